// Large-M blockwise-scaled FP8 GEMM for gfx950: 256 x 256 macro tile, 8 waves (two per SIMD) of 128 x 64.
//
// Why this shape.  Measured on MI355X: one v_mfma_f32_16x16x128_f8f6f4 occupies the matrix pipe for 33 cycles, and a
// wave can issue roughly one instruction every four cycles, so a wave that has to issue the MFMA, its four promotion
// FMAs, its share of LDS reads/writes, global loads, waits and address arithmetic (about 11 instructions per MFMA) is
// issue-bound at ~59 cycles per MFMA when it is alone on its SIMD.  Two waves per SIMD issue different instruction
// types in the same cycle and keep the pipe busy, but then a wave may only own 256 registers.  128 accumulators leave
// no room for staging registers, so the tiles go from global memory straight into LDS with
// global_load_lds_dwordx4 (16-byte direct-to-LDS loads exist on gfx950): no staging registers, no ds_write.
//
// Arithmetic and operand roles are those of the generic kernel in gemm_w8a8.hip: weights are the MFMA A operand,
// tokens the B operand, one MFMA consumes one 128-wide scale block, acc += part * (sa[m,kb] * sb[nb,kb]).
//
// LDS: two stages (separate static arrays, so the compiler can tell a DMA into one stage from reads of the other and
// does not serialize them), each 512 rows x 128 B (rows 0..255 tokens, 256..511 channels) plus 256 token scales.
// A direct-to-LDS load writes lane l's 16 bytes at base + 16 * l, i.e. a wave fills 8 rows of 128 B per instruction;
// the 16-byte chunks of a row are XOR-swizzled with (row & 7) by choosing which chunk each lane FETCHES.  Operand reads
// take chunks q and q + 4 per lane quarter q, the pattern that sustains the LDS's full 256 B/clk.
//
// Schedule of one iteration (block k in stage k % 2): issue the DMA for block k+1 into the other stage, which every
// wave finished reading before the barrier that ended iteration k-1; read fragments and run 32 steps of
// {MFMA of tile t, FMAs of tile t-1}; wait for the DMA, barrier.
#include "gemm_common.h"

namespace mi355 {
namespace {

constexpr int D_THREADS = 512;
constexpr int D_BM = 256, D_BN = 256, D_WM = 128, D_WN = 64;
constexpr int D_MT = D_WM / 16, D_NT = D_WN / 16;  // 8 token tiles x 4 channel tiles per wave
constexpr int D_ROWS = D_BM + D_BN;                // 512 rows of 128 B
constexpr int D_LOADS = D_ROWS / 64;               // 8 direct-to-LDS loads per thread and stage (a wave fills 8 rows each)
constexpr int D_STAGE = D_ROWS * KSTEP;            // 65536 B

__shared__ __attribute__((aligned(1024))) uint8_t d_stage0[D_STAGE];
__shared__ __attribute__((aligned(1024))) uint8_t d_stage1[D_STAGE];
// 256 token scales per stage; the array is twice that long because all 8 waves run the scale fetch (waves 4..7 write a
// second, unused copy): a wave-conditional fetch would put a branch into the K loop, and the compiler then sinks the
// promotion FMAs across it, which serializes the loop and spills
__shared__ __attribute__((aligned(256))) float d_scale0[2 * D_BM];
__shared__ __attribute__((aligned(256))) float d_scale1[2 * D_BM];

__device__ __attribute__((aligned(16))) const uint32_t d_zero16[4] = {0, 0, 0, 0};  // source of chunks past the end of K

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;
// read-only scalars fetched through the constant address space become s_load (own counter, no vmcnt traffic)
typedef const __attribute__((address_space(4))) float* cfloat_ptr;
typedef const __attribute__((address_space(3))) uint8_t* lds_cptr;

// Per-lane LDS base of one stage (typed as an LDS pointer so that tile offsets fold into ds_read immediates).
__device__ __forceinline__ lds_cptr lds_base(const uint8_t* stage, uint32_t off) {
  return (lds_cptr)stage + off;
}
__device__ __forceinline__ u32x4 lds16(lds_cptr p, int imm) {
  return *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(p + imm);
}

struct Frag {
  u32x4 lo, hi;
};
__device__ __forceinline__ v8i as_v8i(const Frag& f) {
  return v8i{(int)f.lo.x, (int)f.lo.y, (int)f.lo.z, (int)f.lo.w, (int)f.hi.x, (int)f.hi.y, (int)f.hi.z, (int)f.hi.w};
}

struct DmaState {
  const uint8_t* a_base;
  const uint8_t* b_base;
  uint32_t goff[D_LOADS];  // byte offset of this lane's chunk from the matrix base (rows clamped); loads 0..3 tokens, 4..7 channels
  int chunk_byte;          // 16 * logical chunk this lane fetches
  const float* sa_ptr;     // &sa[m, 0] for the token whose scale this thread fetches (waves 0..3)
  cfloat_ptr sb_ptr;       // &sb[nb, 0] of this wave's 128-channel block
  int64_t sa_sk, sb_sk;
  int K;
  int wave;
  uint32_t tok_off[2], ch_off[2], sc_off;
};

// Direct-to-LDS load number i (0..7: tile rows, 8: token scales) of K block kb into `stage` / `scale`.
template <bool KFULL>
__device__ __forceinline__ void issue_one(const DmaState& s, int i, uint8_t* stage, float* scale, int kb) {
  if (i < D_LOADS) {
    // scalar base + 32-bit lane offset (saddr form).  The asm keeps the compiler from folding the lane offset into
    // per-lane 64-bit pointers, which costs 16 registers and a 64-bit vector add per load.
    const uint8_t* base = (i < D_LOADS / 2 ? s.a_base : s.b_base) + (uint64_t)kb * KSTEP;
    asm volatile("" : "+s"(base));
    const uint8_t* src = base + s.goff[i];
    if constexpr (!KFULL) {
      if (kb * KSTEP + s.chunk_byte >= s.K) src = reinterpret_cast<const uint8_t*>(d_zero16);
    }
    __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(stage + (i * 64 + s.wave * 8) * KSTEP), 16, 0, 0);
  } else {
    __builtin_amdgcn_global_load_lds((gptr_t)(s.sa_ptr + (int64_t)kb * s.sa_sk), (lptr_t)(scale + s.wave * 64), 4, 0, 0);
  }
}

template <bool KFULL>
__device__ __forceinline__ void issue_block(const DmaState& s, uint8_t* stage, float* scale, int kb) {
#pragma unroll
  for (int i = 0; i <= D_LOADS; ++i) issue_one<KFULL>(s, i, stage, scale, kb);
}

// One K block out of `cur` / `sc_cur`; meanwhile the direct-to-LDS loads of block kb_next go out into `nxt` / `sc_nxt`,
// one per step over the first nine steps: early, so that they have the rest of the iteration to land before the barrier,
// but not in one burst, which would hold the wave until the address unit has taken them (a wave issues in order).
template <bool KFULL>
__device__ __forceinline__ void k_block(const DmaState& s, const uint8_t* cur, const float* sc_cur, float sbv,
                                        float (&acc)[D_NT][D_MT][4], uint8_t* nxt, float* sc_nxt, int kb_next) {
  Frag w[D_NT], tokb[2];
  float scb[2];
  const lds_cptr ch0 = lds_base(cur, s.ch_off[0]), ch1 = lds_base(cur, s.ch_off[1]);
  const lds_cptr tk0 = lds_base(cur, s.tok_off[0]), tk1 = lds_base(cur, s.tok_off[1]);
  // only what the first MFMA needs is read up front (all eight waves hit the LDS at once after the barrier); the
  // other weight fragments follow in steps 0..2
  w[0].lo = lds16(ch0, 0);
  w[0].hi = lds16(ch1, 0);
  tokb[0].lo = lds16(tk0, 0);
  tokb[0].hi = lds16(tk1, 0);
  const float* scp = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(sc_cur) + s.sc_off);
  scb[0] = scp[0] * sbv;
  __builtin_amdgcn_sched_barrier(0);

  v4f part[2];
#pragma unroll
  for (int t = 0; t < D_MT * D_NT; ++t) {
    const int j = t >> 2, i = t & 3;
    part[t & 1] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(as_v8i(w[i]), as_v8i(tokb[j & 1]),
                                                                   v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);  // the MFMA goes first; the rest of the step runs in its shadow
    if (t > 0) {
      const int pj = (t - 1) >> 2, pi = (t - 1) & 3;
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[pi][pj][v] = fmaf(part[(t - 1) & 1][v], scb[pj & 1], acc[pi][pj][v]);
    }
    if (t + 1 < D_NT) {  // weight fragment of the next step (first pass over the channel tiles only)
      w[t + 1].lo = lds16(ch0, (t + 1) * 2048);
      w[t + 1].hi = lds16(ch1, (t + 1) * 2048);
    }
    if (i == 0 && j + 1 < D_MT) {  // next token tile
      tokb[(j + 1) & 1].lo = lds16(tk0, (j + 1) * 2048);
      tokb[(j + 1) & 1].hi = lds16(tk1, (j + 1) * 2048);
    }
    if (i == 1 && j + 1 < D_MT) scb[(j + 1) & 1] = scp[(j + 1) * 16] * sbv;
    if (t <= D_LOADS) issue_one<KFULL>(s, t, nxt, sc_nxt, kb_next);
    __builtin_amdgcn_sched_barrier(0);
  }
  {
    constexpr int t = D_MT * D_NT - 1;
    constexpr int pj = t >> 2, pi = t & 3;
#pragma unroll
    for (int v = 0; v < 4; ++v) acc[pi][pj][v] = fmaf(part[t & 1][v], scb[pj & 1], acc[pi][pj][v]);
  }
}

template <bool KFULL>
__global__ __launch_bounds__(D_THREADS) void fp8_gemm_dma_kernel(const GemmParams p) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: LDS destinations and scale pointers stay scalar
  const int wave_m = wave >> 2, wave_n = wave & 3;
  const int l16 = lane & 15, q = lane >> 4;

  const TileCoord tc = tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n);
  const int m0 = tc.tile_m * D_BM, n0 = tc.tile_n * D_BN;
  const int nkb = p.kb_total;

  DmaState s;
  s.K = p.K;
  s.wave = wave;
  s.a_base = p.a;
  s.b_base = p.b;
  {
    // lane l of a wave lands in row l / 8, physical chunk l % 8 of the 8 rows its instruction fills
    const int lrow = lane >> 3;
    const int logical = (lane & 7) ^ lrow;  // (row & 7) == lrow because every 8-row group starts at a multiple of 8
    s.chunk_byte = logical * 16;
#pragma unroll
    for (int i = 0; i < D_LOADS; ++i) {
      const int row = i * 64 + wave * 8 + lrow;
      if (row < D_BM)
        s.goff[i] = (uint32_t)((int64_t)min(m0 + row, p.M - 1) * p.lda + s.chunk_byte);
      else
        s.goff[i] = (uint32_t)((int64_t)min(n0 + row - D_BM, p.N - 1) * p.ldb + s.chunk_byte);
    }
  }
  s.sa_ptr = p.sa + (int64_t)min(m0 + (tid & (D_BM - 1)), p.M - 1) * p.sa_sm;
  s.sa_sk = p.sa_sk;
  // wave-uniform by construction; readfirstlane tells the compiler so, which turns the per-block fetch into a scalar load
  s.sb_ptr = (cfloat_ptr)(p.sb + (int64_t)__builtin_amdgcn_readfirstlane(min(n0 + wave_n * D_WN, p.N - 1) / 128) * p.sb_sn);
  s.sb_sk = p.sb_sk;
  {
    const int trow = wave_m * D_WM + l16, crow = D_BM + wave_n * D_WN + l16;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      s.tok_off[h] = trow * KSTEP + (((q + 4 * h) ^ (trow & 7)) << 4);
      s.ch_off[h] = crow * KSTEP + (((q + 4 * h) ^ (crow & 7)) << 4);
    }
    s.sc_off = (wave_m * D_WM + l16) * 4;
  }

  float acc[D_NT][D_MT][4];
#pragma unroll
  for (int i = 0; i < D_NT; ++i)
#pragma unroll
    for (int j = 0; j < D_MT; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;

  issue_block<KFULL>(s, d_stage0, d_scale0, 0);
  float sb_cur = s.sb_ptr[0];
  __syncthreads();

  int kb = 0;
  for (; kb + 1 < nkb; kb += 2) {
    // the weight-block scales of the next two blocks are fetched (scalar loads) before anything needs them
    const float sb_1 = s.sb_ptr[(int64_t)(kb + 1) * s.sb_sk];
    const float sb_2 = s.sb_ptr[(int64_t)min(kb + 2, nkb - 1) * s.sb_sk];
    k_block<KFULL>(s, d_stage0, d_scale0, sb_cur, acc, d_stage1, d_scale1, kb + 1);
    __syncthreads();
    // past the end of K the last block is fetched again into a stage nobody reads
    k_block<KFULL>(s, d_stage1, d_scale1, sb_1, acc, d_stage0, d_scale0, min(kb + 2, nkb - 1));
    __syncthreads();
    sb_cur = sb_2;
  }
  if (kb < nkb) k_block<KFULL>(s, d_stage0, d_scale0, sb_cur, acc, d_stage1, d_scale1, kb);

  // the last iterations refetch a block into a stage nobody reads: those writes must not outlive this workgroup's LDS
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // ---- epilogue: lane holds channels n .. n+3 of token m
  const bool vec_ok = ((p.ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
#pragma unroll
  for (int j = 0; j < D_MT; ++j) {
    const int m = m0 + wave_m * D_WM + j * 16 + l16;
    if (m >= p.M) continue;
#pragma unroll
    for (int i = 0; i < D_NT; ++i) {
      const int n = n0 + wave_n * D_WN + i * 16 + 4 * q;
      if (n >= p.N) continue;
      store_out4(p.out, p.out_dtype, (int64_t)m * p.ldo + n, acc[i][j], min(4, p.N - n), vec_ok);
    }
  }
}

}  // namespace

int launch_fp8_dma(GemmParams& p, hipStream_t stream, const char* what) {
  p.tiles_m = (p.M + D_BM - 1) / D_BM;
  p.tiles_n = (p.N + D_BN - 1) / D_BN;
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n));
  if (p.K % KSTEP == 0)
    hipLaunchKernelGGL(fp8_gemm_dma_kernel<true>, grid, dim3(D_THREADS), 0, stream, p);
  else
    hipLaunchKernelGGL(fp8_gemm_dma_kernel<false>, grid, dim3(D_THREADS), 0, stream, p);
  return check_launch(what);
}

}  // namespace mi355
