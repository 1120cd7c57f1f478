// Large-M blockwise-scaled FP8 GEMM for gfx950: 256 (tokens) x 128 (channels) macro tile, 4 waves of 128 x 64.
//
// Same arithmetic and operand roles as the generic kernel in gemm_w8a8.hip (weights = MFMA A operand, tokens =
// B operand, one v_mfma_f32_16x16x128_f8f6f4 per 128-wide scale block, acc += part * (sa * sb)), but the K loop
// is laid out by hand as a software pipeline, because with one wave per SIMD nothing else hides latency:
//
//   block b is   loaded global -> registers      in iteration b-4 (steps 12..23; two register sets alternate)
//                written registers -> LDS         in iteration b-2 (steps 0..11), visible after that barrier
//                read LDS -> operand registers    in the tail of iteration b-1 (weights, first token tile)
//                multiplied                       in iteration b
//
//   three LDS stages of (256 + 128) rows x 128 B make that legal with ONE barrier per iteration: iteration k
//   multiplies stage k%3, prefetches from stage (k+1)%3 and overwrites stage (k+2)%3, which was last read in
//   iteration k-1.  The loader also stores sa[m,kb] * sb[nb,kb] (one float per token) next to the tile, so the
//   inner loop has no scale arithmetic besides the promotion FMAs.
//
//   an iteration is 32 steps (8 token tiles x 4 channel tiles).  Step t issues the MFMA of tile t and, while it
//   runs, the four FMAs that promote tile t-1, plus at most two memory instructions.  __builtin_amdgcn_sched_barrier
//   fences keep the compiler from collapsing that interleave.  The body is branch-free: past the end of K the
//   loads are clamped to the last block and land in a stage nobody reads.
//
//   weight fragments of the next block need registers while the current ones are still in use, so the body is
//   instantiated twice with the two fragment sets swapped (ping-pong) instead of copying 32 registers.
#include "gemm_common.h"

namespace mi355 {
namespace {

constexpr int P_BM = 256, P_BN = 128, P_WM = 128, P_WN = 64;
constexpr int P_MT = P_WM / 16, P_NT = P_WN / 16;  // 8 token tiles x 4 channel tiles per wave
constexpr int P_ROWS = P_BM + P_BN;                // 384 rows of 128 B per stage
constexpr int P_LOADS = P_ROWS / 32;               // 12 16-byte chunks per thread and stage
constexpr int P_STAGE = P_ROWS * KSTEP;            // 49152 B
constexpr int P_NSTAGE = 3;
constexpr size_t P_LDS = (size_t)P_NSTAGE * P_STAGE + (size_t)P_NSTAGE * P_BM * sizeof(float);

struct Frag {
  u32x4 lo, hi;
};

__device__ __forceinline__ v8i as_v8i(const Frag& f) {
  return v8i{(int)f.lo.x, (int)f.lo.y, (int)f.lo.z, (int)f.lo.w, (int)f.hi.x, (int)f.hi.y, (int)f.hi.z, (int)f.hi.w};
}

struct PipeState {
  // loader
  const uint8_t* a_base;         // uniform bases; per-lane 32-bit byte offsets keep the addresses in saddr + voffset form
  const uint8_t* b_base;
  uint32_t goff[P_LOADS];        // row * stride + 16 * chunk, rows clamped to the matrix (loads 0..7 tokens, 8..11 channels)
  const float* sa_ptr;           // &sa[m, 0] of the token this thread loads the scale of
  const float* sb_ptr;           // &sb[nb, 0]
  int64_t sa_sk, sb_sk;
  uint32_t wr_off;               // LDS offset of this thread's chunk in row (tid >> 3); + 4096 per load
  int chunk_byte;                // 16 * (tid & 7)
  int K, kb_last;
  u32x4 stage_regs[2][P_LOADS];  // two register sets: a block is loaded four iterations before it is multiplied
  float stage_sa[2], stage_sb[2];  // raw scale values; multiplied only when written to LDS, so no wait at load time
  // consumer
  uint32_t tok_off[2], ch_off[2];  // swizzled offsets of the first token / channel tile (halves 0 and 1)
  uint32_t sc_off;                 // byte offset of this lane's first token scale inside a stage's scale row
};

// KFULL: K is a multiple of 128, so every chunk of every block is inside the row.
template <bool KFULL, int SET>
__device__ __forceinline__ void load_one(PipeState& s, int i, int kb) {
  kb = min(kb, s.kb_last);
  const uint8_t* base = (i < P_BM / 32 ? s.a_base : s.b_base) + (int64_t)kb * KSTEP;  // wave-uniform
  if constexpr (KFULL) {
    s.stage_regs[SET][i] = *reinterpret_cast<const u32x4*>(base + s.goff[i]);
  } else {
    const bool valid = kb * KSTEP + s.chunk_byte < s.K;  // past the end of the row: read chunk 0 instead, then zero
    const u32x4 v = *reinterpret_cast<const u32x4*>(base + (valid ? s.goff[i] : s.goff[i] - (uint32_t)s.chunk_byte));
    s.stage_regs[SET][i] = valid ? v : u32x4{0, 0, 0, 0};
  }
}

template <int SET>
__device__ __forceinline__ void load_scale(PipeState& s, int kb) {
  kb = min(kb, s.kb_last);
  s.stage_sa[SET] = s.sa_ptr[(int64_t)kb * s.sa_sk];
  s.stage_sb[SET] = s.sb_ptr[(int64_t)kb * s.sb_sk];
}

// One K block.  wc: weight fragments of this block (already in registers); wn: receives the next block's.
// tokb/scb: double-buffered token fragment and its scale; tokb[0]/scb[0] hold token tile 0 of this block on entry
// and of the next block on exit.
template <bool KFULL, int SET>
__device__ __forceinline__ void k_block(PipeState& s, uint8_t* smem, float (&acc)[P_NT][P_MT][4], Frag (&wc)[P_NT],
                                        Frag (&wn)[P_NT], Frag (&tokb)[2], float (&scb)[2], int st_cur, int st_next,
                                        int st_write, int kb_load) {
  const uint8_t* cur = smem + st_cur * P_STAGE;
  const uint8_t* nxt = smem + st_next * P_STAGE;
  uint8_t* wr = smem + st_write * P_STAGE;
  const float* sc_cur = reinterpret_cast<const float*>(smem + P_NSTAGE * P_STAGE + st_cur * P_BM * 4 + s.sc_off);
  const float* sc_nxt = reinterpret_cast<const float*>(smem + P_NSTAGE * P_STAGE + st_next * P_BM * 4 + s.sc_off);
  float* sc_wr = reinterpret_cast<float*>(smem + P_NSTAGE * P_STAGE + st_write * P_BM * 4);

  v4f part[2];
#pragma unroll
  for (int t = 0; t < P_MT * P_NT; ++t) {
    const int j = t >> 2, i = t & 3;
    part[t & 1] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(as_v8i(wc[i]), as_v8i(tokb[j & 1]),
                                                                   v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);  // the MFMA goes first; everything below runs in its shadow
    if (t > 0) {
      const int pj = (t - 1) >> 2, pi = (t - 1) & 3;
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[pi][pj][v] = fmaf(part[(t - 1) & 1][v], scb[pj & 1], acc[pi][pj][v]);
    }
    // ---- memory slots of this step
    if (t < P_LOADS) {  // register set SET, filled two iterations ago -> stage st_write
      *reinterpret_cast<u32x4*>(wr + s.wr_off + t * 4096) = s.stage_regs[SET][t];
      if (t == 0) sc_wr[threadIdx.x] = s.stage_sa[SET] * s.stage_sb[SET];
    } else if (t < 2 * P_LOADS) {  // refill it with the block four ahead
      load_one<KFULL, SET>(s, t - P_LOADS, kb_load);
      if (t == P_LOADS) load_scale<SET>(s, kb_load);
    }
    if (i == 0 && j + 1 < P_MT) {  // next token tile of this block
      tokb[(j + 1) & 1].lo = *reinterpret_cast<const u32x4*>(cur + s.tok_off[0] + (j + 1) * 2048);
      tokb[(j + 1) & 1].hi = *reinterpret_cast<const u32x4*>(cur + s.tok_off[1] + (j + 1) * 2048);
      scb[(j + 1) & 1] = sc_cur[(j + 1) * 16];
    }
    if (t >= 24) {  // next block: one weight half-fragment per step, token tile 0 once its buffer is free
      const int f = (t - 24) >> 1;
      if ((t & 1) == 0)
        wn[f].lo = *reinterpret_cast<const u32x4*>(nxt + s.ch_off[0] + f * 2048);
      else
        wn[f].hi = *reinterpret_cast<const u32x4*>(nxt + s.ch_off[1] + f * 2048);
      if (t == 28) {
        tokb[0].lo = *reinterpret_cast<const u32x4*>(nxt + s.tok_off[0]);
        tokb[0].hi = *reinterpret_cast<const u32x4*>(nxt + s.tok_off[1]);
        scb[0] = sc_nxt[0];
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  {
    constexpr int t = P_MT * P_NT - 1;
    constexpr int pj = t >> 2, pi = t & 3;
#pragma unroll
    for (int v = 0; v < 4; ++v) acc[pi][pj][v] = fmaf(part[t & 1][v], scb[pj & 1], acc[pi][pj][v]);
  }
}

template <bool KFULL>
__global__ __launch_bounds__(THREADS) void fp8_gemm_pipelined_kernel(const GemmParams p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wave_m = wave >> 1, wave_n = wave & 1;
  const int l16 = lane & 15, q = lane >> 4;

  const TileCoord tc = tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n);
  const int m0 = tc.tile_m * P_BM, n0 = tc.tile_n * P_BN;
  const int nkb = p.kb_total;

  PipeState s;
  s.K = p.K;
  s.kb_last = nkb - 1;
  s.a_base = p.a;
  s.b_base = p.b;
  s.chunk_byte = (tid & 7) * 16;
  {
    const int r0 = tid >> 3;
    s.wr_off = r0 * KSTEP + (((tid & 7) ^ (r0 & 7)) << 4);  // rows r0 + 32*i keep (row & 7), so + 4096*i
#pragma unroll
    for (int i = 0; i < P_LOADS; ++i) {
      const int row = r0 + 32 * i;
      if (row < P_BM)
        s.goff[i] = (uint32_t)((int64_t)min(m0 + row, p.M - 1) * p.lda + s.chunk_byte);
      else
        s.goff[i] = (uint32_t)((int64_t)min(n0 + row - P_BM, p.N - 1) * p.ldb + s.chunk_byte);
    }
  }
  s.sa_ptr = p.sa + (int64_t)min(m0 + tid, p.M - 1) * p.sa_sm;
  s.sa_sk = p.sa_sk;
  s.sb_ptr = p.sb + (int64_t)(min(n0, p.N - 1) / 128) * p.sb_sn;
  s.sb_sk = p.sb_sk;
  {
    const int trow = wave_m * P_WM + l16, crow = P_BM + wave_n * P_WN + l16;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      s.tok_off[h] = trow * KSTEP + (((q + 4 * h) ^ (trow & 7)) << 4);
      s.ch_off[h] = crow * KSTEP + (((q + 4 * h) ^ (crow & 7)) << 4);
    }
    s.sc_off = (wave_m * P_WM + l16) * 4;
  }

  float acc[P_NT][P_MT][4];
#pragma unroll
  for (int i = 0; i < P_NT; ++i)
#pragma unroll
    for (int j = 0; j < P_MT; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;

  // ---- prologue: blocks 0 and 1 into stages 0 and 1, block 2 into registers
  float* sc_base = reinterpret_cast<float*>(smem + P_NSTAGE * P_STAGE);
#pragma unroll
  for (int b = 0; b < 2; ++b) {
#pragma unroll
    for (int i = 0; i < P_LOADS; ++i) load_one<KFULL, 0>(s, i, b);
    load_scale<0>(s, b);
#pragma unroll
    for (int i = 0; i < P_LOADS; ++i)
      *reinterpret_cast<u32x4*>(smem + b * P_STAGE + s.wr_off + i * 4096) = s.stage_regs[0][i];
    sc_base[b * P_BM + tid] = s.stage_sa[0] * s.stage_sb[0];
  }
  // same order as in steady state (set 0 entirely before set 1), so that the wait counts the compiler derives
  // for the loop header from this path agree with those of the back edge
#pragma unroll
  for (int i = 0; i < P_LOADS; ++i) {
    load_one<KFULL, 0>(s, i, 2);
    if (i == 0) load_scale<0>(s, 2);
  }
  __builtin_amdgcn_sched_barrier(0);  // keep the scheduler from interleaving the two groups
#pragma unroll
  for (int i = 0; i < P_LOADS; ++i) {
    load_one<KFULL, 1>(s, i, 3);
    if (i == 0) load_scale<1>(s, 3);
  }
  __syncthreads();

  Frag w0[P_NT], w1[P_NT], tokb[2];
  float scb[2];
#pragma unroll
  for (int f = 0; f < P_NT; ++f) {
    w0[f].lo = *reinterpret_cast<const u32x4*>(smem + s.ch_off[0] + f * 2048);
    w0[f].hi = *reinterpret_cast<const u32x4*>(smem + s.ch_off[1] + f * 2048);
  }
  tokb[0].lo = *reinterpret_cast<const u32x4*>(smem + s.tok_off[0]);
  tokb[0].hi = *reinterpret_cast<const u32x4*>(smem + s.tok_off[1]);
  scb[0] = *reinterpret_cast<const float*>(smem + P_NSTAGE * P_STAGE + s.sc_off);

  int st0 = 0, st1 = 1, st2 = 2;  // stage being multiplied, the next one, the one being overwritten
  int kb = 0;
  for (; kb + 1 < nkb; kb += 2) {  // two blocks per trip: the register sets and weight fragments ping-pong
    k_block<KFULL, 0>(s, smem, acc, w0, w1, tokb, scb, st0, st1, st2, kb + 4);
    __syncthreads();
    k_block<KFULL, 1>(s, smem, acc, w1, w0, tokb, scb, st1, st2, st0, kb + 5);
    __syncthreads();
    const int t = st0;
    st0 = st2, st2 = st1, st1 = t;  // rotate by two
  }
  if (kb < nkb) {  // odd number of blocks
    k_block<KFULL, 0>(s, smem, acc, w0, w1, tokb, scb, st0, st1, st2, kb + 4);
  }

  // ---- epilogue: lane holds channels n .. n+3 of token m
  const bool vec_ok = ((p.ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
#pragma unroll
  for (int j = 0; j < P_MT; ++j) {
    const int m = m0 + wave_m * P_WM + j * 16 + l16;
    if (m >= p.M) continue;
#pragma unroll
    for (int i = 0; i < P_NT; ++i) {
      const int n = n0 + wave_n * P_WN + i * 16 + 4 * q;
      if (n >= p.N) continue;
      fp8_channel_epilogue(p, n, acc[i][j]);
      store_out4(p.out, p.out_dtype, (int64_t)m * p.ldo + n, acc[i][j], min(4, p.N - n), vec_ok);
    }
  }
}

}  // namespace

int launch_fp8_pipelined(GemmParams& p, hipStream_t stream, const char* what) {
  p.tiles_m = (p.M + P_BM - 1) / P_BM;
  p.tiles_n = (p.N + P_BN - 1) / P_BN;
  static bool lds_reserved = false;
  if (!lds_reserved) {
    for (const void* fn : {reinterpret_cast<const void*>(fp8_gemm_pipelined_kernel<true>),
                           reinterpret_cast<const void*>(fp8_gemm_pipelined_kernel<false>)}) {
      hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)P_LDS);
      if (e != hipSuccess) {
        set_error("%s: cannot reserve %zu bytes of LDS: %s", what, P_LDS, hipGetErrorString(e));
        return MI355_ERR_LAUNCH;
      }
    }
    lds_reserved = true;
  }
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n));
  if (p.K % KSTEP == 0)
    hipLaunchKernelGGL(fp8_gemm_pipelined_kernel<true>, grid, dim3(THREADS), P_LDS, stream, p);
  else
    hipLaunchKernelGGL(fp8_gemm_pipelined_kernel<false>, grid, dim3(THREADS), P_LDS, stream, p);
  return check_launch(what);
}

}  // namespace mi355
