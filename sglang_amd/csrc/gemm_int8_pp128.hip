// Mid-M per-token x per-channel INT8 GEMM for gfx950: 128 x 256 macro tile, 8 waves, two-phase schedule, THREE LDS stages.
//
// The three-stage kernel of gemm_int8_dma3.hip runs its eight waves in lockstep: after every barrier all of them read LDS
// (the matrix pipe waits), then all of them multiply (LDS waits); a 128 x 256 tile takes 1.14 us per 128-byte K step where
// the 256 x 256 two-phase kernel (gemm_int8_pp.hip) spends 0.73 us on the same amount of work.  This kernel gives the short
// tile the two-phase schedule: waves 0..3 own token rows 0..63, waves 4..7 rows 64..127, each wave 64 channels
// (4 x 4 tiles of 16 x 16); a group alternates a memory phase (the sixteen ds_read_b128 of its next K step, then its six
// direct-to-LDS loads of the K step after next) with a compute phase (32 v_mfma_i32_16x16x64_i8 and nothing else),
// one workgroup barrier per phase, group 1 one phase behind - so while one group multiplies the other reads.
// A K step is 2 phases (~0.7 us), too short for loads that come from HBM to land within one step, hence three stages of
// 48 KB: the loads of step b + 2 go out in the memory phase of step b into the stage step b - 1 was read from (both groups
// finished reading it a barrier ago) and have two K steps to land; each wave waits for its own loads of step b + 1 at the
// end of that phase (s_waitcnt vmcnt(6): the six just issued may be in flight) and the barriers make that hold for all.
// Arithmetic, fragment layout and swizzle are those of gemm_int8_pp.hip.  Optional split along K (int32 partials to the
// workspace, the ordered reduce applies the epilogue).  Requires K % 128 == 0, 16-byte aligned rows, row offsets below 4 GiB.
#include "gemm_common.h"

namespace mi355 {
namespace {

constexpr int J_THREADS = 512;
constexpr int J_BM = 128, J_BN = 256, J_WM = 64, J_WN = 64;
constexpr int J_MT = J_WM / 16, J_NT = J_WN / 16;  // 4 token tiles x 4 channel tiles of 16 x 16 per wave
constexpr int J_ROWS = J_BM + J_BN;
constexpr int J_LOADS = J_ROWS / 64;  // 6 direct-to-LDS loads per wave and K step: 2 of token rows, 4 of channel rows
constexpr int J_STAGE = J_ROWS * KSTEP;

// the three stages are one array: after the K loop it holds the output tile (128 rows x 512 bytes) on its way to memory
__shared__ __attribute__((aligned(1024))) uint8_t j_stages[3 * J_STAGE];
#define j_stage0 (j_stages)
#define j_stage1 (j_stages + J_STAGE)
#define j_stage2 (j_stages + 2 * J_STAGE)
static_assert(3 * J_STAGE >= J_BM * 512, "the output tile is staged in the input stages");

typedef __attribute__((address_space(3))) void* lptr_t;
typedef const __attribute__((address_space(3))) uint8_t* lds_cptr;

__device__ __forceinline__ v4i lds16(lds_cptr p, int imm) {
  const u32x4 v = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(p + imm);
  return v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
}

struct JState {
  const uint8_t* a_base;
  const uint8_t* b_base;
  uint32_t goff[J_LOADS];  // loads 0..1 token rows, 2..5 channel rows
  int wave, kb_last;
  uint32_t tok_off[2], ch_off[2];  // per K half: this lane's 16 bytes in the first token / channel tile
};

// Direct-to-LDS load number i of K step kb (clamped to the last step): tile rows i * 64 + 8 * wave .. + 7 into `stage`.
// Written as an instruction so that the compiler does not count it; it writes m0 (which cannot be named as a clobber:
// reserved register); no compiler-managed use of m0 lies between these statements.
__device__ __forceinline__ void issue_one(const JState& s, int i, uint8_t* stage, int kb) {
  kb = min(kb, s.kb_last);
  const uint8_t* base = (i < J_BM / 64 ? s.a_base : s.b_base) + (uint64_t)kb * KSTEP;  // wave-uniform
  asm volatile("" : "+s"(base));
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)(stage + (i * 64 + s.wave * 8) * KSTEP);
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(s.goff[i]), "s"(base), "s"(lds_addr) : "memory");
}
__device__ __forceinline__ void issue_step(const JState& s, uint8_t* stage, int b) {
#pragma unroll
  for (int i = 0; i < J_LOADS; ++i) issue_one(s, i, stage, b);
}

__device__ __forceinline__ void compute_end() {
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_setprio(2);  // the memory phase that follows runs above the other group's MFMA stream (measured: ~1 %)
  asm volatile("s_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}
// End of a memory phase: its LDS reads have returned and all but the six youngest of this wave's loads have landed.
__device__ __forceinline__ void memory_end() {
  static_assert(J_LOADS == 6, "the wait is written for six loads per K step");
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  __builtin_amdgcn_s_setprio(0);
  __builtin_amdgcn_sched_barrier(0);
}

// Memory phase, operand part: the wave's weight and token fragments of the K step in `cur`.
__device__ __forceinline__ void read_operands(const JState& s, const uint8_t* cur, v4i (&w)[J_NT][2], v4i (&t)[J_MT][2]) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int i = 0; i < J_NT; ++i) w[i][h] = lds16((lds_cptr)cur + s.ch_off[h], i * 2048);
#pragma unroll
    for (int j = 0; j < J_MT; ++j) t[j][h] = lds16((lds_cptr)cur + s.tok_off[h], j * 2048);
  }
}

// Compute phase: 32 MFMAs; a tile's accumulator comes round every sixteenth one.
__device__ __forceinline__ void compute(const v4i (&w)[J_NT][2], const v4i (&t)[J_MT][2], v4i (&acc)[J_NT][J_MT]) {
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int j = 0; j < J_MT; ++j)
#pragma unroll
      for (int i = 0; i < J_NT; ++i) acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[i][h], t[j][h], acc[i][j], 0, 0, 0);
}

// 128-row output tile through LDS (rows of 512 bytes, chunks swizzled as out_tile_put4 writes them): every wave stores 16
// whole rows, two per instruction.  Needs ldo % 8 == 0, a 16-byte aligned output base and n0 + 256 <= N.
__device__ __forceinline__ void out_tile128_store(const uint8_t* tile, void* out, int64_t ldo, int m0, int n0, int M) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int chunk = lane & 31;
  uint16_t* o = reinterpret_cast<uint16_t*>(out);
#pragma unroll 4
  for (int it = 0; it < 8; ++it) {
    const int row = wave * 16 + it * 2 + (lane >> 5);
    const u32x4 v = *reinterpret_cast<const u32x4*>(tile + row * 512 + ((chunk ^ (row & 7)) << 4));
    if (m0 + row < M) *reinterpret_cast<u32x4*>(o + (int64_t)(m0 + row) * ldo + n0 + chunk * 8) = v;
  }
}

template <bool SPLIT>
__global__ __launch_bounds__(J_THREADS) void int8_gemm_pp128_kernel(const GemmParams p) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave >> 2;  // 0: starts computing first; 1: one phase behind.  Also the wave's token half of the tile.
  const int wave_n = wave & 3;
  const int l16 = lane & 15, q = lane >> 4;

  const TileCoord tc = tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n);
  const int m0 = tc.tile_m * J_BM, n0 = tc.tile_n * J_BN;
  const int kb_begin = tc.split * p.kb_per_split;
  const int kb_end = min(p.kb_total, kb_begin + p.kb_per_split);
  const int nkb = kb_end - kb_begin;

  JState s;
  s.wave = wave;
  s.kb_last = kb_end - 1;
  s.a_base = p.a;
  s.b_base = p.b;
  {
    // lane l lands in row l / 8, physical chunk l % 8 of the 8 rows one load fills (rows start at multiples of 8); it
    // fetches the logical chunk that belongs there under the (row & 7) swizzle
    const int lrow = lane >> 3;
    const int chunk_byte = ((lane & 7) ^ lrow) * 16;
#pragma unroll
    for (int i = 0; i < J_LOADS; ++i) {
      const int row = i * 64 + wave * 8 + lrow;
      if (row < J_BM)
        s.goff[i] = (uint32_t)((int64_t)min(m0 + row, p.M - 1) * p.lda + chunk_byte);
      else
        s.goff[i] = (uint32_t)((int64_t)min(n0 + row - J_BM, p.N - 1) * p.ldb + chunk_byte);
    }
    const int trow = grp * J_WM + l16, crow = J_BM + wave_n * J_WN + l16;
#pragma unroll
    for (int h = 0; h < 2; ++h) {  // K half h takes the 16-byte chunk q + 4h of the row
      s.tok_off[h] = trow * KSTEP + (((q + 4 * h) ^ (trow & 7)) << 4);
      s.ch_off[h] = crow * KSTEP + (((q + 4 * h) ^ (crow & 7)) << 4);
    }
  }

  v4i acc[J_NT][J_MT];
#pragma unroll
  for (int i = 0; i < J_NT; ++i)
#pragma unroll
    for (int j = 0; j < J_MT; ++j) acc[i][j] = v4i{0, 0, 0, 0};

  v4i w[J_NT][2], t[J_MT][2];

  // ---- prologue: steps 0 and 1
  issue_step(s, j_stage0, kb_begin);
  issue_step(s, j_stage1, kb_begin + 1);
  asm volatile("s_waitcnt vmcnt(6)\n\ts_barrier" ::: "memory");  // step 0 is in LDS (step 1 may be in flight)
  if (grp == 1) compute_end();  // group 1 runs one phase behind group 0

  // One K step: memory phase (operands of `cur`, loads of the step after next into `nxt2`), compute phase.
  auto k_step = [&](uint8_t* cur, uint8_t* nxt2, int kb) {
    read_operands(s, cur, w, t);
    issue_step(s, nxt2, kb + 2);
    memory_end();
    compute(w, t, acc);
    compute_end();
  };

  int k = 0;
  for (; k + 2 < nkb; k += 3) {
    k_step(j_stage0, j_stage2, kb_begin + k);
    k_step(j_stage1, j_stage0, kb_begin + k + 1);
    k_step(j_stage2, j_stage1, kb_begin + k + 2);
  }
  if (k < nkb) {
    k_step(j_stage0, j_stage2, kb_begin + k);
    if (k + 1 < nkb) k_step(j_stage1, j_stage0, kb_begin + k + 1);
  }
  if (grp == 0) compute_end();  // as many barriers as group 1
  // the last requests refetch the last step into rows nobody reads any more: they must not outlive the workgroup's LDS
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // ---- epilogue: lane holds, for token m = 16 j + l16 of the wave's rows, channels 16 i + 4 q + (0..3) of its columns
  if constexpr (SPLIT) {
#pragma unroll
    for (int j = 0; j < J_MT; ++j) {
      const int m = m0 + grp * J_WM + j * 16 + l16;
      if (m >= p.M) continue;
#pragma unroll
      for (int i = 0; i < J_NT; ++i)
        {
          const int n = n0 + wave_n * J_WN + i * 16 + 4 * q;
          if (n >= p.N) continue;
          const int nvalid = min(4, p.N - n);
          int* wsp = reinterpret_cast<int*>(p.ws) + ((int64_t)tc.split * p.M + m) * p.N + n;
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (v < nvalid) wsp[v] = acc[i][j][v];
        }
    }
    return;
  }
  const bool vec_ok = ((p.ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
  const bool raw = p.out_dtype == MI355_I32;
  if (out_tile_ok(p.out, p.ldo, p.out_dtype, n0, p.N) && (reinterpret_cast<uintptr_t>(p.sb) & 15) == 0 &&
      (p.bias == nullptr || (reinterpret_cast<uintptr_t>(p.bias) & 7) == 0)) {
    // full tile: channel scales and bias by 16- and 8-byte loads, results through LDS, whole rows to memory
    asm volatile("s_barrier" ::: "memory");  // every wave's stray loads have landed: the stages are free
    float sa_j[J_MT];
#pragma unroll
    for (int j = 0; j < J_MT; ++j) sa_j[j] = p.sa[min(m0 + grp * J_WM + j * 16 + l16, p.M - 1)];
#pragma unroll
    for (int i = 0; i < J_NT; ++i) {
      {
        const int col = wave_n * J_WN + i * 16 + 4 * q;
        const v4f sbv = *reinterpret_cast<const v4f*>(p.sb + n0 + col);
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (p.bias) {
          const u32x2 hb = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint16_t*>(p.bias) + n0 + col);
          const uint32_t h[4] = {hb.x & 0xffffu, hb.x >> 16, hb.y & 0xffffu, hb.y >> 16};
#pragma unroll
          for (int v = 0; v < 4; ++v) bv[v] = (p.out_dtype == MI355_BF16) ? bf16_bits_to_f32(h[v]) : f16_bits_to_f32(h[v]);
        }
#pragma unroll
        for (int j = 0; j < J_MT; ++j) {
          float r[4];
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            float x = mul_rn((float)acc[i][j][v], mul_rn(sbv[v], sa_j[j]));
            if (p.bias) x = add_rn(x, bv[v]);
            r[v] = x;
          }
          out_tile_put4(j_stages, grp * J_WM + j * 16 + l16, col, p.out_dtype, r);
        }
      }
    }
    __syncthreads();
    out_tile128_store(j_stages, p.out, p.ldo, m0, n0, p.M);
    return;
  }
#pragma unroll
  for (int j = 0; j < J_MT; ++j) {
    const int m = m0 + grp * J_WM + j * 16 + l16;
    if (m >= p.M) continue;
    const float sa_m = raw ? 1.f : p.sa[m];
#pragma unroll
    for (int i = 0; i < J_NT; ++i) {
      {
        const int n = n0 + wave_n * J_WN + i * 16 + 4 * q;
        if (n >= p.N) continue;
        const int nvalid = min(4, p.N - n);
        if (raw) {
          int* o = reinterpret_cast<int*>(p.out) + (int64_t)m * p.ldo + n;
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (v < nvalid) o[v] = acc[i][j][v];
        } else {
          float r[4];
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int nn = min(n + v, p.N - 1);
            float x = mul_rn((float)acc[i][j][v], mul_rn(p.sb[nn], sa_m));
            if (p.bias) {
              const uint32_t hb = reinterpret_cast<const uint16_t*>(p.bias)[nn];
              x = add_rn(x, (p.out_dtype == MI355_BF16) ? bf16_bits_to_f32(hb) : f16_bits_to_f32(hb));
            }
            r[v] = x;
          }
          store_out4(p.out, p.out_dtype, (int64_t)m * p.ldo + n, r, nvalid, vec_ok);
        }
      }
    }
  }
}

}  // namespace

// Needs 16-byte aligned rows, K % 128 == 0 and row offsets below 4 GiB.  The caller sets p.splits, p.kb_per_split and p.ws.
int launch_int8_pp128(GemmParams& p, hipStream_t stream, const char* what) {
  p.tiles_m = (p.M + J_BM - 1) / J_BM;
  p.tiles_n = (p.N + J_BN - 1) / J_BN;
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n * p.splits));
  if (p.splits > 1)
    hipLaunchKernelGGL(int8_gemm_pp128_kernel<true>, grid, dim3(J_THREADS), 0, stream, p);
  else
    hipLaunchKernelGGL(int8_gemm_pp128_kernel<false>, grid, dim3(J_THREADS), 0, stream, p);
  return check_launch(what);
}

}  // namespace mi355
