// Large-M per-token x per-channel INT8 GEMM for gfx950: 256 x 256 macro tile, 8 waves, two-phase schedule.
//
// The schedule is the one of gemm_fp8_pp.hip: waves 0..3 (token rows 0..127 of the tile) and waves 4..7 (rows 128..255) sit
// one per SIMD each and take turns - while one group runs a compute phase (32 v_mfma_i32_16x16x64_i8, operands in
// registers, nothing else), the other runs a memory phase (LDS operand reads for its next compute phase first, then its
// share of the direct-to-LDS loads of later K steps); a workgroup barrier ends every phase and group 1 starts one phase
// late.  Per 128-byte K step and wave: M0 (weight fragments, token rows of the first four 16-row tiles), C0, M1 (the other
// four token tiles), C1.  Operands leave LDS a phase before they are used, so a 64-row band is requested again early:
//   set A(b) = the four channel bands, token rows 0..63 and 128..191 of step b: requested in M1(b - 2);
//   set B(b) = token rows 64..127 and 192..255: requested in M0(b - 1).
// Loads complete in order: at the end of every memory phase exactly eight younger loads may still be in flight
// (s_waitcnt vmcnt(8)); every set has four phases to land.
// Arithmetic: exact int32 accumulation inside the MFMA.  Both int8 instructions run at the full rate on zeros, but on
// operand values like a model's the chip's power management lets a register-fed stream of 16x16x64 sustain 0.81 of
// 5 POP/s and one of 32x32x32 only 0.65 (measured on all CUs at once), so the kernel is built on 16x16x64: two per
// 16 x 16 tile and K step (16-byte chunk q of both operands' rows, then chunk q + 4), LDS layout, (row & 7) chunk swizzle
// and fragment reads those of gemm_fp8_pp.hip.  Epilogue f32(acc) * (sb[n] * sa[m]) + bias, separately rounded
// (epilogue_per_row_per_col_scale.h:280-303), or the raw accumulators.  Weights are the MFMA A operand and tokens the
// B operand, so a lane holds 4 consecutive channels of ONE token per tile.  Requires K % 128 == 0, 16-byte aligned rows, row offsets below 4 GiB.
#include "gemm_common.h"

namespace mi355 {
namespace {

constexpr int J_THREADS = 512;
constexpr int J_BM = 256, J_BN = 256, J_WM = 128, J_WN = 64;
constexpr int J_MT = J_WM / 16, J_NT = J_WN / 16;  // 8 token tiles x 4 channel tiles of 16 x 16 per wave
constexpr int J_HT = J_MT / 2;                     // token tiles per compute phase
constexpr int J_ROWS = J_BM + J_BN;
constexpr int J_LOADS = J_ROWS / 64;  // 8 direct-to-LDS loads per wave and K step
constexpr int J_STAGE = J_ROWS * KSTEP;
constexpr int J_SET_A = 6, J_SET_B = 2;

// the two stages are one array: after the K loop it holds the output tile on its way to memory
__shared__ __attribute__((aligned(1024))) uint8_t j_stages[2 * J_STAGE];
#define j_stage0 (j_stages)
#define j_stage1 (j_stages + J_STAGE)
static_assert(2 * J_STAGE >= OUT_TILE_BYTES, "the output tile is staged in the two input stages");

typedef __attribute__((address_space(3))) void* lptr_t;
typedef const __attribute__((address_space(3))) uint8_t* lds_cptr;

__device__ __forceinline__ v4i lds16(lds_cptr p, int imm) {
  const u32x4 v = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(p + imm);
  return v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
}

struct JState {
  const uint8_t* a_base;
  const uint8_t* b_base;
  uint32_t goff[J_LOADS];  // loads 0..3 token rows, 4..7 channel rows
  int wave, kb_last;
  uint32_t tok_off[2], ch_off[2];  // per K half: this lane's 16 bytes in the first token / channel tile
};

// Direct-to-LDS load number i of K step kb (clamped to the last step): tile rows i * 64 + 8 * wave .. + 7 into `stage`.
// Written as an instruction so that the compiler does not count it; it writes m0 (which cannot be named as a clobber:
// reserved register); no compiler-managed use of m0 lies between these statements.
__device__ __forceinline__ void issue_one(const JState& s, int i, uint8_t* stage, int kb) {
  kb = min(kb, s.kb_last);
  const uint8_t* base = (i < J_LOADS / 2 ? s.a_base : s.b_base) + (uint64_t)kb * KSTEP;  // wave-uniform
  asm volatile("" : "+s"(base));
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)(stage + (i * 64 + s.wave * 8) * KSTEP);
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(s.goff[i]), "s"(base), "s"(lds_addr) : "memory");
}
__device__ __forceinline__ void issue_set_a(const JState& s, uint8_t* stage, int b) {
#pragma unroll
  for (int i = 4; i < 8; ++i) issue_one(s, i, stage, b);
  issue_one(s, 0, stage, b);
  issue_one(s, 2, stage, b);
}
__device__ __forceinline__ void issue_set_b(const JState& s, uint8_t* stage, int b) {
  issue_one(s, 1, stage, b);
  issue_one(s, 3, stage, b);
}

__device__ __forceinline__ void compute_end() {
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_setprio(2);  // the memory phase that follows runs above the other group's MFMA stream (measured: ~1 %)
  asm volatile("s_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}
// End of a memory phase: its LDS reads have returned and all but the eight youngest of this wave's loads have landed.
__device__ __forceinline__ void memory_end() {
  static_assert(J_SET_A + J_SET_B == 8, "the wait is written for eight loads per K step");
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  __builtin_amdgcn_s_setprio(0);
  __builtin_amdgcn_sched_barrier(0);
}

// Memory phase, operand part: token tiles 4 * HALF .. + 3 of `cur` (and, for HALF == 0, the weight fragments).
template <int HALF>
__device__ __forceinline__ void read_operands(const JState& s, const uint8_t* cur, v4i (&w)[J_NT][2], v4i (&t)[J_HT][2]) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    if constexpr (HALF == 0) {
#pragma unroll
      for (int i = 0; i < J_NT; ++i) w[i][h] = lds16((lds_cptr)cur + s.ch_off[h], i * 2048);
    }
#pragma unroll
    for (int jj = 0; jj < J_HT; ++jj) t[jj][h] = lds16((lds_cptr)cur + s.tok_off[h], (HALF * J_HT + jj) * 2048);
  }
}

// Compute phase: 32 MFMAs; a tile's accumulator comes round every sixteenth one.
template <int HALF>
__device__ __forceinline__ void compute(const v4i (&w)[J_NT][2], const v4i (&t)[J_HT][2], v4i (&acc)[J_NT][J_MT]) {
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int jj = 0; jj < J_HT; ++jj)
#pragma unroll
      for (int i = 0; i < J_NT; ++i)
        acc[i][HALF * J_HT + jj] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[i][h], t[jj][h], acc[i][HALF * J_HT + jj], 0, 0, 0);
}

__global__ __launch_bounds__(J_THREADS) void int8_gemm_pp_kernel(const GemmParams p) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave >> 2;  // 0: starts computing first; 1: one phase behind.  Also the wave's token half of the tile.
  const int wave_n = wave & 3;
  const int l16 = lane & 15, q = lane >> 4;

  const TileCoord tc = tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n);
  const int m0 = tc.tile_m * J_BM, n0 = tc.tile_n * J_BN;
  const int nkb = p.kb_total;

  JState s;
  s.wave = wave;
  s.kb_last = nkb - 1;
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

  v4i w[J_NT][2], t[J_HT][2];

  // ---- prologue: all of step 0 and set A of step 1
  issue_set_a(s, j_stage0, 0);
  issue_set_b(s, j_stage0, 0);
  issue_set_a(s, j_stage1, 1);
  asm volatile("s_waitcnt vmcnt(6)\n\ts_barrier" ::: "memory");  // step 0 is in LDS (set A of step 1 may be in flight)
  if (grp == 1) compute_end();  // group 1 runs one phase behind group 0

  // One K step: M0, C0, M1, C1.  `cur` holds step kb; `nxt` takes set B of step kb + 1, `cur` set A of step kb + 2.
  auto k_step = [&](uint8_t* cur, uint8_t* nxt, int kb) {
    read_operands<0>(s, cur, w, t);
    issue_set_b(s, nxt, kb + 1);
    memory_end();
    compute<0>(w, t, acc);
    compute_end();
    read_operands<1>(s, cur, w, t);
    issue_set_a(s, cur, kb + 2);
    memory_end();
    compute<1>(w, t, acc);
    compute_end();
  };

  int kb = 0;
  for (; kb + 1 < nkb; kb += 2) {
    k_step(j_stage0, j_stage1, kb);
    k_step(j_stage1, j_stage0, kb + 1);
  }
  if (kb < nkb) k_step(j_stage0, j_stage1, kb);
  if (grp == 0) compute_end();  // as many barriers as group 1
  // the last requests refetch the last step into rows nobody reads any more: they must not outlive the workgroup's LDS
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // ---- epilogue: lane holds, for token m = 16 j + l16 of the wave's rows, channels 16 i + 4 q + (0..3) of its columns
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
    out_tile_store(j_stages, p.out, p.ldo, m0, n0, p.M);
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

// Needs 16-byte aligned rows, K % 128 == 0 and row offsets below 4 GiB.
int launch_int8_pp(GemmParams& p, hipStream_t stream, const char* what) {
  p.tiles_m = (p.M + J_BM - 1) / J_BM;
  p.tiles_n = (p.N + J_BN - 1) / J_BN;
  hipLaunchKernelGGL(int8_gemm_pp_kernel, dim3((unsigned)(p.tiles_m * p.tiles_n)), dim3(J_THREADS), 0, stream, p);
  return check_launch(what);
}

}  // namespace mi355
