// Large-M per-token x per-channel INT8 GEMM for gfx950: 256 x 256 macro tile, 8 waves (two per SIMD) of 128 x 64,
// direct-to-LDS loads, v_mfma_i32_32x32x32_i8.
//
// Two static 64 KB LDS stages filled by global_load_lds_dwordx4, one barrier per 128-byte K step, loads of the next step
// interleaved with the MFMAs.  Compared with the FP8 kernels:
//   * the int8 instruction with the full rate on this part is the 32x32x32 one (measured 3.4 POP/s against 2.1 POP/s
//     for 16x16x64), so a wave's 128 x 64 tile is 4 x 2 tiles of 32 x 32 and a K step is four MFMAs per tile;
//   * accumulation is exact int32 inside the MFMA; there are no per-block scales and no promotion FMAs;
//   * operand fragments are 32 rows x 2 K halves per ds_read_b128, and for that shape the chunk swizzle that reads at the
//     LDS's full 256 B/clk is XOR with (row >> 1) & 7 (measured; (row & 7) halves the rate);
//   * epilogue: f32(acc) * (sb[n] * sa[m]) + bias, separately rounded (epilogue_per_row_per_col_scale.h:280-303), or the
//     raw accumulators.
// Weights are the MFMA A operand and tokens the B operand, so a lane holds 4 x 4 consecutive channels of ONE token.
#include "gemm_common.h"

namespace mi355 {
namespace {

typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int I_THREADS = 512;
constexpr int I_BM = 256, I_BN = 256, I_WM = 128, I_WN = 64;
constexpr int I_MT = I_WM / 32, I_NT = I_WN / 32;  // 4 token tiles x 2 channel tiles of 32 x 32 per wave
constexpr int I_ROWS = I_BM + I_BN;
constexpr int I_LOADS = I_ROWS / 64;  // 8 direct-to-LDS loads per thread and stage
constexpr int I_STAGE = I_ROWS * KSTEP;

__shared__ __attribute__((aligned(1024))) uint8_t i_stage0[I_STAGE];
__shared__ __attribute__((aligned(1024))) uint8_t i_stage1[I_STAGE];

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

struct I8State {
  const uint8_t* a_base;
  const uint8_t* b_base;
  uint32_t goff[I_LOADS];  // loads 0..3 token rows, 4..7 channel rows
  int wave;
  uint32_t tok_off[4], ch_off[4];  // per K sub-step s: offset of this lane's 16 bytes in the first token / channel tile
};

__device__ __forceinline__ void issue_one(const I8State& s, int i, uint8_t* stage, int kb) {
  const uint8_t* base = (i < I_LOADS / 2 ? s.a_base : s.b_base) + (int64_t)kb * KSTEP;
  __builtin_amdgcn_global_load_lds((gptr_t)(base + s.goff[i]), (lptr_t)(stage + (i * 64 + s.wave * 8) * KSTEP), 16, 0, 0);
}

__device__ __forceinline__ v4i ld16(const uint8_t* p) {
  const u32x4 v = *reinterpret_cast<const u32x4*>(p);
  return v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
}

// One 128-byte K step out of `cur`; the direct-to-LDS loads of step kb_next go out in between, into `nxt`.
__device__ __forceinline__ void k_step(const I8State& s, const uint8_t* cur, v16i (&acc)[I_NT][I_MT], uint8_t* nxt,
                                       int kb_next) {
  v4i w[I_NT][4];
#pragma unroll
  for (int i = 0; i < I_NT; ++i)
#pragma unroll
    for (int k = 0; k < 4; ++k) w[i][k] = ld16(cur + s.ch_off[k] + i * 4096);
  // token tiles two at a time: a tile's accumulator is then reused every fourth MFMA, far enough apart for the
  // dependent accumulate not to stall
#pragma unroll
  for (int jp = 0; jp < I_MT / 2; ++jp) {
    v4i t[2][4];
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
      for (int k = 0; k < 4; ++k) t[jj][k] = ld16(cur + s.tok_off[k] + (2 * jp + jj) * 4096);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
        for (int i = 0; i < I_NT; ++i)
          acc[i][2 * jp + jj] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w[i][k], t[jj][k], acc[i][2 * jp + jj], 0, 0, 0);
      }
      // two direct-to-LDS loads per group of four MFMAs: 8 loads over the 8 groups of a step
      issue_one(s, jp * 4 + k, nxt, kb_next);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

__global__ __launch_bounds__(I_THREADS) void int8_gemm_dma_kernel(const GemmParams p) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave >> 2, wave_n = wave & 3;
  const int l32 = lane & 31, kh = lane >> 5;

  const TileCoord tc = tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n);
  const int m0 = tc.tile_m * I_BM, n0 = tc.tile_n * I_BN;
  const int nkb = p.kb_total;

  I8State s;
  s.wave = wave;
  s.a_base = p.a;
  s.b_base = p.b;
  {
    // lane l lands in row l / 8, physical chunk l % 8 of the 8 rows one instruction fills; rows start at multiples of 8,
    // so (row >> 1) & 7 == (4 * wave + (l >> 4)) & 7 for every instruction of this wave
    const int lrow = lane >> 3;
    const int key = (4 * wave + (lane >> 4)) & 7;
    const int chunk_byte = ((lane & 7) ^ key) * 16;
#pragma unroll
    for (int i = 0; i < I_LOADS; ++i) {
      const int row = i * 64 + wave * 8 + lrow;
      if (row < I_BM)
        s.goff[i] = (uint32_t)((int64_t)min(m0 + row, p.M - 1) * p.lda + chunk_byte);
      else
        s.goff[i] = (uint32_t)((int64_t)min(n0 + row - I_BM, p.N - 1) * p.ldb + chunk_byte);
    }
    const int trow = wave_m * I_WM + l32, crow = I_BM + wave_n * I_WN + l32;
#pragma unroll
    for (int k = 0; k < 4; ++k) {  // K sub-step k takes the 16-byte chunk 2k + kh of the row
      s.tok_off[k] = trow * KSTEP + (((2 * k + kh) ^ ((trow >> 1) & 7)) << 4);
      s.ch_off[k] = crow * KSTEP + (((2 * k + kh) ^ ((crow >> 1) & 7)) << 4);
    }
  }

  v16i acc[I_NT][I_MT];
#pragma unroll
  for (int i = 0; i < I_NT; ++i)
#pragma unroll
    for (int j = 0; j < I_MT; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

#pragma unroll
  for (int i = 0; i < I_LOADS; ++i) issue_one(s, i, i_stage0, 0);
  __syncthreads();

  int kb = 0;
  for (; kb + 1 < nkb; kb += 2) {
    k_step(s, i_stage0, acc, i_stage1, kb + 1);
    __syncthreads();
    k_step(s, i_stage1, acc, i_stage0, min(kb + 2, nkb - 1));  // past the end: refetch the last step, unused
    __syncthreads();
  }
  if (kb < nkb) k_step(s, i_stage0, acc, i_stage1, kb);

  // the last iterations refetch a block into a stage nobody reads: those writes must not outlive this workgroup's LDS
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // ---- epilogue: lane holds, for token m, channels n0 + 32 i + 8 g + 4 kh + (0..3), g = 0..3
  const bool vec_ok = ((p.ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
  const bool raw = p.out_dtype == MI355_I32;
#pragma unroll
  for (int j = 0; j < I_MT; ++j) {
    const int m = m0 + wave_m * I_WM + j * 32 + l32;
    if (m >= p.M) continue;
    const float sa_m = raw ? 1.f : p.sa[m];
#pragma unroll
    for (int i = 0; i < I_NT; ++i) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + wave_n * I_WN + i * 32 + 8 * g + 4 * kh;
        if (n >= p.N) continue;
        const int nvalid = min(4, p.N - n);
        if (raw) {
          int* o = reinterpret_cast<int*>(p.out) + (int64_t)m * p.ldo + n;
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (v < nvalid) o[v] = acc[i][j][4 * g + v];
        } else {
          float r[4];
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int nn = min(n + v, p.N - 1);
            float t = mul_rn((float)acc[i][j][4 * g + v], mul_rn(p.sb[nn], sa_m));
            if (p.bias) {
              const uint32_t hb = reinterpret_cast<const uint16_t*>(p.bias)[nn];
              t = add_rn(t, (p.out_dtype == MI355_BF16) ? bf16_bits_to_f32(hb) : f16_bits_to_f32(hb));
            }
            r[v] = t;
          }
          store_out4(p.out, p.out_dtype, (int64_t)m * p.ldo + n, r, nvalid, vec_ok);
        }
      }
    }
  }
}

}  // namespace

// Needs 16-byte aligned rows, K % 128 == 0 and row offsets below 4 GiB.
int launch_int8_dma(GemmParams& p, hipStream_t stream, const char* what) {
  p.tiles_m = (p.M + I_BM - 1) / I_BM;
  p.tiles_n = (p.N + I_BN - 1) / I_BN;
  hipLaunchKernelGGL(int8_gemm_dma_kernel, dim3((unsigned)(p.tiles_m * p.tiles_n)), dim3(I_THREADS), 0, stream, p);
  return check_launch(what);
}

}  // namespace mi355
