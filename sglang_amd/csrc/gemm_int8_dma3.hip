// Mid-M per-token x per-channel INT8 GEMM for gfx950: 64 x 256, 128 x 128 or 64 x 128 macro tile, 8 waves, THREE LDS stages
// (the 128 x 256 tile of this family is served by the two-phase kernel of gemm_int8_pp128.hip, which is a quarter faster).
//
// The loop structure is the one of gemm_fp8_dma3.hip: the direct-to-LDS loads of K step k+2 are issued while step k is
// multiplied, the wait before the bare s_barrier that ends iteration k covers step k+1 only (s_waitcnt vmcnt(LOADS), the
// loads per wave and iteration being a constant), loads, wait and barrier are written as instructions.  The arithmetic
// is the one of gemm_int8_pp.hip: v_mfma_i32_16x16x64_i8, two per 16 x 16 tile and 128-byte K step (chunk q of both
// operands' rows, then chunk q + 4), exact int32 accumulation, (row & 7) chunk swizzle.  A wave owns (BM / 2) x (BN / 4)
// outputs; the 128-channel tiles fill the chip for layers with few channels (K=4096 -> N=6144 at 256 tokens: 17 against 24 us).
// Optional split along K: int32 partials to the workspace, the ordered reduce applies the epilogue.
// Requires K % 128 == 0, 16-byte aligned rows, row offsets below 4 GiB.
#include "gemm_common.h"

namespace mi355 {
namespace {

constexpr int U_THREADS = 512;

typedef __attribute__((address_space(3))) void* lptr_t;
typedef const __attribute__((address_space(3))) uint8_t* lds_cptr;


__device__ __forceinline__ v4i lds16(lds_cptr p, int imm) {
  const u32x4 v = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(p + imm);
  return v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
}

template <int BM, int BN>
struct U8State {
  static constexpr int LOADS = (BM + BN) / 64;
  const uint8_t* a_base;
  const uint8_t* b_base;
  uint32_t goff[LOADS];
  int wave, kb_last;
  uint32_t tok_off[2], ch_off[2];  // per K half: this lane's 16 bytes in the first token / channel tile
};

// Writes m0, which cannot be listed as a clobber (reserved register); no compiler-managed use of m0 lies in the K loop.
template <int BM, int BN>
__device__ __forceinline__ void issue_one(const U8State<BM, BN>& s, int i, uint8_t* stage, int kb) {
  kb = min(kb, s.kb_last);
  const uint8_t* base = (i < BM / 64 ? s.a_base : s.b_base) + (uint64_t)kb * KSTEP;  // wave-uniform
  asm volatile("" : "+s"(base));
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)(stage + (i * 64 + s.wave * 8) * KSTEP);
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(s.goff[i]), "s"(base), "s"(lds_addr) : "memory");
}

// One 128-byte K step out of `cur`; the loads of step kb_next go out in between, into `nxt`.
template <int BM, int BN>
__device__ __forceinline__ void k_step(const U8State<BM, BN>& s, const uint8_t* cur, v4i (&acc)[BN / 64][BM / 32], uint8_t* nxt,
                                       int kb_next) {
  constexpr int MT = BM / 32, U_NT = BN / 64, LOADS = U8State<BM, BN>::LOADS;  // a wave owns BN / 4 channels = U_NT tiles of 16
  v4i w[U_NT][2], t[MT][2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int i = 0; i < U_NT; ++i) w[i][h] = lds16((lds_cptr)cur + s.ch_off[h], i * 2048);
#pragma unroll
    for (int j = 0; j < MT; ++j) t[j][h] = lds16((lds_cptr)cur + s.tok_off[h], j * 2048);
  }
  int issued = 0;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int j = 0; j < MT; ++j) {
#pragma unroll
      for (int i = 0; i < U_NT; ++i)
        acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[i][h], t[j][h], acc[i][j], 0, 0, 0);
      if (issued < LOADS) issue_one<BM, BN>(s, issued++, nxt, kb_next);
      if (issued < LOADS && MT == 2) issue_one<BM, BN>(s, issued++, nxt, kb_next);  // 4 groups only: two loads per group
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// Everything but the YOUNGER youngest loads has landed; then the workgroup barrier.
template <int YOUNGER>
__device__ __forceinline__ void wait_and_barrier() {
  static_assert(YOUNGER >= 3 && YOUNGER <= 24, "(stages - 2) x LOADS, LOADS = (BM + BN) / 64");
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(YOUNGER) : "memory");
}

// S: LDS stages.  Three; four for 128 x 128 tiles (32 KB a stage: the workgroup has the CU to itself either way); six for
// 64 x 128 tiles where the launch has at most one workgroup per CU (otherwise two workgroups of three stages share the CU),
// then with one barrier per two K blocks - as in the FP8 kernel of the same structure (gemm_fp8_dma3.hip).
template <int BM, bool SPLIT, int BN, int S = 3>
__global__ __launch_bounds__(U_THREADS) void int8_gemm_dma3_kernel(const GemmParams p) {
  static_assert(BN == 128 || BN == 256, "channel tile");
  constexpr int WM = BM / 2, MT = WM / 16, U_WN = BN / 4, U_NT = U_WN / 16, LOADS = U8State<BM, BN>::LOADS;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave >> 2, wave_n = wave & 3;
  const int l16 = lane & 15, q = lane >> 4;

  const TileCoord tc = tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n);
  const int m0 = tc.tile_m * BM, n0 = tc.tile_n * BN;
  const int kb_begin = tc.split * p.kb_per_split;
  const int kb_end = min(p.kb_total, kb_begin + p.kb_per_split);
  const int nkb = kb_end - kb_begin;

  // S stages of (BM token rows + BN channel rows) x 128 bytes, sized per tile shape: three stages of a 64 x 128 tile take
  // 72 KB, so two such workgroups share a CU's 160 KB
  static_assert(S >= 3 && S * (BM + BN) * KSTEP <= 160 * 1024, "the stages must fit the CU's LDS");
  __shared__ __attribute__((aligned(1024))) uint8_t u_stage[S][(BM + BN) * KSTEP];
  // PAIRED (six stages): one barrier per two K blocks; iteration k requests block k + S - 2 into the stage that iteration
  // k - 2 read, and the wait in front of the barrier covers the two blocks of the next pair
  constexpr bool PAIRED = S == 6;
  constexpr int AHEAD = PAIRED ? S - 2 : S - 1;
  constexpr int YOUNGER = (PAIRED ? S - 4 : S - 2) * LOADS;
  U8State<BM, BN> s;
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
    for (int i = 0; i < LOADS; ++i) {
      const int row = i * 64 + wave * 8 + lrow;
      if (row < BM)
        s.goff[i] = (uint32_t)((int64_t)min(m0 + row, p.M - 1) * p.lda + chunk_byte);
      else
        s.goff[i] = (uint32_t)((int64_t)min(n0 + row - BM, p.N - 1) * p.ldb + chunk_byte);
    }
    const int trow = wave_m * WM + l16, crow = BM + wave_n * U_WN + l16;
#pragma unroll
    for (int h = 0; h < 2; ++h) {  // K half h takes the 16-byte chunk q + 4h of the row
      s.tok_off[h] = trow * KSTEP + (((q + 4 * h) ^ (trow & 7)) << 4);
      s.ch_off[h] = crow * KSTEP + (((q + 4 * h) ^ (crow & 7)) << 4);
    }
  }

  v4i acc[U_NT][MT];
#pragma unroll
  for (int i = 0; i < U_NT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[i][j] = v4i{0, 0, 0, 0};

#pragma unroll
  for (int b = 0; b < AHEAD; ++b)
#pragma unroll
    for (int i = 0; i < LOADS; ++i) issue_one<BM, BN>(s, i, u_stage[b], kb_begin + b);
  wait_and_barrier<YOUNGER>();

  int k = 0;
  for (; k + S - 1 < nkb; k += S) {
#pragma unroll
    for (int u = 0; u < S; ++u) {
      k_step<BM, BN>(s, u_stage[u], acc, u_stage[(u + AHEAD) % S], kb_begin + k + u + AHEAD);
      if (!PAIRED || (u & 1)) wait_and_barrier<YOUNGER>();
    }
  }
#pragma unroll
  for (int u = 0; u < S - 1; ++u) {  // up to S - 1 blocks left, in stages 0 ..
    if (k + u < nkb) {
      k_step<BM, BN>(s, u_stage[u], acc, u_stage[(u + AHEAD) % S], kb_begin + k + u + AHEAD);
      if ((!PAIRED || (u & 1)) && k + u + 1 < nkb) wait_and_barrier<YOUNGER>();
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // stray refetches must not outlive the workgroup's LDS

  // ---- epilogue: lane holds, for token m = 16 j + l16 of the wave's rows, channels 16 i + 4 q + (0..3) of its columns
  const bool vec_ok = ((p.ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
  const bool raw = p.out_dtype == MI355_I32;
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int m = m0 + wave_m * WM + j * 16 + l16;
    if (m >= p.M) continue;
    float sa_m = 1.f;
    if constexpr (!SPLIT) {
      if (!raw) sa_m = p.sa[m];
    }
#pragma unroll
    for (int i = 0; i < U_NT; ++i) {
      {
        const int n = n0 + wave_n * U_WN + i * 16 + 4 * q;
        if (n >= p.N) continue;
        const int nvalid = min(4, p.N - n);
        if constexpr (SPLIT) {
          int* wsp = reinterpret_cast<int*>(p.ws) + ((int64_t)tc.split * p.M + m) * p.N + n;
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (v < nvalid) wsp[v] = acc[i][j][v];
        } else if (raw) {
          int* o = reinterpret_cast<int*>(p.out) + (int64_t)m * p.ldo + n;
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (v < nvalid) o[v] = acc[i][j][v];
        } else {
          float r[4];
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int nn = min(n + v, p.N - 1);
            float t = mul_rn((float)acc[i][j][v], mul_rn(p.sb[nn], sa_m));
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

template <int BM, int BN>
int launch_bm(GemmParams& p, hipStream_t stream, const char* what) {
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n * p.splits));
  if (BM + BN == 192 && (int64_t)p.tiles_m * p.tiles_n * p.splits > NUM_CUS) {
    if (p.splits > 1) hipLaunchKernelGGL((int8_gemm_dma3_kernel<BM, true, BN, 3>), grid, dim3(U_THREADS), 0, stream, p);
    else hipLaunchKernelGGL((int8_gemm_dma3_kernel<BM, false, BN, 3>), grid, dim3(U_THREADS), 0, stream, p);
  } else {
    constexpr int S = BM + BN == 192 ? 6 : BM + BN == 256 ? 4 : 3;
    if (p.splits > 1) hipLaunchKernelGGL((int8_gemm_dma3_kernel<BM, true, BN, S>), grid, dim3(U_THREADS), 0, stream, p);
    else hipLaunchKernelGGL((int8_gemm_dma3_kernel<BM, false, BN, S>), grid, dim3(U_THREADS), 0, stream, p);
  }
  return check_launch(what);
}

}  // namespace

// Tiling and split are those of the FP8 mid-M kernel (dma3_plan): same tile shapes, same byte model.  The 128 x 256 tile is
// not built here: the two-phase 128-token kernel (gemm_int8_pp128.hip) serves it.
int launch_int8_dma3(GemmParams& p, int bm, int bn, hipStream_t stream, const char* what) {
  if (bn == 128) return bm == 64 ? launch_bm<64, 128>(p, stream, what) : launch_bm<128, 128>(p, stream, what);
  if (bm == 128) return launch_int8_pp128(p, stream, what);
  return launch_bm<64, 256>(p, stream, what);
}

}  // namespace mi355
