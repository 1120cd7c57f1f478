// Blockwise-scaled FP8 GEMM and per-token/per-channel INT8 GEMM for gfx950 (MI355X).
//
// One LDS-staged MFMA skeleton serves both:
//   * 256 threads = 4 waves per workgroup, macro tile BM (tokens) x BN (output channels) x 128 (K bytes);
//   * both operands are K-contiguous bytes; a K step of 128 bytes per row is staged through LDS in a
//     double buffer: global_load_dwordx4 -> registers -> ds_write_b128, the loads for step k+1 are in
//     flight while step k is multiplied;
//   * LDS rows are 128 bytes, the eight 16-byte chunks of a row are XOR-swizzled with (row & 7) so both
//     the cooperative writes and the MFMA operand reads (16 rows x one chunk per ds_read_b128) are free
//     of bank conflicts;
//   * the weight tile is the MFMA "A" operand and the token tile the "B" operand, so a lane's four
//     accumulator registers are four consecutive output channels of ONE token: the per-token scale is a
//     single value per lane and M-tile, and the output store is 4 contiguous elements;
//   * FP8: v_mfma_f32_16x16x128_f8f6f4 consumes exactly one 128-wide scale block, its result is promoted
//     into the fp32 accumulator with one FMA per element: acc += part * (sa[m,kb] * sb[nb,kb])
//     (python/sglang/srt/layers/quantization/fp8_kernel.py:749-758);
//   * INT8: two v_mfma_i32_16x16x64_i8 per K step accumulate exactly in int32; the epilogue is
//     f32(acc) * (sb[n] * sa[m]) + bias (epilogue_per_row_per_col_scale.h:280-303);
//   * small token counts stream the weight once with a split along K: partial tiles go to a caller
//     workspace and a second kernel adds them in a fixed order (deterministic, no atomics);
//   * workgroups are renumbered so that each of the 8 XCDs (own L2) works on a contiguous, M-grouped
//     patch of output tiles.
#include <mutex>

#include "gemm_common.h"

namespace mi355 {
namespace {

// IS_FP8: blockwise-scaled fp8 (fp32 accumulators) or int8 (int32 accumulators).
// BM x BN macro tile, WGM x WGN waves (WGM * WGN == 4).
// ALIGNED: rows of both operands start on 16-byte boundaries and K % 16 == 0, so 16-byte loads are legal.
// SPLIT: write raw partial accumulators to the workspace instead of the epilogue.
template <bool IS_FP8, int BM, int BN, int WGM, int WGN, bool ALIGNED, bool SPLIT>
__global__ __launch_bounds__(THREADS) void gemm_kernel(const GemmParams p) {
  static_assert(WGM * WGN == 4, "four waves per workgroup");
  constexpr int WM = BM / WGM, WN = BN / WGN;
  constexpr int MT = WM / 16, NT = WN / 16;
  static_assert(MT >= 1 && NT >= 1 && 128 % WN == 0, "a wave's channels must lie inside one 128-wide scale block");
  constexpr int ROWS = BM + BN;
  constexpr int LOADS = (ROWS + 31) / 32;  // 16-byte chunks per thread and stage
  constexpr bool LAST_PARTIAL = (ROWS % 32) != 0;  // the last pass covers fewer than 32 rows
  constexpr int STAGE_BYTES = ROWS * KSTEP;
  using AccT = typename std::conditional<IS_FP8, float, int>::type;

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint8_t* tiles = smem;                                                 // [2][ROWS][128]
  float* s_scale = reinterpret_cast<float*>(smem + 2 * STAGE_BYTES);     // [2][BM] (fp8 only)

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave / WGN, wave_n = wave % WGN;
  const int l16 = lane & 15, q = lane >> 4;

  const TileCoord tc = tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n);
  const int tile_m = tc.tile_m, tile_n = tc.tile_n, split = tc.split;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int kb_begin = split * p.kb_per_split;
  const int kb_end = min(p.kb_total, kb_begin + p.kb_per_split);

  // ---- loader set-up: thread owns chunk (tid & 7) of rows (tid >> 3) + 32 * i
  const int chunk = tid & 7;
  const uint8_t* gptr[LOADS];
  uint32_t lds_off[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int row = min((tid >> 3) + 32 * i, ROWS - 1);  // rows < BM are tokens, the rest channels
    if (row < BM) {
      const int m = min(m0 + row, p.M - 1);  // rows past the edge re-read the last valid row; never stored
      gptr[i] = p.a + (int64_t)m * p.lda + chunk * 16;
    } else {
      const int n = min(n0 + row - BM, p.N - 1);
      gptr[i] = p.b + (int64_t)n * p.ldb + chunk * 16;
    }
    lds_off[i] = row * KSTEP + ((chunk ^ (row & 7)) << 4);
  }
  const float* sa_ptr = nullptr;
  if constexpr (IS_FP8) {
    if (tid < BM) sa_ptr = p.sa + (int64_t)min(m0 + tid, p.M - 1) * p.sa_sm;
  }

  u32x4 stage_regs[LOADS];
  float stage_scale = 0.f;

  auto load_global = [&](int kb) {
    const int kbyte = kb * KSTEP + chunk * 16;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const uint8_t* src = gptr[i] + (int64_t)kb * KSTEP;
      if constexpr (ALIGNED) {
        stage_regs[i] = (kbyte < p.K) ? *reinterpret_cast<const u32x4*>(src) : u32x4{0, 0, 0, 0};
      } else {
        // arbitrary K and row strides: byte loads with a bound on every byte
        uint32_t w[4] = {0, 0, 0, 0};
        for (int j = 0; j < 16; ++j)
          if (kbyte + j < p.K) w[j >> 2] |= (uint32_t)src[j] << (8 * (j & 3));
        stage_regs[i] = u32x4{w[0], w[1], w[2], w[3]};
      }
    }
    if constexpr (IS_FP8) {
      if (tid < BM) stage_scale = sa_ptr[(int64_t)kb * p.sa_sk];
    }
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      if (LAST_PARTIAL && i == LOADS - 1 && (tid >> 3) + 32 * i >= ROWS) continue;
      *reinterpret_cast<u32x4*>(tiles + buf * STAGE_BYTES + lds_off[i]) = stage_regs[i];
    }
    if constexpr (IS_FP8) {
      if (tid < BM) s_scale[buf * BM + tid] = stage_scale;
    }
  };

  AccT acc[NT][MT][4];
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0;

  // operand fragment addresses inside a stage (swizzled); constant over K.  Lane quarter q takes the 16-byte
  // chunks q and q + 4 of a row: with this mapping a ds_read_b128 runs at the full 256 B/clk of the gfx950 LDS
  // (chunks 2q, 2q+1 measure at half of that).  Both operands use the same mapping, so the dot product is unchanged.
  uint32_t tok_off[MT][2], ch_off[NT][2];
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int row = wave_m * WM + j * 16 + l16;
#pragma unroll
    for (int h = 0; h < 2; ++h) tok_off[j][h] = row * KSTEP + (((q + 4 * h) ^ (row & 7)) << 4);
  }
#pragma unroll
  for (int i = 0; i < NT; ++i) {
    const int row = BM + wave_n * WN + i * 16 + l16;
#pragma unroll
    for (int h = 0; h < 2; ++h) ch_off[i][h] = row * KSTEP + (((q + 4 * h) ^ (row & 7)) << 4);
  }
  // one 128x128 weight block holds all of this wave's channels
  const int nb = min(n0 + wave_n * WN, p.N - 1) / 128;

  if (kb_begin < kb_end) {
    load_global(kb_begin);
    store_lds(0);
  }
  __syncthreads();

  for (int kb = kb_begin; kb < kb_end; ++kb) {
    const int buf = (kb - kb_begin) & 1;
    const bool more = kb + 1 < kb_end;
    if (more) load_global(kb + 1);

    const uint8_t* st = tiles + buf * STAGE_BYTES;
    u32x4 tok[MT][2];
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      tok[j][0] = *reinterpret_cast<const u32x4*>(st + tok_off[j][0]);
      tok[j][1] = *reinterpret_cast<const u32x4*>(st + tok_off[j][1]);
    }
    if constexpr (IS_FP8) {
      const float sbv = p.sb[(int64_t)nb * p.sb_sn + (int64_t)kb * p.sb_sk];
      float sc[MT];
#pragma unroll
      for (int j = 0; j < MT; ++j) sc[j] = s_scale[buf * BM + wave_m * WM + j * 16 + l16] * sbv;
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        const u32x4 c0 = *reinterpret_cast<const u32x4*>(st + ch_off[i][0]);
        const u32x4 c1 = *reinterpret_cast<const u32x4*>(st + ch_off[i][1]);
        const v8i wfrag = {(int)c0.x, (int)c0.y, (int)c0.z, (int)c0.w, (int)c1.x, (int)c1.y, (int)c1.z, (int)c1.w};
#pragma unroll
        for (int j = 0; j < MT; ++j) {
          const v8i tfrag = {(int)tok[j][0].x, (int)tok[j][0].y, (int)tok[j][0].z, (int)tok[j][0].w,
                             (int)tok[j][1].x, (int)tok[j][1].y, (int)tok[j][1].z, (int)tok[j][1].w};
          const v4f part =
              __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wfrag, tfrag, v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[i][j][v] = fmaf(part[v], sc[j], acc[i][j][v]);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        const u32x4 c0 = *reinterpret_cast<const u32x4*>(st + ch_off[i][0]);
        const u32x4 c1 = *reinterpret_cast<const u32x4*>(st + ch_off[i][1]);
        const v4i w0 = {(int)c0.x, (int)c0.y, (int)c0.z, (int)c0.w};
        const v4i w1 = {(int)c1.x, (int)c1.y, (int)c1.z, (int)c1.w};
#pragma unroll
        for (int j = 0; j < MT; ++j) {
          v4i c = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
          const v4i t0 = {(int)tok[j][0].x, (int)tok[j][0].y, (int)tok[j][0].z, (int)tok[j][0].w};
          const v4i t1 = {(int)tok[j][1].x, (int)tok[j][1].y, (int)tok[j][1].z, (int)tok[j][1].w};
          c = __builtin_amdgcn_mfma_i32_16x16x64_i8(w0, t0, c, 0, 0, 0);
          c = __builtin_amdgcn_mfma_i32_16x16x64_i8(w1, t1, c, 0, 0, 0);
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[i][j][v] = c[v];
        }
      }
    }

    if (more) store_lds(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: lane holds channels n = nbase + 4q .. +3 of token m = mbase + l16
  const bool vec_ok = ((p.ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int m = m0 + wave_m * WM + j * 16 + l16;
    if (m >= p.M) continue;
    float sa_m = 1.f;
    if constexpr (!IS_FP8 && !SPLIT) {
      if (p.out_dtype != MI355_I32) sa_m = p.sa[m];
    }
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const int n = n0 + wave_n * WN + i * 16 + 4 * q;
      if (n >= p.N) continue;
      const int nvalid = min(4, p.N - n);
      if constexpr (SPLIT) {
        AccT* w = reinterpret_cast<AccT*>(p.ws) + ((int64_t)split * p.M + m) * p.N + n;
#pragma unroll
        for (int v = 0; v < 4; ++v)
          if (v < nvalid) w[v] = acc[i][j][v];
      } else if constexpr (IS_FP8) {
        fp8_channel_epilogue(p, n, acc[i][j]);
        store_out4(p.out, p.out_dtype, (int64_t)m * p.ldo + n, acc[i][j], nvalid, vec_ok);
      } else {
        if (p.out_dtype == MI355_I32) {
          int* o = reinterpret_cast<int*>(p.out) + (int64_t)m * p.ldo + n;
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (v < nvalid) o[v] = acc[i][j][v];
        } else {
          float r[4];
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int nn = min(n + v, p.N - 1);
            // separately rounded multiply and add: the contract is mul, mul, add, not a fused multiply-add
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

// Sums the split-K partial tiles in ascending split order and applies the epilogue.  The partial tiles are fetched eight at
// a time before they are added: with one load per addition the kernel is a chain of memory latencies (4.6 us for 7 splits).
constexpr int REDUCE_BATCH = 8;
template <bool IS_FP8>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const GemmParams p) {
  const int64_t total = (int64_t)p.M * p.N;
  const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (idx >= total) return;
  // N % 4 == 0 is required for the split path, so the four elements share a row
  const int m = (int)(idx / p.N);
  const int n = (int)(idx - (int64_t)m * p.N);
  if constexpr (IS_FP8) {
    const float* w = reinterpret_cast<const float*>(p.ws) + idx;
    v4f s = {0.f, 0.f, 0.f, 0.f};  // 0 + first partial is exact, so the sum is the one that starts from the first partial
    for (int k0 = 0; k0 < p.splits; k0 += REDUCE_BATCH) {
      v4f t[REDUCE_BATCH];
#pragma unroll
      for (int j = 0; j < REDUCE_BATCH; ++j)
        t[j] = *reinterpret_cast<const v4f*>(w + (int64_t)min(k0 + j, p.splits - 1) * total);
#pragma unroll
      for (int j = 0; j < REDUCE_BATCH; ++j)
        if (k0 + j < p.splits) s[0] += t[j][0], s[1] += t[j][1], s[2] += t[j][2], s[3] += t[j][3];
    }
    float r[4] = {s[0], s[1], s[2], s[3]};
    fp8_channel_epilogue(p, n, r);
    const bool vec_ok = ((p.ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
    store_out4(p.out, p.out_dtype, (int64_t)m * p.ldo + n, r, 4, vec_ok);
  } else {
    const int* w = reinterpret_cast<const int*>(p.ws) + idx;
    v4i s = {0, 0, 0, 0};
    for (int k0 = 0; k0 < p.splits; k0 += REDUCE_BATCH) {
      v4i t[REDUCE_BATCH];
#pragma unroll
      for (int j = 0; j < REDUCE_BATCH; ++j)
        t[j] = *reinterpret_cast<const v4i*>(w + (int64_t)min(k0 + j, p.splits - 1) * total);
#pragma unroll
      for (int j = 0; j < REDUCE_BATCH; ++j)
        if (k0 + j < p.splits) s[0] += t[j][0], s[1] += t[j][1], s[2] += t[j][2], s[3] += t[j][3];
    }
    if (p.out_dtype == MI355_I32) {
      int* o = reinterpret_cast<int*>(p.out) + (int64_t)m * p.ldo + n;
      for (int v = 0; v < 4; ++v) o[v] = s[v];
      return;
    }
    const float sa_m = p.sa[m];
    float r[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      float t = mul_rn((float)s[v], mul_rn(p.sb[n + v], sa_m));
      if (p.bias) {
        const uint32_t hb = reinterpret_cast<const uint16_t*>(p.bias)[n + v];
        t = add_rn(t, (p.out_dtype == MI355_BF16) ? bf16_bits_to_f32(hb) : f16_bits_to_f32(hb));
      }
      r[v] = t;
    }
    const bool vec_ok = ((p.ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
    store_out4(p.out, p.out_dtype, (int64_t)m * p.ldo + n, r, 4, vec_ok);
  }
}

// ---------------------------------------------------------------------------------------------
struct Plan {
  int bm, bn, splits, kb_per_split;
};

// Tile and split selection.  Large token counts are MFMA-bound and want the biggest tile; small ones
// stream the weight once and want enough workgroups in flight to cover HBM latency.
Plan make_plan(int64_t M, int64_t N, int64_t K) {
  Plan pl;
  pl.bn = 128;
  if (M <= 16) pl.bm = 16;
  else if (M <= 32) pl.bm = 32;
  else if (M <= 64) pl.bm = 64;
  else if (M <= 1024) pl.bm = 128;
  else pl.bm = 256;
  const int64_t kb_total = (K + KSTEP - 1) / KSTEP;
  const int64_t tiles = ((M + pl.bm - 1) / pl.bm) * ((N + pl.bn - 1) / pl.bn);
  int splits = 1;
  if (N % 4 == 0 && tiles < 2 * NUM_CUS) {
    // aim at ~4 workgroups per CU, keep at least 4 K steps per split
    int64_t want = (4 * NUM_CUS + tiles - 1) / tiles;
    int64_t max_by_k = kb_total / 4 > 0 ? kb_total / 4 : 1;
    splits = (int)(want < max_by_k ? want : max_by_k);
    if (splits < 1) splits = 1;
    if (splits > 32) splits = 32;
  }
  pl.kb_per_split = (int)((kb_total + splits - 1) / splits);
  pl.splits = (int)((kb_total + pl.kb_per_split - 1) / pl.kb_per_split);
  if (pl.splits < 1) pl.splits = 1;
  return pl;
}

size_t scale_relayout_bytes(int64_t M, int64_t K);

// Upper bound over the kernels a shape may be routed to (the choice also depends on pointer alignment, which is not
// known here).
size_t workspace_bytes(int64_t M, int64_t N, int64_t K, bool is_fp8) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const Plan pl = make_plan(M, N, K);
  size_t need = pl.splits > 1 ? (size_t)pl.splits * (size_t)M * (size_t)N * 4u : 0;
  if (M > 16 && K % KSTEP == 0) {
    const Dma3Plan dp = dma3_plan(M, N, K, !is_fp8);  // (an upper bound: the dispatcher may still pick another kernel)
    const size_t dneed = dp.splits > 1 ? (size_t)dp.splits * (size_t)M * (size_t)N * 4u : 0;
    if (dneed > need) need = dneed;
  }
  if (decode_supported(M, N, K)) {
    const int ds = decode_splits(M, N, K);
    const size_t dneed = ds > 1 ? (size_t)ds * (size_t)M * (size_t)N * 4u : 0;
    if (dneed > need) need = dneed;
  }
  if (is_fp8 && (M > 16 || (double)M >= route_constants().decode_dma3_min_tokens)) need += scale_relayout_bytes(M, K);  // the direct-to-LDS kernels may have to re-lay the token scales out
  return need;
}

template <bool IS_FP8, int BM, int BN, int WGM, int WGN, bool ALIGNED, bool SPLIT>
int launch_tile_inst(const GemmParams& p, unsigned grid, size_t lds, hipStream_t stream, const char* what) {
  auto kfn = gemm_kernel<IS_FP8, BM, BN, WGM, WGN, ALIGNED, SPLIT>;
  if (lds > 64 * 1024) {
    // more than 64 KB of dynamic LDS has to be granted once per kernel; concurrent first calls may both ask, which is harmless
    static std::once_flag once;
    static hipError_t granted = hipSuccess;
    std::call_once(once, [&] {
      granted = hipFuncSetAttribute(reinterpret_cast<const void*>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    });
    if (granted != hipSuccess) {
      set_error("%s: cannot reserve %zu bytes of LDS: %s", what, lds, hipGetErrorString(granted));
      return MI355_ERR_LAUNCH;
    }
  }
  hipLaunchKernelGGL(kfn, dim3(grid), dim3(THREADS), lds, stream, p);
  return check_launch(what);
}

template <bool IS_FP8, int BM, int BN, int WGM, int WGN>
int launch_tile(GemmParams& p, bool aligned, hipStream_t stream, const char* what) {
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const unsigned grid = (unsigned)(p.tiles_m * p.tiles_n * p.splits);
  const size_t lds = 2 * (size_t)(BM + BN) * KSTEP + (IS_FP8 ? 2 * BM * sizeof(float) : 0);
  const bool split = p.splits > 1;
  if (aligned)
    return split ? launch_tile_inst<IS_FP8, BM, BN, WGM, WGN, true, true>(p, grid, lds, stream, what)
                 : launch_tile_inst<IS_FP8, BM, BN, WGM, WGN, true, false>(p, grid, lds, stream, what);
  return split ? launch_tile_inst<IS_FP8, BM, BN, WGM, WGN, false, true>(p, grid, lds, stream, what)
               : launch_tile_inst<IS_FP8, BM, BN, WGM, WGN, false, false>(p, grid, lds, stream, what);
}

// Which kernel serves a problem, with which tiling.  One function decides for the launcher and for the plan query, so
// what the query reports is what runs.
enum RouteKernel { RK_DECODE = 0, RK_DMA3, RK_PINGPONG, RK_PIPELINED, RK_GENERIC, RK_WAVESPLIT, RK_PP128 };
const char* const ROUTE_NAMES[] = {"decode", "dma3", "pingpong", "pipelined", "generic", "decode_wavesplit", "pingpong128"};

struct Route {
  int kernel;
  int bm, bn;
  int splits, kb_per_split;
  int groups_per_wg;  // decode only
  bool aligned;
};

// Decode sizes: the kernel that splits K over the waves of a workgroup instead of over workgroups, where it was
// measured faster than the streaming kernel (the numbers stand beside the thresholds in route_constants.h).
bool wavesplit_preferred(bool is_fp8, int64_t M, int64_t N, int64_t K) {
  if (!decode_supported(M, N, K)) return true;  // channels in whole 16s but not 128s: the streaming kernel cannot run
  const RouteConstants& rc = route_constants();
  if ((double)(K / KSTEP) < rc.wavesplit_min_kblocks) return false;
  if (!is_fp8) return true;
  if ((double)N * (double)K <= rc.wavesplit_small_weight_bytes) return N / 16 >= NUM_CUS || (double)M <= rc.wavesplit_small_weight_max_tokens;
  if (!wavesplit_two_tiles(true, M, N, K)) return (double)M <= rc.wavesplit_large_weight_max_tokens;
  return (double)M <= ((double)(K / KSTEP) > rc.wavesplit_two_tile_long_k_blocks ? rc.wavesplit_long_k_max_tokens : rc.wavesplit_two_tile_max_tokens);
}

// The mid-M kernel at decode sizes: the channel tile that gives the most unsplit 64-token tiles in one round (at most one per
// CU, at least the measured minimum), 0 if none does.
int decode_dma3_channel_tile(bool is_fp8, int64_t N) {
  const RouteConstants& rc = route_constants();
  const double min_workgroups = is_fp8 ? rc.decode_dma3_min_workgroups : rc.decode_dma3_int8_min_workgroups;
  int bn = 0;
  int64_t most = 0;
  for (int c = 256; c >= 128; c -= is_fp8 ? 64 : 128) {
    const int64_t tiles = (N + c - 1) / c;
    if ((double)tiles >= min_workgroups && tiles <= NUM_CUS && tiles > most) most = tiles, bn = c;
  }
  return bn;
}

// `aligned`: both operand base pointers and row strides are multiples of 16 bytes and K % 16 == 0.
// `fused_quant`: the tokens arrive unquantized and the kernel is to quantize them itself, which only the streaming
// decode kernel can.
Route choose_route(bool is_fp8, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, bool aligned, bool fused_quant = false) {
  Route r{};
  r.aligned = aligned;
  const bool small_b = N * ldb < (1ll << 32);                 // kernels that address rows by 32-bit byte offsets
  const bool small_offsets = M * lda < (1ll << 32) && small_b;
  const bool to_wavesplit = !fused_quant && wavesplit_supported(M, N, K) && aligned && small_b && wavesplit_preferred(is_fp8, M, N, K);
  if (!fused_quant && M <= 16 && K % KSTEP == 0 && aligned && small_offsets) {
    // decode sizes on the mid-M kernel (one 64-token tile, K unsplit) where that fills the chip in one round.  FP8: instead
    // of the streaming kernel whenever that one would split K, instead of the wave-split kernel with 192-channel tiles and
    // long K.  INT8: from a dozen tokens on.
    const RouteConstants& rc = route_constants();
    const bool long_k = (double)(K / KSTEP) > rc.decode_dma3_wavesplit_min_kblocks;
    if ((double)M >= (is_fp8 ? rc.decode_dma3_min_tokens : long_k ? rc.decode_dma3_int8_long_k_min_tokens : rc.decode_dma3_int8_min_tokens)) {
      const int bn = decode_dma3_channel_tile(is_fp8, N);
      const bool instead = !is_fp8 ? true
                           : to_wavesplit ? (bn == 192 && (double)(K / KSTEP) > rc.decode_dma3_wavesplit_min_kblocks)
                                          : (decode_supported(M, N, K) && decode_splits(M, N, K) > 1);
      if (instead && bn != 0) {
        r.kernel = RK_DMA3, r.bm = 64, r.bn = bn, r.splits = 1, r.kb_per_split = (int)(K / KSTEP);
        return r;
      }
    }
  }
  if (to_wavesplit) {
    const WavesplitShape ws = wavesplit_shape(K);
    r.kernel = RK_WAVESPLIT, r.bm = 16, r.bn = wavesplit_two_tiles(is_fp8, M, N, K) ? 32 : 16, r.splits = 1;
    r.kb_per_split = (int)((K + KSTEP - 1) / KSTEP);
    r.groups_per_wg = ws.waves;  // waves that share a workgroup's K
    return r;
  }
  if (decode_supported(M, N, K) && aligned && small_b) {  // barrier-free weight streaming
    r.kernel = RK_DECODE, r.bm = 16, r.bn = 128;
    r.splits = decode_splits(M, N, K);
    r.kb_per_split = decode_kb_per_range();
    r.groups_per_wg = decode_groups_per_wg(N, r.splits);
    return r;
  }
  const int64_t tiles_256 = ((M + 255) / 256) * ((N + 255) / 256);
  if (M > 16 && (M <= 1024 || tiles_256 < NUM_CUS) && K % KSTEP == 0 && aligned && small_offsets) {
    // mid-M, or many tokens but too few channels for 256 x 256 tiles: three-stage direct-to-LDS kernel with 64- or 128-token
    // tiles, when its tiling fills the chip well enough
    // It beats the generic kernel for every layer measured (K=1536..18432 -> N=576..28672 at 24..4096 tokens: e.g. 9 against
    // 25 us for K=2048 -> N=7168 at 128 tokens, 23 against 68 us for K=7168 -> N=576 at 2048), its 64 x 128 tiles and K
    // splits filling the chip where the channels alone do not; without splits (N not a multiple of 4) the older
    // chip-filling score decides.
    const Dma3Plan dp = dma3_plan(M, N, K, !is_fp8);
    // Above 128 tokens the two-phase 256 x 256 kernel competes: a round of its tiles takes (K blocks) x 1.39 us + 11 us
    // (INT8: 1.46 us per block), whatever part of the tile is filled and however many CUs the round uses, so it wins
    // where the channels alone give it a round's worth of tiles (measured: K=7168 -> N=36864 at M=256: 89 against 141 us,
    // M=1024: 260 against 308 us; INT8 K=4096 -> N=28672 at M=512: 59 against 94 us) and loses for few channels.
    if (M > 128) {
      const RouteConstants& rc = route_constants();
      const double pp_us = (double)((tiles_256 + NUM_CUS - 1) / NUM_CUS) * ((double)(K / KSTEP) * (is_fp8 ? rc.pp_fp8_us_per_kblock : rc.pp_int8_us_per_kblock) + rc.pp_us_per_tile);
      if (pp_us < dp.time_us) {
        r.kernel = RK_PINGPONG, r.bm = 256, r.bn = 256, r.splits = 1, r.kb_per_split = (int)(K / KSTEP);
        return r;
      }
    }
    if (N % 4 == 0 || dp.efficiency >= route_constants().dma3_min_efficiency) {
      // INT8: the 128 x 256 tile of this family is the two-phase 128-token kernel (gemm_int8_pp128.hip)
      r.kernel = (!is_fp8 && dp.bm == 128 && dp.bn == 256) ? RK_PP128 : RK_DMA3;
      r.bm = dp.bm, r.bn = dp.bn, r.splits = dp.splits, r.kb_per_split = dp.kb_per_split;
      return r;
    }
  }
  const Plan pl = make_plan(M, N, K);
  r.kernel = RK_GENERIC, r.bm = pl.bm, r.bn = pl.bn, r.splits = pl.splits, r.kb_per_split = pl.kb_per_split;
  const int64_t tiles_128 = ((M + 255) / 256) * ((N + 127) / 128);
  if (pl.bm == 256 && pl.splits == 1 && aligned && small_offsets) {
    if (is_fp8) {
      // 256 x 256 tiles (8 waves in two alternating groups) when they still give every CU a workgroup, else 256 x 128
      if (tiles_256 >= NUM_CUS) {
        r.kernel = RK_PINGPONG, r.bn = 256;
        return r;
      }
      if (tiles_128 >= NUM_CUS) {
        r.kernel = RK_PIPELINED;
        return r;
      }
    } else if (K % KSTEP == 0 && tiles_256 >= NUM_CUS / 2) {
      r.kernel = RK_PINGPONG, r.bn = 256;
      return r;
    }
  }
  if (r.bm == 256 && tiles_128 < NUM_CUS) r.bm = 128;  // too few 256-row tiles to fill the chip
  return r;
}

// out[kb * ld_out + m] = sa[m * sa_sm + kb * sa_sk]: token scales re-laid out M-major with a row pitch that is a multiple
// of four floats.  One 32 x 32 tile per workgroup through LDS, so that reads and writes are both contiguous for either
// input layout.
__global__ __launch_bounds__(256) void relayout_scales_kernel(const float* sa, int64_t sa_sm, int64_t sa_sk, float* out,
                                                              int64_t ld_out, int M, int KB) {
  __shared__ float tile[32][33];
  const int m0 = blockIdx.x * 32, k0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  const bool k_fast = sa_sk < sa_sm;                       // which index is contiguous in the input
#pragma unroll
  for (int r = ty; r < 32; r += 8) {
    const int m = k_fast ? m0 + r : m0 + tx, kb = k_fast ? k0 + tx : k0 + r;
    if (m < M && kb < KB) tile[kb - k0][m - m0] = sa[(int64_t)m * sa_sm + (int64_t)kb * sa_sk];
  }
  __syncthreads();
#pragma unroll
  for (int r = ty; r < 32; r += 8) {
    const int m = m0 + tx, kb = k0 + r;
    if (m < M && kb < KB) out[(int64_t)kb * ld_out + m] = tile[r][tx];
  }
}


// The direct-to-LDS kernels (two-phase large-M, three-stage mid-M) read token scales M-major with 16-byte loads.  Scales
// that are not laid out that way (K-major, as per_token_group_quant_fp8 returns them by default; a pitch or base that is
// not a multiple of 16 bytes) are first copied into the head of the workspace.
size_t scale_relayout_bytes(int64_t M, int64_t K) {
  const size_t b = (size_t)((M + 3) & ~3ll) * (size_t)((K + KSTEP - 1) / KSTEP) * 4u;
  return (b + 255) & ~(size_t)255;  // what follows in the workspace stays 256-byte aligned
}
bool fp8_scales_conform(const GemmParams& p) {
  return p.sa_sm == 1 && (p.sa_sk & 3) == 0 && p.sa_sk >= ((p.M + 3) & ~3) && (reinterpret_cast<uintptr_t>(p.sa) & 15) == 0;
}
bool route_wants_m_major_scales(bool is_fp8, const Route& r) {
  return is_fp8 && (r.kernel == RK_PINGPONG || r.kernel == RK_DMA3);
}

// Workspace bytes the chosen route needs for this call: a re-laid-out copy of the token scales (first) and split-K
// partial sums (after it).
size_t route_workspace_need(bool is_fp8, const Route& r, const GemmParams& p) {
  size_t need = r.splits > 1 ? (size_t)r.splits * (size_t)p.M * (size_t)p.N * 4u : 0;
  if (!p.ue8m0 && route_wants_m_major_scales(is_fp8, r) && !fp8_scales_conform(p)) need += scale_relayout_bytes(p.M, p.K);
  return need;
}

bool operands_aligned(const GemmParams& p) {
  return (p.K % 16 == 0) && (p.lda % 16 == 0) && (p.ldb % 16 == 0) && ((reinterpret_cast<uintptr_t>(p.a) & 15) == 0) &&
         ((reinterpret_cast<uintptr_t>(p.b) & 15) == 0);
}

template <bool IS_FP8>
int run_gemm(GemmParams& p, void* workspace, size_t workspace_bytes_given, hipStream_t stream, const char* what) {
  p.kb_total = (p.K + KSTEP - 1) / KSTEP;
  const bool aligned = operands_aligned(p);
  const Route r = choose_route(IS_FP8, p.M, p.N, p.K, p.lda, p.ldb, aligned, p.x16 != nullptr);
  p.splits = r.splits;
  p.kb_per_split = r.kb_per_split;
  const size_t need = route_workspace_need(IS_FP8, r, p);
  if (need > 0) {
    MI355_REQUIRE(workspace != nullptr && workspace_bytes_given >= need, MI355_ERR_WORKSPACE,
                  "%s: needs a workspace of %zu bytes, got %zu", what, need, workspace_bytes_given);
    MI355_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15) == 0, MI355_ERR_WORKSPACE,
                  "%s: workspace must be 16-byte aligned", what);
    p.ws = workspace;
  }
  if (!p.ue8m0 && route_wants_m_major_scales(IS_FP8, r) && !fp8_scales_conform(p)) {
    float* dst = static_cast<float*>(workspace);
    const int64_t ld = (p.M + 3) & ~3;
    hipLaunchKernelGGL(relayout_scales_kernel, dim3((unsigned)((p.M + 31) / 32), (unsigned)((p.kb_total + 31) / 32)), dim3(256), 0,
                       stream, p.sa, p.sa_sm, p.sa_sk, dst, ld, p.M, p.kb_total);
    const int rc0 = check_launch(what);
    if (rc0 != MI355_OK) return rc0;
    p.sa = dst, p.sa_sm = 1, p.sa_sk = ld;
    p.ws = static_cast<uint8_t*>(workspace) + scale_relayout_bytes(p.M, p.K);
  }
  int rc;
  switch (r.kernel) {
    case RK_DECODE:
      rc = IS_FP8 ? launch_fp8_decode(p, r.groups_per_wg, stream, what) : launch_int8_decode(p, r.groups_per_wg, stream, what);
      break;
    case RK_WAVESPLIT: return IS_FP8 ? launch_fp8_wavesplit(p, stream, what) : launch_int8_wavesplit(p, stream, what);
    case RK_PP128:
      if constexpr (IS_FP8) {
        set_error("%s: the 128-token two-phase kernel is built for INT8", what);
        return MI355_ERR_UNSUPPORTED;
      } else {
        rc = launch_int8_pp128(p, stream, what);
      }
      break;
    case RK_DMA3:
      if constexpr (IS_FP8) rc = p.ue8m0 ? launch_fp8_dma3_ue8m0(p, r.bm, r.bn, stream, what) : launch_fp8_dma3(p, r.bm, r.bn, stream, what);
      else rc = launch_int8_dma3(p, r.bm, r.bn, stream, what);
      break;
    case RK_PINGPONG: return IS_FP8 ? launch_fp8_pp(p, stream, what) : launch_int8_pp(p, stream, what);
    case RK_PIPELINED: return launch_fp8_pipelined(p, stream, what);
    default:
      // the generic kernel runs its own ordered reduce
      switch (r.bm) {
        case 16: rc = launch_tile<IS_FP8, 16, 128, 1, 4>(p, aligned, stream, what); break;
        case 32: rc = launch_tile<IS_FP8, 32, 128, 1, 4>(p, aligned, stream, what); break;
        case 64: rc = launch_tile<IS_FP8, 64, 128, 1, 4>(p, aligned, stream, what); break;
        case 128: rc = launch_tile<IS_FP8, 128, 128, 2, 2>(p, aligned, stream, what); break;
        default: rc = launch_tile<IS_FP8, 256, 128, 2, 2>(p, aligned, stream, what); break;
      }
  }
  if (rc != MI355_OK || p.splits == 1) return rc;
  const int64_t quads = ((int64_t)p.M * p.N + 3) / 4;
  hipLaunchKernelGGL(splitk_reduce_kernel<IS_FP8>, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, stream, p);
  return check_launch(what);
}

// ---- the constants table: defaults, the per-thread override of a perturbed plan query, names
const RouteConstants g_route_defaults{};
thread_local const RouteConstants* g_route_override = nullptr;
const char* const ROUTE_CONSTANT_NAMES[ROUTE_CONSTANT_COUNT] = {
    "pp_fp8_us_per_kblock", "pp_int8_us_per_kblock", "pp_us_per_tile", "dma3_hbm_bytes_per_us",
    "dma3_tile_us[fp8][128x256]", "dma3_tile_us[fp8][64x256]", "dma3_tile_us[fp8][128x128]", "dma3_tile_us[fp8][64x128]",
    "dma3_tile_us[fp8][128x192]", "dma3_tile_us[fp8][64x192]",
    "dma3_tile_us[int8][128x256]", "dma3_tile_us[int8][64x256]", "dma3_tile_us[int8][128x128]", "dma3_tile_us[int8][64x128]",
    "dma3_tile_us[int8][unused]", "dma3_tile_us[int8][unused2]",
    "dma3_latency_us[fp8][128x256]", "dma3_latency_us[fp8][64x256]", "dma3_latency_us[fp8][128x128]", "dma3_latency_us[fp8][64x128]",
    "dma3_latency_us[fp8][128x192]", "dma3_latency_us[fp8][64x192]",
    "dma3_latency_us[int8][128x256]", "dma3_latency_us[int8][64x256]", "dma3_latency_us[int8][128x128]", "dma3_latency_us[int8][64x128]",
    "dma3_latency_us[int8][unused]", "dma3_latency_us[int8][unused2]",
    "dma3_busy_chip_factor", "dma3_long_row_factor", "dma3_split_fixed_us", "dma3_split_per_split_us", "dma3_min_efficiency",
    "dma3_small_tile_factor", "wavesplit_min_kblocks", "wavesplit_small_weight_bytes", "wavesplit_small_weight_max_tokens",
    "wavesplit_large_weight_max_tokens", "wavesplit_two_tile_min_workgroups", "wavesplit_two_tile_min_tokens",
    "wavesplit_two_tile_long_k_blocks", "wavesplit_two_tile_max_tokens", "wavesplit_long_k_max_tokens",
    "decode_dma3_min_tokens", "decode_dma3_wavesplit_min_kblocks", "decode_dma3_int8_long_k_min_tokens", "decode_dma3_int8_min_tokens",
    "decode_dma3_int8_min_workgroups",
    "decode_dma3_min_workgroups",
    "linear_producer_min_decode_splits", "fused_quant_long_k_blocks", "fused_quant_short_k_blocks", "fused_quant_short_k_max_tokens"};

// LDS stages of the mid-M kernel's pipeline for this plan (0 for the other kernels, whose depth is fixed).
int route_stages(bool is_fp8, const Route& r, int64_t M, int64_t N) {
  if (r.kernel != RK_DMA3) return 0;
  const int64_t workgroups = ((M + r.bm - 1) / r.bm) * ((N + r.bn - 1) / r.bn) * r.splits;
  return dma3_stages(r.bm, r.bn, workgroups);  // the INT8 kernel of the same structure follows the same rule
}

int describe_route(bool is_fp8, int64_t M, int64_t N, int64_t K, int aligned, char* buf, size_t buf_len, const char* what) {
  clear_error();
  MI355_REQUIRE(buf != nullptr && buf_len > 0, MI355_ERR_INVALID_ARGUMENT, "%s: no buffer", what);
  MI355_REQUIRE(M > 0 && N > 0 && K > 0 && M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31),
                MI355_ERR_INVALID_ARGUMENT, "%s: shape out of range", what);
  const Route r = choose_route(is_fp8, M, N, K, K, K, aligned != 0 && K % 16 == 0);
  const int n = snprintf(buf, buf_len, "kernel=%s bm=%d bn=%d splits=%d kb_per_split=%d groups_per_wg=%d aligned=%d stages=%d",
                         ROUTE_NAMES[r.kernel], r.bm, r.bn, r.splits, r.kb_per_split, r.groups_per_wg, (int)r.aligned,
                         route_stages(is_fp8, r, M, N));
  MI355_REQUIRE(n > 0 && (size_t)n < buf_len, MI355_ERR_INVALID_ARGUMENT, "%s: buffer of %zu bytes is too small", what,
                buf_len);
  return MI355_OK;
}

}  // namespace

const RouteConstants& route_constants() { return g_route_override ? *g_route_override : g_route_defaults; }
const char* route_constant_name(int index) {
  return index >= 0 && index < ROUTE_CONSTANT_COUNT ? ROUTE_CONSTANT_NAMES[index] : nullptr;
}
}  // namespace mi355

using namespace mi355;

extern "C" int mi355_route_constant_count(void) { return ROUTE_CONSTANT_COUNT; }
extern "C" const char* mi355_route_constant_name(int index) { return route_constant_name(index); }
extern "C" double mi355_route_constant_value(int index) {
  return index >= 0 && index < ROUTE_CONSTANT_COUNT ? reinterpret_cast<const double*>(&g_route_defaults)[index] : 0.0;
}
extern "C" int mi355_gemm_plan_perturbed(int is_fp8, int64_t M, int64_t N, int64_t K, int aligned, int constant_index, double factor,
                                         char* buf, size_t buf_len) {
  const char* what = "mi355_gemm_plan_perturbed";
  clear_error();
  MI355_REQUIRE(constant_index >= 0 && constant_index < ROUTE_CONSTANT_COUNT && factor > 0.0, MI355_ERR_INVALID_ARGUMENT,
                "%s: constant index 0..%d and a positive factor", what, ROUTE_CONSTANT_COUNT - 1);
  RouteConstants rc = g_route_defaults;
  reinterpret_cast<double*>(&rc)[constant_index] *= factor;
  g_route_override = &rc;
  const int status = describe_route(is_fp8 != 0, M, N, K, aligned, buf, buf_len, what);
  g_route_override = nullptr;
  return status;
}

extern "C" size_t mi355_fp8_blockwise_mm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  return workspace_bytes(M, N, K, true);
}

namespace {

// Argument checks and parameter block shared by the two FP8 entry points.  Returns MI355_OK with `empty` set when there
// is nothing to do.
int fp8_mm_params(const char* what, const void* a, const void* b, const float* sa, const float* sb, void* out,
                  int out_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t sa_sm, int64_t sa_sk,
                  int64_t sb_sn, int64_t sb_sk, int64_t ldo, GemmParams& p, bool& empty) {
  clear_error();
  empty = false;
  MI355_REQUIRE(M >= 0 && N >= 0 && K >= 0, MI355_ERR_INVALID_ARGUMENT, "%s: negative shape", what);
  MI355_REQUIRE(out_dtype == MI355_BF16 || out_dtype == MI355_F16 || out_dtype == MI355_F32,
                MI355_ERR_INVALID_ARGUMENT, "%s: out_dtype must be bfloat16, float16 or float32", what);
  if (M == 0 || N == 0) {
    empty = true;
    return MI355_OK;
  }
  MI355_REQUIRE(K > 0, MI355_ERR_INVALID_ARGUMENT, "%s: K must be positive", what);
  MI355_REQUIRE(a && b && sa && sb && out, MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  MI355_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), MI355_ERR_INVALID_ARGUMENT,
                "%s: dimensions must fit in 31 bits", what);
  MI355_REQUIRE(lda >= K && ldb >= K && ldo >= N, MI355_ERR_INVALID_ARGUMENT,
                "%s: row strides smaller than the row length", what);
  p = GemmParams{};
  p.a = static_cast<const uint8_t*>(a);
  p.b = static_cast<const uint8_t*>(b);
  p.sa = sa, p.sb = sb, p.bias = nullptr, p.out = out, p.ws = nullptr;
  p.M = (int)M, p.N = (int)N, p.K = (int)K;
  p.lda = lda, p.ldb = ldb, p.ldo = ldo;
  p.sa_sm = sa_sm, p.sa_sk = sa_sk, p.sb_sn = sb_sn, p.sb_sk = sb_sk;
  p.out_dtype = out_dtype;
  return MI355_OK;
}

// ---- scratch of the entry point that allocates nothing.  One array per GPU (every device that loads this code object
// holds its own copy at its own address); the name below is only a host-side handle, the device address comes from
// hipGetSymbolAddress, once per device, and is what kernels and host calls are given.
constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)MI355_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) uint8_t scratch[NOALLOC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
std::mutex symbol_mutex;
void* scratch_ptr[MAX_DEVICES];     // guarded by symbol_mutex
void* unit_scale_ptr[MAX_DEVICES];  // guarded by symbol_mutex

// A weight-block scale of one for the per-token x per-channel FP8 GEMM, which runs on the blockwise kernels: every block
// reads this same float (strides 0).
static __device__ __align__(16) float unit_scale[4] = {1.0f, 1.0f, 1.0f, 1.0f};

// Device addresses of the two arrays above on the current device, looked up on first use (or by mi355_qlinear_init) and
// kept.  The first lookup on a device may make the runtime load the code object, which allocates: it is refused while
// `stream` is being captured into a graph, where the caller is told to initialise the device before the capture.
int symbols_of_current_device(void** scratch_out, const float** unit_out, hipStream_t stream, bool check_capture, const char* what) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    set_error("%s: cannot identify the current device (%s, device %d)", what, hipGetErrorString(e), dev);
    return MI355_ERR_LAUNCH;
  }
  std::lock_guard<std::mutex> lock(symbol_mutex);
  if (scratch_ptr[dev] == nullptr || unit_scale_ptr[dev] == nullptr) {
    if (check_capture) {
      hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
      e = hipStreamIsCapturing(stream, &capturing);
      if (e != hipSuccess || capturing != hipStreamCaptureStatusNone) {
        set_error("%s: device %d is not initialised and the stream is being captured: call mi355_qlinear_init() on this device "
                  "before the capture (%s)", what, dev, hipGetErrorString(e));
        return MI355_ERR_LAUNCH;
      }
    }
    void *p = nullptr, *q = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e == hipSuccess) e = hipGetSymbolAddress(&q, HIP_SYMBOL(unit_scale));
    if (e != hipSuccess || p == nullptr || q == nullptr) {
      set_error("%s: cannot resolve the library's device arrays on device %d: %s", what, dev, hipGetErrorString(e));
      return MI355_ERR_LAUNCH;
    }
    scratch_ptr[dev] = p, unit_scale_ptr[dev] = q;
  }
  if (scratch_out) *scratch_out = scratch_ptr[dev];
  if (unit_out) *unit_out = static_cast<const float*>(unit_scale_ptr[dev]);
  return MI355_OK;
}

}  // namespace

extern "C" int mi355_fp8_blockwise_mm(const void* a, const void* b, const float* sa, const float* sb, void* out,
                                      int out_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                                      int64_t sa_sm, int64_t sa_sk, int64_t sb_sn, int64_t sb_sk, int64_t ldo,
                                      void* workspace, size_t workspace_bytes_given, void* stream) {
  const char* what = "mi355_fp8_blockwise_mm";
  GemmParams p;
  bool empty;
  const int rc = fp8_mm_params(what, a, b, sa, sb, out, out_dtype, M, N, K, lda, ldb, sa_sm, sa_sk, sb_sn, sb_sk, ldo, p, empty);
  if (rc != MI355_OK || empty) return rc;
  return run_gemm<true>(p, workspace, workspace_bytes_given, static_cast<hipStream_t>(stream), what);
}

namespace {

// Packed exponents as fp32 scales 2^(byte - 127), for the kernels that take those; byte kb & 3 of word kb >> 2 belongs to
// K block kb.  Byte 0 is 2^-127 (a subnormal float), byte 255 NaN.  One launch for both operands:
//   tokens   sa_out[kb * ldm + m]  from sa_words[(kb >> 2) * sa_kw + m]                  (threads 0 .. M * KB - 1)
//   weights  sb_out[nb * KB + kb]  from sb_words[(kb >> 2) * sb_kw + 128 * nb * sb_row]  (the block's first row; the rest)
__device__ __forceinline__ float ue8m0_to_f32(uint32_t word, int kb) {
  const uint32_t byte = (word >> ((kb & 3) * 8)) & 0xffu;
  return __uint_as_float(byte == 0 ? 0x00400000u : (byte == 255 ? 0x7fc00000u : byte << 23));
}
__global__ __launch_bounds__(256) void unpack_ue8m0_kernel(const uint32_t* sa_words, int64_t sa_kw, float* sa_out, int64_t ldm,
                                                           int M, const uint32_t* sb_words, int64_t sb_row, int64_t sb_kw,
                                                           float* sb_out, int NB, int KB) {
  int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t n_tok = (int64_t)M * KB;
  if (idx < n_tok) {
    // consecutive threads walk tokens: the words are contiguous over tokens, and so is the M-major output
    const int kb = (int)(idx / M), m = (int)(idx - (int64_t)kb * M);
    sa_out[(int64_t)kb * ldm + m] = ue8m0_to_f32(sa_words[(int64_t)(kb >> 2) * sa_kw + m], kb);
    return;
  }
  idx -= n_tok;
  if (idx >= (int64_t)NB * KB) return;
  const int nb = (int)(idx / KB), kb = (int)(idx - (int64_t)nb * KB);
  sb_out[idx] = ue8m0_to_f32(sb_words[(int64_t)(kb >> 2) * sb_kw + (int64_t)nb * 128 * sb_row], kb);
}

size_t ue8m0_unpacked_bytes(int64_t M, int64_t N, int64_t K) {
  const int64_t kb = (K + KSTEP - 1) / KSTEP;
  const size_t b = ((size_t)((M + 3) & ~3ll) * (size_t)kb + (size_t)((N + 127) / 128) * (size_t)kb) * 4u;
  return (b + 255) & ~(size_t)255;
}

}  // namespace

extern "C" size_t mi355_fp8_blockwise_mm_ue8m0_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  return ue8m0_unpacked_bytes(M, N, K) + workspace_bytes(M, N, K, true);
}

extern "C" int mi355_fp8_blockwise_mm_ue8m0(const void* a, const void* b, const void* sa_words, const void* sb_words,
                                            const void* bias, void* out, int out_dtype, int64_t M, int64_t N, int64_t K, int64_t lda,
                                            int64_t ldb, int64_t sa_sk, int64_t sb_sn, int64_t sb_sk, int64_t ldo,
                                            void* workspace, size_t workspace_bytes_given, void* stream) {
  const char* what = "mi355_fp8_blockwise_mm_ue8m0";
  GemmParams p;
  bool empty;
  // strides of the packed words stand in for the fp32 scale strides of the shared argument check
  int rc = fp8_mm_params(what, a, b, static_cast<const float*>(sa_words), static_cast<const float*>(sb_words), out, out_dtype, M,
                         N, K, lda, ldb, 1, sa_sk, sb_sn, sb_sk, ldo, p, empty);
  if (rc != MI355_OK || empty) return rc;
  MI355_REQUIRE(((reinterpret_cast<uintptr_t>(sa_words) | reinterpret_cast<uintptr_t>(sb_words)) & 3) == 0,
                MI355_ERR_INVALID_ARGUMENT, "%s: scale words must be 4-byte aligned", what);
  MI355_REQUIRE(bias == nullptr || out_dtype != MI355_F32, MI355_ERR_INVALID_ARGUMENT,
                "%s: a bias needs a 16-bit output type (it has the output's type)", what);
  p.bias = bias;
  hipStream_t st = static_cast<hipStream_t>(stream);
  p.kb_total = (p.K + KSTEP - 1) / KSTEP;
  const Route r = choose_route(true, p.M, p.N, p.K, p.lda, p.ldb, operands_aligned(p));
  const bool words_conform = (sa_sk & 3) == 0 && sa_sk >= ((M + 3) & ~3ll) && (reinterpret_cast<uintptr_t>(sa_words) & 15) == 0;
  if (r.kernel == RK_PINGPONG && K % KSTEP == 0 && words_conform) {
    // the MFMA applies both exponents itself: no scale arithmetic at all
    p.splits = 1, p.kb_per_split = p.kb_total;
    return launch_fp8_pp_ue8m0(p, st, what);
  }
  if (r.kernel == RK_WAVESPLIT && K % KSTEP == 0) {
    // decode sizes on the wave-split kernel: the same, one launch, no workspace
    return launch_fp8_wavesplit_ue8m0(p, st, what);
  }
  if ((r.kernel == RK_DMA3 && K % KSTEP == 0 && words_conform) || r.kernel == RK_DECODE) {
    // mid-M and streaming decode: the same kernels with the exponents applied by the MFMA; the workspace only holds
    // split-K partial sums (the decode kernel reads the words with ordinary loads: any pitch will do)
    p.ue8m0 = 1;
    return run_gemm<true>(p, workspace, workspace_bytes_given, st, what);
  }
  // every other shape: exponents to fp32 scales in the head of the workspace (tokens M-major, weights one row per
  // 128-channel block, read from the block's first channel), then the fp32-scale kernels
  const size_t head = ue8m0_unpacked_bytes(M, N, K);
  MI355_REQUIRE(workspace != nullptr && workspace_bytes_given >= head, MI355_ERR_WORKSPACE,
                "%s: needs a workspace of at least %zu bytes, got %zu", what, head, workspace_bytes_given);
  MI355_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15) == 0, MI355_ERR_WORKSPACE, "%s: workspace must be 16-byte aligned", what);
  const int KB = p.kb_total;
  const int64_t ldm = (M + 3) & ~3ll;
  const int NB = (int)((N + 127) / 128);
  float* sa_f = static_cast<float*>(workspace);
  float* sb_f = sa_f + ldm * KB;
  hipLaunchKernelGGL(unpack_ue8m0_kernel, dim3((unsigned)(((int64_t)(M + NB) * KB + 255) / 256)), dim3(256), 0, st,
                     static_cast<const uint32_t*>(sa_words), sa_sk, sa_f, ldm, (int)M, static_cast<const uint32_t*>(sb_words), sb_sn,
                     sb_sk, sb_f, NB, KB);
  rc = check_launch(what);
  if (rc != MI355_OK) return rc;
  p.sa = sa_f, p.sa_sm = 1, p.sa_sk = ldm;
  p.sb = sb_f, p.sb_sn = KB, p.sb_sk = 1;
  return run_gemm<true>(p, static_cast<uint8_t*>(workspace) + head, workspace_bytes_given - head, st, what);
}

extern "C" int mi355_fp8_blockwise_mm_kloop_ceiling(const void* a, const void* b, const float* sa, const float* sb, void* out,
                                                    int out_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                                                    int64_t sa_sm, int64_t sa_sk, int64_t sb_sn, int64_t sb_sk, int64_t ldo,
                                                    void* stream) {
  const char* what = "mi355_fp8_blockwise_mm_kloop_ceiling";
  GemmParams p;
  bool empty;
  const int rc = fp8_mm_params(what, a, b, sa, sb, out, out_dtype, M, N, K, lda, ldb, sa_sm, sa_sk, sb_sn, sb_sk, ldo, p, empty);
  if (rc != MI355_OK || empty) return rc;
  p.kb_total = (p.K + KSTEP - 1) / KSTEP;
  const Route r = choose_route(true, p.M, p.N, p.K, p.lda, p.ldb, operands_aligned(p));
  MI355_REQUIRE(r.kernel == RK_PINGPONG && K % KSTEP == 0 && K >= 4 * KSTEP && fp8_scales_conform(p), MI355_ERR_UNSUPPORTED,
                "%s: only for shapes that take the two-phase kernel, K a multiple of 128 and at least 512, token scales M-major "
                "with a pitch that is a multiple of four floats and a 16-byte aligned base", what);
  p.splits = 1, p.kb_per_split = p.kb_total;
  return launch_fp8_pp_noload(p, static_cast<hipStream_t>(stream), what);
}

extern "C" int mi355_fp8_blockwise_mm_noalloc(const void* a, const void* b, const float* sa, const float* sb, void* out,
                                              int out_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                                              int64_t sa_sm, int64_t sa_sk, int64_t sb_sn, int64_t sb_sk, int64_t ldo,
                                              void* stream) {
  const char* what = "mi355_fp8_blockwise_mm_noalloc";
  GemmParams p;
  bool empty;
  int rc = fp8_mm_params(what, a, b, sa, sb, out, out_dtype, M, N, K, lda, ldb, sa_sm, sa_sk, sb_sn, sb_sk, ldo, p, empty);
  if (rc != MI355_OK || empty) return rc;
  // the same plan the launcher will make: how many partial-sum bytes it needs
  const Route r = choose_route(true, p.M, p.N, p.K, p.lda, p.ldb, operands_aligned(p));
  const size_t need = route_workspace_need(true, r, p);
  MI355_REQUIRE(need <= NOALLOC_SCRATCH_BYTES, MI355_ERR_WORKSPACE,
                "%s: M=%lld N=%lld K=%lld needs %zu bytes of scratch (split-K partial sums), the built-in scratch holds %zu; use "
                "mi355_fp8_blockwise_mm with a caller workspace",
                what, (long long)M, (long long)N, (long long)K, need, NOALLOC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (need > 0) {
    rc = symbols_of_current_device(&ws, nullptr, static_cast<hipStream_t>(stream), true, what);
    if (rc != MI355_OK) return rc;
  }
  // every partial sum that the reduce kernel reads is written by this call first, so nothing has to be cleared
  return run_gemm<true>(p, ws, need > 0 ? NOALLOC_SCRATCH_BYTES : 0, static_cast<hipStream_t>(stream), what);
}

extern "C" int mi355_qlinear_init(void) {
  clear_error();
  return symbols_of_current_device(nullptr, nullptr, nullptr, false, "mi355_qlinear_init");
}

extern "C" size_t mi355_fp8_scaled_mm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  return workspace_bytes(M, N, K, true);
}

extern "C" int mi355_fp8_scaled_mm(const void* a, const void* b, const float* sa, const float* sb, const void* bias,
                                   void* out, int out_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                                   int64_t ldo, void* workspace, size_t workspace_bytes_given, void* stream) {
  const char* what = "mi355_fp8_scaled_mm";
  clear_error();
  MI355_REQUIRE(out_dtype == MI355_BF16 || out_dtype == MI355_F16, MI355_ERR_INVALID_ARGUMENT,
                "%s: out_dtype must be bfloat16 or float16", what);
  const float* one = nullptr;
  if (M > 0 && N > 0) {
    const int rc1 = symbols_of_current_device(nullptr, &one, static_cast<hipStream_t>(stream), true, what);
    if (rc1 != MI355_OK) return rc1;
  }
  GemmParams p;
  bool empty;
  // token scale: one value per token for every K block (stride 0 along K); weight-block scale: one
  const int rc = fp8_mm_params(what, a, b, sa, one, out, out_dtype, M, N, K, lda, ldb, /*sa_sm*/ 1, /*sa_sk*/ 0, 0, 0, ldo, p, empty);
  if (rc != MI355_OK || empty) return rc;
  MI355_REQUIRE(sb != nullptr, MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  p.col_scale = sb;
  p.bias = bias;
  p.kb_total = (p.K + KSTEP - 1) / KSTEP;
  const Route r = choose_route(true, p.M, p.N, p.K, p.lda, p.ldb, operands_aligned(p));
  if (r.kernel == RK_PINGPONG && K % KSTEP == 0) {
    // large M: accumulate in the MFMA with unit scales, apply both scales once in the epilogue (the reference's order)
    p.row_scale = sa;
    p.sa = reinterpret_cast<const float*>(p.a);  // readable filler for the schedule's scale-load slots
    p.sa_sk = 0;
    p.splits = 1, p.kb_per_split = p.kb_total;
    return launch_fp8_pp_rowcol(p, static_cast<hipStream_t>(stream), what);
  }
  return run_gemm<true>(p, workspace, workspace_bytes_given, static_cast<hipStream_t>(stream), what);
}

namespace {
size_t align256(size_t b) { return (b + 255) & ~(size_t)255; }

// One-call linear where the streaming decode kernel can quantize the tokens itself: is that faster than a quantizer launch
// plus the kernel the GEMM alone would take?  Always where that kernel is the streaming one (a launch saved, nothing else
// changes); against the wave-split kernel by measurement.
// One-call linear at decode sizes: the mid-M kernel with producer waves where the GEMM alone takes that kernel, and beyond:
// for fewer tokens than the GEMM's own threshold on the same shape, and where the streaming kernel would split K into many
// ranges (the alternatives here are the streaming kernel with the quantizer in its prologue or two launches, not the bare
// wave-split kernel).  Returns the GEMM's plan otherwise.
Route linear_producer_route(int64_t M, int64_t N, int64_t K, int64_t ldw) {
  Route plain = choose_route(true, M, N, K, K, ldw, true);
  if (plain.kernel == RK_DMA3 || M > 16 || K % KSTEP != 0 || N * ldw >= (1ll << 32)) return plain;
  const RouteConstants& rc = route_constants();
  const int bn = decode_dma3_channel_tile(true, N);
  if (bn == 0) return plain;
  const bool few_tokens = (double)M < rc.decode_dma3_min_tokens &&
                          choose_route(true, (int64_t)rc.decode_dma3_min_tokens, N, K, K, ldw, true).kernel == RK_DMA3;
  const bool many_ranges = decode_supported(M, N, K) && (double)decode_splits(M, N, K) >= rc.linear_producer_min_decode_splits;
  if (few_tokens || many_ranges) plain.kernel = RK_DMA3, plain.bm = 64, plain.bn = bn, plain.splits = 1, plain.kb_per_split = (int)(K / KSTEP);
  return plain;
}

bool fused_quant_preferred(int64_t M, int64_t N, int64_t K, int64_t ldw) {
  const int plain = choose_route(true, M, N, K, K, ldw, true).kernel;
  if (plain == RK_DMA3) return false;  // the mid-M kernel at decode sizes beats the streaming kernel by more than a launch
  if (plain != RK_WAVESPLIT) return true;
  const RouteConstants& rc = route_constants();
  const double kb = (double)(K / KSTEP);
  if (kb > rc.fused_quant_long_k_blocks) return false;
  return !(kb <= rc.fused_quant_short_k_blocks && (double)M > rc.fused_quant_short_k_max_tokens);
}
}  // namespace

extern "C" size_t mi355_fp8_block_linear_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const size_t kb = (size_t)((K + KSTEP - 1) / KSTEP);
  return align256((size_t)M * (size_t)K) + align256((size_t)((M + 3) & ~3ll) * kb * 4u) + workspace_bytes(M, N, K, true);
}

namespace {
int block_linear(const char* what, const void* x, int x_dtype, int quant_mode, const void* w, const float* w_scale, int64_t ws_sn,
                 int64_t ws_sk, const void* bias, void* out, int out_dtype, int64_t M, int64_t N, int64_t K, int64_t ldw,
                 int64_t ldo, void* workspace, size_t workspace_bytes_given, void* stream) {
  clear_error();
  MI355_REQUIRE(quant_mode == MI355_QUANT_DIV || quant_mode == MI355_QUANT_RCP, MI355_ERR_INVALID_ARGUMENT,
                "%s: quant_mode must be MI355_QUANT_DIV or MI355_QUANT_RCP", what);
  MI355_REQUIRE(M >= 0 && N >= 0 && K >= 0, MI355_ERR_INVALID_ARGUMENT, "%s: negative shape", what);
  MI355_REQUIRE(out_dtype == MI355_BF16 || out_dtype == MI355_F16, MI355_ERR_INVALID_ARGUMENT,
                "%s: out_dtype must be bfloat16 or float16", what);
  if (M == 0 || N == 0) return MI355_OK;
  MI355_REQUIRE(K > 0 && K % KSTEP == 0, MI355_ERR_INVALID_ARGUMENT,
                "%s: K must be a positive multiple of the quantization group (128)", what);
  MI355_REQUIRE(x && w && w_scale && out, MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  const size_t need = mi355_fp8_block_linear_workspace_bytes(M, N, K);
  MI355_REQUIRE(workspace != nullptr && workspace_bytes_given >= need, MI355_ERR_WORKSPACE,
                "%s: needs a workspace of %zu bytes, got %zu", what, need, workspace_bytes_given);
  MI355_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, MI355_ERR_WORKSPACE,
                "%s: workspace must be 256-byte aligned", what);
  // workspace: [codes M x K][token scales, M-major, pitch align4(M)][what the GEMM needs]
  uint8_t* q = static_cast<uint8_t*>(workspace);
  const size_t q_bytes = align256((size_t)M * (size_t)K);
  float* sa = reinterpret_cast<float*>(q + q_bytes);
  const int64_t pitch = (M + 3) & ~3ll;
  const size_t sa_bytes = align256((size_t)pitch * (size_t)(K / KSTEP) * 4u);
  // Decode sizes: the GEMM kernel quantizes the tokens of each K range itself (same arithmetic), no quantizer launch -
  // except where a quantizer launch in front of the wave-split kernel is measured faster (route_constants.h).
  const bool ptr_ok = x_dtype != MI355_F32 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0 && ldw % 16 == 0;
  if (ptr_ok && M <= 16) {
    const Route plain = linear_producer_route(M, N, K, ldw);
    if (plain.kernel == RK_DMA3) {  // one round of unsplit 64-token tiles: producer waves of that kernel quantize the tokens
      GemmParams p;
      bool empty;
      const int rc = fp8_mm_params(what, x, w, w_scale, w_scale, out, out_dtype, M, N, K, K, ldw, 1, (M + 3) & ~3ll, ws_sn, ws_sk, ldo, p, empty);
      if (rc != MI355_OK || empty) return rc;
      p.bias = bias;
      p.x16 = x, p.ldx = K, p.x_dtype = x_dtype, p.x_by_reciprocal = quant_mode == MI355_QUANT_RCP;
      p.kb_total = K / KSTEP, p.splits = 1, p.kb_per_split = p.kb_total;
      return launch_fp8_dma3_quant(p, plain.bn, static_cast<hipStream_t>(stream), what);
    }
  }
  if (ptr_ok && choose_route(true, M, N, K, K, ldw, true, true).kernel == RK_DECODE && fused_quant_preferred(M, N, K, ldw)) {
    GemmParams p;
    bool empty;
    // a / sa are not read by the kernel in this mode; they only have to satisfy the checks
    int rc = fp8_mm_params(what, x, w, w_scale, w_scale, out, out_dtype, M, N, K, K, ldw, 1, (M + 3) & ~3ll, ws_sn, ws_sk, ldo, p, empty);
    if (rc != MI355_OK || empty) return rc;
    p.bias = bias;
    p.x16 = x, p.ldx = K, p.x_dtype = x_dtype, p.x_by_reciprocal = quant_mode == MI355_QUANT_RCP;
    return run_gemm<true>(p, workspace, workspace_bytes_given, static_cast<hipStream_t>(stream), what);
  }
  // quantize with q = x / s, the arithmetic of the reference's column-major path (fp8_kernel.py:164-212 via fp8_utils.py:201-203),
  // or with q = x * (1 / s), that of its row-major path (fp8_kernel.py:156-158); the scale layout here is the library's own
  int rc = mi355_group_quant_8bit(x, x_dtype, q, MI355_FP8_E4M3FN, sa, M, K, KSTEP, 1e-10f, -448.0f, 448.0f, quant_mode,
                                  MI355_SCALE_F32, 0.0f, 1, pitch, stream);
  if (rc != MI355_OK) return rc;
  GemmParams p;
  bool empty;
  rc = fp8_mm_params(what, q, w, sa, w_scale, out, out_dtype, M, N, K, K, ldw, 1, pitch, ws_sn, ws_sk, ldo, p, empty);
  if (rc != MI355_OK || empty) return rc;
  p.bias = bias;
  return run_gemm<true>(p, q + q_bytes + sa_bytes, workspace_bytes_given - q_bytes - sa_bytes, static_cast<hipStream_t>(stream), what);
}
}  // namespace

extern "C" int mi355_fp8_block_linear(const void* x, int x_dtype, const void* w, const float* w_scale, int64_t ws_sn,
                                      int64_t ws_sk, const void* bias, void* out, int out_dtype, int64_t M, int64_t N,
                                      int64_t K, int64_t ldw, int64_t ldo, void* workspace, size_t workspace_bytes_given,
                                      void* stream) {
  return block_linear("mi355_fp8_block_linear", x, x_dtype, MI355_QUANT_DIV, w, w_scale, ws_sn, ws_sk, bias, out, out_dtype, M, N,
                      K, ldw, ldo, workspace, workspace_bytes_given, stream);
}

extern "C" int mi355_fp8_block_linear_mode(const void* x, int x_dtype, int quant_mode, const void* w, const float* w_scale,
                                           int64_t ws_sn, int64_t ws_sk, const void* bias, void* out, int out_dtype, int64_t M,
                                           int64_t N, int64_t K, int64_t ldw, int64_t ldo, void* workspace,
                                           size_t workspace_bytes_given, void* stream) {
  return block_linear("mi355_fp8_block_linear_mode", x, x_dtype, quant_mode, w, w_scale, ws_sn, ws_sk, bias, out, out_dtype, M, N,
                      K, ldw, ldo, workspace, workspace_bytes_given, stream);
}

extern "C" int mi355_fp8_block_linear_plan(int64_t M, int64_t N, int64_t K, char* buf, size_t buf_len) {
  const char* what = "mi355_fp8_block_linear_plan";
  clear_error();
  MI355_REQUIRE(buf != nullptr && buf_len > 0, MI355_ERR_INVALID_ARGUMENT, "%s: no buffer", what);
  MI355_REQUIRE(M > 0 && N > 0 && K > 0 && M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31) && K % KSTEP == 0,
                MI355_ERR_INVALID_ARGUMENT, "%s: shape out of range (K must be a multiple of 128)", what);
  const Route plain = linear_producer_route(M, N, K, K);
  const bool producer = M <= 16 && plain.kernel == RK_DMA3;  // the mid-M kernel's producer waves quantize
  const bool fused = producer || (choose_route(true, M, N, K, K, K, true, true).kernel == RK_DECODE && fused_quant_preferred(M, N, K, K));
  const Route r = producer ? plain : choose_route(true, M, N, K, K, K, true, fused);
  const int n = snprintf(buf, buf_len, "kernel=%s bm=%d bn=%d splits=%d kb_per_split=%d groups_per_wg=%d aligned=%d stages=%d quantizer=%s",
                         ROUTE_NAMES[r.kernel], r.bm, r.bn, r.splits, r.kb_per_split, r.groups_per_wg, (int)r.aligned,
                         route_stages(true, r, M, N), fused ? "fused" : "launch");
  MI355_REQUIRE(n > 0 && (size_t)n < buf_len, MI355_ERR_INVALID_ARGUMENT, "%s: buffer of %zu bytes is too small", what, buf_len);
  return MI355_OK;
}

extern "C" size_t mi355_int8_scaled_mm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  return workspace_bytes(M, N, K, false);
}

extern "C" int mi355_int8_scaled_mm(const void* a, const void* b, const float* sa, const float* sb, const void* bias,
                                    void* out, int out_dtype, int64_t M, int64_t N, int64_t K, int64_t lda,
                                    int64_t ldb, int64_t ldo, void* workspace, size_t workspace_bytes_given,
                                    void* stream) {
  const char* what = "mi355_int8_scaled_mm";
  clear_error();
  MI355_REQUIRE(M >= 0 && N >= 0 && K >= 0, MI355_ERR_INVALID_ARGUMENT, "%s: negative shape", what);
  MI355_REQUIRE(out_dtype == MI355_BF16 || out_dtype == MI355_F16 || out_dtype == MI355_I32,
                MI355_ERR_INVALID_ARGUMENT, "%s: out_dtype must be bfloat16 or float16 (int32 for raw accumulators)",
                what);
  if (M == 0 || N == 0) return MI355_OK;
  MI355_REQUIRE(K > 0, MI355_ERR_INVALID_ARGUMENT, "%s: K must be positive", what);
  MI355_REQUIRE(a && b && out, MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  MI355_REQUIRE(out_dtype == MI355_I32 || (sa && sb), MI355_ERR_INVALID_ARGUMENT, "%s: scales missing", what);
  MI355_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 17), MI355_ERR_INVALID_ARGUMENT,
                "%s: K must stay below 131072 so that int32 accumulation cannot overflow", what);
  MI355_REQUIRE(lda >= K && ldb >= K && ldo >= N, MI355_ERR_INVALID_ARGUMENT,
                "%s: row strides smaller than the row length", what);
  GemmParams p{};
  p.a = static_cast<const uint8_t*>(a);
  p.b = static_cast<const uint8_t*>(b);
  p.sa = sa, p.sb = sb, p.bias = bias, p.out = out, p.ws = nullptr;
  p.M = (int)M, p.N = (int)N, p.K = (int)K;
  p.lda = lda, p.ldb = ldb, p.ldo = ldo;
  p.out_dtype = out_dtype;
  return run_gemm<false>(p, workspace, workspace_bytes_given, static_cast<hipStream_t>(stream), what);
}

extern "C" size_t mi355_int8_linear_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  return align256((size_t)M * (size_t)K) + align256((size_t)M * 4u) + workspace_bytes(M, N, K, false);
}

extern "C" int mi355_int8_linear(const void* x, int x_dtype, const void* w, const float* w_scale, const void* bias, void* out,
                                 int out_dtype, int64_t M, int64_t N, int64_t K, int64_t ldw, int64_t ldo, void* workspace,
                                 size_t workspace_bytes_given, void* stream) {
  const char* what = "mi355_int8_linear";
  clear_error();
  MI355_REQUIRE(M >= 0 && N >= 0 && K >= 0, MI355_ERR_INVALID_ARGUMENT, "%s: negative shape", what);
  MI355_REQUIRE(out_dtype == MI355_BF16 || out_dtype == MI355_F16, MI355_ERR_INVALID_ARGUMENT,
                "%s: out_dtype must be bfloat16 or float16", what);
  if (M == 0 || N == 0) return MI355_OK;
  MI355_REQUIRE(K > 0 && K < (1ll << 17) && M < (1ll << 31) && N < (1ll << 31), MI355_ERR_INVALID_ARGUMENT,
                "%s: K must be positive and below 131072 so that int32 accumulation cannot overflow", what);
  MI355_REQUIRE(x && w && w_scale && out, MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  MI355_REQUIRE(ldw >= K && ldo >= N, MI355_ERR_INVALID_ARGUMENT, "%s: row strides smaller than the row length", what);
  const size_t need = mi355_int8_linear_workspace_bytes(M, N, K);
  MI355_REQUIRE(workspace != nullptr && workspace_bytes_given >= need, MI355_ERR_WORKSPACE,
                "%s: needs a workspace of %zu bytes, got %zu", what, need, workspace_bytes_given);
  MI355_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, MI355_ERR_WORKSPACE,
                "%s: workspace must be 256-byte aligned", what);
  // workspace: [codes M x K][token scales M][what the GEMM needs]
  uint8_t* q = static_cast<uint8_t*>(workspace);
  const size_t q_bytes = align256((size_t)M * (size_t)K);
  float* sa = reinterpret_cast<float*>(q + q_bytes);
  const size_t sa_bytes = align256((size_t)M * 4u);
  const int rc = mi355_per_token_quant_int8(x, x_dtype, q, sa, M, K, stream);
  if (rc != MI355_OK) return rc;
  GemmParams p{};
  p.a = q;
  p.b = static_cast<const uint8_t*>(w);
  p.sa = sa, p.sb = w_scale, p.bias = bias, p.out = out, p.ws = nullptr;
  p.M = (int)M, p.N = (int)N, p.K = (int)K;
  p.lda = K, p.ldb = ldw, p.ldo = ldo;
  p.out_dtype = out_dtype;
  return run_gemm<false>(p, q + q_bytes + sa_bytes, workspace_bytes_given - q_bytes - sa_bytes, static_cast<hipStream_t>(stream), what);
}

extern "C" size_t mi355_fp8_per_token_linear_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  return align256((size_t)M * (size_t)K) + align256((size_t)M * 4u) + mi355_fp8_scaled_mm_workspace_bytes(M, N, K);
}

extern "C" int mi355_fp8_per_token_linear(const void* x, int x_dtype, const void* w, const float* w_scale, const void* bias,
                                          void* out, int out_dtype, int64_t M, int64_t N, int64_t K, int64_t ldw, int64_t ldo,
                                          void* workspace, size_t workspace_bytes_given, void* stream) {
  const char* what = "mi355_fp8_per_token_linear";
  clear_error();
  MI355_REQUIRE(M >= 0 && N >= 0 && K >= 0, MI355_ERR_INVALID_ARGUMENT, "%s: negative shape", what);
  MI355_REQUIRE(out_dtype == MI355_BF16 || out_dtype == MI355_F16, MI355_ERR_INVALID_ARGUMENT,
                "%s: out_dtype must be bfloat16 or float16", what);
  if (M == 0 || N == 0) return MI355_OK;
  MI355_REQUIRE(K > 0 && M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), MI355_ERR_INVALID_ARGUMENT,
                "%s: K must be positive and every dimension fit in 31 bits", what);
  MI355_REQUIRE(x && w && w_scale && out, MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  const size_t need = mi355_fp8_per_token_linear_workspace_bytes(M, N, K);
  MI355_REQUIRE(workspace != nullptr && workspace_bytes_given >= need, MI355_ERR_WORKSPACE,
                "%s: needs a workspace of %zu bytes, got %zu", what, need, workspace_bytes_given);
  MI355_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, MI355_ERR_WORKSPACE,
                "%s: workspace must be 256-byte aligned", what);
  // workspace: [codes M x K][token scales M][what the GEMM needs]
  uint8_t* q = static_cast<uint8_t*>(workspace);
  const size_t q_bytes = align256((size_t)M * (size_t)K);
  float* sa = reinterpret_cast<float*>(q + q_bytes);
  const size_t sa_bytes = align256((size_t)M * 4u);
  const int rc = mi355_per_token_quant_fp8(x, x_dtype, q, sa, M, K, stream);
  if (rc != MI355_OK) return rc;
  return mi355_fp8_scaled_mm(q, w, sa, w_scale, bias, out, out_dtype, M, N, K, K, ldw, ldo, q + q_bytes + sa_bytes,
                             workspace_bytes_given - q_bytes - sa_bytes, stream);
}

extern "C" size_t mi355_fp8_block_linear_ue8m0_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const size_t words = (size_t)(((K + KSTEP - 1) / KSTEP + 3) / 4);
  return align256((size_t)M * (size_t)K) + align256((size_t)((M + 3) & ~3ll) * words * 4u) +
         mi355_fp8_blockwise_mm_ue8m0_workspace_bytes(M, N, K);
}

extern "C" int mi355_fp8_block_linear_ue8m0(const void* x, int x_dtype, const void* w, const void* sb_words, int64_t sb_sn,
                                            int64_t sb_sk, const void* bias, void* out, int out_dtype, int64_t M, int64_t N,
                                            int64_t K, int64_t ldw, int64_t ldo, void* workspace, size_t workspace_bytes_given,
                                            void* stream) {
  const char* what = "mi355_fp8_block_linear_ue8m0";
  clear_error();
  MI355_REQUIRE(M >= 0 && N >= 0 && K >= 0, MI355_ERR_INVALID_ARGUMENT, "%s: negative shape", what);
  MI355_REQUIRE(out_dtype == MI355_BF16 || out_dtype == MI355_F16, MI355_ERR_INVALID_ARGUMENT,
                "%s: out_dtype must be bfloat16 or float16", what);
  if (M == 0 || N == 0) return MI355_OK;
  MI355_REQUIRE(K > 0 && K % KSTEP == 0, MI355_ERR_INVALID_ARGUMENT,
                "%s: K must be a positive multiple of the quantization group (128)", what);
  MI355_REQUIRE(x && w && sb_words && out, MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  const size_t need = mi355_fp8_block_linear_ue8m0_workspace_bytes(M, N, K);
  MI355_REQUIRE(workspace != nullptr && workspace_bytes_given >= need, MI355_ERR_WORKSPACE,
                "%s: needs a workspace of %zu bytes, got %zu", what, need, workspace_bytes_given);
  MI355_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, MI355_ERR_WORKSPACE,
                "%s: workspace must be 256-byte aligned", what);
  // workspace: [codes M x K][token scale words, packed along tokens, pitch align4(M)][what the GEMM needs]
  uint8_t* q = static_cast<uint8_t*>(workspace);
  const size_t q_bytes = align256((size_t)M * (size_t)K);
  void* sa_words = q + q_bytes;
  const int64_t pitch = (M + 3) & ~3ll;
  const size_t sa_bytes = align256((size_t)pitch * (size_t)((K / KSTEP + 3) / 4) * 4u);
  // q = x * (448 / amax) with the scale rounded up to a power of two: per_token_group_quant_8bit_v2.cu:77-78 with scale_ue8m0
  const int rc = mi355_group_quant_8bit(x, x_dtype, q, MI355_FP8_E4M3FN, sa_words, M, K, KSTEP, 1e-10f, -448.0f, 448.0f,
                                        MI355_QUANT_MUL, MI355_SCALE_UE8M0_PACKED, 0.0f, 1, pitch, stream);
  if (rc != MI355_OK) return rc;
  return mi355_fp8_blockwise_mm_ue8m0(q, w, sa_words, sb_words, bias, out, out_dtype, M, N, K, K, ldw, pitch, sb_sn, sb_sk, ldo,
                                      q + q_bytes + sa_bytes, workspace_bytes_given - q_bytes - sa_bytes, stream);
}

extern "C" int mi355_fp8_blockwise_mm_plan(int64_t M, int64_t N, int64_t K, int aligned, char* buf, size_t buf_len) {
  return describe_route(true, M, N, K, aligned, buf, buf_len, "mi355_fp8_blockwise_mm_plan");
}

extern "C" int mi355_int8_scaled_mm_plan(int64_t M, int64_t N, int64_t K, int aligned, char* buf, size_t buf_len) {
  return describe_route(false, M, N, K, aligned, buf, buf_len, "mi355_int8_scaled_mm_plan");
}
