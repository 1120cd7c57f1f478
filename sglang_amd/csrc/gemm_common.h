// Shared declarations of the gfx950 GEMM kernels: vector types, launch parameters, output store, tile order.
#pragma once

#include <type_traits>

#include "common.h"
#include "route_constants.h"

namespace mi355 {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int KSTEP = 128;   // bytes of K per row and stage
constexpr int THREADS = 256;
constexpr int GROUP_M = 8;    // M-tiles per group in the tile order

constexpr int NUM_CUS = 256;

struct GemmParams {
  const uint8_t* a;  // tokens   [M, K], row stride lda
  const uint8_t* b;  // channels [N, K], row stride ldb
  const float* sa;
  const float* sb;
  const void* bias;        // optional [N] in the output dtype (INT8 GEMM; per-channel FP8 epilogue)
  const float* col_scale;  // FP8 only, optional [N]: per-channel scale applied in the epilogue (fp8_scaled_mm)
  const float* row_scale;  // FP8 two-phase kernel in its epilogue-scaled mode only: per-token scale [M]
  const void* x16;         // FP8 decode kernel only, optional: unquantized tokens [M, K] (x_dtype, row stride ldx elements);
  int64_t ldx;             // when set, the kernel quantizes them per 1 x 128 group itself and ignores a / sa
  int x_dtype;
  int x_by_reciprocal;     // the fused quantizer computes q = x * (1 / s) instead of q = x / s
  void* out;
  void* ws;  // split-K partial tiles: [splits][M][N] fp32 or int32
  int M, N, K;
  int64_t lda, ldb, ldo;
  int64_t sa_sm, sa_sk, sb_sn, sb_sk;
  int kb_total, kb_per_split, splits;
  int tiles_m, tiles_n;
  int out_dtype;
  int ue8m0;  // FP8 only: sa / sb are packed exponent words and the route's kernel applies them in the MFMA (set by the UE8M0 entry point)
};

// ---------------------------------------------------------------------------------------------
// Puts a wave-uniform value into a vector register HERE.  The MFMA takes its scale operands from vector registers and reads
// all 64 lanes whatever EXEC says; the compiler, which knows neither, may sink an MFMA whose result only a guarded store
// uses into that store's divergent region together with the scalar-to-vector copy of its scale, and the copy then skips
// the inactive lanes (rows of the operand that the active lanes' results still depend on).  Call it where every lane is active.
__device__ __forceinline__ int in_vgpr(int x) {
  asm volatile("" : "+v"(x));
  return x;
}

// ---- 1 x 128 group quantization inside a GEMM kernel (the one-call linear at decode sizes): 16 lanes hold a group, 8
// elements each, with the arithmetic of the group quantizer's reference path (amax floored at 1e-10, s = amax / 448,
// q = e4m3fn(clamp(x / s)), group_quant.hip).
// max over the 16 lanes of a DPP row
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true)));
  return v;
}
// x / s, correctly rounded, given r = RN(1 / s): two Markstein steps, as in the group quantizer (group_quant.hip), where
// the conditions under which this equals the `/` operator are stated and checked.
__device__ __forceinline__ float div_by_shared(float x, float s, float r) {
  float q = x * r;
  q = fmaf(fmaf(-q, s, x), r, q);
  q = fmaf(fmaf(-q, s, x), r, q);
  return q;
}
// The lane's eight 16-bit elements (raw) of a group spread over its DPP row -> their eight e4m3fn codes and the group's scale
// (the same value in all 16 lanes).  Every lane of the row must be active.  by_reciprocal: q = x * (1 / s) as the
// reference's row-major-scale quantizer computes it (fp8_kernel.py:156-158), else the true division of its M-major one.
__device__ __forceinline__ u32x2 quantize_group_lane(const u32x4& raw, int x_dtype, bool by_reciprocal, float& scale) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  float v[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = x_dtype == MI355_BF16 ? __uint_as_float(w[i] << 16) : f16_bits_to_f32(w[i] & 0xffffu);
    v[2 * i + 1] = x_dtype == MI355_BF16 ? __uint_as_float(w[i] & 0xffff0000u) : f16_bits_to_f32(w[i] >> 16);
  }
  float amax = 1e-10f;
#pragma unroll
  for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(v[e]));
  amax = row16_max(amax);
  const float sc = amax / 448.0f;
  const float rcp = 1.0f / sc;
  float t[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) t[e] = fminf(fmaxf(by_reciprocal ? v[e] * rcp : div_by_shared(v[e], sc, rcp), -448.0f), 448.0f);
  int c0 = __builtin_amdgcn_cvt_pk_fp8_f32(t[0], t[1], 0, false);
  c0 = __builtin_amdgcn_cvt_pk_fp8_f32(t[2], t[3], c0, true);
  int c1 = __builtin_amdgcn_cvt_pk_fp8_f32(t[4], t[5], 0, false);
  c1 = __builtin_amdgcn_cvt_pk_fp8_f32(t[6], t[7], c1, true);
  scale = sc;
  return u32x2{(uint32_t)c0, (uint32_t)c1};
}

__device__ __forceinline__ void store_out4(void* out, int out_dtype, int64_t off, const float* r, int nvalid,
                                           bool vec_ok) {
  if (out_dtype == MI355_F32) {
    float* o = reinterpret_cast<float*>(out) + off;
    if (nvalid == 4 && vec_ok) {
      *reinterpret_cast<v4f*>(o) = v4f{r[0], r[1], r[2], r[3]};
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (i < nvalid) o[i] = r[i];
    }
    return;
  }
  const bool bf = out_dtype == MI355_BF16;
  const uint32_t w0 = bf ? pack_bf16x2(r[0], r[1]) : pack_f16x2(r[0], r[1]);
  const uint32_t w1 = bf ? pack_bf16x2(r[2], r[3]) : pack_f16x2(r[2], r[3]);
  uint16_t* o = reinterpret_cast<uint16_t*>(out) + off;
  if (nvalid == 4 && vec_ok) {
    *reinterpret_cast<u32x2*>(o) = u32x2{w0, w1};
  } else {
    const uint32_t h[4] = {w0 & 0xffffu, w0 >> 16, w1 & 0xffffu, w1 >> 16};
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < nvalid) o[i] = (uint16_t)h[i];
  }
}


// ---- 256 x 256 output tile of 16-bit elements through LDS.
// A lane's accumulators are four consecutive channels of one token: stored straight from registers, a wave instruction
// writes 16 or 32 separate 32-byte pieces, and a tile takes ~12 us.  Instead every wave writes its results into a
// [256 tokens][512 bytes] image of the tile in LDS (16-byte chunks XOR-swizzled with the row so that neither side has
// bank conflicts), and after a barrier each wave stores 32 whole rows, two rows of 512 contiguous bytes per instruction.
constexpr int OUT_TILE_BYTES = 256 * 512;

__device__ __forceinline__ uint32_t pack2_16(int out_dtype, float lo, float hi) {
  return out_dtype == MI355_BF16 ? pack_bf16x2(lo, hi) : pack_f16x2(lo, hi);
}
// four consecutive channels starting at tile column `col` (a multiple of 4) of tile row `row`
__device__ __forceinline__ void out_tile_put4(uint8_t* tile, int row, int col, int out_dtype, const float* r) {
  const int chunk = col >> 3, half = (col >> 2) & 1;
  *reinterpret_cast<u32x2*>(tile + row * 512 + ((chunk ^ (row & 7)) << 4) + half * 8) =
      u32x2{pack2_16(out_dtype, r[0], r[1]), pack2_16(out_dtype, r[2], r[3])};
}
// Called by all 512 threads after a barrier that follows the last out_tile_put4.  Needs ldo % 8 == 0, a 16-byte aligned
// output base and n0 + 256 <= N; rows at or past M are skipped.
__device__ __forceinline__ void out_tile_store(const uint8_t* tile, void* out, int64_t ldo, int m0, int n0, int M) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int chunk = lane & 31;
  uint16_t* o = reinterpret_cast<uint16_t*>(out);
#pragma unroll 4
  for (int it = 0; it < 16; ++it) {
    const int row = wave * 32 + it * 2 + (lane >> 5);
    const u32x4 v = *reinterpret_cast<const u32x4*>(tile + row * 512 + ((chunk ^ (row & 7)) << 4));
    if (m0 + row < M) *reinterpret_cast<u32x4*>(o + (int64_t)(m0 + row) * ldo + n0 + chunk * 8) = v;
  }
}
__device__ __forceinline__ bool out_tile_ok(const void* out, int64_t ldo, int out_dtype, int n0, int N) {
  return (out_dtype == MI355_BF16 || out_dtype == MI355_F16) && (ldo & 7) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0 &&
         n0 + 256 <= N;
}

// Optional per-channel epilogue of the FP8 kernels: r[v] = col_scale[n + v] * r[v] + bias[n + v] for the four consecutive
// channels n .. n + 3 (channels at or past N repeat the last one; they are never stored).
__device__ __forceinline__ void fp8_channel_epilogue(const GemmParams& p, int n, float* r) {
  if (p.col_scale == nullptr && p.bias == nullptr) return;
  const bool whole = n + 4 <= p.N;
  if (p.col_scale) {
    if (whole && (reinterpret_cast<uintptr_t>(p.col_scale + n) & 15) == 0) {
      const v4f c = *reinterpret_cast<const v4f*>(p.col_scale + n);
#pragma unroll
      for (int v = 0; v < 4; ++v) r[v] = c[v] * r[v];
    } else {
#pragma unroll
      for (int v = 0; v < 4; ++v) r[v] = p.col_scale[min(n + v, p.N - 1)] * r[v];
    }
  }
  if (p.bias) {
    const uint16_t* b = reinterpret_cast<const uint16_t*>(p.bias);
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const uint32_t h = b[min(n + v, p.N - 1)];
      r[v] += (p.out_dtype == MI355_BF16) ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
    }
  }
}

struct TileCoord {
  int tile_m, tile_n, split;
};

// Workgroup -> output tile.  Consecutive workgroup ids go round-robin to the 8 XCDs (each with its own L2), so
// ids are first renumbered to give every XCD a contiguous range; inside a range tiles are walked GROUP_M
// M-tiles at a time, so that the tiles an XCD works on concurrently share weight and token rows in its L2.
__device__ __forceinline__ TileCoord tile_of_block(int bid, int total, int tiles_m, int tiles_n) {
  const int per = total >> 3;
  if (bid < per * 8) bid = (bid & 7) * per + (bid >> 3);
  const int tiles_mn = tiles_m * tiles_n;
  TileCoord c;
  c.split = bid / tiles_mn;
  const int lid = bid - c.split * tiles_mn;
  const int per_group = GROUP_M * tiles_n;
  const int group = lid / per_group;
  const int first_m = group * GROUP_M;
  const int gm = min(tiles_m - first_m, GROUP_M);
  const int in_group = lid - group * per_group;
  c.tile_m = first_m + in_group % gm;
  c.tile_n = in_group / gm;
  return c;
}

// Large-M blockwise FP8 GEMM (256 x 128 tile, three LDS stages, software-pipelined); gemm_fp8_pipelined.hip.
// Needs 16-byte aligned rows and K % 16 == 0.  Returns an MI355_* status.
int launch_fp8_pipelined(GemmParams& p, hipStream_t stream, const char* what);

// Large-M blockwise FP8 GEMM (256 x 256 tile, 8 waves in two groups that alternate compute and memory phases);
// gemm_fp8_pp.hip.  Same requirements.
int launch_fp8_pp(GemmParams& p, hipStream_t stream, const char* what);
// The K loop of launch_fp8_pp without its global loads: a measurement aid (see gemm_fp8_pp.hip).  K % 128 == 0.
int launch_fp8_pp_noload(GemmParams& p, hipStream_t stream, const char* what);
// The same kernel for packed power-of-two (UE8M0) scales on both operands, applied by the MFMA itself: p.sa / p.sb point
// to 32-bit words of four exponent bytes (see fp8_gemm_pp_kernel).  K % 128 == 0.
int launch_fp8_pp_ue8m0(GemmParams& p, hipStream_t stream, const char* what);
// The same kernel with one scale per token (p.row_scale) and per channel (p.col_scale) applied after the K loop, which
// then carries no scale arithmetic; p.sa must point to >= 4 * M readable, 16-byte aligned bytes.  K % 128 == 0.
int launch_fp8_pp_rowcol(GemmParams& p, hipStream_t stream, const char* what);
// Token scales must be M-major with a pitch that is a multiple of four floats and a 16-byte aligned base.


// Mid-M blockwise FP8 GEMM (64/128 x 256 tile, 8 waves, three LDS stages, hand-issued direct-to-LDS loads);
// gemm_fp8_dma3.hip.  Needs 16-byte aligned rows, K % 128 == 0, row offsets below 4 GiB.  dma3_plan() gives the split it
// wants; the caller sets p.splits, p.kb_per_split and p.ws accordingly.
struct Dma3Plan {
  int bm, bn, splits, kb_per_split;  // bn: 256, 192 (FP8 only) or 128, whichever models fastest
  double efficiency;  // modelled fraction of the streaming time that is useful (balance, partial sums, pipeline fill)
  double time_us;     // modelled duration of the chosen plan
};
Dma3Plan dma3_plan(int64_t M, int64_t N, int64_t K, bool is_int8 = false);
int dma3_stages(int bm, int bn, int64_t workgroups);  // LDS stages the FP8 kernel runs such a launch with (3, 4 or 6)
int launch_fp8_dma3(GemmParams& p, int bm, int bn, hipStream_t stream, const char* what);  // bm: 64 or 128, bn: 128, 192 or 256, from dma3_plan()
// The same for packed UE8M0 scales on both operands (p.sa / p.sb point to the words, p.sa_sk / p.sb_sn / p.sb_sk are word
// strides; token words M-major with a pitch that is a multiple of four words), applied by the MFMA.
int launch_fp8_dma3_ue8m0(GemmParams& p, int bm, int bn, hipStream_t stream, const char* what);
// One-call linear at decode sizes on this kernel: a producer wave quantizes the unquantized tokens (p.x16, M <= 16) block by block.
int launch_fp8_dma3_quant(GemmParams& p, int bn, hipStream_t stream, const char* what);

// Grouped problems on the tile bodies of the dense kernels: token rows of all experts stacked in one matrix, one weight
// matrix per expert.  `g` describes expert 0 (a, out, b, sb, and sa = the re-laid-out token scales: M-major, every
// expert's first row moved to column ((row0 + 3) & ~3) + 4 * expert so that each expert starts on a whole quad); N, K,
// strides and kb_total are common to all experts; splits = 1.  `tiles` is written on the device from the problem sizes:
// tiles[0].x = number of token tiles of this launch, then one record per token tile: {expert, first stacked row of the
// expert, rows of the expert, first row of the tile in the expert}.
struct GroupedParams {
  GemmParams g;
  const v4i* tiles;
  int64_t b_expert_stride;   // bytes between consecutive experts' weight matrices
  int64_t sb_expert_stride;  // floats between consecutive experts' weight-block scales
  int max_tiles_m;           // upper bound on the number of records; the grid is max_tiles_m * tiles_n
  int out_elem;              // bytes per output element
};
// Workgroup -> (token tile record, channel tile) and the parameter block of that tile's expert.  The grid is sized for the
// largest possible number of token tiles; workgroups past the real number (known only on the device) leave at once.  The
// ids below it are renumbered so that each XCD gets a contiguous range (as in tile_of_block; it has to be the real
// number, or the XCDs that are handed the high ids would get nothing but empty workgroups); inside a range GROUPED_GM
// token tiles at a time are walked over all channel tiles, token tile fastest, so that the token tiles of one expert
// that use the same weight rows run together on one XCD's L2.  Returns false for a workgroup without a tile.
constexpr int GROUPED_GM = 4;
__device__ __forceinline__ bool grouped_tile_of_block(const GroupedParams& gp, GemmParams& p, int& m0, int& tile_n) {
  const int count = min(__builtin_amdgcn_readfirstlane(gp.tiles[0].x), gp.max_tiles_m);
  const int total = count * gp.g.tiles_n;
  int bid = blockIdx.x;
  if (bid >= total) return false;
  const int per = total >> 3;
  if (bid < per * 8) bid = (bid & 7) * per + (bid >> 3);
  const int span = GROUPED_GM * gp.g.tiles_n;
  const int grp = bid / span, r = bid - grp * span;
  const int gm = min(GROUPED_GM, count - grp * GROUPED_GM);
  tile_n = r / gm;
  const v4i rec = gp.tiles[1 + grp * GROUPED_GM + r % gm];
  const int e = __builtin_amdgcn_readfirstlane(rec.x);
  const int row0 = __builtin_amdgcn_readfirstlane(rec.y);
  m0 = __builtin_amdgcn_readfirstlane(rec.w);
  p = gp.g;
  p.a += (int64_t)row0 * p.lda;
  p.b += (int64_t)e * gp.b_expert_stride;
  p.sb += (int64_t)e * gp.sb_expert_stride;
  p.sa += ((row0 + 3) & ~3) + 4 * e;
  p.out = reinterpret_cast<uint8_t*>(p.out) + (int64_t)row0 * p.ldo * gp.out_elem;
  p.M = __builtin_amdgcn_readfirstlane(rec.z);
  return true;
}
int launch_fp8_grouped_dma3(GroupedParams& gp, int bm, hipStream_t stream, const char* what);  // gemm_fp8_dma3.hip; bm: 64 or 128
int launch_fp8_grouped_pp(GroupedParams& gp, hipStream_t stream, const char* what);            // gemm_fp8_pp.hip: 256-row tiles
int launch_int8_dma3(GemmParams& p, int bm, int bn, hipStream_t stream, const char* what);  // gemm_int8_dma3.hip: same tiling, int8 MFMA, int32 partials

// Large-M INT8 GEMM (256 x 256 tile, 8 waves in two groups that alternate compute and memory phases, direct-to-LDS loads,
// 16x16x64 MFMA); gemm_int8_pp.hip.  Needs 16-byte aligned rows, K % 128 == 0 and row offsets below 4 GiB.
int launch_int8_pp(GemmParams& p, hipStream_t stream, const char* what);
// Mid-M INT8 GEMM (128 x 256 tile, the two-phase schedule over three LDS stages); gemm_int8_pp128.hip.  Same requirements;
// optional split along K: the caller sets p.splits, p.kb_per_split and p.ws (int32 partials, ordered reduce afterwards).
int launch_int8_pp128(GemmParams& p, hipStream_t stream, const char* what);

// Small-M blockwise FP8 GEMM streaming the weight through wave-private LDS, no barriers; gemm_fp8_decode.hip.
// decode_splits() is the split count it wants for a shape; the caller sets p.splits, p.kb_per_split and p.ws.
int decode_splits(int64_t M, int64_t N, int64_t K);
int decode_kb_per_range();  // K blocks per split (the last range may be shorter)
bool decode_supported(int64_t M, int64_t N, int64_t K);
int decode_groups_per_wg(int64_t N, int splits);  // consecutive 128-channel groups one workgroup walks
int launch_fp8_decode(GemmParams& p, int groups_per_wg, hipStream_t stream, const char* what);
int launch_int8_decode(GemmParams& p, int groups_per_wg, hipStream_t stream, const char* what);  // same kernel, int8 MFMA, int32 partials

// Decode (M <= 16) GEMMs for small weights (gemm_decode_wavesplit.hip): 16 channels per workgroup, K split over its waves
// and summed inside the workgroup - one launch, no workspace.  K % 128 == 0, N % 16 == 0, 16-byte aligned rows.
struct WavesplitShape {
  int waves, blocks_per_round;
};
WavesplitShape wavesplit_shape(int64_t K);
bool wavesplit_two_tiles(bool is_fp8, int64_t M, int64_t N, int64_t K);  // 32 channels per workgroup instead of 16
bool wavesplit_supported(int64_t M, int64_t N, int64_t K);
int launch_fp8_wavesplit(GemmParams& p, hipStream_t stream, const char* what);
int launch_int8_wavesplit(GemmParams& p, hipStream_t stream, const char* what);
// The FP8 kernel with packed power-of-two scales on both operands, applied by the MFMA (p.sa / p.sb point to the words,
// p.sa_sk / p.sb_sn / p.sb_sk are word strides; see decode_wavesplit_kernel).
int launch_fp8_wavesplit_ue8m0(GemmParams& p, hipStream_t stream, const char* what);

}  // namespace mi355
