// Grouped blockwise-scaled FP8 GEMM for gfx950: the expert GEMMs of a mixture-of-experts layer in one call.
//
// What the reference's fp8_blockwise_scaled_grouped_mm computes (sgl-kernel/csrc/moe/fp8_blockwise_moe_kernel.cu:650-810,
// per-expert operand addresses as in sgl-kernel/csrc/moe/cutlass_moe_helper.cu:37-69): token rows of all experts are
// stacked in one matrix a [total_m, K] with their 1 x 128 group scales [total_m, K / 128]; expert e owns the rows
// expert_offsets[e] .. + problem_sizes[e][0], multiplies them with its own weight b[e] [N, K] (128 x 128 block scales
// scales_b[e] [N / 128, K / 128]) and writes the same rows of out [total_m, N].  problem_sizes and expert_offsets live
// on the device (they come out of the routing kernel), so the tile schedule is built on the device too:
//   1. grouped_plan_kernel  - one workgroup; prefix sums over the experts' tile counts turn the problem sizes into one
//      record per token tile (expert, rows, position) in two tables, 256-row tiles and 64/128-row tiles, each headed by
//      its number of records; sizes are clamped into the stacked matrix, so inconsistent routing data cannot make a later kernel read
//      or write out of bounds;
//   2. grouped_relayout_scales_kernel - token scales re-laid out M-major (what the direct-to-LDS GEMMs read with 16-byte
//      loads), every expert padded to start on a whole quad of rows;
//   3. fp8_grouped_pp_kernel (gemm_fp8_pp.hip), the two-phase 256 x 256 tile kernel, over the first table, then
//      fp8_grouped_dma3_kernel (gemm_fp8_dma3.hip), the three-stage (64 or 128) x 256 tile kernel, over the second:
//      one workgroup per (token tile, channel tile).  The first launch is left out when no expert can have more than
//      128 rows.
// Where the reference takes device arrays of per-expert pointers, strides and scale layouts as scratch that its own
// set-up kernel fills, this interface takes the base pointers and strides and keeps its scratch in the workspace.
#include "gemm_common.h"

namespace mi355 {
namespace {

size_t align256(size_t b) { return (b + 255) & ~(size_t)255; }

// Tile heights.  An expert's rows are cut into 256-row tiles for the two-phase kernel; what is left (fewer than 256 rows)
// becomes one more 256-row tile when it is more than 128 rows, otherwise 64- or 128-row tiles for the three-stage kernel
// (one height per call, chosen on the host from the average rows per expert).  Measured on the dense kernels: per output
// element a 128-row tile costs 1.5x and a 64-row tile 2.3x of a 256-row tile when both are bound by the matrix pipe.
constexpr int BIG = 256;

struct ExpertTiles {
  int row0, rows, big, small, small_first;  // tiles of each kind; first row (inside the expert) of the small tiles
};
__device__ __forceinline__ ExpertTiles expert_tiles(const int32_t* problem_sizes, const int32_t* expert_offsets, int e, int E,
                                                    int total_m, int bm) {
  ExpertTiles t{0, 0, 0, 0, 0};
  if (e >= E) return t;
  t.row0 = min(max(expert_offsets[e], 0), total_m);
  t.rows = min(max(problem_sizes[3 * e], 0), total_m - t.row0);
  t.big = t.rows / BIG;
  const int rest = t.rows - t.big * BIG;
  if (rest > 128) t.big += 1;
  else t.small = (rest + bm - 1) / bm;
  t.small_first = t.big * BIG;
  return t;
}

__global__ __launch_bounds__(256) void grouped_plan_kernel(const int32_t* problem_sizes, const int32_t* expert_offsets, int E,
                                                           int total_m, int bm, v4i* big_tiles, int max_big, v4i* small_tiles,
                                                           int max_small) {
  __shared__ int scan_b[256], scan_s[256];
  int base_b = 0, base_s = 0;
  for (int c = 0; c < E; c += 256) {
    const int e = c + (int)threadIdx.x;
    const ExpertTiles t = expert_tiles(problem_sizes, expert_offsets, e, E, total_m, bm);
    scan_b[threadIdx.x] = t.big, scan_s[threadIdx.x] = t.small;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {  // inclusive prefix sums
      const int vb = (int)threadIdx.x >= d ? scan_b[threadIdx.x - d] : 0;
      const int vs = (int)threadIdx.x >= d ? scan_s[threadIdx.x - d] : 0;
      __syncthreads();
      scan_b[threadIdx.x] += vb, scan_s[threadIdx.x] += vs;
      __syncthreads();
    }
    const int first_b = base_b + scan_b[threadIdx.x] - t.big, first_s = base_s + scan_s[threadIdx.x] - t.small;
    for (int j = 0; j < t.big; ++j)
      if (first_b + j < max_big) big_tiles[1 + first_b + j] = v4i{e, t.row0, t.rows, j * BIG};
    for (int j = 0; j < t.small; ++j)
      if (first_s + j < max_small) small_tiles[1 + first_s + j] = v4i{e, t.row0, t.rows, t.small_first + j * bm};
    base_b += scan_b[255], base_s += scan_s[255];
    __syncthreads();
  }
  // record 0 of each table: how many follow (consistent routing data never exceeds the bounds)
  if (threadIdx.x == 0) {
    big_tiles[0] = v4i{min(base_b, max_big), 0, 0, 0};
    small_tiles[0] = v4i{min(base_s, max_small), 0, 0, 0};
  }
}

// out[kb * pitch + col(e) + m] = sa[(row0 + m) * sa_sm + kb * sa_sk], col(e) = ((row0 + 3) & ~3) + 4 * e.
// Up to 128 rows x 32 K blocks per workgroup, through LDS so that both sides are contiguous.  blockIdx.x walks the two
// halves of every 256-row tile record, then the small tile records.
__global__ __launch_bounds__(256) void grouped_relayout_scales_kernel(const float* sa, int64_t sa_sm, int64_t sa_sk, float* out,
                                                                      int64_t pitch, int KB, int bm, const v4i* big_tiles,
                                                                      int max_big, const v4i* small_tiles) {
  __shared__ float tile[32][129];
  const bool is_big = (int)blockIdx.x < 2 * max_big;
  const int idx = is_big ? (int)(blockIdx.x >> 1) : (int)blockIdx.x - 2 * max_big;
  const v4i* table = is_big ? big_tiles : small_tiles;
  if (idx >= table[0].x) return;
  const v4i rec = table[1 + idx];
  const int first = rec.w + (is_big ? (int)(blockIdx.x & 1) * 128 : 0);  // first row, inside the expert
  const int rows = min(is_big ? 128 : bm, rec.z - first);
  if (rows <= 0) return;
  const int k0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const float* src = sa + (int64_t)(rec.y + first) * sa_sm;
  if (k0 + tx < KB)
    for (int r = ty; r < rows; r += 8) tile[tx][r] = src[(int64_t)r * sa_sm + (int64_t)(k0 + tx) * sa_sk];
  __syncthreads();
  float* dst = out + ((rec.y + 3) & ~3) + 4 * rec.x + first;
  for (int i = threadIdx.x; i < 32 * 128; i += 256) {
    const int kk = i >> 7, m = i & 127;
    if (m < rows && k0 + kk < KB) dst[(int64_t)(k0 + kk) * pitch + m] = tile[kk][m];
  }
}

struct GroupedPlan {
  int bm;                  // height of the small tiles
  int max_big, max_small;  // upper bounds on the number of tile records of each kind
  int64_t pitch;           // floats per K block in the re-laid-out token scales
  size_t big_bytes, small_bytes, scale_bytes;
};

GroupedPlan grouped_plan(int64_t E, int64_t total_m, int64_t K) {
  GroupedPlan pl;
  pl.bm = total_m > 64 * E ? 128 : 64;  // by the average rows per expert; the sizes themselves are on the device
  pl.max_big = (int)(total_m / 129);    // every 256-row tile covers more than 128 rows
  // an expert leaves at most 128 rows to small tiles, and every small tile covers at least one row
  pl.max_small = (int)std::min<int64_t>(total_m, E * (128 / pl.bm));
  // the last expert's column is at most align4(total_m) - rows + 4 (E - 1) + 3, and the GEMM reads whole quads up to
  // align4(rows) past it: one more quad of slack keeps that inside the row (and inside the workspace for the last row)
  pl.pitch = ((total_m + 3) & ~3ll) + 4 * E + 4;
  pl.big_bytes = align256((size_t)(pl.max_big + 1) * sizeof(v4i));  // record 0 holds the count
  pl.small_bytes = align256((size_t)(pl.max_small + 1) * sizeof(v4i));
  pl.scale_bytes = align256((size_t)pl.pitch * (size_t)((K + KSTEP - 1) / KSTEP) * 4u);
  return pl;
}

}  // namespace
}  // namespace mi355

using namespace mi355;

extern "C" size_t mi355_fp8_blockwise_scaled_grouped_mm_workspace_bytes(int64_t num_experts, int64_t total_m, int64_t N,
                                                                        int64_t K) {
  if (num_experts <= 0 || total_m <= 0 || N <= 0 || K <= 0) return 0;
  const GroupedPlan pl = grouped_plan(num_experts, total_m, K);
  return pl.big_bytes + pl.small_bytes + pl.scale_bytes;
}

extern "C" int mi355_fp8_blockwise_scaled_grouped_mm_plan(int64_t num_experts, int64_t total_m, int64_t N, int64_t K, char* buf,
                                                          size_t buf_len) {
  const char* what = "mi355_fp8_blockwise_scaled_grouped_mm_plan";
  clear_error();
  MI355_REQUIRE(buf && buf_len > 0, MI355_ERR_INVALID_ARGUMENT, "%s: no buffer", what);
  MI355_REQUIRE(num_experts > 0 && total_m > 0 && N > 0 && K > 0, MI355_ERR_INVALID_ARGUMENT, "%s: empty problem", what);
  const GroupedPlan pl = grouped_plan(num_experts, total_m, K);
  snprintf(buf, buf_len, "kernel=grouped_pingpong+grouped_dma3 small_tile=%dx256 max_big_tiles=%d max_small_tiles=%d tiles_n=%lld",
           pl.bm, pl.max_big, pl.max_small, (long long)((N + 255) / 256));
  return MI355_OK;
}

extern "C" int mi355_fp8_blockwise_scaled_grouped_mm(const void* a, const void* b, const float* scales_a, const float* scales_b,
                                                     void* out, int out_dtype, const int32_t* problem_sizes,
                                                     const int32_t* expert_offsets, int64_t num_experts, int64_t total_m,
                                                     int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t b_expert_stride,
                                                     int64_t sa_sm, int64_t sa_sk, int64_t sb_expert_stride, int64_t sb_sn,
                                                     int64_t sb_sk, int64_t ldo, void* workspace, size_t workspace_bytes,
                                                     void* stream) {
  const char* what = "mi355_fp8_blockwise_scaled_grouped_mm";
  clear_error();
  MI355_REQUIRE(num_experts >= 0 && total_m >= 0 && N >= 0 && K >= 0, MI355_ERR_INVALID_ARGUMENT, "%s: negative shape", what);
  MI355_REQUIRE(out_dtype == MI355_BF16 || out_dtype == MI355_F16, MI355_ERR_INVALID_ARGUMENT,
                "%s: out_dtype must be bfloat16 or float16", what);
  if (num_experts == 0 || total_m == 0 || N == 0) return MI355_OK;
  MI355_REQUIRE(K > 0, MI355_ERR_INVALID_ARGUMENT, "%s: K must be positive", what);
  MI355_REQUIRE(a && b && scales_a && scales_b && out && problem_sizes && expert_offsets, MI355_ERR_INVALID_ARGUMENT,
                "%s: null pointer", what);
  MI355_REQUIRE(lda >= K && ldb >= K && ldo >= N, MI355_ERR_INVALID_ARGUMENT, "%s: row strides smaller than the row length", what);
  MI355_REQUIRE(K % KSTEP == 0, MI355_ERR_UNSUPPORTED, "%s: K must be a multiple of 128", what);
  MI355_REQUIRE(lda % 16 == 0 && ldb % 16 == 0 && b_expert_stride % 16 == 0 && (reinterpret_cast<uintptr_t>(a) & 15) == 0 &&
                    (reinterpret_cast<uintptr_t>(b) & 15) == 0,
                MI355_ERR_UNSUPPORTED, "%s: operand rows and expert strides must be 16-byte aligned", what);
  MI355_REQUIRE(num_experts < (1 << 24) && total_m < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31) &&
                    total_m * lda < (1ll << 32) && N * ldb < (1ll << 32),
                MI355_ERR_INVALID_ARGUMENT, "%s: dimensions out of range (row offsets must stay below 4 GiB)", what);
  const GroupedPlan pl = grouped_plan(num_experts, total_m, K);
  MI355_REQUIRE(((int64_t)pl.max_big + pl.max_small) * ((N + 255) / 256) < (1ll << 31), MI355_ERR_INVALID_ARGUMENT,
                "%s: too many tiles", what);
  const size_t need = pl.big_bytes + pl.small_bytes + pl.scale_bytes;
  MI355_REQUIRE(workspace && workspace_bytes >= need, MI355_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", what,
                need, workspace_bytes);
  MI355_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, MI355_ERR_INVALID_ARGUMENT,
                "%s: workspace must be 256-byte aligned", what);

  hipStream_t st = static_cast<hipStream_t>(stream);
  uint8_t* wsp = static_cast<uint8_t*>(workspace);
  v4i* big_tiles = reinterpret_cast<v4i*>(wsp);
  v4i* small_tiles = reinterpret_cast<v4i*>(wsp + pl.big_bytes);
  float* sa_mm = reinterpret_cast<float*>(wsp + pl.big_bytes + pl.small_bytes);
  const int KB = (int)(K / KSTEP);
  hipLaunchKernelGGL(grouped_plan_kernel, dim3(1), dim3(256), 0, st, problem_sizes, expert_offsets, (int)num_experts, (int)total_m,
                     pl.bm, big_tiles, pl.max_big, small_tiles, pl.max_small);
  int rc = check_launch(what);
  if (rc != MI355_OK) return rc;
  hipLaunchKernelGGL(grouped_relayout_scales_kernel, dim3((unsigned)(2 * pl.max_big + pl.max_small), (unsigned)((KB + 31) / 32)),
                     dim3(256), 0, st, scales_a, sa_sm, sa_sk, sa_mm, pl.pitch, KB, pl.bm, big_tiles, pl.max_big, small_tiles);
  rc = check_launch(what);
  if (rc != MI355_OK) return rc;

  GroupedParams gp{};
  gp.g.a = static_cast<const uint8_t*>(a);
  gp.g.b = static_cast<const uint8_t*>(b);
  gp.g.sa = sa_mm, gp.g.sb = scales_b, gp.g.out = out;
  gp.g.M = 0, gp.g.N = (int)N, gp.g.K = (int)K;
  gp.g.lda = lda, gp.g.ldb = ldb, gp.g.ldo = ldo;
  gp.g.sa_sm = 1, gp.g.sa_sk = pl.pitch, gp.g.sb_sn = sb_sn, gp.g.sb_sk = sb_sk;
  gp.g.kb_total = KB;
  gp.g.out_dtype = out_dtype;
  gp.b_expert_stride = b_expert_stride;
  gp.sb_expert_stride = sb_expert_stride;
  gp.out_elem = 2;
  if (pl.max_big > 0) {
    gp.tiles = big_tiles, gp.max_tiles_m = pl.max_big;
    rc = launch_fp8_grouped_pp(gp, st, what);
    if (rc != MI355_OK) return rc;
  }
  gp.tiles = small_tiles, gp.max_tiles_m = pl.max_small;
  return launch_fp8_grouped_dma3(gp, pl.bm, st, what);
}
