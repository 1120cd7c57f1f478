// Grouped blockwise-scaled FP8 GEMM for gfx950: the expert GEMMs of a mixture-of-experts layer in one call.
//
// What the reference's fp8_blockwise_scaled_grouped_mm computes (sgl-kernel/csrc/moe/fp8_blockwise_moe_kernel.cu:650-810,
// per-expert operand addresses as in sgl-kernel/csrc/moe/cutlass_moe_helper.cu:37-69): token rows of all experts are
// stacked in one matrix a [total_m, K] with their 1 x 128 group scales [total_m, K / 128]; expert e owns the rows
// expert_offsets[e] .. + problem_sizes[e][0], multiplies them with its own weight b[e] [N, K] (128 x 128 block scales
// scales_b[e] [N / 128, K / 128]) and writes the same rows of out [total_m, N].  problem_sizes and expert_offsets live
// on the device (they come out of the routing kernel), so the tile schedule is built on the device too:
//   1. grouped_plan_kernel  - one workgroup; a prefix sum over the experts' tile counts turns the problem sizes into one
//      record per token tile (expert, rows, position), unused records marked; sizes are clamped into the stacked matrix,
//      so inconsistent routing data cannot make a later kernel read or write out of bounds;
//   2. grouped_relayout_scales_kernel - token scales re-laid out M-major (what the direct-to-LDS GEMM reads with 16-byte
//      loads), every expert padded to start on a whole quad of rows;
//   3. fp8_grouped_dma3_kernel (gemm_fp8_dma3.hip) - the three-stage (64 or 128) x 256 tile kernel, one workgroup per
//      (token tile, channel tile).
// Where the reference takes device arrays of per-expert pointers, strides and scale layouts as scratch that its own
// set-up kernel fills, this interface takes the base pointers and strides and keeps its scratch in the workspace.
#include "gemm_common.h"

namespace mi355 {
namespace {

size_t align256(size_t b) { return (b + 255) & ~(size_t)255; }

__global__ __launch_bounds__(256) void grouped_plan_kernel(const int32_t* problem_sizes, const int32_t* expert_offsets, int E,
                                                           int total_m, int bm, v4i* tiles, int max_tiles) {
  __shared__ int scan[256];
  int base = 0;
  for (int c = 0; c < E; c += 256) {
    const int e = c + (int)threadIdx.x;
    int row0 = 0, rows = 0;
    if (e < E) {
      row0 = min(max(expert_offsets[e], 0), total_m);
      rows = min(max(problem_sizes[3 * e], 0), total_m - row0);
    }
    const int nt = (rows + bm - 1) / bm;
    scan[threadIdx.x] = nt;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {  // inclusive prefix sum
      const int v = (int)threadIdx.x >= d ? scan[threadIdx.x - d] : 0;
      __syncthreads();
      scan[threadIdx.x] += v;
      __syncthreads();
    }
    const int first = base + scan[threadIdx.x] - nt;
    for (int j = 0; j < nt; ++j)
      if (first + j < max_tiles) tiles[first + j] = v4i{e, row0, rows, j * bm};
    base += scan[255];
    __syncthreads();
  }
  for (int i = min(base, max_tiles) + (int)threadIdx.x; i < max_tiles; i += 256) tiles[i] = v4i{-1, 0, 0, 0};
}

// out[kb * pitch + col(e) + m] = sa[(row0 + m) * sa_sm + kb * sa_sk], col(e) = ((row0 + 3) & ~3) + 4 * e.
// One token tile x 32 K blocks per workgroup, through LDS so that both sides are contiguous.
__global__ __launch_bounds__(256) void grouped_relayout_scales_kernel(const float* sa, int64_t sa_sm, int64_t sa_sk, float* out,
                                                                      int64_t pitch, int KB, int bm, const v4i* tiles) {
  __shared__ float tile[32][129];
  const v4i rec = tiles[blockIdx.x];
  if (rec.x < 0) return;
  const int rows = min(bm, rec.z - rec.w);
  const int k0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const float* src = sa + (int64_t)(rec.y + rec.w) * sa_sm;
  if (k0 + tx < KB)
    for (int r = ty; r < rows; r += 8) tile[tx][r] = src[(int64_t)r * sa_sm + (int64_t)(k0 + tx) * sa_sk];
  __syncthreads();
  float* dst = out + ((rec.y + 3) & ~3) + 4 * rec.x + rec.w;
  for (int i = threadIdx.x; i < 32 * bm; i += 256) {
    const int kk = i / bm, m = i - kk * bm;
    if (m < rows && k0 + kk < KB) dst[(int64_t)(k0 + kk) * pitch + m] = tile[kk][m];
  }
}

struct GroupedPlan {
  int bm;            // token-tile height
  int max_tiles_m;   // upper bound on the number of token tiles: every expert adds at most one partial tile
  int64_t pitch;     // floats per K block in the re-laid-out token scales
  size_t table_bytes, scale_bytes;
};

GroupedPlan grouped_plan(int64_t E, int64_t total_m, int64_t K) {
  GroupedPlan pl;
  pl.bm = total_m > 64 * E ? 128 : 64;  // by the average rows per expert; the sizes themselves are on the device
  pl.max_tiles_m = (int)(total_m / pl.bm + std::min<int64_t>(E, total_m));
  pl.pitch = ((total_m + 3) & ~3ll) + 4 * E;
  pl.table_bytes = align256((size_t)pl.max_tiles_m * sizeof(v4i));
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
  return pl.table_bytes + pl.scale_bytes;
}

extern "C" int mi355_fp8_blockwise_scaled_grouped_mm_plan(int64_t num_experts, int64_t total_m, int64_t N, int64_t K, char* buf,
                                                          size_t buf_len) {
  const char* what = "mi355_fp8_blockwise_scaled_grouped_mm_plan";
  clear_error();
  MI355_REQUIRE(buf && buf_len > 0, MI355_ERR_INVALID_ARGUMENT, "%s: no buffer", what);
  MI355_REQUIRE(num_experts > 0 && total_m > 0 && N > 0 && K > 0, MI355_ERR_INVALID_ARGUMENT, "%s: empty problem", what);
  const GroupedPlan pl = grouped_plan(num_experts, total_m, K);
  snprintf(buf, buf_len, "kernel=grouped_dma3 tile=%dx256 max_tiles_m=%d tiles_n=%lld", pl.bm, pl.max_tiles_m,
           (long long)((N + 255) / 256));
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
  MI355_REQUIRE((int64_t)pl.max_tiles_m * ((N + 255) / 256) < (1ll << 31), MI355_ERR_INVALID_ARGUMENT, "%s: too many tiles", what);
  const size_t need = pl.table_bytes + pl.scale_bytes;
  MI355_REQUIRE(workspace && workspace_bytes >= need, MI355_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", what,
                need, workspace_bytes);
  MI355_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, MI355_ERR_INVALID_ARGUMENT,
                "%s: workspace must be 256-byte aligned", what);

  hipStream_t st = static_cast<hipStream_t>(stream);
  v4i* tiles = static_cast<v4i*>(workspace);
  float* sa_mm = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + pl.table_bytes);
  const int KB = (int)(K / KSTEP);
  hipLaunchKernelGGL(grouped_plan_kernel, dim3(1), dim3(256), 0, st, problem_sizes, expert_offsets, (int)num_experts, (int)total_m,
                     pl.bm, tiles, pl.max_tiles_m);
  int rc = check_launch(what);
  if (rc != MI355_OK) return rc;
  hipLaunchKernelGGL(grouped_relayout_scales_kernel, dim3((unsigned)pl.max_tiles_m, (unsigned)((KB + 31) / 32)), dim3(256), 0, st,
                     scales_a, sa_sm, sa_sk, sa_mm, pl.pitch, KB, pl.bm, tiles);
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
  gp.tiles = tiles;
  gp.b_expert_stride = b_expert_stride;
  gp.sb_expert_stride = sb_expert_stride;
  gp.max_tiles_m = pl.max_tiles_m;
  gp.out_elem = 2;
  return launch_fp8_grouped_dma3(gp, pl.bm, st, what);
}
