// Measurement aid, not an operator: the fp8 matrix-instruction streams of the large-M GEMM kernels with every operand
// held in registers - no LDS, no global loads, no barriers - on all CUs at once.  What such a stream sustains is what the
// chip's power management lets the matrix pipes do on given operand VALUES (the shader clock under it drops well below
// its nominal 2.4 GHz on real operands and not at all on zeros), i.e. the ceiling for any schedule of these instructions.
//   mode 0  v_mfma_f32_16x16x128_f8f6f4 with C = 0 and four promotion FMAs per result, FMAs two results behind the MFMAs
//           (the compute phase of the fp32-scale kernel, gemm_fp8_pp.hip)
//   mode 1  the same MFMA accumulating in place, scales applied by the instruction (the compute phase of the UE8M0 kernel)
//   mode 2  the same MFMA with C = 0 and no vector arithmetic (results only kept alive)
// Each of the 8 waves of a workgroup (two per SIMD, as in the kernels) holds four weight and four token fragments and
// runs `iters` rounds of their 16 products.
#include "common.h"

namespace mi355 {
namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

template <int MODE>
__global__ __launch_bounds__(512) void mfma_stream_kernel(const uint8_t* a, const uint8_t* b, float* out, int iters) {
  const int l = threadIdx.x & 63, wave = threadIdx.x >> 6;
  v8i w[4], t[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int* pa = reinterpret_cast<const int*>(a + ((wave * 4 + i) * 64 + l) * 32);
    const int* pb = reinterpret_cast<const int*>(b + ((wave * 4 + i) * 64 + l) * 32);
#pragma unroll
    for (int x = 0; x < 8; ++x) w[i][x] = pa[x], t[i][x] = pb[x];
  }
  float sc[4] = {1.0f + l * 1e-3f, 0.5f, 0.25f + wave, 2.0f};
  v4f acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
    if constexpr (MODE == 1) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(w[i], t[j], acc[i][j], 0, 0, 0, 127, 0, 127);
    } else {
      v4f part[3];
#pragma unroll
      for (int s = 0; s < 18; ++s) {
        if (s < 16) {
          part[s % 3] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(w[s & 3], t[s >> 2], v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (s > 1) {
          const int pj = (s - 2) >> 2, pi = (s - 2) & 3;
          if constexpr (MODE == 0) {
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[pi][pj][v] = fmaf(part[(s - 2) % 3][v], sc[pj], acc[pi][pj][v]);
          } else {
            asm volatile("" ::"v"(part[(s - 2) % 3]));
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    asm volatile("" : "+v"(w[0]), "+v"(t[0]));  // keeps the loop a loop
  }
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) sum += acc[i][j][v];
  out[blockIdx.x * 512 + threadIdx.x] = sum;
}

}  // namespace
}  // namespace mi355

using namespace mi355;

extern "C" int mi355_probe_fp8_mfma_stream(int mode, int workgroups, int iters, const void* a, const void* b, void* out,
                                           void* stream) {
  const char* what = "mi355_probe_fp8_mfma_stream";
  clear_error();
  MI355_REQUIRE(mode >= 0 && mode <= 2 && workgroups > 0 && workgroups <= 65536 && iters > 0, MI355_ERR_INVALID_ARGUMENT,
                "%s: mode 0..2, 1..65536 workgroups, iters > 0", what);
  MI355_REQUIRE(a && b && out, MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint8_t* pa = static_cast<const uint8_t*>(a);
  const uint8_t* pb = static_cast<const uint8_t*>(b);
  float* po = static_cast<float*>(out);
  switch (mode) {
    case 0: hipLaunchKernelGGL(mfma_stream_kernel<0>, dim3(workgroups), dim3(512), 0, st, pa, pb, po, iters); break;
    case 1: hipLaunchKernelGGL(mfma_stream_kernel<1>, dim3(workgroups), dim3(512), 0, st, pa, pb, po, iters); break;
    default: hipLaunchKernelGGL(mfma_stream_kernel<2>, dim3(workgroups), dim3(512), 0, st, pa, pb, po, iters); break;
  }
  return check_launch(what);
}
