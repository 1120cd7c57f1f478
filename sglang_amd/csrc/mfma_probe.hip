// Measurement aid, not an operator: the fp8 matrix-instruction streams of the large-M GEMM kernels with every operand
// held in registers - no LDS, no global loads, no barriers - on all CUs at once.  What such a stream sustains is what the
// chip's power management lets the matrix pipes do on given operand VALUES (the shader clock under it drops well below
// its nominal 2.4 GHz on real operands and not at all on zeros), i.e. the ceiling for any schedule of these instructions.
//   mode 0  v_mfma_f32_16x16x128_f8f6f4 with C = 0 and four promotion FMAs per result, FMAs two results behind the MFMAs
//           (the compute phase of the fp32-scale kernel, gemm_fp8_pp.hip)
//   mode 1  the same MFMA accumulating in place, scales applied by the instruction (the compute phase of the UE8M0 kernel)
//   mode 2  the same MFMA with C = 0 and no vector arithmetic (results only kept alive)
//   mode 3  v_mfma_f32_32x32x64_f8f6f4 with C = 0 and no vector arithmetic, the same FLOP per round (8 instructions)
// and of the INT8 kernels (mi355_probe_int8_mfma_stream; the same bytes reinterpreted as int8 fragments of 16 bytes):
//   mode 0  v_mfma_i32_16x16x64_i8 accumulating in place (32 per round; what the INT8 kernels use)
//   mode 1  v_mfma_i32_32x32x32_i8 accumulating in place (16 per round)
// Each of the 8 waves of a workgroup (two per SIMD, as in the kernels) holds four weight and four token fragments and
// runs `iters` rounds of their 16 products.
#include "common.h"

namespace mi355 {
namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

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
  if constexpr (MODE == 3) {
    v16f zero, keep;
#pragma unroll
    for (int v = 0; v < 16; ++v) zero[v] = 0.f, keep[v] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int s = 0; s < 8; ++s) {  // 8 instructions of 2 * 32 * 32 * 64 FLOP
        const v16f part = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w[s & 3], t[s >> 1], zero, 0, 0, 0, 0, 0, 0);
        asm volatile("" ::"v"(part));
        if (s == 7) keep = part;
      }
      asm volatile("" : "+v"(w[0]), "+v"(t[0]));
    }
    float sum = 0.f;
#pragma unroll
    for (int v = 0; v < 16; ++v) sum += keep[v];
    out[blockIdx.x * 512 + threadIdx.x] = sum;
    return;
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

template <int MODE>
__global__ __launch_bounds__(512) void int8_mfma_stream_kernel(const uint8_t* a, const uint8_t* b, int* out, int iters) {
  const int l = threadIdx.x & 63, wave = threadIdx.x >> 6;
  v4i w[8], t[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int* pa = reinterpret_cast<const int*>(a + ((wave * 8 + i) * 64 + l) * 16);
    const int* pb = reinterpret_cast<const int*>(b + ((wave * 8 + i) * 64 + l) * 16);
#pragma unroll
    for (int x = 0; x < 4; ++x) w[i][x] = pa[x], t[i][x] = pb[x];
  }
  int sum = 0;
  if constexpr (MODE == 0) {  // 4 x 4 tiles of 16 x 16, two K steps of 64
    v4i acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = v4i{0, 0, 0, 0};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[i * 2 + ks], t[j * 2 + ks], acc[i][j], 0, 0, 0);
      asm volatile("" : "+v"(w[0]), "+v"(t[0]));
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) sum += acc[i][j][v];
  } else {  // 2 x 2 tiles of 32 x 32, four K steps of 32
    v16i acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int i = 0; i < 2; ++i) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w[i * 4 + ks], t[j * 4 + ks], acc[i][j], 0, 0, 0);
      asm volatile("" : "+v"(w[0]), "+v"(t[0]));
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) sum += acc[i][j][v];
  }
  out[blockIdx.x * 512 + threadIdx.x] = sum;
}

}  // namespace
}  // namespace mi355

using namespace mi355;

extern "C" int mi355_probe_fp8_mfma_stream(int mode, int workgroups, int iters, const void* a, const void* b, void* out,
                                           void* stream) {
  const char* what = "mi355_probe_fp8_mfma_stream";
  clear_error();
  MI355_REQUIRE(mode >= 0 && mode <= 3 && workgroups > 0 && workgroups <= 65536 && iters > 0, MI355_ERR_INVALID_ARGUMENT,
                "%s: mode 0..3, 1..65536 workgroups, iters > 0", what);
  MI355_REQUIRE(a && b && out, MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint8_t* pa = static_cast<const uint8_t*>(a);
  const uint8_t* pb = static_cast<const uint8_t*>(b);
  float* po = static_cast<float*>(out);
  switch (mode) {
    case 0: hipLaunchKernelGGL(mfma_stream_kernel<0>, dim3(workgroups), dim3(512), 0, st, pa, pb, po, iters); break;
    case 1: hipLaunchKernelGGL(mfma_stream_kernel<1>, dim3(workgroups), dim3(512), 0, st, pa, pb, po, iters); break;
    case 2: hipLaunchKernelGGL(mfma_stream_kernel<2>, dim3(workgroups), dim3(512), 0, st, pa, pb, po, iters); break;
    default: hipLaunchKernelGGL(mfma_stream_kernel<3>, dim3(workgroups), dim3(512), 0, st, pa, pb, po, iters); break;
  }
  return check_launch(what);
}

extern "C" int mi355_probe_int8_mfma_stream(int mode, int workgroups, int iters, const void* a, const void* b, void* out,
                                            void* stream) {
  const char* what = "mi355_probe_int8_mfma_stream";
  clear_error();
  MI355_REQUIRE(mode >= 0 && mode <= 1 && workgroups > 0 && workgroups <= 65536 && iters > 0, MI355_ERR_INVALID_ARGUMENT,
                "%s: mode 0..1, 1..65536 workgroups, iters > 0", what);
  MI355_REQUIRE(a && b && out, MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint8_t* pa = static_cast<const uint8_t*>(a);
  const uint8_t* pb = static_cast<const uint8_t*>(b);
  int* po = static_cast<int*>(out);
  if (mode == 0) hipLaunchKernelGGL(int8_mfma_stream_kernel<0>, dim3(workgroups), dim3(512), 0, st, pa, pb, po, iters);
  else hipLaunchKernelGGL(int8_mfma_stream_kernel<1>, dim3(workgroups), dim3(512), 0, st, pa, pb, po, iters);
  return check_launch(what);
}
