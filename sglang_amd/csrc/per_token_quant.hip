// Per-token (per-row) symmetric 8-bit quantizers for gfx950.
//
// One workgroup per row: 16-byte loads, |x| max over the row (DPP inside a wave, LDS across the four
// waves), then
//   INT8: q = round-half-away(x * (127 / absmax)) with absmax floored at 1e-10 and scale = absmax / 127, as in
//         python/sglang/srt/layers/quantization/int8_kernel.py:47-50;
//   FP8:  scale = absmax / 448 (no floor), q = e4m3fn(clamp(x * (1 / scale))) rounded to nearest even, a row of zeros
//         gives scale 0 and zeros, as in sgl-kernel/csrc/gemm/per_token_quant_fp8.cu:15-85.
//   FP8, whole row as ONE quantization group (per_token_group_quant_fp8 with group_size == K, what the reference
//         quantizes a 16-bit checkpoint's weights with at load time, python/sglang/srt/layers/quantization/fp8.py:368-375):
//         scale = max(absmax, eps) / 448 and either q = e4m3fn(clamp(x * (1 / scale))), the arithmetic of the Triton kernel
//         python/sglang/srt/layers/quantization/fp8_kernel.py:122-161, or q = e4m3fn(clamp(x / scale)) with a true
//         division, the arithmetic of sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:25-114.
// Rows of up to 8192 two-byte elements stay in registers between the two phases; longer rows are
// re-read (from L2).
// Two-byte inputs with rows of at most 8192 elements (every hidden size of the benchmark models) take a second kernel: one
// WAVE per row, four rows per workgroup, the row in registers (up to 16 x 16 bytes per lane), no LDS and no barrier -
// 16384 workgroups of one short row each spend a visible share of their life starting up and at the barrier.
#include "common.h"

namespace mi355 {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <int DT>
__device__ __forceinline__ void unpack16(const u32x4& r, float* f) {
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
  if constexpr (DT == MI355_F32) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(w[i]);
  } else if constexpr (DT == MI355_BF16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(w[i] << 16);
      f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = f16_bits_to_f32(w[i] & 0xffffu);
      f[2 * i + 1] = f16_bits_to_f32(w[i] >> 16);
    }
  }
}

__device__ __forceinline__ float wave_allreduce_max(float v) {
  // row_shr-free butterfly inside 16-lane rows, then across rows with ds_swizzle-free readlane
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true)));
  float r = fmaxf(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0)),
                  __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16)));
  r = fmaxf(r, __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32)));
  r = fmaxf(r, __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48)));
  return r;
}

// Sum over the wave, the same value in every lane (butterfly over 16-lane rows, then the four rows in lane order).
__device__ __forceinline__ float wave_allreduce_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true));
  float r = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0)) + __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  r += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  r += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return r;
}

// The row sum leaves in the input's type (int8_kernel.py:52-54: `x_sum.to(x_sum_ptr.dtype.element_ty)`).
template <int DT>
__device__ __forceinline__ void store_row_sum(void* x_sum, int64_t row, float v) {
  if constexpr (DT == MI355_F32) reinterpret_cast<float*>(x_sum)[row] = v;
  else reinterpret_cast<uint16_t*>(x_sum)[row] = (uint16_t)(DT == MI355_BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v));
}

// Scale of a row from its |x| maximum (written by the caller) and the factor the elements are multiplied with.
template <bool FP8_OUT>
__device__ __forceinline__ float row_scale(float amax, float& mul) {
  if constexpr (FP8_OUT) {
    const float scale = amax / 448.0f;
    mul = (scale == 0.f) ? 0.f : 1.0f / scale;
    return scale;
  } else {
    mul = 127.0f / amax;
    return amax / 127.0f;
  }
}

// One 16-byte vector of input -> 4 or 8 codes at d.  DIVIDE: `mul` is the scale and the elements are divided by it.
template <int DT, bool FP8_OUT, bool STREAM, bool DIVIDE = false>
__device__ __forceinline__ void emit_vector(const u32x4& raw, float mul, int8_t* d) {
  constexpr int VEC = (DT == MI355_F32) ? 4 : 8;
  float f[VEC];
  unpack16<DT>(raw, f);
  uint32_t w[VEC / 4];
#pragma unroll
  for (int j = 0; j < VEC / 4; ++j) {
    uint32_t pk = 0;
    if constexpr (FP8_OUT) {
      float t[4];
#pragma unroll
      for (int b = 0; b < 4; ++b) t[b] = fmaxf(fminf(DIVIDE ? f[4 * j + b] / mul : f[4 * j + b] * mul, 448.0f), -448.0f);
      int c = __builtin_amdgcn_cvt_pk_fp8_f32(t[0], t[1], 0, false);
      c = __builtin_amdgcn_cvt_pk_fp8_f32(t[2], t[3], c, true);
      pk = (uint32_t)c;
    } else {
#pragma unroll
      for (int b = 0; b < 4; ++b) pk |= ((uint32_t)(int)roundf(f[4 * j + b] * mul) & 0xffu) << (8 * b);
    }
    w[j] = pk;
  }
  if constexpr (VEC == 8) {
    if constexpr (STREAM) __builtin_nontemporal_store(u32x2{w[0], w[1]}, reinterpret_cast<u32x2*>(d));
    else *reinterpret_cast<u32x2*>(d) = u32x2{w[0], w[1]};
  } else {
    *reinterpret_cast<uint32_t*>(d) = w[0];
  }
}

// One wave per row, the row in registers: NV vectors of eight two-byte elements per lane (K <= 512 * NV).
// SUM (INT8 only): also the fp32 sum of the row, rounded to the input's type (per_token_quant_int8(cal_sum=True)).
template <int DT, bool FP8_OUT, int NV, bool SUM = false>
__global__ __launch_bounds__(256) void per_token_quant_wave_kernel(const void* x, int8_t* q, float* s, int64_t M, int64_t K,
                                                                   void* x_sum = nullptr) {
  static_assert(DT != MI355_F32, "two-byte inputs");
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const int nvec = (int)(K / 8);
  const u32x4* src = reinterpret_cast<const u32x4*>(x) + row * nvec;
  u32x4 keep[NV];
  float amax = FP8_OUT ? 0.f : 1e-10f;
  [[maybe_unused]] float total = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = lane + 64 * i;
    keep[i] = (v < nvec) ? __builtin_nontemporal_load(src + v) : u32x4{0, 0, 0, 0};
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    float f[8];
    unpack16<DT>(keep[i], f);
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(f[j]));
    if constexpr (SUM) {
#pragma unroll
      for (int j = 0; j < 8; ++j) total += f[j];
    }
  }
  amax = wave_allreduce_max(amax);
  float mul;
  const float scale = row_scale<FP8_OUT>(amax, mul);
  if (lane == 0) s[row] = scale;
  if constexpr (SUM) {
    total = wave_allreduce_sum(total);
    if (lane == 0) store_row_sum<DT>(x_sum, row, total);
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = lane + 64 * i;
    if (v < nvec) emit_vector<DT, FP8_OUT, true>(keep[i], mul, q + row * K + (int64_t)v * 8);
  }
}

// ROW_GROUP (FP8 only): the row is one quantization group: absmax floored at eps; DIVIDE: elements are divided by the
// scale instead of multiplied by its reciprocal.
template <int DT, bool FP8_OUT, bool ROW_GROUP = false, bool DIVIDE = false, bool SUM = false>
__global__ __launch_bounds__(256) void per_token_quant_kernel(const void* x, int8_t* q, float* s, int64_t K, float eps,
                                                              void* x_sum = nullptr) {
  static_assert(FP8_OUT || !ROW_GROUP, "whole-row groups are built for FP8 codes");
  static_assert(ROW_GROUP || !DIVIDE, "division is a mode of the whole-row group");
  constexpr int VEC = (DT == MI355_F32) ? 4 : 8;
  constexpr int KEEP = 4;  // vectors per thread kept in registers
  __shared__ float wave_max[4];
  __shared__ float wave_sum[4];
  [[maybe_unused]] float total = 0.f;
  const int64_t row = blockIdx.x;
  const int64_t nvec = K / VEC;
  const u32x4* src = reinterpret_cast<const u32x4*>(x) + row * nvec;
  u32x4 keep[KEEP];
  float amax = ROW_GROUP ? eps : (FP8_OUT ? 0.f : 1e-10f);
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int64_t v = threadIdx.x + 256 * i;
    keep[i] = (v < nvec) ? src[v] : u32x4{0, 0, 0, 0};
    float f[VEC];
    unpack16<DT>(keep[i], f);
#pragma unroll
    for (int j = 0; j < VEC; ++j) amax = fmaxf(amax, fabsf(f[j]));
    if constexpr (SUM) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) total += f[j];
    }
  }
  for (int64_t v = threadIdx.x + 256 * KEEP; v < nvec; v += 256) {
    float f[VEC];
    unpack16<DT>(src[v], f);
#pragma unroll
    for (int j = 0; j < VEC; ++j) amax = fmaxf(amax, fabsf(f[j]));
    if constexpr (SUM) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) total += f[j];
    }
  }
  amax = wave_allreduce_max(amax);
  if constexpr (SUM) total = wave_allreduce_sum(total);
  if ((threadIdx.x & 63) == 0) {
    wave_max[threadIdx.x >> 6] = amax;
    if constexpr (SUM) wave_sum[threadIdx.x >> 6] = total;
  }
  __syncthreads();
  if constexpr (SUM) {
    if (threadIdx.x == 0) store_row_sum<DT>(x_sum, row, (wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3]));
  }
  amax = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
  float mul;
  float scale = row_scale<FP8_OUT>(amax, mul);
  if constexpr (ROW_GROUP) {
    scale = amax / 448.0f;  // amax >= eps > 0
    mul = DIVIDE ? scale : 1.0f / scale;
  }
  if (threadIdx.x == 0) s[row] = scale;

  auto emit = [&](const u32x4& raw, int64_t v) { emit_vector<DT, FP8_OUT, false, DIVIDE>(raw, mul, q + row * K + v * VEC); };
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int64_t v = threadIdx.x + 256 * i;
    if (v < nvec) emit(keep[i], v);
  }
  for (int64_t v = threadIdx.x + 256 * KEEP; v < nvec; v += 256) emit(src[v], v);
}

}  // namespace
}  // namespace mi355

namespace mi355 {
namespace {

template <bool FP8_OUT, bool ROW_GROUP = false, bool DIVIDE = false, bool SUM = false>
int per_token_quant(const char* what, const void* x, int x_dtype, void* q, float* s, int64_t M, int64_t K, void* stream,
                    float eps = 0.f, void* x_sum = nullptr) {
  clear_error();
  MI355_REQUIRE(M >= 0 && K >= 0, MI355_ERR_INVALID_ARGUMENT, "%s: negative shape", what);
  MI355_REQUIRE(x_dtype == MI355_F32 || x_dtype == MI355_F16 || x_dtype == MI355_BF16, MI355_ERR_INVALID_ARGUMENT,
                "%s: input must be float32, float16 or bfloat16", what);
  if (M == 0 || K == 0) return MI355_OK;
  MI355_REQUIRE(x && q && s && (!SUM || x_sum), MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  MI355_REQUIRE((K * (int64_t)dtype_size(x_dtype)) % 16 == 0, MI355_ERR_UNSUPPORTED,
                "%s: a row must span a multiple of 16 input bytes", what);
  MI355_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)q % 8 == 0), MI355_ERR_INVALID_ARGUMENT,
                "%s: input must be 16-byte and output 8-byte aligned", what);
  MI355_REQUIRE(M < (1ll << 31), MI355_ERR_INVALID_ARGUMENT, "%s: too many rows", what);
  hipStream_t st = static_cast<hipStream_t>(stream);
  int8_t* qq = static_cast<int8_t*>(q);
  if (!ROW_GROUP && x_dtype != MI355_F32 && K <= 8192) {  // one wave per row
    const dim3 grid((unsigned)((M + 3) / 4));
    const int nv = (int)((K / 8 + 63) / 64);
#define MI355_WAVE_ROWS(DT, NV) \
  hipLaunchKernelGGL((per_token_quant_wave_kernel<DT, FP8_OUT, NV, SUM>), grid, dim3(256), 0, st, x, qq, s, M, K, x_sum)
    if (x_dtype == MI355_BF16) {
      if (nv <= 4) MI355_WAVE_ROWS(MI355_BF16, 4);
      else if (nv <= 8) MI355_WAVE_ROWS(MI355_BF16, 8);
      else MI355_WAVE_ROWS(MI355_BF16, 16);
    } else {
      if (nv <= 4) MI355_WAVE_ROWS(MI355_F16, 4);
      else if (nv <= 8) MI355_WAVE_ROWS(MI355_F16, 8);
      else MI355_WAVE_ROWS(MI355_F16, 16);
    }
#undef MI355_WAVE_ROWS
    return check_launch(what);
  }
  switch (x_dtype) {
    case MI355_F32:
      hipLaunchKernelGGL((per_token_quant_kernel<MI355_F32, FP8_OUT, ROW_GROUP, DIVIDE, SUM>), dim3((unsigned)M), dim3(256), 0, st, x, qq, s, K, eps, x_sum);
      break;
    case MI355_F16:
      hipLaunchKernelGGL((per_token_quant_kernel<MI355_F16, FP8_OUT, ROW_GROUP, DIVIDE, SUM>), dim3((unsigned)M), dim3(256), 0, st, x, qq, s, K, eps, x_sum);
      break;
    default:
      hipLaunchKernelGGL((per_token_quant_kernel<MI355_BF16, FP8_OUT, ROW_GROUP, DIVIDE, SUM>), dim3((unsigned)M), dim3(256), 0, st, x, qq, s, K, eps, x_sum);
  }
  return check_launch(what);
}

}  // namespace
}  // namespace mi355

extern "C" int mi355_per_token_quant_int8(const void* x, int x_dtype, void* q, float* s, int64_t M, int64_t K,
                                          void* stream) {
  return mi355::per_token_quant<false>("mi355_per_token_quant_int8", x, x_dtype, q, s, M, K, stream);
}

extern "C" int mi355_per_token_quant_int8_sum(const void* x, int x_dtype, void* q, float* s, void* x_sum, int64_t M, int64_t K,
                                              void* stream) {
  return mi355::per_token_quant<false, false, false, true>("mi355_per_token_quant_int8_sum", x, x_dtype, q, s, M, K, stream, 0.f, x_sum);
}

extern "C" int mi355_per_token_quant_fp8(const void* x, int x_dtype, void* q, float* s, int64_t M, int64_t K,
                                         void* stream) {
  return mi355::per_token_quant<true>("mi355_per_token_quant_fp8", x, x_dtype, q, s, M, K, stream);
}

extern "C" int mi355_row_group_quant_fp8(const void* x, int x_dtype, void* q, float* s, int64_t M, int64_t K, float eps,
                                         int mode, void* stream) {
  const char* what = "mi355_row_group_quant_fp8";
  mi355::clear_error();
  MI355_REQUIRE(eps > 0.f, MI355_ERR_INVALID_ARGUMENT, "%s: eps must be positive (it is the floor of the row maximum)", what);
  MI355_REQUIRE(mode == MI355_QUANT_DIV || mode == MI355_QUANT_RCP, MI355_ERR_INVALID_ARGUMENT,
                "%s: mode must be MI355_QUANT_DIV or MI355_QUANT_RCP", what);
  if (mode == MI355_QUANT_DIV) return mi355::per_token_quant<true, true, true>(what, x, x_dtype, q, s, M, K, stream, eps);
  return mi355::per_token_quant<true, true, false>(what, x, x_dtype, q, s, M, K, stream, eps);
}
