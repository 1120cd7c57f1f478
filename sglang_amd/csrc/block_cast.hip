// Weight-side 128 x 128 block quantization for gfx950: the two kernels a block-FP8 checkpoint needs when it is
// re-quantized to power-of-two (UE8M0) scales at load time.
//
//   block_cast:    x [m, n] (bf16/fp16/fp32, row-major) -> q [m, n] e4m3fn, s [ceil(m/128), ceil(n/128)] fp32 with
//                  amax = max(1e-4, max |x| over the block), s = 2^ceil(log2(amax / 448)), q = e4m3fn(x * (1 / s))
//                  (per_block_cast_to_fp8 + ceil_to_ue8m0, python/sglang/srt/layers/quantization/fp8_utils.py:487-505; the
//                  reference pads the tensor with zeros to whole blocks, which changes no maximum).  ceil(log2(.)) is taken
//                  from the exponent and mantissa bits, i.e. exactly; no clamp is needed because |x / s| <= 448.
//   block_dequant: q [n, k] e4m3fn, s [ceil(n/128), ceil(k/128)] -> out [n, k] = T(float(q) * s)
//                  (block_quant_dequant, fp8_utils.py:392-413).
// One workgroup per block, streaming (nontemporal) loads and stores: 152 -> 145 us for a [36864, 7168] bf16 weight.  A
// workgroup that walks over several blocks and requests the next one before it reduces the one in hand was tried and is
// slower (173 us and more: twice the registers, half the workgroups per CU).  Both kernels stream every byte once: bound
// by HBM; they run once per weight at load time.
#include "common.h"

namespace mi355 {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <int DT>
__device__ __forceinline__ float load_elem(const void* x, int64_t i) {
  if constexpr (DT == MI355_F32) return reinterpret_cast<const float*>(x)[i];
  const uint32_t h = reinterpret_cast<const uint16_t*>(x)[i];
  return DT == MI355_BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
}

template <int DT>
__device__ __forceinline__ void store_elem(void* o, int64_t i, float v) {
  if constexpr (DT == MI355_F32)
    reinterpret_cast<float*>(o)[i] = v;
  else
    reinterpret_cast<uint16_t*>(o)[i] = (uint16_t)(DT == MI355_BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v));
}

__device__ __forceinline__ float wave_max64(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  return v;
}

// Eight consecutive values starting at element index `idx` (columns c .. c + 7 of a row of length n); values past the
// row's end read as zero.  VEC: idx is a multiple of 8 elements from a 16-byte aligned base and n % 8 == 0.
template <int DT, bool VEC>
__device__ __forceinline__ void load8(const void* x, int64_t idx, int64_t c, int64_t n, bool row_ok, float* f) {
  if constexpr (VEC) {
    if (!row_ok || c >= n) {
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = 0.f;
      return;
    }
    if constexpr (DT == MI355_F32) {
      const u32x4 a = reinterpret_cast<const u32x4*>(reinterpret_cast<const float*>(x) + idx)[0];
      const u32x4 b = reinterpret_cast<const u32x4*>(reinterpret_cast<const float*>(x) + idx)[1];
      const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = __uint_as_float(w[j]);
    } else {
      const u32x4 a = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(x) + idx));
      const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        f[2 * j] = DT == MI355_BF16 ? __uint_as_float(w[j] << 16) : f16_bits_to_f32(w[j] & 0xffffu);
        f[2 * j + 1] = DT == MI355_BF16 ? __uint_as_float(w[j] & 0xffff0000u) : f16_bits_to_f32(w[j] >> 16);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = (row_ok && c + j < n) ? load_elem<DT>(x, idx + j) : 0.f;
  }
}

// A block is 128 rows of 16 eight-value vectors; thread t takes vectors t, t + 256, ... (sixteen consecutive threads
// cover one row of the block: 256 contiguous bytes of a 16-bit input).
template <int DT, bool VEC>
__global__ __launch_bounds__(256) void block_cast_kernel(const void* x, uint8_t* q, float* s, int64_t m, int64_t n,
                                                         int64_t blocks_n) {
  __shared__ float part[4];
  const int64_t bm = blockIdx.x / blocks_n, bn = blockIdx.x - bm * blocks_n;
  float v[8][8];
  float amax = 0.f;
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int i = threadIdx.x + 256 * it;
    const int64_t row = bm * 128 + (i >> 4), c = bn * 128 + (i & 15) * 8;
    load8<DT, VEC>(x, row * n + c, c, n, row < m, v[it]);
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[it][j]));
  }
  amax = wave_max64(amax);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3])), 1e-4f);
  const uint32_t bits = __float_as_uint(amax / 448.0f);
  const int e = (int)((bits >> 23) & 0xffu) - 127 + ((bits & 0x7fffffu) != 0u);
  const float inv = __uint_as_float((uint32_t)(127 - e) << 23);
  if (threadIdx.x == 0) s[blockIdx.x] = __uint_as_float((uint32_t)(e + 127) << 23);
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int i = threadIdx.x + 256 * it;
    const int64_t row = bm * 128 + (i >> 4), c = bn * 128 + (i & 15) * 8;
    if (row >= m || c >= n) continue;
    int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(v[it][0] * inv, v[it][1] * inv, 0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(v[it][2] * inv, v[it][3] * inv, w0, true);
    int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(v[it][4] * inv, v[it][5] * inv, 0, false);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(v[it][6] * inv, v[it][7] * inv, w1, true);
    uint8_t* d = q + row * n + c;
    if constexpr (VEC) {
      __builtin_nontemporal_store(u32x2{(uint32_t)w0, (uint32_t)w1}, reinterpret_cast<u32x2*>(d));
    } else {
      const uint32_t w[2] = {(uint32_t)w0, (uint32_t)w1};
#pragma unroll
      for (int b = 0; b < 8; ++b)
        if (c + b < n) d[b] = (uint8_t)(w[b >> 2] >> (8 * (b & 3)));
    }
  }
}

// Same vector-to-thread map as block_cast_kernel: sixteen consecutive threads cover one 128-value row of the block.
template <int DT>
__global__ __launch_bounds__(256) void block_dequant_kernel(const uint8_t* q, const float* s, void* out, int64_t n,
                                                            int64_t k, int64_t blocks_k) {
  const int64_t bn = blockIdx.x / blocks_k, bk = blockIdx.x - bn * blocks_k;
  const float sc = s[blockIdx.x];
  const bool vec = k % 8 == 0 && (reinterpret_cast<uintptr_t>(q) & 7) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int i = threadIdx.x + 256 * it;
    const int64_t row = bn * 128 + (i >> 4), c = bk * 128 + (i & 15) * 8;
    if (row >= n || c >= k) continue;
    const int64_t idx = row * k + c;
    if (vec) {
      const u32x2 w = *reinterpret_cast<const u32x2*>(q + idx);
      float f[8];
      f[0] = __builtin_amdgcn_cvt_f32_fp8((int)w.x, 0), f[1] = __builtin_amdgcn_cvt_f32_fp8((int)w.x, 1);
      f[2] = __builtin_amdgcn_cvt_f32_fp8((int)w.x, 2), f[3] = __builtin_amdgcn_cvt_f32_fp8((int)w.x, 3);
      f[4] = __builtin_amdgcn_cvt_f32_fp8((int)w.y, 0), f[5] = __builtin_amdgcn_cvt_f32_fp8((int)w.y, 1);
      f[6] = __builtin_amdgcn_cvt_f32_fp8((int)w.y, 2), f[7] = __builtin_amdgcn_cvt_f32_fp8((int)w.y, 3);
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = mul_rn(f[j], sc);
      if constexpr (DT == MI355_F32) {
        float* o = reinterpret_cast<float*>(out) + idx;
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = f[j];
      } else {
        u32x4 o;
        if constexpr (DT == MI355_BF16)
          o = u32x4{pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7])};
        else
          o = u32x4{pack_f16x2(f[0], f[1]), pack_f16x2(f[2], f[3]), pack_f16x2(f[4], f[5]), pack_f16x2(f[6], f[7])};
        *reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(out) + idx) = o;
      }
    } else {
      for (int j = 0; j < 8 && c + j < k; ++j)
        store_elem<DT>(out, idx + j, mul_rn(__builtin_amdgcn_cvt_f32_fp8((int)q[idx + j], 0), sc));
    }
  }
}

}  // namespace
}  // namespace mi355

using namespace mi355;

extern "C" int mi355_block_cast_to_fp8(const void* x, int x_dtype, void* q, float* s, int64_t m, int64_t n, void* stream) {
  const char* what = "mi355_block_cast_to_fp8";
  clear_error();
  MI355_REQUIRE(m >= 0 && n >= 0, MI355_ERR_INVALID_ARGUMENT, "%s: negative shape", what);
  MI355_REQUIRE(x_dtype == MI355_F32 || x_dtype == MI355_F16 || x_dtype == MI355_BF16, MI355_ERR_INVALID_ARGUMENT,
                "%s: input must be float32, float16 or bfloat16", what);
  if (m == 0 || n == 0) return MI355_OK;
  MI355_REQUIRE(x && q && s, MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  const int64_t blocks_m = (m + 127) / 128, blocks_n = (n + 127) / 128;
  MI355_REQUIRE(blocks_m * blocks_n < (1ll << 31), MI355_ERR_INVALID_ARGUMENT, "%s: too many blocks for one launch", what);
  const dim3 grid((unsigned)(blocks_m * blocks_n));
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint8_t* qq = static_cast<uint8_t*>(q);
  const bool vec = n % 8 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)q % 8 == 0;
#define MI355_LAUNCH_CAST(DT_)                                                                                      \
  do {                                                                                                              \
    if (vec)                                                                                                        \
      hipLaunchKernelGGL((block_cast_kernel<DT_, true>), grid, dim3(256), 0, st, x, qq, s, m, n, blocks_n);         \
    else                                                                                                            \
      hipLaunchKernelGGL((block_cast_kernel<DT_, false>), grid, dim3(256), 0, st, x, qq, s, m, n, blocks_n);        \
  } while (0)
  switch (x_dtype) {
    case MI355_F32: MI355_LAUNCH_CAST(MI355_F32); break;
    case MI355_F16: MI355_LAUNCH_CAST(MI355_F16); break;
    default: MI355_LAUNCH_CAST(MI355_BF16);
  }
#undef MI355_LAUNCH_CAST
  return check_launch(what);
}

extern "C" int mi355_block_dequant_fp8(const void* q, const float* s, void* out, int out_dtype, int64_t n, int64_t k,
                                       void* stream) {
  const char* what = "mi355_block_dequant_fp8";
  clear_error();
  MI355_REQUIRE(n >= 0 && k >= 0, MI355_ERR_INVALID_ARGUMENT, "%s: negative shape", what);
  MI355_REQUIRE(out_dtype == MI355_F32 || out_dtype == MI355_F16 || out_dtype == MI355_BF16, MI355_ERR_INVALID_ARGUMENT,
                "%s: output must be float32, float16 or bfloat16", what);
  if (n == 0 || k == 0) return MI355_OK;
  MI355_REQUIRE(q && s && out, MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  const int64_t blocks_n = (n + 127) / 128, blocks_k = (k + 127) / 128;
  MI355_REQUIRE(blocks_n * blocks_k < (1ll << 31), MI355_ERR_INVALID_ARGUMENT, "%s: too many blocks for one launch", what);
  const dim3 grid((unsigned)(blocks_n * blocks_k));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint8_t* qq = static_cast<const uint8_t*>(q);
  switch (out_dtype) {
    case MI355_F32: hipLaunchKernelGGL(block_dequant_kernel<MI355_F32>, grid, dim3(256), 0, st, qq, s, out, n, k, blocks_k); break;
    case MI355_F16: hipLaunchKernelGGL(block_dequant_kernel<MI355_F16>, grid, dim3(256), 0, st, qq, s, out, n, k, blocks_k); break;
    default: hipLaunchKernelGGL(block_dequant_kernel<MI355_BF16>, grid, dim3(256), 0, st, qq, s, out, n, k, blocks_k);
  }
  return check_launch(what);
}
