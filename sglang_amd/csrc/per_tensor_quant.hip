// Per-tensor FP8 quantization for gfx950: one fp32 scale for the whole activation tensor.
//
//   dynamic:  scale = max|x| / 448 over all elements, then q = e4m3fn(clamp(x * (1 / scale)))
//             (sgl-kernel/csrc/gemm/per_tensor_quant_fp8.cu:10-45: block maxima merged with an atomic max into the scale
//             word, which the caller zeroes first, as the reference's Python wrapper does; :48-100: the quantize pass);
//   static:   the scale is given, only the quantize pass runs (the same arithmetic as static_quant_fp8,
//             python/sglang/srt/layers/quantization/fp8_kernel.py:593-632), optionally copying the scale into one slot
//             per row (its REPEAT_SCALE output, the per-token shape fp8_scaled_mm wants).
// Both passes stream one contiguous range per workgroup with 16-byte loads; the maximum is order-independent and the division by 448
// monotonic, so the atomic merge of per-workgroup quotients gives exactly max|x| / 448.  A tensor of zeros has scale 0,
// 1 / scale = inf and 0 * inf = NaN, which the reference's clamp (fmin, then fmax) turns into +448: kept, bit for bit.
#include "common.h"

namespace mi355 {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <int DT>
__device__ __forceinline__ float elem_f32(const void* x, int64_t i) {
  if constexpr (DT == MI355_F32) return reinterpret_cast<const float*>(x)[i];
  const uint32_t h = reinterpret_cast<const uint16_t*>(x)[i];
  return DT == MI355_BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
}

// 16 bytes = VEC elements
template <int DT>
__device__ __forceinline__ void unpack_vec(const u32x4& r, float* f) {
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
  if constexpr (DT == MI355_F32) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(w[i]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = DT == MI355_BF16 ? __uint_as_float(w[i] << 16) : f16_bits_to_f32(w[i] & 0xffffu);
      f[2 * i + 1] = DT == MI355_BF16 ? __uint_as_float(w[i] & 0xffff0000u) : f16_bits_to_f32(w[i] >> 16);
    }
  }
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  return v;
}

// One contiguous range per workgroup, eight 16-byte loads in flight per thread, 1024 threads: 512 workgroups read
// 235 MB in 39 us (6.0 TB/s).  The number of workgroups matters more than anything else here, because every one ends
// with an atomic on the ONE scale word and those serialize at ~11 ns each: 2048 workgroups of 256 threads took 50 us,
// 8192 took 108 us.  A workgroup whose maximum does not exceed what the word already holds skips the atomic.
constexpr int ABSMAX_THREADS = 1024;
constexpr int ABSMAX_MAX_WGS = 512;
constexpr int ABSMAX_UNROLL = 8;

template <int DT>
__global__ __launch_bounds__(ABSMAX_THREADS) void per_tensor_absmax_kernel(const void* x, float* scale, int64_t n) {
  constexpr int VEC = (DT == MI355_F32) ? 4 : 8;
  constexpr int U = ABSMAX_UNROLL;
  __shared__ float part[ABSMAX_THREADS / 64];
  const int64_t nvec = n / VEC;
  const int64_t per = (nvec + gridDim.x - 1) / gridDim.x;
  const int64_t begin = (int64_t)blockIdx.x * per, end = min(nvec, begin + per);
  const u32x4* src = reinterpret_cast<const u32x4*>(x);
  auto take = [&](const u32x4& raw, float m) {
    float f[VEC];
    unpack_vec<DT>(raw, f);
#pragma unroll
    for (int j = 0; j < VEC; ++j) m = fmaxf(m, fabsf(f[j]));
    return m;
  };
  float m = 0.f;
  int64_t v = begin + threadIdx.x;
  for (; v + (U - 1) * ABSMAX_THREADS < end; v += U * ABSMAX_THREADS) {
    u32x4 r[U];
#pragma unroll
    for (int u = 0; u < U; ++u) r[u] = src[v + u * ABSMAX_THREADS];
#pragma unroll
    for (int u = 0; u < U; ++u) m = take(r[u], m);
  }
  for (; v < end; v += ABSMAX_THREADS) m = take(src[v], m);
  // the elements behind the last whole 16 bytes
  for (int64_t i = nvec * VEC + (int64_t)blockIdx.x * ABSMAX_THREADS + threadIdx.x; i < n; i += (int64_t)gridDim.x * ABSMAX_THREADS)
    m = fmaxf(m, fabsf(elem_f32<DT>(x, i)));
  m = wave_max(m);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < ABSMAX_THREADS / 64; ++w) m = fmaxf(m, part[w]);
    // non-negative floats order like their bit patterns (a NaN maximum ends up largest and stays)
    const unsigned int mine = __float_as_uint(m / 448.0f);
    unsigned int* word = reinterpret_cast<unsigned int*>(scale);
    if (mine > __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(word, mine);
  }
}

__device__ __forceinline__ float clamp448(float v) { return fmaxf(fminf(v, 448.0f), -448.0f); }

// The quantize pass walks the tensor like the absmax pass before it - the same contiguous range per workgroup, in the same
// order - with streaming loads: what the first pass left in the caches is then still there when the second arrives
// (both passes: 108 -> 96 us on 235 MB of bf16; with a grid-stride second pass 102 us, with streaming loads in the
// FIRST pass 106 us, walking the ranges backwards 99 us).
template <int DT>
__global__ __launch_bounds__(ABSMAX_THREADS) void per_tensor_quant_kernel(const void* x, uint8_t* q, const float* scale, int64_t n,
                                                                          float* scale_rows, int64_t rows) {
  constexpr int VEC = (DT == MI355_F32) ? 4 : 8;
  constexpr int U = ABSMAX_UNROLL, T = ABSMAX_THREADS;
  const int64_t gid = (int64_t)blockIdx.x * T + threadIdx.x, stride = (int64_t)gridDim.x * T;
  const float s = *scale;
  const float inv = 1.0f / s;
  if (scale_rows != nullptr)
    for (int64_t r = gid; r < rows; r += stride) scale_rows[r] = s;
  const int64_t nvec = n / VEC;
  const u32x4* src = reinterpret_cast<const u32x4*>(x);
  auto emit = [&](const u32x4& raw, int64_t v) {
    float f[VEC];
    unpack_vec<DT>(raw, f);
    uint32_t w[VEC / 4];
#pragma unroll
    for (int j = 0; j < VEC / 4; ++j) {
      int c = __builtin_amdgcn_cvt_pk_fp8_f32(clamp448(f[4 * j] * inv), clamp448(f[4 * j + 1] * inv), 0, false);
      c = __builtin_amdgcn_cvt_pk_fp8_f32(clamp448(f[4 * j + 2] * inv), clamp448(f[4 * j + 3] * inv), c, true);
      w[j] = (uint32_t)c;
    }
    if constexpr (VEC == 8)
      __builtin_nontemporal_store(u32x2{w[0], w[1]}, reinterpret_cast<u32x2*>(q + v * VEC));
    else
      *reinterpret_cast<uint32_t*>(q + v * VEC) = w[0];
  };
  const int64_t per = (nvec + gridDim.x - 1) / gridDim.x;
  const int64_t begin = (int64_t)blockIdx.x * per, end = min(nvec, begin + per);
  int64_t v = begin + threadIdx.x;
  for (; v + (U - 1) * T < end; v += U * T) {  // eight loads in flight per thread
    u32x4 r[U];
#pragma unroll
    for (int u = 0; u < U; ++u) r[u] = __builtin_nontemporal_load(src + v + u * T);
#pragma unroll
    for (int u = 0; u < U; ++u) emit(r[u], v + u * T);
  }
  for (; v < end; v += T) emit(src[v], v);
  for (int64_t i = nvec * VEC + gid; i < n; i += stride) {
    const float t = clamp448(elem_f32<DT>(x, i) * inv);
    q[i] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(t, t, 0, false) & 0xff);
  }
}

template <int DT>
void launch_both(const void* x, uint8_t* q, float* scale, int64_t n, bool is_static, float* scale_rows, int64_t rows,
                 hipStream_t st) {
  // both passes use the same grid, so that a workgroup of the second pass re-reads what its namesake of the first pass read
  const int64_t per_wg = (int64_t)ABSMAX_THREADS * ABSMAX_UNROLL * ((DT == MI355_F32) ? 4 : 8);
  const unsigned grid = (unsigned)std::max<int64_t>(1, std::min<int64_t>((n + per_wg - 1) / per_wg, ABSMAX_MAX_WGS));
  if (!is_static) hipLaunchKernelGGL(per_tensor_absmax_kernel<DT>, dim3(grid), dim3(ABSMAX_THREADS), 0, st, x, scale, n);
  hipLaunchKernelGGL(per_tensor_quant_kernel<DT>, dim3(grid), dim3(ABSMAX_THREADS), 0, st, x, q, scale, n, scale_rows, rows);
}

}  // namespace
}  // namespace mi355

using namespace mi355;

extern "C" int mi355_per_tensor_quant_fp8(const void* x, int x_dtype, void* q, float* scale, int64_t numel, int is_static,
                                          float* scale_rows, int64_t rows, void* stream) {
  const char* what = "mi355_per_tensor_quant_fp8";
  clear_error();
  MI355_REQUIRE(numel >= 0 && rows >= 0, MI355_ERR_INVALID_ARGUMENT, "%s: negative size", what);
  MI355_REQUIRE(x_dtype == MI355_F32 || x_dtype == MI355_F16 || x_dtype == MI355_BF16, MI355_ERR_INVALID_ARGUMENT,
                "%s: input must be float32, float16 or bfloat16", what);
  MI355_REQUIRE(scale != nullptr, MI355_ERR_INVALID_ARGUMENT, "%s: null scale", what);
  MI355_REQUIRE(scale_rows == nullptr || is_static, MI355_ERR_INVALID_ARGUMENT,
                "%s: the per-row copy of the scale is an option of the static mode", what);
  if (numel == 0) return MI355_OK;
  MI355_REQUIRE(x && q, MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  MI355_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)q % 8 == 0) && ((uintptr_t)scale % 4 == 0), MI355_ERR_INVALID_ARGUMENT,
                "%s: input must be 16-byte and output 8-byte aligned", what);
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint8_t* qq = static_cast<uint8_t*>(q);
  float* sr = scale_rows;
  switch (x_dtype) {
    case MI355_F32: launch_both<MI355_F32>(x, qq, scale, numel, is_static != 0, sr, rows, st); break;
    case MI355_F16: launch_both<MI355_F16>(x, qq, scale, numel, is_static != 0, sr, rows, st); break;
    default: launch_both<MI355_BF16>(x, qq, scale, numel, is_static != 0, sr, rows, st);
  }
  return check_launch(what);
}
