// silu(gate) * up fused in front of the 1 x 128 FP8 group quantizer, plain and masked (expert-major) layouts, for gfx950.
//
// What the reference's v2 quantizer does with fuse_silu_and_mul (sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:
// :250-392, schedulers :133-238): the input row holds 2 * H values, gate | up; the value that is quantized is
//   v = T( float(T(silu(float(gate)))) * float(up) ),   silu(g) = g / (1 + exp(-g)),   T = the input's 16-bit type,
// then, per group of 128 values, amax = max(1e-10, max |v|), e = ceil(log2(amax / 448)), code = e4m3fn(clamp(v * 2^-e)),
// and the scale leaves as the exponent byte e + 127, four to a 32-bit word, words column-major (token index fastest).
// The reference only builds this combination (column-major packed UE8M0 scales, group 128 in its callers); so does this file.
// Masked layout: x [E, T, 2H], tokens t >= masked_m[e] of expert e are neither read nor written.
//
// exp is evaluated by a fixed sequence of individually rounded fp32 operations (det_expf below), the same sequence the
// CPU oracle uses, so results are reproducible bit for bit; it is within 1 ulp of exp.  (The reference uses the GPU's
// approximate exp intrinsic and compares its kernels with a tolerance.)
//
// One 16-lane row of a wave per group (8 values per lane: one 16-byte load of gate, one of up, one 8-byte store), 16
// groups of one token per workgroup.  The kernel moves 4 B in and 1 B out per value: bound by HBM.
#include "common.h"

namespace mi355 {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float det_expf(float x) {
  if (x > 88.72284f) return __builtin_inff();
  if (x < -103.97208f) return 0.0f;
  const float n = rintf(mul_rn(x, 1.44269504f));
  float r = fmaf(n, -0.693145751953125f, x);
  r = fmaf(n, -1.42860682e-6f, r);
  float p = 1.98412698e-4f;
  p = fmaf(p, r, 1.38888889e-3f);
  p = fmaf(p, r, 8.33333333e-3f);
  p = fmaf(p, r, 4.16666667e-2f);
  p = fmaf(p, r, 1.66666667e-1f);
  p = fmaf(p, r, 0.5f);
  p = fmaf(p, r, 1.0f);
  p = fmaf(p, r, 1.0f);
  return ldexpf(p, (int)n);
}

template <int DT>
__device__ __forceinline__ void unpack8(const u32x4& r, float* f) {
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = DT == MI355_BF16 ? __uint_as_float(w[i] << 16) : f16_bits_to_f32(w[i] & 0xffffu);
    f[2 * i + 1] = DT == MI355_BF16 ? __uint_as_float(w[i] & 0xffff0000u) : f16_bits_to_f32(w[i] >> 16);
  }
}

// round a float to T and back
template <int DT>
__device__ __forceinline__ float round_to_t(float v) {
  if constexpr (DT == MI355_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(v));
  return f16_bits_to_f32(f32_to_f16_bits(v));
}

__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true)));
  return v;
}

struct SiluQuantParams {
  const void* x;         // [E, T, 2H]
  uint8_t* q;            // [E, T, H]
  uint8_t* s;            // exponent bytes: word (e, t, kw) at ((e * s_e + kw * s_k + t) * 4), byte kg & 3
  const int32_t* masked_m;  // [E] or nullptr
  int64_t E, T, H;
  int64_t s_e, s_k;      // strides in 32-bit words
  int gpr, chunks;       // groups per row (H / 128), 16-group chunks per row
};

template <int DT>
__device__ __forceinline__ void quant_groups_of_row(const SiluQuantParams& p, int64_t e, int64_t t, int chunk) {
  const int lane = threadIdx.x & 15;
  const int kg = chunk * 16 + (threadIdx.x >> 4);  // group inside the row
  if (kg >= p.gpr) return;
  const int64_t row = e * p.T + t;
  const u32x4* gate = reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.x) + row * 2 * p.H + (int64_t)kg * 128) + lane;
  const u32x4* up = reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.x) + row * 2 * p.H + p.H + (int64_t)kg * 128) + lane;
  const u32x4 rg = __builtin_nontemporal_load(gate);
  const u32x4 ru = __builtin_nontemporal_load(up);
  float g[8], u[8], v[8];
  unpack8<DT>(rg, g);
  unpack8<DT>(ru, u);
  float amax = 1e-10f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float sl = g[j] / (1.0f + det_expf(-g[j]));
    v[j] = round_to_t<DT>(mul_rn(round_to_t<DT>(sl), u[j]));  // the product of two T values is exact in fp32
    amax = fmaxf(amax, fabsf(v[j]));
  }
  amax = row16_max(amax);
  const uint32_t bits = __float_as_uint(mul_rn(amax, 1.0f / 448.0f));
  const int ex = (int)((bits >> 23) & 0xffu) - 127 + ((bits & 0x7fffffu) != 0u);  // ceil(log2(amax / 448))
  const float mul = __uint_as_float((uint32_t)(127 - ex) << 23);
  float c[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) c[j] = fminf(fmaxf(mul_rn(v[j], mul), -448.0f), 448.0f);
  int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], 0, false);
  w0 = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], w0, true);
  int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(c[4], c[5], 0, false);
  w1 = __builtin_amdgcn_cvt_pk_fp8_f32(c[6], c[7], w1, true);
  __builtin_nontemporal_store(u32x2{(uint32_t)w0, (uint32_t)w1},
                              reinterpret_cast<u32x2*>(p.q + row * p.H + (int64_t)kg * 128 + lane * 8));
  if (lane == 0) {
    uint8_t* sb = p.s + ((e * p.s_e + (int64_t)(kg >> 2) * p.s_k + t) << 2) + (kg & 3);
    *sb = (uint8_t)(ex + 127);
    if (kg == p.gpr - 1)  // unused bytes of the last word read as exponent 0
      for (int b = (kg & 3) + 1; b < 4; ++b) sb[b - (kg & 3)] = 0;
  }
}

template <int DT>
__global__ __launch_bounds__(256) void silu_mul_quant_kernel(const SiluQuantParams p) {
  // blockIdx.x walks (row, chunk) pairs of the flat [E * T] rows
  const int64_t item = blockIdx.x;
  const int64_t row = item / p.chunks;
  quant_groups_of_row<DT>(p, row / p.T, row % p.T, (int)(item - row * p.chunks));
}

template <int DT>
__global__ __launch_bounds__(256) void silu_mul_quant_masked_kernel(const SiluQuantParams p) {
  const int64_t e = blockIdx.z;
  const int64_t valid = min((int64_t)p.masked_m[e], p.T);
  for (int64_t t = blockIdx.y; t < valid; t += gridDim.y) quant_groups_of_row<DT>(p, e, t, (int)blockIdx.x);
}

}  // namespace
}  // namespace mi355

using namespace mi355;

extern "C" int mi355_silu_mul_group_quant_fp8(const void* x, int x_dtype, void* q, void* s_words, int64_t E, int64_t T,
                                              int64_t H, const int32_t* masked_m, int64_t s_expert_stride,
                                              int64_t s_k_stride, void* stream) {
  const char* what = "mi355_silu_mul_group_quant_fp8";
  clear_error();
  MI355_REQUIRE(E >= 0 && T >= 0 && H >= 0, MI355_ERR_INVALID_ARGUMENT, "%s: negative shape", what);
  MI355_REQUIRE(x_dtype == MI355_F16 || x_dtype == MI355_BF16, MI355_ERR_INVALID_ARGUMENT,
                "%s: input must be float16 or bfloat16", what);
  if (E == 0 || T == 0 || H == 0) return MI355_OK;
  MI355_REQUIRE(x && q && s_words, MI355_ERR_INVALID_ARGUMENT, "%s: null pointer", what);
  MI355_REQUIRE(H % 128 == 0, MI355_ERR_UNSUPPORTED, "%s: the hidden size must be a multiple of the group size 128", what);
  MI355_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)q % 8 == 0) && ((uintptr_t)s_words % 4 == 0), MI355_ERR_INVALID_ARGUMENT,
                "%s: input must be 16-byte, output 8-byte and scales 4-byte aligned", what);
  MI355_REQUIRE(E * T < (1ll << 31) && H < (1ll << 31), MI355_ERR_INVALID_ARGUMENT, "%s: shape out of range", what);
  SiluQuantParams p;
  p.x = x, p.q = static_cast<uint8_t*>(q), p.s = static_cast<uint8_t*>(s_words), p.masked_m = masked_m;
  p.E = E, p.T = T, p.H = H, p.s_e = s_expert_stride, p.s_k = s_k_stride;
  p.gpr = (int)(H / 128), p.chunks = (p.gpr + 15) / 16;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (masked_m == nullptr) {
    const int64_t items = E * T * p.chunks;
    MI355_REQUIRE(items < (1ll << 31), MI355_ERR_INVALID_ARGUMENT, "%s: too many groups for one launch", what);
    const dim3 grid((unsigned)items);
    if (x_dtype == MI355_BF16)
      hipLaunchKernelGGL(silu_mul_quant_kernel<MI355_BF16>, grid, dim3(256), 0, st, p);
    else
      hipLaunchKernelGGL(silu_mul_quant_kernel<MI355_F16>, grid, dim3(256), 0, st, p);
  } else {
    MI355_REQUIRE(E <= 65535, MI355_ERR_INVALID_ARGUMENT, "%s: at most 65535 experts", what);
    const dim3 grid((unsigned)p.chunks, (unsigned)std::min<int64_t>(T, 1024), (unsigned)E);
    if (x_dtype == MI355_BF16)
      hipLaunchKernelGGL(silu_mul_quant_masked_kernel<MI355_BF16>, grid, dim3(256), 0, st, p);
    else
      hipLaunchKernelGGL(silu_mul_quant_masked_kernel<MI355_F16>, grid, dim3(256), 0, st, p);
  }
  return check_launch(what);
}
