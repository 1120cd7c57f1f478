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
// T(silu(g)) is a function of a 16-bit input: it is LOOKED UP.  Evaluated per element (an exp and an IEEE division, ~38
// vector operations per value) the kernel was bound by the vector ALUs at about half of the memory bandwidth; one LDS read
// per value leaves ~10 operations and the kernel bound by HBM.  The two tables (bfloat16, float16: 128 KB each) are
// computed at build time by gen_silu_table.cpp with one fixed sequence of individually rounded fp32 operations - the
// definition the CPU oracle restates, so results are reproducible bit for bit (the reference uses its GPU's approximate
// exp intrinsic and compares its kernels with a tolerance) - and are part of the code object: nothing is initialised at
// run time.  A workgroup copies its table into LDS once and then walks groups: 256 workgroups of 1024 threads (one per CU,
// the table takes 128 of the CU's 160 KB), a 16-lane row of a wave per group (8 values per lane: one 16-byte load of
// gate, one of up, eight LDS lookups, one 8-byte store), the loads of the next group requested before the current one is
// processed.  The kernel moves 4 B in and 1 B out per value.
#include "common.h"

namespace mi355 {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __attribute__((aligned(16))) const uint16_t g_silu_table[2][65536] = {
#include "silu_table.inc"
};

// round a float to T and back
template <int DT>
__device__ __forceinline__ float round_to_t(float v) {
  if constexpr (DT == MI355_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(v));
  return f16_bits_to_f32(f32_to_f16_bits(v));
}
template <int DT>
__device__ __forceinline__ float t_bits_to_f32(uint32_t h) {
  if constexpr (DT == MI355_BF16) return bf16_bits_to_f32(h);
  return f16_bits_to_f32(h);
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
  int gpr;               // groups per row (H / 128)
  FastDiv div_gpr;
};

constexpr int SQ_THREADS = 1024;
constexpr int SQ_GROUPS = SQ_THREADS / 16;  // groups a workgroup handles per step

struct GroupLoads {
  u32x4 gate, up;
};

// Expert `e` has `rows` rows to quantize (all T, or masked_m[e]); the workgroup takes groups first, first + stride, ...
// of the rows * gpr groups, 64 at a time.
// gate and up of group gi of expert e (16 bytes each per lane)
__device__ __forceinline__ void fetch_group(const SiluQuantParams& p, int64_t e, int64_t gi, GroupLoads& l) {
  const int lane = threadIdx.x & 15;
  const int64_t t = fastdiv((uint32_t)gi, p.div_gpr);
  const int kg = (int)(gi - t * p.gpr);
  const uint16_t* row = reinterpret_cast<const uint16_t*>(p.x) + (e * p.T + t) * 2 * p.H + (int64_t)kg * 128;
  l.gate = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(row) + lane);
  l.up = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(row + p.H) + lane);
}

// `preloaded`: `cur` already holds the first group's loads (requested before the table was copied).
template <int DT>
__device__ __forceinline__ void quant_expert(const SiluQuantParams& p, const uint16_t* tbl, int64_t e, int64_t rows, int64_t first,
                                             int64_t stride, GroupLoads& cur, bool preloaded) {
  const int lane = threadIdx.x & 15;
  const int64_t groups = rows * p.gpr;
  int64_t gi = first + (threadIdx.x >> 4);
  GroupLoads nxt, nxt2;  // two groups ahead: three 32-byte requests per lane in flight
  if (gi < groups && !preloaded) fetch_group(p, e, gi, cur);
  if (gi + stride < groups) fetch_group(p, e, gi + stride, nxt);
  for (; gi < groups; gi += stride) {
    const int64_t gn = gi + 2 * stride;
    if (gn < groups) fetch_group(p, e, gn, nxt2);
    const int64_t t = fastdiv((uint32_t)gi, p.div_gpr);
    const int kg = (int)(gi - t * p.gpr);
    const uint32_t wg[4] = {cur.gate.x, cur.gate.y, cur.gate.z, cur.gate.w};
    const uint32_t wu[4] = {cur.up.x, cur.up.y, cur.up.z, cur.up.w};
    float v[8];
    float amax = 1e-10f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t gb = (j & 1) ? (wg[j >> 1] >> 16) : (wg[j >> 1] & 0xffffu);
      const uint32_t ub = (j & 1) ? (wu[j >> 1] >> 16) : (wu[j >> 1] & 0xffffu);
      const float sl = t_bits_to_f32<DT>(tbl[gb]);                    // T(silu(gate))
      v[j] = round_to_t<DT>(mul_rn(sl, t_bits_to_f32<DT>(ub)));       // the product of two T values is exact in fp32
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
    const int64_t row = e * p.T + t;
    __builtin_nontemporal_store(u32x2{(uint32_t)w0, (uint32_t)w1},
                                reinterpret_cast<u32x2*>(p.q + row * p.H + (int64_t)kg * 128 + lane * 8));
    if (lane == 0) {
      uint8_t* sb = p.s + ((e * p.s_e + (int64_t)(kg >> 2) * p.s_k + t) << 2) + (kg & 3);
      *sb = (uint8_t)(ex + 127);
      if (kg == p.gpr - 1)  // unused bytes of the last word read as exponent 0
        for (int b = (kg & 3) + 1; b < 4; ++b) sb[b - (kg & 3)] = 0;
    }
    cur = nxt;
    nxt = nxt2;
  }
}

// grid (X, Y): workgroup (x, y) takes experts y, y + Y, ... and of each the groups 64 x, 64 (x + X), ...
template <int DT>
__global__ __launch_bounds__(SQ_THREADS) void silu_mul_quant_kernel(const SiluQuantParams p) {
  __shared__ __attribute__((aligned(16))) uint16_t tbl[65536];
  // the first group's loads go out before the table is copied, so that the copy does not delay the stream's start
  GroupLoads cur;
  const int64_t first = (int64_t)blockIdx.x * SQ_GROUPS, stride = (int64_t)gridDim.x * SQ_GROUPS;
  {
    const int64_t e0 = blockIdx.y;
    const int64_t rows0 = p.masked_m ? min((int64_t)p.masked_m[e0], p.T) : p.T;
    if (first + (threadIdx.x >> 4) < rows0 * p.gpr) fetch_group(p, e0, first + (threadIdx.x >> 4), cur);
  }
  {
    const u32x4* src = reinterpret_cast<const u32x4*>(g_silu_table[DT == MI355_BF16 ? 0 : 1]);
    u32x4* dst = reinterpret_cast<u32x4*>(tbl);
#pragma unroll
    for (int i = 0; i < 65536 * 2 / 16 / SQ_THREADS; ++i) dst[i * SQ_THREADS + threadIdx.x] = src[i * SQ_THREADS + threadIdx.x];
  }
  __syncthreads();
  for (int64_t e = blockIdx.y; e < p.E; e += gridDim.y) {
    const int64_t rows = p.masked_m ? min((int64_t)p.masked_m[e], p.T) : p.T;
    quant_expert<DT>(p, tbl, e, rows, first, stride, cur, e == (int64_t)blockIdx.y);
  }
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
  p.s_e = s_expert_stride, p.s_k = s_k_stride;
  p.gpr = (int)(H / 128);
  p.div_gpr = make_fastdiv((uint32_t)p.gpr);
  p.H = H;
  // 256 workgroups in all (one per CU: the table fills most of a CU's LDS): a workgroup walks whole experts, so that
  // masked rows cost nothing
  p.E = E, p.T = T;
  MI355_REQUIRE(T * p.gpr < (1ll << 31), MI355_ERR_INVALID_ARGUMENT, "%s: too many groups per expert", what);
  const int gy = (int)std::min<int64_t>(E, 256);
  const int gx = (int)std::max<int64_t>(1, std::min<int64_t>(256 / gy, (T * p.gpr + SQ_GROUPS - 1) / SQ_GROUPS));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)gx, (unsigned)gy);
  if (x_dtype == MI355_BF16)
    hipLaunchKernelGGL(silu_mul_quant_kernel<MI355_BF16>, grid, dim3(SQ_THREADS), 0, st, p);
  else
    hipLaunchKernelGGL(silu_mul_quant_kernel<MI355_F16>, grid, dim3(SQ_THREADS), 0, st, p);
  return check_launch(what);
}
