// Per-token-group 8-bit quantizer for gfx950 (MI355X).
//
// Bandwidth-bound streaming kernel.  One group of `group` elements is owned by LPG adjacent
// lanes of a wave (LPG <= 16, i.e. never wider than one DPP row); each lane keeps its share
// of the group in registers, so the input is read exactly once:
//   16-byte coalesced loads -> |x| max in fp32 -> row-local DPP all-reduce -> scale ->
//   multiply or IEEE divide -> clamp -> v_cvt_pk_fp8_f32 (OCP e4m3 on gfx950) -> packed stores.
// Every thread processes UNROLL groups whose loads are all issued before the first use, which
// is what keeps enough bytes in flight to cover HBM latency.
//
// Arithmetic follows, bit for bit, sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:25-114 (DIV),
// sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:54-90,:250-392 (MUL) and
// python/sglang/srt/layers/quantization/fp8_kernel.py:121-212 (RCP / DIV), evaluated in IEEE fp32.
#include <hip/hip_fp16.h>

#include "common.h"

namespace mi355 {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct QuantParams {
  const void* x;
  uint8_t* q;
  void* s;
  uint32_t num_groups;     // M * K / group
  FastDiv groups_per_row;  // K / group
  float eps, qmin, qmax, inv_qmax, pow2_floor;
  int64_t s_stride_row, s_stride_col;
};

// max over the LPG lanes of a group, result in every lane.  Pure DPP (no LDS traffic).
template <int LPG>
__device__ __forceinline__ float group_allreduce_max(float v) {
  // quad_perm [1,0,3,2] = 0xB1, [2,3,0,1] = 0x4E, row_half_mirror = 0x141, row_mirror = 0x140
  if constexpr (LPG >= 2)
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true)));
  if constexpr (LPG >= 4)
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true)));
  if constexpr (LPG >= 8)
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true)));
  if constexpr (LPG >= 16)
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true)));
  return v;
}

template <typename T>
struct Elem;
template <>
struct Elem<float> {
  static constexpr int VEC = 4;
  static __device__ __forceinline__ void unpack(const u32x4& r, float* f) {
    f[0] = __uint_as_float(r.x), f[1] = __uint_as_float(r.y), f[2] = __uint_as_float(r.z), f[3] = __uint_as_float(r.w);
  }
};
struct bf16_tag {};
struct f16_tag {};
template <>
struct Elem<bf16_tag> {
  static constexpr int VEC = 8;
  static __device__ __forceinline__ void unpack(const u32x4& r, float* f) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(w[i] << 16);
      f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};
template <>
struct Elem<f16_tag> {
  static constexpr int VEC = 8;
  static __device__ __forceinline__ void unpack(const u32x4& r, float* f) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = f16_bits_to_f32(w[i] & 0xffffu);
      f[2 * i + 1] = f16_bits_to_f32(w[i] >> 16);
    }
  }
};

__device__ __forceinline__ int log2_ceil_bits(float x) {
  uint32_t u = __float_as_uint(x);
  return (int)((u >> 23) & 0xffu) - 127 + ((u & 0x7fffffu) != 0u);
}
__device__ __forceinline__ float pow2_int(int e) { return __uint_as_float((uint32_t)(e + 127) << 23); }

// Streaming stores.  Written as instructions because the optimizer drops the nontemporal hint of
// __builtin_nontemporal_store in this kernel, and the hint is worth ~8 % of bandwidth here (the output is never re-read).
__device__ __forceinline__ void store_nt(void* p, u32x2 v) {
  asm volatile("global_store_dwordx2 %0, %1, off nt" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void store_nt(void* p, uint32_t v) {
  asm volatile("global_store_dword %0, %1, off nt" ::"v"(p), "v"(v) : "memory");
}

// x / s, correctly rounded, for many x sharing one divisor s, given r = RN(1 / s).
// q0 = RN(x * r) is within 2 ulp of the quotient; each step q += RN(x - q * s) * r (the residual is exact in an FMA)
// at least squares the relative error, so after two steps the result is the correctly rounded quotient (Markstein's
// iteration, the same refinement the hardware divide expansion uses, minus its per-element reciprocal and range
// scaling).  Needs no range scaling here: |x / s| <= qmax * (1 + 2^-23), s and r are normal for every amax >= eps,
// and results below 2^-11 (where a subnormal residual could lose bits) convert to zero in either output format.
// Checked on the device against the `/` operator for every bf16 and fp16 x under 65536 divisors.
__device__ __forceinline__ float div_shared(float x, float s, float r) {
  float q = x * r;
  q = fmaf(fmaf(-q, s, x), r, q);
  q = fmaf(fmaf(-q, s, x), r, q);
  return q;
}

// T: element tag; LPG lanes per group; ITERS 16-byte vectors per lane and group.
// QUAD (UNROLL == 4 only): the four groups of a thread are four CONSECUTIVE groups of one row, so their scales leave as
// one 16-byte store (fp32, row-major) or one 32-bit word (packed UE8M0) instead of four 4-byte or 1-byte stores; the host
// selects it when groups per row and the group count are multiples of four and the scale layout is one of those two.
template <typename T, int LPG, int ITERS, int MODE, bool UE8M0, bool FP8_OUT, int UNROLL, bool QUAD>
__global__ __launch_bounds__(256) void group_quant_kernel(const QuantParams p) {
  static_assert(!QUAD || UNROLL == 4, "a quad is four groups");
  constexpr int VEC = Elem<T>::VEC;
  constexpr int GROUP = LPG * ITERS * VEC;
  constexpr int GROUPS_PER_PASS = 256 / LPG;
  constexpr int G_STEP = QUAD ? 1 : GROUPS_PER_PASS;  // distance between a thread's consecutive groups
  const uint32_t lane = threadIdx.x % LPG;
  // QUAD: quads past the end redo the last quad (same values to the same addresses), like single groups do below
  const uint32_t g_first = QUAD ? min(blockIdx.x * GROUPS_PER_PASS + threadIdx.x / LPG, p.num_groups / 4 - 1) * 4
                                : blockIdx.x * (GROUPS_PER_PASS * UNROLL) + threadIdx.x / LPG;
  float quad_scale[QUAD ? 4 : 1];

  u32x4 raw[UNROLL][ITERS];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    // Past the last group the lanes redo the last group (same values to the same addresses): the body stays free of
    // branches, which keeps the stores nontemporal and the loop fully unrolled.
    const uint32_t g = min(g_first + u * G_STEP, p.num_groups - 1);
    const u32x4* src = reinterpret_cast<const u32x4*>(p.x) + (size_t)g * (LPG * ITERS) + lane;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      raw[u][it] = __builtin_nontemporal_load(src + it * LPG);
    }
  }

#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const uint32_t g = min(g_first + u * G_STEP, p.num_groups - 1);
    float v[ITERS][VEC];
    float amax = p.eps;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      Elem<T>::unpack(raw[u][it], v[it]);
#pragma unroll
      for (int j = 0; j < VEC; ++j) amax = fmaxf(amax, fabsf(v[it][j]));
    }
    amax = group_allreduce_max<LPG>(amax);

    float s_val, mul = 0.f;
    if constexpr (MODE == MI355_QUANT_MUL) {
      if constexpr (UE8M0) {
        const int e = log2_ceil_bits(amax * p.inv_qmax);
        s_val = pow2_int(e);
        mul = pow2_int(-e);
      } else {
        s_val = amax * p.inv_qmax;
        mul = p.qmax / amax;
      }
    } else {
      s_val = amax / p.qmax;
      if constexpr (UE8M0) {
        const int e = log2_ceil_bits(fmaxf(s_val, p.pow2_floor));
        s_val = pow2_int(e);
        mul = pow2_int(-e);  // dividing by 2^e and multiplying by 2^-e round identically
      } else if constexpr (MODE == MI355_QUANT_RCP) {
        mul = 1.0f / s_val;
      }
    }
    constexpr bool USE_DIV = (MODE == MI355_QUANT_DIV) && !UE8M0;
    float rcp = 0.f;
    if constexpr (USE_DIV) rcp = 1.0f / s_val;  // correctly rounded; shared by the whole group

    {
      uint8_t* dst = p.q + (size_t)g * GROUP + (size_t)lane * VEC;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        float t[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float y = USE_DIV ? div_shared(v[it][j], s_val, rcp) : v[it][j] * mul;
          t[j] = fminf(fmaxf(y, p.qmin), p.qmax);
        }
        uint32_t w[VEC / 4];
#pragma unroll
        for (int j = 0; j < VEC / 4; ++j) {
          if constexpr (FP8_OUT) {
            int pk = __builtin_amdgcn_cvt_pk_fp8_f32(t[4 * j], t[4 * j + 1], 0, false);
            pk = __builtin_amdgcn_cvt_pk_fp8_f32(t[4 * j + 2], t[4 * j + 3], pk, true);
            w[j] = (uint32_t)pk;
          } else {
            w[j] = ((uint32_t)(int)t[4 * j] & 0xffu) | (((uint32_t)(int)t[4 * j + 1] & 0xffu) << 8) |
                   (((uint32_t)(int)t[4 * j + 2] & 0xffu) << 16) | (((uint32_t)(int)t[4 * j + 3] & 0xffu) << 24);
          }
        }
        uint8_t* d = dst + (size_t)it * (LPG * VEC);
        if constexpr (VEC == 8)
          store_nt(d, u32x2{w[0], w[1]});
        else
          store_nt(d, w[0]);
      }
      if constexpr (QUAD) {
        quad_scale[u] = s_val;
      } else if (lane == 0) {
        const uint32_t row = fastdiv(g, p.groups_per_row);
        const uint32_t kg = g - row * p.groups_per_row.div;
        if constexpr (UE8M0) {
          uint8_t* sb = reinterpret_cast<uint8_t*>(p.s) + (size_t)(kg >> 2) * (size_t)p.s_stride_col * 4u +
                        (size_t)row * 4u + (kg & 3u);
          *sb = (uint8_t)(__float_as_uint(s_val) >> 23);
          if (kg == p.groups_per_row.div - 1)
            for (uint32_t t = (kg & 3u) + 1; t < 4; ++t) sb[t - (kg & 3u)] = 0;
        } else {
          reinterpret_cast<float*>(p.s)[(int64_t)row * p.s_stride_row + (int64_t)kg * p.s_stride_col] = s_val;
        }
      }
    }
  }
  if constexpr (QUAD) {
    if (lane == 0) {
      if constexpr (UE8M0) {
        const uint32_t row = fastdiv(g_first, p.groups_per_row);
        const uint32_t kg = g_first - row * p.groups_per_row.div;  // a multiple of four
        uint32_t word = 0;
#pragma unroll
        for (int u = 0; u < 4; ++u) word |= (__float_as_uint(quad_scale[u]) >> 23) << (8 * u);
        *reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(p.s) + (size_t)(kg >> 2) * (size_t)p.s_stride_col * 4u +
                                     (size_t)row * 4u) = word;
      } else {
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p.s) + g_first) =
            f32x4{quad_scale[0], quad_scale[1], quad_scale[2], quad_scale[3]};
      }
    }
  }
}

template <typename T, int LPG, int ITERS, int MODE, bool UE8M0, bool FP8_OUT>
int launch(const QuantParams& p, hipStream_t stream) {
  // Fewer groups per thread when each group already spans several vectors per lane.
  constexpr int UNROLL = (ITERS >= 4) ? 1 : (ITERS == 2 ? 2 : 4);
  constexpr int GROUPS_PER_BLOCK = (256 / LPG) * UNROLL;
  const uint32_t blocks = (p.num_groups + GROUPS_PER_BLOCK - 1) / GROUPS_PER_BLOCK;
  if constexpr (UNROLL == 4) {
    // four consecutive groups of a row per thread when their scales are adjacent in memory: fp32 scales indexed by the
    // flat group number, or packed exponents (four k-groups per word)
    const uint32_t gpr = p.groups_per_row.div;
    const bool flat_f32 = !UE8M0 && p.s_stride_col == 1 && p.s_stride_row == (int64_t)gpr &&
                          (reinterpret_cast<uintptr_t>(p.s) & 15) == 0;
    const bool packed = UE8M0 && (reinterpret_cast<uintptr_t>(p.s) & 3) == 0;
    if (gpr % 4 == 0 && p.num_groups % 4 == 0 && (flat_f32 || packed)) {
      hipLaunchKernelGGL((group_quant_kernel<T, LPG, ITERS, MODE, UE8M0, FP8_OUT, UNROLL, true>), dim3(blocks), dim3(256), 0,
                         stream, p);
      return check_launch("mi355_group_quant_8bit");
    }
  }
  hipLaunchKernelGGL((group_quant_kernel<T, LPG, ITERS, MODE, UE8M0, FP8_OUT, UNROLL, false>), dim3(blocks), dim3(256), 0,
                     stream, p);
  return check_launch("mi355_group_quant_8bit");
}

template <typename T, int LPG, int ITERS>
int dispatch_mode(const QuantParams& p, int mode, bool ue8m0, bool fp8_out, hipStream_t stream) {
#define MI355_CASE(MODE_, UE_, FP8_)                                     \
  if (mode == MODE_ && ue8m0 == UE_ && fp8_out == FP8_) {                \
    return launch<T, LPG, ITERS, MODE_, UE_, FP8_>(p, stream);           \
  }
  MI355_CASE(MI355_QUANT_DIV, false, true)
  MI355_CASE(MI355_QUANT_RCP, false, true)
  MI355_CASE(MI355_QUANT_MUL, false, true)
  // with a power-of-two scale the three modes differ only in how the exponent is found
  MI355_CASE(MI355_QUANT_DIV, true, true)
  MI355_CASE(MI355_QUANT_RCP, true, true)
  MI355_CASE(MI355_QUANT_MUL, true, true)
  MI355_CASE(MI355_QUANT_DIV, false, false)
  MI355_CASE(MI355_QUANT_RCP, false, false)
  MI355_CASE(MI355_QUANT_MUL, false, false)
#undef MI355_CASE
  set_error("mi355_group_quant_8bit: int8 output with UE8M0 scales is not supported");
  return MI355_ERR_UNSUPPORTED;
}

template <typename T>
int dispatch_shape(const QuantParams& p, int nvec, int mode, bool ue8m0, bool fp8_out, hipStream_t stream) {
  switch (nvec) {
    case 1: return dispatch_mode<T, 1, 1>(p, mode, ue8m0, fp8_out, stream);
    case 2: return dispatch_mode<T, 2, 1>(p, mode, ue8m0, fp8_out, stream);
    case 4: return dispatch_mode<T, 4, 1>(p, mode, ue8m0, fp8_out, stream);
    case 8: return dispatch_mode<T, 8, 1>(p, mode, ue8m0, fp8_out, stream);
    case 16: return dispatch_mode<T, 16, 1>(p, mode, ue8m0, fp8_out, stream);
    case 32: return dispatch_mode<T, 16, 2>(p, mode, ue8m0, fp8_out, stream);
    case 64: return dispatch_mode<T, 16, 4>(p, mode, ue8m0, fp8_out, stream);
    case 128: return dispatch_mode<T, 16, 8>(p, mode, ue8m0, fp8_out, stream);
  }
  set_error("mi355_group_quant_8bit: group must be a power of two spanning 16..2048 bytes of input");
  return MI355_ERR_UNSUPPORTED;
}

}  // namespace
}  // namespace mi355

extern "C" int mi355_group_quant_8bit(const void* x, int x_dtype, void* q, int q_dtype, void* s, int64_t M, int64_t K,
                                      int group, float eps, float qmin, float qmax, int mode, int scale_kind,
                                      float pow2_floor, int64_t s_stride_row, int64_t s_stride_col, void* stream) {
  using namespace mi355;
  clear_error();
  MI355_REQUIRE(M >= 0 && K >= 0, MI355_ERR_INVALID_ARGUMENT, "mi355_group_quant_8bit: negative shape");
  MI355_REQUIRE(group > 0 && K % group == 0, MI355_ERR_INVALID_ARGUMENT,
                "mi355_group_quant_8bit: the last dimension (%lld) must be divisible by group (%d)", (long long)K,
                group);
  MI355_REQUIRE(x_dtype == MI355_F32 || x_dtype == MI355_F16 || x_dtype == MI355_BF16, MI355_ERR_INVALID_ARGUMENT,
                "mi355_group_quant_8bit: input must be float32, float16 or bfloat16");
  MI355_REQUIRE(q_dtype == MI355_FP8_E4M3FN || q_dtype == MI355_I8, MI355_ERR_INVALID_ARGUMENT,
                "mi355_group_quant_8bit: output must be float8_e4m3fn or int8");
  MI355_REQUIRE(mode >= MI355_QUANT_DIV && mode <= MI355_QUANT_MUL, MI355_ERR_INVALID_ARGUMENT,
                "mi355_group_quant_8bit: unknown mode %d", mode);
  MI355_REQUIRE(scale_kind == MI355_SCALE_F32 || scale_kind == MI355_SCALE_UE8M0_PACKED, MI355_ERR_INVALID_ARGUMENT,
                "mi355_group_quant_8bit: unknown scale_kind %d", scale_kind);
  if (M == 0 || K == 0) return MI355_OK;
  MI355_REQUIRE(x && q && s, MI355_ERR_INVALID_ARGUMENT, "mi355_group_quant_8bit: null pointer");
  MI355_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)q % 8 == 0), MI355_ERR_INVALID_ARGUMENT,
                "mi355_group_quant_8bit: input must be 16-byte and output 8-byte aligned");
  const int64_t num_groups = M * (K / group);
  MI355_REQUIRE(num_groups < (1ll << 31), MI355_ERR_INVALID_ARGUMENT,
                "mi355_group_quant_8bit: more than 2^31 groups in one call");
  const size_t gbytes = (size_t)group * dtype_size(x_dtype);
  MI355_REQUIRE(gbytes % 16 == 0, MI355_ERR_UNSUPPORTED,
                "mi355_group_quant_8bit: group must span a multiple of 16 input bytes");

  QuantParams p;
  p.x = x;
  p.q = static_cast<uint8_t*>(q);
  p.s = s;
  p.num_groups = (uint32_t)num_groups;
  p.groups_per_row = make_fastdiv((uint32_t)(K / group));
  p.eps = eps;
  p.qmin = qmin;
  p.qmax = qmax;
  p.inv_qmax = 1.0f / qmax;
  p.pow2_floor = pow2_floor;
  p.s_stride_row = s_stride_row;
  p.s_stride_col = s_stride_col;
  const bool ue8m0 = scale_kind == MI355_SCALE_UE8M0_PACKED;
  const bool fp8_out = q_dtype == MI355_FP8_E4M3FN;
  const int nvec = (int)(gbytes / 16);
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (x_dtype) {
    case MI355_F32: return dispatch_shape<float>(p, nvec, mode, ue8m0, fp8_out, st);
    case MI355_F16: return dispatch_shape<f16_tag>(p, nvec, mode, ue8m0, fp8_out, st);
    default: return dispatch_shape<bf16_tag>(p, nvec, mode, ue8m0, fp8_out, st);
  }
}
