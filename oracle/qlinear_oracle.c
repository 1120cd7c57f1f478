/*
 * CPU oracle for the quantized-linear hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a plain-C, IEEE-fp32 restatement of the reference's arithmetic.
 * It is the checker the HIP kernels are compared with; it is never part of the
 * product path.  Only tests, the smoke check and the benchmark's CPU-baseline
 * leg may load it.
 *
 * Build:  gcc -O2 -fno-fast-math -ffp-contract=off -fopenmp -shared -fPIC
 * (-ffp-contract=off matters: a fused multiply-add would change roundings).
 *
 * What each function follows (paths relative to the reference tree):
 *   oracle_group_quant        sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:25-114      (mode DIV, "v1")
 *                             sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:54-90,
 *                               :250-392                                                     (mode MUL, "v2")
 *                             python/sglang/srt/layers/quantization/fp8_kernel.py:121-161    (mode RCP, Triton row-major)
 *                             python/sglang/srt/layers/quantization/fp8_kernel.py:164-212    (mode DIV, Triton col-major)
 *   oracle_fp8_blockwise_mm   sgl-kernel/tests/test_fp8_blockwise_gemm.py:19-59 (baseline_scaled_mm),
 *                             python/sglang/test/test_block_fp8.py:273-325 (native_w8a8_block_fp8_matmul),
 *                             python/sglang/srt/layers/quantization/fp8_kernel.py:749-758 (per-K-block promotion)
 *   oracle_int8_mm_acc        exact integer matmul (sgl-kernel/csrc/gemm/int8_gemm_kernel.cu:663-697 contract)
 *   oracle_int8_epilogue      sgl-kernel/csrc/cutlass_extensions/epilogue/epilogue_per_row_per_col_scale.h:273-303,
 *                             sgl-kernel/csrc/gemm/int8_gemm_kernel.cu:449-476 (sm90 order),
 *                             sgl-kernel/tests/test_int8_gemm.py:11-17 (torch order)
 *   oracle_per_token_quant_int8  python/sglang/srt/layers/quantization/int8_kernel.py:28-52
 *   oracle_per_token_quant_fp8   sgl-kernel/csrc/gemm/per_token_quant_fp8.cu:15-85
 *   oracle_silu_mul              sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:32-40, :318-331 (the activation the v2
 *                                quantizer fuses in front of oracle_group_quant: T(silu(float(gate))) * up, in T)
 *   oracle_block_cast_to_fp8     python/sglang/srt/layers/quantization/fp8_utils.py:487-505 (per_block_cast_to_fp8, ceil_to_ue8m0)
 *   oracle_block_dequant_fp8     python/sglang/srt/layers/quantization/fp8_utils.py:392-413 (block_quant_dequant)
 *   oracle_per_tensor_quant_fp8  sgl-kernel/csrc/gemm/per_tensor_quant_fp8.cu:10-100,
 *                                python/sglang/srt/layers/quantization/fp8_kernel.py:593-632 (static_quant_fp8)
 *   oracle_fp8_scaled_mm         sgl-kernel/csrc/gemm/fp8_gemm_kernel.cu:529-547, :1450-1532
 *
 * Parity status: every function here is pinned by tests/test_oracle_*.py against
 * torch's CPU float8/bfloat16/half conversions, torch fp32/fp64 matmul, exact
 * integer arithmetic, brute force and the known-answer construction of
 * test/srt/quant/test_fp8_kernel.py:24-45.  The one thing no test can pin is the
 * *order* of the fp32 additions inside a 128-wide K block of the FP8 GEMM: the
 * reference leaves it to the tensor cores, and compares with a tolerance only.
 * The oracle sums each block in double precision ("parity unpinned" for that
 * summation order; the GPU kernel is held to the reference's tolerance instead).
 * Likewise "parity unpinned": the bits of exp inside oracle_silu_mul.  The reference calls the GPU's approximate
 * __expf there (per_token_group_quant_8bit_v2.cu:32-40) and compares its kernels with a tolerance; oracle_expf is one
 * fixed definition, pinned to fp64 exp within 1 ulp, and oracle_silu_mul is pinned against torch's silu up to isolated
 * one-unit differences after the rounding to the 16-bit type.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

enum { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2, DT_FP8_E4M3FN = 3, DT_I8 = 4, DT_I32 = 5 };
enum { QUANT_DIV = 0, QUANT_RCP = 1, QUANT_MUL = 2 };
enum { SCALE_F32 = 0, SCALE_UE8M0_PACKED = 1 };
enum { EPI_COL_ROW = 0, EPI_ROW_COL_ACC = 1, EPI_TORCH = 2 };

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ---------------------------------------------------------------- conversions */

float oracle_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

float oracle_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1f;
  uint32_t man = h & 0x3ffu;
  if (exp == 0x1f) return u2f(sign | 0x7f800000u | (man << 13));
  if (exp == 0) {
    if (man == 0) return u2f(sign);
    /* subnormal half = man * 2^-24, exact in fp32 */
    float v = (float)man * 5.9604644775390625e-08f;
    return sign ? -v : v;
  }
  return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

/* float -> bfloat16, round to nearest even, NaN kept quiet. */
uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

/* float -> IEEE half, round to nearest even, overflow to infinity. */
uint16_t oracle_f32_to_f16(float f) {
  uint32_t u = f2u(f);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 -> inf (65520 handled by rounding) */
  if (a < 0x38800000u) {                                     /* below the smallest normal half 2^-14 */
    if (a < 0x33000000u) return sign;                        /* < 2^-25 rounds to zero */
    uint32_t e = a >> 23;
    uint32_t m = (a & 0x7fffffu) | 0x800000u;
    uint32_t shift = 126u - e; /* result = m >> shift in units of 2^-24, shift in [14,24] */
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1u);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | q);
  }
  uint32_t r = a - 0x38000000u; /* rebias 127 -> 15 */
  uint32_t q = r >> 13;
  uint32_t rem = r & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
  return (uint16_t)(sign | q); /* a carry into the exponent, up to infinity, is the correct rounding */
}

/*
 * float -> OCP FP8 E4M3 ("e4m3fn"): 1 sign, 4 exponent (bias 7), 3 mantissa bits,
 * no infinities, 0x7f/0xff = NaN, largest finite 448 (0x7e).  Round to nearest even.
 * Magnitudes that round above 448 become NaN (the format has no infinity); callers
 * on this path clamp to [-448, 448] first, as the reference does.
 */
uint8_t oracle_e4m3fn_encode(float f) {
  uint32_t u = f2u(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  uint32_t a = u & 0x7fffffffu;
  if (a >= 0x43f00000u) return (uint8_t)(sign | 0x7fu); /* |f| >= 480, inf or NaN */
  if (a < 0x3c800000u) {                                /* below the smallest normal 2^-6: subnormal grid of 2^-9 */
    if (a < 0x3a000000u) return sign;                   /* < 2^-11 rounds to zero; 2^-10 is the first tie */
    uint32_t e = a >> 23;
    uint32_t m = (a & 0x7fffffu) | 0x800000u;
    uint32_t shift = 141u - e; /* value = m * 2^(e-150); units of 2^-9 -> m >> (141 - e), shift in [21,25] */
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1u);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint8_t)(sign | q);
  }
  uint32_t r = a - 0x3c000000u; /* rebias 127 -> 7 */
  uint32_t q = r >> 20;
  uint32_t rem = r & 0xfffffu;
  if (rem > 0x80000u || (rem == 0x80000u && (q & 1u))) q++;
  return (uint8_t)(sign | q); /* q == 0x7f can only come from (464, 480): NaN, as in the format */
}

float oracle_e4m3fn_decode(uint8_t b) {
  uint32_t sign = (uint32_t)(b & 0x80u) << 24;
  uint32_t exp = (b >> 3) & 0xfu;
  uint32_t man = b & 7u;
  if (exp == 0xf && man == 7) return u2f(sign | 0x7fc00000u);
  if (exp == 0) {
    float v = (float)man * 0.001953125f; /* man * 2^-9 */
    return sign ? -v : v;
  }
  return u2f(sign | ((exp + 120u) << 23) | (man << 20));
}

/* Batch forms of the scalar conversions, for exhaustive comparisons with a library routine. */
void oracle_e4m3fn_encode_n(const float* in, uint8_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_e4m3fn_encode(in[i]);
}
void oracle_e4m3fn_decode_n(const uint8_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_e4m3fn_decode(in[i]);
}
void oracle_f32_to_bf16_n(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_f32_to_bf16(in[i]);
}
void oracle_f32_to_f16_n(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_f32_to_f16(in[i]);
}
void oracle_f16_to_f32_n(const uint16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_f16_to_f32(in[i]);
}

static inline float load_as_f32(const void* p, int dtype, size_t i) {
  switch (dtype) {
    case DT_F32: return ((const float*)p)[i];
    case DT_F16: return oracle_f16_to_f32(((const uint16_t*)p)[i]);
    default: return oracle_bf16_to_f32(((const uint16_t*)p)[i]);
  }
}

static inline void store_from_f32(void* p, int dtype, size_t i, float v) {
  switch (dtype) {
    case DT_F32: ((float*)p)[i] = v; break;
    case DT_F16: ((uint16_t*)p)[i] = oracle_f32_to_f16(v); break;
    default: ((uint16_t*)p)[i] = oracle_f32_to_bf16(v);
  }
}

/* ceil(log2(x)) for a positive normal float, by its bits:
 * per_token_group_quant_8bit_v2.cu:61-66 (fast_log2_ceil). */
static inline int log2_ceil_bits(float x) {
  uint32_t u = f2u(x);
  int e = (int)((u >> 23) & 0xffu);
  return e - 127 + ((u & 0x7fffffu) != 0);
}

static inline float pow2_int(int e) { return u2f((uint32_t)(e + 127) << 23); }

/* ---------------------------------------------------------------- group quantizer */

/*
 * x [M, K] contiguous; one scale per `group` consecutive elements of a row.
 *   amax = fmaxf-fold of |x| starting from eps       (v1 :45,:80; v2 :331-346; Triton :155)
 *   DIV: s = amax / qmax;          q = x / s          (v1 :86,:110)
 *   RCP: s = amax / qmax;          q = x * (1.0f / s) (Triton row-major :156-158)
 *   MUL: s = amax * (1.0f / qmax); q = x * (qmax / amax)  (v2 :77-78,:369-375)
 * Power-of-two scales (ue8m0 != 0):
 *   DIV: s = 2^ceil(log2(max(s, pow2_floor)))         (v1 :88 with pow2_floor = 1e-10f; Triton :207-208 with 0)
 *   MUL: e = ceil(log2(amax * (1.0f / qmax))), s = 2^e, multiplier 2^-e   (v2 :73-75)
 *   stored byte = biased exponent of s                (v1 :94, v2 :84-90)
 * q is clamped with fmaxf/fminf to [qmin, qmax] and converted: e4m3fn by RNE,
 * int8 by truncation toward zero (v1 :111 `DST_DTYPE(q_val)`, v2 :384).
 * Scale placement:
 *   SCALE_F32:           s[row * s_stride_row + kg * s_stride_col]  (floats)
 *   SCALE_UE8M0_PACKED:  bytes; address (kg/4) * s_stride_col * 4 + row * 4 + kg % 4
 *                        (v1 :54-61, v2 :305-315); the unused bytes of a row's last
 *                        word are zeroed (v2 :322-329).
 */
int oracle_group_quant(const void* x, int x_dtype, void* q, int q_dtype, void* s, int64_t M, int64_t K, int group,
                       float eps, float qmin, float qmax, int mode, int scale_kind, float pow2_floor,
                       int64_t s_stride_row, int64_t s_stride_col) {
  if (group <= 0 || K % group != 0) return 1;
  if (q_dtype != DT_FP8_E4M3FN && q_dtype != DT_I8) return 2;
  const int64_t G = K / group;
  const int ue8m0 = (scale_kind == SCALE_UE8M0_PACKED);
  const float inv_qmax = 1.0f / qmax;
#pragma omp parallel for schedule(static)
  for (int64_t row = 0; row < M; ++row) {
    for (int64_t kg = 0; kg < G; ++kg) {
      const size_t base = (size_t)row * (size_t)K + (size_t)kg * (size_t)group;
      float amax = eps;
      for (int j = 0; j < group; ++j) amax = fmaxf(amax, fabsf(load_as_f32(x, x_dtype, base + j)));
      float s_val, mul = 0.0f;
      if (mode == QUANT_MUL) {
        if (ue8m0) {
          int e = log2_ceil_bits(amax * inv_qmax);
          s_val = pow2_int(e);
          mul = pow2_int(-e);
        } else {
          s_val = amax * inv_qmax;
          mul = qmax / amax;
        }
      } else {
        s_val = amax / qmax;
        if (ue8m0) s_val = pow2_int(log2_ceil_bits(fmaxf(s_val, pow2_floor)));
        if (mode == QUANT_RCP) mul = 1.0f / s_val;
      }
      if (ue8m0) {
        uint8_t* sb = (uint8_t*)s;
        size_t off = (size_t)(kg / 4) * (size_t)s_stride_col * 4u + (size_t)row * 4u + (size_t)(kg % 4);
        sb[off] = (uint8_t)(f2u(s_val) >> 23);
        if (kg == G - 1)
          for (int64_t t = (kg % 4) + 1; t < 4; ++t) sb[off - (size_t)(kg % 4) + (size_t)t] = 0;
      } else {
        ((float*)s)[row * s_stride_row + kg * s_stride_col] = s_val;
      }
      for (int j = 0; j < group; ++j) {
        float v = load_as_f32(x, x_dtype, base + j);
        float t = (mode == QUANT_DIV) ? v / s_val : v * mul;
        t = fminf(fmaxf(t, qmin), qmax);
        if (q_dtype == DT_FP8_E4M3FN)
          ((uint8_t*)q)[base + j] = oracle_e4m3fn_encode(t);
        else
          ((int8_t*)q)[base + j] = (int8_t)t;
      }
    }
  }
  return 0;
}

/* ---------------------------------------------------------------- per-token int8 quantizer */

/* x [M, K] -> q int8 [M, K], s float [M]:  absmax floored at 1e-10, s = absmax / 127,
 * q = round-half-away-from-zero(x * (127 / absmax))   (int8_kernel.py:47-50, libdevice.round). */
int oracle_per_token_quant_int8(const void* x, int x_dtype, int8_t* q, float* s, int64_t M, int64_t K) {
#pragma omp parallel for schedule(static)
  for (int64_t row = 0; row < M; ++row) {
    float amax = 1e-10f;
    for (int64_t j = 0; j < K; ++j) amax = fmaxf(amax, fabsf(load_as_f32(x, x_dtype, (size_t)row * K + j)));
    s[row] = amax / 127.0f;
    float mul = 127.0f / amax;
    for (int64_t j = 0; j < K; ++j) {
      float t = load_as_f32(x, x_dtype, (size_t)row * K + j) * mul;
      q[(size_t)row * K + j] = (int8_t)roundf(t);
    }
  }
  return 0;
}

/* x [M, K] -> q e4m3fn [M, K], s float [M]:  s = max|x| / 448 (no floor), q = RNE(clamp(x * (1 / s), -448, 448)),
 * and a row of zeros gives s = 0, q = 0 (sgl-kernel/csrc/gemm/per_token_quant_fp8.cu:15-85, the warp-per-token kernel;
 * its small-batch sibling :91-160 divides by the scale without the zero test and would produce NaN for such a row). */
int oracle_per_token_quant_fp8(const void* x, int x_dtype, uint8_t* q, float* s, int64_t M, int64_t K) {
#pragma omp parallel for schedule(static)
  for (int64_t row = 0; row < M; ++row) {
    float amax = 0.f;
    for (int64_t j = 0; j < K; ++j) amax = fmaxf(amax, fabsf(load_as_f32(x, x_dtype, (size_t)row * K + j)));
    const float scale = amax / 448.0f;
    s[row] = scale;
    const float inv = (scale == 0.f) ? 0.f : 1.0f / scale;
    for (int64_t j = 0; j < K; ++j) {
      float t = load_as_f32(x, x_dtype, (size_t)row * K + j) * inv;
      t = fmaxf(fminf(t, 448.0f), -448.0f);
      q[(size_t)row * K + j] = oracle_e4m3fn_encode(t);
    }
  }
  return 0;
}

/* x [m, n] -> q e4m3fn [m, n], s fp32 [ceil(m/128), ceil(n/128)]: per 128 x 128 block amax = max(1e-4, max |x|),
 * s = 2^ceil(log2(amax / 448)), q = RNE(x * (1 / s))  (fp8_utils.py:487-505; the reference zero-pads to whole blocks and
 * takes log2 / ceil / pow in fp32 tensor ops - here ceil(log2) comes from the exponent and mantissa bits, the exact value). */
int oracle_block_cast_to_fp8(const void* x, int x_dtype, uint8_t* q, float* s, int64_t m, int64_t n) {
  const int64_t bm = (m + 127) / 128, bn = (n + 127) / 128;
#pragma omp parallel for schedule(static) collapse(2)
  for (int64_t i = 0; i < bm; ++i)
    for (int64_t j = 0; j < bn; ++j) {
      const int64_t r1 = (i + 1) * 128 < m ? (i + 1) * 128 : m, c1 = (j + 1) * 128 < n ? (j + 1) * 128 : n;
      float amax = 0.f;
      for (int64_t r = i * 128; r < r1; ++r)
        for (int64_t c = j * 128; c < c1; ++c) amax = fmaxf(amax, fabsf(load_as_f32(x, x_dtype, (size_t)(r * n + c))));
      amax = fmaxf(amax, 1e-4f);
      const float t = amax / 448.0f;
      int e;
      const float mant = frexpf(t, &e); /* t = mant * 2^e, mant in [0.5, 1) */
      const int ce = (mant == 0.5f) ? e - 1 : e; /* ceil(log2 t) */
      const float sf = ldexpf(1.0f, ce), inv = ldexpf(1.0f, -ce);
      s[i * bn + j] = sf;
      for (int64_t r = i * 128; r < r1; ++r)
        for (int64_t c = j * 128; c < c1; ++c)
          q[r * n + c] = oracle_e4m3fn_encode(load_as_f32(x, x_dtype, (size_t)(r * n + c)) * inv);
    }
  return 0;
}

/* q [n, k] e4m3fn, s [ceil(n/128), ceil(k/128)] -> out [n, k] = T(float(q) * s)  (fp8_utils.py:392-413). */
int oracle_block_dequant_fp8(const uint8_t* q, const float* s, void* out, int out_dtype, int64_t n, int64_t k) {
  const int64_t bk = (k + 127) / 128;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < n; ++r)
    for (int64_t c = 0; c < k; ++c)
      store_from_f32(out, out_dtype, (size_t)(r * k + c), oracle_e4m3fn_decode(q[r * k + c]) * s[(r / 128) * bk + c / 128]);
  return 0;
}

/* exp(x) in single precision from individually rounded fp32 operations only (multiply, round-to-integer, fused
 * multiply-add, scaling by a power of two), so that a GPU evaluating the same sequence gets the same bits: n = rint(x *
 * log2(e)), r = x - n * ln2 in two FMA steps (ln2 split so that n * hi is exact), Taylor polynomial of degree 7 in Horner
 * form with FMAs (|r| <= 0.3466: truncation below 6e-9), times 2^n.  Within 1 ulp of exp on the whole range. */
float oracle_expf(float x) {
  if (x > 88.72284f) return INFINITY;
  if (x < -103.97208f) return 0.0f;
  const float n = rintf(x * 1.44269504f);
  float r = fmaf(n, -0.693145751953125f, x);
  r = fmaf(n, -1.42860682e-6f, r);
  float p = 1.98412698e-4f; /* 1/5040 */
  p = fmaf(p, r, 1.38888889e-3f); /* 1/720 */
  p = fmaf(p, r, 8.33333333e-3f); /* 1/120 */
  p = fmaf(p, r, 4.16666667e-2f); /* 1/24 */
  p = fmaf(p, r, 1.66666667e-1f); /* 1/6 */
  p = fmaf(p, r, 0.5f);
  p = fmaf(p, r, 1.0f);
  p = fmaf(p, r, 1.0f);
  return ldexpf(p, (int)n);
}

/* x [rows, 2 * H] (gate | up halves of each row) -> out [rows, H] in the same 16-bit type T:
 *   out = T( float(T(silu(float(gate)))) * float(up) ),  silu(g) = g / (1 + exp(-g))
 * i.e. the activation is rounded to T, then multiplied by `up` in T (one rounding of the exact product), as
 * per_token_group_quant_8bit_v2.cu:318-331 does with its element type.  The reference evaluates exp with the GPU's
 * approximate intrinsic (:32-40), whose bits differ between its own kernels, and compares with a tolerance
 * (sgl-kernel/tests/test_per_token_group_quant_8bit.py:153-168); here exp is oracle_expf. */
int oracle_silu_mul(const void* x, int dtype, void* out, int64_t rows, int64_t H) {
  if (dtype != DT_BF16 && dtype != DT_F16) return 1;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t j = 0; j < H; ++j) {
      const float g = load_as_f32(x, dtype, (size_t)(r * 2 * H + j));
      const float u = load_as_f32(x, dtype, (size_t)(r * 2 * H + H + j));
      const float sl = g / (1.0f + oracle_expf(-g));
      store_from_f32(out, dtype, (size_t)(r * H + j), sl);               /* T(silu) */
      const float st = load_as_f32(out, dtype, (size_t)(r * H + j));
      store_from_f32(out, dtype, (size_t)(r * H + j), st * u);           /* exact product, one rounding */
    }
  }
  return 0;
}

/* x (n elements) -> q e4m3fn, one scale for the tensor.  Dynamic (is_static == 0): *scale = max|x| / 448 (the reference
 * merges per-block quotients with an atomic max into a zeroed word: the same value, division by 448 being monotonic);
 * then in both modes q = RNE(fmax(fmin(x * (1 / *scale), 448), -448))  (sgl-kernel/csrc/gemm/per_tensor_quant_fp8.cu:10-100;
 * python/sglang/srt/layers/quantization/fp8_kernel.py:593-632 has the same arithmetic for a given scale).  fmin/fmax return
 * the other operand for a NaN, so a zero tensor quantized dynamically (0 * inf) comes out as +448, as in the reference. */
int oracle_per_tensor_quant_fp8(const void* x, int x_dtype, uint8_t* q, float* scale, int64_t n, int is_static) {
  if (!is_static) {
    float amax = 0.f;
    for (int64_t i = 0; i < n; ++i) amax = fmaxf(amax, fabsf(load_as_f32(x, x_dtype, (size_t)i)));
    *scale = amax / 448.0f;
  }
  const float inv = 1.0f / *scale;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float t = load_as_f32(x, x_dtype, (size_t)i) * inv;
    t = fmaxf(fminf(t, 448.0f), -448.0f);
    q[i] = oracle_e4m3fn_encode(t);
  }
  return 0;
}

/*
 * Per-token x per-channel FP8 GEMM:  out[m, n] = cast( sa[m] * (sb[n] * sum_k a[m,k] * b[n,k]) + bias[n] )
 * (sgl-kernel/csrc/gemm/fp8_gemm_kernel.cu:1450-1532; epilogue order of its sm90 visitor tree :529-547: the weight scale
 * multiplies the accumulator, the token scale multiplies that, the bias is added in the same fused step).  The sum over
 * K is exact in double here; bias, if any, has the output dtype.  abs_out, if not NULL, receives
 * |sa[m] * sb[n]| * sum_k |a * b| (fp32).
 */
int oracle_fp8_scaled_mm(const uint8_t* a, const uint8_t* b, const float* sa, const float* sb, const void* bias, void* out,
                         int out_dtype, float* abs_out, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                         int64_t ldo) {
  float lut[256];
  for (int i = 0; i < 256; ++i) lut[i] = oracle_e4m3fn_decode((uint8_t)i);
#pragma omp parallel for schedule(static) collapse(2)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      double acc = 0.0, mag = 0.0;
      const uint8_t* ar = a + m * lda;
      const uint8_t* br = b + n * ldb;
      for (int64_t k = 0; k < K; ++k) {
        const double prod = (double)lut[ar[k]] * (double)lut[br[k]];
        acc += prod;
        mag += fabs(prod);
      }
      float t = sb[n] * (float)acc;
      t = sa[m] * t;
      if (bias) t = t + load_as_f32(bias, out_dtype, (size_t)n);
      store_from_f32(out, out_dtype, (size_t)(m * ldo + n), t);
      if (abs_out) abs_out[m * N + n] = fabsf(sa[m] * sb[n]) * (float)mag;
    }
  }
  return 0;
}

/* ---------------------------------------------------------------- blockwise FP8 GEMM */

/*
 * out[m, n] = cast( sum_kb ( sum_{k in kb} a[m,k] * b[n,k] ) * sa[m,kb] * sb[n/128, kb] )
 *   a  [M, K] e4m3fn bytes, row stride lda
 *   b  [N, K] e4m3fn bytes, row stride ldb (the weight as stored; `mat_b` of
 *      fp8_blockwise_scaled_mm is this matrix viewed transposed)
 *   sa element (m, kb) at sa[m * sa_sm + kb * sa_sk];  sb element (nb, kb) at sb[nb * sb_sn + kb * sb_sk]
 *   K and N may have ragged last blocks (fp8_kernel.py:738-751 masks the tails).
 * The inner block sum is exact in double; the promotion `acc += partial * sa * sb`
 * is evaluated as ((float)partial * sa) * sb in fp32 like fp8_kernel.py:758, and
 * accumulated in fp32 over K blocks in ascending order.
 * If abs_out != NULL it receives sum_kb sum_k |a*b| * |sa*sb| (fp32), the magnitude
 * against which a tolerance for summation-order differences can be scaled.
 */
int oracle_fp8_blockwise_mm(const uint8_t* a, const uint8_t* b, const float* sa, const float* sb, void* out,
                            int out_dtype, float* abs_out, int64_t M, int64_t N, int64_t K, int64_t lda,
                            int64_t ldb, int64_t sa_sm, int64_t sa_sk, int64_t sb_sn, int64_t sb_sk, int64_t ldo) {
  float lut[256];
  for (int i = 0; i < 256; ++i) lut[i] = oracle_e4m3fn_decode((uint8_t)i);
  const int64_t KB = (K + 127) / 128;
#pragma omp parallel for schedule(static) collapse(2)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      const uint8_t* ar = a + (size_t)m * lda;
      const uint8_t* br = b + (size_t)n * ldb;
      float acc = 0.0f, aacc = 0.0f;
      for (int64_t kb = 0; kb < KB; ++kb) {
        int64_t k1 = (kb + 1) * 128 < K ? (kb + 1) * 128 : K;
        double p = 0.0, pa = 0.0;
        for (int64_t k = kb * 128; k < k1; ++k) {
          double t = (double)lut[ar[k]] * (double)lut[br[k]];
          p += t;
          pa += fabs(t);
        }
        float s_a = sa[m * sa_sm + kb * sa_sk];
        float s_b = sb[(n / 128) * sb_sn + kb * sb_sk];
        acc += ((float)p * s_a) * s_b;
        aacc += ((float)pa * fabsf(s_a)) * fabsf(s_b);
      }
      size_t o = (size_t)m * ldo + n;
      if (out_dtype == DT_BF16)
        ((uint16_t*)out)[o] = oracle_f32_to_bf16(acc);
      else if (out_dtype == DT_F16)
        ((uint16_t*)out)[o] = oracle_f32_to_f16(acc);
      else
        ((float*)out)[o] = acc;
      if (abs_out) abs_out[(size_t)m * N + n] = aacc;
    }
  }
  return 0;
}

/* ---------------------------------------------------------------- INT8 GEMM */

/* acc[m, n] = sum_k a[m,k] * b[n,k], exact in int32 (|acc| <= 128*128*K < 2^31 for K < 131072). */
int oracle_int8_mm_acc(const int8_t* a, const int8_t* b, int32_t* acc, int64_t M, int64_t N, int64_t K, int64_t lda,
                       int64_t ldb) {
#pragma omp parallel for schedule(static) collapse(2)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      const int8_t* ar = a + (size_t)m * lda;
      const int8_t* br = b + (size_t)n * ldb;
      int32_t s = 0;
      for (int64_t k = 0; k < K; ++k) s += (int32_t)ar[k] * (int32_t)br[k];
      acc[(size_t)m * N + n] = s;
    }
  }
  return 0;
}

/*
 * Epilogue orders that exist in the reference (all fp32):
 *   EPI_COL_ROW      r = f32(acc) * (sb[n] * sa[m])   (+ f32(bias[n]))   epilogue_per_row_per_col_scale.h:280-303
 *   EPI_ROW_COL_ACC  r = sa[m] * (sb[n] * f32(acc))   (+ f32(bias[n]))   int8_gemm_kernel.cu:449-476
 *   EPI_TORCH        r = (f32(acc) * sa[m]) * sb[n]   (+ f32(bias[n]))   tests/test_int8_gemm.py:11-17
 * bias has the output dtype (int8_gemm_kernel.cu:694).  Output cast is RNE.
 */
int oracle_int8_epilogue(const int32_t* acc, const float* sa, const float* sb, const void* bias, void* out,
                         int out_dtype, int order, int64_t M, int64_t N, int64_t ldo) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      float f = (float)acc[(size_t)m * N + n];
      float r;
      if (order == EPI_COL_ROW)
        r = f * (sb[n] * sa[m]);
      else if (order == EPI_ROW_COL_ACC)
        r = sa[m] * (sb[n] * f);
      else
        r = (f * sa[m]) * sb[n];
      if (bias) r = r + load_as_f32(bias, out_dtype, (size_t)n);
      size_t o = (size_t)m * ldo + n;
      if (out_dtype == DT_BF16)
        ((uint16_t*)out)[o] = oracle_f32_to_bf16(r);
      else if (out_dtype == DT_F16)
        ((uint16_t*)out)[o] = oracle_f32_to_f16(r);
      else
        ((float*)out)[o] = r;
    }
  }
  return 0;
}

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void oracle_set_num_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n);
#else
  (void)n;
#endif
}
