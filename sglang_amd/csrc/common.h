// Shared host/device helpers of the gfx950 quantized-linear kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "mi355_qlinear.h"

namespace mi355 {

// ---- error reporting (host) -------------------------------------------------------------
void set_error(const char* fmt, ...);  // defined in error.cpp; stores a thread-local message
void clear_error();

#define MI355_REQUIRE(cond, code, ...) \
  do {                                 \
    if (!(cond)) {                     \
      ::mi355::set_error(__VA_ARGS__); \
      return (code);                   \
    }                                  \
  } while (0)

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return MI355_ERR_LAUNCH;
  }
  return MI355_OK;
}

inline size_t dtype_size(int dt) {
  switch (dt) {
    case MI355_F32: return 4;
    case MI355_I32: return 4;
    case MI355_F16: return 2;
    case MI355_BF16: return 2;
    default: return 1;
  }
}

// Division of a 31-bit unsigned numerator by a run-time constant with one multiply-high and a shift.
struct FastDiv {
  uint32_t mul, shift, div;
};
inline FastDiv make_fastdiv(uint32_t d) {
  // ceil(2^(32+s) / d) with s = ceil(log2 d); exact for numerators below 2^31.
  FastDiv f;
  f.div = d;
  uint32_t s = 0;
  while ((1ull << s) < d) ++s;
  f.shift = s;
  f.mul = (uint32_t)((((1ull << 32) * ((1ull << s) - d)) / d) + 1);
  return f;
}

// ---- device helpers ---------------------------------------------------------------------
__device__ __forceinline__ uint32_t fastdiv(uint32_t n, const FastDiv& f) {
  uint32_t t = __umulhi(n, f.mul);
  return (t + n) >> f.shift;  // n < 2^31, so t + n cannot overflow
}

// Separately rounded fp32 multiply and add, written as instructions: the INT8 epilogue contract is mul, mul, add, and no
// compiler setting or code motion may fuse two of them into an FMA (a fused result differs in the last bit of the 16-bit
// output about once in 10^5 elements).
__device__ __forceinline__ float mul_rn(float a, float b) {
  float r;
  asm("v_mul_f32_e32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ float add_rn(float a, float b) {
  float r;
  asm("v_add_f32_e32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// Two fp32 values to packed bf16 (lo in bits 0..15), round to nearest even, NaN stays NaN: the conversion instruction of
// gfx950 (one instruction per pair instead of about six integer operations per value).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  uint32_t r;
  asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));
  return r;
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) { return pack_bf16x2(f, f) & 0xffffu; }

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  return (uint32_t)__half_as_ushort(__float2half_rn(f));
}

__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) { return f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16); }

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
  return __half2float(__ushort_as_half((unsigned short)h));
}

}  // namespace mi355
