// Shared host/device helpers of the fp8k library (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "../../include/fp8k.h"

namespace fp8k {

// ---------------------------------------------------------------- host: errors
int fail(int code, const char* fmt, ...);
void clear_error();
int num_cu();  // compute units of the current device (256 when no device is visible)

#define FP8K_REQUIRE(cond, ...)                                   \
  do {                                                            \
    if (!(cond)) return ::fp8k::fail(FP8K_ERR_INVALID, __VA_ARGS__); \
  } while (0)

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(FP8K_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return FP8K_OK;
}

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// ---------------------------------------------------------------- device: types
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned short u16;

constexpr float kFp8Max = 448.0f;

// ---------------------------------------------------------------- device: conversions
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// float -> bf16 bits, round to nearest even (NaN stays a quiet NaN): gfx950 converts in hardware, two values per
// v_cvt_pk_bf16_f32 (the add / shift / select sequence it replaces was most of a GEMM tile's write-out time)
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(unsigned short, (__bf16)f);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const v2f v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;
  return (uint32_t) __builtin_bit_cast(unsigned short, h);
}
__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
  return (float)__builtin_bit_cast(_Float16, (unsigned short)b);
}

// two floats -> two OCP e4m3fn bytes in the low / high half of a dword (v_cvt_pk_fp8_f32, RNE)
__device__ __forceinline__ uint32_t cvt_pk_fp8_lo(float a, float b, uint32_t old) {
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, false);
}
__device__ __forceinline__ uint32_t cvt_pk_fp8_hi(float a, float b, uint32_t old) {
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, true);
}
__device__ __forceinline__ uint32_t cvt4_fp8(float a, float b, float c, float d) {
  // the low-half convert keeps the upper 16 bits of `old`, which the high-half convert overwrites
  return cvt_pk_fp8_hi(c, d, cvt_pk_fp8_lo(a, b, __float_as_uint(a)));
}

// ---------------------------------------------------------------- device: DPP lane exchange
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float,
                            __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7-i inside each 8
constexpr int kDppMirror = 0x140;     // lane i <-> 15-i inside each 16

// max of NON-NEGATIVE floats over aligned groups of LANES consecutive lanes; every lane of the group
// gets the result.  Non-negative floats order like their bit patterns, so the exchange uses integer
// max, which folds into one DPP instruction per step (no NaN canonicalisation in between).
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_umax(uint32_t v) {
  return max(v, (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xf, 0xf, false));
}
template <int LANES>
__device__ __forceinline__ float group_max(float f) {
  uint32_t v = __float_as_uint(f);
  if (LANES >= 2) v = dpp_umax<kDppXor1>(v);
  if (LANES >= 4) v = dpp_umax<kDppXor2>(v);
  if (LANES >= 8) v = dpp_umax<kDppHalfMirror>(v);
  if (LANES >= 16) v = dpp_umax<kDppMirror>(v);
  if (LANES >= 32) v = max(v, (uint32_t)__shfl_xor((int)v, 16));
  if (LANES >= 64) v = max(v, (uint32_t)__shfl_xor((int)v, 32));
  return __uint_as_float(v);
}

// silu in float32 and the rounding of a float to the element type DT (identity for float32): shared by
// silu_and_mul and by the group quant that fuses it, so that both produce the same 16-bit values
// exp(-v) through the hardware exp2 and the quotient through the hardware reciprocal: the library routines cost
// three times the instructions, and the fused silu + quant kernel is bound by them, not by memory (the reference's
// fused kernel takes __expf the same way, per_token_group_quant_8bit_v2.cu:32-39).  Measured against float64 the
// result is within 2 float32 ulp for |v| < 8; below v = -8, where silu(v) = v * exp(v) is itself tiny, the rounding
// of the exponent -v*log2(e) adds |v| * 1e-7 of relative error - far inside a 16-bit output's rounding.
__device__ __forceinline__ float silu_f32(float v) {
  const float e = __builtin_amdgcn_exp2f(v * -1.4426950408889634f);
  // 1 + e may reach 2^128, whose reciprocal the hardware would flush to zero: divide by (1 + e) * 2^-32 and scale
  // back (exact, powers of two).  e = inf gives v * 0 = -0, and NaN for v = -inf as the quotient -inf / inf does.
  return v * (__builtin_amdgcn_rcpf((1.0f + e) * 0x1p-32f) * 0x1p-32f);
}

// gelu in float32, the reference's expression term for term: v * (0.5 * (1 + erf(v / sqrt 2)))
// (sgl-kernel/csrc/elementwise/activation.cu:62-67), erf from the device math library
__device__ __forceinline__ float gelu_f32(float v) { return v * (0.5f * (1.0f + erff(v * 0.70710678118654752440f))); }

template <int DT>
__device__ __forceinline__ float round_to(float v) {
  if (DT == FP8K_BF16) return __uint_as_float(f32_to_bf16_bits(v) << 16);
  if (DT == FP8K_F16) return f16_bits_to_f32(f32_to_f16_bits(v));
  return v;
}

}  // namespace fp8k
