// The exact arithmetic of the FP8 group quantisation, shared by the quant kernels and by the GEMM epilogue that
// quantises its own output: scale = amax / 448 correctly rounded, bytes = RNE_e4m3fn(clamp(x / scale)) bit-identical
// to an IEEE divide followed by the cast.
#pragma once

#include "fp8k_common.h"

namespace fp8k {

// q = RNE_e4m3fn(clamp(RN32(a / sc))) for 8 values - bit-identical to an IEEE float32 divide followed by the
// cast - without a divide and without a branch.  The quotient is bracketed by two multiplies with reciprocals
// (relative half-width 2^-20, far wider than the 2^-22 error of x * rcp(sc)); the cast is monotonic, so where
// both ends give the same byte the exact quotient does too.  Where they differ, for 16-bit inputs the answer
// follows from number theory instead of a divide.  Let amax = ma * 2^ea and x = mx * 2^ex with integer
// mantissas below 2^11, and Q0 = 448 x / amax, the quotient by the UNROUNDED scale.  Q0 is a rational with
// denominator ma, so it is either exactly a rounding boundary m = (2t+1) * 2^i of the cast or at least 2^-16
// (relative) away from every boundary; the bracket (2^-19) plus the rounding of the scale (2^-24) cannot
// bridge that, hence a differing byte means Q0 == m, a structural tie (0.3 % of real activations).  What the
// reference then produces depends only on how the scale was rounded, e = sc * 448 - amax (exact in one fma):
//   * e == 0 (ma is a multiple of 7, one group in seven): the quotient is m itself, round-half-to-even picks
//     the code with a clear low bit;
//   * e != 0: 7 does not divide ma, so 7 divides 2t+1, and the cast's boundaries only offer 2t+1 = 21 (normal
//     range, lower code even) and 7 (subnormal range, upper code even).  The float32 quotient m / (1 + e/amax)
//     rounds to m unless |e/amax| exceeds half an ulp at m, 2^-20/21 resp. 2^-22/7; equality would need
//     7 | ma.  So: scale rounded up by more than 2^-22/7 -> always the lower code; rounded down by more than
//     2^-20/21 -> always the upper code; otherwise the tie goes to the even code.
// All three cases are lane-group uniform selects and three bit operations per word.  Scales outside
// [2^-100, 2^100] (reachable only with a non-default eps or non-finite data) and float32 inputs, whose
// mantissas are too long for the argument, set `redo`: the caller recomputes those lanes with the real divide.
template <bool SHORT_MANTISSA>
__device__ __forceinline__ uint2 quant8_bracket(const float (&a)[8], float sc, float amax, bool& redo) {
  const float r = __builtin_amdgcn_rcpf(sc);  // 1 ulp
  const float r_lo = r * (1.0f - 0x1p-20f);
  const float r_hi = r * (1.0f + 0x1p-20f);
  const uint32_t l0 = cvt4_fp8(a[0] * r_lo, a[1] * r_lo, a[2] * r_lo, a[3] * r_lo);
  const uint32_t l1 = cvt4_fp8(a[4] * r_lo, a[5] * r_lo, a[6] * r_lo, a[7] * r_lo);
  const uint32_t h0 = cvt4_fp8(a[0] * r_hi, a[1] * r_hi, a[2] * r_hi, a[3] * r_hi);
  const uint32_t h1 = cvt4_fp8(a[4] * r_hi, a[5] * r_hi, a[6] * r_hi, a[7] * r_hi);
  const bool safe = (__float_as_uint(sc) - 0x0D800000u) < (0x71800000u - 0x0D800000u);
  if (!SHORT_MANTISSA) {
    redo = !safe | (l0 != h0) | (l1 != h1);
    return make_uint2(l0, l1);
  }
  redo = !safe;
  const float e = __builtin_fmaf(sc, kFp8Max, -amax);                   // exact
  const bool take_lower = __builtin_fmaf(e, 0x1.cp24f, -amax) > 0.0f;   // e/amax >  2^-22/7   (7 * 2^22)
  const bool take_upper = __builtin_fmaf(e, 0x1.5p24f, amax) < 0.0f;    // e/amax < -2^-20/21  (21 * 2^20)
  // default: bytes whose low-end code is odd take the high-end code (equal bytes are unaffected)
  const uint32_t s0 = take_lower ? 0u : (take_upper ? 0xFFFFFFFFu : (l0 & 0x01010101u) * 0xFFu);
  const uint32_t s1 = take_lower ? 0u : (take_upper ? 0xFFFFFFFFu : (l1 & 0x01010101u) * 0xFFu);
  return make_uint2((h0 & s0) | (l0 & ~s0), (h1 & s1) | (l1 & ~s1));
}

// the same 8 values through the IEEE divide (cold path)
__device__ __forceinline__ uint2 quant8_divide(const float (&a)[8], float sc) {
  float y[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float t = a[i] / sc;  // correctly rounded (no fast-math in this build)
    t = t < -kFp8Max ? -kFp8Max : t;  // NaN falls through, as torch.clamp does
    t = t > kFp8Max ? kFp8Max : t;
    y[i] = t;
  }
  return make_uint2(cvt4_fp8(y[0], y[1], y[2], y[3]), cvt4_fp8(y[4], y[5], y[6], y[7]));
}

// amax / 448, correctly rounded.  FAST: q0 = a*y, r = a - 448*q0 (exact in one fma), q1 = q0 + r*y with
// y = RN(1/448) - the classic reciprocal-refinement quotient, which is correctly rounded for this
// divisor; it is used where amax is a 16-bit float (every possible operand is covered by a test
// that walks all of them), float32 inputs take the full IEEE divide.
template <bool FAST>
__device__ __forceinline__ float div448(float a) {
  if (!FAST) return a / kFp8Max;
  constexpr float y = 1.0f / 448.0f;
  const float q0 = a * y;
  const float r = __builtin_fmaf(-q0, kFp8Max, a);
  return __builtin_fmaf(r, y, q0);
}

}  // namespace fp8k
