// Bit-level minifloat encode/decode shared by the minifloat cast and the MXFP kernels.
// Follows the reference's integer arithmetic step by step (nn/quantizers/_minifloat_mx/fake.py:11-149),
// including its source-specific behaviour: the fp32 mantissa is truncated to 15 bits before rounding, a
// fraction that rounds up to 2^F is OR-ed into the exponent field (so the carry is lost when that field is
// odd), and subnormal fractions are shifted with truncation.
#pragma once
#include "common.hpp"

namespace mase {

struct MinifloatMxFmt {
  int E, F;
  int bias, e_hi, frac_hi;
  int is_finite;
  int round_mode;  // 0 rn, 1 ru, 2 rd, 3 rz
};

__device__ __forceinline__ uint32_t minifloat_mx_encode(float x, const MinifloatMxFmt& m) {
  uint32_t xb = f2bits(x);
  bool neg = x < 0.0f;  // -0.0 and NaN are "not negative"
  uint32_t ab = xb & 0x7FFFFFFFu;
  bool ftz = (ab & 0x7F800000u) == 0;
  // frexp of the flushed magnitude: exponent e with significand in [1,2); Inf/NaN give the library's
  // frexp exponent 0 -> e = -1 (only reachable for formats with inf/nan, where it is overridden below)
  int e = (int)(ab >> 23) - 127;
  uint32_t m23 = ab & 0x7FFFFFu;
  bool is_inf = ab == 0x7F800000u, is_nan = ab > 0x7F800000u;
  if (is_inf || is_nan) e = -1;
  if (ftz) { e = -1; m23 = 0; }
  bool under = e < -m.bias;
  bool over = e > (m.e_hi - m.bias);
  int ye = e + m.bias;
  int yf;
  if (m.round_mode == 3) {
    yf = (int)(m23 >> (23 - m.F));
  } else {
    uint32_t m15 = m23 >> 8;
    int sh = 15 - m.F;
    uint32_t fl = m15 >> sh;
    uint32_t rem = m15 & ((1u << sh) - 1u);
    uint32_t half = 1u << (sh - 1);
    if (m.round_mode == 0) yf = (int)(fl + ((rem > half || (rem == half && (fl & 1u))) ? 1u : 0u));
    else if (m.round_mode == 1) yf = (int)(fl + (rem ? 1u : 0u));
    else yf = (int)fl;
  }
  if (ye == 0 && yf != 0) yf = (yf | (1 << m.F)) >> 1;
  if (under) { yf = 0; ye = 0; }
  if (over) { yf = m.frac_hi; ye = m.e_hi; }
  if (ftz) { yf = 0; ye = 0; }
  if (!m.is_finite) {
    if (is_inf) { yf = 0; ye = m.e_hi; }
    if (is_nan) { yf = (1 << m.F) - 1; ye = m.e_hi; }
  }
  uint32_t y = ((uint32_t)ye << m.F) | (uint32_t)yf;
  if (neg) y += 1u << (m.E + m.F);
  return y & 0xFFFFu;
}

__device__ __forceinline__ float minifloat_mx_decode(uint32_t c, const MinifloatMxFmt& m) {
  bool sgn = (c >> (m.E + m.F)) & 1u;
  c &= 0x7FFFu;
  int xe = (int)((c >> m.F) & ((1u << m.E) - 1u));
  int xf = (int)(c & ((1u << m.F) - 1u));
  bool sub = (xe == 0) && (xf != 0);
  bool zero = (xe == 0) && (xf == 0);
  int ye = xe - m.bias + (sub ? 1 : 0);
  float fr = (float)xf / (float)(1 << m.F);
  if (!sub) fr += 1.0f;
  float y = ldexpf(fr, ye);
  if (!m.is_finite && xe == (1 << m.E) - 1) y = (xf == 0) ? __builtin_inff() : qnan();
  if (zero) y = 0.0f;
  return sgn ? -y : y;
}

// Integer form of decode(encode(x)) on the fp32 bit fields, for elements whose code is an ordinary one:
//   ye = exponent field + bias - 127; fraction 23 -> 15 bits by truncation, 15 -> F bits in the format's rounding
//   mode; a carry out of the fraction is OR-ed into the exponent field; ye > e_hi saturates; ye == 0 takes the
//   shifted fraction, ye < 0 gives zero; the value is the code's [exponent|fraction] field moved to fp32's place
//   (codes with exponent field 0: the integer fraction times 2^(1-bias-F)).
// Returns false for what is left to the stepwise functions: fp32 subnormals and non-finite inputs, codes of the
// inf/nan exponent of a format that has them and, with INLINE_SUB = false (formats whose subnormal range is
// rarely reached), every code with exponent field 0.
template <bool INLINE_SUB>
__device__ __forceinline__ bool minifloat_mx_fast(float x, const MinifloatMxFmt& m, uint32_t addc, uint32_t tie, int ye_limit,
                                                float& y) {
  const int F = m.F;
  const uint32_t xb = f2bits(x + 0.0f);  // -0.0 is "not negative" in the encode
  const uint32_t ab = xb & 0x7FFFFFFFu;
  const uint32_t Ef = ab >> 23;
  const int ye = (int)Ef + (m.bias - 127);
  const int shn = 15 - F;
  const uint32_t m15 = (ab >> 8) & 0x7FFFu;
  const uint32_t yf = (m15 + addc + ((m15 >> shn) & tie)) >> shn;  // 0 .. 2^F
  const uint32_t cn = ((uint32_t)ye << F) | yf;
  const uint32_t cmax = ((uint32_t)m.e_hi << F) | (uint32_t)m.frac_hi;
  const uint32_t rebias = (uint32_t)(127 - m.bias) << 23;
  const bool ordinary = (Ef - 1u < 254u) || ab == 0;
  if constexpr (!INLINE_SUB) {
    const uint32_t c = ye > m.e_hi ? cmax : cn;
    const uint32_t yn = (c << (23 - F)) + rebias;
    y = bits2f(ab == 0 ? 0u : ((xb & 0x80000000u) | yn));
    return ordinary && (ye > 0 || ab == 0) && ye < ye_limit;
  }
  const uint32_t cs = yf ? ((yf | (1u << F)) >> 1) : 0u;
  uint32_t c = ye > 0 ? cn : (ye == 0 ? cs : 0u);
  c = ye > m.e_hi ? cmax : c;
  c = ab == 0 ? 0u : c;
  const uint32_t yn = (c << (23 - F)) + rebias;
  const uint32_t ys = f2bits(ldexpf((float)c, 1 - m.bias - F));
  y = bits2f((xb & 0x80000000u) | ((c >> F) != 0 ? yn : ys));
  return ordinary && ye < ye_limit;
}

// decode(encode(x)) for 8 elements: the integer form for all of them and one rarely taken branch that redoes the
// lane's elements with the stepwise functions
__device__ __forceinline__ void minifloat_mx_qdq8(const float* x, float* y, const MinifloatMxFmt& m) {
  const int shn = 15 - m.F;
  // rounding of the 15-bit fraction as one addition: nearest-even, up (any remainder), down / toward zero
  const uint32_t addc = m.round_mode == 0 ? (1u << (shn - 1)) - 1u : (m.round_mode == 1 ? (1u << shn) - 1u : 0u);
  const uint32_t tie = m.round_mode == 0 ? 1u : 0u;
  // formats with inf/nan codes: an element that reaches the top ordinary exponent may carry into the inf/nan one
  const int ye_limit = m.is_finite ? 0x7FFFFFFF : m.e_hi;
  bool ok = true;
  if (m.bias < 12) {  // uniform
#pragma unroll
    for (int j = 0; j < 8; ++j) ok &= minifloat_mx_fast<true>(x[j], m, addc, tie, ye_limit, y[j]);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) ok &= minifloat_mx_fast<false>(x[j], m, addc, tie, ye_limit, y[j]);
  }
  if (__builtin_expect(!ok, 0)) {
#pragma unroll
    for (int j = 0; j < 8; ++j) y[j] = minifloat_mx_decode(minifloat_mx_encode(x[j], m), m);
  }
}

}  // namespace mase
