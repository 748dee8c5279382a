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

}  // namespace mase
