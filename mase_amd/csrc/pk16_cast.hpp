// Minifloat cast of 16-bit elements (bf16 / fp16) in their own bit patterns, two elements per 32-bit register,
// with packed 16-bit integer instructions.  Shared by the stand-alone cast and by the MXFP quantizer on 16-bit tensors.
//
// For an element whose code is an ordinary one (exponent field of the code in [1, e_hi]) the cast only rounds the
// element's mantissa (MB bits: 7 for bf16, 10 for fp16) to F bits:
//   t  = |x| + round_add + tie_bit          (a carry out of the mantissa bumps the exponent field)
//   y  = t with the dropped mantissa bits cleared
//   the format ORs a carry into its exponent field, so a carry is lost when that field is odd: y -= one exponent step
//   y  = min(y, largest value of the format), sign put back (a zero keeps no sign)
// SUB = true also handles the binade below the format's normal range, where the format shifts the rounded fraction
// right by one with truncation (rounded fraction 0 -> zero; a carry -> 1.0 * 2^e; otherwise the lowest kept mantissa
// bit is cleared), and everything below that binade, which becomes a signed zero.
#pragma once
#include "common.hpp"
#include "minifloat_mx.hpp"

namespace mase {

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u16x2 as_u16x2(uint32_t v) { return __builtin_bit_cast(u16x2, v); }
__device__ __forceinline__ uint32_t as_u32(u16x2 v) { return __builtin_bit_cast(uint32_t, v); }

// 0xFFFF in the halves where a (as a signed 16-bit number) is negative
__device__ __forceinline__ uint32_t neg_mask2(uint32_t a) {
  typedef short i16x2 __attribute__((ext_vector_type(2)));
  const i16x2 fifteen = {15, 15};
  return __builtin_bit_cast(uint32_t, __builtin_bit_cast(i16x2, a) >> fifteen);
}

// what depends on the format and the rounding mode only
struct Pk16Format {
  uint32_t round_add2;  // per half: what is added before the dropped bits are cleared
  uint32_t tie2;        // 0x00010001 for round-to-nearest-even, else 0
  uint32_t keep2;       // per half: mask of sign-less bits that survive
  uint32_t keep_sub2;   // keep2 without its lowest mantissa bit
  uint32_t exp_lsb2;    // per half: lowest bit of the exponent field
  uint32_t exp_mask2;   // per half: the exponent field
  int drop;             // mantissa bits dropped
};

// what also depends on the scale the elements are cast at (per-half bit patterns, both halves equal)
struct Pk16Range {
  uint32_t odd_k2;    // exp_lsb2 if the code's exponent field is odd when the element's is even, else 0
  uint32_t max2;      // the format's largest value
  uint32_t lo_thr2;   // lowest pattern with an ordinary code
  uint32_t sub_thr2;  // lowest pattern of the binade below (SUB)
};

template <int MB>
inline Pk16Format make_pk16_format(int F, int round_mode) {
  Pk16Format f;
  const uint32_t one = 0x00010001u;
  const int drop = MB - F;
  const uint32_t add = drop == 0 ? 0u : (round_mode == 0 ? (1u << (drop - 1)) - 1u : (round_mode == 1 ? (1u << drop) - 1u : 0u));
  f.drop = drop;
  f.round_add2 = add * one;
  f.tie2 = (round_mode == 0 && drop > 0) ? one : 0u;
  f.keep2 = (0x7FFFu & ~((1u << drop) - 1u)) * one;
  f.keep_sub2 = f.keep2 & ~((1u << drop) * one);
  f.exp_lsb2 = (1u << MB) * one;
  f.exp_mask2 = (0x7FFFu & ~((1u << MB) - 1u)) * one;
  return f;
}

// Everything pk16_cast needs for format m on elements of dtype DT, and the domain it covers: an element e is handled
// iff e == 0 or lo_thr <= |e| < hi_thr (bit patterns); `sub`: the binade below the format's normal range can be taken
// in line (pk16_cast<MB, true>), which moves the lower end of the domain down to T's own smallest normal.  Returns
// false when the packed form does not apply.
// A format with more fraction bits than T has mantissa bits (F > MB) rounds nothing inside its normal range; its
// largest value, 2^top * (2 - 2^-F), is not a value of T and rounds to 2^(top+1) (T's infinity when top is T's last
// binade) when the result is stored, so that is what elements beyond the range become.
struct Pk16CastParams {
  Pk16Format f;
  Pk16Range r;
  uint32_t lo_thr, hi_thr;
  bool sub;
};

template <int DT>
inline bool make_pk16_cast_params(const MinifloatMxFmt& m, Pk16CastParams& q) {
  constexpr int MB = (DT == MASE_DT_BF16) ? 7 : 10, EB = (DT == MASE_DT_BF16) ? 127 : 15;
  constexpr int kMaxField = (DT == MASE_DT_BF16) ? 254 : 30;
  const int top = m.e_hi - m.bias + EB;      // exponent field (in T) of the format's largest binade
  const int bottom = 1 - m.bias + EB;        // and of its smallest normal binade
  if (top > kMaxField || top < 1) return false;
  const bool wide = m.F > MB;
  const int F = wide ? MB : m.F;
  const uint32_t one = 0x00010001u;
  q.f = make_pk16_format<MB>(F, m.round_mode);
  q.r.odd_k2 = (((m.bias - EB) & 1) ? (1u << MB) : 0u) * one;
  q.r.max2 = (wide ? ((uint32_t)(top + 1) << MB)
                   : (((uint32_t)top << MB) | ((uint32_t)m.frac_hi << q.f.drop))) * one;
  q.lo_thr = (uint32_t)(bottom < 1 ? 1 : bottom) << MB;
  q.r.lo_thr2 = q.lo_thr * one;
  q.r.sub_thr2 = ((uint32_t)(bottom - 1 < 1 ? 1 : bottom - 1) << MB) * one;
  // Inf/NaN inputs, and for a format with inf/nan codes every element of its top ordinary binade
  q.hi_thr = m.is_finite ? ((uint32_t)(kMaxField + 1) << MB) : ((uint32_t)top << MB);
  // in-line handling of the binade below the normal range when ordinary data reaches it and it exists in T
  q.sub = !wide && m.bias < 12 && q.lo_thr > (2u << MB) && m.F >= 1;
  return true;
}

// One register (two elements).  lo_acc / hi_acc collect min(|x| - 1) (a zero wraps to 0xFFFF) and max(|x|) for the
// caller's domain check.
template <int MB, bool SUB>
__device__ __forceinline__ uint32_t pk16_cast(uint32_t w, const Pk16Format& f, const Pk16Range& r, u16x2& lo_acc,
                                              u16x2& hi_acc) {
  const uint32_t ab = w & 0x7FFF7FFFu;
  const u16x2 drop2 = {(unsigned short)f.drop, (unsigned short)f.drop};
  const uint32_t lsb = as_u32(as_u16x2(ab) >> drop2) & f.tie2;
  const uint32_t t = as_u32(as_u16x2(ab) + as_u16x2(f.round_add2) + as_u16x2(lsb));
  const uint32_t tm = t & f.keep2;
  const uint32_t fix = (tm ^ ab) & (ab ^ r.odd_k2) & f.exp_lsb2;  // carry into an odd exponent field of the code
  u16x2 ya = as_u16x2(tm) - as_u16x2(fix);
  ya = __builtin_elementwise_min(ya, as_u16x2(r.max2));
  uint32_t yv = as_u32(ya);
  if constexpr (SUB) {
    const uint32_t below_lo = neg_mask2(as_u32(as_u16x2(ab) - as_u16x2(r.lo_thr2)));
    const uint32_t below_sub = neg_mask2(as_u32(as_u16x2(ab) - as_u16x2(r.sub_thr2)));
    const uint32_t eonly = ab & f.exp_mask2;
    const uint32_t carry = neg_mask2(((tm ^ ab) & f.exp_lsb2) << (15 - MB));
    uint32_t ys = (carry & eonly) | (~carry & tm & f.keep_sub2);
    const uint32_t z = tm ^ eonly;  // zero iff the rounded fraction is zero (and there was no carry)
    ys &= neg_mask2(z | as_u32(as_u16x2(0u) - as_u16x2(z)));
    yv = (below_lo & ys) | (~below_lo & yv);
    yv &= ~below_sub;
  }
  const uint32_t nz = as_u32(as_u16x2(ab) + as_u16x2(0x7FFF7FFFu));  // bit 15 of a half: the element is not zero
  lo_acc = __builtin_elementwise_min(lo_acc, as_u16x2(ab) - as_u16x2(0x00010001u));
  hi_acc = __builtin_elementwise_max(hi_acc, as_u16x2(ab));
  return yv | (w & nz & 0x80008000u);
}

}  // namespace mase
