// Per-block arithmetic of the MXFP quantizer (nn/quantizers/mxfp/fake.py:12-104), shared by the stand-alone
// quantize-dequantize / packing kernels and by kernels that quantize values they have just produced.
#pragma once
#include "common.hpp"
#include "minifloat_mx.hpp"

namespace mase {

struct MxfpParams {
  MinifloatMxFmt m;
  int el_emax;
  const uint32_t* tab;  // fp32 table (floor half is used)
};

// state 0: all flushed, 1: regular (sh valid), 2: NaN block
template <typename... Meta>
__device__ __forceinline__ int mxfp_block_scale(uint32_t mbits, const MxfpParams& p, int& sh, const Meta&... meta) {
  // the lookup runs for every lane (see WaveLog2), on a stand-in when the maximum is zero or not finite
  const bool special = (mbits == 0) || (mbits >= 0x7F800000u);
  const int kf = floor_log2_lib(special ? 0x3F800000u : mbits, p.tab, meta...);
  if (mbits == 0) return 0;
  if (mbits >= 0x7F800000u) return 2;
  sh = min(max(kf - p.el_emax, -127), 128);
  return 1;
}

__device__ __forceinline__ float mxfp_element(float t, int state, int sh, const MxfpParams& p, uint32_t& code) {
  code = 0;
  if (state == 0) return 0.0f;
  if (state == 2) return qnan();
  code = minifloat_mx_encode(ldexpf(t, -sh), p.m);
  return minifloat_mx_decode(code, p.m) * pow2f(sh);
}

__device__ __forceinline__ float flush_subnormal(float x) {
  return ((f2bits(x) & 0x7F800000u) == 0) ? 0.0f : x;
}

// Integer fast path of mxfp_element for an element of a regular block (state 1): the same steps as
// minifloat_mx_encode / minifloat_mx_decode written on the bit fields of the already flushed fp32 input.
//   exponent field of t / 2^sh is  ef = exp(t) - sh  (ldexp is exact while ef stays >= 1)
//   fraction: 23 -> 15 bits by truncation, 15 -> F bits round-half-even; a carry out of the fraction is OR-ed
//   into the exponent field (lost when that field is odd), exponent field 0 takes the truncating shift
//   value = code's [exponent|fraction] field moved to fp32's, exponent rebased by sh + 127 - bias
// Takes the raw (unflushed) input bits.  Returns false (caller takes mxfp_element) when t / 2^sh leaves the
// fp32 normal range, which only happens for elements more than 2^100 below the block maximum.
// INLINE_SUB = false leaves codes with exponent field 0 (elements more than 2^(el_emax + bias) below the block
// maximum) to the caller's slow path as well: right for the wide-exponent formats (e4m3, e5m2), where such
// elements are rare, and it halves the instruction count; the narrow-exponent formats handle them in line.
template <bool INLINE_SUB>
__device__ __forceinline__ bool mxfp_element_fast(uint32_t xb, int sh, const MxfpParams& p, uint32_t& code,
                                                  uint32_t& ybits) {
  const int F = p.m.F;
  const uint32_t ab = xb & 0x7FFFFFFFu;
  const uint32_t sgn32 = xb & 0x80000000u;
  const int ef = (int)(ab >> 23) - sh;
  const int ye = ef - 127 + p.m.bias;
  const int shn = 15 - F;
  const uint32_t m15 = (ab >> 8) & 0x7FFFu;
  const uint32_t yf = (m15 + ((1u << (shn - 1)) - 1u) + ((m15 >> shn) & 1u)) >> shn;  // 0 .. 2^F
  const uint32_t cn = ((uint32_t)ye << F) | yf;
  if constexpr (!INLINE_SUB) {
    const bool zero = (ab >> 23) == 0;  // zero or an fp32 subnormal, which the reference flushes to +0
    const uint32_t yn = sgn32 | ((cn << (23 - F)) + ((uint32_t)(sh + 127 - p.m.bias) << 23));
    ybits = zero ? 0u : yn;
    code = zero ? 0u : (cn | (sgn32 >> (31 - p.m.E - F)));
    return zero || ye > 0;  // ye > 0 implies ef > 0 (bias <= 127)
  }
  const uint32_t cs = yf ? ((yf | (1u << F)) >> 1) : 0u;
  uint32_t c = ye > 0 ? cn : (ye == 0 ? cs : 0u);
  const bool zero = (ab >> 23) == 0;  // zero or an fp32 subnormal, which the reference flushes to +0
  if (zero) c = 0;
  // decode: normal codes move as a bit field; codes with exponent field 0 are integers times a power of two
  const uint32_t yn = (c << (23 - F)) + ((uint32_t)(sh + 127 - p.m.bias) << 23);
  const uint32_t ys = f2bits(ldexpf((float)c, 1 - p.m.bias - F + sh));
  const uint32_t sg = zero ? 0u : sgn32;
  ybits = sg | ((c >> F) != 0 ? yn : ys);
  code = c | (sg >> (31 - p.m.E - F));
  // ye <= e_hi always holds in a regular block: sh >= floor(log2 max) - el_emax unless clamped from above,
  // which fp32 exponents cannot reach
  return zero || ef > 0;
}

// N elements of one block in any state: fast path for all of them, and one (rarely taken) branch that redoes
// the lane's elements with the step-by-step functions when the block is not regular or any element fell out
// of the fast path's range
template <bool INLINE_SUB, int N>
__device__ __forceinline__ void mxfp_elements(const float* x, int state, int sh, const MxfpParams& p, uint32_t* code,
                                              float* y) {
  bool slow = state != 1;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    uint32_t yb;
    slow |= !mxfp_element_fast<INLINE_SUB>(f2bits(x[j]), sh, p, code[j], yb);
    y[j] = bits2f(yb);
  }
  if (__builtin_expect(slow, 0)) {
#pragma unroll
    for (int j = 0; j < N; ++j) y[j] = mxfp_element(flush_subnormal(x[j]), state, sh, p, code[j]);
  }
}

}  // namespace mase
