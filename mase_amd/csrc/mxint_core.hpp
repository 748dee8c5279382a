// Per-block arithmetic of the MXINT quantizer (nn/quantizers/mxint/fake.py:11-80), shared by the stand-alone
// quantize-dequantize kernels and by kernels that quantize values they have just produced.
#pragma once
#include "common.hpp"

namespace mase {

struct MxintParams {
  int qshift;     // b - 1
  int bias;       // 2^(s-1) - 1
  int scale_max;  // 2^s - 1
  float lo, hi;   // clamp bounds as T represents them
  const uint32_t* tab;
};

// state 0: regular block (k, kc valid); 1: 2^k overflows T (also an infinite maximum): x/2^k is +-0;
// 2: the maximum is NaN.
template <int DT, typename... Meta>
__device__ __forceinline__ int block_exponent(uint32_t mbits, const MxintParams& p, int& k, int& kc,
                                              const Meta&... meta) {
  using TR = DTypeTraits<DT>;
  mbits = max(mbits, TR::kTinyBits);
  // the lookup runs for every lane (see WaveLog2), on a stand-in when the maximum is not finite
  const int kf = ceil_log2_lib(mbits >= 0x7F800000u ? 0x3F800000u : mbits, p.tab, meta...);
  if (mbits > 0x7F800000u) return 2;
  k = (mbits == 0x7F800000u) ? 1024 : kf;
  kc = min(max(k + p.bias, 0), p.scale_max) - p.bias;
  return (k > TR::kMaxPow2) ? 1 : 0;
}

// one element: dequantized value (fp32, rounded to T by the store) and its integer code
template <int DT>
__device__ __forceinline__ float mxint_element(float x, int state, int k, int kc, const MxintParams& p, int& code) {
  using TR = DTypeTraits<DT>;
  code = 0;
  if (state == 0) {
    float r = rintf(ldexpf(x, p.qshift - k));
    r = fminf(fmaxf(r, p.lo), p.hi);
    code = (int)r;
    return ldexpf(r, kc - p.qshift);
  }
  if (state == 2) return qnan();
  // x / inf: +-0 for finite x, NaN otherwise; then (+-0 / 2^(b-1)) * 2^kc, NaN when 2^kc is inf in T
  bool finite = (f2bits(x) & 0x7FFFFFFFu) < 0x7F800000u;
  if (!finite || kc > TR::kMaxPow2) return qnan();
  return bits2f(f2bits(x) & 0x80000000u);
}

}  // namespace mase
