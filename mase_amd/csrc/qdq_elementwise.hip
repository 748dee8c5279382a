// Element-wise quantize-dequantize kernels for gfx950: fixed point, minifloat (denorm / ieee flavours) and
// the bit-level minifloat cast used by the MX formats.
//
// The two minifloat flavours are restated operation by operation: each reference op on a tensor of dtype
// T is "fp32 op, then round to T", written R(.) below, because with narrow T the intermediate values
// (2^e underflowing to 0 in fp16, clamp bounds that T cannot represent, ...) are part of the result.
#include "common.hpp"
#include "minifloat_mx.hpp"
#include "pk16_cast.hpp"

namespace mase {
namespace {

// ---------------------------------------------------------------------------------------------
// generic driver: 8 elements per lane through 16-byte accesses, one element per lane for the tail
// ---------------------------------------------------------------------------------------------
// fp32 items are two 16-byte vectors.  Inside a complete group of 64 items (one wavefront) lane l takes vectors l
// and l + 64 of the group's 128, so that each access of the wavefront covers 1 KB of consecutive memory; the items
// of the incomplete last group take adjacent vectors.
// SPLIT is set when input and output are both fp32 (the two sides must agree on which elements an item holds).
template <bool SPLIT>
__device__ __forceinline__ size_t vec4_first(size_t i8, size_t n8) {
  if constexpr (!SPLIT) return 2 * i8;
  return ((i8 | 63) < n8) ? ((i8 & ~(size_t)63) * 2 + (i8 & 63)) : 2 * i8;
}
template <bool SPLIT>
__device__ __forceinline__ size_t vec4_step(size_t i8, size_t n8) {
  if constexpr (!SPLIT) return 1;
  return ((i8 | 63) < n8) ? 64 : 1;
}

template <int DT, bool SPLIT>
__device__ __forceinline__ void load8(const void* p, size_t i8, size_t n8, float* x) {
  using TR = DTypeTraits<DT>;
  if constexpr (TR::kVec == 4) {
    const uint4* q = (const uint4*)p + vec4_first<SPLIT>(i8, n8);
    uint4 a = load_nt(q), b = load_nt(q + vec4_step<SPLIT>(i8, n8));
    TR::unpack(a, x);
    TR::unpack(b, x + 4);
  } else {
    uint4 a = load_nt((const uint4*)p + i8);
    TR::unpack(a, x);
  }
}
template <int DT, bool SPLIT>
__device__ __forceinline__ void store8(void* p, size_t i8, size_t n8, const float* y) {
  using TR = DTypeTraits<DT>;
  if constexpr (TR::kVec == 4) {
    uint4* q = (uint4*)p + vec4_first<SPLIT>(i8, n8);
    store_nt(q, TR::pack(y));
    store_nt(q + vec4_step<SPLIT>(i8, n8), TR::pack(y + 4));
  } else {
    store_nt((uint4*)p + i8, TR::pack(y));
  }
}

// One item of 8 elements per lane (16 bytes of a 16-bit type, 32 of fp32), 64-lane work-groups: the shape
// that streams best on this part.  Lanes past the vector part each take one element of the unaligned tail.
// Every lane runs the functor on all 8 slots (the log2 lookups inside are wave-wide register permutes and
// need all lanes present); unused slots hold 1.0.
constexpr int kEwThreads = 64;

template <int DTI, int DTO, typename F>
__global__ __launch_bounds__(kEwThreads) void elementwise_kernel(const void* __restrict__ in, void* __restrict__ out,
                                                                 size_t n8, size_t numel, F f) {
  constexpr bool kSplit = DTypeTraits<DTI>::kVec == 4 && DTypeTraits<DTO>::kVec == 4;
  WaveLog2 meta;
  if constexpr (F::kUsesTable) meta.init(f.tab, F::kTableHalf);
  const size_t t = (size_t)blockIdx.x * kEwThreads + threadIdx.x;
  const size_t tail = n8 * 8 + (t - n8);
  const bool vec = t < n8;
  const bool one = !vec && tail < numel;
  float x[8], y[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) x[j] = 1.0f;
  if (vec) load8<DTI, kSplit>(in, t, n8, x);
  else if (one) x[0] = DTypeTraits<DTI>::load1(in, tail);
  if constexpr (F::kBatch) {
    f.batch8(x, y);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) y[j] = f(x[j], meta);
  }
  if (vec) store8<DTO, kSplit>(out, t, n8, y);
  else if (one) DTypeTraits<DTO>::store1(out, tail, y[0]);
}

template <int DTI, int DTO, typename F>
int launch_elementwise(const void* in, void* out, size_t numel, const F& f, hipStream_t st) {
  size_t n8 = (aligned16(in) && aligned16(out)) ? numel / 8 : 0;
  size_t threads = n8 + (numel - n8 * 8);
  hipLaunchKernelGGL((elementwise_kernel<DTI, DTO, F>), dim3(blocks_for(threads, kEwThreads)), dim3(kEwThreads), 0, st,
                     in, out, n8, numel, f);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

// clamp as "min(max(a, lo), hi)" with the library's scalar-compare semantics: NaN propagates and
// -0.0 is not replaced by a +0.0 bound.
__device__ __forceinline__ float clamp_cmp(float a, float lo, float hi) {
  a = (a < lo) ? lo : a;
  a = (a > hi) ? hi : a;
  return a;
}

// ---------------------------------------------------------------------------------------------
// fixed point: integer.py:10-66
// ---------------------------------------------------------------------------------------------
template <int DT>
struct IntegerOp {
  static constexpr bool kUsesTable = false;
  static constexpr int kTableHalf = 0;
  static constexpr bool kBatch = false;
  const uint32_t* tab;
  int frac;
  int use_floor;
  float lo, hi;
  __device__ __forceinline__ float operator()(float x, const WaveLog2&) const {
    float t = DTypeTraits<DT>::round(ldexpf(x, frac));  // x * 2^f underflows differently in narrow T
    float r = use_floor ? floorf(t) : rintf(t);
    r = clamp_cmp(r, lo, hi);
    return ldexpf(r, -frac);  // rounded to T by the store
  }
};

// ---------------------------------------------------------------------------------------------
// minifloat denorm / ieee: minifloat.py:7-68 and :120-182
// ---------------------------------------------------------------------------------------------
template <int DT, bool IEEE>
struct MinifloatOp {
  using TR = DTypeTraits<DT>;
  static constexpr bool kUsesTable = true;
  static constexpr int kTableHalf = IEEE ? kLog2TabHalf : 0;  // floor thresholds (ieee) or ceil thresholds (denorm)
  static constexpr bool kBatch = false;
  const uint32_t* tab;
  int mb;
  float e_lo, e_hi;  // exponent clamp (as floats; representable in every T for exponent_width <= 8)
  float qmax;        // 2^mb - 1 as T represents it
  float shift;       // 2^mb
  uint32_t close_thr;
  float neg_bias;    // -exponent_bias as T represents it (ieee)
  int fast_ok;       // every intermediate of a finite element is exact in T (set by the launcher): value-level path
  int e_lo_i, e_hi_i;

  __device__ static __forceinline__ float R(float f) { return TR::round(f); }

  // library log2 of a T value followed by ceil (denorm) or floor (ieee), as a float
  template <bool WAVE = true>
  __device__ __forceinline__ float log2_rounded(float l, const WaveLog2& w) const {
    const uint32_t b = f2bits(l);
    // the lookup runs for every lane (wave-wide register permute), on a stand-in for zero / non-finite values
    const bool special = (b == 0) || (b >= 0x7F800000u);
    const uint32_t bb = special ? 0x3F800000u : b;
    float k;
    if constexpr (WAVE) k = (float)(IEEE ? floor_log2_lib(bb, tab, w) : ceil_log2_lib(bb, tab, w));
    else k = (float)(IEEE ? floor_log2_lib(bb, tab) : ceil_log2_lib(bb, tab));  // table from memory: any lane subset
    if (b == 0) return -__builtin_inff();
    if (b >= 0x7F800000u) return (b == 0x7F800000u) ? __builtin_inff() : qnan();  // l >= 0 here or NaN
    return k;
  }
  // x / p for p = 2^k evaluated in T: an exact scaling while p is a finite non-zero power of two (the quotient
  // of an IEEE division by a power of two is the correctly rounded scaled value, which is what ldexp gives);
  // zero, infinite or NaN p take the division
  __device__ static __forceinline__ float div_pow2(float x, float p) {
    const uint32_t pb = f2bits(p);
    const uint32_t ex = pb >> 23;  // p >= 0 here
    if (__builtin_expect((pb & 0x7FFFFFu) == 0 && ex >= 1 && ex <= 254, 1)) return ldexpf(x, 127 - (int)ex);
    return x / p;
  }
  // 2^e evaluated in T for an integer-valued float e
  __device__ static __forceinline__ float pow2_T(float e) {
    if (e != e) return e;
    if (e > (float)TR::kMaxPow2) return __builtin_inff();
    if (e < -160.0f) return 0.0f;
    return R(ldexpf(1.0f, (int)e));
  }

  // Value-level evaluation of a finite element when the launcher has established that no intermediate needs a
  // rounding to T (mantissa no wider than T's, 2^e and the smallest grid step representable in T): with k the
  // rounded logarithm of R(|x| + 1e-9),
  //   e = clamp(k, e_lo, e_hi);  man = R(|x| / 2^e);  ms = R(man * 2^mb)
  //   denorm: q = clamp(rint(ms), 0, qmax),                         |y| = q * 2^(e-mb)
  //   ieee:   e != -bias: q = clamp(rint(ms - 2^mb), 0, qmax),       |y| = (2^mb + q) * 2^(e-mb)
  //           e == -bias: q = clamp(rint(ms / 2), 0, qmax),          |y| = q * 2^(e-mb+1)
  //   result = isclose(x, 0) ? (x == 0 ? +0 : x) : copysign(|y|, x)
  // (for close elements 0*y + x keeps x, except that +0 + -0 is +0; for the others y carries the sign of
  // x + 1e-9, which is the sign of x, and adding 0*x changes nothing).
  __device__ __forceinline__ float fast(float x, uint32_t ab, float val, int k) const {
    const int e = min(max(k, e_lo_i), e_hi_i);
    const float man = R(ldexpf(val, -e));
    const float ms = R(ldexpf(man, mb));
    float yabs;
    if constexpr (!IEEE) {
      const float q = fminf(fmaxf(rintf(ms), 0.0f), qmax);
      yabs = ldexpf(q, e - mb);
    } else {
      const bool normal = (float)e != neg_bias;
      const float a = normal ? R(ms - shift) : R(ms * 0.5f);
      const float q = fminf(fmaxf(rintf(a), 0.0f), qmax);
      yabs = normal ? ldexpf(shift + q, e - mb) : ldexpf(q, e - mb + 1);
    }
    if (ab <= close_thr) return (ab == 0) ? 0.0f : x;
    return bits2f(f2bits(yabs) | (f2bits(x) & 0x80000000u));
  }

  __device__ __forceinline__ float operator()(float x, const WaveLog2& t) const {
    float val = fabsf(x);
    float l = R(val + 1e-9f);
    const float lr = log2_rounded(l, t);  // the table lookup inside runs for every lane, before any divergence
    if (fast_ok) {  // uniform
      const uint32_t ab = f2bits(val);
      if (__builtin_expect(ab < 0x7F800000u, 1)) return fast(x, ab, val, (int)lr);
    }
    return stepwise(x, val, lr);
  }

  // the same element evaluated with the table read from memory: callable from a divergent branch
  __device__ __forceinline__ float stepwise_from_memory(float x) const {
    const float val = fabsf(x);
    const WaveLog2 unused{};
    return stepwise(x, val, log2_rounded<false>(R(val + 1e-9f), unused));
  }

  // operation-by-operation evaluation; lr = rounded library logarithm of R(|x| + 1e-9)
  __device__ __forceinline__ float stepwise(float x, float val, float lr) const {
    float xs = R(x + 1e-9f);
    float sgn = (xs > 0.0f) ? 1.0f : ((xs < 0.0f) ? -1.0f : xs);
    float e = clamp_cmp(lr, e_lo, e_hi);
    float p2 = pow2_T(e);
    float man = R(div_pow2(val, p2));
    float mant;
    if constexpr (!IEEE) {
      float q = clamp_cmp(rintf(R(man * shift)), 0.0f, qmax);
      mant = R(ldexpf(q, -mb));  // q / 2^mb
    } else {
      bool normal = !(e == neg_bias);
      float ms = R(man * shift);
      float a1 = clamp_cmp(rintf(R(ms - shift)), 0.0f, qmax);
      float a2 = clamp_cmp(rintf(R(ms * 0.5f)), 0.0f, qmax);
      float q = normal ? R(a1 + R(0.0f * a2)) : R(R(0.0f * a1) + a2);
      const float qs = R(ldexpf(q, -mb));  // q / 2^mb
      float m1 = R(1.0f + qs);
      float m2 = R(qs * 2.0f);
      mant = normal ? R(m1 + R(0.0f * m2)) : R(R(0.0f * m1) + m2);
    }
    float y = R(R(sgn * p2) * mant);
    bool close = (f2bits(val) <= close_thr);
    return close ? R(R(0.0f * y) + x) : R(y + R(0.0f * x));
  }
};

// ---------------------------------------------------------------------------------------------
// minifloat denorm / ieee, value-level kernel.  Preconditions (checked by the launcher): fast_ok of the op (no
// intermediate needs rounding to T) and the exponent clamp range inside [-32, 31].  Then, with k the rounded library
// logarithm and e = clamp(k, e_lo, e_hi),
//   denorm: |y| = min(rint(|x| * 2^(mb-e)), qmax) * 2^(e-mb)
//   ieee:   e != e_lo: |y| = (2^mb + clamp(rint(|x| * 2^(mb-e) - 2^mb), 0, qmax)) * 2^(e-mb)
//           e == e_lo: |y| = min(rint(|x| * 2^(mb-e-1)), qmax) * 2^(e-mb+1)
// (two exact scalings by powers of two collapse into one; where the stepwise form would round a subnormal
// intermediate the product is far below 1/2 and rounds to 0 either way).  rint on the grid is done in place by
// adding and subtracting 1.5 * 2^(23+e-mb), and the clamps are applied to |y| itself.  k comes from one add and one shift: lane L
// keeps, for the biased exponent E = L (mod 64) in [95, 158], delta = 2^23 - 1 - thr (ceil flavour: k = E-127 + (M >
// thr)) or 2^23 - thr (floor flavour: M >= thr), so that (bits + delta) >> 23 = E + carry.  Exponents outside the
// window read some other lane's delta and come out as E or E + 1, which the clamp maps to the same bound as the true
// k.  EPS selects how log2's argument R(|x| + 1e-9) is formed: 0 = it equals |x| for every element whose k can land
// inside the clamp range (fp16 always; bf16 when e_lo >= -20), 1 = fp32 add, 2 = add and round to bf16.
// Non-finite elements take the stepwise evaluation with the table read from memory.
// ---------------------------------------------------------------------------------------------
constexpr int kValueItems = 2;

template <int DT, bool IEEE, int EPS>
__global__ __launch_bounds__(kEwThreads) void minifloat_value_kernel(const void* __restrict__ in, void* __restrict__ out,
                                                                     size_t n8, MinifloatOp<DT, IEEE> op) {
  using TR = DTypeTraits<DT>;
  const int lane = (int)(threadIdx.x & 63);
  // this lane's biased exponent in [95, 158] and its delta
  const int E_l = 95 + ((lane - 95) & 63);
  const uint32_t thr = op.tab[(IEEE ? kLog2TabHalf : 0) + 149 + (E_l - 127)];
  const uint32_t delta = IEEE ? (0x800000u - thr) : (0x7FFFFFu - thr);
  // kValueItems items per lane, 64 items apart, all loaded before the first is worked on: with one item per lane the
  // wavefronts a CU can hold keep too few bytes in flight once an item takes ~140 instructions
  const size_t t0 = (size_t)blockIdx.x * (kEwThreads * kValueItems) + threadIdx.x;
  float xs[kValueItems][8];
#pragma unroll
  for (int u = 0; u < kValueItems; ++u) {
    const size_t t = t0 + (size_t)u * kEwThreads;
    load8<DT, true>(in, t < n8 ? t : n8 - 1, n8, xs[u]);  // every lane takes part in the register permutes
  }
  // clamp bounds of the exponent in place, and the constants that turn (e + 127) << 23 into the rounding constant
  // and into the upper bound of |y| (mb >= 1 for the denorm flavour, checked by the launcher)
  const uint32_t lo_f = (uint32_t)(op.e_lo_i + 127) << 23, hi_f = ((uint32_t)(op.e_hi_i + 127) << 23) | 0x7FFFFFu;
  uint32_t k_magic = ((uint32_t)(23 - op.mb) << 23) + 0x400000u;
  uint32_t k_cap = IEEE ? (0x800000u - (0x800000u >> op.mb))                    // (2 - 2^-mb) * 2^e
                              : (0x800000u - (0x1000000u >> op.mb)) - 0x800000u;      // (2 - 2^(1-mb)) * 2^(e-1)
  [[maybe_unused]] const float cap_sub = op.mb == 0 ? 0.0f : bits2f(lo_f + (0x800000u - (0x1000000u >> op.mb)));
  // one scalar each: left visible, the sums would be taken apart again into two vector additions per element
  asm volatile("" : "+s"(k_magic), "+s"(k_cap));
#pragma unroll
  for (int u = 0; u < kValueItems; ++u) {
  const size_t t = t0 + (size_t)u * kEwThreads;
  const bool live = t < n8;
  float* x = xs[u];
  float y[8];
  uint32_t worst = 0;
  uint32_t lbs[8], ds[8];
  // all eight permutes are issued before the first result is needed
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const uint32_t ab = f2bits(x[j]) & 0x7FFFFFFFu;
    uint32_t lb = ab;
    if constexpr (EPS == 1) lb = f2bits(bits2f(ab) + 1e-9f);
    if constexpr (EPS == 2) lb = f2bits(TR::round(bits2f(ab) + 1e-9f));
    lbs[j] = lb;
    // the permute takes its source lane from address bits 7:2 and ignores the rest: (lb >> 23) mod 64
    ds[j] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(lb >> 21), (int)delta);
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const uint32_t xb = f2bits(x[j]);
    const uint32_t lb = lbs[j], d = ds[j];
    const uint32_t ab = (EPS == 0) ? lb : (xb & 0x7FFFFFFFu);
    const float val = bits2f(ab);
    worst = max(worst, ab);
    // e clamped, kept in place as the exponent field: ebs = (e + 127) << 23
    // (the ieee flavour clamps at e_lo + 1 instead: an element with e == e_lo is rounded on the grid of e_lo + 1)
    const uint32_t kraw = lb + d;
    uint32_t c;
    asm("v_med3_u32 %0, %1, %2, %3" : "=v"(c) : "v"(kraw), "s"(IEEE ? lo_f + 0x800000u : lo_f), "v"(hi_f));  // one scalar operand at most
    const uint32_t ebs = c & 0x7F800000u;
    // rounding to the grid 2^(e-mb) by adding and subtracting 1.5 * 2^(23+e-mb) (exact while |x| < 2^(22+e-mb);
    // beyond that the result only has to stay at or above the upper clamp bound, which it does)
    float yabs;
    if constexpr (!IEEE) {
      const float C = bits2f(ebs + k_magic);
      const float r = (val + C) - C;
      // r >= +0: the order of the bit patterns is the order of the values, and an integer minimum needs no
      // canonicalizing move of the bound first
      yabs = bits2f(min(f2bits(r), ebs + k_cap));  // qmax * 2^(e-mb)
    } else {
      // e == e_lo: grid 2^(e-mb+1), range [0, qmax * 2^(e-mb+1)];  otherwise [2^e, (2^(mb+1) - 1) * 2^(e-mb)]
      const bool sub = kraw < lo_f + 0x800000u;
      const float C = bits2f(ebs + k_magic);
      const uint32_t lo = sub ? 0u : ebs;
      const uint32_t hi = sub ? f2bits(cap_sub) : ebs + k_cap;
      const float r = (val + C) - C;
      // r, lo, hi >= +0: clamped as bit patterns (same order as the values, no canonicalizing moves)
      yabs = bits2f(min(max(f2bits(r), lo), hi));
    }
    const uint32_t yb = (f2bits(yabs) & 0x7FFFFFFFu) | (xb & 0x80000000u);
    // isclose(x, 0): the element passes through, and both zeros become +0 (x + 0.0).  A bitwise select: a
    // conditional here would be compiled into a branch around the arithmetic, with a wait for each permute
    const uint32_t xz = f2bits(x[j] + 0.0f);
    const uint32_t keep = (uint32_t)-(int32_t)(ab <= op.close_thr);
    y[j] = bits2f((xz & keep) | (yb & ~keep));
  }
  if (__builtin_expect(worst >= 0x7F800000u, 0)) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      // an opaque copy: terms of the rare path must not be shared with (and so computed on) the common path
      float xj = x[j];
      asm volatile("" : "+v"(xj));
      if ((f2bits(xj) & 0x7FFFFFFFu) >= 0x7F800000u) y[j] = op.stepwise_from_memory(xj);
    }
  }
  if (live) store8<DT, true>(out, t, n8, y);
  }
}

// ---------------------------------------------------------------------------------------------
// bit-level minifloat cast: _minifloat_mx/fake.py:11-149 (encode to a code, decode it back)
// ---------------------------------------------------------------------------------------------
struct MinifloatMxOp {
  static constexpr bool kUsesTable = false;
  static constexpr int kTableHalf = 0;
  static constexpr bool kBatch = true;
  const uint32_t* tab;
  MinifloatMxFmt m;
  __device__ __forceinline__ float operator()(float x, const WaveLog2&) const {
    return minifloat_mx_decode(minifloat_mx_encode(x, m), m);
  }

  __device__ __forceinline__ void batch8(const float* x, float* y) const { minifloat_mx_qdq8(x, y, m); }
};

// ---------------------------------------------------------------------------------------------
// Bit-level minifloat cast of a 16-bit tensor to the same dtype with the packed 16-bit form (pk16_cast.hpp: about 9
// instructions per element instead of 30, 17 with the in-line handling of the format's subnormal binade).  Lanes
// holding an element outside its domain (Inf/NaN, inputs subnormal in the tensor dtype, the inf/nan exponent of a
// format that has one and, without SUB, codes with exponent field 0) redo their 8 elements with the fp32 form.
// ---------------------------------------------------------------------------------------------
struct MinifloatPk16Params {
  Pk16Format f;
  Pk16Range r;
  uint32_t lo_thr, hi_thr;  // an element e is in the domain iff e == 0 or lo_thr <= |e| < hi_thr (bit patterns)
  MinifloatMxFmt m;
};

template <int DT, bool SUB>
__global__ __launch_bounds__(kEwThreads) void minifloat_mx_pk16_kernel(const uint4* __restrict__ in,
                                                                       uint4* __restrict__ out, size_t n8,
                                                                       MinifloatPk16Params p) {
  constexpr int MB = (DT == MASE_DT_BF16) ? 7 : 10;
  // kValueItems items per lane, 64 items apart, all loaded first (more bytes in flight per wavefront)
  const size_t i0 = (size_t)blockIdx.x * (kEwThreads * kValueItems) + threadIdx.x;
  uint4 vs[kValueItems];
#pragma unroll
  for (int u = 0; u < kValueItems; ++u) {
    const size_t i = i0 + (size_t)u * kEwThreads;
    vs[u] = i < n8 ? load_nt(in + i) : make_uint4(0, 0, 0, 0);
  }
#pragma unroll
  for (int u = 0; u < kValueItems; ++u) {
  const size_t i = i0 + (size_t)u * kEwThreads;
  if (i >= n8) return;
  const uint4 v = vs[u];
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  uint32_t r[4];
  u16x2 lo_acc = as_u16x2(0xFFFFFFFFu), hi_acc = as_u16x2(0u);
#pragma unroll
  for (int j = 0; j < 4; ++j) r[j] = pk16_cast<MB, SUB>(w[j], p.f, p.r, lo_acc, hi_acc);
  const uint32_t lo = min((uint32_t)lo_acc.x, (uint32_t)lo_acc.y), hi = max((uint32_t)hi_acc.x, (uint32_t)hi_acc.y);
  uint4 o = make_uint4(r[0], r[1], r[2], r[3]);
  // SUB: only inputs that are subnormal in T itself (or non-finite) are left over
  const uint32_t lowest = SUB ? (1u << MB) : p.lo_thr;
  if (__builtin_expect(lo + 1u < lowest || hi >= p.hi_thr, 0)) {
    float x[8], y[8];
    DTypeTraits<DT>::unpack(v, x);
    minifloat_mx_qdq8(x, y, p.m);
    o = DTypeTraits<DT>::pack(y);
  }
  store_nt(out + i, o);
  }
}

template <typename MakeOp>
int dispatch_same_dtype(int dtype, MakeOp&& mk) {
  switch (dtype) {
    case MASE_DT_F32: return mk.template run<MASE_DT_F32>();
    case MASE_DT_BF16: return mk.template run<MASE_DT_BF16>();
    case MASE_DT_F16: return mk.template run<MASE_DT_F16>();
    default: return MASE_ERR_DTYPE;
  }
}

struct IntegerRun {
  const void* in; void* out; size_t numel; int dtype, width, frac, is_signed, use_floor; hipStream_t st;
  template <int DT> int run() {
    IntegerOp<DT> op;
    op.tab = nullptr;
    op.frac = frac;
    op.use_floor = use_floor;
    double lo = is_signed ? -(double)(1ull << (width - 1)) : 0.0;
    double hi = is_signed ? (double)((1ull << (width - 1)) - 1) : (double)((1ull << width) - 1);
    op.lo = mase_round_scalar_to_dtype(lo, dtype);
    op.hi = mase_round_scalar_to_dtype(hi, dtype);
    return launch_elementwise<DT, DT>(in, out, numel, op, st);
  }
};

struct MinifloatRun {
  const void* in; void* out; size_t numel; int dtype, width, ew, bias, ieee; const uint32_t* tab; hipStream_t st;
  template <int DT, bool IEEE> int go() {
    MinifloatOp<DT, IEEE> op;
    op.tab = tab;
    op.mb = width - ew - 1;
    op.e_lo = (float)(-bias);
    op.e_hi = (float)((1 << ew) - 1 - bias);
    op.qmax = mase_round_scalar_to_dtype((double)((1 << op.mb) - 1), dtype);
    op.shift = (float)(1 << op.mb);
    op.close_thr = mase_isclose_zero_threshold_bits(dtype);
    op.neg_bias = -mase_round_scalar_to_dtype((double)bias, dtype);
    op.e_lo_i = -bias;
    op.e_hi_i = (1 << ew) - 1 - bias;
    // exactness conditions of the value-level path: significand of the result fits T, 2^e_hi finite in T, the
    // smallest grid step 2^(e_lo - mb) exactly representable in T (fp16: down to its smallest subnormal), the
    // clamp bounds and -bias exact in T
    const int sig_T = (DT == MASE_DT_F32) ? 24 : (DT == MASE_DT_BF16 ? 8 : 11);
    const int max_e = DTypeTraits<DT>::kMaxPow2;
    const int min_step = (DT == MASE_DT_F16) ? -24 : -126;
    const int sig = op.mb + (IEEE ? 1 : 0);
    op.fast_ok = sig <= sig_T && op.e_hi_i <= max_e && op.e_lo_i - op.mb >= min_step &&
                 op.qmax == (float)((1 << op.mb) - 1) && op.neg_bias == (float)(-bias) && bias < 256;
    // value-level kernel on the 16-byte-aligned vector part, the general kernel on what is left
    const bool window = op.e_lo_i >= -32 && op.e_hi_i <= 31 && op.mb <= 16 && (IEEE ? op.e_hi_i > op.e_lo_i : op.mb >= 1);
    size_t done = 0;
    if (op.fast_ok && window && aligned16(in) && aligned16(out) && numel >= 8) {
      const size_t n8 = numel / 8;
      const int eps = (DT == MASE_DT_F16) ? 0 : (DT == MASE_DT_F32 ? 1 : (op.e_lo_i >= -20 ? 0 : 2));
      const dim3 grid(blocks_for(n8, kEwThreads * kValueItems)), block(kEwThreads);
      if (eps == 0) hipLaunchKernelGGL((minifloat_value_kernel<DT, IEEE, 0>), grid, block, 0, st, in, out, n8, op);
      else if (eps == 1) hipLaunchKernelGGL((minifloat_value_kernel<DT, IEEE, 1>), grid, block, 0, st, in, out, n8, op);
      else hipLaunchKernelGGL((minifloat_value_kernel<DT, IEEE, 2>), grid, block, 0, st, in, out, n8, op);
      if (hipGetLastError() != hipSuccess) return MASE_ERR_LAUNCH;
      done = n8 * 8;
      if (done == numel) return MASE_OK;
    }
    const size_t eb = DTypeTraits<DT>::kBytes;
    return launch_elementwise<DT, DT>((const char*)in + done * eb, (char*)out + done * eb, numel - done, op, st);
  }
  template <int DT> int run() { return ieee ? go<DT, true>() : go<DT, false>(); }
};

struct MinifloatMxRun {
  const void* in; void* out; size_t numel; int out_dtype; MinifloatMxFmt m; hipStream_t st;
  // parameters of the packed 16-bit kernel, or false when the format does not fit it
  template <int DT> bool pk16_params(MinifloatPk16Params& q, bool& sub) const {
    Pk16CastParams c;
    if (!make_pk16_cast_params<DT>(m, c)) return false;
    q.f = c.f;
    q.r = c.r;
    q.lo_thr = c.lo_thr;
    q.hi_thr = c.hi_thr;
    q.m = m;
    sub = c.sub;
    return true;
  }
  template <int DTI> int run() {
    MinifloatMxOp op;
    op.tab = nullptr;
    op.m = m;
    if constexpr (DTI != MASE_DT_F32) {
      MinifloatPk16Params q;
      bool sub = false;
      if (out_dtype == DTI && aligned16(in) && aligned16(out) && numel >= 8 && pk16_params<DTI>(q, sub)) {
        const size_t n8 = numel / 8;
        const dim3 grid(blocks_for(n8, kEwThreads * kValueItems)), block(kEwThreads);
        if (sub) hipLaunchKernelGGL((minifloat_mx_pk16_kernel<DTI, true>), grid, block, 0, st, (const uint4*)in, (uint4*)out, n8, q);
        else hipLaunchKernelGGL((minifloat_mx_pk16_kernel<DTI, false>), grid, block, 0, st, (const uint4*)in, (uint4*)out, n8, q);
        if (hipGetLastError() != hipSuccess) return MASE_ERR_LAUNCH;
        if (n8 * 8 == numel) return MASE_OK;
        return launch_elementwise<DTI, DTI>((const char*)in + n8 * 16, (char*)out + n8 * 16, numel - n8 * 8, op, st);
      }
    }
    switch (out_dtype) {
      case MASE_DT_F32: return launch_elementwise<DTI, MASE_DT_F32>(in, out, numel, op, st);
      case MASE_DT_BF16: return launch_elementwise<DTI, MASE_DT_BF16>(in, out, numel, op, st);
      case MASE_DT_F16: return launch_elementwise<DTI, MASE_DT_F16>(in, out, numel, op, st);
      default: return MASE_ERR_DTYPE;
    }
  }
};

}  // namespace
}  // namespace mase

extern "C" int mase_integer_qdq(const void* in, void* out, size_t numel, int dtype, int width, int frac_width,
                                int is_signed, int use_floor, void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (in == nullptr || out == nullptr) return MASE_ERR_NULL;
  if (width < 1 || width > 32 || frac_width < -64 || frac_width > 64) return MASE_ERR_PARAM;
  IntegerRun r{in, out, numel, dtype, width, frac_width, is_signed, use_floor, (hipStream_t)stream};
  return dispatch_same_dtype(dtype, r);
}

extern "C" int mase_minifloat_qdq(const void* in, void* out, size_t numel, int dtype, int width, int exponent_width,
                                  int exponent_bias, int ieee, const uint32_t* log2_tab, void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (in == nullptr || out == nullptr || log2_tab == nullptr) return MASE_ERR_NULL;
  if (exponent_width < 1 || exponent_width > 8 || width - exponent_width - 1 < 0 || width - exponent_width - 1 > 23)
    return MASE_ERR_PARAM;
  int bias = exponent_bias < 0 ? (1 << (exponent_width - 1)) - 1 : exponent_bias;
  if (bias > 255) return MASE_ERR_PARAM;
  MinifloatRun r{in, out, numel, dtype, width, exponent_width, bias, ieee, log2_tab, (hipStream_t)stream};
  return dispatch_same_dtype(dtype, r);
}

extern "C" int mase_minifloat_mx_qdq(const void* in, void* out, size_t numel, int in_dtype, int out_dtype, int exp_bits,
                                     int frac_bits, int is_finite, int round_mode, void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (in == nullptr || out == nullptr) return MASE_ERR_NULL;
  if (exp_bits <= 0 || frac_bits <= 0 || exp_bits + frac_bits >= 16 || round_mode < 0 || round_mode > 3)
    return MASE_ERR_PARAM;
  if (exp_bits > 8) return MASE_ERR_PARAM;  // exponent range beyond fp32's is not representable in the decode
  MinifloatMxFmt m;
  m.E = exp_bits;
  m.F = frac_bits;
  m.bias = (1 << (exp_bits - 1)) - 1;
  m.e_hi = is_finite ? (1 << exp_bits) - 1 : (1 << exp_bits) - 2;
  m.frac_hi = (1 << frac_bits) - 1;
  m.is_finite = is_finite;
  m.round_mode = round_mode;
  MinifloatMxRun r{in, out, numel, out_dtype, m, (hipStream_t)stream};
  return dispatch_same_dtype(in_dtype, r);
}
