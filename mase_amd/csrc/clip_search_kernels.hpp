// Clip search of the MX quantizers for gfx950: quantile_search=True of mxint_quantizer / mxfp_quantizer without
// calibration activations (nn/quantizers/mxint/mxint.py:40-143, nn/quantizers/mxfp/mxfp.py:40-105), which is how
// LinearMXInt quantizes its weight when config["clip_search"] is set (nn/quantized/modules/linear.py:925-933).
//
// Per block of B elements the reference quantizes 11 times, with the block's scale taken from the 1.0, 0.995, 0.99,
// 0.97, 0.95, 0.93, 0.90, 0.80, 0.70, 0.60 and 0.50 quantile of |x| instead of the maximum, and keeps the candidate with
// the smallest error.  It does so with some thirty tensor passes over an [11, n_blocks, B] intermediate; here one
// work-item owns one block: the B (16, 32 or 64) magnitudes are sorted in registers (bitonic network), the quantiles interpolated,
// the candidates with distinct scales evaluated with the device functions of the plain quantizers, and the winner
// written once.
//
// What is reproduced exactly:
//   * the quantile: rank = fl32(q) * (B-1) in fp32, weight w = rank - floor(rank), value = fma(w, hi - lo, lo) for
//     w < 0.5 and fma(w - 1, hi - lo, hi) otherwise (the library's interpolation, measured on its CPU build);
//   * MXINT: the candidate from ceil(log2()) of the quantile rounded to the tensor dtype T, the error as
//     round_T(sqrt(sum round_T(y - x)^2)), the first smallest error wins (argmin);
//   * MXFP: the reference scores a candidate by  q = code / 2^(F-1) * 2^(scale - 127)  with `code` the element's bit
//     pattern as an integer and the power evaluated in uint8 arithmetic (1 << (scale - 127) for scale in 127..134, else
//     0), error = round_T(sum round_T(round_T(q - x)^2)), and replaces the incumbent only on a strictly smaller error;
//     that scoring is kept as it is, so the same candidate wins.  A zero quantile in a block that is not all zero gives
//     the scale byte 255 (the conversion of -inf wraps) and a candidate that dequantizes to NaN, as in the reference.
// What is not: the order in which the library adds the 32 squares (vector lanes, then a tree; it differs between its
// CPU builds and its GPU kernels).  Here they are added in element order with fp32 fma.  Two candidates whose errors
// differ by less than that rounding can therefore swap; the tests bound this.
// Inf / NaN inputs are not specified.  `ref` is the tensor in its original flattening: the reference measures the error
// of the blocks taken along block_dim against the blocks of the plain flattening (the same thing when block_dim is the
// last dimension).
#include "common.hpp"
//
// This header holds the kernels; clip_search_mx*_b*.hip each instantiate one quantizer family for one block size (the
// sorting networks make these the slowest kernels of the library to compile, so they are spread over translation
// units), and clip_search.hip holds the entry points.
#pragma once
#include "common.hpp"
#include "mxint_core.hpp"
#include "mxfp_core.hpp"

#include <type_traits>

namespace mase {
namespace {

constexpr int kCand = 11;
constexpr double kClipPercentiles[kCand] = {1.0, 0.995, 0.99, 0.97, 0.95, 0.93, 0.90, 0.80, 0.70, 0.60, 0.50};

// interpolation plan of candidate P for blocks of B elements (all in fp32, as the library computes it)
template <int B, int P>
struct ClipRank {
  static constexpr float q = (float)kClipPercentiles[P];
  static constexpr float rank = q * (float)(B - 1);
  static constexpr int lo = (int)rank;
  static constexpr int hi = ((float)lo < rank) ? lo + 1 : lo;
  static constexpr float w = rank - (float)lo;
  static constexpr bool small = w < 0.5f;
  static constexpr float coeff = small ? w : w - 1.0f;
  static constexpr int base = small ? lo : hi;
};

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

template <int B>
__device__ __forceinline__ void sort_ascending(uint32_t* s) {
  constexpr int LOGB = (B == 16) ? 4 : (B == 32) ? 5 : 6;
#pragma unroll
  for (int lk = 1; lk <= LOGB; ++lk) {
#pragma unroll
    for (int lj = lk - 1; lj >= 0; --lj) {
#pragma unroll
      for (int i = 0; i < B; ++i) {
        const int l = i ^ (1 << lj);
        if (l > i) {
          const bool up = (i & (1 << lk)) == 0;
          const uint32_t a = s[i], b = s[l];
          const uint32_t mn = min(a, b), mx = max(a, b);
          s[i] = up ? mn : mx;
          s[l] = up ? mx : mn;
        }
      }
    }
  }
}

template <int DT, int B>
__device__ __forceinline__ void load_block(const void* p, size_t blk, float* x) {
  using TR = DTypeTraits<DT>;
  constexpr int V = TR::kVec;
  const uint4* v = (const uint4*)p + blk * (B / V);
#pragma unroll
  for (int j = 0; j < B / V; ++j) TR::unpack(v[j], x + j * V);
}

template <int B, int P>
__device__ __forceinline__ float clip_quantile(const uint32_t* s) {
  using R = ClipRank<B, P>;
  return __builtin_fmaf(R::coeff, bits2f(s[R::hi]) - bits2f(s[R::lo]), bits2f(s[R::base]));
}

// index of the next candidate after P whose exponent differs from `cur` (kCand when there is none); the exponents
// fall monotonically with the percentile, so equal ones are neighbours
__device__ __forceinline__ int next_distinct(const int* key, int P, int cur) {
  int nxt = kCand;
#pragma unroll
  for (int j = kCand - 1; j >= 1; --j) nxt = (j > P && key[j] != cur) ? j : nxt;
  return nxt;
}

__device__ __forceinline__ int select_key(const int* key, int P) {
  int v = key[0];
#pragma unroll
  for (int j = 1; j < kCand; ++j) v = (P == j) ? key[j] : v;
  return v;
}

// Candidates with the same exponent are the same candidate, and with the first-minimum rule only the first of them
// can win: a work-item evaluates each distinct exponent once (typically 3 of the 11), in percentile order.
template <int DT, int B>
// (Blocks of 32: the allocator is asked for three wavefronts per SIMD, i.e. at most 168 registers; left alone it takes
// 186 to 216 and two wavefronts fit.  bf16: 267 -> 222 us on 8 x 2048 x 4096, same results; the fp16 form would spill
// and was measured slower, so it keeps its registers.)
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu((B == 32 && DT != MASE_DT_F16) ? 3 : 1))) void mxint_clip_search_kernel(const void* __restrict__ in, const void* __restrict__ ref,
                                                               void* __restrict__ out, uint8_t* __restrict__ choice,
                                                               size_t n_blocks, MxintParams p) {
  using TR = DTypeTraits<DT>;
  constexpr int V = TR::kVec;
  constexpr int kNanKey = 4096, kOverflowKey = 2048;  // block_exponent states 2 and 1 (k > any finite exponent)
  const size_t blk = (size_t)blockIdx.x * 64 + threadIdx.x;
  if (blk >= n_blocks) return;
  float x[B], r[B], best_y[B];
  load_block<DT, B>(in, blk, x);
  load_block<DT, B>(ref, blk, r);
  int key[kCand];
  {
    uint32_t s[B];
#pragma unroll
    for (int i = 0; i < B; ++i) s[i] = f2bits(x[i]) & 0x7FFFFFFFu;
    sort_ascending<B>(s);
    static_for<0, kCand>([&](auto pc) __attribute__((always_inline)) {
      constexpr int P = decltype(pc)::value;
      const uint32_t mbits = f2bits(TR::round(clip_quantile<B, P>(s)));
      int k = 0, kc = 0;
      const int state = block_exponent<DT>(mbits, p, k, kc);
      key[P] = (state == 2) ? kNanKey : (k >= 1024 ? kOverflowKey : k);
    });
  }
  float best_err = 0.0f;
  int best = 0;
  int P = 0;
  while (P < kCand) {
    const int cur = select_key(key, P);
    const int state = (cur == kNanKey) ? 2 : (cur > TR::kMaxPow2 ? 1 : 0);
    const int k = (cur == kOverflowKey) ? 1024 : cur;
    const int kc = min(max(k + p.bias, 0), p.scale_max) - p.bias;
    float y[B];
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < B; ++i) {
      int code;
      y[i] = TR::round(mxint_element<DT>(x[i], state, k, kc, p, code));
      const float d = TR::round(y[i] - r[i]);
      acc = __builtin_fmaf(d, d, acc);
    }
    const float err = TR::round(sqrtf(acc));
    const bool take = (P == 0) || (err < best_err);
    best_err = take ? err : best_err;
    best = take ? P : best;
#pragma unroll
    for (int i = 0; i < B; ++i) best_y[i] = take ? y[i] : best_y[i];
    P = next_distinct(key, P, cur);
  }
  uint4* o = (uint4*)out + blk * (B / V);
#pragma unroll
  for (int j = 0; j < B / V; ++j) o[j] = TR::pack(best_y + j * V);
  if (choice != nullptr) choice[blk] = (uint8_t)best;
}

template <int DT, int B>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(B == 32 ? 3 : 1))) void mxfp_clip_search_kernel(const void* __restrict__ in, const void* __restrict__ ref,
                                                              void* __restrict__ out, uint8_t* __restrict__ choice,
                                                              size_t n_blocks, MxfpParams p) {
  using TR = DTypeTraits<DT>;
  constexpr int V = TR::kVec;
  // keys: the shift sh of a regular candidate (-127 .. 127); 128: zero quantile in a block that is not all zero
  // (floor(log2) is -inf, whose int32 conversion minus el_emax wraps to a large positive number: scale byte 255,
  // elements x / inf); kFlushedKey: every element flushed; kNanKey: the quantile is not finite
  constexpr int kFlushedKey = 4096, kNanKey = 2048;
  const size_t blk = (size_t)blockIdx.x * 64 + threadIdx.x;
  if (blk >= n_blocks) return;
  float t[B], r[B], best_y[B];
  load_block<DT, B>(in, blk, t);
  load_block<DT, B>(ref, blk, r);
  int key[kCand];
  {
    uint32_t s[B];
#pragma unroll
    for (int i = 0; i < B; ++i) {
      t[i] = flush_subnormal(t[i]);
      s[i] = f2bits(t[i]) & 0x7FFFFFFFu;
    }
    sort_ascending<B>(s);
    const bool all_flushed = s[B - 1] == 0;
    static_for<0, kCand>([&](auto pc) __attribute__((always_inline)) {
      constexpr int P = decltype(pc)::value;
      int sh = 0;
      const int state = mxfp_block_scale(f2bits(clip_quantile<B, P>(s)), p, sh);  // the lookup runs on a stand-in for 0
      key[P] = all_flushed ? kFlushedKey : (state == 0 ? 128 : (state == 2 ? kNanKey : sh));
    });
  }
  const float code_unit = pow2f(1 - p.m.F);  // 1 / 2^(F-1)
  float best_err = bits2f(0x7F800000u);
  int best = 0;
  int P = 0;
  while (P < kCand) {
    const int cur = select_key(key, P);
    const int state = (cur == kFlushedKey) ? 0 : (cur == kNanKey ? 2 : (cur == 128 ? 3 : 1));
    const int sh = cur;
    const int sc = (state == 0) ? 0 : sh + 127;
    const float unit = ((sc >= 127 && sc <= 134) ? (float)(1 << (sc - 127)) : 0.0f) * code_unit;
    float y[B];
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < B; ++i) {
      uint32_t code;
      if (state == 3) {
        code = minifloat_mx_encode(bits2f(f2bits(t[i]) & 0x80000000u), p.m);
        y[i] = qnan();
      } else {
        y[i] = mxfp_element(t[i], state, sh, p, code);
      }
      const float qs = TR::round((float)code * unit);
      const float d = fabsf(TR::round(qs - r[i]));
      acc += TR::round(d * d);
    }
    const float err = TR::round(acc);
    const bool take = (P == 0) || (err < best_err);  // the incumbent starts as candidate 0 whatever its error
    best_err = (err < best_err) ? err : best_err;
    best = take ? P : best;
#pragma unroll
    for (int i = 0; i < B; ++i) best_y[i] = take ? y[i] : best_y[i];
    P = next_distinct(key, P, cur);
  }
  uint4* o = (uint4*)out + blk * (B / V);
#pragma unroll
  for (int j = 0; j < B / V; ++j) o[j] = TR::pack(best_y + j * V);
  if (choice != nullptr) choice[blk] = (uint8_t)best;
}

// All eleven candidates of every block instead of the winner: what the search scored on calibration outputs needs
// (nn/quantizers/mxint/mxint.py:99-131, nn/quantizers/mxfp/mxfp.py:65-93), where a candidate's error is a norm over whole
// batches of activations times the candidate and is left to matrix products on the host side.  cand[P * numel + i]:
// element i of the tensor quantized with the scale of percentile P.  MXFP also writes the values the reference
// scores, code / 2^(F-1) * 2^(scale - 127) on the integer codes with the power in uint8 arithmetic (see above).
template <int DT, int B>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(B == 32 ? 3 : 1))) void mxint_clip_candidates_kernel(const void* __restrict__ in, void* __restrict__ cand,
                                                                   size_t n_blocks, MxintParams p) {
  using TR = DTypeTraits<DT>;
  constexpr int V = TR::kVec;
  const size_t blk = (size_t)blockIdx.x * 64 + threadIdx.x;
  if (blk >= n_blocks) return;
  float x[B];
  load_block<DT, B>(in, blk, x);
  uint32_t s[B];
#pragma unroll
  for (int i = 0; i < B; ++i) s[i] = f2bits(x[i]) & 0x7FFFFFFFu;
  sort_ascending<B>(s);
  static_for<0, kCand>([&](auto pc) __attribute__((always_inline)) {
    constexpr int P = decltype(pc)::value;
    const uint32_t mbits = f2bits(TR::round(clip_quantile<B, P>(s)));
    int k = 0, kc = 0;
    const int state = block_exponent<DT>(mbits, p, k, kc);
    float y[B];
#pragma unroll
    for (int i = 0; i < B; ++i) {
      int code;
      y[i] = TR::round(mxint_element<DT>(x[i], state, k, kc, p, code));
    }
    uint4* o = (uint4*)cand + ((size_t)P * n_blocks + blk) * (B / V);
#pragma unroll
    for (int j = 0; j < B / V; ++j) o[j] = TR::pack(y + j * V);
  });
}

template <int DT, int B>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(B == 32 ? 3 : 1))) void mxfp_clip_candidates_kernel(const void* __restrict__ in, void* __restrict__ cand,
                                                                  void* __restrict__ score, size_t n_blocks,
                                                                  MxfpParams p) {
  using TR = DTypeTraits<DT>;
  constexpr int V = TR::kVec;
  const size_t blk = (size_t)blockIdx.x * 64 + threadIdx.x;
  if (blk >= n_blocks) return;
  float t[B];
  load_block<DT, B>(in, blk, t);
  uint32_t s[B];
#pragma unroll
  for (int i = 0; i < B; ++i) {
    t[i] = flush_subnormal(t[i]);
    s[i] = f2bits(t[i]) & 0x7FFFFFFFu;
  }
  sort_ascending<B>(s);
  const bool all_flushed = s[B - 1] == 0;
  const float code_unit = pow2f(1 - p.m.F);  // 1 / 2^(F-1)
  static_for<0, kCand>([&](auto pc) __attribute__((always_inline)) {
    constexpr int P = decltype(pc)::value;
    int sh = 0;
    int state = mxfp_block_scale(f2bits(clip_quantile<B, P>(s)), p, sh);
    // states as in the search kernel: 0 all flushed, 1 regular, 2 quantile not finite, 3 zero quantile in a block
    // that is not all zero (scale byte 255, elements x / inf, value NaN)
    state = all_flushed ? 0 : (state == 0 ? 3 : state);
    const int sc = (state == 0) ? 0 : (state == 1 ? sh + 127 : 255);
    const float unit = ((sc >= 127 && sc <= 134) ? (float)(1 << (sc - 127)) : 0.0f) * code_unit;
    float y[B], q[B];
#pragma unroll
    for (int i = 0; i < B; ++i) {
      uint32_t code;
      if (state == 3) {
        code = minifloat_mx_encode(bits2f(f2bits(t[i]) & 0x80000000u), p.m);
        y[i] = qnan();
      } else {
        y[i] = mxfp_element(t[i], state, sh, p, code);
      }
      q[i] = TR::round((float)code * unit);
    }
    uint4* o = (uint4*)cand + ((size_t)P * n_blocks + blk) * (B / V);
    uint4* oq = (uint4*)score + ((size_t)P * n_blocks + blk) * (B / V);
#pragma unroll
    for (int j = 0; j < B / V; ++j) {
      o[j] = TR::pack(y + j * V);
      oq[j] = TR::pack(q + j * V);
    }
  });
}
}  // namespace

// launchers of the instantiations for one block size, defined once each in the clip_search_mx*_b*.hip units
#define MASE_CLIP_DECLARE(B)                                                                                          \
  int clip_mxint_search_b##B(int dtype, const void* in, const void* ref, void* out, uint8_t* choice, size_t n_blocks, \
                             const MxintParams& p, hipStream_t st);                                                   \
  int clip_mxint_candidates_b##B(int dtype, const void* in, void* cand, size_t n_blocks, const MxintParams& p,        \
                                 hipStream_t st);                                                                     \
  int clip_mxfp_search_b##B(int dtype, const void* in, const void* ref, void* out, uint8_t* choice, size_t n_blocks,  \
                            const MxfpParams& p, hipStream_t st);                                                     \
  int clip_mxfp_candidates_b##B(int dtype, const void* in, void* cand, void* score, size_t n_blocks,                  \
                                const MxfpParams& p, hipStream_t st);
MASE_CLIP_DECLARE(16)
MASE_CLIP_DECLARE(32)
MASE_CLIP_DECLARE(64)
#undef MASE_CLIP_DECLARE

#define MASE_CLIP_BY_DTYPE(CALL)                                                     \
  switch (dtype) {                                                                   \
    case MASE_DT_F32: { constexpr int DT = MASE_DT_F32; CALL; break; }               \
    case MASE_DT_BF16: { constexpr int DT = MASE_DT_BF16; CALL; break; }             \
    case MASE_DT_F16: { constexpr int DT = MASE_DT_F16; CALL; break; }               \
    default: return MASE_ERR_DTYPE;                                                  \
  }                                                                                  \
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;

#define MASE_CLIP_DEFINE_MXINT(B)                                                                                      \
  int clip_mxint_search_b##B(int dtype, const void* in, const void* ref, void* out, uint8_t* choice, size_t n_blocks,  \
                             const MxintParams& p, hipStream_t st) {                                                   \
    MASE_CLIP_BY_DTYPE(hipLaunchKernelGGL((mxint_clip_search_kernel<DT, B>), dim3(blocks_for(n_blocks, 64)), dim3(64), \
                                          0, st, in, ref, out, choice, n_blocks, p))                                   \
  }                                                                                                                    \
  int clip_mxint_candidates_b##B(int dtype, const void* in, void* cand, size_t n_blocks, const MxintParams& p,         \
                                 hipStream_t st) {                                                                     \
    MASE_CLIP_BY_DTYPE(hipLaunchKernelGGL((mxint_clip_candidates_kernel<DT, B>), dim3(blocks_for(n_blocks, 64)),       \
                                          dim3(64), 0, st, in, cand, n_blocks, p))                                     \
  }

#define MASE_CLIP_DEFINE_MXFP(B)                                                                                       \
  int clip_mxfp_search_b##B(int dtype, const void* in, const void* ref, void* out, uint8_t* choice, size_t n_blocks,   \
                            const MxfpParams& p, hipStream_t st) {                                                     \
    MASE_CLIP_BY_DTYPE(hipLaunchKernelGGL((mxfp_clip_search_kernel<DT, B>), dim3(blocks_for(n_blocks, 64)), dim3(64),  \
                                          0, st, in, ref, out, choice, n_blocks, p))                                   \
  }                                                                                                                    \
  int clip_mxfp_candidates_b##B(int dtype, const void* in, void* cand, void* score, size_t n_blocks,                   \
                                const MxfpParams& p, hipStream_t st) {                                                 \
    MASE_CLIP_BY_DTYPE(hipLaunchKernelGGL((mxfp_clip_candidates_kernel<DT, B>), dim3(blocks_for(n_blocks, 64)),        \
                                          dim3(64), 0, st, in, cand, score, n_blocks, p))                              \
  }

}  // namespace mase
