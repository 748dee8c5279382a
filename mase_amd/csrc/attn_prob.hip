// Attention probabilities of the MX-quantized Llama attention in one pass over the score matrix (gfx950).
//
// Reference sequence (nn/quantized/modules/llama/attention.py:334-393, _eager_attention_forward_mxfp/_mxint), on the
// [batch, heads, q_len, kv_len] result s of the query-key product, every step a full tensor pass in dtype T:
//   w = R(s * scaling);  w = R(w + mask)                         (mask [batch, 1, q_len, kv_len], optional)
//   w = minifloat_cast(w)                                        (softmax_minifloat, functional/softmax.py:41-57)
//   p = R(softmax(float(w), dim=-1))                             (fp32 softmax, cast back to T)
//   p = mx_quantize(p, block 32 along kv_len)                    (MXINT in T arithmetic, MXFP in fp32)
// R(.) rounds to T.  Here one wavefront owns one row: the row stays in registers between the steps, so the tensor
// is read once and written once (2 + 2 bytes per element for 16-bit T, against about 36 for the separate passes).
// HBM-bound; the mask rows are shared by all heads and come from the cache.
//
// The exponentials (hardware exp2 with a compensated argument, about 2 ulp), the order of the row sum and the
// normalisation (multiplication by the reciprocal of the sum) differ from the library's softmax kernel by rounding, so
// results agree with the separate-pass form to the last bits of fp32 before the rounding to T, not bit for bit.
#include "common.hpp"
#include "minifloat_mx.hpp"
#include "mxfp_core.hpp"
#include "mxint_core.hpp"
#include "pk16_cast.hpp"

namespace mase {
namespace {

constexpr int kRowThreads = 64;  // one wavefront per row
constexpr int kChunk = 64 * 8;   // elements of a row handled per step: 8 per lane

struct AttnProbParams {
  const void* scores;
  const void* mask;     // may be null
  void* out;
  size_t rows;          // batch * heads * q_len
  int cols;             // kv_len: a multiple of 32
  int heads, q_len;     // mask row of score row r: (r / (heads * q_len)) * q_len + r % q_len
  size_t mask_row_stride;  // elements between mask rows
  float scaling;
  int cast_on;          // 0: softmax on the masked scores as they are
  MinifloatMxFmt cast;
  int pk_on;            // 16-bit T: the cast runs on packed 16-bit patterns (pk16_cast.hpp) with these parameters
  Pk16CastParams pk;
  int mx_kind;          // 0 none, 1 MXINT, 2 MXFP
  MxintParams qi;
  MxfpParams qf;
};

template <int DT>
__device__ __forceinline__ void load_row8(const void* base, size_t elem, float* x) {
  using TR = DTypeTraits<DT>;
  const uint4* q = (const uint4*)((const char*)base + elem * TR::kBytes);
  if constexpr (TR::kVec == 4) {
    TR::unpack(q[0], x);
    TR::unpack(q[1], x + 4);
  } else {
    TR::unpack(load_nt(q), x);
  }
}

// exp(x) for x <= 0: exp2 of x * log2(e), with the rounding error of that product fed back to first order
__device__ __forceinline__ float exp_neg(float x) {
  const float kLog2e = 1.4426950408889634f, kLog2eLo = 1.925963033500227e-8f, kLn2 = 0.6931471805599453f;
  x = fmaxf(x, -150.0f);  // exp(-150) is 0 in fp32; keeps -inf (masked, or beyond the row) out of the error term
  const float t = x * kLog2e;
  const float r = __builtin_fmaf(x, kLog2e, -t) + x * kLog2eLo;  // x * log2(e) - t
  const float y = __builtin_amdgcn_exp2f(t);
  return __builtin_fmaf(y, r * kLn2, y);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

template <int DT, int NCH>
__global__ __launch_bounds__(kRowThreads) void attn_prob_kernel(AttnProbParams p) {
  using TR = DTypeTraits<DT>;
  const int lane = (int)(threadIdx.x & 63);
  const size_t row = blockIdx.x;
  const char* srow = (const char*)p.scores + row * (size_t)p.cols * TR::kBytes;
  const size_t per_batch = (size_t)p.heads * (size_t)p.q_len;
  const size_t mrow = (row / per_batch) * (size_t)p.q_len + row % (size_t)p.q_len;
  const char* mbase = p.mask ? (const char*)p.mask + mrow * p.mask_row_stride * TR::kBytes : nullptr;
  WaveLog2 meta_i, meta_f;
  if (p.mx_kind == 1) meta_i.init(p.qi.tab, 0);
  if (p.mx_kind == 2) meta_f.init(p.qf.tab, kLog2TabHalf);

  float w[NCH][8];
  float row_max = -__builtin_inff();
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e0 = (c * 64 + lane) * 8;
    const bool live = e0 < p.cols;  // uniform over each group of 4 lanes (cols is a multiple of 32)
    float s[8], m[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) { s[j] = 0.0f; m[j] = 0.0f; }
    if (live) {
      load_row8<DT>(srow, (size_t)e0, s);
      if (mbase) load_row8<DT>(mbase, (size_t)e0, m);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float v = TR::round(s[j] * p.scaling);
      if (mbase) v = TR::round(v + m[j]);
      s[j] = v;
    }
    if (p.cast_on) {
      bool done = false;
      if constexpr (DT != MASE_DT_F32) {
        if (p.pk_on) {  // the masked scores are values of T: cast their bit patterns two per register
          constexpr int MB = (DT == MASE_DT_BF16) ? 7 : 10;
          uint4 v;
          if constexpr (DT == MASE_DT_BF16) {
            v = make_uint4(pack_bf16_exact(s[0], s[1]), pack_bf16_exact(s[2], s[3]), pack_bf16_exact(s[4], s[5]),
                           pack_bf16_exact(s[6], s[7]));
          } else {
            v = TR::pack(s);
          }
          const uint32_t w[4] = {v.x, v.y, v.z, v.w};
          uint32_t r[4];
          u16x2 lo_acc = as_u16x2(0xFFFFFFFFu), hi_acc = as_u16x2(0u);
          if (p.pk.sub) {
#pragma unroll
            for (int j = 0; j < 4; ++j) r[j] = pk16_cast<MB, true>(w[j], p.pk.f, p.pk.r, lo_acc, hi_acc);
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) r[j] = pk16_cast<MB, false>(w[j], p.pk.f, p.pk.r, lo_acc, hi_acc);
          }
          const uint32_t lo = min((uint32_t)lo_acc.x, (uint32_t)lo_acc.y), hi = max((uint32_t)hi_acc.x, (uint32_t)hi_acc.y);
          const uint32_t lowest = p.pk.sub ? (1u << MB) : p.pk.lo_thr;
          // a lane with an element outside the packed form's domain takes the step-by-step cast below
          done = !(lo + 1u < lowest || hi >= p.pk.hi_thr);
          if (done) TR::unpack(make_uint4(r[0], r[1], r[2], r[3]), s);
        }
      }
      if (!done) {
        float y[8];
        minifloat_mx_qdq8(s, y, p.cast);
#pragma unroll
        for (int j = 0; j < 8; ++j) s[j] = TR::round(y[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      w[c][j] = live ? s[j] : -__builtin_inff();
      row_max = fmaxf(row_max, w[c][j]);
    }
  }
  row_max = wave_max(row_max);
  float sum = 0.0f;
#pragma unroll
  for (int c = 0; c < NCH; ++c)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      w[c][j] = exp_neg(w[c][j] - row_max);
      sum += w[c][j];
    }
  sum = wave_sum(sum);
  const float inv_sum = 1.0f / sum;

#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e0 = (c * 64 + lane) * 8;
    const bool live = e0 < p.cols;
    float x[8], y[8];
    uint32_t mbits = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      x[j] = TR::round(w[c][j] * inv_sum);
      mbits = max(mbits, f2bits(x[j]) & 0x7FFFFFFFu);
    }
    if (p.mx_kind == 1) {
      // MXINT block of 32 = 4 lanes; arithmetic of qdq_mxint's vector kernel
      const uint32_t mx = group_max_u32<4>(mbits);
      int k = 0, kc = 0;
      const int state = block_exponent<DT>(mx, p.qi, k, kc, meta_i);
      int code;
      if (state == 0) {
        const int up = p.qi.qshift - k, dn = kc - p.qi.qshift;
#pragma unroll
        for (int j = 0; j < 8; ++j) y[j] = ldexpf(fminf(fmaxf(rintf(ldexpf(x[j], up)), p.qi.lo), p.qi.hi), dn);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) y[j] = mxint_element<DT>(x[j], state, k, kc, p.qi, code);
      }
    } else if (p.mx_kind == 2) {
      const uint32_t flushed = ((mbits & 0x7F800000u) == 0) ? 0u : mbits;  // per lane; a larger lane decides anyway
      const uint32_t mx = group_max_u32<4>(flushed);
      int sh = 0;
      const int state = mxfp_block_scale(mx, p.qf, sh, meta_f);
      uint32_t codes[8];
      if (p.qf.m.E >= 4) mxfp_elements<false, 8>(x, state, sh, p.qf, codes, y);
      else mxfp_elements<true, 8>(x, state, sh, p.qf, codes, y);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = x[j];
    }
    if (live) {
      uint4* q = (uint4*)((char*)p.out + (row * (size_t)p.cols + (size_t)e0) * TR::kBytes);
      if constexpr (TR::kVec == 4) {
        q[0] = TR::pack(y);
        q[1] = TR::pack(y + 4);
      } else {
        store_nt(q, TR::pack(y));
      }
    }
  }
}

template <int DT>
int launch_attn_prob(const AttnProbParams& p, hipStream_t st) {
  const int nch = (p.cols + kChunk - 1) / kChunk;
  const dim3 grid((unsigned)p.rows), block(kRowThreads);
  if (nch <= 1) hipLaunchKernelGGL((attn_prob_kernel<DT, 1>), grid, block, 0, st, p);
  else if (nch <= 2) hipLaunchKernelGGL((attn_prob_kernel<DT, 2>), grid, block, 0, st, p);
  else if (nch <= 4) hipLaunchKernelGGL((attn_prob_kernel<DT, 4>), grid, block, 0, st, p);
  else if (nch <= 8) hipLaunchKernelGGL((attn_prob_kernel<DT, 8>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((attn_prob_kernel<DT, 16>), grid, block, 0, st, p);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

}  // namespace
}  // namespace mase

extern "C" int mase_attn_softmax_mx(const void* scores, const void* mask, void* out, size_t batch, size_t heads,
                                    size_t q_len, size_t kv_len, size_t mask_row_stride, int dtype, float scaling,
                                    int cast_exp_bits, int cast_frac_bits, int cast_is_finite, int cast_round_mode,
                                    int mx_kind, int mx_p0, int mx_p1, const uint32_t* log2_tab_dtype,
                                    const uint32_t* log2_tab_f32, void* stream) {
  using namespace mase;
  const size_t rows = batch * heads * q_len;
  if (rows == 0 || kv_len == 0) return MASE_OK;
  if (scores == nullptr || out == nullptr) return MASE_ERR_NULL;
  if (kv_len % 32 != 0 || kv_len > 16 * (size_t)kChunk || rows > 0x7FFFFFFFull) return MASE_ERR_SHAPE;
  if (mask != nullptr && (mask_row_stride < kv_len || mask_row_stride % 8 != 0)) return MASE_ERR_SHAPE;
  if (!aligned16(scores) || !aligned16(out) || (mask != nullptr && !aligned16(mask))) return MASE_ERR_ALIGN;
  if (dtype < 0 || dtype > 2) return MASE_ERR_DTYPE;
  AttnProbParams p{};
  p.scores = scores;
  p.mask = mask;
  p.out = out;
  p.rows = rows;
  p.cols = (int)kv_len;
  p.heads = (int)heads;
  p.q_len = (int)q_len;
  p.mask_row_stride = mask_row_stride;
  p.scaling = scaling;
  p.cast_on = cast_exp_bits > 0;
  if (p.cast_on) {
    if (cast_frac_bits <= 0 || cast_exp_bits > 8 || cast_exp_bits + cast_frac_bits >= 16 || cast_round_mode < 0 ||
        cast_round_mode > 3)
      return MASE_ERR_PARAM;
    p.cast.E = cast_exp_bits;
    p.cast.F = cast_frac_bits;
    p.cast.bias = (1 << (cast_exp_bits - 1)) - 1;
    p.cast.e_hi = cast_is_finite ? (1 << cast_exp_bits) - 1 : (1 << cast_exp_bits) - 2;
    p.cast.frac_hi = (1 << cast_frac_bits) - 1;
    p.cast.is_finite = cast_is_finite;
    p.cast.round_mode = cast_round_mode;
    if (dtype == MASE_DT_BF16) p.pk_on = make_pk16_cast_params<MASE_DT_BF16>(p.cast, p.pk) ? 1 : 0;
    else if (dtype == MASE_DT_F16) p.pk_on = make_pk16_cast_params<MASE_DT_F16>(p.cast, p.pk) ? 1 : 0;
  }
  p.mx_kind = mx_kind;
  if (mx_kind == 1) {
    if (log2_tab_dtype == nullptr) return MASE_ERR_NULL;
    if (mx_p0 < 2 || mx_p0 > 24) return MASE_ERR_PARAM;
    p.qi.qshift = mx_p0 - 1;
    p.qi.bias = 127;
    p.qi.scale_max = 255;
    p.qi.lo = mase_round_scalar_to_dtype(-(double)(1 << (mx_p0 - 1)), dtype);
    p.qi.hi = mase_round_scalar_to_dtype((double)((1 << (mx_p0 - 1)) - 1), dtype);
    p.qi.tab = log2_tab_dtype;
  } else if (mx_kind == 2) {
    if (log2_tab_f32 == nullptr) return MASE_ERR_NULL;
    const int E = mx_p0, F = mx_p1;
    const bool legal = (E == 4 && F == 3) || (E == 5 && F == 2) || (E == 2 && F == 3) || (E == 3 && F == 2) ||
                       (E == 2 && F == 1) || (E == 1 && F == 2);
    if (!legal) return MASE_ERR_PARAM;
    p.qf.m.E = E;
    p.qf.m.F = F;
    p.qf.m.bias = (1 << (E - 1)) - 1;
    p.qf.m.e_hi = (1 << E) - 1;
    p.qf.m.frac_hi = (1 << F) - 1;
    p.qf.m.is_finite = 1;
    p.qf.m.round_mode = 0;
    p.qf.el_emax = p.qf.m.e_hi - p.qf.m.bias;
    p.qf.tab = log2_tab_f32;
  } else if (mx_kind != 0) {
    return MASE_ERR_PARAM;
  }
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case MASE_DT_F32: return launch_attn_prob<MASE_DT_F32>(p, st);
    case MASE_DT_BF16: return launch_attn_prob<MASE_DT_BF16>(p, st);
    default: return launch_attn_prob<MASE_DT_F16>(p, st);
  }
}
