// Row-wise and element-wise layers around the quantized Linears of a Llama block, each in one pass (gfx950):
//   RMSNorm with optional minifloat casts of the input and of the weight (nn/quantized/modules/llama/rms_norm.py:72-84;
//   with both casts off: the plain RMSNorm, models/llama/modeling_llama.py:79-93)
//   rotary embedding x * cos + rotate_half(x) * sin (nn/quantized/functional/rope.py:8-27; the minifloat cast of
//   rope_minifloat applies to the small cos / sin tables and is done by the caller)
//   SiLU(cast(gate)) * up (nn/quantized/modules/llama/mlp.py:60-62 with functional/silu.py:41-57; cast off: the plain
//   SwiGLU product, models/llama/modeling_llama.py:219-236)
// RMSNorm and the SwiGLU product can also hand their result on already MXINT-quantized (blocks of 32 along the last
// dimension, the arithmetic of qdq_mxint's vector kernel on the values rounded to T): what the LinearMXInt that
// consumes them would compute from the stored tensor in a pass of its own (nn/quantized/modules/linear.py:956-972).
// Every intermediate is rounded to the tensor dtype T where the separate tensor operations would round it.  Both are
// HBM-bound: the tensor is read once and written once, against 10-20 passes of the separate operations.
#include "common.hpp"
#include "minifloat_mx.hpp"
#include "mxint_core.hpp"

namespace mase {
namespace {

constexpr int kRowThreads = 64;

struct CastSpec {
  int on;
  MinifloatMxFmt m;
};

struct RmsNormParams {
  const void* x;
  const void* weight;
  void* out;
  const void* residual;  // when set: the row normalised is x + residual, rounded to the dtype and also stored to sum_out
  void* sum_out;
  size_t rows;
  int cols;  // multiple of 8, at most 8192
  float eps;
  CastSpec x_cast, w_cast;
  MxintParams mx;  // MX instantiation only
};

// MXINT quantize-dequantize of the 8 values a lane has just produced (already rounded to T); a block of 32 is the 4
// lanes of a group.  Every lane of the wavefront must take part (register permutes).
template <int DT>
__device__ __forceinline__ void mxint_block32(float* v, const MxintParams& q, const WaveLog2& meta) {
  uint32_t mbits = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) mbits = max(mbits, f2bits(v[j]) & 0x7FFFFFFFu);
  const uint32_t mx = group_max_u32<4>(mbits);
  int k = 0, kc = 0;
  const int state = block_exponent<DT>(mx, q, k, kc, meta);
  if (state == 0) {
    const int up = q.qshift - k, dn = kc - q.qshift;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = ldexpf(fminf(fmaxf(rintf(ldexpf(v[j], up)), q.lo), q.hi), dn);
  } else {
    int code;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = mxint_element<DT>(v[j], state, k, kc, q, code);
  }
}

template <int DT>
__device__ __forceinline__ void load_vec8(const void* base, size_t elem, float* x) {
  using TR = DTypeTraits<DT>;
  const uint4* q = (const uint4*)((const char*)base + elem * TR::kBytes);
  if constexpr (TR::kVec == 4) {
    TR::unpack(q[0], x);
    TR::unpack(q[1], x + 4);
  } else {
    TR::unpack(q[0], x);
  }
}
template <int DT>
__device__ __forceinline__ void store_vec8(void* base, size_t elem, const float* y) {
  using TR = DTypeTraits<DT>;
  uint4* q = (uint4*)((char*)base + elem * TR::kBytes);
  if constexpr (TR::kVec == 4) {
    q[0] = TR::pack(y);
    q[1] = TR::pack(y + 4);
  } else {
    q[0] = TR::pack(y);
  }
}

template <int DT>
__device__ __forceinline__ void cast8(float* v, const CastSpec& c) {
  if (!c.on) return;
  float y[8];
  minifloat_mx_qdq8(v, y, c.m);
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = DTypeTraits<DT>::round(y[j]);
}

// WPR wavefronts per row (one work-group); the row stays in registers (NCH chunks of 64 lanes x 8 elements per
// wavefront, chunk c of wavefront w at element ((c * WPR + w) * 64 + lane) * 8).  Rows of more than 1536 elements are
// spread over 4 wavefronts: 16 or 32 elements per lane instead of 64 keep the register count low enough for 8
// wavefronts per SIMD, which is what hides the one load - compute - store round trip of each wavefront.  MX: the
// output is the MXINT quantize-dequantize of the normalised row (cols a multiple of 32).  The weight chunks are requested
// together with the row's, so that their latency passes during the reduction instead of after it.
template <int DT, int NCH, bool MX = false, int WPR = 1>
__global__ __launch_bounds__(kRowThreads * WPR) void rmsnorm_kernel(RmsNormParams p) {
  using TR = DTypeTraits<DT>;
  const int lane = (int)(threadIdx.x & 63);
  const int wave = (int)(threadIdx.x >> 6);
  const size_t row = blockIdx.x;
  const size_t base = row * (size_t)p.cols;
  WaveLog2 meta;
  if constexpr (MX) meta.init(p.mx.tab, 0);
  float h[NCH][8], wv[NCH][8];
  float ss = 0.0f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e0 = ((c * WPR + wave) * 64 + lane) * 8;
#pragma unroll
    for (int j = 0; j < 8; ++j) h[c][j] = 0.0f, wv[c][j] = 0.0f;
    if (e0 < p.cols) {
      load_vec8<DT>(p.x, base + (size_t)e0, h[c]);
      load_vec8<DT>(p.weight, (size_t)e0, wv[c]);
      if (p.residual != nullptr) {
        float res[8];
        load_vec8<DT>(p.residual, base + (size_t)e0, res);
#pragma unroll
        for (int j = 0; j < 8; ++j) h[c][j] = TR::round(h[c][j] + res[j]);
        store_vec8<DT>(p.sum_out, base + (size_t)e0, h[c]);
      }
      cast8<DT>(h[c], p.x_cast);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += h[c][j] * h[c][j];
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) ss += __shfl_xor(ss, o, 64);
  if constexpr (WPR > 1) {
    __shared__ float part[WPR];
    if (lane == 0) part[wave] = ss;
    __syncthreads();
    ss = 0.0f;
#pragma unroll
    for (int w = 0; w < WPR; ++w) ss += part[w];  // the same order in every wavefront
  }
  const float r = rsqrtf(ss / (float)p.cols + p.eps);
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e0 = ((c * WPR + wave) * 64 + lane) * 8;
    const bool live = e0 < p.cols;
    if constexpr (!MX) {
      if (!live) continue;
    }
    float y[8];
    if (live) cast8<DT>(wv[c], p.w_cast);
#pragma unroll
    for (int j = 0; j < 8; ++j) y[j] = wv[c][j] * TR::round(h[c][j] * r);  // weight * hidden.to(dtype), rounded by the store
    if constexpr (MX) {
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = TR::round(y[j]);
      mxint_block32<DT>(y, p.mx, meta);
    }
    if (live) store_vec8<DT>(p.out, base + (size_t)e0, y);
  }
}

template <int DT, bool MX, int WPR>
int launch_rmsnorm_wpr(const RmsNormParams& p, int nch, hipStream_t st) {
  const dim3 grid((unsigned)p.rows), block(kRowThreads * WPR);
  if (nch <= 1) hipLaunchKernelGGL((rmsnorm_kernel<DT, 1, MX, WPR>), grid, block, 0, st, p);
  else if (nch <= 2) hipLaunchKernelGGL((rmsnorm_kernel<DT, 2, MX, WPR>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((rmsnorm_kernel<DT, 4, MX, WPR>), grid, block, 0, st, p);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

template <int DT, bool MX = false>
int launch_rmsnorm(const RmsNormParams& p, hipStream_t st) {
  const int nch = (p.cols + 511) / 512;  // chunks of 64 lanes x 8 elements in a row (cols <= 8192: at most 16)
  if (nch <= 3) return launch_rmsnorm_wpr<DT, MX, 1>(p, nch, st);
  return launch_rmsnorm_wpr<DT, MX, 4>(p, (nch + 3) / 4, st);
}

struct SiluMulParams {
  const void* gate;
  const void* up;
  void* out;
  size_t n8;
  CastSpec cast;
  MxintParams mx;  // MX instantiation only
};

// silu(x) = x / (1 + exp(-x)) evaluated in fp32
__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + expf(-x)); }

// MX: the output is the MXINT quantize-dequantize of the product (blocks of 32 consecutive elements: numel a multiple
// of 32, so the 4 lanes of a block are live or dead together)
template <int DT, bool MX = false>
__global__ __launch_bounds__(kRowThreads) void silu_mul_kernel(SiluMulParams p) {
  using TR = DTypeTraits<DT>;
  const size_t i = (size_t)blockIdx.x * kRowThreads + threadIdx.x;
  const bool live = i < p.n8;
  if constexpr (!MX) {
    if (!live) return;
  }
  WaveLog2 meta;
  if constexpr (MX) meta.init(p.mx.tab, 0);
  float g[8], u[8], y[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) g[j] = u[j] = 0.0f;
  if (live) {
    load_vec8<DT>(p.gate, i * 8, g);
    load_vec8<DT>(p.up, i * 8, u);
    cast8<DT>(g, p.cast);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) y[j] = TR::round(silu_f32(g[j])) * u[j];
  if constexpr (MX) {
#pragma unroll
    for (int j = 0; j < 8; ++j) y[j] = TR::round(y[j]);
    mxint_block32<DT>(y, p.mx, meta);
  }
  if (live) store_vec8<DT>(p.out, i * 8, y);
}

// silu(gate) * up for 16-bit tensors with silu read from a table.  R(silu(g)) is a function of the 16 bits of g alone,
// and evaluating it (an exponential and a division per element) costs the kernel above a third of its time; here the
// table of all 65536 results (filled once per dtype by silu_table_kernel with the very expression the kernel above
// evaluates, so the results are the same bit for bit) sits in LDS, 128 KB, one work-group of 16 wavefronts per CU,
// each walking the tensor with the stride of the grid.
constexpr int kLutThreads = 1024;

template <int DT>
__global__ __launch_bounds__(256) void silu_table_kernel(uint16_t* __restrict__ table) {
  using TR = DTypeTraits<DT>;
  static_assert(DT != MASE_DT_F32, "a table over the 16 bits of a value");
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;  // the grid covers exactly 65536 patterns
  float v[8], y[8];
  TR::unpack(make_uint4(i, 0u, 0u, 0u), v);  // element 0: the low half of the first dword
#pragma unroll
  for (int j = 0; j < 8; ++j) y[j] = TR::round(silu_f32(v[j]));
  table[i] = (uint16_t)(TR::pack(y).x & 0xFFFFu);
}

struct SiluLutParams {
  const uint4* gate;
  const uint4* up;
  uint4* out;
  size_t n8;
  const uint4* table;   // 65536 x 16 bits
  MxintParams mx;
};

template <int DT>
__global__ __launch_bounds__(kLutThreads) void silu_mul_lut_kernel(SiluLutParams p) {
  using TR = DTypeTraits<DT>;
  extern __shared__ __attribute__((aligned(16))) uint16_t lut[];
  for (int i = threadIdx.x; i < 65536 * 2 / 16; i += kLutThreads) ((uint4*)lut)[i] = p.table[i];
  WaveLog2 meta;
  meta.init(p.mx.tab, 0);
  __syncthreads();
  const size_t stride = (size_t)gridDim.x * kLutThreads;
  // the loop bound is the same for all lanes of a wavefront: every lane takes part in the block maximum
  for (size_t base = (size_t)blockIdx.x * kLutThreads + (threadIdx.x & ~63u); base < p.n8; base += stride) {
    const size_t i = base + (threadIdx.x & 63u);
    const bool live = i < p.n8;
    uint4 gq = make_uint4(0, 0, 0, 0), uq = make_uint4(0, 0, 0, 0);
    if (live) {
      gq = load_nt(p.gate + i);
      uq = load_nt(p.up + i);
    }
    const uint32_t gw[4] = {gq.x, gq.y, gq.z, gq.w};
    uint32_t sw[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) sw[j] = (uint32_t)lut[gw[j] & 0xFFFFu] | ((uint32_t)lut[gw[j] >> 16] << 16);
    float s[8], u[8], y[8];
    TR::unpack(make_uint4(sw[0], sw[1], sw[2], sw[3]), s);
    TR::unpack(uq, u);
#pragma unroll
    for (int j = 0; j < 8; ++j) y[j] = TR::round(s[j] * u[j]);
    mxint_block32<DT>(y, p.mx, meta);
    if (live) store_nt(p.out + i, TR::pack(y));
  }
}

struct RopeParams {
  const void* x;
  const void* cos;
  const void* sin;
  void* out;
  int B, H, T, D;                 // D: head_dim, a multiple of 16 (two halves of whole 16-byte vectors)
  size_t xs_b, xs_h, xs_t;        // element strides of x and out (last dimension contiguous)
  size_t cs_b, cs_t;              // element strides of the cos / sin tables [B or 1, T, D]
};

// out = R(R(x * cos) + R(rotate_half(x) * sin)), rotate_half(x) = cat(-x[D/2:], x[:D/2]); each lane takes 8 elements
// of the lower half of one (b, h, t) row and the 8 elements half a row away, which are each other's partners, so
// every element is read once.  Grid: x over the (head, vector) pairs of one token (heads of a token lie next to each
// other in a projection's output), y and z the token (b * T + t = z * 32768 + y: uniform per work-group, so the
// divisions by T are scalar).
template <int DT>
__global__ __launch_bounds__(256) void rope_kernel(RopeParams p) {
  using TR = DTypeTraits<DT>;
  const uint32_t half_vecs = (uint32_t)p.D / 16;  // 8-element vectors in half a row
  const uint32_t hv = blockIdx.x * 256u + threadIdx.x;
  if (hv >= (uint32_t)p.H * half_vecs) return;
  const uint32_t token = blockIdx.z * 32768u + blockIdx.y;
  if (token >= (uint32_t)p.B * (uint32_t)p.T) return;
  const uint32_t b = token / (uint32_t)p.T, t = token - b * (uint32_t)p.T;
  const uint32_t h = hv / half_vecs, v = hv - h * half_vecs;
  const size_t row = (size_t)b * p.xs_b + (size_t)h * p.xs_h + (size_t)t * p.xs_t;
  const size_t crow = (size_t)b * p.cs_b + (size_t)t * p.cs_t;
  const int d0 = (int)v * 8, half = p.D / 2;
  float xl[8], xh[8], cl[8], ch[8], sl[8], sh[8], yl[8], yh[8];
  load_vec8<DT>(p.x, row + d0, xl);
  load_vec8<DT>(p.x, row + d0 + half, xh);
  load_vec8<DT>(p.cos, crow + d0, cl);
  load_vec8<DT>(p.cos, crow + d0 + half, ch);
  load_vec8<DT>(p.sin, crow + d0, sl);
  load_vec8<DT>(p.sin, crow + d0 + half, sh);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    yl[j] = TR::round(xl[j] * cl[j]) + TR::round(-xh[j] * sl[j]);
    yh[j] = TR::round(xh[j] * ch[j]) + TR::round(xl[j] * sh[j]);
  }
  store_vec8<DT>(p.out, row + d0, yl);
  store_vec8<DT>(p.out, row + d0 + half, yh);
}

bool fill_cast(CastSpec& c, int exp_bits, int frac_bits, int is_finite, int round_mode) {
  c.on = exp_bits > 0;
  if (!c.on) return true;
  if (frac_bits <= 0 || exp_bits > 8 || exp_bits + frac_bits >= 16 || round_mode < 0 || round_mode > 3) return false;
  c.m.E = exp_bits;
  c.m.F = frac_bits;
  c.m.bias = (1 << (exp_bits - 1)) - 1;
  c.m.e_hi = is_finite ? (1 << exp_bits) - 1 : (1 << exp_bits) - 2;
  c.m.frac_hi = (1 << frac_bits) - 1;
  c.m.is_finite = is_finite;
  c.m.round_mode = round_mode;
  return true;
}

}  // namespace
}  // namespace mase

extern "C" int mase_rmsnorm_minifloat(const void* x, const void* weight, void* out, size_t rows, size_t cols, int dtype,
                                      float eps, int x_exp_bits, int x_frac_bits, int x_is_finite, int x_round_mode,
                                      int w_exp_bits, int w_frac_bits, int w_is_finite, int w_round_mode, void* stream) {
  using namespace mase;
  if (rows == 0 || cols == 0) return MASE_OK;
  if (x == nullptr || weight == nullptr || out == nullptr) return MASE_ERR_NULL;
  if (cols % 8 != 0 || cols > 8192 || rows > 0x7FFFFFFFull) return MASE_ERR_SHAPE;
  if (!aligned16(x) || !aligned16(weight) || !aligned16(out)) return MASE_ERR_ALIGN;
  if (dtype < 0 || dtype > 2) return MASE_ERR_DTYPE;
  RmsNormParams p{};
  p.x = x;
  p.weight = weight;
  p.out = out;
  p.rows = rows;
  p.cols = (int)cols;
  p.eps = eps;
  if (!fill_cast(p.x_cast, x_exp_bits, x_frac_bits, x_is_finite, x_round_mode) ||
      !fill_cast(p.w_cast, w_exp_bits, w_frac_bits, w_is_finite, w_round_mode))
    return MASE_ERR_PARAM;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case MASE_DT_F32: return launch_rmsnorm<MASE_DT_F32>(p, st);
    case MASE_DT_BF16: return launch_rmsnorm<MASE_DT_BF16>(p, st);
    default: return launch_rmsnorm<MASE_DT_F16>(p, st);
  }
}

extern "C" int mase_silu_mul_minifloat(const void* gate, const void* up, void* out, size_t numel, int dtype, int exp_bits,
                                       int frac_bits, int is_finite, int round_mode, void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (gate == nullptr || up == nullptr || out == nullptr) return MASE_ERR_NULL;
  if (numel % 8 != 0) return MASE_ERR_SHAPE;
  if (!aligned16(gate) || !aligned16(up) || !aligned16(out)) return MASE_ERR_ALIGN;
  if (dtype < 0 || dtype > 2) return MASE_ERR_DTYPE;
  SiluMulParams p{};
  p.gate = gate;
  p.up = up;
  p.out = out;
  p.n8 = numel / 8;
  if (!fill_cast(p.cast, exp_bits, frac_bits, is_finite, round_mode)) return MASE_ERR_PARAM;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(blocks_for(p.n8, (size_t)kRowThreads)), block(kRowThreads);
  switch (dtype) {
    case MASE_DT_F32: hipLaunchKernelGGL((silu_mul_kernel<MASE_DT_F32>), grid, block, 0, st, p); break;
    case MASE_DT_BF16: hipLaunchKernelGGL((silu_mul_kernel<MASE_DT_BF16>), grid, block, 0, st, p); break;
    default: hipLaunchKernelGGL((silu_mul_kernel<MASE_DT_F16>), grid, block, 0, st, p); break;
  }
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

namespace mase {
namespace {
bool fill_mxint(MxintParams& q, int element_bits, int dtype, const uint32_t* tab) {
  if (element_bits < 2 || element_bits > 24 || tab == nullptr) return false;
  q.qshift = element_bits - 1;
  q.bias = 127;
  q.scale_max = 255;
  q.lo = mase_round_scalar_to_dtype(-(double)(1 << (element_bits - 1)), dtype);
  q.hi = mase_round_scalar_to_dtype((double)((1 << (element_bits - 1)) - 1), dtype);
  q.tab = tab;
  return true;
}
}  // namespace
}  // namespace mase

extern "C" int mase_rmsnorm_mxint(const void* x, const void* weight, void* out, size_t rows, size_t cols, int dtype,
                                  float eps, int element_bits, const uint32_t* log2_tab, void* stream) {
  using namespace mase;
  if (rows == 0 || cols == 0) return MASE_OK;
  if (x == nullptr || weight == nullptr || out == nullptr || log2_tab == nullptr) return MASE_ERR_NULL;
  if (cols % 32 != 0 || cols > 8192 || rows > 0x7FFFFFFFull) return MASE_ERR_SHAPE;
  if (!aligned16(x) || !aligned16(weight) || !aligned16(out)) return MASE_ERR_ALIGN;
  if (dtype < 0 || dtype > 2) return MASE_ERR_DTYPE;
  RmsNormParams p{};
  p.x = x;
  p.weight = weight;
  p.out = out;
  p.rows = rows;
  p.cols = (int)cols;
  p.eps = eps;
  if (!fill_mxint(p.mx, element_bits, dtype, log2_tab)) return MASE_ERR_PARAM;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case MASE_DT_F32: return launch_rmsnorm<MASE_DT_F32, true>(p, st);
    case MASE_DT_BF16: return launch_rmsnorm<MASE_DT_BF16, true>(p, st);
    default: return launch_rmsnorm<MASE_DT_F16, true>(p, st);
  }
}

extern "C" int mase_add_rmsnorm_mxint(const void* x, const void* residual, const void* weight, void* sum_out, void* out,
                                      size_t rows, size_t cols, int dtype, float eps, int element_bits,
                                      const uint32_t* log2_tab, void* stream) {
  using namespace mase;
  if (rows == 0 || cols == 0) return MASE_OK;
  if (x == nullptr || residual == nullptr || weight == nullptr || sum_out == nullptr || out == nullptr || log2_tab == nullptr)
    return MASE_ERR_NULL;
  if (cols % 32 != 0 || cols > 8192 || rows > 0x7FFFFFFFull) return MASE_ERR_SHAPE;
  if (!aligned16(x) || !aligned16(residual) || !aligned16(weight) || !aligned16(sum_out) || !aligned16(out)) return MASE_ERR_ALIGN;
  if (dtype < 0 || dtype > 2) return MASE_ERR_DTYPE;
  RmsNormParams p{};
  p.x = x;
  p.residual = residual;
  p.sum_out = sum_out;
  p.weight = weight;
  p.out = out;
  p.rows = rows;
  p.cols = (int)cols;
  p.eps = eps;
  if (!fill_mxint(p.mx, element_bits, dtype, log2_tab)) return MASE_ERR_PARAM;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case MASE_DT_F32: return launch_rmsnorm<MASE_DT_F32, true>(p, st);
    case MASE_DT_BF16: return launch_rmsnorm<MASE_DT_BF16, true>(p, st);
    default: return launch_rmsnorm<MASE_DT_F16, true>(p, st);
  }
}

extern "C" int mase_silu_mul_mxint(const void* gate, const void* up, void* out, size_t numel, int dtype,
                                   int element_bits, const uint32_t* log2_tab, void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (gate == nullptr || up == nullptr || out == nullptr || log2_tab == nullptr) return MASE_ERR_NULL;
  if (numel % 32 != 0) return MASE_ERR_SHAPE;
  if (!aligned16(gate) || !aligned16(up) || !aligned16(out)) return MASE_ERR_ALIGN;
  if (dtype < 0 || dtype > 2) return MASE_ERR_DTYPE;
  SiluMulParams p{};
  p.gate = gate;
  p.up = up;
  p.out = out;
  p.n8 = numel / 8;
  if (!fill_mxint(p.mx, element_bits, dtype, log2_tab)) return MASE_ERR_PARAM;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(blocks_for(p.n8, (size_t)kRowThreads)), block(kRowThreads);
  switch (dtype) {
    case MASE_DT_F32: hipLaunchKernelGGL((silu_mul_kernel<MASE_DT_F32, true>), grid, block, 0, st, p); break;
    case MASE_DT_BF16: hipLaunchKernelGGL((silu_mul_kernel<MASE_DT_BF16, true>), grid, block, 0, st, p); break;
    default: hipLaunchKernelGGL((silu_mul_kernel<MASE_DT_F16, true>), grid, block, 0, st, p); break;
  }
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

extern "C" int mase_silu_table(void* table, int dtype, void* stream) {
  using namespace mase;
  if (table == nullptr) return MASE_ERR_NULL;
  if (!aligned16(table)) return MASE_ERR_ALIGN;
  if (dtype != MASE_DT_BF16 && dtype != MASE_DT_F16) return MASE_ERR_DTYPE;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MASE_DT_BF16) hipLaunchKernelGGL((silu_table_kernel<MASE_DT_BF16>), dim3(256), dim3(256), 0, st, (uint16_t*)table);
  else hipLaunchKernelGGL((silu_table_kernel<MASE_DT_F16>), dim3(256), dim3(256), 0, st, (uint16_t*)table);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

extern "C" int mase_silu_mul_mxint_lut(const void* gate, const void* up, void* out, size_t numel, int dtype,
                                       int element_bits, const uint32_t* log2_tab, const void* silu_table, void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (gate == nullptr || up == nullptr || out == nullptr || log2_tab == nullptr || silu_table == nullptr) return MASE_ERR_NULL;
  if (numel % 32 != 0) return MASE_ERR_SHAPE;
  if (!aligned16(gate) || !aligned16(up) || !aligned16(out) || !aligned16(silu_table)) return MASE_ERR_ALIGN;
  if (dtype != MASE_DT_BF16 && dtype != MASE_DT_F16) return MASE_ERR_DTYPE;
  SiluLutParams p{};
  p.gate = (const uint4*)gate;
  p.up = (const uint4*)up;
  p.out = (uint4*)out;
  p.n8 = numel / 8;
  p.table = (const uint4*)silu_table;
  if (!fill_mxint(p.mx, element_bits, dtype, log2_tab)) return MASE_ERR_PARAM;
  const int n_cu = device_cu_count();
  if (n_cu <= 0) return MASE_ERR_LAUNCH;
  constexpr int kLutBytes = 65536 * 2;
  static std::atomic<uint64_t> attr_done{0};
  if (!device_setup_done(attr_done)) {
    if (hipFuncSetAttribute((const void*)silu_mul_lut_kernel<MASE_DT_BF16>, hipFuncAttributeMaxDynamicSharedMemorySize, kLutBytes) != hipSuccess ||
        hipFuncSetAttribute((const void*)silu_mul_lut_kernel<MASE_DT_F16>, hipFuncAttributeMaxDynamicSharedMemorySize, kLutBytes) != hipSuccess)
      return MASE_ERR_LAUNCH;
    mark_device_setup_done(attr_done);
  }
  const size_t wgs_needed = blocks_for(p.n8, (size_t)kLutThreads);
  const dim3 grid((unsigned)(wgs_needed < (size_t)n_cu ? wgs_needed : (size_t)n_cu)), block(kLutThreads);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MASE_DT_BF16) hipLaunchKernelGGL((silu_mul_lut_kernel<MASE_DT_BF16>), grid, block, kLutBytes, st, p);
  else hipLaunchKernelGGL((silu_mul_lut_kernel<MASE_DT_F16>), grid, block, kLutBytes, st, p);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

extern "C" int mase_rope(const void* x, const void* cos, const void* sin, void* out, size_t B, size_t H, size_t T, size_t D,
                         size_t x_stride_b, size_t x_stride_h, size_t x_stride_t, size_t cs_stride_b, size_t cs_stride_t,
                         int dtype, void* stream) {
  using namespace mase;
  if (B == 0 || H == 0 || T == 0 || D == 0) return MASE_OK;
  if (x == nullptr || cos == nullptr || sin == nullptr || out == nullptr) return MASE_ERR_NULL;
  if (D % 16 != 0 || D > 4096 || B * H * T > 0x7FFFFFFFull || B * T > 65535ull * 32768ull) return MASE_ERR_SHAPE;
  if ((x_stride_b | x_stride_h | x_stride_t | cs_stride_b | cs_stride_t) % 8 != 0) return MASE_ERR_SHAPE;
  if (!aligned16(x) || !aligned16(cos) || !aligned16(sin) || !aligned16(out)) return MASE_ERR_ALIGN;
  if (dtype < 0 || dtype > 2) return MASE_ERR_DTYPE;
  RopeParams p{};
  p.x = x;
  p.cos = cos;
  p.sin = sin;
  p.out = out;
  p.B = (int)B;
  p.H = (int)H;
  p.T = (int)T;
  p.D = (int)D;
  p.xs_b = x_stride_b;
  p.xs_h = x_stride_h;
  p.xs_t = x_stride_t;
  p.cs_b = cs_stride_b;
  p.cs_t = cs_stride_t;
  hipStream_t st = (hipStream_t)stream;
  const size_t tokens = B * T;  // < 2^31 (checked above)
  const dim3 grid(blocks_for(H * (D / 16), (size_t)256), (unsigned)(tokens < 32768 ? tokens : 32768),
                  (unsigned)((tokens + 32767) / 32768)), block(256);
  switch (dtype) {
    case MASE_DT_F32: hipLaunchKernelGGL((rope_kernel<MASE_DT_F32>), grid, block, 0, st, p); break;
    case MASE_DT_BF16: hipLaunchKernelGGL((rope_kernel<MASE_DT_BF16>), grid, block, 0, st, p); break;
    default: hipLaunchKernelGGL((rope_kernel<MASE_DT_F16>), grid, block, 0, st, p); break;
  }
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}
