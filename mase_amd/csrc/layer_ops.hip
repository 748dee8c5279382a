// Row-wise and element-wise layers around the quantized Linears of a Llama block, each in one pass (gfx950):
//   RMSNorm with optional minifloat casts of the input and of the weight (nn/quantized/modules/llama/rms_norm.py:72-84;
//   with both casts off: the plain RMSNorm, models/llama/modeling_llama.py:79-93)
//   SiLU(cast(gate)) * up (nn/quantized/modules/llama/mlp.py:60-62 with functional/silu.py:41-57; cast off: the plain
//   SwiGLU product, models/llama/modeling_llama.py:219-236)
// Every intermediate is rounded to the tensor dtype T where the separate tensor operations would round it.  Both are
// HBM-bound: the tensor is read once and written once, against 10-20 passes of the separate operations.
#include "common.hpp"
#include "minifloat_mx.hpp"

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
  size_t rows;
  int cols;  // multiple of 8, at most 8192
  float eps;
  CastSpec x_cast, w_cast;
};

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

// one wavefront per row; the row stays in registers (NCH chunks of 64 lanes x 8 elements)
template <int DT, int NCH>
__global__ __launch_bounds__(kRowThreads) void rmsnorm_kernel(RmsNormParams p) {
  using TR = DTypeTraits<DT>;
  const int lane = (int)(threadIdx.x & 63);
  const size_t row = blockIdx.x;
  const size_t base = row * (size_t)p.cols;
  float h[NCH][8];
  float ss = 0.0f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e0 = (c * 64 + lane) * 8;
#pragma unroll
    for (int j = 0; j < 8; ++j) h[c][j] = 0.0f;
    if (e0 < p.cols) {
      load_vec8<DT>(p.x, base + (size_t)e0, h[c]);
      cast8<DT>(h[c], p.x_cast);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += h[c][j] * h[c][j];
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) ss += __shfl_xor(ss, o, 64);
  const float r = rsqrtf(ss / (float)p.cols + p.eps);
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e0 = (c * 64 + lane) * 8;
    if (e0 >= p.cols) continue;
    float w[8], y[8];
    load_vec8<DT>(p.weight, (size_t)e0, w);
    cast8<DT>(w, p.w_cast);
#pragma unroll
    for (int j = 0; j < 8; ++j) y[j] = w[j] * TR::round(h[c][j] * r);  // weight * hidden.to(dtype), rounded by the store
    store_vec8<DT>(p.out, base + (size_t)e0, y);
  }
}

template <int DT>
int launch_rmsnorm(const RmsNormParams& p, hipStream_t st) {
  const int nch = (p.cols + 511) / 512;
  const dim3 grid((unsigned)p.rows), block(kRowThreads);
  if (nch <= 1) hipLaunchKernelGGL((rmsnorm_kernel<DT, 1>), grid, block, 0, st, p);
  else if (nch <= 2) hipLaunchKernelGGL((rmsnorm_kernel<DT, 2>), grid, block, 0, st, p);
  else if (nch <= 4) hipLaunchKernelGGL((rmsnorm_kernel<DT, 4>), grid, block, 0, st, p);
  else if (nch <= 8) hipLaunchKernelGGL((rmsnorm_kernel<DT, 8>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((rmsnorm_kernel<DT, 16>), grid, block, 0, st, p);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

struct SiluMulParams {
  const void* gate;
  const void* up;
  void* out;
  size_t n8;
  CastSpec cast;
};

// silu(x) = x / (1 + exp(-x)) evaluated in fp32
__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + expf(-x)); }

template <int DT>
__global__ __launch_bounds__(kRowThreads) void silu_mul_kernel(SiluMulParams p) {
  using TR = DTypeTraits<DT>;
  const size_t i = (size_t)blockIdx.x * kRowThreads + threadIdx.x;
  if (i >= p.n8) return;
  float g[8], u[8], y[8];
  load_vec8<DT>(p.gate, i * 8, g);
  load_vec8<DT>(p.up, i * 8, u);
  cast8<DT>(g, p.cast);
#pragma unroll
  for (int j = 0; j < 8; ++j) y[j] = TR::round(silu_f32(g[j])) * u[j];
  store_vec8<DT>(p.out, i * 8, y);
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
