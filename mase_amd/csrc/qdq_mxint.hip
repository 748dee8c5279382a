// MXINT quantize-dequantize (and optional packing) for gfx950.
//
// Reference arithmetic (nn/quantizers/mxint/fake.py:11-80), per block of B consecutive elements, b =
// element_bits, s = scale_bits, bias = 2^(s-1)-1, all in the tensor dtype T:
//   mx  = max(max|x|, tiny(T));  k = ceil(log2(mx)) as the library rounds it in T
//   m_i = clamp(rne(x_i / 2^k * 2^(b-1)), -2^(b-1), 2^(b-1)-1)        (bounds cast to T)
//   kc  = clamp(k + bias, 0, 2^s-1) - bias
//   y_i = m_i / 2^(b-1) * 2^kc
// Scaling by powers of two is exact in fp32 registers; the only roundings are rne() and the final
// conversion to T (which matters only for subnormal results).  x_i/2^k can be inexact only when it is
// subnormal, and then m_i is 0 either way.  When 2^k overflows T (or the maximum is Inf) the reference
// computes x/inf = +-0 and then +-0 * 2^kc, which is NaN when 2^kc is inf as well and +-0 otherwise; a NaN
// maximum makes the whole block NaN.  The same cases are reproduced here.
//
// Bandwidth-bound: one 16-byte load and one 16-byte store per lane, latency hidden by occupancy (few
// registers, many small work-groups), block maximum by DPP inside the wavefront, no LDS.
#include "common.hpp"
#include "mxint_core.hpp"

#ifndef MASE_RUN_THREADS
#define MASE_RUN_THREADS 64
#endif
#ifndef MASE_MXINT_NARROW_ITEMS
#define MASE_MXINT_NARROW_ITEMS 1
#endif

namespace mase {
namespace {

// work-group size of the vector kernel: small groups stream best on this part
constexpr int kRunThreads = MASE_RUN_THREADS;

// One 16-byte vector per lane.  LPB lanes share one block (B = LPB * kVec) or one lane holds SUB blocks
// (B = kVec / SUB).  For bf16 the dequantized value m * 2^(kc-b+1) has at most 8 significant bits (m is the
// rne of an 8-bit-significand input), so it is packed by truncation unless it would be subnormal.
// out-of-place store of V fp32 registers as DTO elements at vector index idx
template <int DTO, int V>
__device__ __forceinline__ void store_vec(void* out, size_t idx, const float* y, bool exact_bf16) {
  using TO = DTypeTraits<DTO>;
  if constexpr (DTO == MASE_DT_F32) {
    store_nt((uint4*)out + idx * (V / 4), TO::pack(y));
    if constexpr (V == 8) store_nt((uint4*)out + idx * 2 + 1, TO::pack(y + 4));
  } else if constexpr (V == 8) {
    if (DTO == MASE_DT_BF16 && exact_bf16) {
      uint4 o;
      o.x = pack_bf16_exact(y[0], y[1]);
      o.y = pack_bf16_exact(y[2], y[3]);
      o.z = pack_bf16_exact(y[4], y[5]);
      o.w = pack_bf16_exact(y[6], y[7]);
      store_nt((uint4*)out + idx, o);
    } else {
      store_nt((uint4*)out + idx, TO::pack(y));
    }
  } else {  // 4 sixteen-bit results: 8 bytes
    uint2 o;
    if constexpr (DTO == MASE_DT_BF16) {
      o.x = f32_to_bf16_bits(y[0]) | (f32_to_bf16_bits(y[1]) << 16);
      o.y = f32_to_bf16_bits(y[2]) | (f32_to_bf16_bits(y[3]) << 16);
    } else {
      o.x = f32_to_f16_bits(y[0]) | (f32_to_f16_bits(y[1]) << 16);
      o.y = f32_to_f16_bits(y[2]) | (f32_to_f16_bits(y[3]) << 16);
    }
    store_nt((uint2*)out + idx, o);
  }
}

// ITEMS vectors per lane, a work-group's width apart, all loaded before the first is worked on: a wavefront then has
// ITEMS KB in flight instead of one, which is what a latency-bound stream needs when the stores are narrower than the
// loads (fp32 in, 16-bit out).
template <int DT, int DTO, int LPB, int SUB, int T, int ITEMS>
__global__ __launch_bounds__(T) void mxint_qdq_vec_kernel(const uint4* __restrict__ in, void* __restrict__ out,
                                                          int8_t* __restrict__ codes, uint8_t* __restrict__ scales,
                                                          size_t n_vec, MxintParams p) {
  using TR = DTypeTraits<DT>;
  constexpr int V = TR::kVec;
  constexpr int EPS = V / SUB;  // elements per sub-block held by this lane
  const size_t idx0 = (size_t)blockIdx.x * (T * ITEMS) + threadIdx.x;
  uint4 raws[ITEMS];
#pragma unroll
  for (int u = 0; u < ITEMS; ++u) {
    const size_t i = idx0 + (size_t)u * T;
    raws[u] = i < n_vec ? load_nt(in + i) : make_uint4(0, 0, 0, 0);
  }
  WaveLog2 meta;
  meta.init(p.tab, 0);
#pragma unroll
  for (int u = 0; u < ITEMS; ++u) {
    const size_t idx = idx0 + (size_t)u * T;
    const bool live = idx < n_vec;  // whole blocks are live or dead together: n_vec is a multiple of LPB
    const uint4 raw = raws[u];
    float x[V], y[V];
    int c[V];
    TR::unpack(raw, x);
    bool exact_bf16 = (DT == MASE_DT_BF16);  // 8-bit-significand inputs: results need no rounding to bf16
#pragma unroll
    for (int s = 0; s < SUB; ++s) {
      uint32_t m;
      if constexpr (SUB == 1) {
        m = group_max_u32<LPB>(vec_absmax_bits<DT>(raw));
      } else {
        m = 0;
#pragma unroll
        for (int j = 0; j < EPS; ++j) m = max(m, f2bits(x[s * EPS + j]) & 0x7FFFFFFFu);
      }
      int k = 0, kc = 0;
      const int state = block_exponent<DT>(m, p, k, kc, meta);
      if (state == 0) {
        const int up = p.qshift - k, dn = kc - p.qshift;
        exact_bf16 = exact_bf16 && (dn >= -126);
#pragma unroll
        for (int j = 0; j < EPS; ++j) {
          float r = fminf(fmaxf(rintf(ldexpf(x[s * EPS + j], up)), p.lo), p.hi);
          c[s * EPS + j] = (int)r;
          y[s * EPS + j] = ldexpf(r, dn);
        }
      } else {
#pragma unroll
        for (int j = 0; j < EPS; ++j) y[s * EPS + j] = mxint_element<DT>(x[s * EPS + j], state, k, kc, p, c[s * EPS + j]);
      }
      if (codes != nullptr && live) {
        int sb = (state == 0) ? min(max(kc - p.qshift + 134, 0), 255) : 255;
        if constexpr (LPB > 1) {
          if ((idx & (LPB - 1)) == 0) scales[idx / LPB] = (uint8_t)sb;
        } else {
          scales[idx * SUB + s] = (uint8_t)sb;
        }
      }
    }
    if (!live) continue;
    store_vec<DTO, V>(out, idx, y, exact_bf16);
    if (codes != nullptr) {
      if constexpr (V == 4) {
        ((uint32_t*)codes)[idx] = (uint32_t)(c[0] & 0xFF) | ((uint32_t)(c[1] & 0xFF) << 8) | ((uint32_t)(c[2] & 0xFF) << 16) |
                                  ((uint32_t)(c[3] & 0xFF) << 24);
      } else {
        uint2 w;
        w.x = (uint32_t)(c[0] & 0xFF) | ((uint32_t)(c[1] & 0xFF) << 8) | ((uint32_t)(c[2] & 0xFF) << 16) |
              ((uint32_t)(c[3] & 0xFF) << 24);
        w.y = (uint32_t)(c[4] & 0xFF) | ((uint32_t)(c[5] & 0xFF) << 8) | ((uint32_t)(c[6] & 0xFF) << 16) |
              ((uint32_t)(c[7] & 0xFF) << 24);
        ((uint2*)codes)[idx] = w;
      }
    }
  }
}

// Any block size / alignment: one work-item per block, two passes over its elements.
template <int DT, int DTO>
__global__ __launch_bounds__(kThreads) void mxint_qdq_generic_kernel(const void* __restrict__ in, void* __restrict__ out,
                                                                     int8_t* __restrict__ codes,
                                                                     uint8_t* __restrict__ scales, size_t n_blocks,
                                                                     int B, MxintParams p) {
  using TR = DTypeTraits<DT>;
  size_t blk = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (blk >= n_blocks) return;
  size_t off = blk * (size_t)B;
  uint32_t m = 0;
  for (int j = 0; j < B; ++j) m = max(m, f2bits(TR::load1(in, off + j)) & 0x7FFFFFFFu);
  int k = 0, kc = 0;
  int state = block_exponent<DT>(m, p, k, kc);
  for (int j = 0; j < B; ++j) {
    int code;
    DTypeTraits<DTO>::store1(out, off + j, mxint_element<DT>(TR::load1(in, off + j), state, k, kc, p, code));
    if (codes != nullptr) codes[off + j] = (int8_t)code;
  }
  if (codes != nullptr) scales[blk] = (uint8_t)((state == 0) ? min(max(kc - p.qshift + 134, 0), 255) : 255);
}

template <int DT, int DTO>
int launch_mxint(const void* in, void* out, int8_t* codes, uint8_t* scales, size_t numel, int B, const MxintParams& p,
                 hipStream_t st) {
  using TR = DTypeTraits<DT>;
  constexpr int V = TR::kVec;
  const bool pow2 = (B & (B - 1)) == 0;
  const bool vec_ok = pow2 && B <= 64 * V && (numel % V) == 0 && aligned16(in) && aligned16(out) &&
                      (codes == nullptr || (((uintptr_t)codes) & 7u) == 0);
  if (vec_ok) {
    size_t n_vec = numel / V;
    // more than one vector per lane was measured slower for every dtype pair of this kernel (fp32 -> bf16 on 4096^2: 17.6, 18.5, 19.6 us with 1, 2, 4)
    constexpr int kItems = (DT == MASE_DT_F32 && DTO != MASE_DT_F32) ? MASE_MXINT_NARROW_ITEMS : 1;
    dim3 grid(blocks_for(n_vec, (size_t)kRunThreads * kItems)), block(kRunThreads);
#define MASE_MXINT_CASE(LPB_, SUB_)                                                                               \
  hipLaunchKernelGGL((mxint_qdq_vec_kernel<DT, DTO, LPB_, SUB_, kRunThreads, kItems>), grid, block, 0, st,         \
                     (const uint4*)in, out, codes, scales, n_vec, p)
    if (B >= V) {
      switch (B / V) {
        case 1: MASE_MXINT_CASE(1, 1); break;
        case 2: MASE_MXINT_CASE(2, 1); break;
        case 4: MASE_MXINT_CASE(4, 1); break;
        case 8: MASE_MXINT_CASE(8, 1); break;
        case 16: MASE_MXINT_CASE(16, 1); break;
        case 32: MASE_MXINT_CASE(32, 1); break;
        default: MASE_MXINT_CASE(64, 1); break;
      }
    } else {
      switch (V / B) {
        case 2: MASE_MXINT_CASE(1, 2); break;
        case 4: MASE_MXINT_CASE(1, 4); break;
        default:
          if constexpr (V == 8) MASE_MXINT_CASE(1, 8);
          break;
      }
    }
#undef MASE_MXINT_CASE
  } else {
    size_t n_blocks = numel / (size_t)B;
    hipLaunchKernelGGL((mxint_qdq_generic_kernel<DT, DTO>), dim3(blocks_for(n_blocks, kThreads)), dim3(kThreads), 0, st, in,
                       out, codes, scales, n_blocks, B, p);
  }
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

}  // namespace
}  // namespace mase

namespace mase {
namespace {
template <int DT>
int launch_mxint_out(int out_dtype, const void* in, void* out, int8_t* codes, uint8_t* scales, size_t numel, int B,
                     const MxintParams& p, hipStream_t st) {
  switch (out_dtype) {
    case MASE_DT_F32: return launch_mxint<DT, MASE_DT_F32>(in, out, codes, scales, numel, B, p, st);
    case MASE_DT_BF16: return launch_mxint<DT, MASE_DT_BF16>(in, out, codes, scales, numel, B, p, st);
    case MASE_DT_F16: return launch_mxint<DT, MASE_DT_F16>(in, out, codes, scales, numel, B, p, st);
    default: return MASE_ERR_DTYPE;
  }
}
}  // namespace
}  // namespace mase

extern "C" int mase_mxint_qdq(const void* in, void* out, int8_t* codes, uint8_t* scales, size_t numel, int dtype,
                              int out_dtype, int block_size, int element_bits, int scale_bits,
                              const uint32_t* log2_tab, void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (in == nullptr || out == nullptr || log2_tab == nullptr) return MASE_ERR_NULL;
  if ((codes == nullptr) != (scales == nullptr)) return MASE_ERR_NULL;
  if (block_size <= 0 || numel % (size_t)block_size != 0) return MASE_ERR_SHAPE;
  if (element_bits < 2 || element_bits > 24 || scale_bits < 1 || scale_bits > 8) return MASE_ERR_PARAM;
  if (codes != nullptr && element_bits > 8) return MASE_ERR_PARAM;
  if (dtype != MASE_DT_F32 && dtype != MASE_DT_BF16 && dtype != MASE_DT_F16) return MASE_ERR_DTYPE;
  if (out_dtype != MASE_DT_F32 && out_dtype != MASE_DT_BF16 && out_dtype != MASE_DT_F16) return MASE_ERR_DTYPE;
  MxintParams p;
  p.qshift = element_bits - 1;
  p.bias = (1 << (scale_bits - 1)) - 1;
  p.scale_max = (1 << scale_bits) - 1;
  p.lo = mase_round_scalar_to_dtype(-(double)(1 << (element_bits - 1)), dtype);
  p.hi = mase_round_scalar_to_dtype((double)((1 << (element_bits - 1)) - 1), dtype);
  p.tab = log2_tab;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case MASE_DT_F32: return launch_mxint_out<MASE_DT_F32>(out_dtype, in, out, codes, scales, numel, block_size, p, st);
    case MASE_DT_BF16: return launch_mxint_out<MASE_DT_BF16>(out_dtype, in, out, codes, scales, numel, block_size, p, st);
    default: return launch_mxint_out<MASE_DT_F16>(out_dtype, in, out, codes, scales, numel, block_size, p, st);
  }
}
