// MXFP quantize-dequantize (and optional packing) for gfx950.
//
// Reference arithmetic (nn/quantizers/mxfp/fake.py:12-104), always in fp32 whatever the tensor dtype, per
// block of B consecutive elements, element format (E, F) with el_emax = 2^E-1-bias_E (finite elements,
// round-to-nearest):
//   t_i  = x_i with fp32 subnormals flushed to +0
//   sh   = clamp(floor(log2(max|t|)) - el_emax, -127, 128)       (log2 as the library rounds it in fp32)
//   c_i  = minifloat_encode(t_i / 2^sh)                           (bit-level, see minifloat_mx.hpp)
//   y_i  = minifloat_decode(c_i) * 2^sh, converted to the output dtype;  scale byte = sh + 127
// An all-flushed block has scale byte 0 and decodes to +0.  A block holding Inf/NaN decodes to NaN in the
// reference (its int32 conversion of log2 wraps to the largest scale, 0 * inf), and does here.
#include "common.hpp"
#include "minifloat_mx.hpp"
#include "mxfp_core.hpp"
#include "pk16_cast.hpp"

namespace mase {
namespace {

constexpr int kVecThreads = 64;

// largest magnitude (fp32 bits) of the flushed elements of one 16-byte input vector
template <int DTI>
__device__ __forceinline__ uint32_t vec_flushed_absmax(const uint4& v) {
  const uint32_t m = vec_absmax_bits<DTI>(v);
  return ((m & 0x7F800000u) == 0) ? 0u : m;  // a subnormal maximum means every element is flushed
}

// One 16-byte vector of the wider side per lane, 64-lane work-groups (the shape that streams best on this
// part); a block of B elements spans LPB lanes, or a lane holds SUB blocks.  No lane leaves before the table
// lookups: they are wave-wide register permutes.
template <int DTI, int DTO, int LPB, int SUB, bool CODES>
__global__ __launch_bounds__(kVecThreads) void mxfp_qdq_vec_kernel(const void* __restrict__ in, void* __restrict__ out,
                                                                   uint8_t* __restrict__ codes,
                                                                   uint8_t* __restrict__ scales, size_t n_vec,
                                                                   MxfpParams p) {
  using TI = DTypeTraits<DTI>;
  using TO = DTypeTraits<DTO>;
  // work in units of 8 elements when either side is a 16-bit type, else 4
  constexpr int V = (TI::kVec == 8 || TO::kVec == 8) ? 8 : 4;
  constexpr int EPS = V / SUB;
  const size_t idx = (size_t)blockIdx.x * kVecThreads + threadIdx.x;
  const bool live = idx < n_vec;
  WaveLog2 meta;
  meta.init(p.tab, kLog2TabHalf);
  float x[V], y[V];
  uint32_t c[V];
  uint4 raw[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
  if (live) {
    if constexpr (TI::kVec == V) {
      raw[0] = load_nt((const uint4*)in + idx);
    } else {  // fp32 input, 8 per item
      raw[0] = load_nt((const uint4*)in + 2 * idx);
      raw[1] = load_nt((const uint4*)in + 2 * idx + 1);
    }
  }
  TI::unpack(raw[0], x);
  if constexpr (TI::kVec != V) TI::unpack(raw[1], x + 4);
#pragma unroll
  for (int s = 0; s < SUB; ++s) {
    uint32_t m = 0;
    if constexpr (SUB == 1) {  // the lane's whole item belongs to one block: packed maximum of the raw vector(s)
      m = vec_flushed_absmax<DTI>(raw[0]);
      if constexpr (TI::kVec != V) m = max(m, vec_flushed_absmax<DTI>(raw[1]));
    } else {
#pragma unroll
      for (int j = 0; j < EPS; ++j) m = max(m, f2bits(flush_subnormal(x[s * EPS + j])) & 0x7FFFFFFFu);
    }
    m = group_max_u32<LPB>(m);
    int sh = 0;
    const int state = mxfp_block_scale(m, p, sh, meta);
    if (p.m.E >= 4)  // uniform: wide-exponent formats
      mxfp_elements<false, EPS>(x + s * EPS, state, sh, p, c + s * EPS, y + s * EPS);
    else
      mxfp_elements<true, EPS>(x + s * EPS, state, sh, p, c + s * EPS, y + s * EPS);
    if (CODES && live) {
      int sb = (state == 1) ? sh + 127 : (state == 0 ? 0 : 255);
      if constexpr (LPB > 1) {
        if ((idx & (LPB - 1)) == 0) scales[idx / LPB] = (uint8_t)sb;
      } else {
        scales[idx * SUB + s] = (uint8_t)sb;
      }
    }
  }
  if (!live) return;
  if constexpr (TO::kVec == V) {
    store_nt((uint4*)out + idx, TO::pack(y));
  } else {
    store_nt((uint4*)out + 2 * idx, TO::pack(y));
    store_nt((uint4*)out + 2 * idx + 1, TO::pack(y + 4));
  }
  if constexpr (CODES) {
    if constexpr (V == 4) {
      ((uint32_t*)codes)[idx] = c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24);
    } else {
      uint2 w;
      w.x = c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24);
      w.y = c[4] | (c[5] << 8) | (c[6] << 16) | (c[7] << 24);
      ((uint2*)codes)[idx] = w;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// MXFP quantize-dequantize of a 16-bit tensor to the same dtype with the packed 16-bit cast (pk16_cast.hpp).
// Dividing an element by 2^sh, casting it and multiplying by 2^sh again is, in the element's own bit pattern, the
// cast with its thresholds moved up by sh exponent steps: the block's scale only changes per-lane constants (largest
// value, lowest ordinary pattern, parity of the code's exponent field), the elements are never rescaled.
// LPB lanes of 8 elements share a block.  SUBN handles the binade below the format's normal range in line (needed
// for the narrow-exponent formats, where it lies a few binades under the block maximum).  A lane redoes its elements
// with the fp32 form when its block is not regular (all flushed, non-finite) or when it holds an element outside the
// packed form's domain (subnormal in the tensor dtype or, without SUBN, below the format's normal range).
// ---------------------------------------------------------------------------------------------
struct MxfpPk16Params {
  Pk16Format f;
  int top0, bot0;     // exponent fields (in T) of the format's largest / smallest normal binade at scale 2^0
  uint32_t maxfrac;   // mantissa bits of the format's largest value
  int parity0;        // (format bias - T bias) & 1
};

constexpr int kPk16Items = 2;

template <int DT, int LPB, bool SUBN>
__global__ __launch_bounds__(kVecThreads) void mxfp_qdq_pk16_kernel(const uint4* __restrict__ in, uint4* __restrict__ out,
                                                                    size_t n_vec, MxfpParams p, MxfpPk16Params q) {
  using TR = DTypeTraits<DT>;
  constexpr int MB = (DT == MASE_DT_BF16) ? 7 : 10;
  WaveLog2 meta;
  meta.init(p.tab, kLog2TabHalf);
  // kPk16Items vectors per lane, a work-group's width apart, all loaded first (more bytes in flight per wavefront)
  const size_t idx0 = (size_t)blockIdx.x * (kVecThreads * kPk16Items) + threadIdx.x;
  uint4 raws[kPk16Items];
#pragma unroll
  for (int u = 0; u < kPk16Items; ++u) {
    const size_t idx = idx0 + (size_t)u * kVecThreads;
    raws[u] = idx < n_vec ? load_nt(in + idx) : make_uint4(0, 0, 0, 0);
  }
#pragma unroll
  for (int u = 0; u < kPk16Items; ++u) {
  const size_t idx = idx0 + (size_t)u * kVecThreads;
  const bool live = idx < n_vec;  // whole blocks are live or dead together: n_vec is a multiple of LPB
  const uint4 raw = raws[u];
  const uint32_t m = group_max_u32<LPB>(vec_flushed_absmax<DT>(raw));
  int sh = 0;
  const int state = mxfp_block_scale(m, p, sh, meta);
  // the cast's thresholds at this block's scale
  const uint32_t one = 0x00010001u;
  const int botf = q.bot0 + sh;
  Pk16Range r;
  r.odd_k2 = (((q.parity0 - sh) & 1) ? (1u << MB) : 0u) * one;
  r.max2 = (((uint32_t)min(max(q.top0 + sh, 1), 0xFF) << MB) | q.maxfrac) * one;
  const uint32_t lo_thr = (uint32_t)min(max(botf, 1), 0xFF) << MB;
  r.lo_thr2 = lo_thr * one;
  r.sub_thr2 = ((uint32_t)min(max(botf - 1, 1), 0xFF) << MB) * one;
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  uint32_t y[4];
  u16x2 lo_acc = as_u16x2(0xFFFFFFFFu), hi_acc = as_u16x2(0u);
#pragma unroll
  for (int j = 0; j < 4; ++j) y[j] = pk16_cast<MB, SUBN>(w[j], q.f, r, lo_acc, hi_acc);
  const uint32_t lo = min((uint32_t)lo_acc.x, (uint32_t)lo_acc.y);
  uint4 o = make_uint4(y[0], y[1], y[2], y[3]);
  // outside the packed form's domain: elements subnormal in T, elements whose quotient by 2^sh leaves the fp32 normal
  // range (bf16 shares fp32's exponent field: field <= sh; a quotient that underflows to zero loses its sign in the
  // reference) and, without SUBN, elements below the format's normal range
  uint32_t lowest = SUBN ? (1u << MB) : lo_thr;
  if constexpr (DT == MASE_DT_BF16) lowest = max(lowest, (uint32_t)min(max(sh + 1, 1), 0xFF) << MB);
  if (__builtin_expect(state != 1 || lo + 1u < lowest, 0)) {
    float x[8], z[8];
    uint32_t c[8];
    TR::unpack(raw, x);
    mxfp_elements<true, 8>(x, state, sh, p, c, z);  // the form that handles codes with exponent field 0 in line
    o = TR::pack(z);
  }
  if (live) store_nt(out + idx, o);
  }
}

template <int DTI, int DTO>
__global__ __launch_bounds__(kThreads) void mxfp_qdq_generic_kernel(const void* __restrict__ in, void* __restrict__ out,
                                                                    uint8_t* __restrict__ codes,
                                                                    uint8_t* __restrict__ scales, size_t n_blocks,
                                                                    int B, MxfpParams p) {
  size_t blk = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (blk >= n_blocks) return;
  size_t off = blk * (size_t)B;
  uint32_t m = 0;
  for (int j = 0; j < B; ++j) m = max(m, f2bits(flush_subnormal(DTypeTraits<DTI>::load1(in, off + j))) & 0x7FFFFFFFu);
  int sh = 0;
  int state = mxfp_block_scale(m, p, sh);
  for (int j = 0; j < B; ++j) {
    uint32_t c;
    float y = mxfp_element(flush_subnormal(DTypeTraits<DTI>::load1(in, off + j)), state, sh, p, c);
    DTypeTraits<DTO>::store1(out, off + j, y);
    if (codes != nullptr) codes[off + j] = (uint8_t)c;
  }
  if (codes != nullptr) scales[blk] = (uint8_t)((state == 1) ? sh + 127 : (state == 0 ? 0 : 255));
}

template <int DTI, int DTO>
int launch_mxfp(const void* in, void* out, uint8_t* codes, uint8_t* scales, size_t numel, int B, const MxfpParams& p,
                hipStream_t st) {
  constexpr int V = (DTypeTraits<DTI>::kVec == 8 || DTypeTraits<DTO>::kVec == 8) ? 8 : 4;
  const bool pow2 = (B & (B - 1)) == 0;
  const bool vec_ok = pow2 && B <= 64 * V && (numel % V) == 0 && aligned16(in) && aligned16(out) &&
                      (codes == nullptr || (((uintptr_t)codes) & 7u) == 0);
  if (vec_ok) {
    size_t n_vec = numel / V;
    dim3 grid(blocks_for(n_vec, (size_t)kVecThreads)), block(kVecThreads);
    if constexpr (DTI == DTO && DTI != MASE_DT_F32) {
      // packed 16-bit form: same dtype in and out, no codes wanted, a block is 1, 2, 4 or 8 lanes of 8 elements
      constexpr int MB = (DTI == MASE_DT_BF16) ? 7 : 10, EB = (DTI == MASE_DT_BF16) ? 127 : 15;
      const int lpb = B / 8;
      if (codes == nullptr && B % 8 == 0 && lpb <= 8 && p.m.F <= MB) {
        MxfpPk16Params q;
        q.f = make_pk16_format<MB>(p.m.F, 0);
        q.top0 = p.m.e_hi - p.m.bias + EB;
        q.bot0 = 1 - p.m.bias + EB;
        q.maxfrac = (uint32_t)p.m.frac_hi << q.f.drop;
        q.parity0 = (p.m.bias - EB) & 1;
        const uint4* src = (const uint4*)in;
        uint4* dst = (uint4*)out;
        const dim3 grid_pk(blocks_for(n_vec, (size_t)kVecThreads * kPk16Items));
#define MASE_MXFP_PK(LPB_)                                                                                          \
  do {                                                                                                              \
    if (p.m.E >= 4)                                                                                                 \
      hipLaunchKernelGGL((mxfp_qdq_pk16_kernel<DTI, LPB_, false>), grid_pk, block, 0, st, src, dst, n_vec, p, q);   \
    else                                                                                                            \
      hipLaunchKernelGGL((mxfp_qdq_pk16_kernel<DTI, LPB_, true>), grid_pk, block, 0, st, src, dst, n_vec, p, q);    \
  } while (0)
        switch (lpb) {
          case 1: MASE_MXFP_PK(1); break;
          case 2: MASE_MXFP_PK(2); break;
          case 4: MASE_MXFP_PK(4); break;
          default: MASE_MXFP_PK(8); break;
        }
#undef MASE_MXFP_PK
        return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
      }
    }
#define MASE_MXFP_CASE(LPB_, SUB_)                                                                               \
  do {                                                                                                           \
    if (codes != nullptr)                                                                                        \
      hipLaunchKernelGGL((mxfp_qdq_vec_kernel<DTI, DTO, LPB_, SUB_, true>), grid, block, 0, st, in, out, codes,  \
                         scales, n_vec, p);                                                                      \
    else                                                                                                         \
      hipLaunchKernelGGL((mxfp_qdq_vec_kernel<DTI, DTO, LPB_, SUB_, false>), grid, block, 0, st, in, out, codes, \
                         scales, n_vec, p);                                                                      \
  } while (0)
    if (B >= V) {
      switch (B / V) {
        case 1: MASE_MXFP_CASE(1, 1); break;
        case 2: MASE_MXFP_CASE(2, 1); break;
        case 4: MASE_MXFP_CASE(4, 1); break;
        case 8: MASE_MXFP_CASE(8, 1); break;
        case 16: MASE_MXFP_CASE(16, 1); break;
        case 32: MASE_MXFP_CASE(32, 1); break;
        default: MASE_MXFP_CASE(64, 1); break;
      }
    } else {
      switch (V / B) {
        case 2: MASE_MXFP_CASE(1, 2); break;
        case 4: MASE_MXFP_CASE(1, 4); break;
        default:
          if constexpr (V == 8) MASE_MXFP_CASE(1, 8);
          break;
      }
    }
#undef MASE_MXFP_CASE
  } else {
    size_t n_blocks = numel / (size_t)B;
    hipLaunchKernelGGL((mxfp_qdq_generic_kernel<DTI, DTO>), dim3(blocks_for(n_blocks, kThreads)), dim3(kThreads), 0, st,
                       in, out, codes, scales, n_blocks, B, p);
  }
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

// ---------------------------------------------------------------------------------------------
// Packing for the block-scaled matrix instructions (v_mfma_scale_f32_*_f8f6f4).
//
// Codes and scales are first computed exactly as above (so they decode to the reference's values), then
// adapted to what the hardware formats can express: the reference's element formats are "all finite" (the top
// exponent field holds ordinary values), whereas OCP e4m3 reserves S.1111.111 for NaN and e5m2 reserves the
// whole top exponent field.  A block that uses such a code is re-expressed with the next scale (scale + 1)
// and every element halved: exact for elements with exponent field >= 2, round-to-nearest-even into the
// subnormal range below that (error <= 2^-10 of an element unit while the block maximum is >= 2^8 units).
// 8-bit codes are stored one per byte, 4-bit codes two per byte (even element in the low nibble).
// ---------------------------------------------------------------------------------------------
template <int E, int F>
__device__ __forceinline__ uint32_t halve_code(uint32_t c) {
  const uint32_t sgn = c & (1u << (E + F));
  uint32_t e = (c >> F) & ((1u << E) - 1u);
  uint32_t f = c & ((1u << F) - 1u);
  if (e >= 2) {
    e -= 1;
  } else {
    uint32_t v = (e == 1) ? ((1u << F) + f) : f;
    uint32_t q = (v >> 1) + ((v & 1u) & ((v >> 1) & 1u));  // round half to even
    if (q == (1u << F)) { e = 1; f = 0; }
    else { e = 0; f = q; }
  }
  return sgn | (e << F) | f;
}

template <int E, int F>
__device__ __forceinline__ bool code_is_reserved(uint32_t c) {
  const uint32_t e = (c >> F) & ((1u << E) - 1u);
  const uint32_t f = c & ((1u << F) - 1u);
  if constexpr (E == 4 && F == 3) return e == 15u && f == 7u;  // OCP e4m3: NaN
  if constexpr (E == 5 && F == 2) return e == 31u;             // OCP e5m2: Inf / NaN
  return false;
}

// TILED (8-bit codes only): the codes of a [rows, K] matrix go to the image the tiled block-scaled GEMM copies from,
// [row tile of 256][K tile of 128][row][128 B] with the 16-byte chunks of a row segment exchanged by
// chunk ^= (row >> 1) & 7 (the GEMM's LDS swizzle); k8 = K / 8 lanes per row.  Scales stay row-major.
template <int DTI, int E, int F, bool TILED = false>
__global__ __launch_bounds__(64) void mxfp_pack_kernel(const void* __restrict__ in, uint8_t* __restrict__ codes,
                                                       uint8_t* __restrict__ scales, size_t n8, MxfpParams p,
                                                       uint32_t k8) {
  static_assert(!TILED || E + F + 1 == 8, "the tiled image is written for 8-bit codes");
  using TI = DTypeTraits<DTI>;
  const size_t idx = (size_t)blockIdx.x * 64 + threadIdx.x;  // 8 elements per lane, 4 lanes per block of 32
  const bool live = idx < n8;
  WaveLog2 meta;
  meta.init(p.tab, kLog2TabHalf);
  float x[8];
  uint4 raw[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
  if (live) {
    if constexpr (TI::kVec == 8) {
      raw[0] = load_nt((const uint4*)in + idx);
    } else {
      raw[0] = load_nt((const uint4*)in + 2 * idx);
      raw[1] = load_nt((const uint4*)in + 2 * idx + 1);
    }
  }
  TI::unpack(raw[0], x);
  if constexpr (TI::kVec != 8) TI::unpack(raw[1], x + 4);
  uint32_t m = vec_flushed_absmax<DTI>(raw[0]);
  if constexpr (TI::kVec != 8) m = max(m, vec_flushed_absmax<DTI>(raw[1]));
  m = group_max_u32<4>(m);
  int sh = 0;
  const int state = mxfp_block_scale(m, p, sh, meta);
  uint32_t c[8];
  float y_unused[8];
  mxfp_elements<(E < 4), 8>(x, state, sh, p, c, y_unused);
  // any element may hold the reserved code, not only the largest: a fraction carry that the encoder loses
  // in an odd exponent field leaves the block maximum below a neighbour's code
  uint32_t reserved = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) reserved |= code_is_reserved<E, F>(c[j]) ? 1u : 0u;
  reserved = group_max_u32<4>(reserved);
  int sb = (state == 1) ? sh + 127 : (state == 0 ? 0 : 255);
  if (state == 1 && reserved) {
    sb = min(sb + 1, 254);
#pragma unroll
    for (int j = 0; j < 8; ++j) c[j] = halve_code<E, F>(c[j]);
  }
  if (!live) return;
  if ((idx & 3) == 0) scales[idx >> 2] = (uint8_t)sb;
  if constexpr (E + F + 1 <= 4) {
    uint32_t w = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) w |= (c[j] & 0xFu) << (4 * j);
    ((uint32_t*)codes)[idx] = w;
  } else {
    uint2 w;
    w.x = c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24);
    w.y = c[4] | (c[5] << 8) | (c[6] << 16) | (c[7] << 24);
    if constexpr (TILED) {
      const size_t m = idx / k8;
      const uint32_t k0 = (uint32_t)(idx - m * k8) * 8u;  // byte (= element) position in the row
      const uint32_t r = (uint32_t)m & 255u, kin = k0 & 127u;
      const size_t tile = (m >> 8) * (size_t)(k8 >> 4) + (k0 >> 7);
      const uint32_t at = r * 128u + ((((kin >> 4) ^ ((r >> 1) & 7u)) << 4) | (kin & 15u));
      *(uint2*)(codes + tile * 32768 + at) = w;
    } else {
      ((uint2*)codes)[idx] = w;
    }
  }
}

template <int DTI>
int launch_mxfp_pack(const void* in, uint8_t* codes, uint8_t* scales, size_t numel, int E, int F, const MxfpParams& p,
                     hipStream_t st) {
  const size_t n8 = numel / 8;
  const dim3 grid(blocks_for(n8, 64)), block(64);
  if (E == 4 && F == 3) hipLaunchKernelGGL((mxfp_pack_kernel<DTI, 4, 3>), grid, block, 0, st, in, codes, scales, n8, p, 0u);
  else if (E == 5 && F == 2) hipLaunchKernelGGL((mxfp_pack_kernel<DTI, 5, 2>), grid, block, 0, st, in, codes, scales, n8, p, 0u);
  else if (E == 2 && F == 1) hipLaunchKernelGGL((mxfp_pack_kernel<DTI, 2, 1>), grid, block, 0, st, in, codes, scales, n8, p, 0u);
  else return MASE_ERR_PARAM;
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

template <int DTI>
int launch_mxfp_pack_tiled(const void* in, uint8_t* codes, uint8_t* scales, size_t rows, size_t K, int E, int F,
                           const MxfpParams& p, hipStream_t st) {
  const size_t n8 = rows * K / 8;
  const dim3 grid(blocks_for(n8, 64)), block(64);
  const uint32_t k8 = (uint32_t)(K / 8);
  if (E == 4 && F == 3)
    hipLaunchKernelGGL((mxfp_pack_kernel<DTI, 4, 3, true>), grid, block, 0, st, in, codes, scales, n8, p, k8);
  else if (E == 5 && F == 2)
    hipLaunchKernelGGL((mxfp_pack_kernel<DTI, 5, 2, true>), grid, block, 0, st, in, codes, scales, n8, p, k8);
  else return MASE_ERR_PARAM;
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

template <int DTI>
int launch_mxfp_out(int out_dtype, const void* in, void* out, uint8_t* codes, uint8_t* scales, size_t numel, int B,
                    const MxfpParams& p, hipStream_t st) {
  switch (out_dtype) {
    case MASE_DT_F32: return launch_mxfp<DTI, MASE_DT_F32>(in, out, codes, scales, numel, B, p, st);
    case MASE_DT_BF16: return launch_mxfp<DTI, MASE_DT_BF16>(in, out, codes, scales, numel, B, p, st);
    case MASE_DT_F16: return launch_mxfp<DTI, MASE_DT_F16>(in, out, codes, scales, numel, B, p, st);
    default: return MASE_ERR_DTYPE;
  }
}

}  // namespace
}  // namespace mase

extern "C" int mase_mxfp_qdq(const void* in, void* out, uint8_t* codes, uint8_t* scales, size_t numel, int in_dtype,
                             int out_dtype, int block_size, int exp_bits, int frac_bits, const uint32_t* log2_tab,
                             void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (in == nullptr || out == nullptr || log2_tab == nullptr) return MASE_ERR_NULL;
  if ((codes == nullptr) != (scales == nullptr)) return MASE_ERR_NULL;
  if (block_size <= 0 || numel % (size_t)block_size != 0) return MASE_ERR_SHAPE;
  // legal element formats of the reference (nn/quantizers/mxfp/meta.py:41)
  const int legal[6][2] = {{4, 3}, {5, 2}, {2, 3}, {3, 2}, {2, 1}, {1, 2}};
  bool ok = false;
  for (auto& l : legal) ok = ok || (l[0] == exp_bits && l[1] == frac_bits);
  if (!ok) return MASE_ERR_PARAM;
  MxfpParams p;
  p.m.E = exp_bits;
  p.m.F = frac_bits;
  p.m.bias = (1 << (exp_bits - 1)) - 1;
  p.m.e_hi = (1 << exp_bits) - 1;
  p.m.frac_hi = (1 << frac_bits) - 1;
  p.m.is_finite = 1;
  p.m.round_mode = 0;
  p.el_emax = p.m.e_hi - p.m.bias;
  p.tab = log2_tab;
  hipStream_t st = (hipStream_t)stream;
  switch (in_dtype) {
    case MASE_DT_F32: return launch_mxfp_out<MASE_DT_F32>(out_dtype, in, out, codes, scales, numel, block_size, p, st);
    case MASE_DT_BF16: return launch_mxfp_out<MASE_DT_BF16>(out_dtype, in, out, codes, scales, numel, block_size, p, st);
    case MASE_DT_F16: return launch_mxfp_out<MASE_DT_F16>(out_dtype, in, out, codes, scales, numel, block_size, p, st);
    default: return MASE_ERR_DTYPE;
  }
}

extern "C" int mase_mxfp_pack(const void* in, uint8_t* codes, uint8_t* scales, size_t numel, int in_dtype, int exp_bits,
                              int frac_bits, const uint32_t* log2_tab, void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (in == nullptr || codes == nullptr || scales == nullptr || log2_tab == nullptr) return MASE_ERR_NULL;
  if (numel % 32 != 0) return MASE_ERR_SHAPE;
  if (!aligned16(in) || (((uintptr_t)codes) & 7u) != 0) return MASE_ERR_ALIGN;
  if (!((exp_bits == 4 && frac_bits == 3) || (exp_bits == 5 && frac_bits == 2) || (exp_bits == 2 && frac_bits == 1)))
    return MASE_ERR_PARAM;
  MxfpParams p;
  p.m.E = exp_bits;
  p.m.F = frac_bits;
  p.m.bias = (1 << (exp_bits - 1)) - 1;
  p.m.e_hi = (1 << exp_bits) - 1;
  p.m.frac_hi = (1 << frac_bits) - 1;
  p.m.is_finite = 1;
  p.m.round_mode = 0;
  p.el_emax = p.m.e_hi - p.m.bias;
  p.tab = log2_tab;
  hipStream_t st = (hipStream_t)stream;
  switch (in_dtype) {
    case MASE_DT_F32: return launch_mxfp_pack<MASE_DT_F32>(in, codes, scales, numel, exp_bits, frac_bits, p, st);
    case MASE_DT_BF16: return launch_mxfp_pack<MASE_DT_BF16>(in, codes, scales, numel, exp_bits, frac_bits, p, st);
    case MASE_DT_F16: return launch_mxfp_pack<MASE_DT_F16>(in, codes, scales, numel, exp_bits, frac_bits, p, st);
    default: return MASE_ERR_DTYPE;
  }
}

extern "C" int mase_mxfp_pack_tiled(const void* in, uint8_t* tiled_codes, uint8_t* scales, size_t rows, size_t K,
                                    int in_dtype, int exp_bits, int frac_bits, const uint32_t* log2_tab, void* stream) {
  using namespace mase;
  if (rows == 0 || K == 0) return MASE_OK;
  if (in == nullptr || tiled_codes == nullptr || scales == nullptr || log2_tab == nullptr) return MASE_ERR_NULL;
  if (K % 128 != 0 || rows > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  if (!aligned16(in) || (((uintptr_t)tiled_codes) & 15u) != 0) return MASE_ERR_ALIGN;
  if (!((exp_bits == 4 && frac_bits == 3) || (exp_bits == 5 && frac_bits == 2))) return MASE_ERR_PARAM;
  MxfpParams p;
  p.m.E = exp_bits;
  p.m.F = frac_bits;
  p.m.bias = (1 << (exp_bits - 1)) - 1;
  p.m.e_hi = (1 << exp_bits) - 1;
  p.m.frac_hi = (1 << frac_bits) - 1;
  p.m.is_finite = 1;
  p.m.round_mode = 0;
  p.el_emax = p.m.e_hi - p.m.bias;
  p.tab = log2_tab;
  hipStream_t st = (hipStream_t)stream;
  switch (in_dtype) {
    case MASE_DT_F32: return launch_mxfp_pack_tiled<MASE_DT_F32>(in, tiled_codes, scales, rows, K, exp_bits, frac_bits, p, st);
    case MASE_DT_BF16: return launch_mxfp_pack_tiled<MASE_DT_BF16>(in, tiled_codes, scales, rows, K, exp_bits, frac_bits, p, st);
    case MASE_DT_F16: return launch_mxfp_pack_tiled<MASE_DT_F16>(in, tiled_codes, scales, rows, K, exp_bits, frac_bits, p, st);
    default: return MASE_ERR_DTYPE;
  }
}
