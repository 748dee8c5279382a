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
#include <algorithm>
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

// The same packing for a 16-bit tensor and a wide-exponent element format (e4m3, e5m2) on the packed 16-bit cast:
// the cast value's [exponent | kept mantissa bits] field, rebased from the tensor dtype's exponent bias at this block's
// scale to the code's, IS the code, so codes come out two per register without the elements ever being widened.
// One lane owns one block of 32 (four 16-byte vectors, 64 consecutive bytes): the block's scale and the cast's
// per-block constants are computed once per 32 elements.
// A block uses a reserved code iff one of its cast values reaches the format's top code (e4m3) or top binade (e5m2):
// seen on the cast values' running maximum; such a block is rebased one exponent step higher, which halves every code
// with exponent field >= 2 exactly.  A vector of 8 elements is encoded on the fp32 form instead where the
// quantize-dequantize kernel would do so (block not regular, element subnormal in T or below the format's normal
// range) and, in a re-expressed block, when it may hold a code with exponent field 1 (whose half is a rounded
// subnormal); its codes are then halved as codes.
// The row of block b (< 2^31) is b / kb by multiplication: row = mulhi(b, kb_magic) >> kb_shift with
// kb_magic = ceil(2^(31 + l) / kb), kb_shift = l - 1, l = ceil(log2 kb) >= 2 (exact for 31-bit dividends).
template <int DT, int E, int F, bool TILED>
__global__ __launch_bounds__(kVecThreads) void mxfp_pack_pk16_kernel(const uint4* __restrict__ in,
                                                                     uint8_t* __restrict__ codes,
                                                                     uint8_t* __restrict__ scales, uint32_t n_blocks,
                                                                     MxfpParams p, MxfpPk16Params q, uint32_t kb,
                                                                     uint32_t kb_magic, uint32_t kb_shift) {
  static_assert(E + F + 1 == 8 && E >= 4, "8-bit codes of a wide-exponent format");
  using TR = DTypeTraits<DT>;
  constexpr int MB = (DT == MASE_DT_BF16) ? 7 : 10, EB = (DT == MASE_DT_BF16) ? 127 : 15;
  constexpr uint32_t one = 0x00010001u;
  WaveLog2 meta;
  meta.init(p.tab, kLog2TabHalf);
  const uint32_t lane = threadIdx.x;
  const uint32_t blk = blockIdx.x * (uint32_t)kVecThreads + lane;
  const bool live = blk < n_blocks;
  // Load v of a quad of lanes (4q .. 4q+3) reads the 64 bytes of block 4q + v, 16 per lane, so every load touches
  // runs of 64 bytes; a 4 x 4 exchange inside the quad (two butterfly steps on quad permutes) then gives each lane
  // the four vectors of its own block.  n_blocks is a multiple of 4 (the launcher's condition).
  uint4 raw[4];
  {
    const uint32_t quad_blk = blk - (lane & 3u);
#pragma unroll
    for (int v = 0; v < 4; ++v)
      raw[v] = live ? load_nt(in + (size_t)(quad_blk + v) * 4 + (lane & 3u)) : make_uint4(0, 0, 0, 0);
    uint32_t t[4][4];  // [register][dword]
#pragma unroll
    for (int v = 0; v < 4; ++v) { t[v][0] = raw[v].x; t[v][1] = raw[v].y; t[v][2] = raw[v].z; t[v][3] = raw[v].w; }
    const bool odd = (lane & 1u) != 0, upper = (lane & 2u) != 0;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
#pragma unroll
      for (int r0 = 0; r0 < 4; r0 += 2) {  // lanes i, i^1 exchange registers (r0, r0+1)
        const uint32_t got = dpp_mov<0xB1>(odd ? t[r0][d] : t[r0 + 1][d]);
        t[r0][d] = odd ? got : t[r0][d];
        t[r0 + 1][d] = odd ? t[r0 + 1][d] : got;
      }
#pragma unroll
      for (int r0 = 0; r0 < 2; ++r0) {  // lanes i, i^2 exchange registers (r0, r0+2)
        const uint32_t got = dpp_mov<0x4E>(upper ? t[r0][d] : t[r0 + 2][d]);
        t[r0][d] = upper ? got : t[r0][d];
        t[r0 + 2][d] = upper ? t[r0 + 2][d] : got;
      }
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) raw[v] = make_uint4(t[v][0], t[v][1], t[v][2], t[v][3]);
  }
  // block maximum: packed over the 16 registers, then as flushed fp32 bits
  uint32_t pm = 0;
#pragma unroll
  for (int v = 0; v < 4; ++v)
    pm = pk_max_u16(pm, pk_max_u16(pk_max_u16(raw[v].x & 0x7FFF7FFFu, raw[v].y & 0x7FFF7FFFu),
                                   pk_max_u16(raw[v].z & 0x7FFF7FFFu, raw[v].w & 0x7FFF7FFFu)));
  pm = max(pm & 0xFFFFu, pm >> 16);
  uint32_t m;
  if constexpr (DT == MASE_DT_BF16) m = pm << 16;
  else m = f2bits(f16_bits_to_f32(pm));
  if ((m & 0x7F800000u) == 0) m = 0;  // a subnormal maximum means every element is flushed
  int sh = 0;
  const int state = mxfp_block_scale(m, p, sh, meta);
  const int botf = q.bot0 + sh;
  const uint32_t topf = (uint32_t)min(max(q.top0 + sh, 1), 0xFF);
  Pk16Range r;
  r.odd_k2 = (((q.parity0 - sh) & 1) ? (1u << MB) : 0u) * one;
  r.max2 = ((topf << MB) | q.maxfrac) * one;
  const uint32_t lo_thr = (uint32_t)min(max(botf, 1), 0xFF) << MB;
  r.lo_thr2 = lo_thr * one;
  r.sub_thr2 = 0;
  uint32_t y[4][4], lo[4];
  u16x2 top_acc = as_u16x2(0u);
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const uint32_t w[4] = {raw[v].x, raw[v].y, raw[v].z, raw[v].w};
    u16x2 lo_acc = as_u16x2(0xFFFFFFFFu), hi_acc = as_u16x2(0u);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      y[v][j] = pk16_cast<MB, false>(w[j], q.f, r, lo_acc, hi_acc);
      top_acc = __builtin_elementwise_max(top_acc, as_u16x2(y[v][j] & 0x7FFF7FFFu));
    }
    lo[v] = min((uint32_t)lo_acc.x, (uint32_t)lo_acc.y);
  }
  const uint32_t top_y = max((uint32_t)top_acc.x, (uint32_t)top_acc.y);
  // the element that takes a reserved code lies in the block's top binade, so its cast value is valid unless the whole
  // block is subnormal in T, and then every vector takes the fp32 form and reports from its codes
  const bool top_reserved = top_y >= ((E == 4) ? ((topf << MB) | q.maxfrac) : (topf << MB));
  uint32_t lowest = lo_thr;
  if constexpr (DT == MASE_DT_BF16) lowest = max(lowest, (uint32_t)min(max(sh + 1, 1), 0xFF) << MB);
  if (top_reserved) lowest += 1u << MB;
  uint32_t cc[4][4];  // codes, two per register (one per 16-bit half)
  uint32_t fp32_form = 0, flag = 0;
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    if (__builtin_expect(state != 1 || lo[v] + 1u < lowest, 0)) {
      float x[8], z[8];
      uint32_t c[8];
      TR::unpack(raw[v], x);
      mxfp_elements<true, 8>(x, state, sh, p, c, z);  // the form that handles codes with exponent field 0 in line
#pragma unroll
      for (int j = 0; j < 8; ++j) flag |= code_is_reserved<E, F>(c[j]) ? 1u : 0u;
#pragma unroll
      for (int j = 0; j < 4; ++j) cc[v][j] = c[2 * j] | (c[2 * j + 1] << 16);
      fp32_form |= 1u << v;
    }
  }
  const bool reserved = state == 1 && (top_reserved || flag != 0);
  const uint32_t rebase2 = ((uint32_t)((sh + (reserved ? 1 : 0) + EB - p.m.bias) << F) & 0xFFFFu) * one;
  const u16x2 drop2 = {(unsigned short)q.f.drop, (unsigned short)q.f.drop};
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    if (__builtin_expect((fp32_form >> v) & 1u, 0)) {
      if (reserved) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t a = cc[v][j] & 0x007F007Fu;
          const uint32_t small = neg_mask2(as_u32(as_u16x2(a) - as_u16x2((2u << F) * one)));  // exponent field < 2
          const uint32_t h_big = as_u32(as_u16x2(a) - as_u16x2((1u << F) * one));
          const uint32_t half = (a >> 1) & 0x003F003Fu;
          const uint32_t h_small = half + (a & half & one);  // the value of such a code is the code: round half even
          cc[v][j] = (small & h_small) | (~small & h_big) | (cc[v][j] & 0x00800080u);
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t ya = y[v][j] & 0x7FFF7FFFu;
        const uint32_t nz = neg_mask2(as_u32(as_u16x2(ya) + as_u16x2(0x7FFF7FFFu)));  // halves that are not zero
        const uint32_t field = as_u32((as_u16x2(ya) >> drop2) - as_u16x2(rebase2));
        cc[v][j] = (field & nz & 0x007F007Fu) | ((y[v][j] >> 8) & 0x00800080u);
      }
    }
  }
  const int sb = (state == 1) ? min(sh + 127 + (reserved ? 1 : 0), 254) : (state == 0 ? 0 : 255);
  if (live) scales[blk] = (uint8_t)sb;
  uint4 o[2];  // the block's 32 code bytes
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    o[h].x = __builtin_amdgcn_perm(cc[2 * h][1], cc[2 * h][0], 0x06040200u);
    o[h].y = __builtin_amdgcn_perm(cc[2 * h][3], cc[2 * h][2], 0x06040200u);
    o[h].z = __builtin_amdgcn_perm(cc[2 * h + 1][1], cc[2 * h + 1][0], 0x06040200u);
    o[h].w = __builtin_amdgcn_perm(cc[2 * h + 1][3], cc[2 * h + 1][2], 0x06040200u);
  }
  // A quad's four blocks are one 128-byte run of codes (tiled image: one row of one K tile, whose 16-byte chunks are
  // exchanged by chunk ^= swizzle of the row).  Store h of lane j writes chunk 4h + j of the quad, fetched from the
  // lane that produced it (lane (4h + j) / 2, its vector (4h + j) % 2), so a quad writes runs of 64 bytes.
  const uint32_t j = lane & 3u;
  uint8_t* line;
  uint32_t sw = 0;
  if constexpr (TILED) {
    const uint32_t quad_blk = blk - j;
    const uint32_t mrow = __umulhi(quad_blk, kb_magic) >> kb_shift;
    const uint32_t k0 = (quad_blk - mrow * kb) * 32u;  // byte (= element) position in the row: a multiple of 128
    const uint32_t rr = mrow & 255u;
    sw = (rr >> 1) & 7u;
    line = codes + ((size_t)(mrow >> 8) * (kb >> 2) + (k0 >> 7)) * 32768 + rr * 128u;
  } else {
    line = codes + (size_t)(blk - j) * 32;
  }
  const bool second = (lane & 1u) != 0;
  uint4 d0, d1;
  {
    const uint32_t a0 = dpp_mov<0x50>(o[0].x), b0 = dpp_mov<0x50>(o[1].x), a1 = dpp_mov<0x50>(o[0].y), b1 = dpp_mov<0x50>(o[1].y);
    const uint32_t a2 = dpp_mov<0x50>(o[0].z), b2 = dpp_mov<0x50>(o[1].z), a3 = dpp_mov<0x50>(o[0].w), b3 = dpp_mov<0x50>(o[1].w);
    d0 = make_uint4(second ? b0 : a0, second ? b1 : a1, second ? b2 : a2, second ? b3 : a3);  // from lane j / 2
  }
  {
    const uint32_t a0 = dpp_mov<0xFA>(o[0].x), b0 = dpp_mov<0xFA>(o[1].x), a1 = dpp_mov<0xFA>(o[0].y), b1 = dpp_mov<0xFA>(o[1].y);
    const uint32_t a2 = dpp_mov<0xFA>(o[0].z), b2 = dpp_mov<0xFA>(o[1].z), a3 = dpp_mov<0xFA>(o[0].w), b3 = dpp_mov<0xFA>(o[1].w);
    d1 = make_uint4(second ? b0 : a0, second ? b1 : a1, second ? b2 : a2, second ? b3 : a3);  // from lane 2 + j / 2
  }
  if (live) {
    *(uint4*)(line + ((j ^ sw) << 4)) = d0;
    *(uint4*)(line + (((4u + j) ^ sw) << 4)) = d1;
  }
}

template <int DT, bool TILED>
bool launch_mxfp_pack_pk16(const void* in, uint8_t* codes, uint8_t* scales, size_t n8, int E, int F,
                           const MxfpParams& p, uint32_t k8, hipStream_t st) {
  if constexpr (DT == MASE_DT_F32) {
    return false;
  } else {
    constexpr int MB = (DT == MASE_DT_BF16) ? 7 : 10, EB = (DT == MASE_DT_BF16) ? 127 : 15;
    if (!((E == 4 && F == 3) || (E == 5 && F == 2)) || !aligned16(in) || !aligned16(codes)) return false;
    const size_t n_blocks = n8 / 4;
    const uint32_t kb = k8 / 4;
    // quads of lanes read and write four consecutive blocks together
    if (n_blocks == 0 || (n_blocks & 3) != 0 || n_blocks >= (1ull << 31) || (TILED && kb < 4)) return false;
    MxfpPk16Params q;
    q.f = make_pk16_format<MB>(p.m.F, 0);
    q.top0 = p.m.e_hi - p.m.bias + EB;
    q.bot0 = 1 - p.m.bias + EB;
    q.maxfrac = (uint32_t)p.m.frac_hi << q.f.drop;
    q.parity0 = (p.m.bias - EB) & 1;
    uint32_t magic = 0, shift = 0;
    if (TILED) {
      uint32_t l = 0;
      while ((1ull << l) < kb) ++l;
      magic = (uint32_t)(((1ull << (31 + l)) + kb - 1) / kb);
      shift = l - 1;
    }
    const dim3 grid(blocks_for(n_blocks, (size_t)kVecThreads)), block(kVecThreads);
    if (E == 4)
      hipLaunchKernelGGL((mxfp_pack_pk16_kernel<DT, 4, 3, TILED>), grid, block, 0, st, (const uint4*)in, codes, scales,
                         (uint32_t)n_blocks, p, q, kb, magic, shift);
    else
      hipLaunchKernelGGL((mxfp_pack_pk16_kernel<DT, 5, 2, TILED>), grid, block, 0, st, (const uint4*)in, codes, scales,
                         (uint32_t)n_blocks, p, q, kb, magic, shift);
    return true;
  }
}

template <int DTI>
int launch_mxfp_pack(const void* in, uint8_t* codes, uint8_t* scales, size_t numel, int E, int F, const MxfpParams& p,
                     hipStream_t st) {
  const size_t n8 = numel / 8;
  if (launch_mxfp_pack_pk16<DTI, false>(in, codes, scales, n8, E, F, p, 0u, st))
    return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
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
  if (launch_mxfp_pack_pk16<DTI, true>(in, codes, scales, n8, E, F, p, k8, st))
    return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
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
