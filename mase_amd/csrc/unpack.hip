// Dequantization of packed MX tensors for gfx950: element codes (one byte each) and one shared-exponent byte per
// block back to a floating-point tensor.  This is the "compose" half of the reference's quantizers
// (nn/quantizers/mxint/fake.py:59-80 compose_mxint_tensor, nn/quantizers/mxfp/fake.py:75-104) applied to the packed
// outputs of mase_mxint_qdq / mase_mxfp_qdq, so that a checkpoint can hold 8.25 bits per weight and be loaded without
// running the quantizer again.  HBM-bound: 1 + 1/B bytes read and 2 or 4 written per element.
#include "common.hpp"
#include "minifloat_mx.hpp"

namespace mase {
namespace {

constexpr int kUnpackThreads = 64;

struct UnpackParams {
  int kind;            // 0 MXINT, 1 MXFP
  int block_size;
  MinifloatMxFmt m;    // MXFP element format
};

// value of one element; scale is the block's shared-exponent byte
__device__ __forceinline__ float unpack_value(uint32_t code, uint32_t scale, const UnpackParams& p) {
  if (p.kind == 0) return ldexpf((float)(int)(int8_t)code, (int)scale - 134);
  if (scale == 255u) return qnan();  // block with a non-finite maximum
  return minifloat_mx_decode(code, p.m) * pow2f((int)scale - 127);
}

template <int DTO>
__device__ __forceinline__ void store16(void* out, size_t i16, const float* y) {
  using TO = DTypeTraits<DTO>;
  constexpr int kVecs = 16 / TO::kVec;
  uint4* q = (uint4*)out + i16 * kVecs;
#pragma unroll
  for (int v = 0; v < kVecs; ++v) store_nt(q + v, TO::pack(y + v * TO::kVec));
}

// 16 codes (one 16-byte load) per lane; block_size is a multiple of 16, so a lane's codes share one scale
template <int DTO>
__global__ __launch_bounds__(kUnpackThreads) void mx_unpack_vec_kernel(const uint8_t* __restrict__ codes,
                                                                       const uint8_t* __restrict__ scales,
                                                                       void* __restrict__ out, size_t n16,
                                                                       UnpackParams p) {
  const size_t i = (size_t)blockIdx.x * kUnpackThreads + threadIdx.x;
  if (i >= n16) return;
  const uint4 c = load_nt((const uint4*)codes + i);
  const uint32_t scale = scales[(i * 16) / (size_t)p.block_size];
  const uint32_t w[4] = {c.x, c.y, c.z, c.w};
  float y[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) y[j] = unpack_value((w[j >> 2] >> (8 * (j & 3))) & 0xFFu, scale, p);
  store16<DTO>(out, i, y);
}

// any block size / alignment: one element per lane
template <int DTO>
__global__ __launch_bounds__(256) void mx_unpack_scalar_kernel(const uint8_t* __restrict__ codes,
                                                               const uint8_t* __restrict__ scales, void* __restrict__ out,
                                                               size_t numel, UnpackParams p) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= numel) return;
  DTypeTraits<DTO>::store1(out, i, unpack_value(codes[i], scales[i / (size_t)p.block_size], p));
}

template <int DTO>
int launch_unpack(const uint8_t* codes, const uint8_t* scales, void* out, size_t numel, const UnpackParams& p,
                  hipStream_t st) {
  if (p.block_size % 16 == 0 && aligned16(codes) && aligned16(out)) {
    const size_t n16 = numel / 16;  // numel is a multiple of block_size
    hipLaunchKernelGGL((mx_unpack_vec_kernel<DTO>), dim3(blocks_for(n16, kUnpackThreads)), dim3(kUnpackThreads), 0, st,
                       codes, scales, out, n16, p);
  } else {
    hipLaunchKernelGGL((mx_unpack_scalar_kernel<DTO>), dim3(blocks_for(numel, 256)), dim3(256), 0, st, codes, scales,
                       out, numel, p);
  }
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

}  // namespace
}  // namespace mase

extern "C" int mase_mx_unpack(const uint8_t* codes, const uint8_t* scales, void* out, size_t numel, int block_size,
                              int out_dtype, int kind, int p0, int p1, void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (codes == nullptr || scales == nullptr || out == nullptr) return MASE_ERR_NULL;
  if (block_size < 1 || numel % (size_t)block_size != 0) return MASE_ERR_SHAPE;
  UnpackParams p{};
  p.kind = kind;
  p.block_size = block_size;
  if (kind == 0) {
    if (p0 < 2 || p0 > 8) return MASE_ERR_PARAM;  // element_bits: codes are one signed byte
  } else if (kind == 1) {
    const int E = p0, F = p1;
    if (E <= 0 || F <= 0 || E + F > 7) return MASE_ERR_PARAM;  // sign|exp|frac in one byte
    p.m.E = E;
    p.m.F = F;
    p.m.bias = (1 << (E - 1)) - 1;
    p.m.e_hi = (1 << E) - 1;
    p.m.frac_hi = (1 << F) - 1;
    p.m.is_finite = 1;
    p.m.round_mode = 0;
  } else {
    return MASE_ERR_PARAM;
  }
  hipStream_t st = (hipStream_t)stream;
  switch (out_dtype) {
    case MASE_DT_F32: return launch_unpack<MASE_DT_F32>(codes, scales, out, numel, p, st);
    case MASE_DT_BF16: return launch_unpack<MASE_DT_BF16>(codes, scales, out, numel, p, st);
    case MASE_DT_F16: return launch_unpack<MASE_DT_F16>(codes, scales, out, numel, p, st);
    default: return MASE_ERR_DTYPE;
  }
}
