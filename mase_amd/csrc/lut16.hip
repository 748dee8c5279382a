// Element-wise functions of 16-bit tensors by table lookup (gfx950).
//
// A quantize-dequantize of a bf16 / fp16 element that depends on nothing but the element (fixed point, the minifloat
// flavours, the bit-level minifloat cast) is a function from 65536 bit patterns to 65536 bit patterns.  The caller
// builds the 128 KB table once per format by running the arithmetic kernel on all 65536 inputs, so the table is
// bit-identical to that kernel by construction; applying it costs one gather per element from a table that stays in
// the caches, a few instructions instead of 20-30, and the pass runs at the speed of the copy.
#include "common.hpp"

namespace mase {
namespace {

constexpr int kLutThreads = 64;

// 8 elements (one 16-byte vector) per lane
__global__ __launch_bounds__(kLutThreads) void lut16_kernel(const uint4* __restrict__ in, uint4* __restrict__ out,
                                                            size_t n8, const uint16_t* __restrict__ lut) {
  const size_t i = (size_t)blockIdx.x * kLutThreads + threadIdx.x;
  if (i >= n8) return;
  const uint4 v = load_nt(in + i);
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  uint32_t r[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t lo = lut[w[j] & 0xFFFFu], hi = lut[w[j] >> 16];
    r[j] = lo | (hi << 16);
  }
  store_nt(out + i, make_uint4(r[0], r[1], r[2], r[3]));
}

__global__ __launch_bounds__(256) void lut16_tail_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out,
                                                         size_t numel, const uint16_t* __restrict__ lut) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < numel) out[i] = lut[in[i]];
}

}  // namespace
}  // namespace mase

extern "C" int mase_lut16_apply(const void* in, void* out, size_t numel, const uint16_t* table, void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (in == nullptr || out == nullptr || table == nullptr) return MASE_ERR_NULL;
  if ((((uintptr_t)in) & 1u) != 0 || (((uintptr_t)out) & 1u) != 0 || (((uintptr_t)table) & 1u) != 0) return MASE_ERR_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  size_t done = 0;
  if (aligned16(in) && aligned16(out) && numel >= 8) {
    const size_t n8 = numel / 8;
    hipLaunchKernelGGL(lut16_kernel, dim3(blocks_for(n8, kLutThreads)), dim3(kLutThreads), 0, st, (const uint4*)in,
                       (uint4*)out, n8, table);
    done = n8 * 8;
  }
  if (done < numel)
    hipLaunchKernelGGL(lut16_tail_kernel, dim3(blocks_for(numel - done, 256)), dim3(256), 0, st,
                       (const uint16_t*)in + done, (uint16_t*)out + done, numel - done, table);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}
