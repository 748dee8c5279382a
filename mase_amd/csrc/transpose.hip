// Transposed copy of the trailing two dimensions of a 16-bit tensor for gfx950: in[o][i][r][c] -> out[o][i][c][r],
// r padded with zeros to a multiple of 64.  The tiled matrix-core kernels contract rows with rows
// (C = A B^T); an operand that arrives as [K, N] rows (the values of an attention block, the second operand of
// torch.matmul / torch.bmm, nn/quantized/modules/llama/attention.py:449, nn/quantized/functional/matmul.py:437-512) is
// turned into [N, K] rows by this copy, and the zero padding makes K a whole number of the kernels' K tiles.
// HBM-bound: 2 B read + 2 B written per element; 64 x 64 tiles through LDS, 16-byte accesses on both sides.
#include "common.hpp"

namespace mase {
namespace {

struct TransposeParams {
  const unsigned char* in;
  unsigned char* out;
  int rows, cols, rows_padded;     // r, c, r rounded up to a multiple of 64
  int inner;                       // batch index = outer * inner + i
  size_t in_so, in_si, in_sr;      // byte strides of the input: outer, inner, row (columns are contiguous)
};

constexpr int kTT = 64;            // tile edge
constexpr int kTPitch = kTT + 2;   // LDS row pitch in elements: 33 words, so a column walk touches 32 different banks

__global__ __launch_bounds__(256) void transpose16_kernel(TransposeParams p) {
  __shared__ uint16_t tile[kTT][kTPitch];
  const int r0 = (int)blockIdx.x * kTT, c0 = (int)blockIdx.y * kTT;
  const int b = (int)blockIdx.z, bo = b / p.inner, bi = b - bo * p.inner;
  const unsigned char* src = p.in + (size_t)bo * p.in_so + (size_t)bi * p.in_si;
  unsigned char* dst = p.out + (size_t)b * (size_t)p.cols * (size_t)p.rows_padded * 2;
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int i = (int)threadIdx.x + u * 256;
    const int r = i >> 3, c8 = (i & 7) * 8;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (r0 + r < p.rows && c0 + c8 < p.cols) v = *(const uint4*)(src + (size_t)(r0 + r) * p.in_sr + (size_t)(c0 + c8) * 2);
    uint32_t* row = (uint32_t*)&tile[r][c8];  // 4-byte aligned: the pitch and c8 are even
    row[0] = v.x; row[1] = v.y; row[2] = v.z; row[3] = v.w;
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int i = (int)threadIdx.x + u * 256;
    const int c = i >> 3, r8 = (i & 7) * 8;
    if (c0 + c >= p.cols) continue;
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = (uint32_t)tile[r8 + 2 * e][c] | ((uint32_t)tile[r8 + 2 * e + 1][c] << 16);
    *(uint4*)(dst + ((size_t)(c0 + c) * p.rows_padded + (size_t)(r0 + r8)) * 2) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

}  // namespace
}  // namespace mase

extern "C" int mase_transpose16(const void* in, void* out, size_t batch_outer, size_t batch_inner, size_t rows, size_t cols,
                                size_t rows_padded, size_t in_stride_outer, size_t in_stride_inner, size_t in_stride_row,
                                void* stream) {
  using namespace mase;
  if (batch_outer == 0 || batch_inner == 0 || rows == 0 || cols == 0) return MASE_OK;
  if (in == nullptr || out == nullptr) return MASE_ERR_NULL;
  if (cols % 8 != 0 || rows_padded % kTT != 0 || rows_padded < rows || rows_padded - rows >= (size_t)kTT) return MASE_ERR_SHAPE;
  if (rows > (1u << 30) || cols > (1u << 30) || batch_outer * batch_inner > 65535 || batch_inner > (1u << 30) ||
      (cols + kTT - 1) / kTT > 65535)
    return MASE_ERR_SHAPE;
  if (in_stride_row < cols) return MASE_ERR_SHAPE;
  if (!aligned16(in) || !aligned16(out) || in_stride_outer % 8 || in_stride_inner % 8 || in_stride_row % 8) return MASE_ERR_ALIGN;
  TransposeParams p;
  p.in = (const unsigned char*)in;
  p.out = (unsigned char*)out;
  p.rows = (int)rows;
  p.cols = (int)cols;
  p.rows_padded = (int)rows_padded;
  p.inner = (int)batch_inner;
  p.in_so = in_stride_outer * 2;
  p.in_si = in_stride_inner * 2;
  p.in_sr = in_stride_row * 2;
  const dim3 grid((unsigned)(rows_padded / kTT), (unsigned)((cols + kTT - 1) / kTT), (unsigned)(batch_outer * batch_inner));
  hipLaunchKernelGGL(transpose16_kernel, grid, dim3(256), 0, (hipStream_t)stream, p);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}
