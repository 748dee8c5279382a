// Calibration kernels of the benchmark (bench.py), built into bench_support/libmase_bench.so: NOT part of the product
// library or its C ABI, and without counterpart in the reference.
//   bench_copy_bytes               plain streaming copy: the achievable-bandwidth ceiling and the scale of the hardware
//                                  byte counters
//   bench_probe_mfma_bf16 / _bf16_16x16 / _f8f4  issue rate of a matrix instruction on register operands, nothing else
//                                  running
//   bench_constant_rate_counter_khz
// Status codes: 0 ok, negative = the product library's error codes (include/mase_amd.h).
//
// The matrix-core probe: the rate at which the matrix cores of this GPU accept
// v_mfma_f32_32x32x16_bf16 when nothing else runs (no memory traffic, no LDS, operands held in registers), as a
// function of the operand VALUES.  The rate depends on them: with zero or small-integer operands the instruction
// issues close to its nominal 32 cycles, with operands whose mantissa and exponent bits vary it is held back by the
// power management of the part.  That second figure, not the published peak, is what a GEMM on real data can approach.
#include "../mase_amd/csrc/common.hpp"

namespace mase {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}

// operands: 0 zeros, 1 small integers, 2 uniform in [-2, 2) with full mantissas.  Each wavefront issues 8 * iters
// instructions on two accumulator chains; out receives one float per lane so that nothing is optimised away, and after
// those the first wavefront's loop duration on the shader-clock counter and on the constant-rate counter (two int64).
__global__ __launch_bounds__(512) void probe_mfma_bf16_kernel(float* out, int iters, int operands) {
  const int lane = threadIdx.x & 63;
  bf16x8_t a[4], b[4];
#pragma unroll
  for (int s = 0; s < 4; ++s)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t h1 = probe_hash(threadIdx.x * 64 + s * 8 + i + blockIdx.x * 7919), h2 = probe_hash(h1 + 12345);
      float va = 0.0f, vb = 0.0f;
      if (operands == 1) { va = (float)((lane + i) & 7); vb = (float)((lane - i) & 3); }
      if (operands == 2) {
        va = (float)(int)(h1 >> 8) * (1.0f / 4194304.0f) - 2.0f;
        vb = (float)(int)(h2 >> 8) * (1.0f / 4194304.0f) - 2.0f;
      }
      a[s][i] = (__bf16)va;
      b[s][i] = (__bf16)vb;
    }
  f32x16_t acc[2];
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[c][r] = 0.0f;
  const long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s], b[s], acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(s + 1) & 3], b[s], acc[1], 0, 0, 0);
    }
  }
  float r = 0.0f;
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int k = 0; k < 16; ++k) r += acc[c][k];
  const long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = r;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    long long* t = (long long*)(out + (size_t)gridDim.x * blockDim.x);
    t[0] = c1 - c0;
    t[1] = w1 - w0;
  }
}

// The same for v_mfma_f32_16x16x32_bf16, the instruction of the tiled GEMM on the fragment-ordered weight: the same
// multiply-adds per cycle (16 instructions of half the work per iteration), on four times as many accumulator chains
// of a quarter of the size.  With varying operand bits it is held back less than the 32x32x16 instruction.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(512) void probe_mfma_bf16_16x16_kernel(float* out, int iters, int operands) {
  const int lane = threadIdx.x & 63;
  bf16x8_t a[4], b[4];
#pragma unroll
  for (int s = 0; s < 4; ++s)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t h1 = probe_hash(threadIdx.x * 64 + s * 8 + i + blockIdx.x * 7919), h2 = probe_hash(h1 + 12345);
      float va = 0.0f, vb = 0.0f;
      if (operands == 1) { va = (float)((lane + i) & 7); vb = (float)((lane - i) & 3); }
      if (operands == 2) {
        va = (float)(int)(h1 >> 8) * (1.0f / 4194304.0f) - 2.0f;
        vb = (float)(int)(h2 >> 8) * (1.0f / 4194304.0f) - 2.0f;
      }
      a[s][i] = (__bf16)va;
      b[s][i] = (__bf16)vb;
    }
  f32x4_t acc[8];
#pragma unroll
  for (int c = 0; c < 8; ++c)
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[c][r] = 0.0f;
  const long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int c = 2 * s, d = (2 * s + 4) & 7;
      acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s], b[s], acc[c], 0, 0, 0);
      acc[c + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[(s + 1) & 3], b[s], acc[c + 1], 0, 0, 0);
      acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[(s + 2) & 3], b[s], acc[d], 0, 0, 0);
      acc[d + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[(s + 3) & 3], b[s], acc[d + 1], 0, 0, 0);
    }
  }
  float r = 0.0f;
#pragma unroll
  for (int c = 0; c < 8; ++c)
#pragma unroll
    for (int k = 0; k < 4; ++k) r += acc[c][k];
  const long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = r;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    long long* t = (long long*)(out + (size_t)gridDim.x * blockDim.x);
    t[0] = c1 - c0;
    t[1] = w1 - w0;
  }
}

// The same for v_mfma_scale_f32_32x32x64_f8f6f4 with e4m3 codes in A and e2m1 codes in B (the instruction of the
// MXFP8 x MXFP4 Linear), scales of 1.  operands: 0 zero codes, 2 random codes (the e4m3 NaN code excluded).
typedef int i32x8_t __attribute__((ext_vector_type(8)));
__global__ __launch_bounds__(512) void probe_mfma_f8f4_kernel(float* out, int iters, int operands) {
  i32x8_t a[4], b[4];
#pragma unroll
  for (int s = 0; s < 4; ++s)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t h1 = probe_hash(threadIdx.x * 64 + s * 8 + i + blockIdx.x * 7919), h2 = probe_hash(h1 + 12345);
      a[s][i] = operands == 2 ? (int)(h1 & 0xBFBFBFBFu) : 0;          // exponent field below 1000: never the NaN code
      b[s][i] = (operands == 2 && i < 4) ? (int)h2 : 0;                // 64 e2m1 codes in the first four registers
    }
  f32x16_t acc[2];
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[c][r] = 0.0f;
  const long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      acc[0] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[s], b[s], acc[0], 0, 4, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
      acc[1] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[(s + 1) & 3], b[s], acc[1], 0, 4, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
    }
  }
  float r = 0.0f;
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int k = 0; k < 16; ++k) r += acc[c][k];
  const long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = r;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    long long* t = (long long*)(out + (size_t)gridDim.x * blockDim.x);
    t[0] = c1 - c0;
    t[1] = w1 - w0;
  }
}

__global__ __launch_bounds__(64) void copy_bytes_kernel(const uint4* __restrict__ in, uint4* __restrict__ out, size_t n) {
  size_t i = (size_t)blockIdx.x * 64 + threadIdx.x;
  if (i < n) store_nt(out + i, load_nt(in + i));
}

// each wavefront issues 8 * iters matrix instructions; the bound keeps a mistaken argument from occupying the GPU for
// minutes (2^20 iterations are about a tenth of a second)
constexpr int kMaxProbeIters = 1 << 20;

}  // namespace
}  // namespace mase

// `bytes` a multiple of 16, pointers 16-byte aligned
extern "C" int bench_copy_bytes(const void* in, void* out, size_t bytes, void* stream) {
  using namespace mase;
  if (bytes == 0) return MASE_OK;
  if (in == nullptr || out == nullptr) return MASE_ERR_NULL;
  if ((bytes & 15u) != 0) return MASE_ERR_SHAPE;
  if (!aligned16(in) || !aligned16(out)) return MASE_ERR_ALIGN;
  const size_t n = bytes / 16;
  hipLaunchKernelGGL(copy_bytes_kernel, dim3(blocks_for(n, 64)), dim3(64), 0, (hipStream_t)stream, (const uint4*)in,
                     (uint4*)out, n);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

// work_groups x (4 x wavefronts_per_simd) wavefronts, each issuing 8 * iters instructions (1 <= iters <= 2^20) on
// register operands.  out (16-byte aligned): work_groups * 256 * wavefronts_per_simd floats of scratch followed by two
// int64 the kernel writes: the duration of the first wavefront's loop in shader-clock cycles and in ticks of the
// constant-rate counter.
extern "C" int bench_probe_mfma_bf16(void* out, size_t out_bytes, int work_groups, int wavefronts_per_simd, int iters,
                                    int operands, void* stream) {
  using namespace mase;
  if (out == nullptr) return MASE_ERR_NULL;
  if (work_groups < 1 || work_groups > 65536 || (wavefronts_per_simd != 1 && wavefronts_per_simd != 2) || iters < 1 || iters > kMaxProbeIters ||
      operands < 0 || operands > 2)
    return MASE_ERR_PARAM;
  const int threads = 256 * wavefronts_per_simd;
  if (out_bytes < (size_t)work_groups * threads * sizeof(float) + 16 || !aligned16(out)) return MASE_ERR_WORKSPACE;
  hipLaunchKernelGGL(probe_mfma_bf16_kernel, dim3((unsigned)work_groups), dim3((unsigned)threads), 0, (hipStream_t)stream,
                     (float*)out, iters, operands);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

// as bench_probe_mfma_bf16, with v_mfma_f32_16x16x32_bf16 (16 * iters instructions per wavefront)
extern "C" int bench_probe_mfma_bf16_16x16(void* out, size_t out_bytes, int work_groups, int wavefronts_per_simd, int iters,
                                          int operands, void* stream) {
  using namespace mase;
  if (out == nullptr) return MASE_ERR_NULL;
  if (work_groups < 1 || work_groups > 65536 || (wavefronts_per_simd != 1 && wavefronts_per_simd != 2) || iters < 1 || iters > kMaxProbeIters ||
      operands < 0 || operands > 2)
    return MASE_ERR_PARAM;
  const int threads = 256 * wavefronts_per_simd;
  if (out_bytes < (size_t)work_groups * threads * sizeof(float) + 16 || !aligned16(out)) return MASE_ERR_WORKSPACE;
  hipLaunchKernelGGL(probe_mfma_bf16_16x16_kernel, dim3((unsigned)work_groups), dim3((unsigned)threads), 0, (hipStream_t)stream,
                     (float*)out, iters, operands);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

extern "C" int bench_probe_mfma_f8f4(void* out, size_t out_bytes, int work_groups, int wavefronts_per_simd, int iters,
                                    int operands, void* stream) {
  using namespace mase;
  if (out == nullptr) return MASE_ERR_NULL;
  if (work_groups < 1 || work_groups > 65536 || (wavefronts_per_simd != 1 && wavefronts_per_simd != 2) || iters < 1 || iters > kMaxProbeIters ||
      (operands != 0 && operands != 2))
    return MASE_ERR_PARAM;
  const int threads = 256 * wavefronts_per_simd;
  if (out_bytes < (size_t)work_groups * threads * sizeof(float) + 16 || !aligned16(out)) return MASE_ERR_WORKSPACE;
  hipLaunchKernelGGL(probe_mfma_f8f4_kernel, dim3((unsigned)work_groups), dim3((unsigned)threads), 0, (hipStream_t)stream,
                     (float*)out, iters, operands);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

// rate of the constant-rate counter on the current device in kHz; 0 when the runtime cannot tell
extern "C" int bench_constant_rate_counter_khz(void) {
  int dev = 0, khz = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess) return 0;
  return khz;
}
