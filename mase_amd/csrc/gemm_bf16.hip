// C[M,N] = A[M,K] * B[N,K]^T (+ bias[N]) on gfx950 matrix cores: bf16 operands, fp32 accumulation.
//
// This is the contraction behind the MX Linear forward.  Both operands are K-major (activations [tokens, K],
// weights [out, K]), which is the layout v_mfma_f32_32x32x16_bf16 wants: lane l supplies 8 consecutive
// K-elements of row/column l%32, K-group l/32.  MXINT8 and MXFP values are exactly representable in bf16
// (<= 8 significant bits times a power of two), so feeding them as bf16 computes the same real-number dot
// products as the reference's fp32 GEMM on the quantize-dequantized operands; only the summation order
// differs.
//
// Schedule: 256x256 output tile per work-group (4 wavefronts, 2x2, 128x128 each = 4x4 MFMA tiles, 256
// accumulator registers per lane), K step 32, four LDS stages of 32 KB (128 of the CU's 160 KB).  Operand
// tiles go from HBM/L2 straight into LDS with global_load_lds_dwordx4 (no staging registers, no ds_write);
// the loads of K tile t+3 are issued before the MFMAs of tile t.  A wavefront-wide load deposits 64
// consecutive 16-byte chunks = 16 LDS rows of 64 B, so the bank-conflict swizzle (chunk ^ ((row>>1)&3)) is
// applied on the global-address side: each lane fetches the chunk that belongs at its LDS position.
// Rows beyond M or N are clamped to the last valid row (their products land in accumulators that are never
// stored), so the main loop has no bounds checks.  Work-groups are renumbered so that each XCD
// (blockIdx % 8) owns a contiguous band of tiles and re-reads operand panels from its own L2.
#include "common.hpp"

namespace mase {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256, BK = 32;
constexpr int kStages = 4;
constexpr int kGemmThreads = 256;
constexpr int kRowBytes = BK * 2;                 // 64
constexpr int kTileBytes = BM * kRowBytes;        // 16 KB per operand per stage
constexpr int kStageBytes = 2 * kTileBytes;       // A then B
constexpr int kWaveLoadsPerTile = kTileBytes / 1024 / 4;  // per wavefront per operand per stage = 4

struct GemmParams {
  const unsigned char* A;
  const unsigned char* B;
  const void* bias;
  void* C;
  int M, N, K;
  int out_dtype, bias_dtype;
  int tiles_m, tiles_n;
};

__device__ __forceinline__ int lds_off(int row, int chunk) {
  return row * kRowBytes + ((chunk ^ ((row >> 1) & 3)) << 4);
}

__device__ __forceinline__ float load_bias(const void* bias, int dt, int col) {
  if (dt == MASE_DT_F32) return ((const float*)bias)[col];
  if (dt == MASE_DT_BF16) return bits2f((uint32_t)((const uint16_t*)bias)[col] << 16);
  return f16_bits_to_f32(((const uint16_t*)bias)[col]);
}

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// one wavefront-wide 1 KB copy: lane i's 16 bytes at `g` go to LDS byte offset lds_base + 16*i
__device__ __forceinline__ void async_copy_16(const unsigned char* g, unsigned char* lds_base) {
  __builtin_amdgcn_global_load_lds((gptr_t)g, (lptr_t)lds_base, 16, 0, 0);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  // gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14 ; leave the others at max
  __builtin_amdgcn_s_waitcnt((N & 0xF) | (0x7 << 4) | (0xF << 8) | ((N >> 4) << 14));
}

__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_tn_kernel(GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  // XCD-aware tile numbering (see header comment), then groups of 8 tile rows
  int bid = blockIdx.x;
  const int total = p.tiles_m * p.tiles_n;
  if ((total & 7) == 0) bid = (bid & 7) * (total >> 3) + (bid >> 3);
  constexpr int GROUP_M = 8;
  const int in_group = GROUP_M * p.tiles_n;
  const int first_m = (bid / in_group) * GROUP_M;
  const int gsz = min(p.tiles_m - first_m, GROUP_M);
  const int tile_m = first_m + (bid % in_group) % gsz;
  const int tile_n = (bid % in_group) / gsz;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  // global side of the async copies: wave w fills row groups g = w + 4*j (16 rows each), j = 0..3
  const int cp_row = lane >> 2;                              // row inside the 16-row group
  const int cp_chunk = (lane & 3) ^ ((cp_row >> 1) & 3);     // chunk that belongs at LDS position lane&3
  const size_t ldb = (size_t)p.K * 2;                        // bytes per operand row
  const unsigned char* ga[kWaveLoadsPerTile];
  const unsigned char* gb[kWaveLoadsPerTile];
#pragma unroll
  for (int j = 0; j < kWaveLoadsPerTile; ++j) {
    const int r = (wave + 4 * j) * 16 + cp_row;
    ga[j] = p.A + (size_t)min(m0 + r, p.M - 1) * ldb + cp_chunk * 16;
    gb[j] = p.B + (size_t)min(n0 + r, p.N - 1) * ldb + cp_chunk * 16;
  }
  auto issue_tile = [&](int kt) {
    unsigned char* sa = lds + (kt % kStages) * kStageBytes;
    unsigned char* sb = sa + kTileBytes;
    const size_t koff = (size_t)kt * kRowBytes;
#pragma unroll
    for (int j = 0; j < kWaveLoadsPerTile; ++j) {
      async_copy_16(ga[j] + koff, sa + (wave + 4 * j) * 1024);
      async_copy_16(gb[j] + koff, sb + (wave + 4 * j) * 1024);
    }
  };

  f32x16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int nk = p.K / BK;
  constexpr int kAhead = kStages - 1;  // tiles in flight beyond the one being consumed
#pragma unroll
  for (int t = 0; t < kAhead; ++t)
    if (t < nk) issue_tile(t);

  const int frag_row = lane & 31;
  const int kgrp = lane >> 5;
  for (int kt = 0; kt < nk; ++kt) {
    // tile kt has landed once at most the loads of the tiles issued after it are outstanding
    const int newer = min(nk - 1 - kt, kAhead - 1);
    if (newer >= 2) wait_vmcnt<2 * 2 * kWaveLoadsPerTile>();
    else if (newer == 1) wait_vmcnt<2 * kWaveLoadsPerTile>();
    else wait_vmcnt<0>();
    // everyone's part of tile kt is in LDS, and everyone is done reading tile kt-1.  A bare s_barrier: the
    // fence of __syncthreads() would also wait for the copies of the tiles still in flight.
    __builtin_amdgcn_s_barrier();
    if (kt + kAhead < nk) issue_tile(kt + kAhead);

    const unsigned char* sa = lds + (kt % kStages) * kStageBytes + (wm * 128) * kRowBytes;
    const unsigned char* sb = lds + (kt % kStages) * kStageBytes + kTileBytes + (wn * 128) * kRowBytes;
#pragma unroll
    for (int s = 0; s < BK / 16; ++s) {
      bf16x8_t a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a[i] = __builtin_bit_cast(bf16x8_t, *(const uint4*)(sa + lds_off(i * 32 + frag_row, s * 2 + kgrp)));
        b[i] = __builtin_bit_cast(bf16x8_t, *(const uint4*)(sb + lds_off(i * 32 + frag_row, s * 2 + kgrp)));
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
  }

  // epilogue: acc[i][j][r] is C[row, col] with row = i*32 + (r/4)*8 + kgrp*4 + r%4, col = j*32 + lane%32
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int col = n0 + wn * 128 + j * 32 + frag_row;
    if (col >= p.N) continue;
    const float bv = p.bias ? load_bias(p.bias, p.bias_dtype, col) : 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * 128 + i * 32 + (r >> 2) * 8 + kgrp * 4 + (r & 3);
        if (row >= p.M) continue;
        const float v = acc[i][j][r] + bv;
        const size_t o = (size_t)row * p.N + col;
        if (p.out_dtype == MASE_DT_F32) ((float*)p.C)[o] = v;
        else if (p.out_dtype == MASE_DT_BF16) ((uint16_t*)p.C)[o] = (uint16_t)f32_to_bf16_bits(v);
        else ((uint16_t*)p.C)[o] = (uint16_t)f32_to_f16_bits(v);
      }
    }
  }
}

}  // namespace
}  // namespace mase

extern "C" int mase_gemm_bf16_tn(const void* A, const void* B, const void* bias, void* C, size_t M, size_t N, size_t K,
                                 int out_dtype, int bias_dtype, void* stream) {
  using namespace mase;
  if (M == 0 || N == 0) return MASE_OK;
  if (A == nullptr || B == nullptr || C == nullptr) return MASE_ERR_NULL;
  if (K == 0 || (K % BK) != 0 || M > (1u << 30) || N > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  if (!aligned16(A) || !aligned16(B)) return MASE_ERR_ALIGN;
  if (out_dtype < 0 || out_dtype > 2 || (bias != nullptr && (bias_dtype < 0 || bias_dtype > 2))) return MASE_ERR_DTYPE;
  GemmParams p;
  p.A = (const unsigned char*)A;
  p.B = (const unsigned char*)B;
  p.bias = bias;
  p.C = C;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.out_dtype = out_dtype;
  p.bias_dtype = bias_dtype;
  p.tiles_m = (int)((M + BM - 1) / BM);
  p.tiles_n = (int)((N + BN - 1) / BN);
  static bool attr_set = false;
  const size_t lds_bytes = (size_t)kStages * kStageBytes;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)gemm_bf16_tn_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds_bytes) != hipSuccess)
      return MASE_ERR_LAUNCH;
    attr_set = true;
  }
  hipLaunchKernelGGL(gemm_bf16_tn_kernel, dim3((unsigned)(p.tiles_m * p.tiles_n)), dim3(kGemmThreads), lds_bytes,
                     (hipStream_t)stream, p);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}
