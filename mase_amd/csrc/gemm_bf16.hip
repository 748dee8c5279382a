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
// accumulator registers per lane), K step 64 so that every operand row of a tile is one full 128-byte cache
// line (64-byte rows made the L1 fetch every line twice and bound the loop), two LDS stages of 64 KB.
// Operand tiles go from HBM/L2 straight into LDS with global_load_lds_dwordx4 (no staging registers, no
// ds_write); the copies of K tile t+2 are issued while the last MFMAs of tile t execute.  A wavefront-wide
// load deposits 64 consecutive 16-byte chunks = 8 LDS rows of 128 B, so the bank-conflict swizzle is applied
// on the global-address side: each lane fetches the chunk that belongs at its LDS position.  The swizzle
// is chunk ^ ((row>>1)&7): this LDS serves a ds_read_b128 sixteen lanes at a time out of 64 four-byte
// banks, so the 16-byte slots (address/16 mod 16) of 16 consecutive rows must all differ; rows of equal
// parity share a 128-byte half of the 256-byte bank period and get distinct slots from the XOR.
// Rows beyond M or N are clamped to the last valid row (their products land in accumulators that are never
// stored), so the main loop has no bounds checks.  Work-groups are renumbered so that each XCD
// (blockIdx % 8) owns a contiguous band of tiles and re-reads operand panels from its own L2.
#include "common.hpp"

namespace mase {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kStages = 2;
constexpr int kGemmThreads = 256;
constexpr int kRowBytes = BK * 2;                 // 128: one cache line per operand row per K tile
constexpr int kTileBytes = BM * kRowBytes;        // 32 KB per operand per stage
constexpr int kStageBytes = 2 * kTileBytes;       // A then B
constexpr int kWaveLoadsPerTile = kTileBytes / 1024 / 4;  // per wavefront per operand per stage = 8
constexpr int kLoadsPerTile = 2 * kWaveLoadsPerTile;      // async copies one wavefront issues per K tile = 16
constexpr int kSteps = BK / 16;                   // MFMA K steps per tile = 4

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
  return row * kRowBytes + ((chunk ^ ((row >> 1) & 7)) << 4);
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

template <int OUT_DT>
__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_tn_kernel(GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  // XCD-aware tile numbering (see header comment), then groups of 8 tile rows
  int bid = blockIdx.x;
  const int total = p.tiles_m * p.tiles_n;
#ifndef MASE_GEMM_DBG_NOXCD
  if ((total & 7) == 0) bid = (bid & 7) * (total >> 3) + (bid >> 3);
#endif
#ifndef MASE_GEMM_GROUP_M
#define MASE_GEMM_GROUP_M 4
#endif
  constexpr int GROUP_M = MASE_GEMM_GROUP_M;
  const int in_group = GROUP_M * p.tiles_n;
  const int first_m = (bid / in_group) * GROUP_M;
  const int gsz = min(p.tiles_m - first_m, GROUP_M);
  const int tile_m = first_m + (bid % in_group) % gsz;
  const int tile_n = (bid % in_group) / gsz;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  // global side of the async copies: wave w fills row groups g = w + 4*j (8 rows of 128 B each), j = 0..7
  const int cp_row = lane >> 3;  // row inside the 8-row group
  const size_t ldb = (size_t)p.K * 2;  // bytes per operand row
  const unsigned char* ga[kWaveLoadsPerTile];
  const unsigned char* gb[kWaveLoadsPerTile];
#pragma unroll
  for (int j = 0; j < kWaveLoadsPerTile; ++j) {
    const int r = (wave + 4 * j) * 8 + cp_row;
    const int cp_chunk = (lane & 7) ^ ((r >> 1) & 7);  // chunk that belongs at LDS position lane&7 of row r
    ga[j] = p.A + (size_t)min(m0 + r, p.M - 1) * ldb + cp_chunk * 16;
    gb[j] = p.B + (size_t)min(n0 + r, p.N - 1) * ldb + cp_chunk * 16;
  }
  // Tile numbers past the end are clamped to the last tile: the copy then lands in a stage that nobody
  // reads any more, which keeps the main loop free of branches (and the vmcnt bookkeeping uniform).
  const int nk = p.K / BK;
  // copy number c (0..15) of K tile kt: row group c/2 of A (even c) or B (odd c)
  auto issue_copy = [&](int kt, int c) {
    unsigned char* st = lds + (kt % kStages) * kStageBytes + (c & 1) * kTileBytes;
    const size_t koff = (size_t)min(kt, nk - 1) * kRowBytes;
    const int j = c >> 1;
    async_copy_16(((c & 1) ? gb[j] : ga[j]) + koff, st + (wave + 4 * j) * 1024);
  };

  f32x16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

#pragma unroll
  for (int c = 0; c < kLoadsPerTile; ++c) issue_copy(0, c);
#pragma unroll
  for (int c = 0; c < kLoadsPerTile; ++c) issue_copy(1, c);

  const int frag_row = lane & 31;
  const int kgrp = lane >> 5;
  // fragment f (0..3: A row tile f, 4..7: B column tile f-4) of K step s of tile kt
  auto load_frag = [&](int kt, int s, int f) -> bf16x8_t {
    const unsigned char* st = lds + (kt % kStages) * kStageBytes +
                              ((f < 4) ? (wm * 128) * kRowBytes : kTileBytes + (wn * 128) * kRowBytes);
    return __builtin_bit_cast(bf16x8_t, *(const uint4*)(st + lds_off((f & 3) * 32 + frag_row, s * 2 + kgrp)));
  };

  // Software pipeline, written out instruction by instruction and pinned with scheduling barriers, because a
  // wavefront issues in order: an MFMA occupies the matrix pipe for 32 cycles, and whatever else has to be
  // issued (LDS reads of the next K step, async copies of the tile after next) must sit *between* MFMAs to
  // be free.  Per K tile (4 steps of 16 MFMAs, fragment sets ping-pong between fr[0] and fr[1]):
  //   steps 0..2: MFMAs of step s, interleaved with the 8 LDS reads of step s+1
  //   hand-over (after the MFMAs of step 2 are issued): this wavefront's reads of the tile are complete
  //     (lgkmcnt) and its copies of tile kt+1 have landed (vmcnt); barrier -> tile kt+1 is visible to all
  //     and nobody reads tile kt's stage any more
  //   step 3: MFMAs, interleaved with the LDS reads of step 0 of tile kt+1 and the 16 copies of tile kt+2
  //     (into the stage just vacated), which then have a whole tile's worth of MFMAs to land
  // The barrier is a bare s_barrier: the fence of __syncthreads() would wait for all copies in flight.
  bf16x8_t fr[2][8];
#ifdef MASE_GEMM_DBG_CLOCK
  const long long dbg_c0 = clock64(), dbg_w0 = wall_clock64();
#endif
  wait_vmcnt<kLoadsPerTile>();  // tile 1 may still be in flight
  asm volatile("s_barrier" ::: "memory");
#pragma unroll
  for (int f = 0; f < 8; ++f) fr[0][f] = load_frag(0, 0, f);
  for (int kt = 0; kt < nk; ++kt) {
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      const int cur = s & 1, nxt = cur ^ 1;
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        acc[t >> 2][t & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[cur][t >> 2], fr[cur][4 + (t & 3)],
                                                                     acc[t >> 2][t & 3], 0, 0, 0);
        if (s < kSteps - 1) {
          if (t < 8) fr[nxt][t] = load_frag(kt, s + 1, t);
        } else {
          if (t < 8) {
            fr[nxt][t] = load_frag(kt + 1, 0, t);
          } else {  // the 16 copies of tile kt+2, two per MFMA slot, into the stage just vacated
#ifndef MASE_GEMM_DBG_NOLOAD
            issue_copy(kt + 2, 2 * (t - 8));
            issue_copy(kt + 2, 2 * (t - 8) + 1);
#endif
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (s == kSteps - 2) {
        // all LDS reads of tile kt are in registers; the copies of tile kt+1 (issued one tile ago) have landed
        wait_vmcnt<0>();
#ifndef MASE_GEMM_DBG_NOBARRIER
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#endif
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  wait_vmcnt<0>();  // no copy may still be in flight towards LDS when the work-group retires
#ifdef MASE_GEMM_DBG_CLOCK
  const long long dbg_c1 = clock64(), dbg_w1 = wall_clock64();
#endif

  // Epilogue.  acc[i][j][r] is C[row, col] with row = i*32 + (r/4)*8 + kgrp*4 + r%4, col = j*32 + lane%32:
  // stored directly that would be 256 four-byte stores per lane.  Instead each wavefront transposes one
  // 32-row band at a time through its own LDS slice (32 x 128 fp32, rows padded to 136 floats so that the
  // two half-waves of a ds_write_b32 hit disjoint banks) and writes 4 consecutive columns per lane: a
  // half-wave covers 512 contiguous bytes of a C row.  LDS ops of one wavefront complete in order, so the
  // slice needs no barrier; the one barrier below only separates it from the operand stages.
  asm volatile("s_barrier" ::: "memory");
  constexpr int kStgStride = 136;
  float* stg = (float*)(lds + wave * (32 * kStgStride * 4));
  const int c4 = (lane & 31) * 4;                      // first of this lane's 4 columns inside the wave tile
  const int col0 = n0 + wn * 128 + c4;
  const bool vec_ok = ((p.N & 3) == 0) && ((((uintptr_t)p.C) & 15u) == 0);
  float bv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (p.bias != nullptr) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (col0 + e < p.N) bv[e] = load_bias(p.bias, p.bias_dtype, col0 + e);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        stg[((r >> 2) * 8 + kgrp * 4 + (r & 3)) * kStgStride + j * 32 + frag_row] = acc[i][j][r];
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int rr = q * 2 + kgrp;
      const int row = m0 + wm * 128 + i * 32 + rr;
      const float4 v4 = *(const float4*)(stg + rr * kStgStride + c4);
      const float v[4] = {v4.x + bv[0], v4.y + bv[1], v4.z + bv[2], v4.w + bv[3]};
      if (row >= p.M) continue;
      const size_t o = (size_t)row * p.N + col0;
      if (vec_ok && col0 + 3 < p.N) {
        if constexpr (OUT_DT == MASE_DT_F32) {
          *(float4*)((float*)p.C + o) = make_float4(v[0], v[1], v[2], v[3]);
        } else if constexpr (OUT_DT == MASE_DT_BF16) {
          uint2 w;
          w.x = f32_to_bf16_bits(v[0]) | (f32_to_bf16_bits(v[1]) << 16);
          w.y = f32_to_bf16_bits(v[2]) | (f32_to_bf16_bits(v[3]) << 16);
          *(uint2*)((uint16_t*)p.C + o) = w;
        } else {
          uint2 w;
          w.x = f32_to_f16_bits(v[0]) | (f32_to_f16_bits(v[1]) << 16);
          w.y = f32_to_f16_bits(v[2]) | (f32_to_f16_bits(v[3]) << 16);
          *(uint2*)((uint16_t*)p.C + o) = w;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (col0 + e >= p.N) continue;
          if constexpr (OUT_DT == MASE_DT_F32) ((float*)p.C)[o + e] = v[e];
          else if constexpr (OUT_DT == MASE_DT_BF16) ((uint16_t*)p.C)[o + e] = (uint16_t)f32_to_bf16_bits(v[e]);
          else ((uint16_t*)p.C)[o + e] = (uint16_t)f32_to_f16_bits(v[e]);
        }
      }
    }
  }
#ifdef MASE_GEMM_DBG_CLOCK
  const long long dbg_c2 = clock64(), dbg_w2 = wall_clock64();
  if (blockIdx.x == 7 && tid == 0) {
    float* o = (float*)p.C;
    __threadfence();
    o[0] = (float)(dbg_c1 - dbg_c0); o[1] = (float)(dbg_w1 - dbg_w0);
    o[2] = (float)(dbg_c2 - dbg_c1); o[3] = (float)(dbg_w2 - dbg_w1);
  }
#endif
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
  const void* kernels[3] = {(const void*)gemm_bf16_tn_kernel<MASE_DT_F32>, (const void*)gemm_bf16_tn_kernel<MASE_DT_BF16>,
                            (const void*)gemm_bf16_tn_kernel<MASE_DT_F16>};
  if (!attr_set) {
    for (const void* k : kernels)
      if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess)
        return MASE_ERR_LAUNCH;
    attr_set = true;
  }
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n)), block(kGemmThreads);
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == MASE_DT_F32) hipLaunchKernelGGL(gemm_bf16_tn_kernel<MASE_DT_F32>, grid, block, lds_bytes, st, p);
  else if (out_dtype == MASE_DT_BF16) hipLaunchKernelGGL(gemm_bf16_tn_kernel<MASE_DT_BF16>, grid, block, lds_bytes, st, p);
  else hipLaunchKernelGGL(gemm_bf16_tn_kernel<MASE_DT_F16>, grid, block, lds_bytes, st, p);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}
