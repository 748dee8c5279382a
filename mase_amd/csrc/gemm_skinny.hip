// C[M,N] = A[M,K] * B[N,K]^T (+ bias[N]) for few rows of A (M <= 128): the token-by-token shape of serving, where
// the product is bound by streaming the weight matrix B once from HBM, not by the matrix cores.
//
// The 256x256-tile kernel of gemm_bf16.hip would put such a product on N/256 CUs and walk K serially.  Here the
// work is cut into (32 weight rows) x (a K range) per wavefront.  A wavefront streams its slab of B, and the
// matching K range of up to 32 rows of A, through a private ring of LDS stages with global_load_lds_dwordx4
// (whole 128-byte lines per row, several stages in flight to cover the HBM latency; no barrier anywhere: nothing
// is shared between wavefronts), multiplies with v_mfma_f32_32x32x16_bf16 and writes a 32 x M partial result;
// a second small kernel adds the partial results of the K ranges in a fixed order (deterministic, no atomics),
// adds the bias and converts.  More than 32 rows of A take one pass per group of 32 (B then comes from the
// last-level cache on the later passes).
#include "common.hpp"

namespace mase {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void* lptr_t;

constexpr int kSkinnyThreads = 256;   // 4 wavefronts = 4 slabs of 32 weight rows, same K range
constexpr int kSkChunk = 64;          // K elements per chunk: one 128-byte line per row
// XC = async copies that carry the rows of A (8 rows each): 1..4.  A stage holds the B slab chunk (4 KB) and XC KB
// of A; the ring is as deep as 32 KB per wavefront allow (6 stages for up to 8 rows of A, 4 for 32).
template <int XC>
struct SkGeom {
  static constexpr int kStageBytes = 4096 + XC * 1024;
  static constexpr int kStages = (32 * 1024) / kStageBytes;
  static constexpr int kCopies = 4 + XC;                       // async copies per chunk per wavefront
  static constexpr int kLdsBytes = 4 * kStages * kStageBytes;  // per work-group of 4 wavefronts
};

struct SkinnyParams {
  const unsigned char* A;   // [M, K] bf16, M <= 32 (this pass's rows)
  const unsigned char* B;   // [N, K] bf16
  float* P;                 // [KS, M, N] fp32 partial results
  int M, N, K;
  int kc;                   // K elements per split (multiple of 64)
};

// as in gemm_bf16.hip: 16-byte chunk `chunk` of row `row` (rows of 128 bytes), conflict-free for ds_read_b128
__device__ __forceinline__ int sk_lds_off(int row, int chunk) { return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4); }

// one wavefront-wide 1 KB async copy (issued from inline assembly and tracked by hand with s_waitcnt vmcnt, for the
// reasons given in gemm_bf16.hip); M0 = LDS address, nothing else in this kernel uses M0
__device__ __forceinline__ void sk_async_copy(const unsigned char* base, uint32_t off, uint32_t lds_addr) {
  const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(m0v) : "memory");
}

template <int N>
__device__ __forceinline__ void sk_wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 0xF) | (0x7 << 4) | (0xF << 8) | ((N >> 4) << 14));
}

template <int XC>
__global__ __launch_bounds__(kSkinnyThreads) void gemm_skinny_partial_kernel(SkinnyParams p) {
  using G = SkGeom<XC>;
  constexpr int kSkStages = G::kStages, kSkStageBytes = G::kStageBytes, kSkCopies = G::kCopies;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int r = lane & 31, g = lane >> 5;
  const int n0 = ((int)blockIdx.x * 4 + wave) * 32;
  if (n0 >= p.N) return;  // whole wavefront; there is no barrier in this kernel
  const int ks = blockIdx.y;
  const size_t ld = (size_t)p.K * 2;
  // copy j (0..3) of an operand moves rows 8j .. 8j+7: lane -> row 8j + lane/8, LDS position lane%8
  uint32_t offb[4], offa[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = 8 * j + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    offb[j] = (uint32_t)((size_t)min(n0 + row, p.N - 1) * ld) + chunk * 16;
    offa[j] = (uint32_t)((size_t)min(row, p.M - 1) * ld) + chunk * 16;
  }
  const unsigned char* bbase = p.B + (size_t)ks * p.kc * 2;
  const unsigned char* abase = p.A + (size_t)ks * p.kc * 2;
  unsigned char* ring = lds + wave * (kSkStages * kSkStageBytes);
  const uint32_t ring_addr = (uint32_t)(uintptr_t)(lptr_t)ring;
  const int chunks = p.kc / kSkChunk;
  auto issue = [&](int c) __attribute__((always_inline)) {  // chunk c (clamped: past the end re-copies the last chunk)
    const int cc = min(c, chunks - 1);
    const uint32_t st = ring_addr + (uint32_t)((c % kSkStages) * kSkStageBytes);
#pragma unroll
    for (int j = 0; j < 4; ++j) sk_async_copy(bbase + (size_t)cc * 128, offb[j], st + j * 1024);
#pragma unroll
    for (int j = 0; j < XC; ++j) sk_async_copy(abase + (size_t)cc * 128, offa[j], st + 4096 + j * 1024);
  };

  f32x16_t acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
  for (int c = 0; c < kSkStages - 1; ++c) issue(c);
  for (int c = 0; c < chunks; ++c) {
    // the stage of chunk c-1 is free: its fragments were consumed by the MFMAs of the previous iteration
    issue(c + kSkStages - 1);
    sk_wait_vmcnt<(kSkStages - 1) * kSkCopies>();  // chunk c has landed; the later ones may be in flight
    const unsigned char* st = ring + (c % kSkStages) * kSkStageBytes;
    uint4 w[4], x[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      w[i] = *(const uint4*)(st + sk_lds_off(r, 2 * i + g));
      x[i] = *(const uint4*)(st + 4096 + sk_lds_off(min(r, 8 * XC - 1), 2 * i + g));
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, w[i]), __builtin_bit_cast(bf16x8_t, x[i]),
                                                    acc, 0, 0, 0);
  }
  sk_wait_vmcnt<0>();  // no copy may still be in flight towards LDS when the wavefront retires
  // acc[q*4 + j] = sum_k B[n0 + q*8 + g*4 + j][k] * A[r][k]: for this lane's row m = r of A, four consecutive
  // columns n per q
  float* out = p.P + (size_t)ks * p.M * p.N;
  const int m = r;
  if (m < p.M) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = n0 + q * 8 + g * 4;
      float* o = out + (size_t)m * p.N + n;
      if (n + 3 < p.N && (p.N & 3) == 0) {
        *(float4*)o = make_float4(acc[q * 4], acc[q * 4 + 1], acc[q * 4 + 2], acc[q * 4 + 3]);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (n + j < p.N) o[j] = acc[q * 4 + j];
      }
    }
  }
}

__device__ __forceinline__ float skinny_bias(const void* bias, int dt, int col) {
  if (dt == MASE_DT_F32) return ((const float*)bias)[col];
  if (dt == MASE_DT_BF16) return bits2f((uint32_t)((const uint16_t*)bias)[col] << 16);
  return f16_bits_to_f32(((const uint16_t*)bias)[col]);
}

// C[m][n] = sum over the K ranges, in order, of P[ks][m][n]  (+ bias[n]), converted to the output dtype
template <int OUT_DT>
__global__ __launch_bounds__(256) void gemm_skinny_reduce_kernel(const float* __restrict__ P, void* __restrict__ C,
                                                                 const void* __restrict__ bias, int bias_dtype,
                                                                 size_t mn, int N, int splits) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= mn) return;
  float s = 0.0f;
  for (int k = 0; k < splits; ++k) s += P[(size_t)k * mn + i];
  if (bias != nullptr) s += skinny_bias(bias, bias_dtype, (int)(i % (size_t)N));
  if constexpr (OUT_DT == MASE_DT_F32) ((float*)C)[i] = s;
  else if constexpr (OUT_DT == MASE_DT_BF16) ((uint16_t*)C)[i] = (uint16_t)f32_to_bf16_bits(s);
  else ((uint16_t*)C)[i] = (uint16_t)f32_to_f16_bits(s);
}

// K ranges: enough of them that the machine is filled (about 8 wavefronts per CU), each a whole number of
// 64-element chunks, and all equal
int skinny_splits(int M, int N, int K, int n_cu) {
  const int slabs = (N + 31) / 32;
  const int chunks = K / 64;
  int want = (8 * n_cu + slabs - 1) / slabs;
  // the partial results cost splits * rows * N * 8 bytes of traffic: keep that below a quarter of B's bytes
  const int rows = M < 32 ? M : 32;
  const int cap = K / (16 * rows);
  if (want > cap) want = cap;
  if (want < 1) want = 1;
  int best = 1;
  for (int s = 1; s <= chunks && s <= 64; ++s)
    if (chunks % s == 0 && s <= want) best = s;
  return best;
}

int skinny_cu_count() {
  static int n_cu = 0;
  if (n_cu == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return -1;
    n_cu = prop.multiProcessorCount;
  }
  return n_cu;
}

}  // namespace
}  // namespace mase

extern "C" size_t mase_gemm_bf16_skinny_workspace_bytes(size_t M, size_t N, size_t K) {
  using namespace mase;
  if (M == 0 || N == 0 || K == 0 || (K % 64) != 0 || M > 128) return 0;
  const int n_cu = skinny_cu_count();
  if (n_cu <= 0) return 0;
  return (size_t)skinny_splits((int)M, (int)N, (int)K, n_cu) * M * N * sizeof(float);
}

extern "C" int mase_gemm_bf16_skinny(const void* A, const void* B, const void* bias, void* C, size_t M, size_t N, size_t K,
                                     int out_dtype, int bias_dtype, void* workspace, size_t workspace_bytes,
                                     void* stream) {
  using namespace mase;
  if (M == 0 || N == 0) return MASE_OK;
  if (A == nullptr || B == nullptr || C == nullptr) return MASE_ERR_NULL;
  if (K == 0 || (K % 64) != 0 || M > 128 || N > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  if ((unsigned long long)N * K * 2 > 0xFFFFFFFFull) return MASE_ERR_SHAPE;  // 32-bit byte offsets into B
  if (!aligned16(A) || !aligned16(B)) return MASE_ERR_ALIGN;
  if (out_dtype < 0 || out_dtype > 2 || (bias != nullptr && (bias_dtype < 0 || bias_dtype > 2))) return MASE_ERR_DTYPE;
  const int n_cu = skinny_cu_count();
  if (n_cu <= 0) return MASE_ERR_LAUNCH;
  const int splits = skinny_splits((int)M, (int)N, (int)K, n_cu);
  const size_t need = (size_t)splits * M * N * sizeof(float);
  if (workspace == nullptr || workspace_bytes < need || (((uintptr_t)workspace) & 15u) != 0) return MASE_ERR_WORKSPACE;
  hipStream_t st = (hipStream_t)stream;
  static bool attr_set = false;
  if (!attr_set) {
    const void* ks[4] = {(const void*)gemm_skinny_partial_kernel<1>, (const void*)gemm_skinny_partial_kernel<2>,
                         (const void*)gemm_skinny_partial_kernel<3>, (const void*)gemm_skinny_partial_kernel<4>};
    const int sz[4] = {SkGeom<1>::kLdsBytes, SkGeom<2>::kLdsBytes, SkGeom<3>::kLdsBytes, SkGeom<4>::kLdsBytes};
    for (int i = 0; i < 4; ++i)
      if (hipFuncSetAttribute(ks[i], hipFuncAttributeMaxDynamicSharedMemorySize, sz[i]) != hipSuccess)
        return MASE_ERR_LAUNCH;
    attr_set = true;
  }
  const dim3 grid((unsigned)(((N + 31) / 32 + 3) / 4), (unsigned)splits), block(kSkinnyThreads);
  SkinnyParams p;
  p.B = (const unsigned char*)B;
  p.N = (int)N;
  p.K = (int)K;
  p.kc = (int)K / splits;
  // one pass per group of 32 rows of A; the partial results of a group form a [splits, rows, N] block, and the
  // blocks of successive groups are laid out so that together they read as [splits, M, N] per group offset
  for (size_t m0 = 0; m0 < M; m0 += 32) {
    const size_t rows = (M - m0 < 32) ? (M - m0) : 32;
    p.A = (const unsigned char*)A + m0 * K * 2;
    p.P = (float*)workspace + (size_t)splits * m0 * N;
    p.M = (int)rows;
    const int xc = (int)(rows + 7) / 8;
    if (xc == 1) hipLaunchKernelGGL(gemm_skinny_partial_kernel<1>, grid, block, SkGeom<1>::kLdsBytes, st, p);
    else if (xc == 2) hipLaunchKernelGGL(gemm_skinny_partial_kernel<2>, grid, block, SkGeom<2>::kLdsBytes, st, p);
    else if (xc == 3) hipLaunchKernelGGL(gemm_skinny_partial_kernel<3>, grid, block, SkGeom<3>::kLdsBytes, st, p);
    else hipLaunchKernelGGL(gemm_skinny_partial_kernel<4>, grid, block, SkGeom<4>::kLdsBytes, st, p);
    const size_t mn_g = rows * N;
    const dim3 rgrid_g((unsigned)blocks_for(mn_g, 256));
    void* Cg = (unsigned char*)C + m0 * N * (out_dtype == MASE_DT_F32 ? 4 : 2);
    if (out_dtype == MASE_DT_F32)
      hipLaunchKernelGGL(gemm_skinny_reduce_kernel<MASE_DT_F32>, rgrid_g, dim3(256), 0, st, p.P, Cg, bias, bias_dtype, mn_g, (int)N, splits);
    else if (out_dtype == MASE_DT_BF16)
      hipLaunchKernelGGL(gemm_skinny_reduce_kernel<MASE_DT_BF16>, rgrid_g, dim3(256), 0, st, p.P, Cg, bias, bias_dtype, mn_g, (int)N, splits);
    else
      hipLaunchKernelGGL(gemm_skinny_reduce_kernel<MASE_DT_F16>, rgrid_g, dim3(256), 0, st, p.P, Cg, bias, bias_dtype, mn_g, (int)N, splits);
  }
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}
