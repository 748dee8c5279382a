// C[M,N] = A[M,K] * B[N,K]^T (+ bias[N]) for few rows of A (M <= 128): the token-by-token shape of serving, where
// the product is bound by streaming the weight matrix B once from HBM, not by the matrix cores.
//
// The 256x256-tile kernel of gemm_bf16.hip would put such a product on N/256 CUs and walk K serially.  Here the
// work is cut into (32 weight rows) x (a K range) per wavefront.  A wavefront streams its slab of B, and the
// matching K range of up to 32 rows of A, through a private ring of LDS stages with global_load_lds_dwordx4
// (whole 128-byte lines per row, several stages in flight to cover the HBM latency; no barrier anywhere: nothing
// is shared between wavefronts), multiplies with v_mfma_f32_32x32x16_bf16 and writes a 32 x M partial result;
// a second small kernel adds the partial results of the K ranges in a fixed order (deterministic, no atomics),
// adds the bias and converts; with a single K range the first kernel does that itself and the second is not
// launched.  More than 32 rows of A take one pass per group of 32 (B then comes from the last-level cache on the
// later passes).
#include "common.hpp"

namespace mase {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void* lptr_t;

constexpr int kSkinnyThreads = 256;   // 4 wavefronts = 4 slabs of 32 weight rows, same K range
constexpr int kSkChunk = 64;          // K elements per chunk: one 128-byte line per row
// XC = async copies that carry the rows of A (8 rows each): 1..4.  A stage holds the B slab chunk (4 KB) and XC KB
// of A; the ring is as deep as 40 KB per wavefront allow (8 stages for up to 8 rows of A, 5 for 32).
template <int XC>
struct SkGeom {
  static constexpr int kStageBytes = 4096 + XC * 1024;
  static constexpr int kStages = (40 * 1024) / kStageBytes;
  static constexpr int kCopies = 4 + XC;                       // async copies per chunk per wavefront
  static constexpr int kLdsBytes = 4 * kStages * kStageBytes;  // per work-group of 4 wavefronts
};

// Where a kernel's 32 x M result goes.  With several K ranges: partial sums [range][M][N] in the workspace, which the
// reduce kernel adds in order.  With a single range the kernel finishes the job itself (C != null): the value the
// reduce kernel would compute from the one partial sum (0 + sum, + bias), converted and written to C, and no second
// launch.
struct SkinnyOut {
  float* P;           // [ranges, M, N] fp32 partial results
  void* C;            // [M, N] in out_dtype, or null
  const void* bias;   // [N] in bias_dtype, or null
  int out_dtype, bias_dtype;
};

__device__ __forceinline__ float skinny_bias(const void* bias, int dt, int col) {
  if (dt == MASE_DT_F32) return ((const float*)bias)[col];
  if (dt == MASE_DT_BF16) return bits2f((uint32_t)((const uint16_t*)bias)[col] << 16);
  return f16_bits_to_f32(((const uint16_t*)bias)[col]);
}

__device__ __forceinline__ float skinny_finish(const SkinnyOut& o, float sum, int col) {
  float s = 0.0f;
  s += sum;  // as the reduce kernel starts from zero: a sum of -0 comes out as +0 either way
  if (o.bias != nullptr) s += skinny_bias(o.bias, o.bias_dtype, col);
  return s;
}

__device__ __forceinline__ uint32_t skinny_to16(int dt, float v) {
  return dt == MASE_DT_BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v);
}

// element (m, n) of the result, from a lane that holds single elements
__device__ __forceinline__ void skinny_put(const SkinnyOut& o, int ks, int M, int N, int m, int n, float sum) {
  const size_t i = (size_t)m * N + n;
  if (o.C == nullptr) {
    o.P[(size_t)ks * M * N + i] = sum;
  } else {
    const float v = skinny_finish(o, sum, n);
    if (o.out_dtype == MASE_DT_F32) ((float*)o.C)[i] = v;
    else ((uint16_t*)o.C)[i] = (uint16_t)skinny_to16(o.out_dtype, v);
  }
}

// elements (m, n .. n + 3) of the result, from a lane that holds four consecutive columns
__device__ __forceinline__ void skinny_put4(const SkinnyOut& o, int ks, int M, int N, int m, int n, float s0, float s1,
                                            float s2, float s3) {
  if (n + 3 < N && (N & 3) == 0) {
    const size_t i = (size_t)m * N + n;
    if (o.C == nullptr) {
      *(float4*)(o.P + (size_t)ks * M * N + i) = make_float4(s0, s1, s2, s3);
    } else {
      const float v0 = skinny_finish(o, s0, n), v1 = skinny_finish(o, s1, n + 1), v2 = skinny_finish(o, s2, n + 2),
                  v3 = skinny_finish(o, s3, n + 3);
      if (o.out_dtype == MASE_DT_F32) {
        *(float4*)((float*)o.C + i) = make_float4(v0, v1, v2, v3);
      } else {
        const int dt = o.out_dtype;
        *(uint2*)((uint16_t*)o.C + i) = make_uint2(skinny_to16(dt, v0) | (skinny_to16(dt, v1) << 16),
                                                   skinny_to16(dt, v2) | (skinny_to16(dt, v3) << 16));
      }
    }
  } else {
    const float sv[4] = {s0, s1, s2, s3};
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (n + j < N) skinny_put(o, ks, M, N, m, n + j, sv[j]);
  }
}

struct SkinnyParams {
  const unsigned char* A;   // [M, K] bf16, M <= 32 (this pass's rows)
  const unsigned char* B;   // [N, K] bf16
  SkinnyOut o;
  int M, N, K;
  int kc;                   // K elements per K range (multiple of 64); the last range holds what is left of K
};

// as in gemm_bf16.hip: 16-byte chunk `chunk` of row `row` (rows of 128 bytes), conflict-free for ds_read_b128
__device__ __forceinline__ int sk_lds_off(int row, int chunk) { return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4); }

// one wavefront-wide 1 KB async copy (issued from inline assembly and tracked by hand with s_waitcnt vmcnt, for the
// reasons given in gemm_bf16.hip); M0 = LDS address, nothing else in this kernel uses M0
// (m0 is written inside the statement and not listed as clobbered: the compiler keeps no value in m0 across
// statements on this target, it reloads m0 before each use of its own, and rejects the name in a clobber list as a
// reserved register)
__device__ __forceinline__ void sk_async_copy(const unsigned char* base, uint32_t off, uint32_t lds_addr) {
  const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(m0v) : "memory");
}

// The empty statement behind the wait keeps the compiler from moving an LDS read of the copied data in front of it
// (the wait itself is not a memory operation to the compiler).
template <int N>
__device__ __forceinline__ void sk_wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 0xF) | (0x7 << 4) | (0xF << 8) | ((N >> 4) << 14));
  asm volatile("" ::: "memory");
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
  const int chunks = min(p.kc, p.K - ks * p.kc) / kSkChunk;
  // Work-group b walks its K range starting at chunk b mod chunks and wraps around (its four wavefronts stay in step
  // and share their reads of A).  Weight rows lie K*2 bytes apart,
  // for the usual K a power of two: wavefronts walking in step would all ask for the same few memory channels at any
  // moment (measured on 28672 x 8192: 4.3 TB/s, against 5.7 TB/s for K = 8448 or 7936); rotated, their requests
  // cover the whole period.  The order of a wavefront's sum is a fixed function of its position, so results stay
  // reproducible.
  const int rot = (int)((unsigned)blockIdx.x % (unsigned)chunks);
  auto issue = [&](int c) __attribute__((always_inline)) {  // chunk c (clamped: past the end re-copies the last chunk)
    int cc = min(c, chunks - 1) + rot;
    cc = cc >= chunks ? cc - chunks : cc;
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
  const int m = r;
  if (m < p.M) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
      skinny_put4(p.o, ks, p.M, p.N, m, n0 + q * 8 + g * 4, acc[q * 4], acc[q * 4 + 1], acc[q * 4 + 2], acc[q * 4 + 3]);
  }
}

// ---------------------------------------------------------------------------------------------
// The same product with B held as packed MXINT8: int8 codes [N, K] and one scale byte per 32 codes [N, K/32]
// (value = code * 2^(scale - 134), the packed outputs of the MXINT quantizer).  The weight stream is half the bytes of
// the bf16 image, which is what bounds this product.  A wavefront streams 128-element chunks of its 32 code rows (4 KB),
// their 4 scale bytes per row and the matching chunk of A through its LDS ring; codes become bf16 in registers:
// byte ^ 0x80 is the code plus 128 as an unsigned byte, v_cvt_f32_ubyte converts it, one fma subtracts the 128 and
// applies the block's power-of-two scale, and the exact product is truncated to bf16 (at most 8 significant bits).
// The MFMA operands are therefore the same bf16 values the bf16 path multiplies.  Scale bytes below 8 (weights under
// 2^-119) are treated as zero.
// ---------------------------------------------------------------------------------------------
constexpr int kSqChunk = 128;  // K elements per chunk: one 128-byte line of codes per row
constexpr int kSqWaves = 4;     // wavefronts (slabs of 32 weight rows) per work-group, as in the bf16 kernel
constexpr int kSqThreads = kSqWaves * 64;
template <int XC>
struct SqGeom {
  static constexpr int kCodeBytes = 32 * 128, kScaleBytes = 256, kABytes = XC * 8 * 256;
  static constexpr int kStageBytes = kCodeBytes + kScaleBytes + kABytes;
  static constexpr int kStages = ((160 / kSqWaves) * 1024) / kStageBytes;
  static constexpr int kCopies = 4 + 1 + 2 * XC;
  static constexpr int kLdsBytes = kSqWaves * kStages * kStageBytes;
};

struct SkinnyQParams {
  const unsigned char* A;    // [M, K] bf16, M <= 32
  const unsigned char* Bc;   // [N, K] int8 codes
  const unsigned char* Bs;   // [N, K/32] scale bytes
  SkinnyOut o;
  int M, N, K;
  int kc;                    // K elements per K range (multiple of 128); the last range holds what is left of K
};

__device__ __forceinline__ void sk_async_copy4(const unsigned char* base, uint32_t off, uint32_t lds_addr) {
  const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(off), "s"(base), "s"(m0v) : "memory");
}

// four codes of one dword -> two registers of two bf16 values each (code * scale, exact)
__device__ __forceinline__ void codes4_to_bf16(uint32_t c, float scale, float bias, uint32_t& lo, uint32_t& hi) {
  const uint32_t u = c ^ 0x80808080u;
  const float f0 = __builtin_fmaf((float)(u & 0xFFu), scale, bias);
  const float f1 = __builtin_fmaf((float)((u >> 8) & 0xFFu), scale, bias);
  const float f2 = __builtin_fmaf((float)((u >> 16) & 0xFFu), scale, bias);
  const float f3 = __builtin_fmaf((float)(u >> 24), scale, bias);
  lo = __builtin_amdgcn_perm(f2bits(f1), f2bits(f0), 0x07060302u);  // the upper halves: two bf16 values
  hi = __builtin_amdgcn_perm(f2bits(f3), f2bits(f2), 0x07060302u);
}

template <int XC>
__global__ __launch_bounds__(kSqThreads) void gemm_skinny_mxint8_partial_kernel(SkinnyQParams p) {
  using G = SqGeom<XC>;
  constexpr int S = G::kStages;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int r = lane & 31, g = lane >> 5;
  const int n0 = ((int)blockIdx.x * kSqWaves + wave) * 32;
  if (n0 >= p.N) return;  // whole wavefront; there is no barrier in this kernel
  const int ks = blockIdx.y;
  // codes: copy j (0..3) moves rows 8j .. 8j+7 (128 bytes each): lane -> row 8j + lane/8, LDS chunk position lane%8
  uint32_t offc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = 8 * j + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    offc[j] = (uint32_t)((size_t)min(n0 + row, p.N - 1) * (size_t)p.K) + chunk * 16;
  }
  // scales: lane -> the dword of row lane%32 for this chunk
  const uint32_t offs = (uint32_t)((size_t)min(n0 + r, p.N - 1) * (size_t)(p.K / 32));
  // A: copy j (0 .. 2*XC-1) moves rows 4j .. 4j+3 (256 bytes each): lane -> row 4j + lane/16, LDS chunk position lane%16
  uint32_t offa[2 * XC];
#pragma unroll
  for (int j = 0; j < 2 * XC; ++j) {
    const int row = 4 * j + (lane >> 4);
    const int chunk = (lane & 15) ^ (row & 15);
    offa[j] = (uint32_t)((size_t)min(row, p.M - 1) * (size_t)p.K * 2) + chunk * 16;
  }
  const unsigned char* cbase = p.Bc + (size_t)ks * p.kc;
  const unsigned char* sbase = p.Bs + (size_t)ks * (p.kc / 32);
  const unsigned char* abase = p.A + (size_t)ks * p.kc * 2;
  unsigned char* ring = lds + wave * (S * G::kStageBytes);
  const uint32_t ring_addr = (uint32_t)(uintptr_t)(lptr_t)ring;
  const int chunks = min(p.kc, p.K - ks * p.kc) / kSqChunk;
  const int rot = (int)((unsigned)blockIdx.x % (unsigned)chunks);  // rotated start, as in the bf16 kernel
  auto issue = [&](int c) __attribute__((always_inline)) {  // chunk c (clamped: past the end re-copies the last chunk)
    int cc = min(c, chunks - 1) + rot;
    cc = cc >= chunks ? cc - chunks : cc;
    const uint32_t st = ring_addr + (uint32_t)((c % S) * G::kStageBytes);
#pragma unroll
    for (int j = 0; j < 4; ++j) sk_async_copy(cbase + (size_t)cc * 128, offc[j], st + j * 1024);
    sk_async_copy4(sbase + (size_t)cc * 4, offs, st + G::kCodeBytes);
#pragma unroll
    for (int j = 0; j < 2 * XC; ++j)
      sk_async_copy(abase + (size_t)cc * 256, offa[j], st + G::kCodeBytes + G::kScaleBytes + j * 1024);
  };

  f32x16_t acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
  for (int c = 0; c < S - 1; ++c) issue(c);
  const int arow = min(r, 8 * XC - 1);
  for (int c = 0; c < chunks; ++c) {
    issue(c + S - 1);
    sk_wait_vmcnt<(S - 1) * G::kCopies>();  // chunk c has landed; the later ones may be in flight
    const unsigned char* st = ring + (c % S) * G::kStageBytes;
    const uint32_t sc4 = *(const uint32_t*)(st + G::kCodeBytes + r * 4);  // the row's 4 scale bytes of this chunk
    float scale4[4], bias4[4];  // 2^(byte - 134) and the -128 * scale that removes the code offset, per block of 32
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const uint32_t sb = (sc4 >> (8 * b)) & 0xFFu;
      scale4[b] = bits2f(sb >= 8u ? (sb - 7u) << 23 : 0u);
      bias4[b] = -128.0f * scale4[b];
    }
#pragma unroll
    for (int step = 0; step < 8; ++step) {
      // 8 codes of row r at K offset step*16 + g*8, and the 8 values of A row r at the same K offset
      const uint2 cw = *(const uint2*)(st + r * 128 + ((step ^ ((r >> 1) & 7)) << 4) + g * 8);
      const uint4 xv = *(const uint4*)(st + G::kCodeBytes + G::kScaleBytes + arow * 256 + (((2 * step + g) ^ (arow & 15)) << 4));
      const float scale = scale4[step >> 1], bias = bias4[step >> 1];
      uint4 wv;
      codes4_to_bf16(cw.x, scale, bias, wv.x, wv.y);
      codes4_to_bf16(cw.y, scale, bias, wv.z, wv.w);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, wv), __builtin_bit_cast(bf16x8_t, xv), acc,
                                                    0, 0, 0);
    }
  }
  sk_wait_vmcnt<0>();  // no copy may still be in flight towards LDS when the wavefront retires
  const int m = r;
  if (m < p.M) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
      skinny_put4(p.o, ks, p.M, p.N, m, n0 + q * 8 + g * 4, acc[q * 4], acc[q * 4 + 1], acc[q * 4 + 2], acc[q * 4 + 3]);
  }
}


// The same kernel with the chunk of A shared by the work-group's four wavefronts instead of copied once per wavefront:
// a stage holds the four wavefronts' code chunks and scale bytes and ONE chunk of A, so the ring is about twice as deep
// in the same LDS and A crosses the vector-memory path once per work-group, at the price of one barrier per chunk (each
// wavefront copies a quarter of A's chunk, waits for its own copies and meets the others).  Used for more than 8 rows
// of A, where A's chunk is as large as a wavefront's codes or larger (measured on 28672 x 8192, reduction included:
// 16 rows 67 -> 57 us, 32 rows 76 -> 60 us; with 8 rows or fewer the kernel above, whose ring is then deeper, is as fast
// or faster).
template <int XC>
struct SqsGeom {
  static constexpr int kWaveBytes = 32 * 128 + 256;            // codes and scale bytes of one wavefront's chunk
  static constexpr int kABytes = XC * 8 * 256;                 // the chunk of A: 8 XC rows x 128 bf16
  static constexpr int kStageBytes = kSqWaves * kWaveBytes + kABytes;
  static constexpr int kACopies = (2 * XC + kSqWaves - 1) / kSqWaves;  // of A, per wavefront
  static constexpr int kCopies = 4 + 1 + kACopies;
  static constexpr int kFit = (160 * 1024) / kStageBytes;
  static constexpr int kStages = kFit > 8 ? 8 : kFit;
  static constexpr int kLdsBytes = kStages * kStageBytes;
};

template <int XC>
__global__ __launch_bounds__(kSqThreads) void gemm_skinny_mxint8_shared_kernel(SkinnyQParams p) {
  using G = SqsGeom<XC>;
  constexpr int S = G::kStages;
  static_assert((S - 1) * G::kCopies < 64, "outstanding copies must fit the 6-bit counter");
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int r = lane & 31, g = lane >> 5;
  const int n0 = ((int)blockIdx.x * kSqWaves + wave) * 32;  // rows beyond N are clamped: every wavefront reaches the barriers
  const int ks = blockIdx.y;
  uint32_t offc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = 8 * j + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    offc[j] = (uint32_t)((size_t)min(n0 + row, p.N - 1) * (size_t)p.K) + chunk * 16;
  }
  const uint32_t offs = (uint32_t)((size_t)min(n0 + r, p.N - 1) * (size_t)(p.K / 32));
  // A: copy j (0 .. 2*XC-1) moves rows 4j .. 4j+3 (256 bytes each); this wavefront issues copies wave, wave + 4, ...
  // clamped to the last one (a repeated copy writes the same bytes to the same place)
  uint32_t offa[G::kACopies];
  int ja[G::kACopies];
#pragma unroll
  for (int i = 0; i < G::kACopies; ++i) {
    ja[i] = min(wave + kSqWaves * i, 2 * XC - 1);
    const int row = 4 * ja[i] + (lane >> 4);
    const int chunk = (lane & 15) ^ (row & 15);
    offa[i] = (uint32_t)((size_t)min(row, p.M - 1) * (size_t)p.K * 2) + chunk * 16;
  }
  const unsigned char* cbase = p.Bc + (size_t)ks * p.kc;
  const unsigned char* sbase = p.Bs + (size_t)ks * (p.kc / 32);
  const unsigned char* abase = p.A + (size_t)ks * p.kc * 2;
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)lds;
  const int chunks = min(p.kc, p.K - ks * p.kc) / kSqChunk;
  const int rot = (int)((unsigned)blockIdx.x % (unsigned)chunks);
  constexpr int kOffA = kSqWaves * G::kWaveBytes;
  auto issue = [&](int c) __attribute__((always_inline)) {  // chunk c (clamped: past the end re-copies the last chunk)
    int cc = min(c, chunks - 1) + rot;
    cc = cc >= chunks ? cc - chunks : cc;
    const uint32_t st = lds_addr + (uint32_t)((c % S) * G::kStageBytes);
    const uint32_t mine = st + (uint32_t)(wave * G::kWaveBytes);
#pragma unroll
    for (int j = 0; j < 4; ++j) sk_async_copy(cbase + (size_t)cc * 128, offc[j], mine + j * 1024);
    sk_async_copy4(sbase + (size_t)cc * 4, offs, mine + 4096);
#pragma unroll
    for (int i = 0; i < G::kACopies; ++i) sk_async_copy(abase + (size_t)cc * 256, offa[i], st + kOffA + ja[i] * 1024);
  };

  f32x16_t acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
  for (int c = 0; c < S - 1; ++c) issue(c);
  const int arow = min(r, 8 * XC - 1);
  for (int c = 0; c < chunks; ++c) {
    // This wavefront's copies of chunk c have landed; behind the barrier so have the others' (their parts of A), and
    // every wavefront has finished reading chunk c - 1, whose stage the copies issued next overwrite.
    sk_wait_vmcnt<(S - 2) * G::kCopies>();
    __builtin_amdgcn_s_barrier();
    issue(c + S - 1);
    const unsigned char* st = lds + (c % S) * G::kStageBytes;
    const unsigned char* mine = st + wave * G::kWaveBytes;
    const uint32_t sc4 = *(const uint32_t*)(mine + 4096 + r * 4);  // the row's 4 scale bytes of this chunk
    float scale4[4], bias4[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const uint32_t sb = (sc4 >> (8 * b)) & 0xFFu;
      scale4[b] = bits2f(sb >= 8u ? (sb - 7u) << 23 : 0u);
      bias4[b] = -128.0f * scale4[b];
    }
#pragma unroll
    for (int step = 0; step < 8; ++step) {
      const uint2 cw = *(const uint2*)(mine + r * 128 + ((step ^ ((r >> 1) & 7)) << 4) + g * 8);
      const uint4 xv = *(const uint4*)(st + kOffA + arow * 256 + (((2 * step + g) ^ (arow & 15)) << 4));
      const float scale = scale4[step >> 1], bias = bias4[step >> 1];
      uint4 wv;
      codes4_to_bf16(cw.x, scale, bias, wv.x, wv.y);
      codes4_to_bf16(cw.y, scale, bias, wv.z, wv.w);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, wv), __builtin_bit_cast(bf16x8_t, xv), acc,
                                                    0, 0, 0);
    }
  }
  sk_wait_vmcnt<0>();  // no copy may still be in flight towards LDS when the wavefront retires
  const int m = r;
  if (m < p.M && n0 < p.N) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
      skinny_put4(p.o, ks, p.M, p.N, m, n0 + q * 8 + g * 4, acc[q * 4], acc[q * 4 + 1], acc[q * 4 + 2], acc[q * 4 + 3]);
  }
}

// ---------------------------------------------------------------------------------------------
// The few-rows product on packed MXFP operands with the block-scaled matrix instruction: activations as e4m3 / e5m2
// codes [M, K] and weights as e2m1 codes [N, K/2] (two per byte), one E8M0 scale byte per 32 elements each (the
// layout of mase_mxfp_pack).  The weight stream is 0.53 bytes per element, a quarter of the bf16 image, and the
// instruction dequantizes in hardware: nothing but the copies, four LDS reads and one MFMA per 64 elements of K.
// Operand roles as in gemm_mxfp.hip: A = activations (rows = tokens), B = weights (rows = the wavefront's 32 weight
// rows); a chunk is 128 elements of K = two instructions; the scale dword of a row holds the chunk's 4 block scales,
// lane group g uses byte 2*step + g.
// ---------------------------------------------------------------------------------------------
typedef int i32x8_t __attribute__((ext_vector_type(8)));
template <int XC>
struct SfGeom {
  static constexpr int kWBytes = 32 * 64, kScaleBytes = 256, kXBytes = XC * 8 * 128;
  static constexpr int kStageBytes = kWBytes + kScaleBytes + kXBytes + kScaleBytes;
  static constexpr int kFit = (40 * 1024) / kStageBytes;
  static constexpr int kStages = kFit > 8 ? 8 : kFit;   // outstanding copies stay below the 6-bit counter's range
  static constexpr int kCopies = 2 + 1 + XC + 1;
  static constexpr int kLdsBytes = 4 * kStages * kStageBytes;
};

struct SkinnyFParams {
  const unsigned char* Xc;   // [M, K] 8-bit activation codes, M <= 32
  const unsigned char* Xs;   // [M, K/32]
  const unsigned char* Wc;   // [N, K/2] e2m1 codes
  const unsigned char* Ws;   // [N, K/32]
  SkinnyOut o;
  int M, N, K;
  int kc;                    // K elements per K range (multiple of 128); the last range holds what is left of K
  int rotate;                // shared-chunk kernel: work-group b starts at chunk b mod chunks (pays with a single K range)
};

template <int XC, int CBSZ>
__global__ __launch_bounds__(kSkinnyThreads) void gemm_skinny_mxfp4_partial_kernel(SkinnyFParams p) {
  using G = SfGeom<XC>;
  constexpr int S = G::kStages;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int r = lane & 31, g = lane >> 5;
  const int n0 = ((int)blockIdx.x * 4 + wave) * 32;
  if (n0 >= p.N) return;  // whole wavefront; there is no barrier in this kernel
  const int ks = blockIdx.y;
  // weights: copy j (0, 1) moves rows 16j .. 16j+15 (64 bytes per row per chunk): lane -> row 16j + lane/4, position lane%4
  uint32_t offw[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int row = 16 * j + (lane >> 2);
    const int chunk = (lane & 3) ^ ((row >> 2) & 3);
    offw[j] = (uint32_t)((size_t)min(n0 + row, p.N - 1) * (size_t)(p.K / 2)) + chunk * 16;
  }
  // activations: copy j moves rows 8j .. 8j+7 (128 bytes per row per chunk)
  uint32_t offx[XC];
#pragma unroll
  for (int j = 0; j < XC; ++j) {
    const int row = 8 * j + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    offx[j] = (uint32_t)((size_t)min(row, p.M - 1) * (size_t)p.K) + chunk * 16;
  }
  // scales: lane -> the dword of row lane%32 for this chunk
  const uint32_t offws = (uint32_t)((size_t)min(n0 + r, p.N - 1) * (size_t)(p.K / 32));
  const uint32_t offxs = (uint32_t)((size_t)min(r, p.M - 1) * (size_t)(p.K / 32));
  const unsigned char* wbase = p.Wc + (size_t)ks * (p.kc / 2);
  const unsigned char* xbase = p.Xc + (size_t)ks * p.kc;
  const unsigned char* wsbase = p.Ws + (size_t)ks * (p.kc / 32);
  const unsigned char* xsbase = p.Xs + (size_t)ks * (p.kc / 32);
  unsigned char* ring = lds + wave * (S * G::kStageBytes);
  const uint32_t ring_addr = (uint32_t)(uintptr_t)(lptr_t)ring;
  const int chunks = min(p.kc, p.K - ks * p.kc) / 128;
  constexpr int kOffWs = G::kWBytes, kOffX = G::kWBytes + G::kScaleBytes, kOffXs = kOffX + G::kXBytes;
  auto issue = [&](int c) __attribute__((always_inline)) {  // chunk c (clamped: past the end re-copies the last chunk)
    const int cc = min(c, chunks - 1);
    const uint32_t st = ring_addr + (uint32_t)((c % S) * G::kStageBytes);
#pragma unroll
    for (int j = 0; j < 2; ++j) sk_async_copy(wbase + (size_t)cc * 64, offw[j], st + j * 1024);
    sk_async_copy4(wsbase + (size_t)cc * 4, offws, st + kOffWs);
#pragma unroll
    for (int j = 0; j < XC; ++j) sk_async_copy(xbase + (size_t)cc * 128, offx[j], st + kOffX + j * 1024);
    sk_async_copy4(xsbase + (size_t)cc * 4, offxs, st + kOffXs);
  };

  f32x16_t acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
  for (int c = 0; c < S - 1; ++c) issue(c);
  const int xrow = min(r, 8 * XC - 1);
  for (int c = 0; c < chunks; ++c) {
    issue(c + S - 1);
    sk_wait_vmcnt<(S - 1) * G::kCopies>();  // chunk c has landed; the later ones may be in flight
    const unsigned char* st = ring + (c % S) * G::kStageBytes;
    const int sw = (int)(*(const uint32_t*)(st + kOffWs + r * 4) >> (8 * g));
    const int sx = (int)(*(const uint32_t*)(st + kOffXs + r * 4) >> (8 * g));
#pragma unroll
    for (int step = 0; step < 2; ++step) {
      const uint4 x0 = *(const uint4*)(st + kOffX + xrow * 128 + (((step * 4 + g) ^ ((xrow >> 1) & 7)) << 4));
      const uint4 x1 = *(const uint4*)(st + kOffX + xrow * 128 + (((step * 4 + 2 + g) ^ ((xrow >> 1) & 7)) << 4));
      const uint4 w0 = *(const uint4*)(st + r * 64 + (((step * 2 + g) ^ ((r >> 2) & 3)) << 4));
      i32x8_t a, b;
      a[0] = (int)x0.x; a[1] = (int)x0.y; a[2] = (int)x0.z; a[3] = (int)x0.w;
      a[4] = (int)x1.x; a[5] = (int)x1.y; a[6] = (int)x1.z; a[7] = (int)x1.w;
      b[0] = (int)w0.x; b[1] = (int)w0.y; b[2] = (int)w0.z; b[3] = (int)w0.w;
      b[4] = 0; b[5] = 0; b[6] = 0; b[7] = 0;
      if (step == 0) acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc, CBSZ, 4, 0, sx, 0, sw);
      else acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc, CBSZ, 4, 2, sx, 2, sw);
    }
  }
  sk_wait_vmcnt<0>();  // no copy may still be in flight towards LDS when the wavefront retires
  // acc[q*4 + j] = C[token q*8 + g*4 + j][weight row n0 + r]
  const int n = n0 + r;
  if (n < p.N) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int m = q * 8 + g * 4 + j;
        if (m < p.M) skinny_put(p.o, ks, p.M, p.N, m, n, acc[q * 4 + j]);
      }
  }
}

// The same product with the chunk of activation codes shared by the work-group's four wavefronts.  The kernel above
// copies the activation chunk once per wavefront and chunk, which doubles its copy instructions, and reads the weight
// rows in 64-byte pieces.  Here a stage of the ring holds the four wavefronts' weight chunks of 256 elements of K
// (128 bytes per weight row, 4 copies per 4 KB, plus their scale bytes) and ONE chunk of activation codes and scales,
// of which each wavefront copies a quarter; one barrier per chunk makes the parts visible and frees the stage that
// the next copies overwrite.  Nothing grows with K, so one K range serves any K where the weight has enough rows to
// fill the chip, and every work-group starts up once (28672 x 8192, reduction included: 16 tokens 32 us, 32 tokens
// 36 us; a form that kept the activations of the whole K range in LDS needed two ranges for 16 tokens and four for 32:
// 38 and 48 us).  K % 256 == 0.
// Activation chunk layout: [row][256 B] with the 16-byte granule j of a row stored at position j ^ (row & 15), so that
// the 16 lanes a ds_read_b128 serves together (16 rows, same granule) fall into different banks; scales [32][8 B].
template <int XC>
struct SfsGeom {
  static constexpr int kWaveBytes = 4096 + 256;                 // weight codes and scale bytes of one wavefront's chunk
  static constexpr int kXBytes = XC * 8 * 256;                  // the chunk of activation codes: 8 XC rows x 256
  static constexpr int kXsBytes = 256;                          // their scale bytes: [32 rows][8]
  static constexpr int kStageBytes = 4 * kWaveBytes + kXBytes + kXsBytes;
  static constexpr int kXCopies = (2 * XC + 3) / 4;             // of the activation codes, per wavefront
  static constexpr int kCopies = 4 + 1 + kXCopies + 1;
  static constexpr int kFit = (160 * 1024) / kStageBytes;
  static constexpr int kStages = kFit > 8 ? 8 : kFit;
  static constexpr int kLdsBytes = kStages * kStageBytes;
};

template <int XC, int CBSZ>
__global__ __launch_bounds__(kSkinnyThreads) void gemm_skinny_mxfp4_shared_kernel(SkinnyFParams p) {
  using G = SfsGeom<XC>;
  constexpr int XR = 8 * XC, S = G::kStages;
  static_assert((S - 1) * G::kCopies < 64, "outstanding copies must fit the 6-bit counter");
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int r = lane & 31, g = lane >> 5;
  const int n0 = ((int)blockIdx.x * 4 + wave) * 32;  // rows beyond N are clamped: every wavefront reaches the barriers
  const int ks = blockIdx.y;
  const int nch = min(p.kc, p.K - ks * p.kc) / 256;
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)lds;
  // weights: copy j (0..3) moves rows 8j .. 8j+7 (128 bytes per row per chunk); scales: lane -> row lane/2, dword lane%2
  uint32_t offw[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = 8 * j + (lane >> 3);
    const int gran = (lane & 7) ^ ((row >> 1) & 7);
    offw[j] = (uint32_t)((size_t)min(n0 + row, p.N - 1) * (size_t)(p.K / 2)) + (uint32_t)(gran * 16);
  }
  const uint32_t offws = (uint32_t)((size_t)min(n0 + (lane >> 1), p.N - 1) * (size_t)(p.K / 32)) + (uint32_t)((lane & 1) * 4);
  // activations: copy q (0 .. 2*XC-1) moves rows 4q .. 4q+3 (256 bytes per row per chunk): lane -> row 4q + lane/16,
  // granule lane%16 stored at position granule ^ (row & 15); this wavefront issues copies wave, wave + 4, ... clamped to
  // the last one (a repeated copy writes the same bytes to the same place)
  uint32_t offx[G::kXCopies];
  int qx[G::kXCopies];
#pragma unroll
  for (int i = 0; i < G::kXCopies; ++i) {
    qx[i] = min(wave + 4 * i, 2 * XC - 1);
    const int row = 4 * qx[i] + (lane >> 4);
    const int gran = (lane & 15) ^ (row & 15);
    offx[i] = (uint32_t)((size_t)min(row, p.M - 1) * (size_t)p.K) + (uint32_t)(gran * 16);
  }
  const uint32_t offxs = (uint32_t)((size_t)min(lane >> 1, p.M - 1) * (size_t)(p.K / 32)) + (uint32_t)((lane & 1) * 4);
  const unsigned char* wbase = p.Wc + (size_t)ks * (p.kc / 2);
  const unsigned char* wsbase = p.Ws + (size_t)ks * (p.kc / 32);
  const unsigned char* xbase = p.Xc + (size_t)ks * p.kc;
  const unsigned char* xsbase = p.Xs + (size_t)ks * (p.kc / 32);
  // with one K range per weight row the work-groups start at different chunks, as in the bf16 kernel (16 tokens:
  // 34 -> 32 us); with several ranges the rotation gains nothing or costs time, so the host asks for it only with one
  const int rot = p.rotate ? (int)((unsigned)blockIdx.x % (unsigned)nch) : 0;
  constexpr int kOffX = 4 * G::kWaveBytes, kOffXs = kOffX + G::kXBytes;
  auto issue = [&](int c) __attribute__((always_inline)) {  // chunk c (clamped: past the end re-copies the last chunk)
    int cc = min(c, nch - 1) + rot;
    cc = cc >= nch ? cc - nch : cc;
    const uint32_t st = lds_addr + (uint32_t)((c % S) * G::kStageBytes);
    const uint32_t mine = st + (uint32_t)(wave * G::kWaveBytes);
#pragma unroll
    for (int j = 0; j < 4; ++j) sk_async_copy(wbase + (size_t)cc * 128, offw[j], mine + j * 1024);
    sk_async_copy4(wsbase + (size_t)cc * 8, offws, mine + 4096);
#pragma unroll
    for (int i = 0; i < G::kXCopies; ++i) sk_async_copy(xbase + (size_t)cc * 256, offx[i], st + kOffX + qx[i] * 1024);
    sk_async_copy4(xsbase + (size_t)cc * 8, offxs, st + kOffXs);  // by every wavefront alike: the counts stay uniform
  };
  f32x16_t acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
  for (int c = 0; c < S - 1; ++c) issue(c);
  const int xrow = min(r, XR - 1);
  const int xsw = xrow & 15, wsw = (r >> 1) & 7;
  for (int c = 0; c < nch; ++c) {
    // This wavefront's copies of chunk c have landed; behind the barrier so have the others' (their parts of the
    // activations), and every wavefront has finished reading chunk c - 1, whose stage the copies issued next overwrite.
    sk_wait_vmcnt<(S - 2) * G::kCopies>();
    __builtin_amdgcn_s_barrier();
    issue(c + S - 1);
    const unsigned char* st = lds + (c % S) * G::kStageBytes;
    const unsigned char* mine = st + wave * G::kWaveBytes;
    const unsigned char* xc = st + kOffX + xrow * 256;
    const uint2 swv = *(const uint2*)(mine + 4096 + r * 8);
    const uint2 sxv = *(const uint2*)(st + kOffXs + xrow * 8);
#pragma unroll
    for (int step = 0; step < 4; ++step) {
      const uint4 x0 = *(const uint4*)(xc + (((step * 4 + g) ^ xsw) << 4));
      const uint4 x1 = *(const uint4*)(xc + (((step * 4 + 2 + g) ^ xsw) << 4));
      const uint4 w0 = *(const uint4*)(mine + r * 128 + (((step * 2 + g) ^ wsw) << 4));
      const int sw = (int)((step < 2 ? swv.x : swv.y) >> (8 * g));
      const int sx = (int)((step < 2 ? sxv.x : sxv.y) >> (8 * g));
      i32x8_t a, b;
      a[0] = (int)x0.x; a[1] = (int)x0.y; a[2] = (int)x0.z; a[3] = (int)x0.w;
      a[4] = (int)x1.x; a[5] = (int)x1.y; a[6] = (int)x1.z; a[7] = (int)x1.w;
      b[0] = (int)w0.x; b[1] = (int)w0.y; b[2] = (int)w0.z; b[3] = (int)w0.w;
      b[4] = 0; b[5] = 0; b[6] = 0; b[7] = 0;
      if ((step & 1) == 0) acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc, CBSZ, 4, 0, sx, 0, sw);
      else acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc, CBSZ, 4, 2, sx, 2, sw);
    }
  }
  sk_wait_vmcnt<0>();  // no copy may still be in flight towards LDS when the wavefront retires
  // acc[q*4 + j] = C[token q*8 + g*4 + j][weight row n0 + r]
  const int n = n0 + r;
  if (n < p.N) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int m = q * 8 + g * 4 + j;
        if (m < p.M) skinny_put(p.o, ks, p.M, p.N, m, n, acc[q * 4 + j]);
      }
  }
}


int skinny_splits(int M, int N, int K, int n_cu);

// K elements per range when `chunks` chunks of `chunk` elements are cut into `splits` ranges: equal ranges of whole
// chunks, the last one possibly shorter
int range_elems(int K, int chunk, int splits) { return ((K / chunk) + splits - 1) / splits * chunk; }

// K ranges of the shared-chunk MXFP4 kernel: as many as skinny_splits would take, in whole 256-element chunks, none
// of them empty
int mxfp4_shared_splits(int M, int N, int K, int n_cu) {
  const int chunks = K / 256;
  const int want = skinny_splits(M, N, K / 2, n_cu);
  for (int s = want; s < chunks; ++s)
    if ((s - 1) * range_elems(K, 256, s) < K) return s;
  return chunks;
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

// Number of K ranges for a K of `K / 64` chunks (kernels with longer chunks pass a proportionally smaller K): ranges of
// ceil(chunks / ranges) chunks, the last one possibly shorter.  A work-group takes the CU's whole LDS, so the
// work-groups run in rounds of n_cu; the number of ranges is chosen for the smallest estimated time
//   rounds * (time of one work-group, proportional to its K range)  scaled by  (1 + partial-result traffic / B's bytes)
// where the partial results cost ranges * rows * N * 8 bytes against N * K * 2 of B; ties go to fewer ranges.
int skinny_splits(int M, int N, int K, int n_cu) {
  const int slabs = (N + 31) / 32;
  const int groups = (slabs + 3) / 4;
  const int chunks = K / 64;
  const int rows = M < 32 ? M : 32;
  int best = 1;
  double best_cost = 1e300;
  int last_s = 0;
  for (int len = chunks; len >= 1; --len) {  // candidate range lengths, longest first = fewest ranges first
    const int s = (chunks + len - 1) / len;
    if (s == last_s) continue;
    last_s = s;
    if (s > 64) break;
    const int range = (chunks + s - 1) / s;
    const long wgs = (long)groups * s;
    const long rounds = (wgs + n_cu - 1) / n_cu;
    const double overhead = 4.0 * s * rows / (double)K;
    // a short K range leaves the ring's start-up (a few chunks) exposed
    const double per_wg = (double)range + 4.0;
    const double cost = (double)rounds * per_wg * (1.0 + overhead);
    if (cost < best_cost * 0.999) { best_cost = cost; best = s; }
  }
  return best;
}

// The tail of a pass over up to 32 rows of A: with one K range and a 16-byte aligned output block the kernel has
// written C itself; otherwise the reduce kernel adds the ranges.
void skinny_launch_reduce(const SkinnyOut& o, void* Cg, const void* bias, int out_dtype, int bias_dtype, size_t rows, size_t N,
                          int splits, hipStream_t st) {
  if (o.C != nullptr) return;
  const size_t mn_g = rows * N;
  const dim3 rgrid_g((unsigned)blocks_for(mn_g, 256));
  if (out_dtype == MASE_DT_F32)
    hipLaunchKernelGGL(gemm_skinny_reduce_kernel<MASE_DT_F32>, rgrid_g, dim3(256), 0, st, o.P, Cg, bias, bias_dtype, mn_g, (int)N, splits);
  else if (out_dtype == MASE_DT_BF16)
    hipLaunchKernelGGL(gemm_skinny_reduce_kernel<MASE_DT_BF16>, rgrid_g, dim3(256), 0, st, o.P, Cg, bias, bias_dtype, mn_g, (int)N, splits);
  else
    hipLaunchKernelGGL(gemm_skinny_reduce_kernel<MASE_DT_F16>, rgrid_g, dim3(256), 0, st, o.P, Cg, bias, bias_dtype, mn_g, (int)N, splits);
}

SkinnyOut skinny_out(float* P, void* Cg, const void* bias, int out_dtype, int bias_dtype, int splits) {
  SkinnyOut o;
  o.P = P;
  o.C = (splits == 1 && aligned16(Cg)) ? Cg : nullptr;
  o.bias = bias;
  o.out_dtype = out_dtype;
  o.bias_dtype = bias_dtype;
  return o;
}

int skinny_cu_count() {
  const int n_cu = device_cu_count();
  return n_cu > 0 ? n_cu : -1;
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
  static std::atomic<uint64_t> attr_done{0};
  if (!device_setup_done(attr_done)) {
    const void* ks[4] = {(const void*)gemm_skinny_partial_kernel<1>, (const void*)gemm_skinny_partial_kernel<2>,
                         (const void*)gemm_skinny_partial_kernel<3>, (const void*)gemm_skinny_partial_kernel<4>};
    const int sz[4] = {SkGeom<1>::kLdsBytes, SkGeom<2>::kLdsBytes, SkGeom<3>::kLdsBytes, SkGeom<4>::kLdsBytes};
    for (int i = 0; i < 4; ++i)
      if (hipFuncSetAttribute(ks[i], hipFuncAttributeMaxDynamicSharedMemorySize, sz[i]) != hipSuccess)
        return MASE_ERR_LAUNCH;
    mark_device_setup_done(attr_done);
  }
  const dim3 grid((unsigned)(((N + 31) / 32 + 3) / 4), (unsigned)splits), block(kSkinnyThreads);
  SkinnyParams p;
  p.B = (const unsigned char*)B;
  p.N = (int)N;
  p.K = (int)K;
  p.kc = range_elems((int)K, kSkChunk, splits);
  // one pass per group of 32 rows of A; the partial results of a group form a [splits, rows, N] block, and the
  // blocks of successive groups are laid out so that together they read as [splits, M, N] per group offset
  for (size_t m0 = 0; m0 < M; m0 += 32) {
    const size_t rows = (M - m0 < 32) ? (M - m0) : 32;
    p.A = (const unsigned char*)A + m0 * K * 2;
    void* Cg = (unsigned char*)C + m0 * N * (out_dtype == MASE_DT_F32 ? 4 : 2);
    p.o = skinny_out((float*)workspace + (size_t)splits * m0 * N, Cg, bias, out_dtype, bias_dtype, splits);
    p.M = (int)rows;
    const int xc = (int)(rows + 7) / 8;
    if (xc == 1) hipLaunchKernelGGL(gemm_skinny_partial_kernel<1>, grid, block, SkGeom<1>::kLdsBytes, st, p);
    else if (xc == 2) hipLaunchKernelGGL(gemm_skinny_partial_kernel<2>, grid, block, SkGeom<2>::kLdsBytes, st, p);
    else if (xc == 3) hipLaunchKernelGGL(gemm_skinny_partial_kernel<3>, grid, block, SkGeom<3>::kLdsBytes, st, p);
    else hipLaunchKernelGGL(gemm_skinny_partial_kernel<4>, grid, block, SkGeom<4>::kLdsBytes, st, p);
    skinny_launch_reduce(p.o, Cg, bias, out_dtype, bias_dtype, rows, N, splits, st);
  }
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

extern "C" size_t mase_gemm_mxint8_skinny_workspace_bytes(size_t M, size_t N, size_t K) {
  using namespace mase;
  if (M == 0 || N == 0 || K == 0 || (K % 128) != 0 || M > 128) return 0;
  const int n_cu = skinny_cu_count();
  if (n_cu <= 0) return 0;
  // chunks of 128: the split search works in units of 64, so hand it K / 2
  return (size_t)skinny_splits((int)M, (int)N, (int)(K / 2), n_cu) * M * N * sizeof(float);
}

extern "C" int mase_gemm_mxint8_skinny(const void* A, const int8_t* B_codes, const uint8_t* B_scales, const void* bias,
                                       void* C, size_t M, size_t N, size_t K, int out_dtype, int bias_dtype,
                                       void* workspace, size_t workspace_bytes, void* stream) {
  using namespace mase;
  if (M == 0 || N == 0) return MASE_OK;
  if (A == nullptr || B_codes == nullptr || B_scales == nullptr || C == nullptr) return MASE_ERR_NULL;
  if (K == 0 || (K % 128) != 0 || M > 128 || N > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  if ((unsigned long long)N * K > 0xFFFFFFFFull) return MASE_ERR_SHAPE;  // 32-bit byte offsets into the codes
  if (!aligned16(A) || !aligned16(B_codes) || (((uintptr_t)B_scales) & 3u) != 0) return MASE_ERR_ALIGN;
  if (out_dtype < 0 || out_dtype > 2 || (bias != nullptr && (bias_dtype < 0 || bias_dtype > 2))) return MASE_ERR_DTYPE;
  const int n_cu = skinny_cu_count();
  if (n_cu <= 0) return MASE_ERR_LAUNCH;
  const int splits = skinny_splits((int)M, (int)N, (int)(K / 2), n_cu);
  const size_t need = (size_t)splits * M * N * sizeof(float);
  if (workspace == nullptr || workspace_bytes < need || (((uintptr_t)workspace) & 15u) != 0) return MASE_ERR_WORKSPACE;
  hipStream_t st = (hipStream_t)stream;
  static std::atomic<uint64_t> attr_done{0};
  if (!device_setup_done(attr_done)) {
    // up to 8 rows of A: a ring per wavefront; more: the chunk of A shared by the work-group
    if (hipFuncSetAttribute((const void*)gemm_skinny_mxint8_partial_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            SqGeom<1>::kLdsBytes) != hipSuccess)
      return MASE_ERR_LAUNCH;
    const void* kh[3] = {(const void*)gemm_skinny_mxint8_shared_kernel<2>, (const void*)gemm_skinny_mxint8_shared_kernel<3>,
                         (const void*)gemm_skinny_mxint8_shared_kernel<4>};
    const int szh[3] = {SqsGeom<2>::kLdsBytes, SqsGeom<3>::kLdsBytes, SqsGeom<4>::kLdsBytes};
    for (int i = 0; i < 3; ++i)
      if (hipFuncSetAttribute(kh[i], hipFuncAttributeMaxDynamicSharedMemorySize, szh[i]) != hipSuccess)
        return MASE_ERR_LAUNCH;
    mark_device_setup_done(attr_done);
  }
  const dim3 grid((unsigned)(((N + 31) / 32 + kSqWaves - 1) / kSqWaves), (unsigned)splits), block(kSqThreads);
  SkinnyQParams p;
  p.Bc = (const unsigned char*)B_codes;
  p.Bs = (const unsigned char*)B_scales;
  p.N = (int)N;
  p.K = (int)K;
  p.kc = range_elems((int)K, kSqChunk, splits);
  for (size_t m0 = 0; m0 < M; m0 += 32) {
    const size_t rows = (M - m0 < 32) ? (M - m0) : 32;
    p.A = (const unsigned char*)A + m0 * K * 2;
    void* Cg = (unsigned char*)C + m0 * N * (out_dtype == MASE_DT_F32 ? 4 : 2);
    p.o = skinny_out((float*)workspace + (size_t)splits * m0 * N, Cg, bias, out_dtype, bias_dtype, splits);
    p.M = (int)rows;
    const int xc = (int)(rows + 7) / 8;
    if (xc == 1) hipLaunchKernelGGL(gemm_skinny_mxint8_partial_kernel<1>, grid, block, SqGeom<1>::kLdsBytes, st, p);
    else if (xc == 2) hipLaunchKernelGGL(gemm_skinny_mxint8_shared_kernel<2>, grid, block, SqsGeom<2>::kLdsBytes, st, p);
    else if (xc == 3) hipLaunchKernelGGL(gemm_skinny_mxint8_shared_kernel<3>, grid, block, SqsGeom<3>::kLdsBytes, st, p);
    else hipLaunchKernelGGL(gemm_skinny_mxint8_shared_kernel<4>, grid, block, SqsGeom<4>::kLdsBytes, st, p);
    skinny_launch_reduce(p.o, Cg, bias, out_dtype, bias_dtype, rows, N, splits, st);
  }
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

namespace mase {
namespace {
// K % 256 == 0 takes the shared-chunk kernel, other K the ring-only one
int mxfp4_skinny_splits(size_t M, size_t N, size_t K, int n_cu) {
  if (K % 256 == 0) return mxfp4_shared_splits((int)M, (int)N, (int)K, n_cu);
  return skinny_splits((int)M, (int)N, (int)(K / 2), n_cu);
}
}  // namespace
}  // namespace mase

extern "C" size_t mase_gemm_mxfp4_skinny_workspace_bytes(size_t M, size_t N, size_t K) {
  using namespace mase;
  if (M == 0 || N == 0 || K == 0 || (K % 128) != 0 || M > 128) return 0;
  const int n_cu = skinny_cu_count();
  if (n_cu <= 0) return 0;
  return (size_t)mxfp4_skinny_splits(M, N, K, n_cu) * M * N * sizeof(float);
}

extern "C" int mase_gemm_mxfp4_skinny(const void* A_codes, const void* A_scales, int a_format, const void* B_codes,
                                      const void* B_scales, const void* bias, void* C, size_t M, size_t N, size_t K,
                                      int out_dtype, int bias_dtype, void* workspace, size_t workspace_bytes,
                                      void* stream) {
  using namespace mase;
  if (M == 0 || N == 0) return MASE_OK;
  if (A_codes == nullptr || A_scales == nullptr || B_codes == nullptr || B_scales == nullptr || C == nullptr) return MASE_ERR_NULL;
  if (K == 0 || (K % 128) != 0 || M > 128 || N > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  if ((unsigned long long)N * K / 2 > 0xFFFFFFFFull) return MASE_ERR_SHAPE;
  if (!aligned16(A_codes) || !aligned16(B_codes) || (((uintptr_t)A_scales) & 3u) != 0 || (((uintptr_t)B_scales) & 3u) != 0)
    return MASE_ERR_ALIGN;
  if (a_format != 0 && a_format != 1) return MASE_ERR_PARAM;
  if (out_dtype < 0 || out_dtype > 2 || (bias != nullptr && (bias_dtype < 0 || bias_dtype > 2))) return MASE_ERR_DTYPE;
  const int n_cu = skinny_cu_count();
  if (n_cu <= 0) return MASE_ERR_LAUNCH;
  const int splits = mxfp4_skinny_splits(M, N, K, n_cu);
  const bool shared = (K % 256) == 0;
  const size_t need = (size_t)splits * M * N * sizeof(float);
  if (workspace == nullptr || workspace_bytes < need || (((uintptr_t)workspace) & 15u) != 0) return MASE_ERR_WORKSPACE;
  hipStream_t st = (hipStream_t)stream;
  static std::atomic<uint64_t> attr_done{0};
  if (!device_setup_done(attr_done)) {
    const void* sh[8] = {(const void*)gemm_skinny_mxfp4_shared_kernel<1, 0>, (const void*)gemm_skinny_mxfp4_shared_kernel<2, 0>,
                         (const void*)gemm_skinny_mxfp4_shared_kernel<3, 0>, (const void*)gemm_skinny_mxfp4_shared_kernel<4, 0>,
                         (const void*)gemm_skinny_mxfp4_shared_kernel<1, 1>, (const void*)gemm_skinny_mxfp4_shared_kernel<2, 1>,
                         (const void*)gemm_skinny_mxfp4_shared_kernel<3, 1>, (const void*)gemm_skinny_mxfp4_shared_kernel<4, 1>};
    const int shsz[4] = {SfsGeom<1>::kLdsBytes, SfsGeom<2>::kLdsBytes, SfsGeom<3>::kLdsBytes, SfsGeom<4>::kLdsBytes};
    for (int i = 0; i < 8; ++i)
      if (hipFuncSetAttribute(sh[i], hipFuncAttributeMaxDynamicSharedMemorySize, shsz[i & 3]) != hipSuccess)
        return MASE_ERR_LAUNCH;
    const void* ks[8] = {(const void*)gemm_skinny_mxfp4_partial_kernel<1, 0>, (const void*)gemm_skinny_mxfp4_partial_kernel<2, 0>,
                         (const void*)gemm_skinny_mxfp4_partial_kernel<3, 0>, (const void*)gemm_skinny_mxfp4_partial_kernel<4, 0>,
                         (const void*)gemm_skinny_mxfp4_partial_kernel<1, 1>, (const void*)gemm_skinny_mxfp4_partial_kernel<2, 1>,
                         (const void*)gemm_skinny_mxfp4_partial_kernel<3, 1>, (const void*)gemm_skinny_mxfp4_partial_kernel<4, 1>};
    const int sz[4] = {SfGeom<1>::kLdsBytes, SfGeom<2>::kLdsBytes, SfGeom<3>::kLdsBytes, SfGeom<4>::kLdsBytes};
    for (int i = 0; i < 8; ++i)
      if (hipFuncSetAttribute(ks[i], hipFuncAttributeMaxDynamicSharedMemorySize, sz[i & 3]) != hipSuccess)
        return MASE_ERR_LAUNCH;
    mark_device_setup_done(attr_done);
  }
  const dim3 grid((unsigned)(((N + 31) / 32 + 3) / 4), (unsigned)splits), block(kSkinnyThreads);
  SkinnyFParams p;
  p.Wc = (const unsigned char*)B_codes;
  p.Ws = (const unsigned char*)B_scales;
  p.N = (int)N;
  p.K = (int)K;
  p.kc = range_elems((int)K, shared ? 256 : 128, splits);
  p.rotate = (shared && splits == 1) ? 1 : 0;
  for (size_t m0 = 0; m0 < M; m0 += 32) {
    const size_t rows = (M - m0 < 32) ? (M - m0) : 32;
    p.Xc = (const unsigned char*)A_codes + m0 * K;
    p.Xs = (const unsigned char*)A_scales + m0 * (K / 32);
    void* Cg = (unsigned char*)C + m0 * N * (out_dtype == MASE_DT_F32 ? 4 : 2);
    p.o = skinny_out((float*)workspace + (size_t)splits * m0 * N, Cg, bias, out_dtype, bias_dtype, splits);
    p.M = (int)rows;
    const int xc = (int)(rows + 7) / 8;
#define MASE_SF_LAUNCH(XC_)                                                                                           \
  do {                                                                                                                \
    if (shared) {                                                                                                     \
      if (a_format == 0)                                                                                              \
        hipLaunchKernelGGL((gemm_skinny_mxfp4_shared_kernel<XC_, 0>), grid, block, SfsGeom<XC_>::kLdsBytes, st, p);   \
      else                                                                                                            \
        hipLaunchKernelGGL((gemm_skinny_mxfp4_shared_kernel<XC_, 1>), grid, block, SfsGeom<XC_>::kLdsBytes, st, p);   \
    } else if (a_format == 0) {                                                                                       \
      hipLaunchKernelGGL((gemm_skinny_mxfp4_partial_kernel<XC_, 0>), grid, block, SfGeom<XC_>::kLdsBytes, st, p);     \
    } else {                                                                                                          \
      hipLaunchKernelGGL((gemm_skinny_mxfp4_partial_kernel<XC_, 1>), grid, block, SfGeom<XC_>::kLdsBytes, st, p);     \
    }                                                                                                                 \
  } while (0)
    if (xc == 1) MASE_SF_LAUNCH(1);
    else if (xc == 2) MASE_SF_LAUNCH(2);
    else if (xc == 3) MASE_SF_LAUNCH(3);
    else MASE_SF_LAUNCH(4);
#undef MASE_SF_LAUNCH
    skinny_launch_reduce(p.o, Cg, bias, out_dtype, bias_dtype, rows, N, splits, st);
  }
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}
