// C[M,N] = A[M,K] * B[N,K]^T (+ bias[N]) on gfx950 matrix cores: bf16 operands, fp32 accumulation.
//
// This is the contraction behind the MX Linear forward.  Both operands are K-major (activations [tokens, K],
// weights [out, K]), which is the layout v_mfma_f32_16x16x32_bf16 wants: lane l supplies 8 consecutive
// K-elements of row/column l%16, K-group l/16.  MXINT8 and MXFP values are exactly representable in bf16
// (<= 8 significant bits times a power of two), so feeding them as bf16 computes the same real-number dot
// products as the reference's fp32 GEMM on the quantize-dequantized operands; only the summation order
// differs.
//
// Schedule: 256x256 output tile (4 wavefronts, 2x2, 128x128 each = 8x8 MFMA tiles of 16x16, or 1x4, 256x64 each =
// 16x4 tiles, when B comes in fragment order; 256 accumulator registers per lane either way), K tile 64 so that every operand row of a tile is one full 128-byte cache line (64-byte rows made
// the L1 fetch every line twice and bound the loop), two LDS stages of 64 KB.  Operand tiles go from HBM/L2
// straight into LDS with global_load_lds_dwordx4 (no staging registers, no ds_write).  A wavefront-wide copy
// deposits 64 consecutive 16-byte chunks = 8 LDS rows of 128 B, so the bank-conflict swizzle is applied on
// the global-address side: each lane fetches the chunk that belongs at its LDS position.  The swizzle is
// chunk ^ ((row>>1)&7): this LDS serves a ds_read_b128 sixteen lanes at a time out of 64 four-byte banks, so
// the 16-byte slots (address/16 mod 16) of 16 consecutive rows must all differ; rows of equal parity share a
// 128-byte half of the 256-byte bank period and get distinct slots from the XOR.
// Rows beyond M or N are clamped to the last valid row (their products land in accumulators that are never
// stored), so the main loop has no bounds checks.
//
// The kernel is persistent: one work-group per CU walks a list of output tiles, and the K tiles of all of them
// form one stream through the two stages, so the first K tiles of the next output tile are already being
// copied while the epilogue of the current one runs and its stores drain behind the next main loop.
#include "common.hpp"

#include <type_traits>

namespace mase {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int S = 2;                              // LDS stages
constexpr int kStagesB = 4;                       // stages of A alone (32 KB each) when B comes in fragment order
constexpr int kGemmThreads = 256;
constexpr int kRowBytes = BK * 2;                 // 128: one cache line per operand row per K tile
constexpr int kTileBytes = BM * kRowBytes;        // 32 KB per operand per stage
constexpr int kStageBytes = 2 * kTileBytes;       // A then B
constexpr int kWaveCopies = kTileBytes / 1024 / 4;  // copies per wavefront per operand per K tile = 8
constexpr int kCopies = 2 * kWaveCopies;          // async copies one wavefront issues per K tile = 16
// epilogue staging, separate from the stages: per wavefront 32 rows of 128 bytes, row stride 144 bytes (16-byte
// accesses of 16 consecutive rows at one column offset then fall on 64 different banks)
constexpr int kStgRow = 144;
constexpr int kStgWave = 32 * kStgRow;
constexpr int kLdsBytes = S * kStageBytes + 4 * kStgWave;

struct GemmParams {
  const unsigned char* A;
  const unsigned char* B;
  const unsigned char* Bs;  // BCODES: the scale image that goes with the code image in B
  const void* bias;
  void* C;
  int M, N, K;
  int bias_dtype;
  int tiles_m, tiles_n;
  int splits, kc;  // K is cut into `splits` ranges of kc elements; a work item is one output tile over one range and
                   // (when splits > 1) writes an fp32 partial tile into slice `range` of C, laid out [splits, M, N]
  // BATCHED instantiation only: `batches` independent products, product index = outer * batch_inner + inner; byte
  // strides of the two index parts per operand, and byte strides of an operand row / an output row
  int batches = 1, batch_inner = 1;
  size_t a_so = 0, a_si = 0, b_so = 0, b_si = 0, c_so = 0, c_si = 0;
  size_t lda = 0, ldb = 0, ldc = 0;
};

__device__ __forceinline__ int lds_off(int row, int chunk) {
  return row * kRowBytes + ((chunk ^ ((row >> 1) & 7)) << 4);
}

__device__ __forceinline__ float load_bias(const void* bias, int dt, int col) {
  if (dt == MASE_DT_F32) return ((const float*)bias)[col];
  if (dt == MASE_DT_BF16) return bits2f((uint32_t)((const uint16_t*)bias)[col] << 16);
  return f16_bits_to_f32(((const uint16_t*)bias)[col]);
}

typedef __attribute__((address_space(3))) void* lptr_t;

// One wavefront-wide 1 KB async copy HBM/L2 -> LDS: lane i's 16 bytes at base + off_i land at LDS address
// lds_addr + 16*i (base and lds_addr wavefront-uniform, off_i a 32-bit byte offset).  Issued from inline
// assembly rather than through the compiler's builtin: the compiler orders every LDS read after all async
// copies it knows to be in flight (s_waitcnt vmcnt(0) before each ds_read), which would serialize the
// pipeline; completion is tracked by hand with wait_vmcnt.  M0 carries the LDS base; nothing else in this
// kernel uses M0.
// (m0 is written inside the statement and not listed as clobbered: the compiler keeps no value in m0 across
// statements on this target, it reloads m0 before each use of its own, and rejects the name in a clobber list as a
// reserved register)
__device__ __forceinline__ void async_copy_16(const unsigned char* base, uint32_t off, uint32_t lds_addr) {
  const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(m0v) : "memory");
}

// The lane number, computed where it is needed (two instructions) instead of being kept: the code between output tiles
// then holds no value across the K loop that the register allocator would spill.  A reload from scratch memory is a
// vector-memory load the compiler tracks, and it guards such a load with s_waitcnt vmcnt(0), which also waits for
// every async copy and fragment load in flight.  The asm statement keeps the terms derived from the lane number from
// being hoisted out of their place and into the K loop's live registers.
__device__ __forceinline__ int lane_now() {
  int lane;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane));
  return lane;
}

// An accumulator value moved to an ordinary register at the place of the call.  Left to itself the compiler copies all
// 256 accumulators out of their registers at once when it reaches the epilogue, and spills what that displaces.
__device__ __forceinline__ float acc_read(float a) {
  float v;
  asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
  return v;
}
// The compiler separates a matrix instruction from a read of its result by the wait states the part requires, but it does
// not look inside acc_read's assembly.  An epilogue therefore starts with this: more wait states than the longest
// matrix instruction needs (19) plus the time the last matrix instructions may spend queued behind the ones before them,
// issued after the K loop's last matrix instruction and, both being volatile assembly, before the first acc_read.
__device__ __forceinline__ void acc_read_fence() {
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
}

// acc += B fragment x A fragment with v_mfma_f32_16x16x32_bf16, the accumulator tied to accumulation registers.  Through
// the compiler's builtin the 64 four-register accumulators of the K loop are not kept in place from one trip to the next
// (the loop then opens with some 270 register moves).  As assembly the compiler inserts no wait states for it: an
// accumulator is read again 64 matrix instructions after it was written, the fragments come from loads (completed by
// s_waitcnt), the epilogue starts with acc_read_fence and zeroing ends with acc_write_fence.
__device__ __forceinline__ void mfma16_acc(f32x4_t& acc, const bf16x8_t& b, const bf16x8_t& a) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(b), "v"(a));
}
// wait states between a write of an accumulation register by an ordinary instruction and a matrix instruction that
// reads it as its addend (the part requires 2)
__device__ __forceinline__ void acc_write_fence() { asm volatile("s_nop 3" ::: "memory"); }

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  // gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14 ; leave the others at max
  __builtin_amdgcn_s_waitcnt((N & 0xF) | (0x7 << 4) | (0xF << 8) | ((N >> 4) << 14));
}

// One wavefront-wide 1 KB load HBM/L2 -> registers (16 bytes per lane), issued from inline assembly for the same
// reason as the async copies: the compiler does not know of it, so nothing waits for it except wait_vmcnt.  The
// destination must not be touched before the wait that covers it.
__device__ __forceinline__ void load_16_untracked(bf16x8_t& dst, uint32_t off, const unsigned char* base) {
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(off), "s"(base) : "memory");
}

// One wavefront-wide 512-byte / 128-byte load (8 / 2 bytes per lane) outside the compiler's tracking, as above.
__device__ __forceinline__ void load_8_untracked(uint2& dst, uint32_t off, const unsigned char* base) {
  asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(dst) : "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ void load_4_untracked(uint32_t& dst, uint32_t off, const unsigned char* base) {
  asm volatile("global_load_dword %0, %1, %2" : "=v"(dst) : "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ void load_2_untracked(uint32_t& dst, uint32_t off, const unsigned char* base) {
  asm volatile("global_load_ushort %0, %1, %2" : "=v"(dst) : "v"(off), "s"(base) : "memory");
}

// STREAM: K holds at least S tiles, so the copy stream is never more than one output tile ahead and advances
// without branches; the other instantiation (K = one tile) advances it with the general, branching step.
// BPACK (with STREAM, an even number of K tiles): B is the fragment-ordered image of mase_gemm_bf16_pack_b and its
// fragments go from L2 straight into registers, one K tile ahead of the MFMAs that use them; only A passes through
// LDS, in four stages of 32 KB (the copies landing in LDS while the wavefronts read their fragments is what holds the
// plain kernel back).  The four wavefronts then split the 256 x 256 tile 1 x 4 (each 256 rows x 64 columns: 16 x 4
// tiles of v_mfma_f32_16x16x32_bf16) instead of 2 x 2 (128 x 128), so that no two wavefronts load the same B fragments: the CU's
// vector-memory path carries 32 KB of B per K tile next to A's 32 KB (64 KB with the 2 x 2 split, measured 5 % slower),
// at the price of each wavefront reading all of A from LDS.  That path, not the matrix pipe, is what the K loop waits
// for.
// BCODES (with BPACK): B is an MXINT8 weight as codes + scale bytes in fragment order (mase_gemm_mxint8_pack_b): half
// the bytes of the bf16 image in memory and on the way in; the codes are widened to the same bf16 operand values in
// registers, a K step (half a K tile) ahead of the MFMAs that use them (code + 128 as an unsigned byte ->
// v_cvt_f32_ubyte -> one fma that removes the 128 and applies the block's power-of-two scale -> the upper half of the
// exact fp32 product).
// BATCHED (plain form only): the work items are the output tiles of `batches` independent products with strided
// operands (the score and value products of an attention block, torch.bmm): an item's operand bases and its output
// base follow from its product index; rows of A, B and C have the strides lda, ldb, ldc.
// HALFN (plain form only): output tiles of 256 x 128 for products with at most 128 columns (the value product of an
// attention block with head dimension 128), where a 256-wide tile would spend half of its matrix instructions on
// columns that do not exist.  The wavefronts split the tile 2 x 2 into 128 rows x 64 columns (8 x 4 MFMA tiles, 32
// MFMAs per K step); B's stage holds 128 rows.
template <int OUT_DT, bool STREAM, bool BPACK = false, bool BCODES = false, bool BATCHED = false, bool HALFN = false>
__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_tn_kernel(GemmParams p) {
  constexpr int NI = BPACK ? 8 : 4, NJ = (BPACK || HALFN) ? 2 : 4;  // 32 x 32 tiles of a wavefront: rows x columns
  // All forms compute with v_mfma_f32_16x16x32_bf16 (16 x 4, 8 x 8 or 8 x 4 tiles of 16 x 16 per wavefront, two K
  // steps of 32 per K tile): the same multiply-adds per cycle as the 32x32x16 instruction on paper, but under the board's power
  // limit the part sustains a clock about 8 % higher on it (measured with both instructions on random operands).
  constexpr int kBN = HALFN ? 128 : BN;                           // columns of an output tile
  constexpr int kCopiesB = HALFN ? kWaveCopies / 2 : kWaveCopies;  // copies of B per wavefront per K tile
  static_assert(!BCODES || BPACK, "codes come in fragment order");
  static_assert(!BATCHED || !BPACK, "the batched form takes row-major operands");
  static_assert(!HALFN || !BPACK, "the narrow tile exists in the plain form");
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane_id = tid & 63;
  const int lane = lane_id;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int row_base = BPACK ? 0 : wm * 128, col_base = BPACK ? wave * 64 : wn * (HALFN ? 64 : 128);  // the wavefront's part of the tile
  const int nk = p.kc / BK;

  // ---- this work-group's output tiles.  Work-groups are dealt to the 8 XCDs round-robin; when the counts
  // divide, XCD x owns the contiguous tile range [x*total/8, (x+1)*total/8) and its work-groups walk it
  // together (at any time they hold neighbouring tiles, which share operand rows in that XCD's L2).
  const int tiles_mn = p.tiles_m * p.tiles_n;
  const int total = tiles_mn * (BATCHED ? p.batches : p.splits);
  const int nwg = (int)gridDim.x;
  int t_first, t_step, t_end;
  if ((total & 7) == 0 && (nwg & 7) == 0) {
    const int per_xcd = total >> 3;
    t_first = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
    t_step = nwg >> 3;
    t_end = (((int)blockIdx.x & 7) + 1) * per_xcd;
  } else {
    t_first = (int)blockIdx.x;
    t_step = nwg;
    t_end = total;
  }
  const int n_my = (t_first < t_end) ? (t_end - t_first + t_step - 1) / t_step : 0;
  if (n_my == 0) return;
  constexpr int GROUP_M = 4;  // tiles are walked in groups of 4 tile rows
  const int in_group = GROUP_M * p.tiles_n;
  // (BATCHED: ks is the item's product index; there are no K ranges)
  auto tile_origin = [&](int ord, int& m0, int& n0, int& ks) __attribute__((always_inline)) {  // ord-th item of this work-group
    const int item = t_first + min(ord, n_my - 1) * t_step;
    ks = item / tiles_mn;
    const int t = item - ks * tiles_mn;
    const int first_m = (t / in_group) * GROUP_M;
    const int gsz = min(p.tiles_m - first_m, GROUP_M);
    m0 = (first_m + (t % in_group) % gsz) * BM;
    n0 = ((t % in_group) / gsz) * kBN;
  };

  // ---- global side of the async copies: wave w fills row groups w + 4*j (8 rows of 128 B each), j = 0..7
  const size_t ldb = BATCHED ? p.ldb : (size_t)p.K * 2;  // bytes per operand row
  const size_t lda = BATCHED ? p.lda : ldb;
  uint32_t ga[kWaveCopies], gb[kWaveCopies];  // byte offsets of this lane's chunks from the operand bases
  const unsigned char *copy_a = p.A, *copy_b = p.B;  // operand bases of the item the copy stream is in
  auto set_copy_tile = [&](int ord) __attribute__((always_inline)) {
    int m0, n0, ks;
    tile_origin(ord, m0, n0, ks);
    uint32_t k0 = (uint32_t)ks * (uint32_t)p.kc * 2u;  // byte offset of the item's K range inside a row
    if constexpr (BATCHED) {
      const int bo = ks / p.batch_inner, bi = ks - bo * p.batch_inner;
      copy_a = p.A + (size_t)bo * p.a_so + (size_t)bi * p.a_si;
      copy_b = p.B + (size_t)bo * p.b_so + (size_t)bi * p.b_si;
      k0 = 0;
    }
    const int lane = lane_now();
#pragma unroll
    for (int j = 0; j < kWaveCopies; ++j) {
      const int r = (wave + 4 * j) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ ((r >> 1) & 7);  // chunk that belongs at LDS position lane&7 of row r
      ga[j] = (uint32_t)((size_t)min(m0 + r, p.M - 1) * lda) + chunk * 16 + k0;
      if constexpr (!BPACK) gb[j] = (uint32_t)((size_t)min(n0 + r, p.N - 1) * ldb) + chunk * 16 + k0;
    }
  };
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lptr_t)lds;
  // copy-stream position: K tile c_kt of this work-group's c_ord-th output tile goes to stage c_stage.  Past the
  // last tile the stream keeps re-copying K tiles into stages nobody reads any more, which keeps the main
  // loop free of branches around the copies and the vmcnt bookkeeping uniform.
  // LDS stages: the plain form keeps S stages of A + B; the BPACK form keeps kStagesB stages of A alone (B never
  // passes through LDS), which lets the A copies of a K tile be issued a whole K tile before the hand-over that
  // waits for the K tile before it
  constexpr int kStages = BPACK ? kStagesB : S;
  constexpr int kStride = BPACK ? kTileBytes : kStageBytes;
  auto next_of = [](int st) __attribute__((always_inline)) { return (st + 1 == kStages) ? 0 : st + 1; };
  int c_kt = 0, c_ord = 0, c_stage = 0;
  // copy number c (0..15) of the current K tile: row group c/2 of A (even c) or B (odd c)
  auto issue_copy = [&](int c) __attribute__((always_inline)) {
    if constexpr (BPACK) {
      if (c & 1) return;  // B does not pass through LDS
    }
    if constexpr (HALFN) {
      if ((c & 1) && (c >> 1) >= kCopiesB) return;  // B's stage holds 128 rows: row groups 0..15
    }
    const uint32_t st = lds_base + (uint32_t)(c_stage * kStride) + (c & 1) * kTileBytes;
    const int j = c >> 1;
    async_copy_16(((c & 1) ? copy_b : copy_a) + (size_t)c_kt * kRowBytes, (c & 1) ? gb[j] : ga[j], st + (wave + 4 * j) * 1024);
  };
  auto step_within_tile = [&]() __attribute__((always_inline)) {
    c_stage = next_of(c_stage);
    ++c_kt;
  };
  auto advance_copy_stream = [&]() __attribute__((always_inline)) {
    c_stage = next_of(c_stage);
    if (c_ord >= n_my) return;  // past the end: stay on the final K tile
    if (++c_kt == nk) {
      if (++c_ord < n_my) {
        c_kt = 0;
        set_copy_tile(c_ord);
      } else {
        c_kt = nk - 1;
      }
    }
  };

  constexpr int NI16 = 2 * NI, NJ16 = 2 * NJ;
  f32x4_t acc16[NI16][NJ16];  // [row tile of 16][column tile of 16]
  auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NI16; ++i)
#pragma unroll
      for (int j = 0; j < NJ16; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc16[i][j][r] = 0.0f;
    acc_write_fence();
  };
  zero_acc();

  set_copy_tile(0);
  // the copy stream leads the K loop by S tiles (BPACK: by kStagesB - 1)
#pragma unroll
  for (int t = 0; t < (BPACK ? kStagesB - 1 : S); ++t) {
#pragma unroll
    for (int c = 0; c < kCopies; ++c) issue_copy(c);
    advance_copy_stream();
  }

  // The lane's row and K group within a fragment, which every LDS read of the K loop is addressed with.  Set again
  // from the lane number after each epilogue rather than kept across it: what lives across the epilogue's register
  // demand gets spilled (see lane_now).
  int frag_row = lane & 15;
  int kgrp = lane >> 4;
  // plain forms: fragment f (0..7: A row tile f of the wavefront's 128 rows, 8..15: B column tile f - 8 of its 128
  // columns; narrow form: 8..11 of its 64 columns) of K step ks (32 of the K tile's 64)
  auto load_frag16 = [&](int stage, int ks, int f) __attribute__((always_inline)) -> bf16x8_t {
    const unsigned char* st = lds + stage * kStride + ((f < 8) ? (wm * 128) * kRowBytes : kTileBytes + (wn * (HALFN ? 64 : 128)) * kRowBytes);
    return __builtin_bit_cast(bf16x8_t, *(const uint4*)(st + lds_off((f & 7) * 16 + frag_row, ks * 4 + kgrp)));
  };
  // fragment-ordered forms (only A passes through LDS): fragment f of quarter q of the K tile = rows
  // 128 * (q % 2) + 16 * f .. + 16 of the whole tile at K 32 * (q / 2) .. + 32, lane l supplying row l % 16, K
  // 8 * (l / 16) .. + 8
  auto load_frag = [&](int stage, int q, int f) __attribute__((always_inline)) -> bf16x8_t {
    const unsigned char* st = lds + stage * kStride;
    return __builtin_bit_cast(bf16x8_t, *(const uint4*)(st + lds_off(((q & 1) * 8 + f) * 16 + frag_row, (q >> 1) * 4 + kgrp)));
  };

  // ---- epilogue of one output tile.  The MFMAs take the B fragment as their first operand, so the accumulators hold
  // the tile transposed: acc16[i][j][rr] is C[row, col] with row = i*16 + lane%16 and col = j*16 + (lane/16)*4 + rr,
  // i.e. a lane holds runs of four consecutive columns of one row; a band of 32 rows is made of two row tiles.  Bias is added
  // and the value converted in registers; the runs then pass through the wavefront's own staging rows (32 rows of 128
  // bytes: 64 columns of a 16-bit output, 32 of an fp32 one), from which every lane takes 16 consecutive bytes, so that
  // a store instruction writes 8 rows of 128 contiguous bytes.  Only lanes of one wavefront exchange data (its LDS
  // accesses execute in order, and the writes are waited for before the reads are issued): no barrier.
  auto epilogue = [&](int ord) __attribute__((always_inline)) {
    int m0, n0, ks;
    tile_origin(ord, m0, n0, ks);
    acc_read_fence();
    // partial tiles of K range ks go to slice ks of C (fp32, no bias: the caller's reduction adds it)
    unsigned char* Cs = (unsigned char*)p.C + (size_t)ks * (size_t)p.M * (size_t)p.N * sizeof(float);
    if constexpr (BATCHED) {
      const int bo = ks / p.batch_inner, bi = ks - bo * p.batch_inner;
      Cs = (unsigned char*)p.C + (size_t)bo * p.c_so + (size_t)bi * p.c_si;
    }
    const int lane = lane_now();
    const int r32 = lane & 15, kgrp = lane >> 4;
    const int rrow = lane >> 3, chunk = lane & 7;  // read side: row rrow + 8 * pass, 16-byte piece `chunk` of it
    unsigned char* const stg = lds + S * kStageBytes + wave * kStgWave;
    unsigned char* const stg_w = stg + r32 * kStgRow;
    const unsigned char* const stg_r = stg + rrow * kStgRow + chunk * 16;
    constexpr int kEsz = (OUT_DT == MASE_DT_F32) ? 4 : 2;
    constexpr int kVec = 16 / kEsz;  // elements per 16-byte piece
    // (BATCHED: the host has checked that the output base, its strides and its row stride are multiples of 16 bytes)
    const bool vec_ok = BATCHED ? true : ((p.N & (kVec - 1)) == 0) && ((((uintptr_t)p.C) & 15u) == 0);
    // the wavefront's whole part of the tile lies inside C and takes 16-byte stores (wavefront-uniform)
    const bool interior = vec_ok && m0 + row_base + NI * 32 <= p.M && n0 + col_base + NJ * 32 <= p.N;
    const size_t row_step = BATCHED ? p.ldc : (size_t)p.N * kEsz;  // bytes from one output row to the next
    // where this lane's piece of row 0 of the wavefront's first band goes
    unsigned char* const lane_c = Cs + (size_t)(m0 + row_base + rrow) * row_step + (size_t)(n0 + col_base + chunk * kVec) * kEsz;
    float bv[NJ][4][4];  // bias of the lane's columns
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) bv[j][q][rr] = 0.0f;
    if (p.bias != nullptr) {
      auto fill = [&](auto dtc) __attribute__((always_inline)) {  // the dtype is decided once, not per element
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
              // (bv[j][q] belongs to column tile 2 * j + q / 2 of 16; odd q are not used)
              const int col = n0 + col_base + (2 * j + (q >> 1)) * 16 + kgrp * 4 + rr;
              if (q & 1) continue;
              if (col < p.N) bv[j][q][rr] = load_bias(p.bias, decltype(dtc)::value, col);
            }
      };
      if (p.bias_dtype == MASE_DT_F32) fill(std::integral_constant<int, MASE_DT_F32>{});
      else if (p.bias_dtype == MASE_DT_BF16) fill(std::integral_constant<int, MASE_DT_BF16>{});
      else fill(std::integral_constant<int, MASE_DT_F16>{});
      // The bias loads are the only vector-memory loads the compiler itself tracks in this kernel.  Completing
      // them here, with a wait it can see, keeps it from guarding their registers with s_waitcnt vmcnt(0)
      // inside the K loop, where that would also wait for every async copy in flight.
      wait_vmcnt<0>();
    }
    // one band: kBandTiles MFMA tiles of row tile i side by side = 128 bytes of output per row
    constexpr int kBandTiles = (OUT_DT == MASE_DT_F32) ? 1 : 2;
    constexpr int kBandsPerRowTile = NJ / kBandTiles;
    constexpr int kBands = NI * kBandsPerRowTile;
    auto stage_band = [&](int b) __attribute__((always_inline)) {
      const int i = b / kBandsPerRowTile, jb = b % kBandsPerRowTile;
#pragma unroll
      for (int jj = 0; jj < kBandTiles; ++jj) {
        const int j = jb * kBandTiles + jj;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          // q = 2 * (column tile of 16 within the 32 columns j) + (row tile of 16 within the band)
          const int i16 = 2 * i + (q & 1), j16 = 2 * j + (q >> 1);
          const float* const bq = bv[j][q & 2];
          float v[4];
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) v[rr] = acc_read(acc16[i16][j16][rr]) + bq[rr];
          unsigned char* const dst = stg_w + (q & 1) * 16 * kStgRow + (jj * 32 + (q >> 1) * 16 + kgrp * 4) * kEsz;
          if constexpr (OUT_DT == MASE_DT_F32) {
            *(uint4*)dst = make_uint4(f2bits(v[0]), f2bits(v[1]), f2bits(v[2]), f2bits(v[3]));
          } else if constexpr (OUT_DT == MASE_DT_BF16) {
            *(uint2*)dst = make_uint2(f32x2_to_bf16x2_bits(v[0], v[1]), f32x2_to_bf16x2_bits(v[2], v[3]));
          } else {
            *(uint2*)dst = make_uint2(f32_to_f16_bits(v[0]) | (f32_to_f16_bits(v[1]) << 16),
                                      f32_to_f16_bits(v[2]) | (f32_to_f16_bits(v[3]) << 16));
          }
        }
      }
    };
    // Staging band b + 1 between the issue of band b's reads and their use (the LDS executes a wavefront's accesses in
    // the order of issue, so the next band can be written behind the reads while their data is on its way) pays where
    // the epilogue is a large part of the kernel, the batched form with its few K tiles per output tile (score product
    // of an attention block: 6 % faster); with long K loops it was measured without gain or slightly slower.
    constexpr bool kPipeBands = BATCHED;
    if constexpr (kPipeBands) stage_band(0);
#pragma unroll
    for (int b = 0; b < kBands; ++b) {
      const int i = b / kBandsPerRowTile, jb = b % kBandsPerRowTile;
      if constexpr (!kPipeBands) {
        stage_band(b);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the band is in LDS before any lane reads it
      }
      uint4 w[4];
#pragma unroll
      for (int ps = 0; ps < 4; ++ps) w[ps] = *(const uint4*)(stg_r + ps * 8 * kStgRow);
      if constexpr (kPipeBands) {
        asm volatile("" ::: "memory");
        if (b + 1 < kBands) stage_band(b + 1);
        asm volatile("" ::: "memory");
      }
      // streaming stores: the output is not read again by this kernel and should not displace operand panels
      unsigned char* const dst0 = lane_c + (size_t)(i * 32) * row_step + jb * 128;
      if (__builtin_expect(interior, 1)) {
#pragma unroll
        for (int ps = 0; ps < 4; ++ps) store_nt((uint4*)(dst0 + (size_t)(ps * 8) * row_step), w[ps]);
      } else {
        const int col0 = n0 + col_base + jb * kBandTiles * 32 + chunk * kVec;
#pragma unroll
        for (int ps = 0; ps < 4; ++ps) {
          const int row = m0 + row_base + i * 32 + ps * 8 + rrow;
          unsigned char* const dst = dst0 + (size_t)(ps * 8) * row_step;
          if (row >= p.M) continue;
          if (vec_ok && col0 + kVec - 1 < p.N) {
            store_nt((uint4*)dst, w[ps]);
          } else {
            // element by element, the 16 bytes shifted down as they go (a rolled loop: this path is rare and is
            // kept small so that the code between two K loops stays short)
            uint32_t x0 = w[ps].x, x1 = w[ps].y, x2 = w[ps].z, x3 = w[ps].w;
#pragma unroll 1
            for (int e = 0; e < kVec && col0 + e < p.N; ++e) {
              if constexpr (OUT_DT == MASE_DT_F32) {
                ((uint32_t*)dst)[e] = x0;
                x0 = x1, x1 = x2, x2 = x3;
              } else {
                ((uint16_t*)dst)[e] = (uint16_t)x0;
                x0 = (x0 >> 16) | (x1 << 16), x1 = (x1 >> 16) | (x2 << 16), x2 = (x2 >> 16) | (x3 << 16), x3 >>= 16;
              }
            }
          }
        }
      }
      asm volatile("" ::: "memory");      // lanes exchange data through LDS: no value may be carried across
      __builtin_amdgcn_sched_barrier(0);  // bands stay in program order: bounded register use
    }
  };

  // Software pipeline, written out instruction by instruction and pinned with scheduling barriers, because a
  // wavefront issues in order: an MFMA occupies the matrix pipe for 16 cycles, and whatever else has to be issued (LDS reads of later K steps, async copies of the K tile after
  // next) must sit *between* MFMAs to be free.  Per K tile, in the plain forms: four quarters of matrix instructions:
  //   quarters 0, 1: interleaved with the LDS reads of the fragments the rest of the K tile needs
  //   hand-over (after the MFMAs of quarter 1 are issued): this wavefront's reads of the K tile are complete
  //     (lgkmcnt) and its copies of the next K tile have landed (vmcnt); barrier -> the next K tile is visible
  //     to all and nobody reads this one's stage any more
  //   quarters 2, 3: interleaved with the LDS reads of the next K tile's first fragments and the 16 copies of the K
  //     tile after next into the stage just vacated, one every other slot.
  // Handing the stage over half-way through the K tile (which costs more fragment registers) lets the copies be
  // issued over two quarters instead of one: issued in a burst their data arrives in a burst, the LDS is then busy
  // with the writes when the wavefronts want their fragment reads, and the wavefronts drift apart (measured:
  // the barrier costs nothing without the copies and a quarter of the loop with them in a 16-slot burst).
  // The barrier is a bare s_barrier: the fence of __syncthreads() would wait for all copies in flight.
  // The body must stay a single basic block: with a branch inside, the compiler sinks the MFMAs (whose
  // results are only consumed by the next iteration) below it and the interleave is lost.  Hence the copy
  // stream is advanced by a caller-supplied, branch-free step.
  // The epilogue's stores count in vmcnt like the copies, so the first hand-over of an output tile also waits
  // for the previous tile's stores to be acknowledged.
  bf16x8_t fr[4][8];
  // BPACK: B fragments of two K tiles (the one in use and the one being loaded): [buffer][2 * K step + column tile / 2]
  // [column tile % 2].  Image layout: 1 KB blocks [column tile of 16][K step of 32][lane][8 bf16], lane l = column
  // l % 16, K 8*(l/16)..+8.
  bf16x8_t fb[(BPACK && !BCODES) ? 2 : 1][(BPACK && !BCODES) ? 4 : 1][2];
  // BCODES: the codes of two K tiles [buffer][2 * K step + column tile / 2][column tile % 2] (8 per lane: K step of 32,
  // column tile of 16, lane l = column l % 16, K 8 * (l / 16) .. + 8), the scale bytes of the lane's column in the four
  // column tiles [buffer][K step] (byte ct = column tile ct) and the widened fragments of the two K steps [K step][column
  // tile]
  uint2 fbc[BCODES ? 2 : 1][BCODES ? 4 : 1][2];
  uint32_t fsc[BCODES ? 2 : 1][2];
  uint4 fbq[BCODES ? 2 : 1][BCODES ? 4 : 1];
  uint32_t soff = 0;         // BCODES: this lane's byte offset of K tile 0 of its 64 columns in the scale image
  const unsigned char* s_kbase = p.Bs;
  uint32_t boff[4];          // this lane's byte offset of K step 0 of its four column tiles
  const unsigned char* b_kbase = p.B;  // image address of K tile 0 of the K range of the output tile being loaded
  int b_kt = 0;              // K tile (within the range) whose fragments the current iteration loads
  auto set_b_tile = [&](int ord) __attribute__((always_inline)) {
    int m0, n0, ks;
    tile_origin(ord, m0, n0, ks);
    const int lane = lane_now();
    const int nt_last = (p.N + 31) / 32 - 1;
    constexpr uint32_t kFragBytes = BCODES ? 512u : 1024u;  // one fragment of a wavefront: 8 codes or 8 bf16 per lane
    {
      // four column tiles of 16; the image holds a multiple of 32 columns (those beyond N are zero)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const size_t ct = (size_t)min((n0 + col_base) / 16 + j, 2 * nt_last + 1);
        boff[j] = (uint32_t)(ct * (size_t)(p.K / 32) * kFragBytes) + (uint32_t)lane * (kFragBytes / 64u);
      }
      b_kbase = p.B + (size_t)ks * (size_t)(p.kc / 32) * kFragBytes;
      if constexpr (BCODES) {
        // scale image: 128-byte blocks [64 columns][K tile][column % 16][K step][column / 16]
        const size_t g64 = (size_t)min((n0 + col_base) / 64, (p.N + 63) / 64 - 1);
        soff = (uint32_t)(g64 * (size_t)(p.K / 64) * 128u) + (uint32_t)(lane & 15) * 8u;
        s_kbase = p.Bs + (size_t)ks * (size_t)(p.kc / 64) * 128u;
      }
      b_kt = 0;
    }
  };
  // BCODES: the loads of one half of a K tile's codes (K step st: its scale dword and its four fragments), and the
  // widening.  set_scale puts the scale of the lane's column in column tile ct (K step st of the K tile in buffer
  // `buf`), and the -128 * scale that removes the code offset, into wsc / wbs; widen_quarter makes register r (0..3:
  // two codes) of the fragment of column tile ct ((code - 128) * scale is exact in fp32 and has at most 8 significant
  // bits, so the upper half of the fp32 value is the bf16 value).  A quarter register is 5 vector instructions.
  float wsc[4], wbs[4];
  auto load_codes_half = [&](int buf, int st, int i, const unsigned char* csrc, const unsigned char* ssrc) __attribute__((always_inline)) {
    // i = 0: the scale dword; i = 1..4: the codes of column tile i - 1
    if (i == 0) load_4_untracked(fsc[buf][st], soff + (uint32_t)st * 4u, ssrc);
    else load_8_untracked(fbc[buf][st * 2 + ((i - 1) >> 1)][(i - 1) & 1], boff[i - 1], csrc + (size_t)st * 512);
  };
  // (each in two parts, one for either gap of a slot: three vector instructions fit between two matrix instructions.
  // The parts are volatile assembly: plain arithmetic has no ordering against the matrix instructions or the scheduling
  // barriers when the compiler lays the block out, and it gathered both parts of a slot in one gap.)
  uint32_t wsb = 0;
  float wc0 = 0.0f, wc1 = 0.0f;
  auto set_scale_a = [&](int buf, int st, int ct) __attribute__((always_inline)) {
    const uint32_t w = fsc[buf][st];
    if (ct == 0) asm volatile("v_bfe_u32 %0, %1, 0, 8\n\tv_max_u32 %0, 7, %0" : "=v"(wsb) : "v"(w));
    else if (ct == 1) asm volatile("v_bfe_u32 %0, %1, 8, 8\n\tv_max_u32 %0, 7, %0" : "=v"(wsb) : "v"(w));
    else if (ct == 2) asm volatile("v_bfe_u32 %0, %1, 16, 8\n\tv_max_u32 %0, 7, %0" : "=v"(wsb) : "v"(w));
    else asm volatile("v_bfe_u32 %0, %1, 24, 8\n\tv_max_u32 %0, 7, %0" : "=v"(wsb) : "v"(w));
  };
  auto set_scale_b = [&](int ct) __attribute__((always_inline)) {
    // 2^(scale byte - 134), 0 for scale bytes below 8; and -128 times that
    asm volatile("v_lshl_add_u32 %0, %2, 23, %3\n\tv_mul_f32 %1, 0xc3000000, %0"
                 : "=&v"(wsc[ct]), "=v"(wbs[ct])
                 : "v"(wsb), "v"(0xFC800000u));
  };
  auto set_scale = [&](int buf, int st, int ct) __attribute__((always_inline)) {
    set_scale_a(buf, st, ct);
    set_scale_b(ct);
  };
  auto widen_quarter_a = [&](int buf, int st, int ct, int r) __attribute__((always_inline)) {
    const uint2 c = fbc[buf][st * 2 + (ct >> 1)][ct & 1];
    const uint32_t u = (r & 2) ? c.y : c.x;
    if (r & 1) asm volatile("v_cvt_f32_ubyte2 %0, %2\n\tv_cvt_f32_ubyte3 %1, %2" : "=&v"(wc0), "=v"(wc1) : "v"(u));
    else asm volatile("v_cvt_f32_ubyte0 %0, %2\n\tv_cvt_f32_ubyte1 %1, %2" : "=&v"(wc0), "=v"(wc1) : "v"(u));
  };
  auto widen_quarter_b = [&](int st, int ct, int r) __attribute__((always_inline)) {
    uint32_t v;  // the upper halves of the two products: two bf16
    asm volatile("v_fma_f32 %0, %0, %3, %4\n\tv_fma_f32 %1, %1, %3, %4\n\tv_perm_b32 %2, %1, %0, %5"
                 : "+v"(wc0), "+v"(wc1), "=v"(v)
                 : "v"(wsc[ct]), "v"(wbs[ct]), "s"(0x07060302u));
    if (r == 0) fbq[st][ct].x = v;
    else if (r == 1) fbq[st][ct].y = v;
    else if (r == 2) fbq[st][ct].z = v;
    else fbq[st][ct].w = v;
  };
  auto widen_quarter = [&](int buf, int st, int ct, int r) __attribute__((always_inline)) {
    widen_quarter_a(buf, st, ct, r);
    widen_quarter_b(st, ct, r);
  };
  if constexpr (BCODES) {
    // K tiles 0 and 1 in full; K step 0 of K tile 0 widened
    set_b_tile(0);
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int i = 0; i < 5; ++i) load_codes_half(b, st, i, b_kbase + (size_t)b * 1024, s_kbase + (size_t)b * 128);
    b_kt = 2;
    wait_vmcnt<0>();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
      set_scale(0, 0, ct);
#pragma unroll
      for (int r = 0; r < 4; ++r) widen_quarter(0, 0, ct, r);
    }
  } else if constexpr (BPACK) {
    set_b_tile(0);
#pragma unroll
    for (int i = 0; i < 8; ++i) load_16_untracked(fb[0][i >> 1][i & 1], boff[i & 3], b_kbase + (size_t)(i >> 2) * 1024);
    b_kt = 1;
    wait_vmcnt<0>();
    __builtin_amdgcn_sched_barrier(0);
  } else {
    wait_vmcnt<kWaveCopies + kCopiesB>();  // K tile 0 landed; K tile 1 may still be in flight
  }
  asm volatile("s_barrier" ::: "memory");
  if constexpr (!BPACK) {
    // fragment registers of the plain forms: fr[q][0..3] = the four A row tiles of quarter q (K step q / 2, rows
    // 64 * (q % 2) .. + 64 of the wavefront's 128), fr[2 * ks + c / 4][4 + c % 4] = B column tile c of K step ks
#pragma unroll
    for (int f = 0; f < 4; ++f) fr[0][f] = load_frag16(0, 0, f);
    if constexpr (HALFN) {
      // narrow form: four B column tiles per K step, fr[2 * ks + c / 2][4 + c % 2]
#pragma unroll
      for (int c = 0; c < 4; ++c) fr[c >> 1][4 + (c & 1)] = load_frag16(0, 0, 8 + c);
    } else {
#pragma unroll
      for (int c = 0; c < 8; ++c) fr[c >> 2][4 + (c & 3)] = load_frag16(0, 0, 8 + c);
    }
  } else {
#pragma unroll
    for (int f = 0; f < 8; ++f) fr[0][f] = load_frag(0, 0, f);
  }
  int stage = 0;
  // BPACK form of the K iteration.  The wavefront has two kinds of loads in flight, the B fragment loads into
  // registers and the A copies into LDS.  Each kind retires in order, but the two kinds do NOT retire in order with
  // respect to each other: a younger register load can complete before an older LDS copy (with "all but the 16
  // youngest" as the hand-over test, A tiles were read before they had landed, on shapes whose B image often misses the
  // cache).  One counter covers both, so "at most n outstanding" proves that an A copy has landed only if at least
  // n + 1 younger *A copies* would otherwise have to be pending with it.  Hence four stages of A: the copy stream runs
  // three K tiles ahead, so when a hand-over needs the next K tile, the 16 copies of the two K tiles after it have
  // been issued, and the hand-over waits for "at most 16 outstanding": the next K tile has landed (its copies are older
  // than those 16), while the young copies and up to that many B loads fly on across the barrier.  The B fragments are
  // proven the same way, by counting the *register loads* issued after them.
  // bf16 image: a K tile is four quarters q of 32 matrix instructions 16x16x32: K step q / 2 (32 of the 64 K),
  // rows 128 * (q % 2) .. + 128 (8 row tiles of 16) times the 4 column tiles of 16.  Slot t of a quarter (16 slots)
  // issues the two instructions of row tile t / 2 on the column tiles 2 * (t % 2) and 2 * (t % 2) + 1, with the other
  // work between them.  The B loads of a K tile are issued in the order [K step][column tile]; quarters 0 and 1 need
  // the first four (proven by "at most 4 outstanding" at the head of the K tile: the other four of the batch are
  // younger), quarters 2 and 3 the last four (at most 8 outstanding at the head of quarter 2: the 8 of the next batch,
  // issued during quarter 0, are younger).
  //   quarter 0: LDS reads of quarter 1 (8) and the 8 B loads of the next K tile (their registers were last read one K
  //              tile ago), one each per slot 0..7
  //   quarter 1: LDS reads of quarters 2 and 3 (16); the first 4 of the 8 A copies of the K tile three ahead into the
  //              stage vacated at the previous hand-over, one every fourth slot
  //   quarter 2: the other 4 A copies; then the hand-over: at most 16 loads outstanding, own LDS reads complete, barrier
  //   quarter 3: LDS reads of quarter 0 of the next K tile (8)
  // A wait "at most n outstanding" completes everything but the n youngest operations of either kind.  With all 8 A
  // copies issued in quarter 1 the 8 youngest at the head of quarter 2 were those copies, and the wait there also
  // completed the B loads issued in quarter 0, a third of a K tile after their issue: 8 % of the time at K = 11008,
  // where the B image comes from further away.  With 4 copies issued after that wait, the 8 youngest at the wait are 4
  // copies and the last 4 B loads.
  // Stores of an epilogue only make the waits of the next output tile's first K tile conservative.
  auto k_iteration_b = [&](auto&& advance, auto bufc) __attribute__((always_inline)) {
    constexpr int NB = decltype(bufc)::value;
    const unsigned char* bsrc = b_kbase + (size_t)b_kt * 2048;
    const int stage_next = next_of(stage);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (q == 0) wait_vmcnt<4>();
      else if (q == 2) wait_vmcnt<8>();
      // A matrix instruction has no side effect the compiler would order against the wait: without this it hoists the
      // quarter's first one above the wait that proves its fragment.
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        const int it = (q & 1) * 8 + (t >> 1), jt = 2 * (t & 1), fx = (q >> 1) * 2 + (t & 1);
        mfma16_acc(acc16[it][jt], fb[NB][fx][0], fr[q][t >> 1]);
        if (q == 0) {
          if (t < 8) fr[1][t] = load_frag(stage, 1, t);
        } else if (q == 1) {
          if (t < 8) fr[2][t] = load_frag(stage, 2, t);
          else fr[3][t - 8] = load_frag(stage, 3, t - 8);
        } else if (q == 3) {
          if (t < 8) fr[0][t] = load_frag(stage_next, 0, t);
        }
        __builtin_amdgcn_sched_barrier(0);
        mfma16_acc(acc16[it][jt + 1], fb[NB][fx][1], fr[q][t >> 1]);
        if (q == 0) {
          if (t < 8) load_16_untracked(fb[NB ^ 1][t >> 1][t & 1], boff[t & 3], bsrc + (size_t)(t >> 2) * 1024);
        } else if (q == 1) {
          if ((t & 3) == 3) issue_copy((t >> 2) * 2);
        } else if (q == 2) {
          if ((t & 3) == 1) issue_copy(8 + (t >> 2) * 2);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (q == 2) {
        wait_vmcnt<(kStagesB - 2) * kWaveCopies>();
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    advance();
    stage = stage_next;
    ++b_kt;
  };
  // BCODES form.  The matrix instructions of quarter q read the widened fragments fbq[q / 2][column tile]; the codes
  // themselves are read only by the widening, so a half of a code buffer is free again as soon as its K step has been
  // widened, and the loads run a K tile and a half ahead of their use with two buffers:
  //   quarter 0: LDS reads of quarters 1 and 2 (16); slots 0..4: the loads of K step 0 of the K tile after next (scale
  //              dword + 4 fragments of 8 bytes per lane) into this buffer's K step 0 half (widened during quarter 3 of
  //              the previous K tile); before slot 12: K step 1 of this K tile has landed; slots 12..15: its scales
  //   quarter 1: LDS reads of quarter 3 (8); widening of K step 1 of this K tile, one quarter register per slot; 4 A copies
  //   quarter 2: slots 0..4: the loads of K step 1 of the K tile after next into this buffer's K step 1 half; 4 A
  //              copies; before slot 12: K step 0 of the next K tile has landed; slots 12..15: its scales; hand-over
  //   quarter 3: LDS reads of quarter 0 of the next K tile (8); widening of K step 0 of the next K tile
  // Register loads in issue order: .. H0(k+1) H1(k+1) | H0(k+2) [quarter 0] H1(k+2) [quarter 2] with 5 loads per half.
  // The wait in quarter 0 needs H1(k), after which H0(k+1), H1(k+1), H0(k+2) = 15 register loads were issued; the wait
  // in quarter 2 needs H0(k+1), followed by H1(k+1), H0(k+2), H1(k+2) = 15: "at most 15 outstanding" both times.  What
  // these waits complete besides is at least three quarters of a K tile old.  The hand-over is the one of the bf16
  // image form (the 16 youngest of the A copies belong to later K tiles).
  auto k_iteration_c = [&](auto&& advance, auto bufc) __attribute__((always_inline)) {
    constexpr int NB = decltype(bufc)::value;
    const unsigned char* bsrc = b_kbase + (size_t)b_kt * 1024;
    const unsigned char* ssrc = s_kbase + (size_t)b_kt * 128;
    const int stage_next = next_of(stage);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        if ((q == 0 || q == 2) && t == 12) {
          wait_vmcnt<15>();
          __builtin_amdgcn_sched_barrier(0);  // nothing that reads the codes or scales may be hoisted above the wait
        }
        const int it = (q & 1) * 8 + (t >> 1), jt = 2 * (t & 1);
        mfma16_acc(acc16[it][jt], __builtin_bit_cast(bf16x8_t, fbq[q >> 1][jt]), fr[q][t >> 1]);
        if (q == 0) {
          if (t < 8) fr[1][t] = load_frag(stage, 1, t);
          else fr[2][t - 8] = load_frag(stage, 2, t - 8);
          if (t >= 12) set_scale_a(NB, 1, t - 12);
        } else if (q == 1) {
          if (t < 8) fr[3][t] = load_frag(stage, 3, t);
          widen_quarter_a(NB, 1, t >> 2, t & 3);
        } else if (q == 2) {
          if (t >= 12) set_scale_a(NB ^ 1, 0, t - 12);
        } else {
          if (t < 8) fr[0][t] = load_frag(stage_next, 0, t);
          widen_quarter_a(NB ^ 1, 0, t >> 2, t & 3);
        }
        __builtin_amdgcn_sched_barrier(0);
        mfma16_acc(acc16[it][jt + 1], __builtin_bit_cast(bf16x8_t, fbq[q >> 1][jt + 1]), fr[q][t >> 1]);
        if (q == 0) {
          if (t < 5) load_codes_half(NB, 0, t, bsrc, ssrc);
          if (t >= 12) set_scale_b(t - 12);
        } else if (q == 1) {
          widen_quarter_b(1, t >> 2, t & 3);
          if ((t & 3) == 3) issue_copy((t >> 2) * 2);
        } else if (q == 2) {
          if (t < 5) load_codes_half(NB, 1, t, bsrc, ssrc);
          else if (t < 12 && (t & 1)) issue_copy(8 + ((t - 5) >> 1) * 2);
          if (t >= 12) set_scale_b(t - 12);
        } else {
          widen_quarter_b(0, t >> 2, t & 3);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (q == 2) {
        wait_vmcnt<(kStagesB - 2) * kWaveCopies>();
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    advance();
    stage = stage_next;
    ++b_kt;
  };
  // Plain form (both operands through LDS, wavefronts 2 x 2: 8 x 8 tiles of 16 x 16 each).  A K tile is four quarters
  // of 32 matrix instructions: K step q / 2, A row tiles 4 * (q % 2) .. + 4 against the 8 B column tiles; slot t of a
  // quarter issues row tile t / 4 against the column tiles 2 * (t % 4) and 2 * (t % 4) + 1.
  //   quarter 0: the 16 LDS reads the rest of this K tile needs (A of quarter 1; A of quarter 2 and B of K step 1)
  //   quarter 1: the 4 reads of A of quarter 3; then the hand-over as described above
  //   quarter 2: the 12 reads of the next K tile's quarter 0 (A) and K step 0 (B); 8 of the 16 copies
  //   quarter 3: the other 8 copies
  auto k_iteration = [&](auto&& advance) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        const int ks = q >> 1, it = (q & 1) * 4 + (t >> 2), jt = 2 * (t & 3);
        mfma16_acc(acc16[it][jt], fr[2 * ks + (jt >> 2)][4 + (jt & 3)], fr[q][t >> 2]);
        if (q == 0) {
          if (t < 4) fr[1][t] = load_frag16(stage, 0, 4 + t);
          else if (t < 8) fr[2][t - 4] = load_frag16(stage, 1, t - 4);
          else fr[2 + ((t - 8) >> 2)][4 + ((t - 8) & 3)] = load_frag16(stage, 1, t);
        } else if (q == 1) {
          if (t < 4) fr[3][t] = load_frag16(stage, 1, 4 + t);
        } else if (q == 2) {
          if (t < 4) fr[0][t] = load_frag16(stage ^ 1, 0, t);
          else if (t < 12) fr[(t - 4) >> 2][4 + ((t - 4) & 3)] = load_frag16(stage ^ 1, 0, 4 + t);
        }
        __builtin_amdgcn_sched_barrier(0);
        mfma16_acc(acc16[it][jt + 1], fr[2 * ks + ((jt + 1) >> 2)][4 + ((jt + 1) & 3)], fr[q][t >> 2]);
        if (q == 2) {
          if (t & 1) issue_copy(t >> 1);
        } else if (q == 3) {
          if (t & 1) issue_copy(8 + (t >> 1));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (q == 1) {
        wait_vmcnt<0>();
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    advance();
    stage ^= 1;
  };
  // Narrow form (output tiles of 256 x 128; wavefronts 2 x 2: 8 x 4 tiles of 16 x 16 each): quarters of 16 matrix
  // instructions in 8 slots, slot t on row tile t / 2 of the quarter's four against the column tiles 2 * (t % 2) and
  // 2 * (t % 2) + 1; fr[q][0..3] = A of quarter q, fr[2 * ks + c / 2][4 + c % 2] = B column tile c of K step ks.
  //   quarter 0: the 12 LDS reads the rest of the K tile needs (A of quarters 1 and 2 in the first gap of a slot, B of
  //              K step 1 in the second); quarter 1: A of quarter 3; hand-over
  //   quarters 2, 3: the 8 reads of the next K tile's quarter 0 and K step 0; the 12 copies of the K tile after next,
  //              one per slot (slots of the 4 copies that B does not have stay empty)
  auto k_iteration_h = [&](auto&& advance) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const int ks = q >> 1, it = (q & 1) * 4 + (t >> 1), jt = 2 * (t & 1);
        mfma16_acc(acc16[it][jt], fr[2 * ks + (jt >> 1)][4], fr[q][t >> 1]);
        if (q == 0) {
          if (t < 4) fr[1][t] = load_frag16(stage, 0, 4 + t);
          else fr[2][t - 4] = load_frag16(stage, 1, t - 4);
        } else if (q == 1) {
          if (t < 4) fr[3][t] = load_frag16(stage, 1, 4 + t);
        } else if (q == 2) {
          if (t < 4) fr[0][t] = load_frag16(stage ^ 1, 0, t);
          else fr[(t - 4) >> 1][4 + ((t - 4) & 1)] = load_frag16(stage ^ 1, 0, 8 + (t - 4));
        }
        __builtin_amdgcn_sched_barrier(0);
        mfma16_acc(acc16[it][jt + 1], fr[2 * ks + (jt >> 1)][5], fr[q][t >> 1]);
        if (q == 0) {
          if (t < 4) fr[2 + (t >> 1)][4 + (t & 1)] = load_frag16(stage, 1, 8 + t);
        } else if (q == 2) {
          issue_copy(t);
        } else if (q == 3) {
          issue_copy(8 + t);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (q == 1) {
        wait_vmcnt<0>();
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    advance();
    stage ^= 1;
  };
  auto k_iter_plain = [&](auto&& advance) __attribute__((always_inline)) {
    if constexpr (HALFN) k_iteration_h(advance);
    else k_iteration(advance);
  };
  for (int ord = 0; ord < n_my; ++ord) {
    if constexpr (BPACK) {
      // two K tiles per trip (the fragment buffers alternate); the copy stream as in the plain form below, the B
      // stream one K tile ahead: it moves on to the next output tile before the last K tile of this one
      auto iter = [&](auto bufc, auto&& advance) __attribute__((always_inline)) {
        if constexpr (BCODES) k_iteration_c(advance, bufc);
        else k_iteration_b(advance, bufc);
      };
      // while the copy stream (kStagesB - 1 = 3 K tiles ahead) stays inside this output tile it advances without
      // branches; over the last four K tiles (both, when there are only two) it takes the general step, which moves
      // it on to the next output tile
      int kt = 0;
#pragma unroll 1
      for (; kt + 6 <= nk; kt += 2) {
        iter(std::integral_constant<int, 0>{}, step_within_tile);
        iter(std::integral_constant<int, 1>{}, step_within_tile);
      }
#pragma unroll 1
      for (; kt < nk; kt += 2) {
        // the B stream moves on to the next output tile: one K tile ahead (bf16 image), two ahead (codes)
        if constexpr (BCODES) {
          if (kt + 2 >= nk) set_b_tile(ord + 1);
        }
        iter(std::integral_constant<int, 0>{}, advance_copy_stream);
        if constexpr (!BCODES) {
          if (kt + 2 >= nk) set_b_tile(ord + 1);
        }
        iter(std::integral_constant<int, 1>{}, advance_copy_stream);
      }
    } else if constexpr (STREAM) {
      // the copy stream stands at K tile S of this output tile (or, if nk == S, at K tile 0 of the next)
#pragma unroll 1
      for (int kt = 0; kt < nk - S; ++kt) k_iter_plain(step_within_tile);
      // it moves on to the next output tile (past the last one: harmless re-copies of its first K tiles)
      set_copy_tile(ord + 1);
      c_kt = 0;
#pragma unroll 1
      for (int kt = 0; kt < S; ++kt) k_iter_plain(step_within_tile);
    } else {
      for (int kt = 0; kt < nk; ++kt) k_iter_plain(advance_copy_stream);
    }
    epilogue(ord);
    zero_acc();
    {
      const int l = lane_now();
      frag_row = l & 15;
      kgrp = l >> 4;
    }
  }
  wait_vmcnt<0>();  // no copy may still be in flight towards LDS when the work-group retires
}

// number of work-groups of the persistent kernel: one per CU (each takes the whole LDS of its CU)
int persistent_grid_bf16(int total_tiles) {
  const int n_cu = device_cu_count();
  if (n_cu <= 0) return -1;
  return total_tiles < n_cu ? total_tiles : n_cu;
}

// launch of the persistent kernel for the work items of p (tiles x K ranges), output dtype out_dtype
int launch_gemm_bf16(const GemmParams& p, int out_dtype, hipStream_t st, bool bpack = false, bool bcodes = false,
                     bool batched = false) {
  const size_t lds_bytes = (size_t)kLdsBytes;
  const int nwg = persistent_grid_bf16(p.tiles_m * p.tiles_n * (batched ? p.batches : p.splits));
  if (nwg <= 0) return MASE_ERR_LAUNCH;
  const dim3 grid((unsigned)nwg), block(kGemmThreads);
  const bool stream_fits = p.kc / BK >= S;
#define MASE_GEMM_LAUNCH(DT_, STREAM_)                                                                            \
  do {                                                                                                            \
    static std::atomic<uint64_t> attr_done{0};                                                                    \
    const void* k = (const void*)gemm_bf16_tn_kernel<DT_, STREAM_>;                                               \
    if (!set_dynamic_lds_once(attr_done, k, (int)lds_bytes)) return MASE_ERR_LAUNCH;                              \
    hipLaunchKernelGGL((gemm_bf16_tn_kernel<DT_, STREAM_>), grid, block, lds_bytes, st, p);                       \
  } while (0)
  if (batched) {
    const bool halfn = p.N <= 128;  // the caller has counted tiles_n in tiles of 128 columns then
#define MASE_GEMM_LAUNCH_BATCHED(DT_, STREAM_, HALFN_)                                                            \
  do {                                                                                                            \
    static std::atomic<uint64_t> attr_done{0};                                                                    \
    const void* k = (const void*)gemm_bf16_tn_kernel<DT_, STREAM_, false, false, true, HALFN_>;                   \
    if (!set_dynamic_lds_once(attr_done, k, (int)lds_bytes)) return MASE_ERR_LAUNCH;                              \
    hipLaunchKernelGGL((gemm_bf16_tn_kernel<DT_, STREAM_, false, false, true, HALFN_>), grid, block, lds_bytes,   \
                       st, p);                                                                                    \
  } while (0)
#define MASE_GEMM_LAUNCH_BATCHED_DT(STREAM_, HALFN_)                                                              \
  do {                                                                                                            \
    if (out_dtype == MASE_DT_F32) MASE_GEMM_LAUNCH_BATCHED(MASE_DT_F32, STREAM_, HALFN_);                         \
    else if (out_dtype == MASE_DT_BF16) MASE_GEMM_LAUNCH_BATCHED(MASE_DT_BF16, STREAM_, HALFN_);                  \
    else MASE_GEMM_LAUNCH_BATCHED(MASE_DT_F16, STREAM_, HALFN_);                                                  \
  } while (0)
    if (stream_fits && halfn) MASE_GEMM_LAUNCH_BATCHED_DT(true, true);
    else if (stream_fits) MASE_GEMM_LAUNCH_BATCHED_DT(true, false);
    else if (halfn) MASE_GEMM_LAUNCH_BATCHED_DT(false, true);
    else MASE_GEMM_LAUNCH_BATCHED_DT(false, false);
#undef MASE_GEMM_LAUNCH_BATCHED_DT
#undef MASE_GEMM_LAUNCH_BATCHED
  } else if (bpack && bcodes) {
    if (!stream_fits || ((p.kc / BK) & 1) != 0) return MASE_ERR_SHAPE;
#define MASE_GEMM_LAUNCH_C(DT_)                                                                                   \
  do {                                                                                                            \
    static std::atomic<uint64_t> attr_done{0};                                                                    \
    const void* k = (const void*)gemm_bf16_tn_kernel<DT_, true, true, true>;                                      \
    if (!set_dynamic_lds_once(attr_done, k, (int)lds_bytes)) return MASE_ERR_LAUNCH;                              \
    hipLaunchKernelGGL((gemm_bf16_tn_kernel<DT_, true, true, true>), grid, block, lds_bytes, st, p);              \
  } while (0)
    if (out_dtype == MASE_DT_F32) MASE_GEMM_LAUNCH_C(MASE_DT_F32);
    else if (out_dtype == MASE_DT_BF16) MASE_GEMM_LAUNCH_C(MASE_DT_BF16);
    else MASE_GEMM_LAUNCH_C(MASE_DT_F16);
#undef MASE_GEMM_LAUNCH_C
  } else if (bpack) {
    if (!stream_fits || ((p.kc / BK) & 1) != 0) return MASE_ERR_SHAPE;
#define MASE_GEMM_LAUNCH_B(DT_)                                                                                   \
  do {                                                                                                            \
    static std::atomic<uint64_t> attr_done{0};                                                                    \
    const void* k = (const void*)gemm_bf16_tn_kernel<DT_, true, true>;                                            \
    if (!set_dynamic_lds_once(attr_done, k, (int)lds_bytes)) return MASE_ERR_LAUNCH;                              \
    hipLaunchKernelGGL((gemm_bf16_tn_kernel<DT_, true, true>), grid, block, lds_bytes, st, p);                    \
  } while (0)
    if (out_dtype == MASE_DT_F32) MASE_GEMM_LAUNCH_B(MASE_DT_F32);
    else if (out_dtype == MASE_DT_BF16) MASE_GEMM_LAUNCH_B(MASE_DT_BF16);
    else MASE_GEMM_LAUNCH_B(MASE_DT_F16);
#undef MASE_GEMM_LAUNCH_B
  } else if (stream_fits) {
    if (out_dtype == MASE_DT_F32) MASE_GEMM_LAUNCH(MASE_DT_F32, true);
    else if (out_dtype == MASE_DT_BF16) MASE_GEMM_LAUNCH(MASE_DT_BF16, true);
    else MASE_GEMM_LAUNCH(MASE_DT_F16, true);
  } else {
    if (out_dtype == MASE_DT_F32) MASE_GEMM_LAUNCH(MASE_DT_F32, false);
    else if (out_dtype == MASE_DT_BF16) MASE_GEMM_LAUNCH(MASE_DT_BF16, false);
    else MASE_GEMM_LAUNCH(MASE_DT_F16, false);
  }
#undef MASE_GEMM_LAUNCH
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

// C[m][n] = sum over the K ranges, in order, of P[range][m][n]  (+ bias[n]), converted to the output dtype
template <int OUT_DT>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float* __restrict__ P, void* __restrict__ C,
                                                                 const void* __restrict__ bias, int bias_dtype,
                                                                 size_t mn, int N, int splits) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= mn) return;
  float s = 0.0f;
  for (int k = 0; k < splits; ++k) s += P[(size_t)k * mn + i];
  if (bias != nullptr) s += load_bias(bias, bias_dtype, (int)(i % (size_t)N));
  if constexpr (OUT_DT == MASE_DT_F32) ((float*)C)[i] = s;
  else if constexpr (OUT_DT == MASE_DT_BF16) ((uint16_t*)C)[i] = (uint16_t)f32_to_bf16_bits(s);
  else ((uint16_t*)C)[i] = (uint16_t)f32_to_f16_bits(s);
}

// B[N, K] row-major -> fragment-ordered image: 1 KB blocks [column tile of 16][K step of 32][lane][8 bf16]; lane l
// of a block holds B[tile*16 + l%16][step*32 + 8*(l/16) .. +8], rows beyond N (the image holds a multiple of 32) are zero
__global__ __launch_bounds__(256) void gemm_pack_b_kernel(const uint4* __restrict__ B, uint4* __restrict__ out, int N,
                                                          int K, size_t granules) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= granules) return;
  const int lane = (int)(g & 63);
  const size_t blk = g >> 6;
  const int steps = K / 32;
  const int nt = (int)(blk / (size_t)steps), ks = (int)(blk % (size_t)steps);
  const int row = nt * 16 + (lane & 15);
  uint4 v = make_uint4(0, 0, 0, 0);
  if (row < N) v = B[((size_t)row * K + (size_t)ks * 32 + 8 * (lane >> 4)) / 8];
  out[g] = v;
}

// MXINT8 weight [N, K] (int8 codes, one scale byte per 32 along K) -> fragment-ordered images for the BCODES kernel:
// codes: 512-byte blocks [column tile of 16][K step of 32][lane][8 bytes], lane l of a block holding the codes of
// column tile*16 + l%16 at K = step*32 + 8*(l/16) .. +8, each plus 128 (an unsigned byte); columns beyond N (the image
// holds a multiple of 32) hold 128 (zero).  scales: 128-byte blocks [64 columns][K tile of 64][column % 16][8 bytes],
// byte 4 * s + c of a lane's eight = the scale byte of column 64 * group + 16 * c + column % 16 in block 2 * tile + s;
// columns beyond N (the image holds a multiple of 64) have scale 0.
__global__ __launch_bounds__(256) void gemm_pack_codes_kernel(const uint2* __restrict__ codes, uint2* __restrict__ img, int N,
                                                              int K, size_t granules) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= granules) return;
  const int lane = (int)(g & 63);
  const size_t blk = g >> 6;
  const int steps = K / 32;
  const int nt = (int)(blk / (size_t)steps), ks = (int)(blk % (size_t)steps);
  const int row = nt * 16 + (lane & 15);
  uint2 v = make_uint2(0x80808080u, 0x80808080u);
  if (row < N) {
    v = codes[((size_t)row * K + (size_t)ks * 32 + 8 * (lane >> 4)) / 8];
    v.x ^= 0x80808080u;
    v.y ^= 0x80808080u;
  }
  img[g] = v;
}
// one work-item per (64 columns, K tile, column % 16): its eight scale bytes
__global__ __launch_bounds__(256) void gemm_pack_scales_kernel(const uint8_t* __restrict__ scales, uint2* __restrict__ simg, int N,
                                                               int K, size_t items) {
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= items) return;
  const int c16 = (int)(g & 15);
  const size_t blk = g >> 4;
  const int ktiles = K / 64;
  const int g64 = (int)(blk / (size_t)ktiles), kt = (int)(blk % (size_t)ktiles);
  uint32_t w[2] = {0u, 0u};
#pragma unroll
  for (int st = 0; st < 2; ++st)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int row = g64 * 64 + c * 16 + c16;
      if (row < N) w[st] |= (uint32_t)scales[(size_t)row * (K / 32) + (size_t)kt * 2 + st] << (8 * c);
    }
  simg[g] = make_uint2(w[0], w[1]);
}

// K ranges for a product whose output tiles alone would leave most CUs idle: as many as fill the machine once, each a
// whole number of K tiles and at least 4 of them; 1 when the tiles already fill three quarters of the CUs
int splitk_ranges(size_t M, size_t N, size_t K) {
  const int n_cu = persistent_grid_bf16(1 << 30);
  if (n_cu <= 0 || K % BK != 0) return 1;
  const long tiles = (long)((M + BM - 1) / BM) * (long)((N + BN - 1) / BN);
  if (tiles * 4 >= (long)n_cu * 3) return 1;
  const int kt = (int)(K / BK);
  int best = 1;
  for (int s = 2; s <= 16 && (long)s * tiles <= n_cu; ++s)
    if (kt % s == 0 && kt / s >= 4) best = s;
  return best;
}

}  // namespace
}  // namespace mase

extern "C" int mase_gemm_bf16_tn(const void* A, const void* B, const void* bias, void* C, size_t M, size_t N, size_t K,
                                 int out_dtype, int bias_dtype, void* stream) {
  using namespace mase;
  if (M == 0 || N == 0) return MASE_OK;
  if (A == nullptr || B == nullptr || C == nullptr) return MASE_ERR_NULL;
  if (K == 0 || (K % BK) != 0 || M > (1u << 30) || N > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  // the kernel addresses each operand with a 32-bit byte offset from its base
  if ((unsigned long long)M * K * 2 > 0xFFFFFFFFull || (unsigned long long)N * K * 2 > 0xFFFFFFFFull) return MASE_ERR_SHAPE;
  if (!aligned16(A) || !aligned16(B)) return MASE_ERR_ALIGN;
  if (out_dtype < 0 || out_dtype > 2 || (bias != nullptr && (bias_dtype < 0 || bias_dtype > 2))) return MASE_ERR_DTYPE;
  GemmParams p;
  p.A = (const unsigned char*)A;
  p.B = (const unsigned char*)B;
  p.Bs = nullptr;
  p.bias = bias;
  p.C = C;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.bias_dtype = bias_dtype;
  p.tiles_m = (int)((M + BM - 1) / BM);
  p.tiles_n = (int)((N + BN - 1) / BN);
  p.splits = 1;
  p.kc = (int)K;
  return launch_gemm_bf16(p, out_dtype, (hipStream_t)stream);
}

extern "C" int mase_gemm_bf16_tn_batched(const void* A, const void* B, void* C, size_t batch_outer, size_t batch_inner,
                                         size_t M, size_t N, size_t K, size_t lda, size_t ldb, size_t ldc,
                                         size_t a_stride_outer, size_t a_stride_inner, size_t b_stride_outer,
                                         size_t b_stride_inner, size_t c_stride_outer, size_t c_stride_inner,
                                         int out_dtype, void* stream) {
  using namespace mase;
  if (M == 0 || N == 0 || batch_outer == 0 || batch_inner == 0) return MASE_OK;
  if (A == nullptr || B == nullptr || C == nullptr) return MASE_ERR_NULL;
  if (out_dtype < 0 || out_dtype > 2) return MASE_ERR_DTYPE;
  if (K == 0 || (K % BK) != 0 || M > (1u << 30) || N > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  if (lda < K || ldb < K || ldc < N) return MASE_ERR_SHAPE;
  const unsigned long long esz = out_dtype == MASE_DT_F32 ? 4 : 2;
  // operand rows are fetched in 16-byte pieces at 32-bit byte offsets from the product's operand base; output pieces
  // of 16 bytes are stored whole where they lie inside a row
  if ((unsigned long long)M * lda * 2 > 0xFFFFFFFFull || (unsigned long long)N * ldb * 2 > 0xFFFFFFFFull) return MASE_ERR_SHAPE;
  const size_t bn = N <= 128 ? 128 : BN;  // products of at most 128 columns take output tiles of 256 x 128
  const unsigned long long tiles = (unsigned long long)((M + BM - 1) / BM) * ((N + bn - 1) / bn);
  if (tiles * batch_outer * batch_inner > (1ull << 30) || batch_inner > (1u << 30)) return MASE_ERR_SHAPE;
  if (!aligned16(A) || !aligned16(B) || !aligned16(C)) return MASE_ERR_ALIGN;
  if (lda % 8 || ldb % 8 || a_stride_outer % 8 || a_stride_inner % 8 || b_stride_outer % 8 || b_stride_inner % 8)
    return MASE_ERR_ALIGN;
  if ((ldc * esz) % 16 || (c_stride_outer * esz) % 16 || (c_stride_inner * esz) % 16) return MASE_ERR_ALIGN;
  GemmParams p;
  p.A = (const unsigned char*)A;
  p.B = (const unsigned char*)B;
  p.Bs = nullptr;
  p.bias = nullptr;
  p.C = C;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.bias_dtype = 0;
  p.tiles_m = (int)((M + BM - 1) / BM);
  p.tiles_n = (int)((N + bn - 1) / bn);
  p.splits = 1;
  p.kc = (int)K;
  p.batches = (int)(batch_outer * batch_inner);
  p.batch_inner = (int)batch_inner;
  p.a_so = a_stride_outer * 2; p.a_si = a_stride_inner * 2;
  p.b_so = b_stride_outer * 2; p.b_si = b_stride_inner * 2;
  p.c_so = c_stride_outer * esz; p.c_si = c_stride_inner * esz;
  p.lda = lda * 2; p.ldb = ldb * 2; p.ldc = ldc * esz;
  return launch_gemm_bf16(p, out_dtype, (hipStream_t)stream, false, false, true);
}

extern "C" size_t mase_gemm_bf16_tn_splitk_workspace_bytes(size_t M, size_t N, size_t K) {
  using namespace mase;
  if (M == 0 || N == 0 || K == 0) return 0;
  const int splits = splitk_ranges(M, N, K);
  return splits > 1 ? (size_t)splits * M * N * sizeof(float) : 0;
}

extern "C" int mase_gemm_bf16_tn_splitk(const void* A, const void* B, const void* bias, void* C, size_t M, size_t N,
                                        size_t K, int out_dtype, int bias_dtype, void* workspace, size_t workspace_bytes,
                                        void* stream) {
  using namespace mase;
  if (M == 0 || N == 0) return MASE_OK;
  const int splits = (K % BK == 0) ? splitk_ranges(M, N, K) : 1;
  if (splits <= 1) return mase_gemm_bf16_tn(A, B, bias, C, M, N, K, out_dtype, bias_dtype, stream);
  if (A == nullptr || B == nullptr || C == nullptr) return MASE_ERR_NULL;
  if (M > (1u << 30) || N > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  if ((unsigned long long)M * K * 2 > 0xFFFFFFFFull || (unsigned long long)N * K * 2 > 0xFFFFFFFFull) return MASE_ERR_SHAPE;
  if (!aligned16(A) || !aligned16(B)) return MASE_ERR_ALIGN;
  if (out_dtype < 0 || out_dtype > 2 || (bias != nullptr && (bias_dtype < 0 || bias_dtype > 2))) return MASE_ERR_DTYPE;
  const size_t need = (size_t)splits * M * N * sizeof(float);
  if (workspace == nullptr || workspace_bytes < need || (((uintptr_t)workspace) & 15u) != 0) return MASE_ERR_WORKSPACE;
  GemmParams p;
  p.A = (const unsigned char*)A;
  p.B = (const unsigned char*)B;
  p.Bs = nullptr;
  p.bias = nullptr;
  p.C = workspace;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.bias_dtype = 0;
  p.tiles_m = (int)((M + BM - 1) / BM);
  p.tiles_n = (int)((N + BN - 1) / BN);
  p.splits = splits;
  p.kc = (int)(K / splits);
  hipStream_t st = (hipStream_t)stream;
  const int rc = launch_gemm_bf16(p, MASE_DT_F32, st);
  if (rc != MASE_OK) return rc;
  const size_t mn = M * N;
  const dim3 grid(blocks_for(mn, (size_t)256)), block(256);
  const float* P = (const float*)workspace;
  if (out_dtype == MASE_DT_F32)
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel<MASE_DT_F32>, grid, block, 0, st, P, C, bias, bias_dtype, mn, (int)N, splits);
  else if (out_dtype == MASE_DT_BF16)
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel<MASE_DT_BF16>, grid, block, 0, st, P, C, bias, bias_dtype, mn, (int)N, splits);
  else
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel<MASE_DT_F16>, grid, block, 0, st, P, C, bias, bias_dtype, mn, (int)N, splits);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

extern "C" size_t mase_gemm_bf16_packed_bytes(size_t N, size_t K) {
  if (N == 0 || K == 0 || (K % 32) != 0) return 0;
  return ((N + 31) / 32) * 32 * K * 2;
}

extern "C" int mase_gemm_bf16_pack_b(const void* B, void* B_packed, size_t N, size_t K, void* stream) {
  using namespace mase;
  if (N == 0 || K == 0) return MASE_OK;
  if (B == nullptr || B_packed == nullptr) return MASE_ERR_NULL;
  if ((K % 32) != 0 || N > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  if (!aligned16(B) || !aligned16(B_packed)) return MASE_ERR_ALIGN;
  const size_t granules = mase_gemm_bf16_packed_bytes(N, K) / 16;
  hipLaunchKernelGGL(gemm_pack_b_kernel, dim3(blocks_for(granules, (size_t)256)), dim3(256), 0, (hipStream_t)stream,
                     (const uint4*)B, (uint4*)B_packed, (int)N, (int)K, granules);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

extern "C" int mase_gemm_bf16_tn_packed(const void* A, const void* B_packed, const void* bias, void* C, size_t M,
                                        size_t N, size_t K, int out_dtype, int bias_dtype, void* stream) {
  using namespace mase;
  if (M == 0 || N == 0) return MASE_OK;
  if (A == nullptr || B_packed == nullptr || C == nullptr) return MASE_ERR_NULL;
  if (K == 0 || (K % (2 * BK)) != 0 || M > (1u << 30) || N > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  if ((unsigned long long)M * K * 2 > 0xFFFFFFFFull || (unsigned long long)mase_gemm_bf16_packed_bytes(N, K) > 0xFFFFFFFFull)
    return MASE_ERR_SHAPE;
  if (!aligned16(A) || !aligned16(B_packed)) return MASE_ERR_ALIGN;
  if (out_dtype < 0 || out_dtype > 2 || (bias != nullptr && (bias_dtype < 0 || bias_dtype > 2))) return MASE_ERR_DTYPE;
  GemmParams p;
  p.A = (const unsigned char*)A;
  p.B = (const unsigned char*)B_packed;
  p.Bs = nullptr;
  p.bias = bias;
  p.C = C;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.bias_dtype = bias_dtype;
  p.tiles_m = (int)((M + BM - 1) / BM);
  p.tiles_n = (int)((N + BN - 1) / BN);
  p.splits = 1;
  p.kc = (int)K;
  return launch_gemm_bf16(p, out_dtype, (hipStream_t)stream, true);
}

extern "C" size_t mase_gemm_mxint8_packed_code_bytes(size_t N, size_t K) {
  if (N == 0 || K == 0 || (K % 128) != 0) return 0;
  return ((N + 31) / 32) * 32 * K;
}

extern "C" size_t mase_gemm_mxint8_packed_scale_bytes(size_t N, size_t K) {
  if (N == 0 || K == 0 || (K % 128) != 0) return 0;
  return ((N + 63) / 64) * 64 * (K / 32);
}

extern "C" int mase_gemm_mxint8_pack_b(const int8_t* codes, const uint8_t* scales, void* code_image, void* scale_image,
                                       size_t N, size_t K, void* stream) {
  using namespace mase;
  if (N == 0 || K == 0) return MASE_OK;
  if (codes == nullptr || scales == nullptr || code_image == nullptr || scale_image == nullptr) return MASE_ERR_NULL;
  if ((K % 128) != 0 || N > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  if ((((uintptr_t)codes) & 7u) != 0 || !aligned16(code_image) || (((uintptr_t)scale_image) & 7u) != 0) return MASE_ERR_ALIGN;
  const size_t granules = mase_gemm_mxint8_packed_code_bytes(N, K) / 8;
  hipLaunchKernelGGL(gemm_pack_codes_kernel, dim3(blocks_for(granules, (size_t)256)), dim3(256), 0, (hipStream_t)stream,
                     (const uint2*)codes, (uint2*)code_image, (int)N, (int)K, granules);
  const size_t items = mase_gemm_mxint8_packed_scale_bytes(N, K) / 8;
  hipLaunchKernelGGL(gemm_pack_scales_kernel, dim3(blocks_for(items, (size_t)256)), dim3(256), 0, (hipStream_t)stream,
                     scales, (uint2*)scale_image, (int)N, (int)K, items);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

extern "C" int mase_gemm_mxint8_tn_packed(const void* A, const void* code_image, const void* scale_image, const void* bias,
                                          void* C, size_t M, size_t N, size_t K, int out_dtype, int bias_dtype,
                                          void* stream) {
  using namespace mase;
  if (M == 0 || N == 0) return MASE_OK;
  if (A == nullptr || code_image == nullptr || scale_image == nullptr || C == nullptr) return MASE_ERR_NULL;
  if (K == 0 || (K % (2 * BK)) != 0 || M > (1u << 30) || N > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  if ((unsigned long long)M * K * 2 > 0xFFFFFFFFull ||
      (unsigned long long)mase_gemm_mxint8_packed_code_bytes(N, K) > 0xFFFFFFFFull)
    return MASE_ERR_SHAPE;
  if (!aligned16(A) || !aligned16(code_image) || (((uintptr_t)scale_image) & 7u) != 0) return MASE_ERR_ALIGN;
  if (out_dtype < 0 || out_dtype > 2 || (bias != nullptr && (bias_dtype < 0 || bias_dtype > 2))) return MASE_ERR_DTYPE;
  GemmParams p;
  p.A = (const unsigned char*)A;
  p.B = (const unsigned char*)code_image;
  p.Bs = (const unsigned char*)scale_image;
  p.bias = bias;
  p.C = C;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.bias_dtype = bias_dtype;
  p.tiles_m = (int)((M + BM - 1) / BM);
  p.tiles_n = (int)((N + BN - 1) / BN);
  p.splits = 1;
  p.kc = (int)K;
  return launch_gemm_bf16(p, out_dtype, (hipStream_t)stream, true, true);
}
