// C[M,N] = A[M,K] * B[N,K]^T (+ bias[N]) with MX-format operands on gfx950's block-scaled matrix instruction
// v_mfma_scale_f32_32x32x64_f8f6f4: A holds 8-bit codes (e4m3 or e5m2), B holds 8-bit or 4-bit (e2m1) codes,
// each with one E8M0 scale byte per 32 consecutive K elements, fp32 accumulation.
//
// This is the contraction of LinearMXFP.forward for formats the hardware has (the other formats go through
// the bf16 kernel).  Operand layout of the instruction (measured on the device with one-hot operands):
//   lane l holds row/column l%32; with g = l/32,
//   8-bit codes: registers 0-3 = K elements [16g, 16g+16), registers 4-7 = K elements [32+16g, 32+16g+16)
//   4-bit codes: registers 0-3 = K elements [32g, 32g+32), two per byte, even element in the low nibble
//   scales:      the byte selected in lane l scales K block g (elements [32g, 32g+32)) of row/column l%32
// and the hardware multiplies both scales into each block's partial product, so the result is the dot product
// of the dequantized operands.  Inside the instruction the 8 products of one register pair are aligned to
// the largest of them and truncated about 12 bits below its leading bit before they are added; sums across
// such groups of 8 and across instructions are carried in fp32.
//
// Schedule: the 256x256 tile and the 2x2 wavefronts of 4x4 MFMA tiles are those of the bf16 kernel
// (gemm_bf16.hip); the kernel is persistent (one work-group per CU walks its output tiles).  K tile 128: per stage A 256 x 128 B, B 256 x 64 B (4-bit) or 256 x 128 B (8-bit),
// plus 4 scale bytes per row for each operand = one dword per row per K tile.  Three stages when B is 4-bit
// (50 KB each), two when it is 8-bit (66 KB).  All of it travels HBM/L2 -> LDS with global_load_lds (16-byte
// form for codes, 4-byte form for scales); copies of tile t+S are issued while the last MFMAs of tile t run.
// A lane's scale dword is pre-shifted by 8*(l/32) so that K step s finds its byte at position 2s in both
// half-waves (the byte select of the instruction is an immediate).
#include "common.hpp"

#include <type_traits>

namespace mase {
namespace {

typedef int i32x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int kThreadsG = 256;

struct MxGemmParams {
  const unsigned char* A;
  const unsigned char* B;
  const unsigned char* SA;
  const unsigned char* SB;
  const void* bias;
  void* C;
  int M, N, K;
  int bias_dtype;
  int tiles_m, tiles_n;
};

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// one wavefront-wide async copy HBM/L2 -> LDS: lane i's BYTES bytes at base + off_i land at LDS address
// lds_addr + BYTES*i (base and lds_addr wavefront-uniform, off_i a 32-bit byte offset)
template <int BYTES>
// (m0 is written inside the statement and not listed as clobbered: the compiler keeps no value in m0 across
// statements on this target, it reloads m0 before each use of its own, and rejects the name in a clobber list as a
// reserved register)
__device__ __forceinline__ void async_copy(const unsigned char* base, uint32_t off, uint32_t lds_addr) {
  const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_addr);
  if constexpr (BYTES == 16)
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(m0v) : "memory");
  else
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(off), "s"(base), "s"(m0v) : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt_n() {
  __builtin_amdgcn_s_waitcnt((N & 0xF) | (0x7 << 4) | (0xF << 8) | ((N >> 4) << 14));
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

__device__ __forceinline__ float load_bias_v(const void* bias, int dt, int col) {
  if (dt == MASE_DT_F32) return ((const float*)bias)[col];
  if (dt == MASE_DT_BF16) return bits2f((uint32_t)((const uint16_t*)bias)[col] << 16);
  return f16_bits_to_f32(((const uint16_t*)bias)[col]);
}

// LDS offset of 16-byte chunk `chunk` of row `row` for rows of RB bytes (64 or 128); conflict-free for
// ds_read_b128 on a 64-bank LDS that serves 16 lanes at a time (see gemm_bf16.hip)
template <int RB>
__device__ __forceinline__ int lds_off(int row, int chunk) {
  if constexpr (RB == 128) return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4);
  else return row * 64 + ((chunk ^ ((row >> 2) & 3)) << 4);
}

template <int B_BITS>
struct MxGemmGeom {
  static constexpr int RA = BK;               // bytes per A row per K tile (8-bit codes)
  static constexpr int RB = BK * B_BITS / 8;  // bytes per B row per K tile
  static constexpr int kTileA = BM * RA, kTileB = BN * RB;
  static constexpr int kStage = kTileA + kTileB + 2 * 1024;  // + one scale dword per row for A and for B
  static constexpr int S = (kStage <= 53 * 1024) ? 3 : 2;
  // epilogue staging, separate from the stages (copies of the next tile are in flight during the epilogue):
  // per wavefront 16 rows of 128 bytes, row stride 144 bytes (16-byte accesses of 16 consecutive rows at one column
  // offset then fall on 64 different banks); three stages of the 4-bit form leave room for no more
  static constexpr int kStgRow = 144;
  static constexpr int kStgWave = 16 * kStgRow;        // bytes per wavefront
  static constexpr int kLdsBytes = S * kStage + 4 * kStgWave;
};

// Persistent kernel: one work-group per CU walks a list of output tiles.  The K tiles of all its output tiles
// form one stream through the LDS stages, so the copies of the next output tile's first K tiles are already
// in flight while the epilogue of the current one runs, and its stores drain behind the next main loop.
// STREAM: K holds at least S tiles, so the copy stream is never more than one output tile ahead and advances
// without branches; the other instantiation (short K) advances it with the general, branching step.
// TILED: both code matrices come as the images of mase_mxfp_tile_codes / mase_mxfp_pack_tiled, in which the 32 KB (A) or
// 16 KB (4-bit B) that one K tile of one 256-row tile occupies in an LDS stage lie contiguous and already swizzled, so a
// wavefront's copy reads one 1 KB run instead of 8 or 16 row segments a whole row apart (K bytes: a stride that keeps
// hitting the same L2 channels).  The LDS contents, and with them the result, are those of the row-major form.
template <int B_BITS, int CBSZ, int BLGP, int OUT_DT, bool STREAM, bool TILED = false>
__global__ __launch_bounds__(kThreadsG) void gemm_mxfp_kernel(MxGemmParams p) {
  using G = MxGemmGeom<B_BITS>;
  constexpr int RA = G::RA, RB = G::RB, kTileA = G::kTileA, kTileB = G::kTileB, kStage = G::kStage, S = G::S;
  constexpr int kCopiesA = kTileA / 1024 / 4;          // 16-byte copies per wavefront per tile
  constexpr int kCopiesB = kTileB / 1024 / 4;
  constexpr int kCopies = kCopiesA + kCopiesB + 2;     // + one 4-byte copy each for the A and B scales
  constexpr int kChunksB = RB / 64;                    // 16-byte chunks of B per lane per K step: 2 (8-bit) or 1 (4-bit)
  constexpr int kReads = 8 + 4 * kChunksB;             // ds_read_b128 per K step

  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane_id = tid & 63;
  const int lane = lane_id;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int nk = p.K / BK;

  // ---- this work-group's output tiles.  Work-groups are dealt to the 8 XCDs round-robin; when the counts
  // divide, XCD x owns the contiguous tile range [x*total/8, (x+1)*total/8) and its work-groups walk it
  // together (at any time they hold neighbouring tiles, which share operand rows in that XCD's L2).
  const int total = p.tiles_m * p.tiles_n;
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
  constexpr int GROUP_M = 4;
  const int in_group = GROUP_M * p.tiles_n;
  auto tile_origin = [&](int ord, int& m0, int& n0) {  // ord-th tile of this work-group
    const int t = t_first + min(ord, n_my - 1) * t_step;
    const int first_m = (t / in_group) * GROUP_M;
    const int gsz = min(p.tiles_m - first_m, GROUP_M);
    m0 = (first_m + (t % in_group) % gsz) * BM;
    n0 = ((t % in_group) / gsz) * BN;
  };

  // ---- global side of the async copies (the copy stream runs S K-tiles ahead of the MFMAs)
  const size_t lda = (size_t)p.K;                 // bytes per A row
  const size_t ldbb = (size_t)p.K * B_BITS / 8;   // bytes per B row
  const size_t lds_sc = (size_t)p.K / 32;         // scale bytes per row
  uint32_t ga[kCopiesA], gb[kCopiesB], gsa, gsb;  // byte offsets of this lane's pieces from the operand bases
  auto set_copy_tile = [&](int ord) __attribute__((always_inline)) {
    int m0, n0;
    tile_origin(ord, m0, n0);
    int lane = lane_id;
    asm volatile("" : "+v"(lane));  // keeps the lane-derived terms below out of the K loop's live registers
#pragma unroll
    for (int j = 0; j < kCopiesA; ++j) {  // 8 rows of 128 B per copy
      const int r = (wave + 4 * j) * 8 + (lane >> 3);
      if constexpr (TILED) ga[j] = (uint32_t)(m0 / BM) * (uint32_t)(nk * kTileA) + (wave + 4 * j) * 1024 + lane * 16;
      else ga[j] = (uint32_t)((size_t)min(m0 + r, p.M - 1) * lda) + (((lane & 7) ^ ((r >> 1) & 7)) << 4);
    }
#pragma unroll
    for (int j = 0; j < kCopiesB; ++j) {
      if constexpr (TILED) {
        gb[j] = (uint32_t)(n0 / BN) * (uint32_t)(nk * kTileB) + (wave + 4 * j) * 1024 + lane * 16;
      } else if constexpr (RB == 128) {
        const int r = (wave + 4 * j) * 8 + (lane >> 3);
        gb[j] = (uint32_t)((size_t)min(n0 + r, p.N - 1) * ldbb) + (((lane & 7) ^ ((r >> 1) & 7)) << 4);
      } else {  // 16 rows of 64 B per copy
        const int r = (wave + 4 * j) * 16 + (lane >> 2);
        gb[j] = (uint32_t)((size_t)min(n0 + r, p.N - 1) * ldbb) + (((lane & 3) ^ ((r >> 2) & 3)) << 4);
      }
    }
    // scales: wave w copies the dwords of rows [64w, 64w+64) of each operand
    gsa = (uint32_t)((size_t)min(m0 + wave * 64 + lane, p.M - 1) * lds_sc);
    gsb = (uint32_t)((size_t)min(n0 + wave * 64 + lane, p.N - 1) * lds_sc);
  };

  // The copies are issued from inline assembly rather than through the compiler's builtin: the compiler
  // orders every LDS read after all async copies it knows to be in flight (s_waitcnt vmcnt(0) before each
  // ds_read), which would serialize the pipeline; completion is tracked by hand with wait_vmcnt_n below.
  // M0 carries the wavefront-uniform LDS base; nothing else in this kernel uses M0.
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lptr_t)lds;
  // copy-stream position: K tile c_kt of this work-group's c_ord-th output tile goes to stage c_stage.  Past the
  // last tile the stream keeps re-copying the final K tile into stages nobody reads any more, which keeps
  // the main loop free of branches around the copies and the vmcnt bookkeeping uniform.
  int c_kt = 0, c_ord = 0, c_stage = 0;
  auto issue_copy = [&](int c) __attribute__((always_inline)) {
    const uint32_t st = lds_base + (uint32_t)(c_stage * kStage);
    if (c < kCopiesA) {
      async_copy<16>(p.A + (size_t)c_kt * (TILED ? kTileA : RA), ga[c], st + (wave + 4 * c) * 1024);
    } else if (c < kCopiesA + kCopiesB) {
      const int j = c - kCopiesA;
      async_copy<16>(p.B + (size_t)c_kt * (TILED ? kTileB : RB), gb[j], st + kTileA + (wave + 4 * j) * 1024);
    } else if (c == kCopiesA + kCopiesB) {
      async_copy<4>(p.SA + (size_t)c_kt * 4, gsa, st + kTileA + kTileB + wave * 256);
    } else {
      async_copy<4>(p.SB + (size_t)c_kt * 4, gsb, st + kTileA + kTileB + 1024 + wave * 256);
    }
  };
  auto advance_copy_stream = [&]() __attribute__((always_inline)) {
    c_stage = (c_stage + 1 == S) ? 0 : c_stage + 1;
    if (c_ord >= n_my) return;          // past the end: stay on the final K tile
    if (++c_kt == nk) {
      if (++c_ord < n_my) {
        c_kt = 0;
        set_copy_tile(c_ord);
      } else {
        c_kt = nk - 1;
      }
    }
  };

  f32x16_t acc[4][4];
  auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  };
  zero_acc();

  set_copy_tile(0);
#pragma unroll
  for (int t = 0; t < S; ++t) {
#pragma unroll
    for (int c = 0; c < kCopies; ++c) issue_copy(c);
    advance_copy_stream();
  }

  const int frag_row = lane & 31;
  const int kgrp = lane >> 5;
  // Fragment registers of one K step: A row tile i -> fa[i] (8 dwords), B column tile j -> fb[j] (8 dwords, the
  // upper 4 unused for 4-bit codes).  Read number q of a step: q < 8 -> 16-byte half (q&1) of A tile q>>1;
  // then the B chunks.
  uint4 fa[2][4][2], fb[2][4][2];
  auto load_part = [&](int stage, int s, int set, int q) __attribute__((always_inline)) {
    const unsigned char* st = lds + stage * kStage;
    if (q < 8) {
      const int i = q >> 1, h = q & 1;
      fa[set][i][h] = *(const uint4*)(st + (wm * 128) * RA + lds_off<RA>(i * 32 + frag_row, s * 4 + h * 2 + kgrp));
    } else {
      const int qq = q - 8;
      const int j = qq / kChunksB, h = qq % kChunksB;
      fb[set][j][h] = *(const uint4*)(st + kTileA + (wn * 128) * RB +
                                      lds_off<RB>(j * 32 + frag_row, kChunksB == 2 ? s * 4 + h * 2 + kgrp : s * 2 + kgrp));
    }
  };
  // scale dwords of the current K tile (sa/sb) and of the next one (san/sbn), pre-shifted so that K step s
  // uses byte 2s
  int sa[4], sb[4], san[4], sbn[4];
  auto load_scales = [&](int stage, int* a, int* b) {
    const unsigned char* st = lds + stage * kStage + kTileA + kTileB;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a[i] = (int)(*(const uint32_t*)(st + (wm * 128 + i * 32 + frag_row) * 4) >> (8 * kgrp));
      b[i] = (int)(*(const uint32_t*)(st + 1024 + (wn * 128 + i * 32 + frag_row) * 4) >> (8 * kgrp));
    }
  };
  auto mfma = [&](int set, int s, int t) __attribute__((always_inline)) {
    const int i = t >> 2, j = t & 3;
    i32x8_t a, b;
    a[0] = (int)fa[set][i][0].x; a[1] = (int)fa[set][i][0].y; a[2] = (int)fa[set][i][0].z; a[3] = (int)fa[set][i][0].w;
    a[4] = (int)fa[set][i][1].x; a[5] = (int)fa[set][i][1].y; a[6] = (int)fa[set][i][1].z; a[7] = (int)fa[set][i][1].w;
    b[0] = (int)fb[set][j][0].x; b[1] = (int)fb[set][j][0].y; b[2] = (int)fb[set][j][0].z; b[3] = (int)fb[set][j][0].w;
    if constexpr (kChunksB == 2) {
      b[4] = (int)fb[set][j][1].x; b[5] = (int)fb[set][j][1].y; b[6] = (int)fb[set][j][1].z; b[7] = (int)fb[set][j][1].w;
    } else {
      b[4] = 0; b[5] = 0; b[6] = 0; b[7] = 0;
    }
    // B's fragment goes in as the first operand (formats and scales swapped with it): the accumulators then hold the
    // tile transposed, which is the layout the epilogue wants
    if (s == 0)
      acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, a, acc[i][j], BLGP, CBSZ, 0, sb[j], 0, sa[i]);
    else
      acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, a, acc[i][j], BLGP, CBSZ, 2, sb[j], 2, sa[i]);
  };

  // ---- epilogue of one output tile (the scheme of gemm_bf16.hip).  acc[i][j][q*4 + rr] is C[row, col] with
  // row = i*32 + lane%32 and col = j*32 + q*8 + (lane/32)*4 + rr: a lane holds runs of four consecutive columns of one
  // row.  The runs pass through the wavefront's own staging rows, 16 rows of 128 bytes at a time (the lanes of rows
  // 0-15 of the MFMA tile, then those of rows 16-31), from which every lane takes 16 consecutive bytes.  Only lanes of
  // one wavefront exchange data (its LDS accesses execute in order, and the writes are waited for before the reads are
  // issued): no barrier.
  //   without bias: the values are converted to the output type before staging, so a row of the staging area is 64
  //     columns of a 16-bit output and a store instruction writes 8 rows of 128 contiguous bytes.  (No "+ 0" stands in
  //     for the bias: an accumulator that started at +0 never holds -0, so there is nothing for it to normalise.)
  //   with bias: staged as fp32, 32 columns per row; bias added and the value converted after the read-back, where a
  //     lane's columns are the same for every band (16 bias registers instead of 64).
  auto epilogue = [&](int ord) __attribute__((always_inline)) {
    int m0, n0;
    tile_origin(ord, m0, n0);
    acc_read_fence();
    int lane = lane_id;
    asm volatile("" : "+v"(lane));  // keeps the lane-derived terms below out of the K loop's live registers
    const int r32 = lane & 31, kgrp = lane >> 5;
    const int rrow = lane >> 3, chunk = lane & 7;  // read side: row rrow + 8 * pass, 16-byte piece `chunk` of it
    unsigned char* const stg = lds + S * kStage + wave * G::kStgWave;
    unsigned char* const stg_w = stg + (r32 & 15) * G::kStgRow;
    const unsigned char* const stg_r = stg + rrow * G::kStgRow + chunk * 16;
    constexpr int kEsz = (OUT_DT == MASE_DT_F32) ? 4 : 2;
    const size_t row_step = (size_t)p.N * kEsz;  // bytes from one output row to the next
    unsigned char* const wave_c = (unsigned char*)p.C + ((size_t)(m0 + wm * 128) * p.N + (size_t)(n0 + wn * 128)) * kEsz;
    // `n` consecutive elements (16 or 8 bytes in x0..x3) to row `row`, columns col0.. of C, in one store where that is
    // possible, else element by element, the bytes shifted down as they go (a rolled loop: rare, and kept small so that
    // the code between two K loops stays short)
    auto store_piece = [&](auto nc, int row, int col0, uint32_t x0, uint32_t x1, uint32_t x2, uint32_t x3)
                           __attribute__((always_inline)) {
      constexpr int n = decltype(nc)::value;
      if (row >= p.M) return;
      unsigned char* const dst = (unsigned char*)p.C + ((size_t)row * p.N + (size_t)col0) * kEsz;
      if ((p.N & (n - 1)) == 0 && ((((uintptr_t)p.C) & 15u) == 0) && col0 + n - 1 < p.N) {
        if constexpr (n * kEsz == 16) store_nt((uint4*)dst, make_uint4(x0, x1, x2, x3));
        else store_nt((uint2*)dst, make_uint2(x0, x1));
      } else {
#pragma unroll 1
        for (int e = 0; e < n && col0 + e < p.N; ++e) {
          if constexpr (OUT_DT == MASE_DT_F32) {
            ((uint32_t*)dst)[e] = x0;
            x0 = x1, x1 = x2, x2 = x3;
          } else {
            ((uint16_t*)dst)[e] = (uint16_t)x0;
            x0 = (x0 >> 16) | (x1 << 16), x1 = (x1 >> 16) | (x2 << 16), x2 = (x2 >> 16) | (x3 << 16), x3 >>= 16;
          }
        }
      }
    };
    if (p.bias == nullptr) {
      constexpr int kVec = 16 / kEsz;  // elements per 16-byte piece
      // the wavefront's whole part of the tile lies inside C and takes 16-byte stores (wavefront-uniform)
      const bool interior = ((p.N & (kVec - 1)) == 0) && ((((uintptr_t)p.C) & 15u) == 0) &&
                            m0 + wm * 128 + 128 <= p.M && n0 + wn * 128 + 128 <= p.N;
      unsigned char* const lane_c = wave_c + (size_t)rrow * row_step + chunk * 16;
      // one band: kBandTiles MFMA tiles of row tile i side by side = 128 bytes of output per row, 16 rows at a time
      constexpr int kBandTiles = (OUT_DT == MASE_DT_F32) ? 1 : 2;
      constexpr int kBandsPerRowTile = 4 / kBandTiles;
#pragma unroll
      for (int b = 0; b < 4 * kBandsPerRowTile * 2; ++b) {
        const int i = b / (kBandsPerRowTile * 2), jb = (b >> 1) % kBandsPerRowTile, half = b & 1;
        if ((r32 >> 4) == half) {
#pragma unroll
          for (int jj = 0; jj < kBandTiles; ++jj) {
            const int j = jb * kBandTiles + jj;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float v[4] = {acc_read(acc[i][j][q * 4 + 0]), acc_read(acc[i][j][q * 4 + 1]),
                                  acc_read(acc[i][j][q * 4 + 2]), acc_read(acc[i][j][q * 4 + 3])};
              unsigned char* const dst = stg_w + (jj * 32 + q * 8 + kgrp * 4) * kEsz;
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
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the band is in LDS before any lane reads it
        uint4 w[2];
#pragma unroll
        for (int ps = 0; ps < 2; ++ps) w[ps] = *(const uint4*)(stg_r + ps * 8 * G::kStgRow);
        // streaming stores: the output is not read again by this kernel and should not displace operand panels
        if (__builtin_expect(interior, 1)) {
          unsigned char* const dst0 = lane_c + (size_t)(i * 32 + half * 16) * row_step + jb * 128;
#pragma unroll
          for (int ps = 0; ps < 2; ++ps) store_nt((uint4*)(dst0 + (size_t)(ps * 8) * row_step), w[ps]);
        } else {
#pragma unroll
          for (int ps = 0; ps < 2; ++ps)
            store_piece(std::integral_constant<int, kVec>{}, m0 + wm * 128 + i * 32 + half * 16 + ps * 8 + rrow,
                        n0 + wn * 128 + jb * kBandTiles * 32 + chunk * kVec, w[ps].x, w[ps].y, w[ps].z, w[ps].w);
        }
        asm volatile("" ::: "memory");      // lanes exchange data through LDS: no value may be carried across
        __builtin_amdgcn_sched_barrier(0);  // bands stay in program order: bounded register use
      }
    } else {
      float bv[4][4];  // bias of the four columns this lane reads back, per column tile
      auto fill = [&](auto dtc) __attribute__((always_inline)) {  // the dtype is decided once, not per element
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int col = n0 + wn * 128 + j * 32 + chunk * 4 + e;
            bv[j][e] = col < p.N ? load_bias_v(p.bias, decltype(dtc)::value, col) : 0.0f;
          }
      };
      if (p.bias_dtype == MASE_DT_F32) fill(std::integral_constant<int, MASE_DT_F32>{});
      else if (p.bias_dtype == MASE_DT_BF16) fill(std::integral_constant<int, MASE_DT_BF16>{});
      else fill(std::integral_constant<int, MASE_DT_F16>{});
      // The bias loads are the only vector-memory loads the compiler itself tracks in this kernel.  Completing
      // them here, with a wait it can see, keeps it from guarding their registers with s_waitcnt vmcnt(0)
      // inside the K loop, where that would also wait for every async copy in flight.
      wait_vmcnt_n<0>();
#pragma unroll
      for (int b = 0; b < 32; ++b) {  // band: MFMA tile (i, j), 16 rows at a time
        const int i = b >> 3, j = (b >> 1) & 3, half = b & 1;
        if ((r32 >> 4) == half) {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            *(uint4*)(stg_w + (q * 8 + kgrp * 4) * 4) =
                make_uint4(f2bits(acc_read(acc[i][j][q * 4 + 0])), f2bits(acc_read(acc[i][j][q * 4 + 1])),
                           f2bits(acc_read(acc[i][j][q * 4 + 2])), f2bits(acc_read(acc[i][j][q * 4 + 3])));
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the band is in LDS before any lane reads it
        uint4 w[2];
#pragma unroll
        for (int ps = 0; ps < 2; ++ps) w[ps] = *(const uint4*)(stg_r + ps * 8 * G::kStgRow);
#pragma unroll
        for (int ps = 0; ps < 2; ++ps) {
          const float v[4] = {bits2f(w[ps].x) + bv[j][0], bits2f(w[ps].y) + bv[j][1], bits2f(w[ps].z) + bv[j][2],
                              bits2f(w[ps].w) + bv[j][3]};
          const int row = m0 + wm * 128 + i * 32 + half * 16 + ps * 8 + rrow;
          const int col0 = n0 + wn * 128 + j * 32 + chunk * 4;
          if constexpr (OUT_DT == MASE_DT_F32) {
            store_piece(std::integral_constant<int, 4>{}, row, col0, f2bits(v[0]), f2bits(v[1]), f2bits(v[2]), f2bits(v[3]));
          } else if constexpr (OUT_DT == MASE_DT_BF16) {
            store_piece(std::integral_constant<int, 4>{}, row, col0, f32x2_to_bf16x2_bits(v[0], v[1]),
                        f32x2_to_bf16x2_bits(v[2], v[3]), 0u, 0u);
          } else {
            store_piece(std::integral_constant<int, 4>{}, row, col0, f32_to_f16_bits(v[0]) | (f32_to_f16_bits(v[1]) << 16),
                        f32_to_f16_bits(v[2]) | (f32_to_f16_bits(v[3]) << 16), 0u, 0u);
          }
        }
        asm volatile("" ::: "memory");      // lanes exchange data through LDS: no value may be carried across
        __builtin_amdgcn_sched_barrier(0);  // bands stay in program order: bounded register use
      }
    }
  };

  // Pipeline (see gemm_bf16.hip for the reasoning): per K tile two steps of 16 MFMAs; fragment sets ping-pong.
  //   step 0: MFMAs on set 0, interleaved with the LDS reads of step 1 (set 1)
  //   hand-over: own LDS reads done (lgkmcnt), own copies of the next K tile landed (vmcnt), barrier
  //   step 1: MFMAs on set 1, interleaved with the LDS reads of step 0 and the scales of the next K tile and
  //           with the copies of the K tile S positions ahead into the stage just vacated
  // After the last K tile of an output tile: epilogue, accumulators cleared; the stream carries on.
  // The epilogue's stores count in vmcnt like the copies.  Loads retire in order among themselves, so
  // "at most (S-2)*kCopies outstanding" still proves the next K tile has landed (if one of its loads were
  // pending, all kCopies loads of the K tile after it would be too); it may additionally wait for stores.
  constexpr int kCopiesPerSlot = (kCopies + 15) / 16;
  wait_vmcnt_n<(S - 1) * kCopies>();  // K tile 0 landed; the other stages may still be filling
  asm volatile("s_barrier" ::: "memory");
#pragma unroll
  for (int q = 0; q < kReads; ++q) load_part(0, 0, 0, q);
  load_scales(0, sa, sb);
  int stage = 0;
  // One K tile.  The body must stay a single basic block: with a branch inside, the compiler sinks the MFMAs
  // (whose results are only consumed by the next iteration) below it and the interleave is lost.  Hence the
  // copy stream is advanced by a caller-supplied, branch-free step.
  auto k_iteration = [&](auto&& advance) __attribute__((always_inline)) {
    const int next_stage = (stage + 1 == S) ? 0 : stage + 1;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      mfma(0, 0, t);
      if (t < kReads) load_part(stage, 1, 1, t);
      __builtin_amdgcn_sched_barrier(0);
    }
    wait_vmcnt_n<(S - 2) * kCopies>();  // the next K tile must have landed; later ones may be in flight
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      mfma(1, 1, t);
      if (t < kReads) load_part(next_stage, 0, 0, t);
      if (t == 12) load_scales(next_stage, san, sbn);
#pragma unroll
      for (int c = t * kCopiesPerSlot; c < (t + 1) * kCopiesPerSlot; ++c)
        if (c < kCopies) issue_copy(c);  // into the stage this K tile just vacated (c_stage == stage)
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) { sa[i] = san[i]; sb[i] = sbn[i]; }
    advance();
    stage = next_stage;
  };
  auto step_within_tile = [&]() {
    c_stage = (c_stage + 1 == S) ? 0 : c_stage + 1;
    ++c_kt;
  };
  for (int ord = 0; ord < n_my; ++ord) {
    if constexpr (STREAM) {
      // the copy stream stands at K tile S of this output tile (or, if nk == S, at K tile 0 of the next)
#pragma unroll 1
      for (int kt = 0; kt < nk - S; ++kt) k_iteration(step_within_tile);
      // it moves on to the next output tile (past the last one: harmless re-copies of its first K tiles)
      set_copy_tile(ord + 1);
      c_kt = 0;
#pragma unroll 1
      for (int kt = 0; kt < S; ++kt) k_iteration(step_within_tile);
    } else {
      for (int kt = 0; kt < nk; ++kt) k_iteration(advance_copy_stream);
    }
    epilogue(ord);
    zero_acc();
  }
  wait_vmcnt_n<0>();  // no copy may still be in flight towards LDS when the work-group retires
}

// number of work-groups of the persistent kernel: one per CU (each takes the whole LDS of its CU)
int persistent_grid(int total_tiles) {
  const int n_cu = device_cu_count();
  if (n_cu <= 0) return -1;
  return total_tiles < n_cu ? total_tiles : n_cu;
}

template <int B_BITS, int CBSZ, int BLGP, bool TILED = false>
int launch_mx_gemm(const MxGemmParams& p, int out_dtype, hipStream_t st) {
  const size_t lds_bytes = (size_t)MxGemmGeom<B_BITS>::kLdsBytes;
  const int nwg = persistent_grid(p.tiles_m * p.tiles_n);
  if (nwg <= 0) return MASE_ERR_LAUNCH;
  const dim3 grid((unsigned)nwg), block(kThreadsG);
  const bool stream = p.K / BK >= MxGemmGeom<B_BITS>::S;
#define MASE_MX_LAUNCH(DT_, STREAM_)                                                                              \
  do {                                                                                                            \
    static std::atomic<uint64_t> attr_done{0};                                                                    \
    const void* k = (const void*)gemm_mxfp_kernel<B_BITS, CBSZ, BLGP, DT_, STREAM_, TILED>;                       \
    if (!set_dynamic_lds_once(attr_done, k, (int)lds_bytes)) return MASE_ERR_LAUNCH;                              \
    hipLaunchKernelGGL((gemm_mxfp_kernel<B_BITS, CBSZ, BLGP, DT_, STREAM_, TILED>), grid, block, lds_bytes, st,   \
                       p);                                                                                        \
  } while (0)
  if (stream) {
    if (out_dtype == MASE_DT_F32) MASE_MX_LAUNCH(MASE_DT_F32, true);
    else if (out_dtype == MASE_DT_BF16) MASE_MX_LAUNCH(MASE_DT_BF16, true);
    else MASE_MX_LAUNCH(MASE_DT_F16, true);
  } else {
    if (out_dtype == MASE_DT_F32) MASE_MX_LAUNCH(MASE_DT_F32, false);
    else if (out_dtype == MASE_DT_BF16) MASE_MX_LAUNCH(MASE_DT_BF16, false);
    else MASE_MX_LAUNCH(MASE_DT_F16, false);
  }
#undef MASE_MX_LAUNCH
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

// One thread per 16-byte granule of the image: tile (row tile, K tile), row r of the tile, chunk position cl; the
// source chunk is cl ^ swizzle(r), the source row clamped to the last one as the row-major kernel clamps it.
template <int BITS>
__global__ __launch_bounds__(256) void mxfp_tile_codes_kernel(const unsigned char* __restrict__ codes,
                                                              uint4* __restrict__ tiled, int rows, int K,
                                                              size_t granules) {
  constexpr int kRowBytes = BK * BITS / 8;  // 128 or 64
  constexpr int kChunks = kRowBytes / 16;   // 8 or 4
  const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= granules) return;
  const int nk = K / BK;
  const size_t tile = g / (size_t)(BM * kChunks);
  const int within = (int)(g % (size_t)(BM * kChunks));
  const int r = within / kChunks, cl = within % kChunks;
  const int tm = (int)(tile / (size_t)nk), kt = (int)(tile % (size_t)nk);
  const int sw = (BITS == 8) ? ((r >> 1) & 7) : ((r >> 2) & 3);
  const size_t row = (size_t)min(tm * BM + r, rows - 1);
  const unsigned char* src = codes + row * ((size_t)K * BITS / 8) + (size_t)kt * kRowBytes + ((cl ^ sw) << 4);
  tiled[g] = *(const uint4*)src;
}

}  // namespace
}  // namespace mase

extern "C" size_t mase_mxfp_tiled_bytes(size_t rows, size_t K, int bits) {
  if (rows == 0 || K == 0 || (K % mase::BK) != 0 || (bits != 4 && bits != 8)) return 0;
  return ((rows + mase::BM - 1) / mase::BM) * mase::BM * (K * (size_t)bits / 8);
}

extern "C" int mase_mxfp_tile_codes(const void* codes, void* tiled, size_t rows, size_t K, int bits, void* stream) {
  using namespace mase;
  static_assert(BM == BN, "one image geometry for both operands");
  if (rows == 0 || K == 0) return MASE_OK;
  if (codes == nullptr || tiled == nullptr) return MASE_ERR_NULL;
  if (bits != 4 && bits != 8) return MASE_ERR_PARAM;
  if ((K % BK) != 0 || rows > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  if (!aligned16(codes) || !aligned16(tiled)) return MASE_ERR_ALIGN;
  const size_t granules = mase_mxfp_tiled_bytes(rows, K, bits) / 16;
  const dim3 grid(blocks_for(granules, (size_t)256)), block(256);
  if (bits == 8)
    hipLaunchKernelGGL(mxfp_tile_codes_kernel<8>, grid, block, 0, (hipStream_t)stream, (const unsigned char*)codes,
                       (uint4*)tiled, (int)rows, (int)K, granules);
  else
    hipLaunchKernelGGL(mxfp_tile_codes_kernel<4>, grid, block, 0, (hipStream_t)stream, (const unsigned char*)codes,
                       (uint4*)tiled, (int)rows, (int)K, granules);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

extern "C" int mase_gemm_mxfp4_scaled_tiled(const void* A_tiled, const void* A_scales, int a_format, const void* B_tiled,
                                            const void* B_scales, const void* bias, void* C, size_t M, size_t N,
                                            size_t K, int out_dtype, int bias_dtype, void* stream) {
  using namespace mase;
  if (M == 0 || N == 0) return MASE_OK;
  if (A_tiled == nullptr || B_tiled == nullptr || A_scales == nullptr || B_scales == nullptr || C == nullptr)
    return MASE_ERR_NULL;
  if (K == 0 || (K % BK) != 0 || M > (1u << 30) || N > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  // the kernel addresses each image with a 32-bit byte offset from its base
  if ((unsigned long long)mase_mxfp_tiled_bytes(M, K, 8) > 0xFFFFFFFFull ||
      (unsigned long long)mase_mxfp_tiled_bytes(N, K, 4) > 0xFFFFFFFFull)
    return MASE_ERR_SHAPE;
  if (!aligned16(A_tiled) || !aligned16(B_tiled) || (((uintptr_t)A_scales) & 3u) != 0 || (((uintptr_t)B_scales) & 3u) != 0)
    return MASE_ERR_ALIGN;
  if (out_dtype < 0 || out_dtype > 2 || (bias != nullptr && (bias_dtype < 0 || bias_dtype > 2))) return MASE_ERR_DTYPE;
  if (a_format != 0 && a_format != 1) return MASE_ERR_PARAM;
  MxGemmParams p;
  p.A = (const unsigned char*)A_tiled;
  p.B = (const unsigned char*)B_tiled;
  p.SA = (const unsigned char*)A_scales;
  p.SB = (const unsigned char*)B_scales;
  p.bias = bias;
  p.C = C;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.bias_dtype = bias_dtype;
  p.tiles_m = (int)((M + BM - 1) / BM);
  p.tiles_n = (int)((N + BN - 1) / BN);
  hipStream_t st = (hipStream_t)stream;
  return a_format == 0 ? launch_mx_gemm<4, 0, 4, true>(p, out_dtype, st) : launch_mx_gemm<4, 1, 4, true>(p, out_dtype, st);
}

// a_format / b_format: 0 = e4m3 (8-bit), 1 = e5m2 (8-bit), 4 = e2m1 (4-bit, two codes per byte); A must be 8-bit.
extern "C" int mase_gemm_mxfp_scaled(const void* A, const void* A_scales, int a_format, const void* B,
                                     const void* B_scales, int b_format, const void* bias, void* C, size_t M, size_t N,
                                     size_t K, int out_dtype, int bias_dtype, void* stream) {
  using namespace mase;
  if (M == 0 || N == 0) return MASE_OK;
  if (A == nullptr || B == nullptr || A_scales == nullptr || B_scales == nullptr || C == nullptr) return MASE_ERR_NULL;
  if (K == 0 || (K % BK) != 0 || M > (1u << 30) || N > (1u << 30) || K > (1u << 30)) return MASE_ERR_SHAPE;
  // the kernel addresses each operand with a 32-bit byte offset from its base
  if ((unsigned long long)M * K > 0xFFFFFFFFull || (unsigned long long)N * K > 0xFFFFFFFFull) return MASE_ERR_SHAPE;
  if (!aligned16(A) || !aligned16(B) || (((uintptr_t)A_scales) & 3u) != 0 || (((uintptr_t)B_scales) & 3u) != 0)
    return MASE_ERR_ALIGN;
  if (out_dtype < 0 || out_dtype > 2 || (bias != nullptr && (bias_dtype < 0 || bias_dtype > 2))) return MASE_ERR_DTYPE;
  if ((a_format != 0 && a_format != 1) || (b_format != 0 && b_format != 1 && b_format != 4)) return MASE_ERR_PARAM;
  MxGemmParams p;
  p.A = (const unsigned char*)A;
  p.B = (const unsigned char*)B;
  p.SA = (const unsigned char*)A_scales;
  p.SB = (const unsigned char*)B_scales;
  p.bias = bias;
  p.C = C;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.bias_dtype = bias_dtype;
  p.tiles_m = (int)((M + BM - 1) / BM);
  p.tiles_n = (int)((N + BN - 1) / BN);
  hipStream_t st = (hipStream_t)stream;
  if (a_format == 0 && b_format == 4) return launch_mx_gemm<4, 0, 4>(p, out_dtype, st);
  if (a_format == 1 && b_format == 4) return launch_mx_gemm<4, 1, 4>(p, out_dtype, st);
  if (a_format == 0 && b_format == 0) return launch_mx_gemm<8, 0, 0>(p, out_dtype, st);
  if (a_format == 0 && b_format == 1) return launch_mx_gemm<8, 0, 1>(p, out_dtype, st);
  if (a_format == 1 && b_format == 0) return launch_mx_gemm<8, 1, 0>(p, out_dtype, st);
  return launch_mx_gemm<8, 1, 1>(p, out_dtype, st);
}
