// Causal self-attention core of the decoder layer for gfx950: out = softmax(q k^T * scaling + causal mask) v, bf16
// operands, head dimension 128, fp32 softmax statistics and accumulators, in one pass over the keys (no [T, T] score
// matrix in memory).  Semantics of the reference's Llama attention core on unquantized q / k / v
// (models/llama/modeling_llama.py:362-480: scores in the model dtype, fp32 softmax, probabilities cast back to the
// model dtype before the product with v); here the probabilities are rounded to bf16 before that product too, and the
// row sum divides once at the end, so results agree with the tensor operations to bf16 rounding, not bit for bit.
//
// One work-group (4 wavefronts) owns 128 queries of one (batch, head); a wavefront owns 32 of them.  Key blocks of 64
// are streamed through LDS (K and V as [key][128 d] rows, both double-buffered with async copies).
// Per key block a wavefront computes S^T = K Q^T with v_mfma_f32_32x32x16_bf16 (A = K rows from LDS, B = its Q
// fragments, kept in registers for the whole kernel): a lane then holds, for ONE query (lane % 32), the scores of 32 of
// the 64 keys in its accumulator registers, so the softmax statistics are in-lane but for one exchange with lane ^ 32.
// exp2 of the scaled scores gives P^T, which is already laid out as the B operand of O^T += V^T P^T (the matrix
// instruction's 8 contraction slots of lane group g at step s are accumulator registers 8 (s % 2) .. + 7 of score tile
// s / 2, i.e. keys 16 s + 4 g + 8 (j / 4) + j % 4).  Two work-groups fit a CU (64 KB of LDS, under 256 registers),
// so one wavefront's exponentials overlap the other's matrix instructions.
//
// The V^T fragments of the second product (lane = d, 8 keys each) are made from V's rows by the transposing LDS read
// ds_read_b64_tr_b16, so V needs no transposed copy in memory.
#include "common.hpp"
#include "mxint_core.hpp"

namespace mase {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void* lptr_t;
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4_t lds_s16x4_t;

constexpr int kQB = 128, kKB = 64, kHD = 128;
constexpr int kKBytes = kKB * kHD * 2;       // 16 KB: 64 key rows of 256 bytes
constexpr int kVBytes = kKBytes;             // V like K: 64 key rows of 256 bytes
constexpr int kKRing = 5;                    // K fragment pairs in flight or in use: reads run 4 contraction steps ahead
constexpr float kGrow = 8.0f;                // see the softmax reference point in the kernel

// max of a lane's value and lane ^ 32's, without a trip through the LDS queue (which would wait for the fragment reads
// in flight)
__device__ __forceinline__ float max_with_other_half(float v) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const unsigned a = r[0], b = r[1];  // (a bit cast applied to r[1] directly reads element 0)
  return fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
}

__device__ __forceinline__ uint32_t umax_with_other_half(uint32_t v) {
  const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  const unsigned a = r[0], b = r[1];
  return max(a, b);
}

constexpr int kAttnLds = 2 * kKBytes + 2 * kVBytes;

// lane i's 16 bytes at base + off_i land at LDS address lds_addr + 16 * i; tracked by hand with at_wait_vmcnt
// (m0 is written inside the statement and not listed as clobbered: the compiler keeps no value in m0 across
// statements on this target, it reloads m0 before each use of its own, and rejects the name in a clobber list as a
// reserved register)
__device__ __forceinline__ void at_async_copy_16(const unsigned char* base, uint32_t off, uint32_t lds_addr) {
  const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(m0v) : "memory");
}
template <int N>
__device__ __forceinline__ void at_wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 0xF) | (0x7 << 4) | (0xF << 8) | ((N >> 4) << 14));
}

struct AttnParams {
  const unsigned char* q;
  const unsigned char* k;
  const unsigned char* v;
  unsigned char* out;
  int BH, H, T;
  int rounds, bh_lanes;  // persistent form: work items per work-group, (batch, head) pairs an XCD works on side by side
  size_t q_sb, q_sh, k_sb, k_sh, v_sb, v_sh, o_sb, o_sh;  // byte strides of batch and head
  uint32_t q_st, k_st, v_st, o_st;                        // byte strides of a token
  float c;                                    // scaling * log2(e)
  MxintParams mx;                             // MX instantiation only
  const unsigned char* q_cos;                 // ROPE instantiation only: tables [batch or 1][tokens][128] bf16
  const unsigned char* q_sin;
  size_t cs_sb;                               // byte strides of the tables: batch (0 for a shared table), token
  uint32_t cs_st;
};

// MX: the output is written as the MXINT quantize-dequantize of the bf16 result, blocks of 32 along the head dimension
// (what a LinearMXInt reading the [batch, tokens, heads * 128] result would compute in a pass of its own,
// nn/quantized/modules/linear.py:956-972): the 32 values of a block are the 16 accumulator registers of one d tile in
// lane l and in lane l ^ 32.
// ROPE: q is given before its rotary embedding, which is applied as the fragments are loaded: x cos + rotate_half(x) sin
// with the two products and the sum rounded to bf16 one by one, as mase_rope rounds them
// (nn/quantized/functional/rope.py:17-27); the partner element d +- 64 lies in the same lane's fragment s +- 4.
template <bool MX, bool ROPE>
__global__ __launch_bounds__(256, 2) void attn_causal_fwd_kernel(AttnParams p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int l32 = lane & 31, g = lane >> 5;
  // Work-groups are handed to the 8 XCDs in turn (blockIdx % 8), each XCD with an L2 of its own.  All query blocks of
  // one (batch, head) go to one XCD and run at the same time, walking the keys from the start together, so K and V come
  // from HBM once and from that L2 afterwards.
  // Persistent form (rounds > 0; the host picks it when the counts divide): two work-groups per CU for the whole
  // launch, each taking `rounds` items; an XCD's work-groups cover bh_lanes (batch, head) pairs x all query blocks per
  // round, and a work-group alternates between query block n - 1 - i and query block i, so that all of them have the
  // same number of key blocks to go through and finish together.  Otherwise one item per work-group, the query blocks
  // with the most keys first.
  const int n_qb = p.T / kQB;
  const int n_items = p.rounds > 0 ? p.rounds : 1;
  for (int item = 0; item < n_items; ++item) {
  int bh, qb;
  if (p.rounds > 0) {
    const int xcd = (int)blockIdx.x & 7, wl = (int)blockIdx.x >> 3;
    const int qidx = wl % n_qb;
    bh = (wl / n_qb + p.bh_lanes * item) * 8 + xcd;
    qb = (item & 1) ? qidx : n_qb - 1 - qidx;
  } else if (p.BH % 8 == 0) {
    const int xcd = (int)blockIdx.x & 7, slot = (int)blockIdx.x >> 3;
    bh = (slot / n_qb) * 8 + xcd;
    qb = n_qb - 1 - slot % n_qb;
  } else {
    bh = (int)blockIdx.x / n_qb;
    qb = n_qb - 1 - (int)blockIdx.x % n_qb;
  }
  const int b = bh / p.H, h = bh % p.H;
  const unsigned char* qp = p.q + (size_t)b * p.q_sb + (size_t)h * p.q_sh;
  const unsigned char* kp = p.k + (size_t)b * p.k_sb + (size_t)h * p.k_sh;
  const unsigned char* vp = p.v + (size_t)b * p.v_sb + (size_t)h * p.v_sh;
  // persistent form: the first key block of the work-group's next item is fetched during the last key block of this one
  const bool has_next = item + 1 < n_items;
  const unsigned char *kp_next = kp, *vp_next = vp;
  if (has_next) {
    const int bhn = bh + p.bh_lanes * 8, bn = bhn / p.H, hn = bhn % p.H;
    kp_next = p.k + (size_t)bn * p.k_sb + (size_t)hn * p.k_sh;
    vp_next = p.v + (size_t)bn * p.v_sb + (size_t)hn * p.v_sh;
  }
  const int q0 = qb * kQB + wave * 32;  // this wavefront's first query
  const int qi = q0 + l32;              // this lane's query

  bf16x8_t qf[8];
#pragma unroll
  for (int s = 0; s < 8; ++s) qf[s] = *(const bf16x8_t*)(qp + (size_t)qi * p.q_st + (s * 16 + g * 8) * 2);
  if constexpr (ROPE) {
    const unsigned char* cp = p.q_cos + (size_t)b * p.cs_sb + (size_t)qi * p.cs_st;
    const unsigned char* sp = p.q_sin + (size_t)b * p.cs_sb + (size_t)qi * p.cs_st;
    bf16x8_t rq[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const bf16x8_t cs = *(const bf16x8_t*)(cp + (s * 16 + g * 8) * 2), sn = *(const bf16x8_t*)(sp + (s * 16 + g * 8) * 2);
      const bf16x8_t other = qf[s ^ 4];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        using TR = DTypeTraits<MASE_DT_BF16>;
        const float x = (float)qf[s][e], xp = (float)other[e];
        const float rot = (s < 4) ? -xp : xp;
        rq[s][e] = __builtin_bit_cast(__bf16, (uint16_t)f32_to_bf16_bits(TR::round(x * (float)cs[e]) + TR::round(rot * (float)sn[e])));
      }
    }
#pragma unroll
    for (int s = 0; s < 8; ++s) qf[s] = rq[s];
  }

  // async copies of one key block: 4 of K and 4 of V (4 rows of 256 bytes each) per wavefront.
  // K: LDS position (row, 16-byte slot) holds the row's chunk slot ^ (row % 16), so that the fragment reads of 16 lanes
  // (16 rows, same chunk) spread over the banks.  V: chunk slot ^ 4 * (row % 4): one pass of a transposing read takes
  // 32 bytes (two chunks) of each of 4 consecutive rows for each of two 16-lane groups 32 bytes apart, and with the
  // rows 4 chunks apart those 16 chunks are all different (with K's swizzle rows 2 e and 2 e + 1 shared a pair of
  // chunks: two lanes per bank, measured as bank conflicts in 60 % of the LDS's active cycles).
  uint32_t koff[4], voff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int krow = (wave * 4 + i) * 4 + (lane >> 4);
    koff[i] = (uint32_t)krow * p.k_st + (uint32_t)(((lane & 15) ^ (krow & 15)) << 4);
    voff[i] = (uint32_t)krow * p.v_st + (uint32_t)(((lane & 15) ^ ((krow & 3) << 2)) << 4);
  }
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lptr_t)lds;
  const int nblk = 2 * qb + 2;  // key blocks that hold a key <= the block's last query (even: the last one uses stage 1)
  // copy c (0..7) of key block j: 0-3 K, 4-7 V; j == nblk stands for key block 0 of the next item (stage 0 again)
  auto issue_one = [&](int j, int c) __attribute__((always_inline)) {
    const int i = c & 3;
    const bool nxt = j == nblk;
    const size_t blk = nxt ? 0 : (size_t)j;
    if (c < 4) {
      at_async_copy_16((nxt ? kp_next : kp) + blk * kKB * p.k_st, koff[i],
                       lds_base + (uint32_t)((j & 1) * kKBytes + (wave * 4 + i) * 1024));
    } else {
      at_async_copy_16((nxt ? vp_next : vp) + blk * kKB * p.v_st, voff[i],
                       lds_base + (uint32_t)(2 * kKBytes + (j & 1) * kVBytes + (wave * 4 + i) * 1024));
    }
  };
  auto issue = [&](int j) __attribute__((always_inline)) {
#pragma unroll
    for (int c = 0; c < 8; ++c) issue_one(j, c);
  };

  f32x16_t o[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[dt][r] = 0.0f;
  float m = -__builtin_inff(), lsum = 0.0f;

  if (item == 0) issue(0);  // later items: fetched by the item before
  for (int j = 0; j < nblk; ++j) {
    at_wait_vmcnt<0>();  // this wavefront's copies of block j have landed
    asm volatile("s_barrier" ::: "memory");  // ... everyone's have, and everyone has finished with block j - 1's buffers
    const bool more = j + 1 < nblk || has_next;
    const int key0 = j * kKB;
    const bool skip = key0 > q0 + 31;  // every key of the block lies after every query of this wavefront
    if (skip && more) issue(j + 1);
    if (skip) continue;
    const unsigned char* Kb = lds + (j & 1) * kKBytes;
    const unsigned char* Vb = lds + 2 * kKBytes + (j & 1) * kVBytes;

    // S^T = K Q^T: the K fragments are read kKRing - 1 contraction steps ahead of the matrix instructions that take them,
    // and the wavefront's 8 copies of the next key block go out between those instructions (issued in one run they
    // hold the wavefront for as long as the address path takes to accept them)
    // V fragments (A operand of O^T += V^T P^T: lane = d, 8 keys) come from V's natural [key][d] rows by transposing
    // reads: in a group of 16 lanes, lane 4 e + a points at 4 consecutive d (8 bytes) of key row e, and lane i
    // receives element i % 4 of the windows of lanes i / 4, 4 + i / 4, 8 + i / 4, 12 + i / 4: with the windows at
    // d = c0 + 4 a of keys k0 + e, lane i gets d = c0 + i of keys k0 .. k0 + 3.  Two reads (keys k0 .., k0 + 8 ..) make a
    // fragment.  The reads of steps 0 and 1 go out between the matrix instructions of the first product, those of
    // steps 2 and 3 between the exponentials.
    bf16x8_t vf[4][4];
    auto read_v_one = [&](int s, int dt) __attribute__((always_inline)) {
      const int dbyte = (dt * 32 + (l32 & 16) + 4 * (lane & 3)) * 2;
      const int row0 = 16 * s + 4 * g + ((lane & 15) >> 2), row1 = row0 + 8;
      const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (lds_s16x4_t*)(lptr_t)(Vb + row0 * 256 + (((dbyte >> 4) ^ ((row0 & 3) << 2)) << 4) + (dbyte & 8)));
      const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (lds_s16x4_t*)(lptr_t)(Vb + row1 * 256 + (((dbyte >> 4) ^ ((row1 & 3) << 2)) << 4) + (dbyte & 8)));
      s16x8_t both;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        both[e] = lo[e];
        both[4 + e] = hi[e];
      }
      vf[s][dt] = __builtin_bit_cast(bf16x8_t, both);
    };
    bf16x8_t kf[kKRing][2];  // ring: step s uses kf[s % kKRing]
    auto read_k = [&](int s) __attribute__((always_inline)) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int row = t * 32 + l32;
        kf[s % kKRing][t] = *(const bf16x8_t*)(Kb + row * 256 + (((2 * s + g) ^ (row & 15)) << 4));
      }
    };
#pragma unroll
    for (int s = 0; s < kKRing - 1; ++s) read_k(s);
    f32x16_t sc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[t][r] = 0.0f;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < 8; ++s) {
#pragma unroll
      for (int t = 0; t < 2; ++t) sc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[s % kKRing][t], qf[s], sc[t], 0, 0, 0);
      if (s + kKRing - 1 < 8) read_k(s + kKRing - 1);
      read_v_one(s >> 2, s & 3);
      if (more) issue_one(j + 1, s);
      __builtin_amdgcn_sched_barrier(0);
    }
    // register r of tile t is key key0 + 32 t + 8 (r / 4) + 4 g + r % 4
    if (key0 + kKB - 1 > q0) {  // the block reaches past this wavefront's first query: mask
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = key0 + 32 * t + 8 * (r >> 2) + 4 * g + (r & 3);
          if (key > qi) sc[t][r] = -__builtin_inff();
        }
    }
    float mx = sc[0][0];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sc[t][r]);
    mx = max_with_other_half(mx);  // finite: key0 <= q0 <= this lane's query, so key0 itself is not masked
    // The reference point m of the exponentials moves only when some query of the wavefront has met a score more than
    // kGrow (in the exponent's unit) above it: probabilities then reach 2^kGrow instead of 1, which fp32 sums and the
    // bf16 rounding (relative) do not mind, and most key blocks skip the rescaling of the 64 accumulator registers.
    if (__builtin_amdgcn_ballot_w64((mx - m) * p.c > kGrow) != 0) {
      const float mn = fmaxf(m, mx);
      const float alpha = __builtin_amdgcn_exp2f((m - mn) * p.c);
      m = mn;
      lsum *= alpha;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
    }
    const float mc = m * p.c;
    float psum = 0.0f;
    // Contraction step s of O^T += V^T P^T takes the probabilities of 8 keys per lane: registers 8 (s % 2) .. + 8 of
    // score tile s / 2.  A wavefront that issues matrix instructions back to back waits at each for the pipe to take it,
    // so the 4 of step s are issued one at a time with two exponentials of step s + 1 after each (about what fits under
    // one of them); only step 0's exponentials and step 3's matrix instructions have nothing to share the time with.
    // The V fragments of steps 2 and 3 are read between the exponentials of steps 0, 1 and of step 2.
    auto exp_one = [&](int s, int r) __attribute__((always_inline)) {  // r: 0..7 within step s
      const int t = s >> 1, rr = (s & 1) * 8 + r;
      sc[t][rr] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[t][rr], p.c, -mc));
      psum += sc[t][rr];
      if (t == 0 && (rr & 3) == 3) read_v_one(2, rr >> 2);
      if (s == 2 && (rr & 1) == 1) read_v_one(3, rr >> 1);
    };
#pragma unroll
    for (int r = 0; r < 8; ++r) exp_one(0, r);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int t = s >> 1, r0 = (s & 1) * 8;
      uint4 pw;
      pw.x = f32x2_to_bf16x2_bits(sc[t][r0 + 0], sc[t][r0 + 1]);
      pw.y = f32x2_to_bf16x2_bits(sc[t][r0 + 2], sc[t][r0 + 3]);
      pw.z = f32x2_to_bf16x2_bits(sc[t][r0 + 4], sc[t][r0 + 5]);
      pw.w = f32x2_to_bf16x2_bits(sc[t][r0 + 6], sc[t][r0 + 7]);
      const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, pw);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) {
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[s][dt], pf, o[dt], 0, 0, 0);
        if (s < 3) {
          exp_one(s + 1, 2 * dt);
          exp_one(s + 1, 2 * dt + 1);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    lsum += psum;
  }
  if (!has_next) at_wait_vmcnt<0>();  // no copy may be in flight towards LDS when the work-group retires
  lsum += __shfl_xor(lsum, 32, 64);
  const float inv = 1.0f / lsum;
  // register r of tile dt is d = 32 dt + 8 (r / 4) + 4 g + r % 4: four consecutive d per group of four registers
  unsigned char* op = p.out + (size_t)b * p.o_sb + (size_t)h * p.o_sh + (size_t)qi * p.o_st;
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) {
    float y[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) y[r] = o[dt][r] * inv;
    if constexpr (MX) {
      uint32_t mbits = 0;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        y[r] = DTypeTraits<MASE_DT_BF16>::round(y[r]);  // the quantizer reads the stored bf16 value
        mbits = max(mbits, f2bits(y[r]) & 0x7FFFFFFFu);
      }
      mbits = umax_with_other_half(mbits);
      int k = 0, kc = 0;
      const int state = block_exponent<MASE_DT_BF16>(mbits, p.mx, k, kc);
      if (state == 0) {
        const int up = p.mx.qshift - k, dn = kc - p.mx.qshift;
#pragma unroll
        for (int r = 0; r < 16; ++r) y[r] = ldexpf(fminf(fmaxf(rintf(ldexpf(y[r], up)), p.mx.lo), p.mx.hi), dn);
      } else {
        int code;
#pragma unroll
        for (int r = 0; r < 16; ++r) y[r] = mxint_element<MASE_DT_BF16>(y[r], state, k, kc, p.mx, code);
      }
    }
#pragma unroll
    for (int qq = 0; qq < 4; ++qq) {
      uint2 w;
      w.x = f32x2_to_bf16x2_bits(y[4 * qq], y[4 * qq + 1]);
      w.y = f32x2_to_bf16x2_bits(y[4 * qq + 2], y[4 * qq + 3]);
      *(uint2*)(op + (32 * dt + 8 * qq + 4 * g) * 2) = w;
    }
  }
  }  // items
}

}  // namespace
}  // namespace mase

namespace mase {
namespace {
int attention_causal_impl(const void* q, const void* k, const void* v, void* out, size_t batch, size_t heads,
                          size_t tokens, size_t head_dim, size_t q_stride_b, size_t q_stride_h,
                          size_t q_stride_t, size_t k_stride_b, size_t k_stride_h, size_t k_stride_t,
                          size_t v_stride_b, size_t v_stride_h, size_t v_stride_t, size_t o_stride_b,
                          size_t o_stride_h, size_t o_stride_t, int dtype, float scaling, const void* q_cos,
                          const void* q_sin, size_t cs_stride_b, size_t cs_stride_t, int element_bits,
                          const uint32_t* log2_tab, void* stream) {
  if (batch == 0 || heads == 0 || tokens == 0) return MASE_OK;
  if (q == nullptr || k == nullptr || v == nullptr || out == nullptr) return MASE_ERR_NULL;
  if (dtype != MASE_DT_BF16) return MASE_ERR_DTYPE;
  if (!(scaling > 0.0f) || !(scaling < 3.0e38f)) return MASE_ERR_PARAM;  // the running maximum is taken before scaling
  if (head_dim != 128 || tokens % 128 != 0 || tokens > (1u << 20) || batch * heads > (1u << 20)) return MASE_ERR_SHAPE;
  // strides in elements; rows of 128 elements must be whole 16-byte chunks, a token stride must fit 32 bits in bytes
  const size_t strides[12] = {q_stride_b, q_stride_h, q_stride_t, k_stride_b, k_stride_h, k_stride_t,
                              v_stride_b, v_stride_h, v_stride_t, o_stride_b, o_stride_h, o_stride_t};
  for (size_t s : strides)
    if (s % 8 != 0) return MASE_ERR_ALIGN;
  if (q_stride_t < 128 || k_stride_t < 128 || v_stride_t < 128 || o_stride_t < 128) return MASE_ERR_SHAPE;
  // 32-bit lane offsets: a key block's rows (up to 63 token strides) for k and v, one token stride for q and the output
  if (k_stride_t * 2 * tokens > 0xFFFFFFFFull || v_stride_t * 2 * tokens > 0xFFFFFFFFull ||
      q_stride_t * 2 > 0xFFFFFFFFull || o_stride_t * 2 > 0xFFFFFFFFull)
    return MASE_ERR_SHAPE;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out)) return MASE_ERR_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const bool mx = element_bits != 0, rope = q_cos != nullptr || q_sin != nullptr;
  if (rope) {
    if (q_cos == nullptr || q_sin == nullptr) return MASE_ERR_NULL;
    if (!aligned16(q_cos) || !aligned16(q_sin) || cs_stride_b % 8 != 0 || cs_stride_t % 8 != 0) return MASE_ERR_ALIGN;
    if (cs_stride_t < 128 || cs_stride_t * 2 > 0xFFFFFFFFull) return MASE_ERR_SHAPE;
  }
  const void* kernels[4] = {(const void*)attn_causal_fwd_kernel<false, false>, (const void*)attn_causal_fwd_kernel<true, false>,
                            (const void*)attn_causal_fwd_kernel<false, true>, (const void*)attn_causal_fwd_kernel<true, true>};
  static std::atomic<uint64_t> attr_done{0};
  if (!device_setup_done(attr_done)) {
    for (const void* kfn : kernels)
      if (hipFuncSetAttribute(kfn, hipFuncAttributeMaxDynamicSharedMemorySize, kAttnLds) != hipSuccess) return MASE_ERR_LAUNCH;
    mark_device_setup_done(attr_done);
  }
  const int BH = (int)(batch * heads), T = (int)tokens;
  AttnParams p;
  p.q = (const unsigned char*)q;
  p.k = (const unsigned char*)k;
  p.v = (const unsigned char*)v;
  p.v_sb = v_stride_b * 2; p.v_sh = v_stride_h * 2; p.v_st = (uint32_t)(v_stride_t * 2);
  p.out = (unsigned char*)out;
  p.BH = BH;
  p.H = (int)heads;
  p.T = T;
  p.q_sb = q_stride_b * 2; p.q_sh = q_stride_h * 2; p.q_st = (uint32_t)(q_stride_t * 2);
  p.k_sb = k_stride_b * 2; p.k_sh = k_stride_h * 2; p.k_st = (uint32_t)(k_stride_t * 2);
  p.o_sb = o_stride_b * 2; p.o_sh = o_stride_h * 2; p.o_st = (uint32_t)(o_stride_t * 2);
  p.c = scaling * 1.4426950408889634f;
  if (mx) {
    if (element_bits < 2 || element_bits > 24 || log2_tab == nullptr) return MASE_ERR_PARAM;
    p.mx.qshift = element_bits - 1;
    p.mx.bias = 127;
    p.mx.scale_max = 255;
    p.mx.lo = mase_round_scalar_to_dtype(-(double)(1 << (element_bits - 1)), dtype);
    p.mx.hi = mase_round_scalar_to_dtype((double)((1 << (element_bits - 1)) - 1), dtype);
    p.mx.tab = log2_tab;
  } else {
    p.mx = MxintParams{};
  }
  // persistent form when the work divides evenly over two work-groups per CU (see the kernel)
  p.rounds = 0;
  p.bh_lanes = 0;
  unsigned n_wg = (unsigned)(BH * (T / kQB));
  {
    const int n_cu = device_cu_count();  // of the device the call runs on
    if (n_cu <= 0) return MASE_ERR_LAUNCH;
    const int n_qb = T / kQB, wg_per_xcd = 2 * n_cu / 8;
    if (BH % 8 == 0 && n_cu % 8 == 0 && n_qb <= wg_per_xcd && wg_per_xcd % n_qb == 0) {
      const int lanes = wg_per_xcd / n_qb, per_xcd = BH / 8;
      if (per_xcd % lanes == 0 && per_xcd / lanes >= 2) {
        p.rounds = per_xcd / lanes;
        p.bh_lanes = lanes;
        n_wg = (unsigned)(8 * wg_per_xcd);
      }
    }
  }
  p.q_cos = (const unsigned char*)q_cos;
  p.q_sin = (const unsigned char*)q_sin;
  p.cs_sb = cs_stride_b * 2;
  p.cs_st = (uint32_t)(cs_stride_t * 2);
  const dim3 grid(n_wg), block(256);
  if (mx && rope) hipLaunchKernelGGL((attn_causal_fwd_kernel<true, true>), grid, block, kAttnLds, st, p);
  else if (mx) hipLaunchKernelGGL((attn_causal_fwd_kernel<true, false>), grid, block, kAttnLds, st, p);
  else if (rope) hipLaunchKernelGGL((attn_causal_fwd_kernel<false, true>), grid, block, kAttnLds, st, p);
  else hipLaunchKernelGGL((attn_causal_fwd_kernel<false, false>), grid, block, kAttnLds, st, p);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}
}  // namespace
}  // namespace mase

extern "C" int mase_attention_causal(const void* q, const void* k, const void* v, void* out, size_t batch, size_t heads,
                                     size_t tokens, size_t head_dim, size_t q_stride_b, size_t q_stride_h,
                                     size_t q_stride_t, size_t k_stride_b, size_t k_stride_h, size_t k_stride_t,
                                     size_t v_stride_b, size_t v_stride_h, size_t v_stride_t, size_t o_stride_b,
                                     size_t o_stride_h, size_t o_stride_t, int dtype, float scaling, void* stream) {
  return mase::attention_causal_impl(q, k, v, out, batch, heads, tokens, head_dim, q_stride_b, q_stride_h, q_stride_t,
                                     k_stride_b, k_stride_h, k_stride_t, v_stride_b, v_stride_h, v_stride_t, o_stride_b,
                                     o_stride_h, o_stride_t, dtype, scaling, nullptr, nullptr, 0, 0, 0, nullptr, stream);
}

extern "C" int mase_attention_causal_fused(const void* q, const void* k, const void* v, void* out, size_t batch,
                                           size_t heads, size_t tokens, size_t head_dim, size_t q_stride_b,
                                           size_t q_stride_h, size_t q_stride_t, size_t k_stride_b, size_t k_stride_h,
                                           size_t k_stride_t, size_t v_stride_b, size_t v_stride_h, size_t v_stride_t,
                                           size_t o_stride_b, size_t o_stride_h, size_t o_stride_t, int dtype,
                                           float scaling, const void* q_cos, const void* q_sin, size_t cs_stride_b,
                                           size_t cs_stride_t, int element_bits, const uint32_t* log2_tab, void* stream) {
  return mase::attention_causal_impl(q, k, v, out, batch, heads, tokens, head_dim, q_stride_b, q_stride_h, q_stride_t,
                                     k_stride_b, k_stride_h, k_stride_t, v_stride_b, v_stride_h, v_stride_t, o_stride_b,
                                     o_stride_h, o_stride_t, dtype, scaling, q_cos, q_sin, cs_stride_b, cs_stride_t,
                                     element_bits, log2_tab, stream);
}
