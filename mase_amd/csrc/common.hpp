// Shared device helpers for the gfx950 quantize-dequantize kernels.
//
// All arithmetic is carried in fp32 registers.  Every reference operation on a bf16/fp16 tensor is
// "compute in fp32, round once to the tensor dtype", so a kernel only needs an explicit rounding step
// where the fp32 result is not already representable in the tensor dtype; the places where that can
// happen are listed next to each kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/mase_amd.h"

namespace mase {

constexpr int kThreads = 256;

// ---------------------------------------------------------------------------------------------
// dtype traits: 16-byte vectors of the storage type <-> fp32 registers
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float bits2f(uint32_t b) { return __builtin_bit_cast(float, b); }
__device__ __forceinline__ uint32_t f2bits(float f) { return __builtin_bit_cast(uint32_t, f); }

// fp32 -> bf16, round-to-nearest-even, with the hardware conversion of this part (v_cvt_pk_bf16_f32: two values per
// instruction, first operand in the low half); NaN stays NaN.  Written as a vector conversion, which the compiler
// selects that instruction for, and not as the instruction by name: a vector instruction that reads the result of a
// transcendental one (v_exp_f32, v_rcp_f32, ...) needs a wait state between the two on this part, which the compiler
// inserts for instructions it knows and cannot for the text of an asm statement (seen as a wrong conversion of the
// second of two exponentials, now and then).
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) { return f32x2_to_bf16x2_bits(f, 0.0f) & 0xFFFFu; }
__device__ __forceinline__ float round_to_bf16(float f) { return bits2f(f32x2_to_bf16x2_bits(0.0f, f) & 0xFFFF0000u); }
// fp32 -> fp16 bits, round-to-nearest-even.  Issued as an explicit instruction: when the compiler sees
// "(half)(a * b)" it fuses the pair into a mixed-precision fma with a +0 addend, which turns a -0 product
// into +0 and so loses the sign of zero that the reference keeps.  The s_nop is the wait state that a reader of a
// transcendental instruction's result needs (see above); the compiler does not look inside the statement.
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  uint32_t h;
  asm("s_nop 0\n\tv_cvt_f16_f32 %0, %1" : "=v"(h) : "v"(f));
  return h & 0xFFFFu;
}
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}
__device__ __forceinline__ float round_to_f16(float f) { return f16_bits_to_f32(f32_to_f16_bits(f)); }

// streaming (non-temporal) 16-byte accesses: inputs are read once and outputs never re-read
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_nt(const uint4* p) {
  u32x4_t v = __builtin_nontemporal_load((const u32x4_t*)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void store_nt(uint4* p, const uint4& v) {
  u32x4_t w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, (u32x4_t*)p);
}

typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void store_nt(uint2* p, const uint2& v) {
  u32x2_t w = {v.x, v.y};
  __builtin_nontemporal_store(w, (u32x2_t*)p);
}

template <int DT> struct DTypeTraits;

template <> struct DTypeTraits<MASE_DT_F32> {
  static constexpr int kVec = 4;       // elements per 16-byte vector
  static constexpr int kBytes = 4;
  static constexpr int kMaxPow2 = 127; // largest k with 2^k finite
  static constexpr uint32_t kTinyBits = 0x00800000u;  // finfo.tiny as fp32 bits
  __device__ static __forceinline__ float round(float f) { return f; }
  __device__ static __forceinline__ void unpack(const uint4& v, float* x) {
    x[0] = bits2f(v.x); x[1] = bits2f(v.y); x[2] = bits2f(v.z); x[3] = bits2f(v.w);
  }
  __device__ static __forceinline__ uint4 pack(const float* x) {
    return make_uint4(f2bits(x[0]), f2bits(x[1]), f2bits(x[2]), f2bits(x[3]));
  }
  __device__ static __forceinline__ float load1(const void* p, size_t i) { return ((const float*)p)[i]; }
  __device__ static __forceinline__ void store1(void* p, size_t i, float f) { ((float*)p)[i] = f; }
};

template <> struct DTypeTraits<MASE_DT_BF16> {
  static constexpr int kVec = 8;
  static constexpr int kBytes = 2;
  static constexpr int kMaxPow2 = 127;
  static constexpr uint32_t kTinyBits = 0x00800000u;
  __device__ static __forceinline__ float round(float f) { return round_to_bf16(f); }
  __device__ static __forceinline__ void unpack(const uint4& v, float* x) {
    x[0] = bits2f(v.x << 16); x[1] = bits2f(v.x & 0xFFFF0000u);
    x[2] = bits2f(v.y << 16); x[3] = bits2f(v.y & 0xFFFF0000u);
    x[4] = bits2f(v.z << 16); x[5] = bits2f(v.z & 0xFFFF0000u);
    x[6] = bits2f(v.w << 16); x[7] = bits2f(v.w & 0xFFFF0000u);
  }
  __device__ static __forceinline__ uint4 pack(const float* x) {
    uint4 v;
    v.x = f32x2_to_bf16x2_bits(x[0], x[1]);
    v.y = f32x2_to_bf16x2_bits(x[2], x[3]);
    v.z = f32x2_to_bf16x2_bits(x[4], x[5]);
    v.w = f32x2_to_bf16x2_bits(x[6], x[7]);
    return v;
  }
  __device__ static __forceinline__ float load1(const void* p, size_t i) {
    return bits2f((uint32_t)((const uint16_t*)p)[i] << 16);
  }
  __device__ static __forceinline__ void store1(void* p, size_t i, float f) {
    ((uint16_t*)p)[i] = (uint16_t)f32_to_bf16_bits(f);
  }
};

template <> struct DTypeTraits<MASE_DT_F16> {
  static constexpr int kVec = 8;
  static constexpr int kBytes = 2;
  static constexpr int kMaxPow2 = 15;
  static constexpr uint32_t kTinyBits = 0x38800000u;  // 2^-14 as fp32 bits
  __device__ static __forceinline__ float round(float f) { return round_to_f16(f); }
  __device__ static __forceinline__ float h2f(uint32_t h) { return f16_bits_to_f32(h); }
  __device__ static __forceinline__ uint32_t f2h(float f) { return f32_to_f16_bits(f); }
  __device__ static __forceinline__ void unpack(const uint4& v, float* x) {
    x[0] = h2f(v.x & 0xFFFFu); x[1] = h2f(v.x >> 16);
    x[2] = h2f(v.y & 0xFFFFu); x[3] = h2f(v.y >> 16);
    x[4] = h2f(v.z & 0xFFFFu); x[5] = h2f(v.z >> 16);
    x[6] = h2f(v.w & 0xFFFFu); x[7] = h2f(v.w >> 16);
  }
  __device__ static __forceinline__ uint4 pack(const float* x) {
    uint4 v;
    v.x = f2h(x[0]) | (f2h(x[1]) << 16);
    v.y = f2h(x[2]) | (f2h(x[3]) << 16);
    v.z = f2h(x[4]) | (f2h(x[5]) << 16);
    v.w = f2h(x[6]) | (f2h(x[7]) << 16);
    return v;
  }
  __device__ static __forceinline__ float load1(const void* p, size_t i) { return h2f(((const uint16_t*)p)[i]); }
  __device__ static __forceinline__ void store1(void* p, size_t i, float f) { ((uint16_t*)p)[i] = (uint16_t)f2h(f); }
};

// ---------------------------------------------------------------------------------------------
// wave64 lane exchange: max over aligned groups of LANES consecutive lanes (LANES = 1..64, power of 2)
// quad_perm / row_half_mirror / row_mirror DPP for 2..16 lanes, ds_bpermute beyond a 16-lane row.
// ---------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_mov(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xF, 0xF, false);
}

template <int LANES>
__device__ __forceinline__ uint32_t group_max_u32(uint32_t v) {
  if constexpr (LANES >= 2) v = max(v, dpp_mov<0xB1>(v));   // quad_perm:[1,0,3,2]
  if constexpr (LANES >= 4) v = max(v, dpp_mov<0x4E>(v));   // quad_perm:[2,3,0,1]
  if constexpr (LANES >= 8) v = max(v, dpp_mov<0x141>(v));  // row_half_mirror
  if constexpr (LANES >= 16) v = max(v, dpp_mov<0x140>(v)); // row_mirror
  if constexpr (LANES >= 32) v = max(v, (uint32_t)__shfl_xor((int)v, 16, 64));
  if constexpr (LANES >= 64) v = max(v, (uint32_t)__shfl_xor((int)v, 32, 64));
  return v;
}

// ---------------------------------------------------------------------------------------------
// max |x| over the elements of one 16-byte vector, returned as fp32 bits (NaN compares largest).
// 16-bit types are reduced two at a time with packed 16-bit integer max before widening.
// ---------------------------------------------------------------------------------------------
typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
  u16x2_t r = __builtin_elementwise_max(__builtin_bit_cast(u16x2_t, a), __builtin_bit_cast(u16x2_t, b));
  return __builtin_bit_cast(uint32_t, r);
}

template <int DT>
__device__ __forceinline__ uint32_t vec_absmax_bits(const uint4& v) {
  if constexpr (DT == MASE_DT_F32) {
    return max(max(v.x & 0x7FFFFFFFu, v.y & 0x7FFFFFFFu), max(v.z & 0x7FFFFFFFu, v.w & 0x7FFFFFFFu));
  } else {
    uint32_t m = pk_max_u16(pk_max_u16(v.x & 0x7FFF7FFFu, v.y & 0x7FFF7FFFu),
                            pk_max_u16(v.z & 0x7FFF7FFFu, v.w & 0x7FFF7FFFu));
    m = max(m & 0xFFFFu, m >> 16);
    if constexpr (DT == MASE_DT_BF16) return m << 16;
    // fp16: widen (monotone); Inf/NaN patterns map to fp32 Inf/NaN
    return f2bits(f16_bits_to_f32(m));
  }
}

// two fp32 values that are exactly representable in bf16 -> one packed dword (no rounding step)
__device__ __forceinline__ uint32_t pack_bf16_exact(float lo, float hi) {
  return __builtin_amdgcn_perm(f2bits(hi), f2bits(lo), 0x07060302u);
}

// ---------------------------------------------------------------------------------------------
// ceil(log2(v)) / floor(log2(v)) "as the host library evaluates them in the tensor dtype".
//
// v is a positive, finite, non-zero value of the tensor dtype, given as fp32 bits.  The exact integer
// answer is corrected with per-exponent thresholds measured on the host at start-up:
//   tab[k + 149]        largest normalised 23-bit mantissa M > 0 for which ceil(log2(2^k (1+M/2^23))) == k
//                       (0 when there is none: the exact answer k+1 is what the library returns)
//   tab[288 + k + 149]  smallest M for which floor(log2(2^k (1+M/2^23))) == k+1 (0x800000 when none)
// ---------------------------------------------------------------------------------------------
constexpr int kLog2TabHalf = 288;
// (Words 277..279 of each half hold a host-side summary of the table; the kernels do not read them.)

__device__ __forceinline__ int split_pow2(uint32_t b, uint32_t& M) {
  int E = (int)(b >> 23);
  M = b & 0x7FFFFFu;
  if (E == 0) {  // fp32 subnormal: normalise
    int sh = __clz(M) - 8;
    M = (M << sh) & 0x7FFFFFu;
    E = 1 - sh;
  }
  return E - 127;
}

__device__ __forceinline__ int ceil_log2_lib(uint32_t b, const uint32_t* __restrict__ tab) {
  uint32_t M;
  int k = split_pow2(b, M);
  if (M == 0) return k;
  return (M <= tab[k + 149]) ? k : k + 1;
}

// Wave-resident copy of the table entries for k in [-32, 31] (lane i holds k = i - 32), read with one
// coalesced load per wavefront that is in flight together with the data load.  A lookup is then a
// ds_bpermute (cross-lane read, no memory access); exponents outside the window fall back to the table.
// Every lane of the wavefront must call init() and lookups before any lane exits.
struct WaveLog2 {
  uint32_t reg;
  const uint32_t* tab;
  int half;
  __device__ __forceinline__ void init(const uint32_t* __restrict__ t, int h) {
    tab = t;
    half = h;
    reg = t[h + 149 - 32 + (int)(threadIdx.x & 63)];
  }
  __device__ __forceinline__ uint32_t threshold(int k) const {
    int kb = k + 32;
    uint32_t thr = (uint32_t)__builtin_amdgcn_ds_bpermute((kb & 63) << 2, (int)reg);
    if ((unsigned)kb >= 64u) thr = tab[half + k + 149];
    return thr;
  }
};
__device__ __forceinline__ int ceil_log2_lib(uint32_t b, const uint32_t* __restrict__, const WaveLog2& w) {
  uint32_t M;
  int k = split_pow2(b, M);
  uint32_t thr = w.threshold(k);
  return (M == 0 || M <= thr) ? k : k + 1;
}
__device__ __forceinline__ int floor_log2_lib(uint32_t b, const uint32_t* __restrict__, const WaveLog2& w) {
  uint32_t M;
  int k = split_pow2(b, M);
  return (M >= w.threshold(k)) ? k + 1 : k;
}

__device__ __forceinline__ int floor_log2_lib(uint32_t b, const uint32_t* __restrict__ tab) {
  uint32_t M;
  int k = split_pow2(b, M);
  return (M >= tab[kLog2TabHalf + k + 149]) ? k + 1 : k;
}

// 2^e as fp32 for e in [-149, 127]; callers handle e > 127 themselves
__device__ __forceinline__ float pow2f(int e) {
  return (e >= -126) ? bits2f((uint32_t)(e + 127) << 23) : bits2f(1u << (e + 149));
}

__device__ __forceinline__ float qnan() { return bits2f(0x7FC00000u); }

// host-side launch geometry
static inline unsigned blocks_for(size_t items, size_t per_block) {
  return (unsigned)((items + per_block - 1) / per_block);
}

static inline bool aligned16(const void* p) { return (((uintptr_t)p) & 15u) == 0; }

// ---------------------------------------------------------------------------------------------
// host side: per-device facts looked up once, safely from several host threads
// ---------------------------------------------------------------------------------------------
// number of compute units of the current device (0 on error); cached per device index
inline int device_cu_count() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  std::atomic<int>& slot = cached[dev & 63];
  int n = slot.load(std::memory_order_relaxed);
  if (n > 0 && dev < 64) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
  if (dev < 64) slot.store(n, std::memory_order_relaxed);
  return n;
}

// One bit per device index in a call site's record `done`: whether its once-per-device set-up (a kernel attribute
// belongs to the (kernel, device) pair) has run on the current device.  Two threads may both run an idempotent set-up
// the first time; none reads the bit as set before the set-up has finished.
inline bool device_setup_done(const std::atomic<uint64_t>& done) {
  int dev = 0;
  return hipGetDevice(&dev) == hipSuccess && dev < 64 && (done.load(std::memory_order_acquire) >> dev & 1) != 0;
}
inline void mark_device_setup_done(std::atomic<uint64_t>& done) {
  int dev = 0;
  if (hipGetDevice(&dev) == hipSuccess && dev < 64) done.fetch_or(1ull << dev, std::memory_order_release);
}
// raises one kernel's dynamic-LDS limit once per device
inline bool set_dynamic_lds_once(std::atomic<uint64_t>& done, const void* kernel, int bytes) {
  if (device_setup_done(done)) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return false;
  mark_device_setup_done(done);
  return true;
}

}  // namespace mase
