// Block floating point (MSFP) quantize-dequantize for gfx950.
//
// Reference arithmetic (nn/quantizers/block_fp.py:7-82), every op in the tensor dtype T, per tile
// (blocking: nn/quantizers/utils.py:350-629), mb = width-1, bias = 2^(ew-1)-1 unless given:
//   mx  = max|x| over the tile (ragged edges zero padded)
//   e   = clamp(ceil(log2(mx)), -bias, 2^ew-1-bias)            (log2 as the library rounds it in T)
//   v_i = |x_i| + 1e-9                                          (rounded to T)
//   q_i = clamp(rne(v_i / 2^e * 2^mb), 0, 2^mb-1)               (bounds cast to T)
//   y_i = sign(x_i + 1e-9) * 2^e * (q_i / 2^mb)
//   out = isclose(x_i, 0) ? x_i (with -0 -> +0) : y_i carrying the sign of x_i
// Sign of a zero result: the reference reassembles 2-D weights and 3-D activations with F.fold, which
// *adds* the blocks into a zero buffer, so a -0 becomes +0 there; 1-D and 2-D activation blocking is a
// reshape and keeps -0.  The caller selects the behaviour with `zero_sign_mode`.
// The reference's substitute exponent for all-zero tiles never reaches an output (all elements of such a
// tile take the isclose branch), so tiles are independent.  Power-of-two scalings are exact in fp32
// registers; T-rounding is applied to v_i and to the final product.  Tiles holding NaN, or whose 2^e
// overflows T, come out as NaN like the reference's 0*inf; an Inf element saturates when 2^e is finite.
//
// Two schedules:
//  * run kernel   tile_rows == 1 and cols % tile_cols == 0: tiles are contiguous runs; one pass, 16-byte
//                 loads/stores, tile maximum by DPP inside the wavefront.
//  * tile kernels any tile shape / ragged edge: pass 1 reduces |x| per tile with atomicMax into a caller
//                 workspace, pass 2 quantizes; both are coalesced along the last dimension.
#include "common.hpp"

#include <mutex>

// ---- scratch of the entry point that allocates nothing (mase_block_fp_qdq_static): the per-tile maxima of the
// two-pass schedule, held in the library's own device image.  Each GPU the library runs on keeps its own 4 MiB copy
// until the process ends.  In host code the array's name is only a handle of the symbol, never a device address: the
// address on a device comes from hipGetSymbolAddress, looked up once per device with that device current.
static __device__ __align__(256) uint32_t scratch[MASE_BLOCK_FP_STATIC_MAX_TILES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
uint32_t* g_scratch_ptr[kMaxDevices];

uint32_t* static_scratch_of_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) return nullptr;
    g_scratch_ptr[dev] = (uint32_t*)ptr;
  }
  return g_scratch_ptr[dev];
}
}  // namespace


#ifndef MASE_RUN_THREADS
#define MASE_RUN_THREADS 64
#endif

namespace mase {
namespace {

struct BfpParams {
  int mb;            // mantissa bits = width - 1
  int e_lo, e_hi;    // exponent clamp
  float qmax;        // 2^mb - 1 as T represents it
  uint32_t close_thr;  // |x| bits <= close_thr  <=>  isclose(x, 0)
  uint32_t zero_sign_mask;  // 0x80000000: a zero result keeps the sign of x; 0: it is +0 (see header)
  const uint32_t* tab;
};

// work-group size of the single-pass kernel: small groups stream best on this part
constexpr int kRunThreads = MASE_RUN_THREADS;

// returns 0: zero tile, 1: regular (e valid), 2: NaN tile.  The log2 lookup runs for every lane (on a
// harmless stand-in when the maximum is zero or not finite): the wave-resident table is read with a
// cross-lane operation that needs all lanes of the wavefront to take part.
template <int DT, typename... Meta>
__device__ __forceinline__ int tile_exponent(uint32_t mbits, const BfpParams& p, int& e, const Meta&... meta) {
  using TR = DTypeTraits<DT>;
  const bool special = (mbits == 0) || (mbits >= 0x7F800000u);
  const int k = ceil_log2_lib(special ? 0x3F800000u : mbits, p.tab, meta...);
  if (mbits == 0) return 0;
  if (mbits > 0x7F800000u) return 2;
  // an infinite maximum has log2 = inf, which the clamp brings down to e_hi
  e = (mbits == 0x7F800000u) ? p.e_hi : min(max(k, p.e_lo), p.e_hi);
  return (e > TR::kMaxPow2) ? 2 : 1;
}

template <int DT>
__device__ __forceinline__ float bfp_element(float x, int state, int e, const BfpParams& p) {
  using TR = DTypeTraits<DT>;
  uint32_t xb = f2bits(x);
  uint32_t ab = xb & 0x7FFFFFFFu;
  if (state == 2) return qnan();
  if (ab <= p.close_thr) return (ab == 0) ? 0.0f : x;
  float v = TR::round(bits2f(ab) + 1e-9f);
  float q = fminf(fmaxf(rintf(ldexpf(v, p.mb - e)), 0.0f), p.qmax);
  float y = ldexpf(q, e - p.mb);
  uint32_t smask = (q == 0.0f) ? p.zero_sign_mask : 0x80000000u;
  return bits2f(f2bits(y) | (xb & smask));
}

// One 16-byte vector per lane.  LPB lanes share a tile (tile_cols = LPB * kVec) or one lane holds SUB tiles.
//
// Fast path (taken per tile): in a regular tile the quantized value is computed on the signed input,
//   q = med3(rne(x * 2^(mb-e)), -qmax, qmax),  y = q * 2^(e-mb)          [fp32: |x| + 1e-9 first, sign copied]
// which equals the reference because
//   * fp16: |x| + 1e-9 always rounds back to |x|;  bf16: it does for |x| >= 2^-21, and smaller elements
//     quantize to 0 either way once e >= mb - 19 (tiles with a smaller exponent take the general path);
//   * q has at most 8 significant bits for bf16 inputs, so y is a bf16 value and is packed by truncation;
//   * rne() keeps the sign of zero, which is what zero_sign_mode 0 wants; mode 1 adds +0.0 (-0 -> +0).
// Elements with isclose(x, 0) are selected afterwards: x + 0.0 (the value itself, -0 -> +0).
template <int DT, int LPB, int SUB, int T>
__global__ __launch_bounds__(T) void bfp_run_kernel(const uint4* __restrict__ in, uint4* __restrict__ out,
                                                    size_t n_vec, BfpParams p) {
  using TR = DTypeTraits<DT>;
  constexpr int V = TR::kVec;
  const size_t idx = (size_t)blockIdx.x * T + threadIdx.x;
  const bool live = idx < n_vec;  // whole tiles are live or dead together: n_vec is a multiple of LPB
  const uint4 raw = live ? load_nt(in + idx) : make_uint4(0, 0, 0, 0);
  WaveLog2 meta;
  meta.init(p.tab, 0);
  float x[V], y[V];
  TR::unpack(raw, x);
  if constexpr (SUB == 1) {
    uint32_t m = group_max_u32<LPB>(vec_absmax_bits<DT>(raw));
    int e = 0;
    const int state = tile_exponent<DT>(m, p, e, meta);
    const bool fast = (state == 1) && (DT != MASE_DT_BF16 || e >= p.mb - 19);
    if (fast) {
      const float thr = bits2f(p.close_thr);
      const int up = p.mb - e, dn = e - p.mb;
#pragma unroll
      for (int j = 0; j < V; ++j) {
        float r;
        if constexpr (DT == MASE_DT_F32) {
          float q = fminf(rintf(ldexpf(fabsf(x[j]) + 1e-9f, up)), p.qmax);
          r = bits2f(f2bits(ldexpf(q, dn)) | (f2bits(x[j]) & 0x80000000u));
        } else {
          float q = fminf(fmaxf(rintf(ldexpf(x[j], up)), -p.qmax), p.qmax);
          r = ldexpf(q, dn);
        }
        if (p.zero_sign_mask == 0u) r = r + 0.0f;
        y[j] = (fabsf(x[j]) <= thr) ? (x[j] + 0.0f) : r;
      }
      if (!live) return;
      if constexpr (DT == MASE_DT_BF16) {
        uint4 o;
        o.x = pack_bf16_exact(y[0], y[1]);
        o.y = pack_bf16_exact(y[2], y[3]);
        o.z = pack_bf16_exact(y[4], y[5]);
        o.w = pack_bf16_exact(y[6], y[7]);
        store_nt(out + idx, o);
      } else {
        store_nt(out + idx, TR::pack(y));
      }
      return;
    }
#pragma unroll
    for (int j = 0; j < V; ++j) y[j] = bfp_element<DT>(x[j], state, e, p);
  } else {
    constexpr int EPS = V / SUB;
#pragma unroll
    for (int s = 0; s < SUB; ++s) {
      uint32_t m = 0;
#pragma unroll
      for (int j = 0; j < EPS; ++j) m = max(m, f2bits(x[s * EPS + j]) & 0x7FFFFFFFu);
      int e = 0;
      const int state = tile_exponent<DT>(m, p, e, meta);
#pragma unroll
      for (int j = 0; j < EPS; ++j) y[s * EPS + j] = bfp_element<DT>(x[s * EPS + j], state, e, p);
    }
  }
  if (live) store_nt(out + idx, TR::pack(y));
}

__global__ __launch_bounds__(kThreads) void fill_u32_kernel(uint32_t* __restrict__ p, size_t n, uint32_t v) {
  size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (i < n) p[i] = v;
}

struct TileGeom {
  size_t rows, cols;        // per batch item
  size_t tiles_r, tiles_c;  // tiles per batch item along rows / cols
  int b0, b1;
  size_t col_groups;        // groups of kGroup consecutive columns per row
  size_t total_groups;      // batch * rows * col_groups
};
constexpr int kGroup = 8;

// One work-item per group of kGroup consecutive columns of one row.
template <int DT, int PASS>
__global__ __launch_bounds__(kThreads) void bfp_tile_kernel(const void* __restrict__ in, void* __restrict__ out,
                                                            uint32_t* __restrict__ tile_max, TileGeom g,
                                                            BfpParams p) {
  using TR = DTypeTraits<DT>;
  size_t gid = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (gid >= g.total_groups) return;
  size_t cg = gid % g.col_groups;
  size_t row_all = gid / g.col_groups;  // batch * rows + row
  size_t b = row_all / g.rows, r = row_all % g.rows;
  size_t c0 = cg * kGroup;
  size_t c1 = min(c0 + (size_t)kGroup, g.cols);
  size_t tile_row_base = (b * g.tiles_r + r / g.b0) * g.tiles_c;
  size_t off = row_all * g.cols;
  if constexpr (PASS == 1) {
    size_t cur = c0 / g.b1;
    uint32_t m = 0;
    for (size_t c = c0; c < c1; ++c) {
      size_t t = c / g.b1;
      if (t != cur) {
        if (m) atomicMax(&tile_max[tile_row_base + cur], m);
        cur = t;
        m = 0;
      }
      m = max(m, f2bits(TR::load1(in, off + c)) & 0x7FFFFFFFu);
    }
    if (m) atomicMax(&tile_max[tile_row_base + cur], m);
  } else {
    size_t cur = (size_t)-1;
    int e = 0, state = 0;
    for (size_t c = c0; c < c1; ++c) {
      size_t t = c / g.b1;
      if (t != cur) {
        cur = t;
        state = tile_exponent<DT>(tile_max[tile_row_base + cur], p, e);
      }
      TR::store1(out, off + c, bfp_element<DT>(TR::load1(in, off + c), state, e, p));
    }
  }
}

bool run_path_ok(const void* in, const void* out, size_t numel, size_t cols, int b0, int b1, int V) {
  return b0 == 1 && (b1 & (b1 - 1)) == 0 && b1 <= 64 * V && cols % (size_t)b1 == 0 && numel % (size_t)V == 0 &&
         aligned16(in) && aligned16(out);
}

template <int DT>
int launch_bfp(const void* in, void* out, size_t batch, size_t rows, size_t cols, int b0, int b1, const BfpParams& p,
               void* ws, size_t ws_bytes, hipStream_t st) {
  using TR = DTypeTraits<DT>;
  constexpr int V = TR::kVec;
  size_t numel = batch * rows * cols;
  if (run_path_ok(in, out, numel, cols, b0, b1, V)) {
    size_t n_vec = numel / V;
    dim3 grid(blocks_for(n_vec, kRunThreads)), block(kRunThreads);
#define MASE_BFP_CASE(LPB_, SUB_)                                                                              \
  hipLaunchKernelGGL((bfp_run_kernel<DT, LPB_, SUB_, kRunThreads>), grid, block, 0, st, (const uint4*)in, (uint4*)out, \
                     n_vec, p)
    if (b1 >= V) {
      switch (b1 / V) {
        case 1: MASE_BFP_CASE(1, 1); break;
        case 2: MASE_BFP_CASE(2, 1); break;
        case 4: MASE_BFP_CASE(4, 1); break;
        case 8: MASE_BFP_CASE(8, 1); break;
        case 16: MASE_BFP_CASE(16, 1); break;
        case 32: MASE_BFP_CASE(32, 1); break;
        default: MASE_BFP_CASE(64, 1); break;
      }
    } else {
      switch (V / b1) {
        case 2: MASE_BFP_CASE(1, 2); break;
        case 4: MASE_BFP_CASE(1, 4); break;
        default:
          if constexpr (V == 8) MASE_BFP_CASE(1, 8);
          break;
      }
    }
#undef MASE_BFP_CASE
    return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
  }
  TileGeom g;
  g.rows = rows;
  g.cols = cols;
  g.b0 = b0;
  g.b1 = b1;
  g.tiles_r = (rows + b0 - 1) / b0;
  g.tiles_c = (cols + b1 - 1) / b1;
  g.col_groups = (cols + kGroup - 1) / kGroup;
  g.total_groups = batch * rows * g.col_groups;
  size_t n_tiles = batch * g.tiles_r * g.tiles_c;
  if (ws == nullptr || ws_bytes < n_tiles * sizeof(uint32_t)) return MASE_ERR_WORKSPACE;
  uint32_t* tm = (uint32_t*)ws;
  hipLaunchKernelGGL(fill_u32_kernel, dim3(blocks_for(n_tiles, kThreads)), dim3(kThreads), 0, st, tm, n_tiles, 0u);
  dim3 grid(blocks_for(g.total_groups, kThreads)), block(kThreads);
  hipLaunchKernelGGL((bfp_tile_kernel<DT, 1>), grid, block, 0, st, in, out, tm, g, p);
  hipLaunchKernelGGL((bfp_tile_kernel<DT, 2>), grid, block, 0, st, in, out, tm, g, p);
  return hipGetLastError() == hipSuccess ? MASE_OK : MASE_ERR_LAUNCH;
}

int vec_of(int dtype) { return dtype == MASE_DT_F32 ? 4 : 8; }
int min_pow2_of(int dtype) { return dtype == MASE_DT_F32 ? -149 : (dtype == MASE_DT_BF16 ? -133 : -24); }

}  // namespace
}  // namespace mase

extern "C" size_t mase_block_fp_workspace_bytes(size_t batch, size_t rows, size_t cols, int tile_rows, int tile_cols,
                                                int dtype) {
  using namespace mase;
  if (tile_rows <= 0 || tile_cols <= 0) return 0;
  // the run path additionally needs 16-byte aligned pointers; a caller that cannot guarantee them must
  // provide the workspace, so report the tile-path size whenever the shape alone does not decide
  size_t tiles = batch * ((rows + tile_rows - 1) / tile_rows) * ((cols + tile_cols - 1) / tile_cols);
  return tiles * sizeof(uint32_t);
}

extern "C" int mase_block_fp_qdq(const void* in, void* out, size_t batch, size_t rows, size_t cols, int tile_rows,
                                 int tile_cols, int dtype, int width, int exponent_width, int exponent_bias,
                                 int zero_sign_mode, const uint32_t* log2_tab, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  using namespace mase;
  if (batch == 0 || rows == 0 || cols == 0) return MASE_OK;
  if (in == nullptr || out == nullptr || log2_tab == nullptr) return MASE_ERR_NULL;
  if (tile_rows <= 0 || tile_cols <= 0) return MASE_ERR_SHAPE;
  if (dtype != MASE_DT_F32 && dtype != MASE_DT_BF16 && dtype != MASE_DT_F16) return MASE_ERR_DTYPE;
  if (width < 2 || width > 25 || exponent_width < 1 || exponent_width > 16) return MASE_ERR_PARAM;
  BfpParams p;
  p.mb = width - 1;
  int bias = exponent_bias < 0 ? (1 << (exponent_width - 1)) - 1 : exponent_bias;
  p.e_lo = -bias;
  p.e_hi = (1 << exponent_width) - 1 - bias;
  if (p.e_hi < min_pow2_of(dtype)) return MASE_ERR_PARAM;  // 2^e would underflow to zero in the dtype
  p.qmax = mase_round_scalar_to_dtype((double)((1 << p.mb) - 1), dtype);
  p.close_thr = mase_isclose_zero_threshold_bits(dtype);
  p.zero_sign_mask = zero_sign_mode ? 0u : 0x80000000u;
  p.tab = log2_tab;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case MASE_DT_F32:
      return launch_bfp<MASE_DT_F32>(in, out, batch, rows, cols, tile_rows, tile_cols, p, workspace, workspace_bytes, st);
    case MASE_DT_BF16:
      return launch_bfp<MASE_DT_BF16>(in, out, batch, rows, cols, tile_rows, tile_cols, p, workspace, workspace_bytes, st);
    default:
      return launch_bfp<MASE_DT_F16>(in, out, batch, rows, cols, tile_rows, tile_cols, p, workspace, workspace_bytes, st);
  }
}

extern "C" int mase_block_fp_qdq_static(const void* in, void* out, size_t batch, size_t rows, size_t cols, int tile_rows,
                                        int tile_cols, int dtype, int width, int exponent_width, int exponent_bias,
                                        int zero_sign_mode, const uint32_t* log2_tab, void* stream) {
  using namespace mase;
  if (batch == 0 || rows == 0 || cols == 0) return MASE_OK;
  if (tile_rows <= 0 || tile_cols <= 0) return MASE_ERR_SHAPE;
  const size_t tiles = batch * ((rows + tile_rows - 1) / tile_rows) * ((cols + tile_cols - 1) / tile_cols);
  if (tiles > (size_t)MASE_BLOCK_FP_STATIC_MAX_TILES) return MASE_ERR_WORKSPACE;  // more tile maxima than the static scratch holds
  uint32_t* ws = static_scratch_of_current_device();
  if (ws == nullptr) return MASE_ERR_LAUNCH;
  // the two-pass schedule clears the maxima it uses with a fill kernel before pass 1, so what an earlier call
  // left in the scratch does not matter
  return mase_block_fp_qdq(in, out, batch, rows, cols, tile_rows, tile_cols, dtype, width, exponent_width,
                           exponent_bias, zero_sign_mode, log2_tab, ws,
                           (size_t)MASE_BLOCK_FP_STATIC_MAX_TILES * sizeof(uint32_t), stream);
}
