// Entry points of the clip search of the MX quantizers (kernels and what they reproduce: clip_search_kernels.hpp).
#include "clip_search_kernels.hpp"

namespace mase {
namespace {


MxintParams make_mxint_params(int element_bits, int scale_bits, int dtype, const uint32_t* log2_tab) {
  MxintParams p;
  p.qshift = element_bits - 1;
  p.bias = (1 << (scale_bits - 1)) - 1;
  p.scale_max = (1 << scale_bits) - 1;
  p.lo = mase_round_scalar_to_dtype(-(double)(1 << (element_bits - 1)), dtype);
  p.hi = mase_round_scalar_to_dtype((double)((1 << (element_bits - 1)) - 1), dtype);
  p.tab = log2_tab;
  return p;
}

bool make_mxfp_params(int exp_bits, int frac_bits, const uint32_t* log2_tab, MxfpParams& p) {
  const int legal[6][2] = {{4, 3}, {5, 2}, {2, 3}, {3, 2}, {2, 1}, {1, 2}};  // nn/quantizers/mxfp/meta.py:41
  bool ok = false;
  for (auto& l : legal) ok = ok || (l[0] == exp_bits && l[1] == frac_bits);
  if (!ok) return false;
  p.m.E = exp_bits;
  p.m.F = frac_bits;
  p.m.bias = (1 << (exp_bits - 1)) - 1;
  p.m.e_hi = (1 << exp_bits) - 1;
  p.m.frac_hi = (1 << frac_bits) - 1;
  p.m.is_finite = 1;
  p.m.round_mode = 0;
  p.el_emax = p.m.e_hi - p.m.bias;
  p.tab = log2_tab;
  return true;
}

int clip_args(const void* in, const void* ref, void* out, size_t numel, int dtype, int block_size,
              const uint32_t* log2_tab) {
  if (in == nullptr || ref == nullptr || out == nullptr || log2_tab == nullptr) return MASE_ERR_NULL;
  if (block_size != 16 && block_size != 32 && block_size != 64) return MASE_ERR_PARAM;
  if (numel % (size_t)block_size != 0) return MASE_ERR_SHAPE;
  if (dtype != MASE_DT_F32 && dtype != MASE_DT_BF16 && dtype != MASE_DT_F16) return MASE_ERR_DTYPE;
  if (!aligned16(in) || !aligned16(ref) || !aligned16(out)) return MASE_ERR_ALIGN;
  return MASE_OK;
}

}  // namespace
}  // namespace mase

extern "C" int mase_mxint_clip_search(const void* in, const void* ref, void* out, uint8_t* choice, size_t numel,
                                      int dtype, int block_size, int element_bits, int scale_bits,
                                      const uint32_t* log2_tab, void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (int rc = clip_args(in, ref, out, numel, dtype, block_size, log2_tab)) return rc;
  if (element_bits < 2 || element_bits > 24 || scale_bits < 1 || scale_bits > 8) return MASE_ERR_PARAM;
  const MxintParams p = make_mxint_params(element_bits, scale_bits, dtype, log2_tab);
  const size_t n_blocks = numel / (size_t)block_size;
  hipStream_t st = (hipStream_t)stream;
  switch (block_size) {
    case 16: return clip_mxint_search_b16(dtype, in, ref, out, choice, n_blocks, p, st);
    case 32: return clip_mxint_search_b32(dtype, in, ref, out, choice, n_blocks, p, st);
    default: return clip_mxint_search_b64(dtype, in, ref, out, choice, n_blocks, p, st);
  }
}

extern "C" int mase_mxfp_clip_search(const void* in, const void* ref, void* out, uint8_t* choice, size_t numel,
                                     int dtype, int block_size, int exp_bits, int frac_bits, const uint32_t* log2_tab,
                                     void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (int rc = clip_args(in, ref, out, numel, dtype, block_size, log2_tab)) return rc;
  MxfpParams p;
  if (!make_mxfp_params(exp_bits, frac_bits, log2_tab, p)) return MASE_ERR_PARAM;
  const size_t n_blocks = numel / (size_t)block_size;
  hipStream_t st = (hipStream_t)stream;
  switch (block_size) {
    case 16: return clip_mxfp_search_b16(dtype, in, ref, out, choice, n_blocks, p, st);
    case 32: return clip_mxfp_search_b32(dtype, in, ref, out, choice, n_blocks, p, st);
    default: return clip_mxfp_search_b64(dtype, in, ref, out, choice, n_blocks, p, st);
  }
}

extern "C" int mase_mxint_clip_candidates(const void* in, void* cand, size_t numel, int dtype, int block_size,
                                          int element_bits, int scale_bits, const uint32_t* log2_tab, void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (int rc = clip_args(in, in, cand, numel, dtype, block_size, log2_tab)) return rc;
  if (element_bits < 2 || element_bits > 24 || scale_bits < 1 || scale_bits > 8) return MASE_ERR_PARAM;
  const MxintParams p = make_mxint_params(element_bits, scale_bits, dtype, log2_tab);
  const size_t n_blocks = numel / (size_t)block_size;
  hipStream_t st = (hipStream_t)stream;
  switch (block_size) {
    case 16: return clip_mxint_candidates_b16(dtype, in, cand, n_blocks, p, st);
    case 32: return clip_mxint_candidates_b32(dtype, in, cand, n_blocks, p, st);
    default: return clip_mxint_candidates_b64(dtype, in, cand, n_blocks, p, st);
  }
}

extern "C" int mase_mxfp_clip_candidates(const void* in, void* cand, void* score, size_t numel, int dtype,
                                         int block_size, int exp_bits, int frac_bits, const uint32_t* log2_tab,
                                         void* stream) {
  using namespace mase;
  if (numel == 0) return MASE_OK;
  if (score == nullptr) return MASE_ERR_NULL;
  if (int rc = clip_args(in, in, cand, numel, dtype, block_size, log2_tab)) return rc;
  if (!aligned16(score)) return MASE_ERR_ALIGN;
  MxfpParams p;
  if (!make_mxfp_params(exp_bits, frac_bits, log2_tab, p)) return MASE_ERR_PARAM;
  const size_t n_blocks = numel / (size_t)block_size;
  hipStream_t st = (hipStream_t)stream;
  switch (block_size) {
    case 16: return clip_mxfp_candidates_b16(dtype, in, cand, score, n_blocks, p, st);
    case 32: return clip_mxfp_candidates_b32(dtype, in, cand, score, n_blocks, p, st);
    default: return clip_mxfp_candidates_b64(dtype, in, cand, score, n_blocks, p, st);
  }
}
