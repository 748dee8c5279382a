// The MXINT clip-search kernels for blocks of 16: one translation unit per family and block size, see
// clip_search_kernels.hpp.
#include "clip_search_kernels.hpp"

namespace mase {
MASE_CLIP_DEFINE_MXINT(16)
}  // namespace mase
