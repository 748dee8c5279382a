// Host-only parts of the C ABI: version, error strings, scalar conversions shared by the launchers.
#include "common.hpp"

#include <cmath>
#include <cstring>

namespace {

float host_round_bf16(float f) {
  uint32_t b;
  std::memcpy(&b, &f, 4);
  if ((b & 0x7FFFFFFFu) > 0x7F800000u) return f;
  b = (b + 0x7FFFu + ((b >> 16) & 1u)) & 0xFFFF0000u;
  std::memcpy(&f, &b, 4);
  return f;
}

float host_round_f16(float f) { return (float)(_Float16)f; }

}  // namespace

extern "C" int mase_abi_version(void) { return 1; }

extern "C" const char* mase_error_string(int code) {
  switch (code) {
    case MASE_OK: return "ok";
    case MASE_ERR_NULL: return "a required pointer is NULL";
    case MASE_ERR_SHAPE: return "inconsistent sizes (numel not divisible by the block size, zero dimension, ...)";
    case MASE_ERR_ALIGN: return "pointer not aligned as required";
    case MASE_ERR_DTYPE: return "unknown dtype code";
    case MASE_ERR_PARAM: return "format parameter outside the supported domain";
    case MASE_ERR_LAUNCH: return "HIP runtime rejected the kernel launch";
    case MASE_ERR_WORKSPACE: return "workspace missing or too small";
    default: return "unknown error code";
  }
}

// A Python scalar used as a clamp bound is first converted to the tensor dtype (round to nearest even).
extern "C" float mase_round_scalar_to_dtype(double v, int dtype) {
  float f = (float)v;
  if (dtype == MASE_DT_BF16) return host_round_bf16(f);
  if (dtype == MASE_DT_F16) return host_round_f16(f);
  return f;
}

// isclose(x, 0) with default tolerances is |x| <= atol evaluated in the tensor dtype, atol = 1e-8.
extern "C" uint32_t mase_isclose_zero_threshold_bits(int dtype) {
  float t = mase_round_scalar_to_dtype(1e-8, dtype);
  uint32_t b;
  std::memcpy(&b, &t, 4);
  return b;
}
