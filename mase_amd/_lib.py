"""ctypes binding of ``libmase_amd.so`` (the C ABI declared in ``include/mase_amd.h``).

The library is the only compute path of this package: if it is missing, or a call fails, an exception is
raised.  There is no fallback to framework ops.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_double, c_float, c_int, c_size_t, c_uint32, c_void_p

import torch

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libmase_amd.so")

DT_F32, DT_BF16, DT_F16 = 0, 1, 2
DTYPE_CODE = {torch.float32: DT_F32, torch.bfloat16: DT_BF16, torch.float16: DT_F16}
LOG2_TABLE_WORDS = 576
BLOCK_FP_STATIC_MAX_TILES = 1 << 20


class MaseAmdError(RuntimeError):
    pass


# name -> (restype, argtypes); one entry per symbol declared in include/mase_amd.h
SIGNATURES = {
    "mase_abi_version": (c_int, []),
    "mase_error_string": (c_char_p, [c_int]),
    "mase_mxint_qdq": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mase_block_fp_workspace_bytes": (c_size_t, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int]),
    "mase_block_fp_qdq": (c_int, [c_void_p, c_void_p, c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_size_t, c_void_p]),
    "mase_block_fp_qdq_static": (c_int, [c_void_p, c_void_p, c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mase_integer_qdq": (c_int, [c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "mase_minifloat_qdq": (c_int, [c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mase_minifloat_mx_qdq": (c_int, [c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "mase_mxfp_qdq": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mase_gemm_bf16_tn": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_size_t, c_int, c_int, c_void_p]),
    "mase_transpose16": (c_int, [c_void_p, c_void_p] + [c_size_t] * 8 + [c_void_p]),
    "mase_gemm_bf16_tn_batched": (c_int, [c_void_p, c_void_p, c_void_p] + [c_size_t] * 14 + [c_int, c_void_p]),
    "mase_gemm_bf16_tn_splitk_workspace_bytes": (c_size_t, [c_size_t, c_size_t, c_size_t]),
    "mase_gemm_bf16_tn_splitk": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_size_t, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "mase_gemm_bf16_skinny_workspace_bytes": (c_size_t, [c_size_t, c_size_t, c_size_t]),
    "mase_gemm_bf16_skinny": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_size_t, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "mase_attn_softmax_mx": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_size_t, c_size_t, c_size_t, c_int,
                                     ctypes.c_float, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                                     c_void_p]),
    "mase_rope": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_size_t, c_size_t, c_size_t, c_size_t,
                          c_size_t, c_size_t, c_size_t, c_int, c_void_p]),
    "mase_rmsnorm_minifloat": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_int, c_float, c_int, c_int, c_int,
                                       c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "mase_silu_mul_minifloat": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "mase_attention_causal": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p] + [c_size_t] * 16 + [c_int, c_float, c_void_p]),
    "mase_attention_causal_fused": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p] + [c_size_t] * 16 + [c_int, c_float, c_void_p, c_void_p,
                                            c_size_t, c_size_t, c_int, c_void_p, c_void_p]),
    "mase_rmsnorm_mxint": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_int, c_float, c_int, c_void_p, c_void_p]),
    "mase_add_rmsnorm_mxint": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_int, c_float, c_int,
                                      c_void_p, c_void_p]),
    "mase_silu_mul_mxint": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int, c_void_p, c_void_p]),
    "mase_silu_table": (c_int, [c_void_p, c_int, c_void_p]),
    "mase_silu_mul_mxint_lut": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "mase_mxint_clip_search": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mase_mxfp_clip_search": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mase_mxint_clip_candidates": (c_int, [c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mase_mxfp_clip_candidates": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mase_gemm_bf16_packed_bytes": (c_size_t, [c_size_t, c_size_t]),
    "mase_gemm_bf16_pack_b": (c_int, [c_void_p, c_void_p, c_size_t, c_size_t, c_void_p]),
    "mase_gemm_bf16_tn_packed": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_size_t, c_int, c_int, c_void_p]),
    "mase_gemm_mxint8_packed_code_bytes": (c_size_t, [c_size_t, c_size_t]),
    "mase_gemm_mxint8_packed_scale_bytes": (c_size_t, [c_size_t, c_size_t]),
    "mase_gemm_mxint8_pack_b": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_void_p]),
    "mase_gemm_mxint8_tn_packed": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_size_t,
                                           c_int, c_int, c_void_p]),
    "mase_mx_unpack": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "mase_gemm_mxint8_skinny_workspace_bytes": (c_size_t, [c_size_t, c_size_t, c_size_t]),
    "mase_gemm_mxint8_skinny": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_size_t, c_int,
                                        c_int, c_void_p, c_size_t, c_void_p]),
    "mase_gemm_mxfp4_skinny_workspace_bytes": (c_size_t, [c_size_t, c_size_t, c_size_t]),
    "mase_gemm_mxfp4_skinny": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t,
                                       c_size_t, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "mase_mxfp_pack": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mase_mxfp_tiled_bytes": (c_size_t, [c_size_t, c_size_t, c_int]),
    "mase_mxfp_tile_codes": (c_int, [c_void_p, c_void_p, c_size_t, c_size_t, c_int, c_void_p]),
    "mase_mxfp_pack_tiled": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_int, c_int, c_int, c_void_p,
                                     c_void_p]),
    "mase_gemm_mxfp4_scaled_tiled": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                             c_size_t, c_size_t, c_int, c_int, c_void_p]),
    "mase_gemm_mxfp_scaled": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_size_t, c_size_t, c_size_t, c_int, c_int, c_void_p]),
    "mase_isclose_zero_threshold_bits": (c_uint32, [c_int]),
    "mase_round_scalar_to_dtype": (c_float, [c_double, c_int]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Loads the shared library (once).  Raises MaseAmdError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MaseAmdError(
            f"{LIB_PATH} not found: build it with `python -m mase_amd.build` (hipcc, gfx950). "
            "mase_amd has no CPU or framework fallback."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().mase_error_string(code).decode()
        raise MaseAmdError(f"{what} failed: {msg} (code {code})")


def dtype_code(t: torch.Tensor) -> int:
    try:
        return DTYPE_CODE[t.dtype]
    except KeyError:
        raise MaseAmdError(f"mase_amd kernels support float32, bfloat16 and float16 tensors, got {t.dtype}") from None


def require_device(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise MaseAmdError(
            f"{what}: expected a tensor on a ROCm device, got device '{t.device}'. "
            "mase_amd runs on MI355X only and has no CPU path."
        )


def stream_ptr(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream
