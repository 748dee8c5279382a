"""Host wrappers of the matrix-core contractions."""
from __future__ import annotations

import torch
from torch import Tensor

from . import _lib

GEMM_K_MULTIPLE = 64  # K tile of mase_gemm_bf16_tn


def gemm_bf16_tn(a: Tensor, b: Tensor, bias: Tensor | None, out_dtype: torch.dtype) -> Tensor:
    """``a[M,K] @ b[N,K].T + bias`` with bf16 operands and fp32 accumulation; result in ``out_dtype``."""
    _lib.require_device(a, "gemm_bf16_tn")
    lib = _lib.load()
    assert a.dtype == torch.bfloat16 and b.dtype == torch.bfloat16
    assert a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[1]
    if a.shape[1] % GEMM_K_MULTIPLE:
        # the kernel consumes K in whole tiles; zero columns do not change the product
        pad = GEMM_K_MULTIPLE - a.shape[1] % GEMM_K_MULTIPLE
        a = torch.nn.functional.pad(a, (0, pad))
        b = torch.nn.functional.pad(b, (0, pad))
    a = a.contiguous()
    b = b.contiguous()
    M, K = a.shape
    N = b.shape[0]
    out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    if bias is not None:
        bias = bias.contiguous()
    rc = lib.mase_gemm_bf16_tn(
        a.data_ptr(), b.data_ptr(), bias.data_ptr() if bias is not None else None, out.data_ptr(), M, N, K,
        _lib.DTYPE_CODE[out_dtype], _lib.DTYPE_CODE[bias.dtype] if bias is not None else 0, _lib.stream_ptr(a),
    )
    _lib.check(rc, "mase_gemm_bf16_tn")
    return out
