"""Fused forward of the MX-quantized Linear modules.

``LinearMXInt.forward`` / ``LinearMXFP.forward`` in the reference are ``F.linear(qdq(x), W, b)`` with W already
on the MX grid (``chop/nn/quantized/modules/linear.py:956-972, 877-895``).  Here the activation quantizer writes
its result directly as bf16 (MX values are exact in bf16) and the contraction runs on the matrix cores with
fp32 accumulation, so the real-number dot products are those of the reference; only the summation order differs.
"""
from __future__ import annotations

import torch
from torch import Tensor
from torch.nn import functional as F

from ..._gemm import gemm_bf16_tn


class WeightCache:
    """bf16 image of a module's (already MX-quantized) weight, rebuilt when the parameter changes.

    The image is used only if it is *exact* (``w.to(bf16)`` round-trips); a weight that is not on an MX grid
    (e.g. assigned after ``load_state_dict``, or ``gptq=True``) makes the forward take the plain library GEMM
    in the weight's own dtype instead, which is what the reference computes in that situation.

    Changes are detected through the parameter's storage pointer, shape, dtype, device and version counter
    (``load_state_dict``, ``.to()``, ``weight.copy_()``, ``weight.data = ...`` all change one of them).  An in-place
    edit made through ``weight.data`` bypasses the version counter: call ``invalidate()`` after such an edit.
    """

    def __init__(self):
        self._key = None
        self._w = None

    def invalidate(self):
        self._key = None
        self._w = None

    def get(self, weight: Tensor):
        key = (weight.data_ptr(), weight._version, weight.dtype, weight.device, tuple(weight.shape))
        if key != self._key:
            w = weight.detach()
            if w.dtype == torch.bfloat16:
                wb = w.contiguous()
            else:
                wb = w.to(torch.bfloat16).contiguous()
                if not torch.equal(wb.to(w.dtype), w):
                    wb = None
            self._key, self._w = key, wb
        return self._w


def mx_linear(x: Tensor, weight: Tensor, bias: Tensor | None, quantize_to_bf16, quantize_same_dtype,
              cache: WeightCache) -> Tensor:
    """``F.linear(q(x), weight, bias)``.  ``quantize_to_bf16(x2d)`` returns q(x) as bf16 (exact);
    ``quantize_same_dtype(x)`` returns q(x) in x's dtype (used when the weight has no exact bf16 image)."""
    wb = cache.get(weight) if x.is_cuda and weight.dim() == 2 else None
    if wb is None or x.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        return F.linear(quantize_same_dtype(x), weight, bias)
    lead = x.shape[:-1]
    x2 = x.reshape(-1, x.shape[-1])
    xq = quantize_to_bf16(x2)
    y = gemm_bf16_tn(xq, wb, bias, x.dtype)
    return y.reshape(*lead, weight.shape[0])
