"""Packed checkpoints for MX-quantized Linear weights: element codes (one byte each) and one shared-exponent byte per
block instead of the dequantized fp tensor (8.25 bits per weight for blocks of 32, against 16 or 32).

The reference keeps quantized weights as dequantized floating point in its ``state_dict.pt`` / ``.mz`` checkpoints
(``chop/passes/graph/interface/save_and_load.py:118-148``) and re-runs the quantizer in ``load_state_dict``
(``nn/quantized/modules/linear.py:916-954``).  Here a checkpoint can hold what the quantizer's extract step produces
(``mxint/fake.py:11-56``, ``mxfp/fake.py:12-72``), and loading is the compose step (``mase_mx_unpack``): the loaded
``weight`` equals the quantized weight element for element and no quantizer runs.  MXFP codes carry a sign bit, so
the result is bit-identical; an MXINT code is a two's-complement integer, so a negative element that rounded to zero
(-0.0 in the quantized tensor) comes back as +0.0, every other element bit-identical.

File format: an ordinary ``torch.save`` of a flat ``{name: tensor}`` dict (loadable with ``weights_only=True``).  A
packed weight ``<prefix>.weight`` is replaced by ``<prefix>.weight.mx_codes`` (int8 / uint8, shape of the weight),
``<prefix>.weight.mx_scales`` (uint8, ``[out_features, in_features / block]``) and ``<prefix>.weight.mx_meta``
(int64: format version, kind 0 MXINT / 1 MXFP, block size, p0, p1, dtype code of the weight).  Everything else is
stored as in ``state_dict()``.  A weight is packed only if unpacking the codes reproduces the module's weight
(checked when the checkpoint is written); otherwise it is stored as it is.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch
from torch import Tensor

from .. import _lib
from ..quantizers import _ops
from .modules.linear import LinearMXFP, LinearMXInt

PACKED_FORMAT_VERSION = 1
_DTYPES = {v: k for k, v in _lib.DTYPE_CODE.items()}


def _weight_format(module):
    """(kind, block_size, p0, p1) of a module's weight quantizer, or None when the module does not quantize"""
    if not isinstance(module, (LinearMXInt, LinearMXFP)) or module.bypass or module.gptq:
        return None
    cfg = module.config
    if isinstance(module, LinearMXInt):
        return ("mxint", cfg["weight_block_size"], cfg["weight_width"], 0)
    if isinstance(module, LinearMXFP):
        return ("mxfp", cfg["weight_block_size"], cfg["weight_exponent_width"], cfg["weight_frac_width"])
    return None


def pack_weight(weight: Tensor, kind: str, block_size: int, p0: int, p1: int = 0):
    """Quantize ``weight`` ([out, in], blocks along ``in``) and return ``(dequantized, codes, scales)`` with codes and
    scales shaped ``[out, in]`` and ``[out, in / block_size]``."""
    if kind == "mxint":
        if p0 > 8:
            raise ValueError("packed MXINT codes are one byte: element width must be at most 8")
        deq, codes, scales = _ops.mxint_qdq(weight, block_size, p0, 1, 8, pack=True)
    else:
        deq, codes, scales = _ops.mxfp_qdq(weight, block_size, p0, p1, 1, 8, pack=True)
    return deq, codes.view(weight.shape), scales.view(weight.shape[0], -1)


def unpack_weight(codes: Tensor, scales: Tensor, kind: str, block_size: int, p0: int, p1: int, dtype: torch.dtype) -> Tensor:
    return _ops.mx_unpack(codes, scales, block_size, dtype, kind, p0, p1).view(codes.shape)


def _same_values(a: Tensor, b: Tensor) -> bool:
    return a.dtype == b.dtype and a.shape == b.shape and bool(torch.equal(a, b))


def packed_state_dict(model: torch.nn.Module, float_state_dict: Optional[Dict[str, Tensor]] = None) -> Dict[str, Tensor]:
    """``model.state_dict()`` with the weights of its MX Linear modules packed.

    The codes of a weight come from quantizing ``float_state_dict[<prefix>.weight]`` (the weights the model was
    quantized from) when given, else from quantizing the module's weight again; either way they are kept only if they
    unpack to exactly the module's weight (re-quantizing an MXINT weight moves a block whose largest code is +64 to a
    finer scale where it saturates, so without the original weights some tensors stay unpacked)."""
    sd = dict(model.state_dict())
    for name, module in model.named_modules():
        fmt = _weight_format(module)
        key = f"{name}.weight" if name else "weight"
        if fmt is None or key not in sd or not sd[key].is_cuda:
            continue
        kind, block, p0, p1 = fmt
        w = sd[key]
        if w.dim() != 2 or w.shape[1] % block != 0 or (kind == "mxint" and p0 > 8) or w.dtype not in _lib.DTYPE_CODE:
            continue
        src = float_state_dict[key].to(device=w.device, dtype=w.dtype) if float_state_dict and key in float_state_dict else w
        _, codes, scales = pack_weight(src, kind, block, p0, p1)
        if not _same_values(unpack_weight(codes, scales, kind, block, p0, p1, w.dtype), w):
            continue
        del sd[key]
        sd[key + ".mx_codes"] = codes
        sd[key + ".mx_scales"] = scales
        sd[key + ".mx_meta"] = torch.tensor([PACKED_FORMAT_VERSION, 0 if kind == "mxint" else 1, block, p0, p1,
                                             _lib.DTYPE_CODE[w.dtype]], dtype=torch.int64)
    return sd


def unpacked_state_dict(packed: Dict[str, Tensor], device=None) -> Dict[str, Tensor]:
    """the plain state dict a packed one stands for (weights dequantized on ``device``, default: where the codes are)"""
    out = {}
    for key, value in packed.items():
        if key.endswith(".mx_scales") or key.endswith(".mx_meta"):
            continue
        if not key.endswith(".mx_codes"):
            out[key] = value
            continue
        base = key[: -len(".mx_codes")]
        version, kind, block, p0, p1, dt = (int(v) for v in packed[base + ".mx_meta"].tolist())
        if version != PACKED_FORMAT_VERSION:
            raise ValueError(f"{base}: packed format version {version} is not supported")
        dev = device if device is not None else value.device
        out[base] = unpack_weight(value.to(dev), packed[base + ".mx_scales"].to(dev), "mxint" if kind == 0 else "mxfp",
                                  block, p0, p1, _DTYPES[dt])
    return out


def load_packed_state_dict(model: torch.nn.Module, packed: Dict[str, Tensor], strict: bool = True):
    """Load a packed state dict into a model whose MX Linear modules are already in place (e.g. after the quantize
    pass on an uninitialised model).  Parameters are copied as stored: no quantizer runs.  Returns what
    ``nn.Module.load_state_dict`` returns."""
    device = next((p.device for p in model.parameters()), None)
    result = torch.nn.Module.load_state_dict(model, unpacked_state_dict(packed, device), strict=strict)
    for name, module in model.named_modules():
        key = f"{name}.weight" if name else "weight"
        if isinstance(module, (LinearMXFP, LinearMXInt)) and key + ".mx_codes" in packed:
            module.weights_loaded_quantized(packed[key + ".mx_codes"], packed[key + ".mx_scales"])
        elif isinstance(module, (LinearMXInt, LinearMXFP)):
            module.weights_loaded_quantized()
    return result


def save_packed(model: torch.nn.Module, path: str, float_state_dict: Optional[Dict[str, Tensor]] = None) -> None:
    torch.save({k: v.cpu() for k, v in packed_state_dict(model, float_state_dict).items()}, path)


def load_packed(model: torch.nn.Module, path: str, strict: bool = True):
    return load_packed_state_dict(model, torch.load(path, map_location="cpu", weights_only=True), strict=strict)
