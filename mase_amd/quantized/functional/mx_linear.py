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

from ..._gemm import (MXFP_HW_FORMATS, MXFP_K_MULTIPLE, SKINNY_MAX_ROWS, gemm_bf16_pack_b, gemm_bf16_packed_b_supported,
                      gemm_bf16_takes_packed_b, gemm_bf16_tn, gemm_mxfp4_scaled_tiled, gemm_mxfp4_skinny, gemm_mxfp4_skinny_supported,
                      gemm_mxfp4_tiled_supported, mxfp_pack_tiled, mxfp_tile_codes,
                      gemm_mxfp_scaled, gemm_mxint8_pack_b, gemm_mxint8_packed_supported, gemm_mxint8_skinny,
                      gemm_mxint8_skinny_supported, gemm_mxint8_tn_packed, mxfp_pack)


class WeightCache:
    """bf16 image of a module's (already MX-quantized) weight, rebuilt when the parameter changes.

    The image is used only if it is *exact* (``w.to(bf16)`` round-trips); a weight that is not on an MX grid
    (e.g. assigned after ``load_state_dict``, or ``gptq=True``) makes the forward take the plain library GEMM
    in the weight's own dtype instead, which is what the reference computes in that situation.

    Changes are detected through the parameter's storage pointer, shape, dtype, device and version counter
    (``load_state_dict``, ``.to()``, ``weight.copy_()``, ``weight.data = ...`` all change one of them).  An in-place
    edit made through ``weight.data`` bypasses the version counter: call ``invalidate()`` after such an edit.
    A parameter that is an inference tensor (created under ``torch.inference_mode()``) has no version counter: its
    image is rebuilt on every call rather than trusted.
    """

    def __init__(self):
        self._key = None
        self._w = None
        self._packed = None

    def invalidate(self):
        self._key = None
        self._w = None
        self._packed = None

    def get(self, weight: Tensor):
        key = _tensor_key(weight)
        if key is None or key != self._key:
            w = weight.detach()
            if w.dtype == torch.bfloat16:
                wb = w.contiguous()
            else:
                wb = w.to(torch.bfloat16).contiguous()
                if not torch.equal(wb.to(w.dtype), w):
                    wb = None
            self._key, self._w, self._packed = key, wb, None
        return self._w

    def packed(self):
        """The fragment-ordered copy of the image returned by the last ``get`` (for ``gemm_bf16_tn(b_packed=...)``),
        built on first use: another 2 bytes per weight, spent only by modules that see batches large enough for the
        tiled kernel.  None while a HIP graph is being captured and the copy does not exist yet (it must not be
        allocated from the graph's pool)."""
        if self._packed is None and self._w is not None and gemm_bf16_packed_b_supported(*self._w.shape):
            if torch.cuda.is_current_stream_capturing():
                return None
            self._packed = gemm_bf16_pack_b(self._w)
        return self._packed


def _tensor_key(t: Tensor):
    """identity of a parameter as far as it can be observed without reading it: storage pointer, version counter,
    dtype, device, shape; None for an inference tensor (it has no version counter, so changes cannot be seen and
    nothing derived from it is kept)"""
    if t.is_inference():
        return None
    return (t.data_ptr(), t._version, t.dtype, t.device, tuple(t.shape))


def mx_linear(x: Tensor, weight: Tensor, bias: Tensor | None, quantize_to_bf16, quantize_same_dtype,
              cache: WeightCache, xq: Tensor | None = None) -> Tensor:
    """``F.linear(q(x), weight, bias)``.  ``quantize_to_bf16(x2d)`` returns q(x) as bf16 (exact);
    ``quantize_same_dtype(x)`` returns q(x) in x's dtype (used when the weight has no exact bf16 image).
    ``xq``: q(x) as a bf16 matrix when the caller already has it (sibling projections of one tensor, see
    ``project_shared``)."""
    wb = cache.get(weight) if x.is_cuda and weight.dim() == 2 else None
    if wb is None or x.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        return F.linear(quantize_same_dtype(x), weight, bias)
    lead = x.shape[:-1]
    if xq is None:
        xq = quantize_to_bf16(x.reshape(-1, x.shape[-1]))
    wp = cache.packed() if gemm_bf16_takes_packed_b(xq.shape[0], wb.shape[0], wb.shape[1]) else None
    y = gemm_bf16_tn(xq, wb, bias, x.dtype, b_packed=wp)
    return y.reshape(*lead, weight.shape[0])


def project_shared(x: Tensor, modules) -> list:
    """``[m(x) for m in modules]`` for sibling projections of one tensor (query / key / value, gate / up): modules
    that quantize ``x`` the same way (``activation_key``) receive one quantized copy instead of making their own.
    The copy lives for the duration of this call only; nothing is remembered between calls."""
    outs, key, prepared = [], None, None
    for m in modules:
        k = m.activation_key(x) if hasattr(m, "activation_key") else None
        if k is None:
            outs.append(m(x))
            continue
        if prepared is None or k != key:
            key, prepared = k, m.prepare_activation(x)
        outs.append(m(x, prepared=prepared))
    return outs


def shared_mxint_width(x: Tensor, modules) -> int | None:
    """The element width when every module would turn the bf16 tensor ``x`` into the same MXINT form with blocks of 32
    on its way to the matrix cores (``activation_key``), else None.  A producer of ``x`` that can quantize what it
    writes (``rmsnorm_mxint``, ``silu_mul_mxint``) then hands the modules that form directly:
    ``m(xq, prepared=xq.reshape(-1, K))``: with ``prepared`` given, a module reads only the shape and dtype of its
    first argument."""
    if x.dtype != torch.bfloat16 or not modules:
        return None
    keys = {m.activation_key(x) if hasattr(m, "activation_key") else None for m in modules}
    if len(keys) != 1:
        return None
    key = keys.pop()
    if key is None or key[0] != "mxint" or key[1] != 32:
        return None
    return key[2]


def _weight_key(weight: Tensor):
    return _tensor_key(weight)


class PackedMXFPWeight:
    """Hardware image (element codes + E8M0 block scales) of an MXFP-quantized weight for the block-scaled
    matrix instruction.

    It is packed from the *unquantized* weight when a state dict is loaded (packing the quantized weight again
    could pick a different block scale) and is valid only while the parameter is the tensor that load produced:
    the same identity/version test as ``WeightCache``.  The packed values equal the reference's quantized
    weight except in blocks whose largest element takes the format's top code, which the hardware reserves
    for NaN/Inf (e4m3 0x7F, e5m2 exponent 31): those blocks are stored with the next scale and halved codes,
    which only rounds elements more than 2^9 below the block maximum.  e2m1 has no reserved code and is exact.
    """

    def __init__(self):
        self._key = None
        self.codes = None
        self.scales = None
        self.fmt = None
        self._tiled = None

    def invalidate(self):
        self._key = None
        self.codes = self.scales = self.fmt = self._tiled = None

    def tiled(self, K: int):
        """The e2m1 codes as the tile image the tiled GEMM copies from (``mxfp_tile_codes``), made on the first forward
        that takes that kernel: another 0.5 bytes per weight.  None while a HIP graph is being captured before the
        image exists (it must not come from the graph's memory pool)."""
        if self._tiled is not None and self._tiled[0] is self.codes:
            return self._tiled[1]
        if self.codes is None or torch.cuda.is_current_stream_capturing():
            return None
        self._tiled = (self.codes, mxfp_tile_codes(self.codes, K, 4))
        return self._tiled[1]

    @staticmethod
    def eligible(weight: Tensor, block_size: int, fmt) -> bool:
        return (weight.is_cuda and weight.dim() == 2 and block_size == 32 and tuple(fmt) in MXFP_HW_FORMATS
                and weight.shape[1] % MXFP_K_MULTIPLE == 0
                and weight.dtype in (torch.float32, torch.bfloat16, torch.float16))

    def pack(self, weight: Tensor, fmt):
        self.codes, self.scales = mxfp_pack(weight.detach(), *fmt)
        self.fmt = tuple(fmt)

    def bind(self, weight: Tensor):
        """declare the image current for ``weight`` as it is now (after its in-place quantization)"""
        self._key = _weight_key(weight)

    def from_reference_codes(self, codes: Tensor, scales: Tensor, fmt) -> bool:
        """Build the image from the quantizer's own element codes (one ``sign|exp|frac`` byte per element) and scale
        bytes, e.g. those of a packed checkpoint.  The bit fields are the hardware's; e2m1 codes are put two to a
        byte.  Returns False (no image) when a block uses a code the hardware format reserves."""
        fmt = tuple(fmt)
        codes = codes.contiguous()
        if fmt == (2, 1):
            hw = (codes[..., 0::2] & 0xF) | (codes[..., 1::2] << 4)
        else:
            reserved = ((codes & 0x7F) == 0x7F) if fmt == (4, 3) else (((codes >> 2) & 0x1F) == 0x1F)
            if bool(reserved.any()):
                return False
            hw = codes
        self.codes, self.scales, self.fmt = hw.contiguous(), scales.contiguous(), fmt
        return True

    def decodes_to(self, weight: Tensor) -> bool:
        """whether the image holds exactly the values of ``weight``"""
        from ...quantizers._ops import mx_unpack

        codes = self.codes
        if self.fmt == (2, 1):  # two codes per byte, even element in the low nibble
            codes = torch.stack((codes & 0xF, codes >> 4), dim=-1).reshape(*codes.shape[:-1], -1)
        got = mx_unpack(codes, self.scales, 32, weight.dtype, "mxfp", *self.fmt).view(weight.shape)
        return bool(torch.equal(got, weight))

    def valid_for(self, weight: Tensor) -> bool:
        return self.codes is not None and self._key is not None and self._key == _weight_key(weight)


class PackedMXIntWeight:
    """MXINT8 codes (int8 [N, K]) and scale bytes (uint8 [N, K/32]) of a quantized weight, kept next to the parameter for
    the weight-streaming product of decode-sized batches (half the bytes of the bf16 image).  Valid only while the
    parameter is the tensor the codes were made for (identity / version test, as ``WeightCache``)."""

    def __init__(self):
        self._key = None
        self.codes = None
        self.scales = None

    def invalidate(self):
        self._key = None
        self.codes = self.scales = None

    @staticmethod
    def eligible(weight: Tensor, block_size: int, element_bits: int) -> bool:
        return (weight.is_cuda and weight.dim() == 2 and block_size == 32 and element_bits == 8
                and weight.shape[1] % 128 == 0 and weight.shape[0] * weight.shape[1] < (1 << 32)
                and weight.dtype in (torch.float32, torch.bfloat16, torch.float16))

    def set(self, codes: Tensor, scales: Tensor, weight: Tensor):
        n, k = weight.shape
        self.codes, self.scales = codes.reshape(n, k).contiguous(), scales.reshape(n, k // 32).contiguous()
        self._key = _weight_key(weight)

    def decodes_to(self, weight: Tensor) -> bool:
        from ...quantizers._ops import mx_unpack

        got = mx_unpack(self.codes, self.scales, 32, weight.dtype, "mxint", 8).view(weight.shape)
        return bool(torch.equal(got, weight))

    def valid_for(self, weight: Tensor) -> bool:
        return self.codes is not None and self._key is not None and self._key == _weight_key(weight)


class MXIntCodeImage:
    """An MXINT8 weight as the fragment-ordered code and scale images of the tiled kernel that widens codes in
    registers (``gemm_mxint8_tn_packed``): 1.03 bytes per weight, in place of the bf16 image and its fragment-ordered
    copy (2 + 2 bytes per weight).  Valid only while the parameter is the tensor the codes were made for."""

    def __init__(self):
        self._key = None
        self.codes = self.scales = None
        self.n = 0

    def invalidate(self):
        self._key = None
        self.codes = self.scales = None

    @staticmethod
    def eligible(weight: Tensor, block_size: int, element_bits: int) -> bool:
        return (weight.is_cuda and weight.dim() == 2 and block_size == 32 and element_bits == 8
                and gemm_mxint8_packed_supported(weight.shape[0], weight.shape[1])
                and weight.dtype in (torch.float32, torch.bfloat16, torch.float16))

    def set(self, codes: Tensor, scales: Tensor, weight: Tensor) -> bool:
        """Build the images from row-major codes [N, K] and scale bytes [N, K/32].  False (nothing kept) when a block
        scale is below 2^-126: the kernel takes such weights as zero."""
        n, k = weight.shape
        scales = scales.reshape(n, k // 32)
        if bool((scales < 8).any()):
            self.invalidate()
            return False
        self.codes, self.scales = gemm_mxint8_pack_b(codes.reshape(n, k), scales)
        self.n = n
        self._key = _weight_key(weight)
        return True

    def valid_for(self, weight: Tensor) -> bool:
        return self.codes is not None and self._key is not None and self._key == _weight_key(weight)


def mxint_linear_codes(x: Tensor, image: MXIntCodeImage, bias: Tensor | None, quantize_to_bf16,
                       xq: Tensor | None = None) -> Tensor:
    """``F.linear(q(x), W, b)`` on the tiled kernel with W as MXINT8 code / scale images"""
    lead = x.shape[:-1]
    if xq is None:
        xq = quantize_to_bf16(x.reshape(-1, x.shape[-1]))
    y = gemm_mxint8_tn_packed(xq, image.codes, image.scales, image.n, bias, x.dtype)
    return y.reshape(*lead, image.n)


def mxint_codes_apply(x: Tensor, image: MXIntCodeImage, weight: Tensor) -> bool:
    rows = x.numel() // x.shape[-1] if x.numel() else 0
    return (x.is_cuda and rows > SKINNY_MAX_ROWS and x.dtype in (torch.float32, torch.bfloat16, torch.float16)
            and image.valid_for(weight) and not torch.is_grad_enabled())


def mxint_linear_decode(x: Tensor, packed: PackedMXIntWeight, bias: Tensor | None, quantize_to_bf16,
                        xq: Tensor | None = None) -> Tensor:
    """``F.linear(q(x), W, b)`` for at most 128 rows of activations with W as MXINT8 codes + scales"""
    lead = x.shape[:-1]
    if xq is None:
        xq = quantize_to_bf16(x.reshape(-1, x.shape[-1]))
    y = gemm_mxint8_skinny(xq, packed.codes, packed.scales, bias, x.dtype)
    return y.reshape(*lead, packed.codes.shape[0])


def mxint_decode_applies(x: Tensor, packed: PackedMXIntWeight, weight: Tensor) -> bool:
    rows = x.numel() // x.shape[-1] if x.numel() else 0
    return (x.is_cuda and 0 < rows <= SKINNY_MAX_ROWS and x.dtype in (torch.float32, torch.bfloat16, torch.float16)
            and packed.valid_for(weight) and gemm_mxint8_skinny_supported(rows, weight.shape[0], weight.shape[1])
            and not torch.is_grad_enabled())


def mxfp_native_layout(x: Tensor, packed: PackedMXFPWeight, act_fmt) -> str:
    """which form of the packed activations the block-scaled contraction of ``x`` with this weight takes: "tiled"
    (tile image, for the tiled kernel) or "rows" (row-major codes: the weight-streaming kernel of few rows and the
    row-major tiled kernel)"""
    M, K = (x.numel() // x.shape[-1] if x.numel() else 0), x.shape[-1]
    N = packed.scales.shape[0]
    if (not gemm_mxfp4_skinny_supported(M, N, K, packed.fmt) and gemm_mxfp4_tiled_supported(M, N, K, act_fmt, packed.fmt)
            and packed.tiled(K) is not None):
        return "tiled"
    return "rows"


def mxfp_native_pack(x: Tensor, act_fmt, layout: str):
    """(codes, scales) of the activations in the given layout: one pass over x, 1.03 bytes written per element"""
    x2 = x.reshape(-1, x.shape[-1])
    return mxfp_pack_tiled(x2, *act_fmt) if layout == "tiled" else mxfp_pack(x2, *act_fmt)


def mxfp_linear_native(x: Tensor, packed: PackedMXFPWeight, bias: Tensor | None, act_fmt, prepared=None) -> Tensor:
    """``F.linear(q(x), W, b)`` on the block-scaled matrix instruction: the activations are quantized straight to
    element codes + scales and contracted with the packed weight; accumulation is fp32 and the result is written in
    x's dtype.  ``prepared``: ``mxfp_native_pack(x, act_fmt, mxfp_native_layout(...))`` when the caller has it."""
    lead = x.shape[:-1]
    M, K = x.numel() // x.shape[-1], x.shape[-1]
    N = packed.scales.shape[0]
    layout = mxfp_native_layout(x, packed, act_fmt)
    xc, xs = prepared if prepared is not None else mxfp_native_pack(x, act_fmt, layout)
    if layout == "tiled":
        # both code matrices as tile images (the activations' written directly by the quantizer): same bits, 7 % faster
        y = gemm_mxfp4_scaled_tiled(xc, xs, act_fmt, packed.tiled(K), packed.scales, bias, x.dtype)
    elif gemm_mxfp4_skinny_supported(M, N, K, packed.fmt):
        # decode-sized batch with MXFP4 weights: bound by streaming the weight codes once (0.53 bytes per weight)
        y = gemm_mxfp4_skinny(xc, xs, act_fmt, packed.codes, packed.scales, bias, x.dtype)
    else:
        y = gemm_mxfp_scaled(xc, xs, act_fmt, packed.codes, packed.scales, packed.fmt, bias, x.dtype)
    return y.reshape(*lead, N)
