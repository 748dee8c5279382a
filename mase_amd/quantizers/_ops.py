"""Host side of the quantize-dequantize functions: argument handling, layout, launches through the C ABI.

Mirrors the public functions of the reference's ``chop.nn.quantizers`` (same names, argument meaning,
defaults and error behaviour); the arithmetic itself lives in ``mase_amd/csrc``.
"""
from __future__ import annotations

from math import ceil
from typing import List, Sequence

import torch
from torch import Tensor

from .. import _lib
from .._tables import log2_table


# ------------------------------------------------------------------------------------------------
# Launch state bound once per (entry point, tensor dtype, device): the foreign function, the dtype code and the
# address of the log2 table.  A 20 us kernel is launch-bound unless the host side of a call stays well below that, so
# the common case (a contiguous, 16-byte aligned tensor on the device) skips every lookup that cannot change.
# ------------------------------------------------------------------------------------------------
_launch_state: dict = {}
_raw_stream = torch._C._cuda_getCurrentRawStream


def _state(name: str, dtype: torch.dtype, device: torch.device, tab_dtype=None):
    key = (name, dtype, device)
    st = _launch_state.get(key)
    if st is None:
        lib = _lib.load()
        code = _lib.DTYPE_CODE.get(dtype)
        if code is None:
            raise _lib.MaseAmdError(f"mase_amd kernels support float32, bfloat16 and float16 tensors, got {dtype}")
        tab = log2_table(tab_dtype or dtype, device)  # kept alive by the table cache
        st = _launch_state[key] = (getattr(lib, name), code, tab.data_ptr(), device.index)
    return st


def _fast_reset():
    _launch_state.clear()


def _contig(x: Tensor) -> Tensor:
    x = x.contiguous()
    if x.data_ptr() % 16 != 0:  # views with odd storage offsets: realign so the 16-byte path applies
        x = x.clone(memory_format=torch.contiguous_format)
    return x


# ------------------------------------------------------------------------------------------------
# layout helpers with the semantics of mxfp/helpers.py:8-63
# ------------------------------------------------------------------------------------------------
def _to_block_last_flat(x: Tensor, block_dim: int) -> Tensor:
    nd = x.dim()
    d = block_dim % nd
    if d == nd - 1:
        return _contig(x).view(-1)
    order = [i for i in range(nd) if i != d] + [d]
    return _contig(x.permute(order)).view(-1)


def _from_block_last_flat(flat: Tensor, shape: Sequence[int], block_dim: int) -> Tensor:
    nd = len(shape)
    d = block_dim % nd
    if d == nd - 1:
        return flat.view(shape)
    moved = [s for i, s in enumerate(shape) if i != d] + [shape[d]]
    back = list(range(nd - 1))
    back.insert(d, nd - 1)
    return flat.view(moved).permute(back)


# ------------------------------------------------------------------------------------------------
# MXINT  (reference: mxint/mxint.py:211-251)
# ------------------------------------------------------------------------------------------------
def mxint_qdq(x: Tensor, block_size: int, element_bits: int, block_dim: int, scale_bits: int, pack: bool = False,
              out_dtype: torch.dtype | None = None):
    """Returns the dequantized tensor (in ``out_dtype``, default the input dtype), or
    (dequantized, codes int8, scales uint8) when ``pack``."""
    if not pack and x.is_cuda and (block_dim == -1 or block_dim == x.dim() - 1) and x.is_contiguous():
        ptr = x.data_ptr()
        if not ptr & 15:
            n = x.numel()
            assert n % block_size == 0, f"Input tensor size {n} is not divisible by block size {block_size}."
            fn, code, tab, index = _state("mase_mxint_qdq", x.dtype, x.device)
            if out_dtype is None:
                out, ocode = torch.empty_like(x), code
            else:
                out, ocode = torch.empty_like(x, dtype=out_dtype), _lib.DTYPE_CODE[out_dtype]
            rc = fn(ptr, out.data_ptr(), None, None, n, code, ocode, block_size, element_bits, scale_bits, tab,
                    _raw_stream(index))
            if rc:
                _lib.check(rc, "mase_mxint_qdq")
            return out
    _lib.require_device(x, "mxint_quantizer")
    lib = _lib.load()
    shape = tuple(x.shape)
    nd = len(shape)
    assert block_dim < nd and block_dim >= -nd
    assert x.numel() % block_size == 0, f"Input tensor size {x.numel()} is not divisible by block size {block_size}."
    flat = _to_block_last_flat(x, block_dim)
    out = torch.empty_like(flat, dtype=out_dtype or x.dtype)
    codes = scales = None
    if pack:
        codes = torch.empty(flat.numel(), dtype=torch.int8, device=x.device)
        scales = torch.empty(flat.numel() // block_size, dtype=torch.uint8, device=x.device)
    tab = log2_table(x.dtype, x.device)
    rc = lib.mase_mxint_qdq(
        flat.data_ptr(), out.data_ptr(),
        codes.data_ptr() if pack else None, scales.data_ptr() if pack else None,
        flat.numel(), _lib.dtype_code(x), _lib.dtype_code(out), block_size, element_bits, scale_bits, tab.data_ptr(),
        _lib.stream_ptr(x),
    )
    _lib.check(rc, "mase_mxint_qdq")
    res = _from_block_last_flat(out, shape, block_dim)
    return (res, codes, scales) if pack else res


# ------------------------------------------------------------------------------------------------
# MXFP  (reference: mxfp/mxfp.py:187-230)
# ------------------------------------------------------------------------------------------------
_LEGAL_MXFP = ((4, 3), (5, 2), (2, 3), (3, 2), (2, 1), (1, 2))


def mxfp_qdq(x: Tensor, block_size: int, exp_bits: int, frac_bits: int, block_dim: int, scale_exp_bits: int,
             pack: bool = False, out_dtype: torch.dtype | None = None):
    _lib.require_device(x, "mxfp_quantizer")
    lib = _lib.load()
    assert scale_exp_bits in (8,), f"Invalid scale exponent bits: {scale_exp_bits}. Legal values are: (8,)."
    assert (exp_bits, frac_bits) in _LEGAL_MXFP, (
        f"Invalid element exp/frac bits: {(exp_bits, frac_bits)}. Legal values are: {_LEGAL_MXFP}."
    )
    shape = tuple(x.shape)
    nd = len(shape)
    assert block_dim < nd and block_dim >= -nd
    assert x.numel() % block_size == 0
    flat = _to_block_last_flat(x, block_dim)
    out = torch.empty_like(flat, dtype=out_dtype or x.dtype)
    codes = scales = None
    if pack:
        codes = torch.empty(flat.numel(), dtype=torch.uint8, device=x.device)
        scales = torch.empty(flat.numel() // block_size, dtype=torch.uint8, device=x.device)
    tab = log2_table(torch.float32, x.device)
    dt = _lib.dtype_code(x)
    rc = lib.mase_mxfp_qdq(
        flat.data_ptr(), out.data_ptr(),
        codes.data_ptr() if pack else None, scales.data_ptr() if pack else None,
        flat.numel(), dt, _lib.dtype_code(out), block_size, exp_bits, frac_bits, tab.data_ptr(), _lib.stream_ptr(x),
    )
    _lib.check(rc, "mase_mxfp_qdq")
    res = _from_block_last_flat(out, shape, block_dim)
    return (res, codes, scales) if pack else res


CLIP_SEARCH_BLOCKS = (16, 32, 64)


def _clip_search(name: str, x: Tensor, block_size: int, block_dim: int, tab_dtype, params, return_choice: bool):
    """the search branch of the MX quantizers without calibration activations: blocks along block_dim, the error
    measured against the blocks of the plain flattening (mxint/mxint.py:41-45, :97; mxfp/mxfp.py:41-45, :94-97)"""
    _lib.require_device(x, name)
    lib = _lib.load()
    if block_size not in CLIP_SEARCH_BLOCKS:
        raise NotImplementedError(f"{name}: quantile_search=True is built for block sizes {CLIP_SEARCH_BLOCKS}, got {block_size}")
    shape = tuple(x.shape)
    nd = len(shape)
    assert block_dim < nd and block_dim >= -nd
    assert x.numel() % block_size == 0, f"Input tensor size {x.numel()} is not divisible by block size {block_size}."
    ref = x.contiguous().view(-1)
    flat = _to_block_last_flat(x, block_dim)
    if ref.data_ptr() % 16:  # a view that starts inside an allocation: the kernel reads 16-byte vectors
        ref = ref.clone()
    if flat.data_ptr() % 16:
        flat = flat.clone()
    out = torch.empty_like(flat)
    choice = torch.empty(flat.numel() // block_size, dtype=torch.uint8, device=x.device) if return_choice else None
    tab = log2_table(tab_dtype, x.device)
    fn = getattr(lib, name)
    rc = fn(flat.data_ptr(), ref.data_ptr(), out.data_ptr(), choice.data_ptr() if return_choice else None, flat.numel(),
            _lib.dtype_code(x), block_size, *params, tab.data_ptr(), _lib.stream_ptr(x))
    _lib.check(rc, name)
    res = _from_block_last_flat(out, shape, block_dim)
    return (res, choice) if return_choice else res


def mxint_clip_search(x: Tensor, block_size: int, element_bits: int, block_dim: int, scale_bits: int,
                      return_choice: bool = False):
    return _clip_search("mase_mxint_clip_search", x, block_size, block_dim, x.dtype, (element_bits, scale_bits),
                        return_choice)


def mxfp_clip_search(x: Tensor, block_size: int, exp_bits: int, frac_bits: int, block_dim: int, scale_exp_bits: int,
                     return_choice: bool = False):
    assert scale_exp_bits in (8,), f"Invalid scale exponent bits: {scale_exp_bits}. Legal values are: (8,)."
    assert (exp_bits, frac_bits) in _LEGAL_MXFP, (
        f"Invalid element exp/frac bits: {(exp_bits, frac_bits)}. Legal values are: {_LEGAL_MXFP}."
    )
    return _clip_search("mase_mxfp_clip_search", x, block_size, block_dim, torch.float32, (exp_bits, frac_bits),
                        return_choice)


def _clip_candidates(name: str, x: Tensor, block_size: int, block_dim: int, tab_dtype, params, with_score: bool):
    """the eleven candidates of the search as [11, n_blocks, B] (blocks along block_dim), and for MXFP the values the
    reference scores (same shape)"""
    _lib.require_device(x, name)
    lib = _lib.load()
    if block_size not in CLIP_SEARCH_BLOCKS:
        raise NotImplementedError(f"{name}: quantile_search=True is built for block sizes {CLIP_SEARCH_BLOCKS}, got {block_size}")
    nd = x.dim()
    assert block_dim < nd and block_dim >= -nd
    assert x.numel() % block_size == 0, f"Input tensor size {x.numel()} is not divisible by block size {block_size}."
    flat = _to_block_last_flat(x, block_dim)
    if flat.data_ptr() % 16:
        flat = flat.clone()
    n = flat.numel()
    cand = torch.empty((11, n // block_size, block_size), dtype=x.dtype, device=x.device)
    score = torch.empty_like(cand) if with_score else None
    tab = log2_table(tab_dtype, x.device)
    fn = getattr(lib, name)
    args = [flat.data_ptr(), cand.data_ptr()] + ([score.data_ptr()] if with_score else [])
    rc = fn(*args, n, _lib.dtype_code(x), block_size, *params, tab.data_ptr(), _lib.stream_ptr(x))
    _lib.check(rc, name)
    return cand, score


def _calibration_view(act_tensor: Tensor, block_size: int) -> Tensor:
    """The reference contracts the calibration activations [batches, tokens, B] with blocks of B weights; an
    activation tensor whose last dimension is a multiple of B is viewed as [..., last/B, B] there and then fails in
    the contraction (mxint.py:101-104, :121; mxfp.py:67-72, :86), so only last dimension == B is a usable input."""
    if act_tensor.dim() != 3 or act_tensor.shape[-1] != block_size:
        raise ValueError(f"act_tensor must be [batches, tokens, {block_size}] (the block size), got {tuple(act_tensor.shape)}")
    return act_tensor


_CAL_CHUNK_ELEMS = 1 << 28  # elements of the [11, a, s, rows] product held at a time


def mxint_clip_search_calibrated(x: Tensor, block_size: int, element_bits: int, block_dim: int, scale_bits: int,
                                 act_tensor: Tensor, cali_batch_size: int = 32, return_choice: bool = False):
    """quantile_search=True with act_tensor (mxint/mxint.py:99-143): the candidate of each block of weights whose
    product with the calibration activations is closest to the unquantized block's, the distance being the sum over
    batches of ``cali_batch_size`` samples of the 2-norm over (sample, token).  The candidates come from
    ``mase_mxint_clip_candidates``; the products and norms are the reference's tensor operations on the device, done
    for groups of weight rows so that the [11, samples, tokens, rows] product stays bounded."""
    act = _calibration_view(act_tensor, block_size)
    shape = tuple(x.shape)
    cand, _ = _clip_candidates("mase_mxint_clip_candidates", x, block_size, block_dim, x.dtype,
                               (element_bits, scale_bits), False)
    rows = x.contiguous().flatten().reshape(-1, block_size)          # blocks of the plain flattening (mxint.py:41-45)
    H = rows.shape[0]
    err = torch.zeros((11, H), device=x.device, dtype=x.dtype)
    for b in range(0, act.shape[0], cali_batch_size):
        act_b = act[b:b + cali_batch_size]
        step = max(1, _CAL_CHUNK_ELEMS // max(1, 11 * act_b.shape[0] * act_b.shape[1]))
        for h0 in range(0, H, step):
            h1 = min(H, h0 + step)
            out_orig = torch.matmul(act_b, rows[h0:h1].T)
            out_q = torch.einsum("asb,phb->pash", act_b, cand[:, h0:h1].to(act.dtype))
            err[:, h0:h1] += torch.norm(out_q - out_orig, p=2, dim=(1, 2))
    pick = torch.argmin(err, dim=0)
    chosen = cand[pick, torch.arange(H, device=x.device)]
    out = _from_block_last_flat(chosen.reshape(-1), shape, block_dim).to(x.dtype)
    return (out, pick.to(torch.uint8)) if return_choice else out


def mxfp_clip_search_calibrated(x: Tensor, block_size: int, exp_bits: int, frac_bits: int, block_dim: int,
                                scale_exp_bits: int, act_tensor: Tensor, cali_batch_size: int = 32,
                                return_choice: bool = False):
    """quantile_search=True with act_tensor (mxfp/mxfp.py:40-115): per percentile the reference multiplies the
    activations with its score values (integer codes times the uint8 power, see ``mase_mxfp_clip_candidates``) and
    with the unquantized blocks, takes the 2-norm of the difference over (sample, token) summed over the batches, and
    replaces the incumbent on a strictly smaller error."""
    assert scale_exp_bits in (8,), f"Invalid scale exponent bits: {scale_exp_bits}. Legal values are: (8,)."
    assert (exp_bits, frac_bits) in _LEGAL_MXFP, (
        f"Invalid element exp/frac bits: {(exp_bits, frac_bits)}. Legal values are: {_LEGAL_MXFP}."
    )
    act = _calibration_view(act_tensor, block_size)
    shape = tuple(x.shape)
    cand, score = _clip_candidates("mase_mxfp_clip_candidates", x, block_size, block_dim, torch.float32,
                                   (exp_bits, frac_bits), True)
    rows = x.contiguous().flatten().reshape(-1, block_size)
    H = rows.shape[0]
    best = torch.full([H], float("inf"), device=x.device, dtype=x.dtype)
    pick = torch.zeros(H, dtype=torch.int64, device=x.device)
    for p in range(11):
        q = score[p].to(rows.dtype)
        err = torch.zeros(H, device=x.device, dtype=x.dtype)
        for b in range(0, act.shape[0], cali_batch_size):
            act_b = act[b:b + cali_batch_size]
            out_q = torch.matmul(act_b, q.T)
            out_orig = torch.matmul(act_b, rows.T)
            err += torch.norm(out_q - out_orig, p=2, dim=(0, 1))
        better = err < best
        best = torch.where(better, err, best)
        pick = torch.where(better, torch.full_like(pick, p), pick)
    chosen = cand[pick, torch.arange(H, device=x.device)]
    out = _from_block_last_flat(chosen.reshape(-1), shape, block_dim)
    return (out, pick.to(torch.uint8)) if return_choice else out


def _cast_args(cast):
    """(exp_bits, frac_bits, is_finite, round_mode code) of an optional minifloat cast; exp_bits 0 switches it off"""
    if cast is None:
        return 0, 0, 1, 0
    return int(cast[0]), int(cast[1]), int(bool(cast[2])), _ROUND_MODES[cast[3]]


RMSNORM_MAX_COLS = 8192


def rmsnorm_supported(x: Tensor, weight: Tensor) -> bool:
    return (x.is_cuda and x.dtype in _lib.DTYPE_CODE and weight.dtype == x.dtype and weight.device == x.device
            and weight.dim() == 1 and x.dim() >= 1 and x.shape[-1] == weight.shape[0] and x.shape[-1] % 8 == 0
            and x.shape[-1] <= RMSNORM_MAX_COLS and x.numel() > 0
            and not (torch.is_grad_enabled() and (x.requires_grad or weight.requires_grad)))


def rmsnorm_minifloat(x: Tensor, weight: Tensor, eps: float, x_cast=None, w_cast=None) -> Tensor:
    """``cast(weight) * (cast(x).float() * rsqrt(mean(square) + eps)).to(dtype)`` over the last dimension in one pass
    (``mase_rmsnorm_minifloat``); a cast is (exp_bits, frac_bits, is_finite, round_mode) or None."""
    _lib.require_device(x, "rmsnorm_minifloat")
    lib = _lib.load()
    assert rmsnorm_supported(x, weight)
    xc = _contig(x)
    w = weight.detach().contiguous()
    out = torch.empty_like(xc)
    cols = xc.shape[-1]
    rc = lib.mase_rmsnorm_minifloat(xc.data_ptr(), w.data_ptr(), out.data_ptr(), xc.numel() // cols, cols, _lib.dtype_code(xc),
                                    float(eps), *_cast_args(x_cast), *_cast_args(w_cast), _lib.stream_ptr(xc))
    _lib.check(rc, "mase_rmsnorm_minifloat")
    return out


def silu_mul_supported(gate: Tensor, up: Tensor) -> bool:
    return (gate.is_cuda and gate.dtype in _lib.DTYPE_CODE and up.dtype == gate.dtype and up.shape == gate.shape
            and up.device == gate.device and gate.numel() > 0 and gate.numel() % 8 == 0
            and not (torch.is_grad_enabled() and (gate.requires_grad or up.requires_grad)))


def silu_mul_minifloat(gate: Tensor, up: Tensor, cast=None) -> Tensor:
    """``silu(cast(gate)) * up`` in one pass (``mase_silu_mul_minifloat``)"""
    _lib.require_device(gate, "silu_mul_minifloat")
    lib = _lib.load()
    assert silu_mul_supported(gate, up)
    g, u = _contig(gate), _contig(up)
    out = torch.empty_like(g)
    rc = lib.mase_silu_mul_minifloat(g.data_ptr(), u.data_ptr(), out.data_ptr(), g.numel(), _lib.dtype_code(g),
                                     *_cast_args(cast), _lib.stream_ptr(g))
    _lib.check(rc, "mase_silu_mul_minifloat")
    return out


def rmsnorm_mxint(x: Tensor, weight: Tensor, eps: float, element_bits: int) -> Tensor:
    """``mxint_quantizer(rmsnorm(x), block 32 along the last dimension, element_bits)`` in one pass
    (``mase_rmsnorm_mxint``): the quantized activation the ``LinearMXInt`` modules after the norm would each compute
    from the stored norm output.  The last dimension must be a multiple of 32."""
    _lib.require_device(x, "rmsnorm_mxint")
    lib = _lib.load()
    assert rmsnorm_supported(x, weight) and x.shape[-1] % 32 == 0
    xc = _contig(x)
    w = weight.detach().contiguous()
    out = torch.empty_like(xc)
    cols = xc.shape[-1]
    rc = lib.mase_rmsnorm_mxint(xc.data_ptr(), w.data_ptr(), out.data_ptr(), xc.numel() // cols, cols, _lib.dtype_code(xc),
                                float(eps), int(element_bits), log2_table(xc.dtype, xc.device).data_ptr(),
                                _lib.stream_ptr(xc))
    _lib.check(rc, "mase_rmsnorm_mxint")
    return out


def add_rmsnorm_mxint(x: Tensor, residual: Tensor, weight: Tensor, eps: float, element_bits: int):
    """``s = x + residual`` and ``rmsnorm_mxint(s, weight, eps, element_bits)`` in one pass (``mase_add_rmsnorm_mxint``);
    returns ``(s, quantized norm)``.  Same shapes and dtype for ``x`` and ``residual``."""
    _lib.require_device(x, "add_rmsnorm_mxint")
    lib = _lib.load()
    assert rmsnorm_supported(x, weight) and x.shape[-1] % 32 == 0
    assert residual.shape == x.shape and residual.dtype == x.dtype and residual.device == x.device
    xc, rc_ = _contig(x), _contig(residual)
    w = weight.detach().contiguous()
    s, out = torch.empty_like(xc), torch.empty_like(xc)
    cols = xc.shape[-1]
    rc = lib.mase_add_rmsnorm_mxint(xc.data_ptr(), rc_.data_ptr(), w.data_ptr(), s.data_ptr(), out.data_ptr(),
                                    xc.numel() // cols, cols, _lib.dtype_code(xc), float(eps), int(element_bits),
                                    log2_table(xc.dtype, xc.device).data_ptr(), _lib.stream_ptr(xc))
    _lib.check(rc, "mase_add_rmsnorm_mxint")
    return s, out


SILU_TABLE_MIN_NUMEL = 1 << 23  # from here on the table form of silu * up pays for loading its 128 KB per CU
_silu_tables: dict = {}


def silu_table(dtype: torch.dtype, device: torch.device) -> Tensor:
    """R(silu(x)) for every 16-bit pattern x of ``dtype`` (bf16 / fp16), computed on the device by
    ``mase_silu_table`` with the expression the element-wise kernel evaluates; cached per dtype and device."""
    key = (dtype, str(device))
    if key not in _silu_tables:
        lib = _lib.load()
        tab = torch.empty(65536, dtype=torch.int16, device=device)
        _lib.check(lib.mase_silu_table(tab.data_ptr(), _lib.DTYPE_CODE[dtype], _lib.stream_ptr(tab)), "mase_silu_table")
        _silu_tables[key] = tab
    return _silu_tables[key]


def silu_mul_mxint(gate: Tensor, up: Tensor, element_bits: int, use_table: bool | None = None) -> Tensor:
    """``mxint_quantizer(silu(gate) * up, block 32 along the last dimension, element_bits)`` in one pass
    (``mase_silu_mul_mxint``); the last dimension must be a multiple of 32.  Large 16-bit tensors take the form that
    reads silu from a table (``mase_silu_mul_mxint_lut``, same bits); ``use_table`` forces either form."""
    _lib.require_device(gate, "silu_mul_mxint")
    lib = _lib.load()
    assert silu_mul_supported(gate, up) and gate.shape[-1] % 32 == 0
    g, u = _contig(gate), _contig(up)
    out = torch.empty_like(g)
    sixteen = g.dtype in (torch.bfloat16, torch.float16)
    if use_table is None:
        use_table = sixteen and g.numel() >= SILU_TABLE_MIN_NUMEL
    if use_table:
        assert sixteen, "the table form exists for 16-bit tensors"
        rc = lib.mase_silu_mul_mxint_lut(g.data_ptr(), u.data_ptr(), out.data_ptr(), g.numel(), _lib.dtype_code(g),
                                         int(element_bits), log2_table(g.dtype, g.device).data_ptr(),
                                         silu_table(g.dtype, g.device).data_ptr(), _lib.stream_ptr(g))
        _lib.check(rc, "mase_silu_mul_mxint_lut")
        return out
    rc = lib.mase_silu_mul_mxint(g.data_ptr(), u.data_ptr(), out.data_ptr(), g.numel(), _lib.dtype_code(g),
                                 int(element_bits), log2_table(g.dtype, g.device).data_ptr(), _lib.stream_ptr(g))
    _lib.check(rc, "mase_silu_mul_mxint")
    return out


def attention_causal_supported(q: Tensor, k: Tensor, v: Tensor) -> bool:
    """q, k, v [batch, heads, tokens, 128] bf16 on one device, last dimension contiguous, strides multiples of 8,
    tokens a multiple of 128, no gradient recorded"""
    if not (q.is_cuda and q.dim() == 4 and q.dtype == torch.bfloat16 and q.shape == k.shape == v.shape):
        return False
    if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
        return False
    B, H, T, D = q.shape
    if D != 128 or T == 0 or T % 128 != 0 or B * H == 0:
        return False
    for t in (q, k, v):
        if t.dtype != torch.bfloat16 or t.device != q.device or t.stride(3) != 1 or t.data_ptr() % 16:
            return False
        if any(s % 8 for s in t.stride()[:3]) or t.stride(2) < 128 or t.stride(2) * 2 * T > 0xFFFFFFFF:
            return False
    return True


def attention_causal(q: Tensor, k: Tensor, v: Tensor, scaling: float | None = None, mxint_bits: int | None = None,
                     q_rope: tuple[Tensor, Tensor] | None = None) -> Tensor:
    """``softmax(q k^T * scaling + causal mask) v`` for bf16 [batch, heads, tokens, 128] operands in one pass over the keys
    (``mase_attention_causal``).  Returned as [batch, heads, tokens, 128] over memory laid out [batch, tokens, heads,
    128], so that ``out.transpose(1, 2).reshape(batch, tokens, heads * 128)`` is a view.  ``mxint_bits``: the result is
    written as ``mxint_quantizer(result, block 32 along the head dimension, mxint_bits)``, the form a ``LinearMXInt``
    that reads it would compute itself.  ``q_rope = (cos, sin)``: ``q`` is given before its rotary embedding, which the
    kernel applies as it loads ``q`` (the values of ``rope(q, cos, sin)``; the tables must satisfy ``rope_supported``).
    Both through ``mase_attention_causal_fused``."""
    _lib.require_device(q, "attention_causal")
    lib = _lib.load()
    assert attention_causal_supported(q, k, v)
    B, H, T, D = q.shape
    if scaling is None:
        scaling = D ** -0.5
    out = torch.empty((B, T, H, D), dtype=q.dtype, device=q.device).transpose(1, 2)
    args = (q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), B, H, T, D,
            q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
            v.stride(0), v.stride(1), v.stride(2), out.stride(0), out.stride(1), out.stride(2),
            _lib.dtype_code(q), float(scaling))
    if mxint_bits is None and q_rope is None:
        rc = lib.mase_attention_causal(*args, _lib.stream_ptr(q))
    else:
        cos = sin = None
        cs_b = cs_t = 0
        if q_rope is not None:
            cos, sin = q_rope
            assert rope_supported(q, cos, sin)
            cs_b = cos.stride(0) if cos.dim() == 3 and cos.shape[0] == B and B > 1 else 0
            cs_t = cos.stride(-2)
        tab = log2_table(q.dtype, q.device).data_ptr() if mxint_bits is not None else None
        rc = lib.mase_attention_causal_fused(*args, cos.data_ptr() if cos is not None else None,
                                             sin.data_ptr() if sin is not None else None, cs_b, cs_t,
                                             int(mxint_bits or 0), tab, _lib.stream_ptr(q))
    _lib.check(rc, "mase_attention_causal")
    return out


def rope_supported(x: Tensor, cos: Tensor, sin: Tensor) -> bool:
    """x [B, H, T, D] (any strides with the last dimension contiguous), cos / sin [B or 1, T, D] or [T, D]"""
    if not (x.is_cuda and x.dim() == 4 and x.dtype in _lib.DTYPE_CODE and x.numel() > 0 and x.stride(3) == 1):
        return False
    if torch.is_grad_enabled() and x.requires_grad:
        return False
    B, H, T, D = x.shape
    if D % 16 != 0 or any(s % 8 for s in x.stride()[:3]) or x.data_ptr() % 16:
        return False
    for c in (cos, sin):
        if c.dtype != x.dtype or c.device != x.device or c.dim() not in (2, 3) or c.shape[-1] != D or c.shape[-2] != T:
            return False
        if c.stride(-1) != 1 or c.stride(-2) % 8 or c.data_ptr() % 16:
            return False
        if c.dim() == 3 and (c.shape[0] not in (1, B) or c.stride(0) % 8):
            return False
    return cos.shape == sin.shape and cos.stride() == sin.stride()


def rope(x: Tensor, cos: Tensor, sin: Tensor) -> Tensor:
    """``x * cos + rotate_half(x) * sin`` with the tables broadcast over heads, in one pass (``mase_rope``); the result has
    x's strides."""
    _lib.require_device(x, "rope")
    lib = _lib.load()
    assert rope_supported(x, cos, sin)
    B, H, T, D = x.shape
    out = torch.empty_strided(x.shape, x.stride(), dtype=x.dtype, device=x.device)
    cs_b = cos.stride(0) if cos.dim() == 3 and cos.shape[0] == B and B > 1 else 0
    rc = lib.mase_rope(x.data_ptr(), cos.data_ptr(), sin.data_ptr(), out.data_ptr(), B, H, T, D, x.stride(0), x.stride(1),
                       x.stride(2), cs_b, cos.stride(-2), _lib.dtype_code(x), _lib.stream_ptr(x))
    _lib.check(rc, "mase_rope")
    return out


ATTN_PROB_MAX_KV = 8192


def attn_softmax_mx_supported(scores: Tensor, mask: Tensor | None) -> bool:
    """whether ``attn_softmax_mx`` can take these operands (otherwise the caller runs the separate tensor passes)"""
    if not (scores.is_cuda and scores.dim() == 4 and scores.dtype in _lib.DTYPE_CODE and scores.numel() > 0):
        return False
    B, H, S, T = scores.shape
    if T % 32 != 0 or T > ATTN_PROB_MAX_KV:
        return False
    if mask is None:
        return True
    return (mask.dim() == 4 and mask.dtype == scores.dtype and mask.device == scores.device
            and tuple(mask.shape) == (B, 1, S, T) and mask.stride(3) == 1 and mask.stride(2) % 8 == 0
            and mask.stride(2) >= T and (B == 1 or mask.stride(0) == S * mask.stride(2)) and mask.data_ptr() % 16 == 0)


def attn_softmax_mx(scores: Tensor, mask: Tensor | None, scaling: float, cast: tuple | None, mx: tuple | None) -> Tensor:
    """Quantized attention probabilities from the raw query-key products in one pass (``mase_attn_softmax_mx``).
    ``cast``: (exp_bits, frac_bits, is_finite, round_mode) of the softmax input's minifloat cast or None;
    ``mx``: ("mxint", element_bits) / ("mxfp", exp_bits, frac_bits) for blocks of 32 along the last dim, or None."""
    _lib.require_device(scores, "attn_softmax_mx")
    lib = _lib.load()
    assert attn_softmax_mx_supported(scores, mask)
    scores = scores.contiguous()
    B, H, S, T = scores.shape
    out = torch.empty_like(scores)
    ce, cf, cfin, crm = (0, 0, 1, 0) if cast is None else (int(cast[0]), int(cast[1]), int(bool(cast[2])), _ROUND_MODES[cast[3]])
    kind, p0, p1, tab_t, tab_f = 0, 0, 0, None, None
    if mx is not None and mx[0] == "mxint":
        kind, p0 = 1, int(mx[1])
        tab_t = log2_table(scores.dtype, scores.device).data_ptr()
    elif mx is not None:
        kind, p0, p1 = 2, int(mx[1]), int(mx[2])
        tab_f = log2_table(torch.float32, scores.device).data_ptr()
    rc = lib.mase_attn_softmax_mx(scores.data_ptr(), None if mask is None else mask.data_ptr(), out.data_ptr(), B, H, S, T,
                                  0 if mask is None else mask.stride(2), _lib.dtype_code(scores), float(scaling), ce, cf,
                                  cfin, crm, kind, p0, p1, tab_t, tab_f, _lib.stream_ptr(scores))
    _lib.check(rc, "mase_attn_softmax_mx")
    return out


def mx_unpack(codes: Tensor, scales: Tensor, block_size: int, dtype: torch.dtype, kind: str, p0: int, p1: int = 0) -> Tensor:
    """Dequantize packed MX codes (flat, one byte per element, blocks of ``block_size`` consecutive elements) and
    their scale bytes, as produced by ``mxint_qdq(..., pack=True)`` (``kind="mxint"``, ``p0`` = element bits) or
    ``mxfp_qdq(..., pack=True)`` (``kind="mxfp"``, ``p0``/``p1`` = exponent / fraction bits).  Returns a flat tensor
    of ``dtype`` (reference: compose_mxint_tensor mxint/fake.py:59-80, mxfp compose mxfp/fake.py:75-104)."""
    _lib.require_device(codes, "mx_unpack")
    lib = _lib.load()
    codes, scales = codes.contiguous().reshape(-1), scales.contiguous().reshape(-1)
    assert codes.dtype in (torch.int8, torch.uint8) and scales.dtype == torch.uint8
    assert codes.numel() == scales.numel() * block_size
    out = torch.empty(codes.numel(), dtype=dtype, device=codes.device)
    rc = lib.mase_mx_unpack(codes.data_ptr(), scales.data_ptr(), out.data_ptr(), codes.numel(), int(block_size),
                            _lib.DTYPE_CODE[dtype], {"mxint": 0, "mxfp": 1}[kind], int(p0), int(p1),
                            _lib.stream_ptr(codes))
    _lib.check(rc, "mase_mx_unpack")
    return out


# ------------------------------------------------------------------------------------------------
# block floating point  (reference: block_fp.py:111-142; blocking utils.py:350-629)
# ------------------------------------------------------------------------------------------------
def _infer_block_shape(x_shape: List[int], block_shape: List[int]) -> List[int]:
    nd, nb = len(x_shape), len(block_shape)
    inferred = list(block_shape[-nd:]) if nb >= nd else [-1] * (nd - nb) + list(block_shape)
    return [x_shape[i] if (inferred[i] == -1 or inferred[i] > x_shape[i]) else inferred[i] for i in range(nd)]


def block_fp_geometry(shape: Sequence[int], block_size, skip_first_dim: bool):
    """(batch, rows, cols, tile_rows, tile_cols, folded) the reference's ``block`` dispatch (utils.py:569-592)
    implies; ``folded`` tells whether the reference reassembles the result with ``F.fold``."""
    if isinstance(block_size, int):
        block_size = [block_size]
    block_size = list(block_size)
    nd = len(shape)
    if nd == 1:
        assert skip_first_dim is False, "skip_first_dim must be False for bias to be blocked"
        bs = _infer_block_shape([shape[0]], block_size)
        return 1, 1, shape[0], 1, bs[0], False
    if nd == 2:
        if skip_first_dim:
            bs = _infer_block_shape([1, shape[1]], block_size)
            return 1, shape[0], shape[1], 1, bs[-1], False
        bs = _infer_block_shape([shape[0], shape[1]], block_size)
        return 1, shape[0], shape[1], bs[0], bs[1], True
    if nd == 3:
        if skip_first_dim:
            bs = _infer_block_shape([1, shape[1], shape[2]], block_size)
            return shape[0], shape[1], shape[2], bs[1], bs[2], True
        raise NotImplementedError("block 3d weight is not supported.")
    raise RuntimeError(f"Unsupported x.ndim = {nd}")


_bfp_geometry_cache: dict = {}


def block_fp_qdq(x: Tensor, width: int, exponent_width: int, exponent_bias, block_size, skip_first_dim: bool) -> Tensor:
    if x.is_cuda and x.is_contiguous():
        ptr = x.data_ptr()
        shape = x.shape
        gkey = (shape, tuple(block_size) if isinstance(block_size, (list, tuple)) else block_size, skip_first_dim,
                x.dtype)
        geom = _bfp_geometry_cache.get(gkey)
        if geom is None:
            batch, rows, cols, b0, b1, folded = block_fp_geometry(tuple(shape), block_size, skip_first_dim)
            vec = 4 if x.dtype == torch.float32 else 8
            single_pass = (b0 == 1 and b1 > 0 and (b1 & (b1 - 1)) == 0 and b1 <= 64 * vec and cols % b1 == 0
                           and x.numel() % vec == 0 and x.numel() > 0)
            if len(_bfp_geometry_cache) > 256:
                _bfp_geometry_cache.clear()
            geom = _bfp_geometry_cache[gkey] = (batch, rows, cols, b0, b1, int(folded), single_pass)
        if geom[6] and not ptr & 15:
            fn, code, tab, index = _state("mase_block_fp_qdq", x.dtype, x.device)
            out = torch.empty_like(x)
            bias = -1 if exponent_bias in (None, "none", "None") else int(exponent_bias)
            rc = fn(ptr, out.data_ptr(), geom[0], geom[1], geom[2], geom[3], geom[4], code, width, exponent_width, bias,
                    geom[5], tab, None, 0, _raw_stream(index))
            if rc:
                _lib.check(rc, "mase_block_fp_qdq")
            return out
    _lib.require_device(x, "block_fp_quantizer")
    lib = _lib.load()
    batch, rows, cols, b0, b1, folded = block_fp_geometry(tuple(x.shape), block_size, skip_first_dim)
    if exponent_bias in (None, "none", "None"):
        exponent_bias = -1
    xin = _contig(x)
    out = torch.empty_like(xin)
    if xin.numel() == 0:
        return out
    if b0 <= 0 or b1 <= 0:
        raise RuntimeError(f"invalid block shape {(b0, b1)}")
    dt = _lib.dtype_code(x)
    vec = 4 if x.dtype == torch.float32 else 8
    run_path = b0 == 1 and (b1 & (b1 - 1)) == 0 and b1 <= 64 * vec and cols % b1 == 0 and xin.numel() % vec == 0
    ws = None
    ws_bytes = 0
    if not run_path:
        ws_bytes = lib.mase_block_fp_workspace_bytes(batch, rows, cols, b0, b1, dt)
        ws = torch.empty(max(1, ws_bytes // 4), dtype=torch.int32, device=x.device)
    tab = log2_table(x.dtype, x.device)
    rc = lib.mase_block_fp_qdq(
        xin.data_ptr(), out.data_ptr(), batch, rows, cols, b0, b1, dt, width, exponent_width, int(exponent_bias),
        int(folded), tab.data_ptr(), ws.data_ptr() if ws is not None else None, ws_bytes, _lib.stream_ptr(x),
    )
    _lib.check(rc, "mase_block_fp_qdq")
    return out


# ------------------------------------------------------------------------------------------------
# element-wise formats
# ------------------------------------------------------------------------------------------------
def integer_qdq(x: Tensor, width: int, frac_width, is_signed: bool, use_floor: bool) -> Tensor:
    _lib.require_device(x, "integer_quantizer")
    lib = _lib.load()
    if frac_width is None:
        frac_width = width // 2
    xin = _contig(x)
    out = torch.empty_like(xin)
    rc = lib.mase_integer_qdq(xin.data_ptr(), out.data_ptr(), xin.numel(), _lib.dtype_code(x), int(width),
                              int(frac_width), int(bool(is_signed)), int(bool(use_floor)), _lib.stream_ptr(x))
    _lib.check(rc, "mase_integer_qdq")
    return out


def minifloat_qdq(x: Tensor, width: int, exponent_width: int, exponent_bias, ieee: bool) -> Tensor:
    _lib.require_device(x, "minifloat quantizer")
    lib = _lib.load()
    if exponent_bias in (None, "none", "None"):
        exponent_bias = -1
    xin = _contig(x)
    out = torch.empty_like(xin)
    tab = log2_table(x.dtype, x.device)
    rc = lib.mase_minifloat_qdq(xin.data_ptr(), out.data_ptr(), xin.numel(), _lib.dtype_code(x), int(width),
                                int(exponent_width), int(exponent_bias), int(bool(ieee)), tab.data_ptr(),
                                _lib.stream_ptr(x))
    _lib.check(rc, "mase_minifloat_qdq")
    return out


_ROUND_MODES = {"rn": 0, "ru": 1, "rd": 2, "rz": 3}


def minifloat_mx_qdq(x: Tensor, exp_bits: int, frac_bits: int, is_finite: bool, round_mode: str,
                     output_dtype: torch.dtype | None) -> Tensor:
    _lib.require_device(x, "minifloat_quantizer_sim")
    lib = _lib.load()
    if round_mode not in _ROUND_MODES:
        raise ValueError(f"Unknown rounding mode: {round_mode}")
    xin = _contig(x)
    odt = output_dtype or x.dtype
    out = torch.empty(xin.shape, dtype=odt, device=x.device)
    if odt not in _lib.DTYPE_CODE:
        raise _lib.MaseAmdError(f"unsupported output dtype {odt}")
    rc = lib.mase_minifloat_mx_qdq(xin.data_ptr(), out.data_ptr(), xin.numel(), _lib.dtype_code(x),
                                   _lib.DTYPE_CODE[odt], int(exp_bits), int(frac_bits), int(bool(is_finite)),
                                   _ROUND_MODES[round_mode], _lib.stream_ptr(x))
    _lib.check(rc, "mase_minifloat_mx_qdq")
    return out
