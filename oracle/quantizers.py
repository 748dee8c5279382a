"""Op-for-op torch (CPU) restatement of the reference quantize-dequantize functions.  TEST INFRASTRUCTURE.

Citations are to files under the reference's ``src/chop/nn/quantizers/``.  Every function keeps the
reference's operation order and dtypes, because intermediate rounding (in bf16/fp16) and library
behaviour (``log2`` in the tensor dtype, ``clamp`` casting bounds) are part of the result.
Autograd wrappers (straight-through estimators) are not restated here: the oracle checks forward values.
"""
from __future__ import annotations

from math import ceil
from typing import List, Sequence

import torch
from torch import Tensor
from torch.nn import functional as F


# ----------------------------------------------------------------------------------------------
# shared helpers: mxfp/helpers.py:8-29 (flatten_for_quantize) and :32-63 (permute_for_dequantize)
# ----------------------------------------------------------------------------------------------
def _move_block_dim_last_and_flatten(t: Tensor, block_dim: int) -> Tensor:
    nd = t.dim()
    d = block_dim % nd
    order = [i for i in range(nd) if i != d] + [d]
    return t.permute(order).flatten()


def _restore_from_flat(flat: Tensor, shape: Sequence[int], block_dim: int) -> Tensor:
    nd = len(shape)
    d = block_dim % nd
    moved = [s for i, s in enumerate(shape) if i != d] + [shape[d]]
    t = flat.reshape(moved)
    back = list(range(nd - 1))
    back.insert(d, nd - 1)
    return t.permute(back)


# ----------------------------------------------------------------------------------------------
# MXINT  (mxint/fake.py:11-56 extract, :59-80 compose, mxint/mxint.py:145-169 sim, :211-251 entry)
# ----------------------------------------------------------------------------------------------
def mxint_components(flat: Tensor, block_size: int, element_bits: int, scale_bits: int = 8):
    """(biased clamped scale, integer mantissa), both float tensors of shape [n_blocks,1] / [n_blocks,B].

    mxint/fake.py:11-56 with percentile=1.0.
    """
    B = block_size
    assert flat.numel() % B == 0, f"Input tensor size {flat.numel()} is not divisible by block size {B}."
    x = flat.flatten().reshape(flat.numel() // B, B)
    dt = x.dtype
    # quantile(1.0) over |x| in fp32, cast back (fake.py:36-41)
    mx = x.abs().to(torch.float32).quantile(1.0, dim=1, keepdim=True).to(dt)
    mx = mx.clamp(min=torch.finfo(dt).tiny)  # fake.py:44
    scale = mx.log2().ceil()  # fake.py:45 -- evaluated in dt
    bias = 2 ** (scale_bits - 1) - 1
    x = x / 2**scale  # fake.py:47 (unclamped exponent)
    mant = x * 2 ** (element_bits - 1)  # fake.py:48
    scale = (scale + bias).clamp(min=0, max=2**scale_bits - 1)  # fake.py:49-50
    mant = mant.round().clamp(min=-(2 ** (element_bits - 1)), max=2 ** (element_bits - 1) - 1)  # fake.py:51-54
    return scale, mant


def mxint_quantizer(
    x: Tensor,
    block_size: int,
    element_bits: int,
    block_dim: int = -1,
    scale_bits: int = 8,
    quantile_search: bool = False,
    dtype: torch.dtype | None = None,
) -> Tensor:
    """mxint/mxint.py:211-251 -> MXIntQuantize.forward :183-202 -> mxint_quantizer_sim: else-branch :145-169, or
    the search branch :40-143 without calibration activations."""
    if quantile_search:
        return mxint_clip_search(x, block_size, element_bits, block_dim, scale_bits)[0]
    in_dt = x.dtype
    shape = tuple(x.shape)
    assert -len(shape) <= block_dim < len(shape)
    flat = _move_block_dim_last_and_flatten(x, block_dim)
    scale, mant = mxint_components(flat, block_size, element_bits, scale_bits)
    bias = 2 ** (scale_bits - 1) - 1
    deq = mant / 2 ** (element_bits - 1) * 2 ** (scale - bias)  # fake.py:75-80
    out = _restore_from_flat(deq, shape, block_dim)
    return out.to(dtype or in_dt)


CLIP_PERCENTILES = (1.0, 0.995, 0.99, 0.97, 0.95, 0.93, 0.90, 0.80, 0.70, 0.60, 0.50)  # mxint.py:47-51, mxfp.py:53


def mxint_clip_search(x: Tensor, block_size: int, element_bits: int, block_dim: int = -1, scale_bits: int = 8,
                      act_tensor: Tensor | None = None, cali_batch_size: int = 32):
    """The search branch of mxint_quantizer_sim (mxint/mxint.py:40-143), scored on the weights (act_tensor=None, :97-98)
    or on their products with calibration activations [batches, tokens, B] (:99-131).

    Returns (dequantized tensor, index of the chosen percentile per block, errors [11, n_blocks], candidates
    [11, n_blocks, B]).  The candidates are the blocks taken along block_dim; the error is measured against the blocks of the plain flattening (:41-45, :97),
    which are the same blocks only when block_dim is the last dimension.
    """
    B = block_size
    shape = tuple(x.shape)
    assert -len(shape) <= block_dim < len(shape)
    rows = x.flatten().reshape(-1, B)  # :41-45
    blocks = _move_block_dim_last_and_flatten(x, block_dim).flatten().reshape(-1, B)  # :58-65
    dt = blocks.dtype
    pct = torch.tensor(CLIP_PERCENTILES, dtype=torch.float32)
    mx = blocks.abs().to(torch.float32).quantile(pct, dim=1, keepdim=True).to(dt)  # :68-73  [11, n_blocks, 1]
    mx = mx.clamp(min=torch.finfo(dt).tiny)  # :76
    scale = mx.log2().ceil()  # :77
    bias = 2 ** (scale_bits - 1) - 1
    mant = (blocks / 2**scale) * 2 ** (element_bits - 1)  # :79-80, broadcast to [11, n_blocks, B]
    scale = (scale + bias).clamp(min=0, max=2**scale_bits - 1)  # :81-82
    mant = mant.round().clamp(min=-(2 ** (element_bits - 1)), max=2 ** (element_bits - 1) - 1)  # :83-86
    cand = mant / 2 ** (element_bits - 1) * 2 ** (scale - bias)  # :88-90
    if act_tensor is None:
        err = torch.norm(cand - rows, p=2, dim=-1)  # :97
        pick = torch.argmin(err, dim=0).reshape(-1)  # :98
    else:
        assert act_tensor.shape[-1] == B  # :101-104 views any other width to 4-D, which the contraction below rejects
        err = torch.zeros([len(CLIP_PERCENTILES), rows.shape[0]], dtype=x.dtype)  # :107-111
        for b in range(0, act_tensor.shape[0], cali_batch_size):  # :114-126
            act_b = act_tensor[b:b + cali_batch_size]
            out_orig = torch.matmul(act_b, rows.T)
            out_q = torch.einsum("asb,phb->pash", act_b, cand.to(act_tensor.dtype))
            err += torch.norm(out_q - out_orig, p=2, dim=(1, 2))
        pick = torch.argmin(err, dim=0)  # :128
    chosen = cand[pick, torch.arange(cand.shape[1])]  # :132
    out = _restore_from_flat(chosen, shape, block_dim).to(x.dtype)  # :141-143
    return out, pick, err, cand


# ----------------------------------------------------------------------------------------------
# _minifloat_mx  (fake.py:11-93 extract, :96-149 compose, minifloat.py:12-33 sim)
# ----------------------------------------------------------------------------------------------
def minifloat_mx_extract(x: Tensor, exp_bits: int, frac_bits: int, is_finite: bool, round_mode: str) -> Tensor:
    """float tensor -> uint16 codes.  _minifloat_mx/fake.py:11-93."""
    E, Fb = exp_bits, frac_bits
    assert E > 0 and Fb > 0 and E + Fb < 16  # meta.py:26-29
    bias = (1 << (E - 1)) - 1
    e_hi = (1 << E) - 1 if is_finite else (1 << E) - 2
    e_hi_unb = e_hi - bias
    e_lo_unb = -bias
    frac_hi = (1 << Fb) - 1

    x = x.to(torch.float32)
    neg = x < 0
    xb = x.abs().view(torch.int32)
    ftz = (xb & 0x7F800000) == 0
    xn = torch.where(ftz, 0.0, x)

    fr, ex = xn.abs().frexp()
    fr = fr * 2
    ex = ex - 1
    if not is_finite:
        is_inf = x.isinf()
        is_nan = x.isnan()

    under = ex < e_lo_unb
    over = ex > e_hi_unb
    ye = ex + bias
    yf = fr.view(torch.int32) & 0x7FFFFF
    if round_mode == "rz":
        yf = yf >> (23 - Fb)
    else:
        yf = (yf >> 8).float() / (1 << (15 - Fb))
        if round_mode == "ru":
            yf = yf.ceil()
        elif round_mode == "rd":
            yf = yf.floor()
        elif round_mode == "rn":
            yf = yf.round()
        else:
            raise ValueError(f"Unknown rounding mode: {round_mode}")
        yf = yf.to(torch.int32)

    sub = (ye == 0) & (yf != 0)
    yf = torch.where(sub, (yf | (1 << Fb)) >> 1, yf)
    yf = torch.where(under, 0, yf)
    ye = torch.where(under, 0, ye)
    yf = torch.where(over, frac_hi, yf)
    ye = torch.where(over, e_hi, ye)
    yf = torch.where(ftz, 0, yf)
    ye = torch.where(ftz, 0, ye)
    if not is_finite:
        yf = torch.where(is_inf, 0, yf)
        yf = torch.where(is_nan, (1 << Fb) - 1, yf)
        ye = torch.where(is_inf, e_hi, ye)
        ye = torch.where(is_nan, e_hi, ye)
    y = (ye << Fb) | yf
    y = torch.where(neg, y + (1 << (E + Fb)), y)
    return y.to(torch.uint16)


def minifloat_mx_compose(codes: Tensor, exp_bits: int, frac_bits: int, is_finite: bool, output_dtype: torch.dtype) -> Tensor:
    """uint16 codes -> float tensor.  _minifloat_mx/fake.py:96-149."""
    E, Fb = exp_bits, frac_bits
    sign_mask = 1 << (E + Fb)
    bias = (1 << (E - 1)) - 1
    assert codes.dtype == torch.uint16
    c = codes.to(torch.int32)
    sgn = (c & sign_mask) << (31 - (E + Fb))
    c = c & 0x7FFF
    xe = (c >> Fb) & ((1 << E) - 1)
    xf = c & ((1 << Fb) - 1)
    sub = (xe == 0) & (xf != 0)
    zero = (xe == 0) & (xf == 0)
    if not is_finite:
        nf = xe == ((1 << E) - 1)
        inf = nf & (xf == 0)
        nan = nf & (xf != 0)
    ye = xe - bias
    ye = torch.where(sub, ye + 1, ye)
    ye = torch.exp2(ye)
    yf = xf.to(torch.float32) / (1 << Fb)
    yf = torch.where(sub, yf, yf + 1.0)
    y = ye * yf
    if not is_finite:
        y = torch.where(inf, float("inf"), y)
        y = torch.where(nan, float("nan"), y)
    y = torch.where(zero, 0.0, y)
    y = torch.where(sgn != 0, -y, y)
    return y.to(output_dtype)


def minifloat_quantizer_sim(x: Tensor, exp_bits: int, frac_bits: int, is_finite: bool, round_mode: str,
                            output_dtype: torch.dtype | None = None) -> Tensor:
    """_minifloat_mx/minifloat.py:12-33."""
    codes = minifloat_mx_extract(x, exp_bits, frac_bits, is_finite, round_mode)
    return minifloat_mx_compose(codes, exp_bits, frac_bits, is_finite, output_dtype or x.dtype)


# ----------------------------------------------------------------------------------------------
# MXFP  (mxfp/fake.py:12-72 extract, :75-104 compose, mxfp/mxfp.py:107-115 sim tail, :151-230 entry)
# ----------------------------------------------------------------------------------------------
_LEGAL_MXFP = ((4, 3), (5, 2), (2, 3), (3, 2), (2, 1), (1, 2))  # mxfp/meta.py:41


def mxfp_components(flat: Tensor, block_size: int, exp_bits: int, frac_bits: int, scale_exp_bits: int = 8,
                    is_finite: bool = True, round_mode: str = "rn", percentile: float = 1.0):
    """(scales uint8 [n_blocks,1], element codes uint8 [n_blocks,B]).  mxfp/fake.py:12-72."""
    assert scale_exp_bits in (8,), f"Invalid scale exponent bits: {scale_exp_bits}."  # meta.py:35-39
    assert (exp_bits, frac_bits) in _LEGAL_MXFP, f"Invalid element exp/frac bits: {(exp_bits, frac_bits)}."
    t = flat.float()
    B = block_size
    assert t.numel() % B == 0
    sc_bias = (1 << (scale_exp_bits - 1)) - 1
    sc_hi = (1 << scale_exp_bits) - 1 - sc_bias
    sc_lo = 0 - sc_bias
    el_hi = (1 << exp_bits) - 1 if is_finite else (1 << exp_bits) - 2
    el_bias = (1 << (exp_bits - 1)) - 1
    el_hi_unb = el_hi - el_bias

    t = t.flatten().reshape(t.numel() // B, B)
    ftz = (t.view(torch.int32) & 0x7F800000) == 0
    t = torch.where(ftz, 0.0, t)
    sh = t.abs().quantile(percentile, dim=1, keepdim=True)
    sh = sh.log2().floor().to(torch.int32)
    sh -= el_hi_unb
    sh = sh.clamp(sc_lo, sc_hi)
    sc = sh + sc_bias
    sc = torch.where(ftz.all(dim=1, keepdim=True), 0, sc).to(torch.uint8)
    sc_fp = torch.exp2(sh)
    mf = torch.where(ftz, 0.0, t / sc_fp)
    el = minifloat_mx_extract(mf, exp_bits, frac_bits, is_finite, round_mode)
    el = el.view(torch.uint16).to(torch.uint8)
    return sc, el


def mxfp_quantizer(
    x: Tensor,
    block_size: int,
    element_exp_bits: int,
    element_frac_bits: int,
    block_dim: int = -1,
    scale_exp_bits: int = 8,
    quantile_search: bool = False,
    dtype: torch.dtype | None = None,
) -> Tensor:
    """mxfp/mxfp.py:187-230 -> MXFPQuantize.forward :154-178 (finite elements, "rn") -> sim :107-115, or the search
    branch :40-105 without calibration activations."""
    if quantile_search:
        return mxfp_clip_search(x, block_size, element_exp_bits, element_frac_bits, block_dim, scale_exp_bits, dtype)[0]
    shape = tuple(x.shape)
    assert -len(shape) <= block_dim < len(shape)
    flat = _move_block_dim_last_and_flatten(x, block_dim)
    sc, el = mxfp_components(flat, block_size, element_exp_bits, element_frac_bits, scale_exp_bits, True, "rn")
    sc_bias = (1 << (scale_exp_bits - 1)) - 1
    sc_fp = torch.exp2(sc.to(torch.int32) - sc_bias)  # fake.py:97-98
    mf = minifloat_mx_compose(el.to(torch.uint16), element_exp_bits, element_frac_bits, True, torch.float32)
    deq = (mf * sc_fp).flatten().to(dtype or x.dtype)  # fake.py:102-103
    return _restore_from_flat(deq, shape, block_dim)


def mxfp_clip_search(x: Tensor, block_size: int, element_exp_bits: int, element_frac_bits: int, block_dim: int = -1,
                     scale_exp_bits: int = 8, dtype: torch.dtype | None = None, act_tensor: Tensor | None = None,
                     cali_batch_size: int = 32):
    """The search branch of mxfp_quantizer_sim (mxfp/mxfp.py:40-105), scored on the weights (act_tensor=None, :94-97) or
    on the products with calibration activations [batches, tokens, B] (:65-93).

    Returns (dequantized tensor, index of the chosen percentile per block, errors [11, n_blocks], candidates
    [11, n_blocks, B] dequantized).  The score of a
    candidate is computed, as there, from the element *codes* as integers and with the power of two in the uint8
    arithmetic of the scale tensor (:58-63); an incumbent is replaced only by a strictly smaller score (:99-103).
    """
    B = block_size
    shape = tuple(x.shape)
    assert -len(shape) <= block_dim < len(shape)
    rows = x.flatten().reshape(-1, B)  # :41-45
    flat = _move_block_dim_last_and_flatten(x, block_dim)
    best = torch.full([rows.shape[0]], float("inf"), dtype=x.dtype)  # :46-48
    best_sc, best_el = mxfp_components(flat, B, element_exp_bits, element_frac_bits, scale_exp_bits, True, "rn", 1.0)
    pick = torch.zeros(rows.shape[0], dtype=torch.int64)
    errs, cands = [], []
    sc_bias = 2 ** (scale_exp_bits - 1) - 1

    def compose(sc, el):  # fake.py:75-104
        sc_fp = torch.exp2(sc.to(torch.int32) - sc_bias)
        mf = minifloat_mx_compose(el.to(torch.uint16), element_exp_bits, element_frac_bits, True, torch.float32)
        return (mf * sc_fp).to(dtype or x.dtype)

    for i, pct in enumerate(CLIP_PERCENTILES):
        sc, el = mxfp_components(flat, B, element_exp_bits, element_frac_bits, scale_exp_bits, True, "rn", pct)
        q = el / 2 ** (element_frac_bits - 1) * 2 ** (sc - sc_bias)  # :58-62 (uint8 tensors: sc - bias and 2**() wrap)
        q = q.to(dtype=rows.dtype)  # :63
        if act_tensor is not None:
            assert act_tensor.shape[-1] == B  # :67-72 views any other width to 4-D, which makes the error's shape wrong
            err = torch.zeros(rows.shape[0], dtype=x.dtype)  # :75-77
            for b in range(0, act_tensor.shape[0], cali_batch_size):  # :80-90
                act_b = act_tensor[b:b + cali_batch_size]
                out_q = torch.matmul(act_b, q.T)
                out_orig = torch.matmul(act_b, rows.T)
                err += torch.norm(out_q - out_orig, p=2, dim=(0, 1))
        else:
            q -= rows  # :94
            q.abs_()
            q.pow_(2)
            err = torch.sum(q, 1)  # :97
        errs.append(err)
        cands.append(compose(sc, el))
        better = err < best  # :99
        best[better] = err[better]
        best_sc[better] = sc[better]
        best_el[better] = el[better]
        pick[better] = i
    deq = compose(best_sc, best_el).flatten()  # :107-113
    return _restore_from_flat(deq, shape, block_dim), pick, torch.stack(errs), torch.stack(cands)


# ----------------------------------------------------------------------------------------------
# block / unblock  (utils.py:350-391 shape inference, :394-566 per-rank helpers, :569-629 dispatch)
# ----------------------------------------------------------------------------------------------
def _infer_block_shape(x_shape: List[int], block_shape: List[int]) -> List[int]:
    """utils.py:350-375: right-align, -1 or oversize -> full dim."""
    nd, nb = len(x_shape), len(block_shape)
    inferred = list(block_shape[-nd:]) if nb >= nd else [-1] * (nd - nb) + list(block_shape)
    return [x_shape[i] if (inferred[i] == -1 or inferred[i] > x_shape[i]) else inferred[i] for i in range(nd)]


def _infer_padding(x_shape: List[int], block_shape: List[int]) -> List[int]:
    """utils.py:378-391: right padding per dim, in F.pad order (last dim first)."""
    pad = []
    for xs, bs in zip(x_shape, block_shape):
        if bs == -1 or xs < bs:
            pad += [0, 0]
        else:
            pad += [ceil(xs / bs) * bs - xs, 0]
    return pad[::-1]


def _block(x: Tensor, block_shape: List[int], skip_first_dim: bool):
    """utils.py:569-592.  Returns (blocked, per_block_max, padded_shape, block_shape, kind)."""
    if x.ndim == 1:
        assert skip_first_dim is False, "skip_first_dim must be False for bias to be blocked"
        xs = list(x.shape)
        bs = _infer_block_shape(xs, block_shape)  # utils.py:394-413
        px = F.pad(x, _infer_padding(xs, bs))
        blocked = px.reshape(px.shape[0] // bs[0], bs[0])
        return blocked, blocked.abs().max(dim=1, keepdim=True)[0], list(px.shape), bs, "1d"
    if x.ndim == 2 and skip_first_dim:
        xs = list(x.shape)  # utils.py:435-452
        bs = _infer_block_shape([1, xs[1]], block_shape)
        px = F.pad(x, _infer_padding(xs, bs))
        blocked = px.reshape(xs[0], px.shape[1] // bs[-1], bs[-1])
        return blocked, blocked.abs().max(dim=2, keepdim=True)[0], list(px.shape), bs, "2da"
    if x.ndim == 2:
        xs = list(x.shape)  # utils.py:469-490
        bs = _infer_block_shape(xs, block_shape)
        px = F.pad(x, _infer_padding(xs, bs))
        blocked = F.unfold(px.unsqueeze(0).unsqueeze(0), kernel_size=bs, dilation=1, padding=0, stride=bs).squeeze(0)
        return blocked, blocked.abs().max(dim=0, keepdim=True)[0], list(px.shape), bs, "2dw"
    if x.ndim == 3:
        if not skip_first_dim:
            raise NotImplementedError("block 3d weight is not supported.")
        xs = list(x.shape)  # utils.py:519-545
        one = [1, *xs[1:]]
        bs = _infer_block_shape(one, block_shape)
        px = F.pad(x, _infer_padding(one, bs))
        blocked = F.unfold(px.unsqueeze(1), kernel_size=bs[1:], dilation=1, padding=0, stride=bs[1:])
        return blocked, blocked.abs().max(dim=1, keepdim=True)[0], list(px.shape), bs, "3da"
    raise RuntimeError(f"Unsupported x.ndim = {x.ndim}")


def _unblock(blocked: Tensor, orig_shape: List[int], padded_shape: List[int], bs: List[int], kind: str) -> Tensor:
    """utils.py:595-629 and the per-rank inverses."""
    if kind == "1d":
        x = blocked.flatten()  # utils.py:416-432
    elif kind == "2da":
        x = blocked.flatten(1)  # utils.py:455-466
    elif kind == "2dw":
        x = F.fold(blocked, output_size=padded_shape, kernel_size=bs, dilation=1, padding=0, stride=bs).squeeze(0)
    else:
        x = F.fold(blocked, output_size=padded_shape[1:], kernel_size=bs[1:], dilation=1, padding=0, stride=bs[1:]).squeeze(1)
    return x[tuple(slice(None, s) for s in orig_shape)]


# ----------------------------------------------------------------------------------------------
# block floating point  (block_fp.py:7-82, entry :111-142)
# ----------------------------------------------------------------------------------------------
def block_fp_quantizer(
    x: Tensor,
    width: int = 12,
    exponent_width: int = 8,
    exponent_bias: int | None = None,
    block_size: List[int] | int = [16],
    skip_first_dim: bool = True,
) -> Tensor:
    if isinstance(block_size, int):
        block_size = [block_size]
    orig_shape = list(x.shape)
    blocked, bmax, padded_shape, bs, kind = _block(x, list(block_size), skip_first_dim)
    # block_fp.py:40-44 zero-block fill
    if torch.all(bmax == 0):
        bmax = torch.ones_like(bmax)
    else:
        bmax[bmax == 0] = bmax[bmax != 0].min()
    mbits = width - 1
    if exponent_bias in (None, "none", "None"):
        exponent_bias = 2 ** (exponent_width - 1) - 1
    e_hi = 2**exponent_width - 1 - exponent_bias
    e_lo = -exponent_bias
    m_hi = 2**mbits - 1
    sgn = torch.sign(blocked + 1e-9)  # :55
    val = torch.abs(blocked) + 1e-9  # :57
    e = torch.ceil(torch.log2(bmax)).clamp(min=e_lo, max=e_hi)  # :58-59
    man = val / 2**e  # :61
    shift = 2**mbits
    q = (man * shift).round().clamp(min=0, max=m_hi)  # :63-65
    man = q / shift
    msfp = sgn * (2**e) * man  # :68
    y = _unblock(msfp, orig_shape, padded_shape, bs, kind)
    close = torch.isclose(x, torch.tensor([0.0], dtype=x.dtype, device=x.device))  # :79
    return (~close) * y + close * x  # :80


# ----------------------------------------------------------------------------------------------
# fixed point  (integer.py:10-46 round, :49-66 floor, entries :97-122)
# ----------------------------------------------------------------------------------------------
def _int_bounds(width: int, is_signed: bool):
    return (-(2 ** (width - 1)), 2 ** (width - 1) - 1) if is_signed else (0, 2**width - 1)


def integer_quantizer(x: Tensor, width: int, frac_width: int | None = None, is_signed: bool = True) -> Tensor:
    if frac_width is None:
        frac_width = width // 2
    lo, hi = _int_bounds(width, is_signed)
    scale = 2**frac_width
    return x.mul(scale).round().clamp(min=lo, max=hi).div(scale)


def integer_floor_quantizer(x: Tensor, width: int, frac_width: int | None = None, is_signed: bool = True) -> Tensor:
    if frac_width is None:
        frac_width = width // 2
    lo, hi = _int_bounds(width, is_signed)
    scale = 2**frac_width
    return x.mul(scale).floor().clamp(min=lo, max=hi).div(scale)


# ----------------------------------------------------------------------------------------------
# element-wise minifloat  (minifloat.py:7-68 denorm, :120-182 ieee)
# ----------------------------------------------------------------------------------------------
def minifloat_denorm_quantizer(x: Tensor, width: int, exponent_width: int, exponent_bias: int | None = None) -> Tensor:
    mbits = width - exponent_width - 1
    if exponent_bias in (None, "none", "None"):
        exponent_bias = 2 ** (exponent_width - 1) - 1
    e_hi = 2**exponent_width - 1 - exponent_bias
    e_lo = -exponent_bias
    m_hi = 2**mbits - 1
    sgn = torch.sign(x + 1e-9)  # :46
    val = torch.abs(x)
    e = torch.ceil(torch.log2(val + 1e-9)).clamp(min=e_lo, max=e_hi)  # :50-51
    man = val / 2**e  # :55
    shift = 2**mbits
    q = (man * shift).round().clamp(min=0, max=m_hi)  # :57-61
    man = q / shift
    close = torch.isclose(val, torch.tensor([0.0], dtype=val.dtype, device=val.device))  # :65
    return (~close) * (sgn * (2**e) * man) + close * x  # :66


def minifloat_ieee_quantizer(x: Tensor, width: int, exponent_width: int, exponent_bias: int | None = None) -> Tensor:
    mbits = width - exponent_width - 1
    if exponent_bias in (None, "none", "None"):
        exponent_bias = 2 ** (exponent_width - 1) - 1
    e_hi = 2**exponent_width - 1 - exponent_bias
    e_lo = -exponent_bias
    shift = 2**mbits
    m_hi = 2**mbits - 1
    sgn = torch.sign(x + 1e-9)  # :158
    val = torch.abs(x)
    e = torch.floor(torch.log2(val + 1e-9)).clamp(min=e_lo, max=e_hi)  # :162-163
    man = val / 2**e  # :165
    if isinstance(exponent_bias, (int, float)):
        exponent_bias = torch.tensor([exponent_bias], dtype=e.dtype, device=e.device)  # :171-172
    normal = ~torch.isclose(e, -exponent_bias)  # :173
    q = normal * (man * shift - shift).round().clamp(min=0, max=m_hi) + (~normal) * (man * shift / 2).round().clamp(
        min=0, max=m_hi
    )  # :175-176
    man = normal * (1.0 + q / shift) + (~normal) * (q / shift * 2)  # :177
    close = torch.isclose(val, torch.tensor([0.0], dtype=val.dtype, device=val.device))  # :179
    return (~close) * (sgn * (2**e) * man) + close * x  # :180
