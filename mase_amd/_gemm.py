"""Host wrappers of the matrix-core contractions."""
from __future__ import annotations

import torch
from torch import Tensor

from . import _lib

GEMM_K_MULTIPLE = 64  # K tile of mase_gemm_bf16_tn
SKINNY_MAX_ROWS = 128  # at most this many rows of activations take mase_gemm_bf16_skinny
OPERAND_BYTES_LIMIT = (1 << 32) - 1  # per-call operand size the GEMM entry points accept


PACKED_B_K_MULTIPLE = 128


def gemm_bf16_packed_b_supported(N: int, K: int) -> bool:
    return K % PACKED_B_K_MULTIPLE == 0 and (N + 31) // 32 * 32 * K * 2 <= OPERAND_BYTES_LIMIT


def gemm_bf16_takes_packed_b(M: int, N: int, K: int) -> bool:
    """whether ``gemm_bf16_tn`` would run the tiled kernel on a fragment-ordered B for this shape (not the
    weight-streaming kernel of few rows, not the K-range form of a few hundred rows)"""
    if M <= SKINNY_MAX_ROWS or not gemm_bf16_packed_b_supported(N, K):
        return False
    return 2 * M * K > OPERAND_BYTES_LIMIT or _lib.load().mase_gemm_bf16_tn_splitk_workspace_bytes(M, N, K) == 0


def gemm_bf16_pack_b(b: Tensor) -> Tensor:
    """fragment-ordered image of ``b[N,K]`` (bf16) for ``gemm_bf16_tn(..., b_packed=...)``: ``mase_gemm_bf16_pack_b``"""
    _lib.require_device(b, "gemm_bf16_pack_b")
    lib = _lib.load()
    assert b.dtype == torch.bfloat16 and b.dim() == 2
    b = b.contiguous()
    N, K = b.shape
    nbytes = lib.mase_gemm_bf16_packed_bytes(N, K)
    assert nbytes > 0, "K must be a multiple of 32"
    out = torch.empty(nbytes, dtype=torch.uint8, device=b.device)
    _lib.check(lib.mase_gemm_bf16_pack_b(b.data_ptr(), out.data_ptr(), N, K, _lib.stream_ptr(b)), "mase_gemm_bf16_pack_b")
    return out


def gemm_bf16_tn(a: Tensor, b: Tensor, bias: Tensor | None, out_dtype: torch.dtype, b_packed: Tensor | None = None) -> Tensor:
    """``a[M,K] @ b[N,K].T + bias`` with bf16 operands and fp32 accumulation; result in ``out_dtype``.
    ``b_packed``: the image of ``gemm_bf16_pack_b(b)``, used by the tiled kernel when the shape takes that kernel."""
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
    if M <= SKINNY_MAX_ROWS:
        # few rows (token-by-token serving): the weight-streaming kernel, which spreads N and K over the whole chip
        nbytes = lib.mase_gemm_bf16_skinny_workspace_bytes(M, N, K)
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=a.device)
        rc = lib.mase_gemm_bf16_skinny(
            a.data_ptr(), b.data_ptr(), bias.data_ptr() if bias is not None else None, out.data_ptr(), M, N, K,
            _lib.DTYPE_CODE[out_dtype], _lib.DTYPE_CODE[bias.dtype] if bias is not None else 0, ws.data_ptr(), nbytes,
            _lib.stream_ptr(a),
        )
        _lib.check(rc, "mase_gemm_bf16_skinny")
        return out
    # a few hundred rows: too few output tiles for the chip; K ranges become work items as well
    nbytes = lib.mase_gemm_bf16_tn_splitk_workspace_bytes(M, N, K) if 2 * M * K <= OPERAND_BYTES_LIMIT else 0
    if nbytes:
        ws = torch.empty(nbytes, dtype=torch.uint8, device=a.device)
        rc = lib.mase_gemm_bf16_tn_splitk(
            a.data_ptr(), b.data_ptr(), bias.data_ptr() if bias is not None else None, out.data_ptr(), M, N, K,
            _lib.DTYPE_CODE[out_dtype], _lib.DTYPE_CODE[bias.dtype] if bias is not None else 0, ws.data_ptr(), nbytes,
            _lib.stream_ptr(a),
        )
        _lib.check(rc, "mase_gemm_bf16_tn_splitk")
        return out
    # the kernel addresses an operand with 32-bit byte offsets: activations beyond 4 GiB go in row chunks
    rows_per_call = max(1, min(M, (OPERAND_BYTES_LIMIT // (2 * K)) // 256 * 256 or 1))
    packed = b_packed is not None and gemm_bf16_packed_b_supported(N, K)
    for r0 in range(0, M, rows_per_call):
        r1 = min(M, r0 + rows_per_call)
        args = (bias.data_ptr() if bias is not None else None, out[r0:r1].data_ptr(), r1 - r0, N, K,
                _lib.DTYPE_CODE[out_dtype], _lib.DTYPE_CODE[bias.dtype] if bias is not None else 0, _lib.stream_ptr(a))
        if packed:
            _lib.check(lib.mase_gemm_bf16_tn_packed(a[r0:r1].data_ptr(), b_packed.data_ptr(), *args), "mase_gemm_bf16_tn_packed")
        else:
            _lib.check(lib.mase_gemm_bf16_tn(a[r0:r1].data_ptr(), b.data_ptr(), *args), "mase_gemm_bf16_tn")
    return out


def _batch_strides(t: Tensor):
    """the leading dimensions of a [..., rows, cols] tensor as at most two nested indices: (outer count, inner count,
    outer stride, inner stride) with outer count 1 when one index does; None when they need more than two"""
    merged = []
    for n, st in zip(t.shape[:-2], t.stride()[:-2]):
        if n == 1:
            continue
        if merged and merged[-1][1] == st * n:  # contiguous with respect to the dimension before it: one index
            merged[-1] = (merged[-1][0] * n, st)
        else:
            merged.append((n, st))
    if len(merged) > 2:
        return None
    while len(merged) < 2:
        merged.insert(0, (1, 0))
    return merged[0][0], merged[1][0], merged[0][1], merged[1][1]


def _common_batch_split(tensors):
    """(outer count, inner count, [(outer stride, inner stride) per tensor]) such that every tensor's leading
    dimensions are addressed by the same two nested indices; None when there is no such pair"""
    parts = [_batch_strides(t) for t in tensors]
    if any(p is None for p in parts):
        return None
    two_level = {p[:2] for p in parts if p[0] > 1}
    if len(two_level) > 1:
        return None
    count = parts[0][0] * parts[0][1]
    n_outer, n_inner = two_level.pop() if two_level else (1, count)
    strides = []
    for no, ni, so, si in parts:
        if no * ni != count:
            return None
        # a tensor that needs one index only: the outer index advances it by n_inner inner steps
        strides.append((so, si) if no > 1 else (si * n_inner, si))
    return n_outer, n_inner, strides


def gemm_bf16_tn_batched_supported(a: Tensor, b: Tensor) -> bool:
    """a [..., M, K] and b [..., N, K] bf16 device tensors with equal leading shapes, last dimension contiguous, K a
    multiple of 64, strides multiples of 8, leading dimensions expressible as two nested indices common to both"""
    if not (a.is_cuda and a.device == b.device and a.dtype == b.dtype == torch.bfloat16 and a.dim() == b.dim() >= 3):
        return False
    if a.shape[:-2] != b.shape[:-2] or a.shape[-1] != b.shape[-1] or a.numel() == 0 or b.numel() == 0:
        return False
    if torch.is_grad_enabled() and (a.requires_grad or b.requires_grad):
        return False
    K = a.shape[-1]
    if K % GEMM_K_MULTIPLE:
        return False
    for t in (a, b):
        if t.stride(-1) != 1 or t.stride(-2) < K or any(st % 8 for st in t.stride()[:-1]) or t.data_ptr() % 16:
            return False
        if t.shape[-2] * t.stride(-2) * 2 > OPERAND_BYTES_LIMIT:
            return False
    return _common_batch_split((a, b)) is not None


def gemm_bf16_tn_batched(a: Tensor, b: Tensor, out_dtype: torch.dtype | None = None, out: Tensor | None = None) -> Tensor:
    """``a[..., M, K] @ b[..., N, K]^T`` for every index of the leading dimensions: bf16 operands (strided views are
    taken as they are), fp32 accumulation, one rounding to ``out_dtype`` (``mase_gemm_bf16_tn_batched``).  ``out``: a
    [..., M, N] tensor to write into (last dimension contiguous, e.g. a transposed view of [batch, M, heads, N]
    memory); without it the result is contiguous."""
    _lib.require_device(a, "gemm_bf16_tn_batched")
    lib = _lib.load()
    assert gemm_bf16_tn_batched_supported(a, b)
    lead = tuple(a.shape[:-2])
    M, K, N = a.shape[-2], a.shape[-1], b.shape[-2]
    if out is None:
        out = torch.empty(lead + (M, N), dtype=out_dtype or a.dtype, device=a.device)
        if (N * out.element_size()) % 16:  # rows of whole 16-byte pieces: pad the row stride
            pad = 16 // out.element_size()
            out = torch.empty(lead + (M, (N + pad - 1) // pad * pad), dtype=out.dtype, device=a.device)[..., :N]
    assert tuple(out.shape) == lead + (M, N) and out.stride(-1) == 1 and out.device == a.device
    esz = out.element_size()
    split = _common_batch_split((a, b, out))
    if split is None or out.data_ptr() % 16 or any((st * esz) % 16 for st in out.stride()[:-1]):
        raise _lib.MaseAmdError("gemm_bf16_tn_batched: the output's layout does not fit the operands' (strides of whole "
                                "16-byte pieces, leading dimensions addressed by the same two nested indices)")
    n_outer, n_inner, ((a_so, a_si), (b_so, b_si), (c_so, c_si)) = split
    rc = lib.mase_gemm_bf16_tn_batched(a.data_ptr(), b.data_ptr(), out.data_ptr(), n_outer, n_inner, M, N, K, a.stride(-2),
                                       b.stride(-2), out.stride(-2), a_so, a_si, b_so, b_si, c_so, c_si,
                                       _lib.DTYPE_CODE[out.dtype], _lib.stream_ptr(a))
    _lib.check(rc, "mase_gemm_bf16_tn_batched")
    return out


def transpose_last2(y: Tensor, rows_padded: int) -> Tensor:
    """``y[..., K, N] -> [..., N, rows_padded]`` contiguous, columns K .. rows_padded - 1 zero (``mase_transpose16``
    when the layout allows it: 16-bit elements, N a multiple of 8, last dimension contiguous, strides multiples of 8,
    leading dimensions addressable by two nested indices; a strided copy of the library otherwise)"""
    K, N = y.shape[-2], y.shape[-1]
    out = torch.empty(y.shape[:-2] + (N, rows_padded), dtype=y.dtype, device=y.device)
    split = _batch_strides(y)
    if (y.is_cuda and y.element_size() == 2 and N % 8 == 0 and y.stride(-1) == 1 and rows_padded % 64 == 0
            and 0 <= rows_padded - K < 64 and split is not None and split[0] * split[1] <= 65535
            and not any(st % 8 for st in y.stride()[:-1]) and y.data_ptr() % 16 == 0):
        n_outer, n_inner, s_outer, s_inner = split
        rc = _lib.load().mase_transpose16(y.data_ptr(), out.data_ptr(), n_outer, n_inner, K, N, rows_padded, s_outer, s_inner,
                                          y.stride(-2), _lib.stream_ptr(y))
        _lib.check(rc, "mase_transpose16")
        return out
    if rows_padded != K:
        out[..., K:].zero_()
    out[..., :K].copy_(y.transpose(-1, -2))
    return out


def matmul_bf16(x: Tensor, y: Tensor, out: Tensor | None = None, out_dtype: torch.dtype | None = None) -> Tensor | None:
    """``torch.matmul(x, y)`` for bf16 device tensors x [..., M, K], y [..., K, N] with equal leading dimensions on the
    batched matrix-core kernel of this package (fp32 accumulation, one rounding to ``out_dtype``, bf16 unless given), or None when the operands do
    not fit it (the caller then uses the library's).  y is copied into [..., N, K] rows once (the kernel contracts
    rows with rows); a contraction length that is not a multiple of 64 is padded with zeros in that copy and in a copy
    of x.  ``out``: as in ``gemm_bf16_tn_batched``."""
    if not (x.is_cuda and x.dtype == y.dtype == torch.bfloat16 and x.dim() == y.dim() >= 3 and x.shape[:-2] == y.shape[:-2]
            and x.shape[-1] == y.shape[-2] and x.numel() > 0 and y.numel() > 0):
        return None
    if torch.is_grad_enabled() and (x.requires_grad or y.requires_grad):
        return None
    K = x.shape[-1]
    pad = -K % GEMM_K_MULTIPLE
    if y.stride(-2) == 1 and not pad and y.stride(-1) >= K:  # already rows of K (a transposed view)
        yt = y.transpose(-1, -2)
    else:
        yt = transpose_last2(y, K + pad)
    if pad:
        x = torch.nn.functional.pad(x, (0, pad))
    elif x.stride(-1) != 1 or any(st % 8 for st in x.stride()[:-1]) or x.data_ptr() % 16:
        x = x.contiguous()
    if not gemm_bf16_tn_batched_supported(x, yt):
        return None
    return gemm_bf16_tn_batched(x, yt, out_dtype=out_dtype, out=out)


def gemm_mxint8_packed_supported(N: int, K: int) -> bool:
    return K % PACKED_B_K_MULTIPLE == 0 and (N + 31) // 32 * 32 * K <= OPERAND_BYTES_LIMIT


def gemm_mxint8_pack_b(codes: Tensor, scales: Tensor):
    """fragment-ordered code and scale images of an MXINT8 weight (int8 codes [N,K], uint8 scales [N,K/32]) for
    ``gemm_mxint8_tn_packed``: ``mase_gemm_mxint8_pack_b``"""
    _lib.require_device(codes, "gemm_mxint8_pack_b")
    lib = _lib.load()
    assert codes.dtype == torch.int8 and scales.dtype == torch.uint8 and codes.dim() == 2
    codes, scales = codes.contiguous(), scales.contiguous()
    N, K = codes.shape
    assert scales.shape == (N, K // 32) and gemm_mxint8_packed_supported(N, K)
    img = torch.empty(lib.mase_gemm_mxint8_packed_code_bytes(N, K), dtype=torch.uint8, device=codes.device)
    simg = torch.empty(lib.mase_gemm_mxint8_packed_scale_bytes(N, K), dtype=torch.uint8, device=codes.device)
    _lib.check(lib.mase_gemm_mxint8_pack_b(codes.data_ptr(), scales.data_ptr(), img.data_ptr(), simg.data_ptr(), N, K,
                                           _lib.stream_ptr(codes)), "mase_gemm_mxint8_pack_b")
    return img, simg


def gemm_mxint8_tn_packed(a: Tensor, code_image: Tensor, scale_image: Tensor, N: int, bias: Tensor | None,
                          out_dtype: torch.dtype) -> Tensor:
    """``a[M,K] @ dequant(weight)[N,K].T + bias`` on the tiled kernel with the weight as MXINT8 code / scale images
    (``gemm_mxint8_pack_b``); bf16 activations, fp32 accumulation; the same values as ``gemm_bf16_tn`` on the
    dequantized weight."""
    _lib.require_device(a, "gemm_mxint8_tn_packed")
    lib = _lib.load()
    assert a.dtype == torch.bfloat16 and a.dim() == 2
    a = a.contiguous()
    M, K = a.shape
    assert gemm_mxint8_packed_supported(N, K) and code_image.numel() == lib.mase_gemm_mxint8_packed_code_bytes(N, K)
    out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    if bias is not None:
        bias = bias.contiguous()
    rows_per_call = max(1, min(M, (OPERAND_BYTES_LIMIT // (2 * K)) // 256 * 256 or 1))
    for r0 in range(0, M, rows_per_call):
        r1 = min(M, r0 + rows_per_call)
        rc = lib.mase_gemm_mxint8_tn_packed(
            a[r0:r1].data_ptr(), code_image.data_ptr(), scale_image.data_ptr(), bias.data_ptr() if bias is not None else None,
            out[r0:r1].data_ptr(), r1 - r0, N, K, _lib.DTYPE_CODE[out_dtype],
            _lib.DTYPE_CODE[bias.dtype] if bias is not None else 0, _lib.stream_ptr(a))
        _lib.check(rc, "mase_gemm_mxint8_tn_packed")
    return out


MXINT8_SKINNY_K_MULTIPLE = 128


def gemm_mxint8_skinny_supported(M: int, N: int, K: int) -> bool:
    return 0 < M <= SKINNY_MAX_ROWS and K % MXINT8_SKINNY_K_MULTIPLE == 0 and N * K < (1 << 32)


def gemm_mxint8_skinny(a: Tensor, codes: Tensor, scales: Tensor, bias: Tensor | None, out_dtype: torch.dtype) -> Tensor:
    """``a[M,K] @ dequant(codes, scales)[N,K].T + bias`` for at most 128 rows of bf16 activations, with the weight held
    as MXINT8 codes (int8 [N,K]) and scale bytes (uint8 [N,K/32]): half the weight bytes of the bf16 image."""
    _lib.require_device(a, "gemm_mxint8_skinny")
    lib = _lib.load()
    assert a.dtype == torch.bfloat16 and codes.dtype == torch.int8 and scales.dtype == torch.uint8
    a, codes, scales = a.contiguous(), codes.contiguous(), scales.contiguous()
    M, K = a.shape
    N = codes.shape[0]
    assert codes.shape == (N, K) and scales.shape == (N, K // 32) and gemm_mxint8_skinny_supported(M, N, K)
    out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    if bias is not None:
        bias = bias.contiguous()
    nbytes = lib.mase_gemm_mxint8_skinny_workspace_bytes(M, N, K)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=a.device)
    rc = lib.mase_gemm_mxint8_skinny(
        a.data_ptr(), codes.data_ptr(), scales.data_ptr(), bias.data_ptr() if bias is not None else None, out.data_ptr(),
        M, N, K, _lib.DTYPE_CODE[out_dtype], _lib.DTYPE_CODE[bias.dtype] if bias is not None else 0, ws.data_ptr(), nbytes,
        _lib.stream_ptr(a),
    )
    _lib.check(rc, "mase_gemm_mxint8_skinny")
    return out


# element formats of the block-scaled matrix instruction: (exp_bits, frac_bits) -> format code of the C ABI
MXFP_HW_FORMATS = {(4, 3): 0, (5, 2): 1, (2, 1): 4}
MXFP_K_MULTIPLE = 128  # K tile of mase_gemm_mxfp_scaled


def mxfp_pack(x: Tensor, exp_bits: int, frac_bits: int):
    """Quantize ``x`` (blocks of 32 along the last dim) to packed MXFP codes + E8M0 scales for the matrix
    instruction.  Returns ``(codes uint8 [..., K] or [..., K/2], scales uint8 [..., K/32])``."""
    from ._tables import log2_table

    _lib.require_device(x, "mxfp_pack")
    lib = _lib.load()
    assert (exp_bits, frac_bits) in MXFP_HW_FORMATS
    x = x.contiguous()
    K = x.shape[-1]
    assert K % 32 == 0, "the last dimension must hold whole blocks of 32"
    per_byte = 2 if exp_bits + frac_bits + 1 <= 4 else 1
    codes = torch.empty(*x.shape[:-1], K // per_byte, dtype=torch.uint8, device=x.device)
    scales = torch.empty(*x.shape[:-1], K // 32, dtype=torch.uint8, device=x.device)
    tab = log2_table(torch.float32, x.device)
    rc = lib.mase_mxfp_pack(x.data_ptr(), codes.data_ptr(), scales.data_ptr(), x.numel(), _lib.dtype_code(x),
                            exp_bits, frac_bits, tab.data_ptr(), _lib.stream_ptr(x))
    _lib.check(rc, "mase_mxfp_pack")
    return codes, scales


def gemm_mxfp_scaled(a_codes: Tensor, a_scales: Tensor, a_fmt, b_codes: Tensor, b_scales: Tensor, b_fmt,
                     bias: Tensor | None, out_dtype: torch.dtype) -> Tensor:
    """``dequant(A)[M,K] @ dequant(B)[N,K].T + bias`` on packed MXFP operands (``mxfp_pack`` layout)."""
    _lib.require_device(a_codes, "gemm_mxfp_scaled")
    lib = _lib.load()
    M, K = a_codes.shape[0], a_scales.shape[1] * 32
    N = b_codes.shape[0]
    assert b_scales.shape[1] * 32 == K and K % MXFP_K_MULTIPLE == 0
    out = torch.empty((M, N), dtype=out_dtype, device=a_codes.device)
    if bias is not None:
        bias = bias.contiguous()
    rows_per_call = max(1, min(M, (OPERAND_BYTES_LIMIT // K) // 256 * 256 or 1))  # M*K < 2^32 per call
    for r0 in range(0, M, rows_per_call):
        r1 = min(M, r0 + rows_per_call)
        rc = lib.mase_gemm_mxfp_scaled(
            a_codes[r0:r1].data_ptr(), a_scales[r0:r1].data_ptr(), MXFP_HW_FORMATS[tuple(a_fmt)], b_codes.data_ptr(),
            b_scales.data_ptr(), MXFP_HW_FORMATS[tuple(b_fmt)], bias.data_ptr() if bias is not None else None,
            out[r0:r1].data_ptr(), r1 - r0, N, K, _lib.DTYPE_CODE[out_dtype],
            _lib.DTYPE_CODE[bias.dtype] if bias is not None else 0, _lib.stream_ptr(a_codes),
        )
        _lib.check(rc, "mase_gemm_mxfp_scaled")
    return out


def gemm_mxfp4_tiled_supported(M: int, N: int, K: int, a_fmt, b_fmt) -> bool:
    """Whether ``gemm_mxfp4_scaled_tiled`` takes the product: 8-bit activations, e2m1 weights, whole K tiles and a weight
    image below 2^32 bytes (the activations are cut into row ranges that fit)."""
    return (tuple(a_fmt) in ((4, 3), (5, 2)) and tuple(b_fmt) == (2, 1) and K > 0 and K % MXFP_K_MULTIPLE == 0
            and M > 0 and -(-N // 256) * 256 * K // 2 < (1 << 32) and 256 * K < (1 << 32))


def mxfp_tile_codes(codes: Tensor, K: int, bits: int) -> Tensor:
    """The tile image of a row-major code matrix ``[rows, K * bits / 8]`` (``mase_mxfp_tile_codes``): what the tiled
    block-scaled GEMM copies from.  Done once for a weight."""
    _lib.require_device(codes, "mxfp_tile_codes")
    lib = _lib.load()
    codes = codes.contiguous()
    rows = codes.shape[0]
    assert codes.dtype == torch.uint8 and codes.shape == (rows, K * bits // 8)
    nbytes = lib.mase_mxfp_tiled_bytes(rows, K, bits)
    assert nbytes > 0, "K must be a multiple of 128 and bits 4 or 8"
    tiled = torch.empty(nbytes, dtype=torch.uint8, device=codes.device)
    _lib.check(lib.mase_mxfp_tile_codes(codes.data_ptr(), tiled.data_ptr(), rows, K, bits, _lib.stream_ptr(codes)),
               "mase_mxfp_tile_codes")
    return tiled


def mxfp_pack_tiled(x: Tensor, exp_bits: int, frac_bits: int):
    """``mxfp_pack`` of a 2-D ``x`` [rows, K] to e4m3 / e5m2 with the codes written as the tile image (flat uint8 of
    ``mase_mxfp_tiled_bytes(rows, K, 8)`` bytes; the rows that pad the last tile are left unwritten).  Returns
    ``(tiled codes, scales uint8 [rows, K/32])``."""
    from ._tables import log2_table

    _lib.require_device(x, "mxfp_pack_tiled")
    lib = _lib.load()
    assert x.dim() == 2 and (exp_bits, frac_bits) in ((4, 3), (5, 2))
    x = x.contiguous()
    rows, K = x.shape
    nbytes = lib.mase_mxfp_tiled_bytes(rows, K, 8)
    assert nbytes > 0, "K must be a multiple of 128"
    tiled = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    scales = torch.empty(rows, K // 32, dtype=torch.uint8, device=x.device)
    tab = log2_table(torch.float32, x.device)
    rc = lib.mase_mxfp_pack_tiled(x.data_ptr(), tiled.data_ptr(), scales.data_ptr(), rows, K, _lib.dtype_code(x),
                                  exp_bits, frac_bits, tab.data_ptr(), _lib.stream_ptr(x))
    _lib.check(rc, "mase_mxfp_pack_tiled")
    return tiled, scales


def gemm_mxfp4_scaled_tiled(a_tiled: Tensor, a_scales: Tensor, a_fmt, b_tiled: Tensor, b_scales: Tensor,
                            bias: Tensor | None, out_dtype: torch.dtype) -> Tensor:
    """``gemm_mxfp_scaled`` for e4m3 / e5m2 activations and e2m1 weights with both code matrices as tile images
    (``mxfp_pack_tiled`` / ``mxfp_tile_codes``); the same bits come out."""
    _lib.require_device(a_tiled, "gemm_mxfp4_scaled_tiled")
    lib = _lib.load()
    M, K = a_scales.shape[0], a_scales.shape[1] * 32
    N = b_scales.shape[0]
    assert gemm_mxfp4_tiled_supported(M, N, K, a_fmt, (2, 1)) and b_scales.shape[1] * 32 == K
    assert a_tiled.numel() == lib.mase_mxfp_tiled_bytes(M, K, 8) and b_tiled.numel() == lib.mase_mxfp_tiled_bytes(N, K, 4)
    out = torch.empty((M, N), dtype=out_dtype, device=a_tiled.device)
    if bias is not None:
        bias = bias.contiguous()
    rows_per_call = max(256, (OPERAND_BYTES_LIMIT // K) // 256 * 256)  # whole row tiles, image below 2^32 bytes per call
    for r0 in range(0, M, rows_per_call):
        r1 = min(M, r0 + rows_per_call)
        rc = lib.mase_gemm_mxfp4_scaled_tiled(
            a_tiled.data_ptr() + r0 * K, a_scales[r0:r1].data_ptr(), MXFP_HW_FORMATS[tuple(a_fmt)], b_tiled.data_ptr(),
            b_scales.data_ptr(), bias.data_ptr() if bias is not None else None, out[r0:r1].data_ptr(), r1 - r0, N, K,
            _lib.DTYPE_CODE[out_dtype], _lib.DTYPE_CODE[bias.dtype] if bias is not None else 0,
            _lib.stream_ptr(a_tiled),
        )
        _lib.check(rc, "mase_gemm_mxfp4_scaled_tiled")
    return out


def gemm_mxfp4_skinny_supported(M: int, N: int, K: int, b_fmt) -> bool:
    return 0 < M <= SKINNY_MAX_ROWS and K % 128 == 0 and tuple(b_fmt) == (2, 1) and N * K // 2 < (1 << 32)


def gemm_mxfp4_skinny(a_codes: Tensor, a_scales: Tensor, a_fmt, b_codes: Tensor, b_scales: Tensor, bias: Tensor | None,
                      out_dtype: torch.dtype) -> Tensor:
    """``dequant(A)[M,K] @ dequant(B)[N,K].T + bias`` for at most 128 rows of e4m3 / e5m2 activations and e2m1 weights
    (``mxfp_pack`` layout): the weight-streaming form of ``gemm_mxfp_scaled``."""
    _lib.require_device(a_codes, "gemm_mxfp4_skinny")
    lib = _lib.load()
    a_codes, a_scales = a_codes.contiguous(), a_scales.contiguous()
    b_codes, b_scales = b_codes.contiguous(), b_scales.contiguous()
    M, K = a_codes.shape
    N = b_codes.shape[0]
    assert b_codes.shape == (N, K // 2) and a_scales.shape == (M, K // 32) and b_scales.shape == (N, K // 32)
    assert gemm_mxfp4_skinny_supported(M, N, K, (2, 1)) and tuple(a_fmt) in ((4, 3), (5, 2))
    out = torch.empty((M, N), dtype=out_dtype, device=a_codes.device)
    if bias is not None:
        bias = bias.contiguous()
    nbytes = lib.mase_gemm_mxfp4_skinny_workspace_bytes(M, N, K)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=a_codes.device)
    rc = lib.mase_gemm_mxfp4_skinny(
        a_codes.data_ptr(), a_scales.data_ptr(), MXFP_HW_FORMATS[tuple(a_fmt)], b_codes.data_ptr(), b_scales.data_ptr(),
        bias.data_ptr() if bias is not None else None, out.data_ptr(), M, N, K, _lib.DTYPE_CODE[out_dtype],
        _lib.DTYPE_CODE[bias.dtype] if bias is not None else 0, ws.data_ptr(), nbytes, _lib.stream_ptr(a_codes),
    )
    _lib.check(rc, "mase_gemm_mxfp4_skinny")
    return out
