"""Host-measured ``log2`` correction tables for the kernels.

The reference computes ``ceil(log2(v))`` / ``floor(log2(v))`` with the host math library *in the tensor
dtype* (``mxint/fake.py:45``, ``block_fp.py:58``, ``minifloat.py:50,162``, ``mxfp/fake.py:58``).  That rounded
logarithm lands on an integer for values a few ulps off a power of two, so the result differs from the
exact integer answer there.  The library is accurate to about an ulp but not correctly rounded, so the
affected mantissas are *measured* here, once per dtype, by calling ``torch.log2`` on the CPU for every
candidate, and handed to the kernels as per-exponent thresholds (layout: ``include/mase_amd.h``).
"""
from __future__ import annotations

import numpy as np
import torch

from ._lib import LOG2_TABLE_WORDS

_HALF = 288
_K_MIN, _K_MAX = -149, 127
_cpu_tables: dict[torch.dtype, np.ndarray] = {}
_dev_tables: dict[tuple[torch.dtype, str], torch.Tensor] = {}


def _split(v64: np.ndarray):
    """exact (k, M): v = 2^k * (1 + M / 2^23) for positive finite float64 holding fp32-exact values"""
    mant, exp = np.frexp(v64)
    k = exp.astype(np.int64) - 1
    M = np.rint((mant * 2.0 - 1.0) * float(1 << 23)).astype(np.int64)
    return k, M


def _thresholds(k: np.ndarray, M: np.ndarray, ceil_v: np.ndarray, floor_v: np.ndarray, what: str) -> np.ndarray:
    tab = np.zeros(LOG2_TABLE_WORDS, dtype=np.uint32)
    tab[_HALF:] = 0x800000
    pow2 = M == 0
    if not (np.all(ceil_v[pow2] == k[pow2]) and np.all(floor_v[pow2] == k[pow2])):
        raise RuntimeError(f"{what}: log2 of an exact power of two is not exact on this host")
    for kk in np.unique(k):
        sel = (k == kk) & ~pow2
        if not sel.any():
            continue
        order = np.argsort(M[sel])
        m = M[sel][order]
        c = ceil_v[sel][order]
        f = floor_v[sel][order]
        if not (np.all((c == kk) | (c == kk + 1)) and np.all((f == kk) | (f == kk + 1))):
            raise RuntimeError(f"{what}: log2 off by more than one at exponent {kk}")
        low = c == kk  # ceil came out one too small
        n_low = int(low.sum())
        if n_low and not low[:n_low].all():
            raise RuntimeError(f"{what}: ceil(log2) corrections are not a prefix at exponent {kk}")
        if n_low:
            tab[kk - _K_MIN] = m[n_low - 1]
        high = f == kk + 1  # floor came out one too large
        n_high = int(high.sum())
        if n_high and not high[len(high) - n_high:].all():
            raise RuntimeError(f"{what}: floor(log2) corrections are not a suffix at exponent {kk}")
        if n_high:
            tab[_HALF + kk - _K_MIN] = m[len(m) - n_high]
    _summarise(tab)
    return tab


def _summarise(tab: np.ndarray) -> None:
    """Words 277..279 of each half: the widest exponent interval around k=0 without corrections, and the
    extreme threshold, so that kernels can skip the per-lane table read in the common case."""
    n = _K_MAX - _K_MIN + 1
    for half, neutral in ((0, 0), (_HALF, 0x800000)):
        thr = tab[half:half + n]
        clean = thr == neutral
        lo = hi = 0 - _K_MIN  # biased index of k = 0
        if not clean[lo]:
            lo, hi = 1, 0  # empty interval
        else:
            while lo - 1 >= 0 and clean[lo - 1]:
                lo -= 1
            while hi + 1 < n and clean[hi + 1]:
                hi += 1
        tab[half + 277] = lo
        tab[half + 278] = hi
        tab[half + 279] = thr.max() if half == 0 else thr.min()


def _measure_16bit(dtype: torch.dtype) -> np.ndarray:
    top = 0x7F80 if dtype == torch.bfloat16 else 0x7C00
    bits = torch.arange(1, top, dtype=torch.int32).to(torch.int16)
    v = bits.view(dtype)
    lg = v.log2()
    ceil_v = lg.ceil().float().numpy().astype(np.int64)
    floor_v = lg.floor().float().numpy().astype(np.int64)
    k, M = _split(v.double().numpy())
    return _thresholds(k, M, ceil_v, floor_v, str(dtype))


def _measure_fp32(window: int = 512) -> np.ndarray:
    ks, Ms = [], []
    for k in range(_K_MIN, _K_MAX + 1):
        step = 1 << max(0, -126 - k)  # mantissa granularity (coarser for subnormals)
        n = min(window, ((1 << 23) - 1) // step)
        if n <= 0:
            cand = np.zeros(1, dtype=np.int64)
        else:
            j = np.arange(1, n + 1, dtype=np.int64) * step
            cand = np.unique(np.concatenate([[0], j, (1 << 23) - j]))
            cand = cand[(cand >= 0) & (cand < (1 << 23))]
        ks.append(np.full(cand.shape, k, dtype=np.int64))
        Ms.append(cand)
    k = np.concatenate(ks)
    M = np.concatenate(Ms)
    v64 = np.ldexp(1.0 + M.astype(np.float64) / float(1 << 23), k)
    v = torch.from_numpy(v64).to(torch.float32)
    assert torch.equal(v.double(), torch.from_numpy(v64)), "candidate not exactly representable in fp32"
    lg = v.log2()
    ceil_v = lg.ceil().numpy().astype(np.int64)
    floor_v = lg.floor().numpy().astype(np.int64)
    tab = _thresholds(k, M, ceil_v, floor_v, "torch.float32")
    # the probe window must extend past every correction
    for kk in range(_K_MIN, _K_MAX + 1):
        step = 1 << max(0, -126 - kk)
        n = min(window, ((1 << 23) - 1) // step)
        if n >= window and (tab[kk - _K_MIN] >= window * step or tab[_HALF + kk - _K_MIN] <= (1 << 23) - window * step):
            raise RuntimeError(f"fp32 log2 corrections reach the edge of the probe window at exponent {kk}")
    return tab


def log2_table_cpu(dtype: torch.dtype) -> np.ndarray:
    """uint32[576] table for ``dtype`` measured with torch on this host (cached)."""
    if dtype not in _cpu_tables:
        if dtype == torch.float32:
            _cpu_tables[dtype] = _measure_fp32()
        elif dtype in (torch.bfloat16, torch.float16):
            _cpu_tables[dtype] = _measure_16bit(dtype)
        else:
            raise ValueError(f"no log2 table for {dtype}")
    return _cpu_tables[dtype]


def log2_table(dtype: torch.dtype, device: torch.device) -> torch.Tensor:
    """The table as an int32 tensor on ``device`` (cached per dtype and device)."""
    key = (dtype, str(device))
    if key not in _dev_tables:
        host = torch.from_numpy(log2_table_cpu(dtype).view(np.int32).copy())
        _dev_tables[key] = host.to(device)
    return _dev_tables[key]
