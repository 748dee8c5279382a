"""Shared input builders and bit-exact comparison for the parity tests."""
import numpy as np
import torch

_INT = {torch.float32: torch.int32, torch.bfloat16: torch.int16, torch.float16: torch.int16}


def bits(t: torch.Tensor) -> torch.Tensor:
    return t.detach().cpu().contiguous().view(_INT[t.dtype])


def assert_bits_equal(got: torch.Tensor, want: torch.Tensor, what: str = ""):
    """Bit-exact (so -0.0 != +0.0); NaN matches NaN whatever the payload."""
    got = got.detach().cpu()
    want = want.detach().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    assert got.dtype == want.dtype, f"{what}: dtype {got.dtype} != {want.dtype}"
    gn, wn = got.float().isnan(), want.float().isnan()
    same = (bits(got) == bits(want)) | (gn & wn)
    if not bool(same.all()):
        idx = (~same).flatten().nonzero().flatten()
        i = int(idx[0])
        g, w = got.flatten()[i], want.flatten()[i]
        raise AssertionError(
            f"{what}: {idx.numel()} of {same.numel()} elements differ; first at flat index {i}: "
            f"got {float(g)!r} (0x{int(bits(got).flatten()[i]) & 0xFFFFFFFF:x}) want {float(w)!r} "
            f"(0x{int(bits(want).flatten()[i]) & 0xFFFFFFFF:x})"
        )


def adversarial_fp32_bits(rng: np.random.Generator, n: int, finite_only: bool = True) -> np.ndarray:
    """fp32 patterns: wide-range normals, values next to powers of two, rounding ties, tiny, subnormal, zeros."""
    out = np.empty(n, dtype=np.uint32)
    kind = rng.integers(0, 8, size=n)
    sign = rng.integers(0, 2, size=n).astype(np.uint32) << 31
    exp_mid = rng.integers(100, 150, size=n).astype(np.uint32)
    exp_any = rng.integers(0, 255, size=n).astype(np.uint32)
    man = rng.integers(0, 1 << 23, size=n).astype(np.uint32)
    small_m = rng.integers(0, 8, size=n).astype(np.uint32)
    out[:] = sign | (exp_mid << 23) | man
    k = kind == 1
    out[k] = sign[k] | (exp_any[k] << 23) | man[k]
    k = kind == 2
    out[k] = sign[k] | (exp_mid[k] << 23) | small_m[k]
    k = kind == 3
    out[k] = sign[k] | (exp_mid[k] << 23) | (np.uint32(0x7FFFFF) - small_m[k])
    k = kind == 4
    out[k] = sign[k] | (exp_mid[k] << 23) | (man[k] & np.uint32(0x7F8000))
    k = kind == 5
    out[k] = sign[k] | (exp_mid[k] << 23) | (man[k] & np.uint32(0x7F80FF)) | np.uint32(0x4000)
    k = kind == 6
    out[k] = sign[k] | (rng.integers(0, 3, size=int(k.sum())).astype(np.uint32) << 23) | (man[k] * (small_m[k] & 1))
    return out


def fp32_from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int32).copy()).view(torch.float32)


def adversarial(rng: np.random.Generator, shape, dtype: torch.dtype, block: int = 32) -> torch.Tensor:
    """A tensor of `dtype` mixing N(0,1) rows with adversarial rows (see module doc); finite values only."""
    n = int(np.prod(shape))
    x = torch.from_numpy(rng.standard_normal(n).astype(np.float32))
    adv = fp32_from_bits(adversarial_fp32_bits(rng, n))
    if dtype == torch.float16:
        adv = adv.clamp(-60000, 60000)
    pick = torch.from_numpy(rng.integers(0, 4, size=n // block + 1).repeat(block)[:n])
    x = torch.where(pick == 0, adv, x)
    # blocks scaled to wildly different magnitudes
    scale = torch.from_numpy((2.0 ** rng.integers(-20, 20, size=n // block + 1)).astype(np.float32).repeat(block)[:n])
    x = torch.where(pick == 1, x * scale, x)
    if dtype == torch.float16:
        x = x.clamp(-60000, 60000)
    x = x.to(dtype)
    flat = x.view(-1)
    # exact powers of two and their one-ulp neighbours as block maxima
    nb = n // block
    for b in rng.integers(0, max(nb, 1), size=max(1, nb // 8)):
        p2 = float(2.0 ** int(rng.integers(-10, 12)))
        v = torch.tensor([p2], dtype=dtype)
        d = int(rng.integers(-2, 3))
        v = (v.view(_INT[dtype]) + d).view(dtype)
        lo = int(b) * block
        seg = flat[lo:lo + block]
        seg.mul_(0.01 * p2 / max(float(seg.float().abs().max()), 1e-30))
        flat[lo + int(rng.integers(0, block))] = v if rng.integers(0, 2) else -v
    # zero block, +-0 mix, single non-zero
    if nb >= 3:
        flat[:block] = 0
        flat[block:2 * block] = torch.where(torch.arange(block) % 2 == 0, torch.tensor(-0.0), torch.tensor(0.0)).to(dtype)
        flat[2 * block:3 * block] = 0
        flat[2 * block + 3] = -3.0
    return x.view(shape)
