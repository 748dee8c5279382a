"""GPU tests of the clip search (quantile_search=True without calibration activations) against the oracle.

Every block the kernel writes must be, bit for bit, the oracle's candidate of the index the kernel reports; the
index must be the oracle's except where two candidates' errors agree to within the rounding of the error itself
(the library's summation order over the 32 squares is not reproduced), and those exceptions must be rare."""
import numpy as np
import pytest
import torch

import oracle as O
from helpers import assert_bits_equal

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]
ULP = {torch.float32: 2.0 ** -22, torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}


def search_inputs(seed: int, dtype: torch.dtype, rows: int = 96, cols: int = 256, scale: float = 0.05) -> torch.Tensor:
    """weight-like rows plus blocks with outliers, many zeros, equal magnitudes, wide ranges and tiny values"""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g) * scale
    x[1] *= torch.exp2(torch.randint(-12, 12, (cols,), generator=g).float())          # wide range inside blocks
    x[2, ::32] *= 50                                                                   # one outlier per block
    x[3, ::7] *= 9
    x[4] = torch.where(torch.rand(cols, generator=g) < 0.6, torch.zeros(cols), x[4])   # more than half zeros
    x[5] = torch.where(torch.rand(cols, generator=g) < 0.97, torch.zeros(cols), x[5])  # almost all zeros
    x[6] = 0.0
    x[7] = torch.sign(x[7]) * scale                                                   # equal magnitudes
    x[8] = torch.exp2(torch.randint(-3, 3, (cols,), generator=g).float()) * scale      # powers of two
    x[9] *= 2.0 ** -20
    x[10] *= 2.0 ** 10
    x[11, :64] = torch.linspace(-1, 1, 64) * scale
    if dtype != torch.float16:
        x[12] *= 2.0 ** -100
        x[13] *= 2.0 ** 60
        x[14] *= 2.0 ** -120
    else:
        x = x.clamp(-60000.0, 60000.0)  # Inf inputs are not specified
    return x.to(dtype)


def check_against_oracle(got, choice, oracle_result, dtype, what, min_agree=0.998):
    want, pick, err, cand = oracle_result
    B = cand.shape[-1]
    nb = cand.shape[1]
    choice = choice.cpu().long()
    assert int(choice.max()) <= 10
    # the block written is the oracle's candidate of the reported index
    mine = cand[choice, torch.arange(nb)]
    assert_bits_equal(got, mine.reshape(got.shape).to(dtype), f"{what}: block contents for the reported index")
    agree = choice == pick
    rate = float(agree.double().mean())
    print(f"{what}: same candidate as the oracle in {rate:.5f} of {nb} blocks; histogram {torch.bincount(pick, minlength=11).tolist()}")
    assert rate >= min_agree
    if not bool(agree.all()):
        idx = (~agree).nonzero().flatten()
        e_mine = err[choice[idx], idx].double()
        e_ref = err[pick[idx], idx].double()
        ok = (e_mine - e_ref).abs() <= e_ref.abs() * ULP[dtype] * 2
        assert bool(ok.all()), (what, idx[~ok][:5].tolist(), e_mine[~ok][:5].tolist(), e_ref[~ok][:5].tolist())
    else:
        assert_bits_equal(got, want, what)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits", [8, 4, 2, 6])
def test_mxint_clip_search_matches_the_oracle(dev, dtype, bits):
    from mase_amd.quantizers import _ops

    x = search_inputs(bits, dtype)
    print(f"mxint clip search {dtype} bits={bits}", flush=True)
    got, choice = _ops.mxint_clip_search(x.to(dev), 32, bits, -1, 8, return_choice=True)
    check_against_oracle(got.cpu(), choice, O.mxint_clip_search(x, 32, bits), dtype, f"mxint{bits} {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("fmt", [(2, 1), (4, 3), (5, 2), (3, 2), (2, 3), (1, 2)])
@pytest.mark.parametrize("scale", [0.05, 10.0])
def test_mxfp_clip_search_matches_the_oracle(dev, dtype, fmt, scale):
    """the larger scale puts the scale bytes into 127..134, the only range where the reference's score tells candidates
    apart (elsewhere every candidate scores sum(x^2) and the first one stays)"""
    from mase_amd.quantizers import _ops

    if scale > 1:
        scale = scale * 2.0 ** ((1 << fmt[0]) - 1 - ((1 << (fmt[0] - 1)) - 1))  # times 2^(largest element exponent)
    x = search_inputs(fmt[0] * 8 + fmt[1], dtype, scale=scale)
    print(f"mxfp clip search {dtype} e{fmt[0]}m{fmt[1]} scale={scale}", flush=True)
    got, choice = _ops.mxfp_clip_search(x.to(dev), 32, fmt[0], fmt[1], -1, 8, return_choice=True)
    ref = O.mxfp_clip_search(x, 32, fmt[0], fmt[1])
    check_against_oracle(got.cpu(), choice, ref, dtype, f"mxfp e{fmt[0]}m{fmt[1]} {dtype} x{scale}")
    if scale > 1 and dtype != torch.float16:
        assert int((ref[1] != 0).sum()) > 50  # the case does exercise the other candidates


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_clip_search_along_the_first_dimension(dev, dtype):
    """block_dim = 0: candidates are blocks along dim 0, the error is taken against the blocks of the plain flattening"""
    from mase_amd.quantizers import _ops

    g = torch.Generator().manual_seed(5)
    x = (torch.randn(64, 48, generator=g) * 0.1).to(dtype)
    got, choice = _ops.mxint_clip_search(x.to(dev), 32, 4, 0, 8, return_choice=True)
    want, pick, err, cand = O.mxint_clip_search(x, 32, 4, 0)
    flat = got.cpu().movedim(0, -1).reshape(-1, 32)
    check_against_oracle(flat, choice, (want.movedim(0, -1).reshape(-1, 32), pick, err, cand), dtype, f"mxint4 dim0 {dtype}")
    got, choice = _ops.mxfp_clip_search((x * 300).to(dev), 32, 2, 1, 0, 8, return_choice=True)
    want, pick, err, cand = O.mxfp_clip_search(x * 300, 32, 2, 1, 0)
    flat = got.cpu().movedim(0, -1).reshape(-1, 32)
    check_against_oracle(flat, choice, (want.movedim(0, -1).reshape(-1, 32), pick, err, cand), dtype, f"mxfp4 dim0 {dtype}")


def test_quantizer_entry_points_take_the_search_branch(dev):
    from mase_amd.quantizers import MXFPMeta, MXIntMeta, mxfp_quantizer, mxfp_quantizer_sim, mxint_quantizer, mxint_quantizer_sim

    x = search_inputs(3, torch.bfloat16)
    xd = x.to(dev)
    got = mxint_quantizer(xd, 32, 4, quantile_search=True)
    plain = mxint_quantizer(xd, 32, 4)
    assert not torch.equal(got, plain)
    assert torch.equal(got, mxint_quantizer_sim(xd, -1, MXIntMeta(block_size=32, scale_bits=8, element_bits=4), quantile_search=True))
    want = O.mxint_quantizer(x, 32, 4, quantile_search=True)
    assert float((got.cpu() == want).float().mean()) > 0.995
    # the searched result is never worse than the plain one by the reference's own measure, block by block
    e_s = (got.float() - xd.float()).reshape(-1, 32).norm(dim=1)
    e_p = (plain.float() - xd.float()).reshape(-1, 32).norm(dim=1)
    assert bool((e_s <= e_p * (1 + 2.0 ** -6)).all())
    big = (x.float() * 800).to(torch.bfloat16)
    got = mxfp_quantizer(big.to(dev), 32, 2, 1, quantile_search=True)
    want = O.mxfp_quantizer(big, 32, 2, 1, quantile_search=True)
    same = (got.cpu() == want) | (got.cpu().isnan() & want.isnan())
    assert float(same.float().mean()) > 0.995
    meta = MXFPMeta(block_size=32, scale_exp_bits=8, element_exp_bits=2, element_frac_bits=1, element_is_finite=True,
                    round_mode="rn")
    assert_bits_equal(mxfp_quantizer_sim(big.to(dev), -1, meta, quantile_search=True), got, "sim entry point")
    with pytest.raises(ValueError):   # calibration activations must be [batches, tokens, block size]
        mxint_quantizer_sim(xd, -1, MXIntMeta(block_size=32, scale_bits=8, element_bits=4), act_tensor=xd, quantile_search=True)
    with pytest.raises(NotImplementedError):
        mxint_quantizer(xd, 8, 4, quantile_search=True)
    # a view that does not start on a 16-byte boundary
    base = torch.randn(4 * 64 + 3, generator=torch.Generator().manual_seed(8)).to(torch.bfloat16)
    view = base[3:].view(4, 64)
    assert_bits_equal(mxint_quantizer(base.to(dev)[3:].view(4, 64), 32, 4, quantile_search=True),
                      O.mxint_quantizer(view, 32, 4, quantile_search=True), "unaligned view")
    # straight-through gradient as for the plain quantizer
    xr = xd.float().clone().requires_grad_(True)
    mxint_quantizer(xr, 32, 4, quantile_search=True).sum().backward()
    assert torch.equal(xr.grad, torch.ones_like(xr))


def test_linear_mxint_clip_search_config(dev):
    """LinearMXInt with config["clip_search"]: the weight is quantized with the search when the state dict is loaded
    (nn/quantized/modules/linear.py:916-954)"""
    from mase_amd.quantized.modules.linear import LinearMXInt

    cfg = {"weight_block_size": 32, "weight_width": 4, "data_in_block_size": 32, "data_in_width": 8,
           "bias_block_size": 32, "bias_width": 8, "clip_search": True}
    g = torch.Generator().manual_seed(2)
    w = torch.randn(64, 128, generator=g) * 0.05
    w[:, ::32] *= 6
    b = torch.randn(64, generator=g)
    m = LinearMXInt(128, 64, bias=True, config=cfg, device=dev, dtype=torch.bfloat16)
    m.load_state_dict({"weight": w.to(torch.bfloat16), "bias": b.to(torch.bfloat16)})
    want_w = O.mxint_quantizer(w.to(torch.bfloat16), 32, 4, 1, quantile_search=True)
    want_b = O.mxint_quantizer(b.to(torch.bfloat16), 32, 8, 0, quantile_search=True)
    assert float((m.weight.detach().cpu() == want_w).float().mean()) > 0.995
    assert float((m.bias.detach().cpu() == want_b).float().mean()) > 0.98
    plain = LinearMXInt(128, 64, bias=True, config={**cfg, "clip_search": False}, device=dev, dtype=torch.bfloat16)
    plain.load_state_dict({"weight": w.to(torch.bfloat16), "bias": b.to(torch.bfloat16)})
    assert not torch.equal(plain.weight, m.weight)
    x = torch.randn(8, 128, generator=g).to(torch.bfloat16).to(dev)
    y = m(x)
    ref = O.linear_mxint_forward(x.cpu(), m.weight.detach().cpu(), m.bias.detach().cpu(), cfg)
    assert float((y.cpu().float() - ref.float()).abs().max() / ref.float().abs().max()) < 1e-2


def test_clip_search_on_a_weight_sized_tensor(dev):
    """131072 blocks of a weight-like bf16 tensor: agreement with the oracle's choice where the summation order of the
    32 squares could matter"""
    from mase_amd.quantizers import _ops

    g = torch.Generator().manual_seed(9)
    x = (torch.randn(1024, 4096, generator=g) * 0.02).to(torch.bfloat16)
    got, choice = _ops.mxint_clip_search(x.to(dev), 32, 4, -1, 8, return_choice=True)
    check_against_oracle(got.cpu(), choice, O.mxint_clip_search(x, 32, 4), torch.bfloat16, "mxint4 bf16 [1024,4096]", 0.9995)
    xf = x.float() * 1000
    got, choice = _ops.mxfp_clip_search(xf.to(dev), 32, 2, 1, -1, 8, return_choice=True)
    check_against_oracle(got.cpu(), choice, O.mxfp_clip_search(xf, 32, 2, 1), torch.float32, "mxfp4 f32 [1024,4096]", 0.9995)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B", [16, 64])
def test_clip_search_block_sizes_16_and_64(dev, dtype, B):
    """the search for the other block sizes the MX formats use: same checks as for 32"""
    from mase_amd.quantizers import _ops

    x = search_inputs(B, dtype, rows=48)
    got, choice = _ops.mxint_clip_search(x.to(dev), B, 4, -1, 8, return_choice=True)
    check_against_oracle(got.cpu(), choice, O.mxint_clip_search(x, B, 4), dtype, f"mxint4 B={B} {dtype}", 0.995)
    xf = search_inputs(B + 1, dtype, rows=48, scale=10.0 * 2.0 ** 2)
    got, choice = _ops.mxfp_clip_search(xf.to(dev), B, 2, 1, -1, 8, return_choice=True)
    check_against_oracle(got.cpu(), choice, O.mxfp_clip_search(xf, B, 2, 1), dtype, f"mxfp4 B={B} {dtype}", 0.995)


def _calibration_case(seed, rows, B, dtype, batches=5, tokens=24):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(rows, B, generator=g) * 0.05
    w[::5] *= torch.exp2(torch.randint(-3, 4, (B,), generator=g).float())
    w[3, 0] *= 40                      # an outlier: clipping it pays when the activations of that column are small
    act = torch.randn(batches, tokens, B, generator=g)
    act[..., 0] *= 0.05
    act[..., 1::7] *= 4
    return w.to(dtype), act.to(dtype)


def _check_calibrated(got, choice, ref, dtype, what, min_agree):
    """the tensor written is the oracle's candidate of the reported index, bit for bit; the index is the oracle's except
    where the two errors (norms of matrix products, whose summation order differs between the library's CPU and GPU
    kernels) agree to within a few steps of the dtype"""
    want, pick, err, cand = ref
    nb = cand.shape[1]
    choice = choice.cpu().long()
    mine = cand[choice, torch.arange(nb)]
    assert_bits_equal(got.cpu().reshape(mine.shape), mine.to(dtype), f"{what}: contents for the reported index")
    agree = choice == pick
    rate = float(agree.double().mean())
    print(f"{what}: same candidate as the oracle in {rate:.4f} of {nb} rows; histogram {torch.bincount(pick, minlength=11).tolist()}")
    assert rate >= min_agree, what
    if not bool(agree.all()) and err.dim() == 2:
        idx = (~agree).nonzero().flatten()
        e_mine, e_ref = err[choice[idx], idx].double(), err[pick[idx], idx].double()
        assert bool(((e_mine - e_ref).abs() <= e_ref.abs() * ULP[dtype] * 16).all()), what


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B", [32, 16, 64])
def test_clip_search_scored_on_calibration_outputs(dev, dtype, B):
    """quantile_search=True with act_tensor (mxint.py:99-131, mxfp.py:65-93) through the quantizer entry points, several
    calibration batches (cali_batch_size smaller than the number of samples)"""
    from mase_amd.quantizers import MXFPMeta, MXIntMeta, _ops, mxfp_quantizer_sim, mxint_quantizer_sim

    w, act = _calibration_case(B, 96, B, dtype)
    got, choice = _ops.mxint_clip_search_calibrated(w.to(dev), B, 4, 1, 8, act.to(dev), 2, return_choice=True)
    ref = O.mxint_clip_search(w, B, 4, 1, act_tensor=act, cali_batch_size=2)
    _check_calibrated(got, choice, ref, dtype, f"mxint4 calibrated B={B} {dtype}", 0.9 if dtype == torch.bfloat16 else 0.97)
    assert int((ref[1] != 0).sum()) > 5       # the calibration data does move choices away from the plain maximum
    plain = O.mxint_clip_search(w, B, 4, 1)
    assert not torch.equal(plain[1], ref[1])  # and away from the search scored on the weights alone
    sim = mxint_quantizer_sim(w.to(dev), 1, MXIntMeta(block_size=B, scale_bits=8, element_bits=4), act_tensor=act.to(dev),
                              quantile_search=True, cali_batch_size=2)
    assert torch.equal(sim, got)
    wf = (w.float() * 500).to(dtype)
    got, choice = _ops.mxfp_clip_search_calibrated(wf.to(dev), B, 2, 1, 1, 8, act.to(dev), 2, return_choice=True)
    ref = O.mxfp_clip_search(wf, B, 2, 1, 1, act_tensor=act, cali_batch_size=2)
    # the strict-replace rule compares each percentile's error with the running best: agreement of the final pick
    want, pick = ref[0], ref[1]
    ch = choice.cpu().long()
    assert_bits_equal(got.cpu().reshape(-1, B), ref[3][ch, torch.arange(ch.numel())].to(dtype), "mxfp calibrated contents")
    rate = float((ch == pick).double().mean())
    print(f"mxfp4 calibrated B={B} {dtype}: same candidate in {rate:.4f}")
    assert rate >= (0.85 if dtype == torch.bfloat16 else 0.95)
    meta = MXFPMeta(block_size=B, scale_exp_bits=8, element_exp_bits=2, element_frac_bits=1, element_is_finite=True, round_mode="rn")
    assert torch.equal(mxfp_quantizer_sim(wf.to(dev), 1, meta, act_tensor=act.to(dev), quantile_search=True, cali_batch_size=2), got)
