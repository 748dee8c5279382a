"""Known-answer vectors of tests/golden/known_answers.json (exact rational arithmetic from the format definitions,
see tests/golden/make_known_answers.py) against the CPU oracle (not gpu) and against the HIP kernels (gpu)."""
import json
import os

import numpy as np
import pytest
import torch

import oracle as O

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "known_answers.json")
with open(PATH) as _f:
    KA = json.load(_f)


def from_bits(b):
    return torch.from_numpy(np.array(b, dtype=np.uint32).view(np.float32).copy())


def check(impl, device):
    n = 0
    for c in KA["integer"]:
        x, want = from_bits(c["x"]).to(device), from_bits(c["y"])
        fn = impl.integer_floor_quantizer if c["floor"] else impl.integer_quantizer
        got = fn(x, c["width"], c["frac_width"]).cpu()
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), ("integer", c["width"], c["frac_width"], c["floor"])
        n += 1
    for c in KA["mxint"]:
        x, want = from_bits(c["x"]).to(device), from_bits(c["y"])
        got = impl.mxint_quantizer(x, c["block_size"], c["element_bits"]).cpu()
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), ("mxint", c["element_bits"])
        n += 1
    for c in KA["block_fp"]:
        x, want = from_bits(c["x"]).to(device), from_bits(c["y"])
        got = impl.block_fp_quantizer(x, width=c["width"], exponent_width=c["exponent_width"], exponent_bias=None,
                                      block_size=[c["block"]], skip_first_dim=False).cpu()
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), ("block_fp", c["width"])
        n += 1
    for c in KA["block_fp_bf16"]:   # bf16 bit patterns; 3-D activation blocking [1, block] as in the headline config
        x = torch.tensor(c["x"], dtype=torch.int32).to(torch.int16).view(torch.bfloat16).reshape(1, 1, -1)
        want = torch.tensor(c["y"], dtype=torch.int32).to(torch.int16)
        for shape, bs, skip in (((1, 1, -1), [1, c["block"]], True), ((-1,), [c["block"]], False)):
            got = impl.block_fp_quantizer(x.reshape(shape).to(device), width=c["width"], exponent_width=c["exponent_width"],
                                          exponent_bias=None, block_size=bs, skip_first_dim=skip).cpu()
            g = got.reshape(-1).view(torch.int16)
            if skip:   # F.fold adds the blocks into a zero buffer there: a -0 result becomes +0
                g = torch.where(got.reshape(-1) == 0, torch.zeros_like(g), g)
                w = torch.where(want.view(torch.bfloat16) == 0, torch.zeros_like(want), want)
            else:
                w = want
            assert torch.equal(g, w), ("block_fp_bf16", c["width"], shape)
        n += 1
    for c in KA["mxfp"]:
        x, want = from_bits(c["x"]).to(device), from_bits(c["y"])
        got = impl.mxfp_quantizer(x, c["block_size"], c["exp_bits"], c["frac_bits"]).cpu()
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), ("mxfp", c["exp_bits"], c["frac_bits"])
        n += 1
    for c in KA["minifloat_mx"]:   # expected values from the value-domain closed form (oracle/scalar.py)
        x, want = from_bits(c["x"]).to(device), from_bits(c["y"])
        if impl is O:
            got = impl.minifloat_quantizer_sim(x, c["exp_bits"], c["frac_bits"], c["is_finite"], c["round_mode"])
        else:
            got = impl.minifloat_quantizer_sim(x, impl.MinifloatMeta(c["exp_bits"], c["frac_bits"], c["is_finite"], c["round_mode"]))
        assert torch.equal(got.cpu().view(torch.int32), want.view(torch.int32)), ("minifloat_mx", c["exp_bits"], c["frac_bits"],
                                                                               c["is_finite"], c["round_mode"])
        n += 1
    return n


def test_oracle_reproduces_the_known_answers():
    assert check(O, "cpu") == 32 + 48


@pytest.mark.gpu
def test_kernels_reproduce_the_known_answers(dev):
    import mase_amd.quantizers as Q

    assert check(Q, dev) == 32 + 48


@pytest.mark.gpu
def test_packed_mxfp_scales_match_the_known_answers(dev):
    """the E8M0 scale byte of mase_mxfp_pack for the formats the matrix instruction has; the vectors avoid block
    maxima that round into the reserved top code only by construction of the check (a +1 scale is accepted
    together with the top code present in the expected values)"""
    from mase_amd._gemm import mxfp_pack

    for c in KA["mxfp"]:
        fmt = (c["exp_bits"], c["frac_bits"])
        if fmt not in ((4, 3), (5, 2), (2, 1)):
            continue
        x = from_bits(c["x"]).to(dev).reshape(1, 32)
        _, scales = mxfp_pack(x, *fmt)
        assert int(scales.cpu()[0, 0]) in (c["scale_byte"], c["scale_byte"] + 1)
