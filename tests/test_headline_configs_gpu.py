"""Parity at the headline configurations' full sizes, on the same seeded inputs the benchmark uses.

Configurations 1 and 2 (quantize-dequantize) are compared bit for bit with the CPU oracle over the whole tensor.
Configuration 3 (MXINT8 Linear 4096^3) is compared with the oracle's forward within 1e-2 (measured ~1e-6).
Configuration 4 (MXFP8 x MXFP4 Linear, M=8192 K=8192 N=28672) is too large for the CPU oracle to finish in seconds,
so it is checked on a slice that is: the first 256 activation rows against the first 2048 weight rows, taken from
the full-size operands (rows are independent in both quantizers and in the product), plus size-independent
properties of the full-size result (finite, row slices agree with the sliced computation)."""
import pytest
import torch

import bench
import oracle as O
from oracle import linear as OL
from helpers import assert_bits_equal

pytestmark = pytest.mark.gpu


def rel_err(y, ref):
    return float((y.double().cpu() - ref.double()).abs().max() / ref.double().abs().max())


def test_config1_mxint_qdq_full_size_bit_exact(dev):
    import mase_amd.quantizers as Q

    x = bench.make_mxint_input(torch)
    assert x.shape == (4096, 4096) and x.dtype == torch.float32
    assert_bits_equal(Q.mxint_quantizer(x.to(dev), 32, 8), O.mxint_quantizer(x, 32, 8), "config 1")


def test_config2_block_fp_qdq_full_size_bit_exact(dev):
    import mase_amd.quantizers as Q

    x = bench.make_bfp_input(torch)
    assert x.shape == (8, 2048, 4096) and x.dtype == torch.bfloat16
    kw = bench.BfpQdq.kw
    got = Q.block_fp_quantizer(x.to(dev), **kw)
    want = O.block_fp_quantizer(x.clone(), **kw)
    assert_bits_equal(got, want, "config 2")
    # size-independent property: every output block of 16 holds multiples of one power of two (its grid step)
    blk = got.float().reshape(-1, 16)
    step = torch.exp2(torch.floor(torch.log2(blk.abs().amax(1, keepdim=True).clamp_min(1e-30))) - 6)
    sample = slice(0, 1 << 16)
    assert bool(((blk[sample] / step[sample]) == (blk[sample] / step[sample]).round()).all())


def test_config3_mxint_linear_full_size(dev):
    from mase_amd.quantized import LinearMXInt

    w = bench.MxintLinear()
    x, wt, b = w.make(torch)
    m = LinearMXInt(w.K, w.N, bias=True, device=dev, config=dict(w.cfg))
    m.load_state_dict({"weight": wt, "bias": b})
    qw, qb = OL.mxint_prepare_weights(wt, b, w.cfg)
    assert_bits_equal(m.weight.data, qw, "config 3 weight")
    e = rel_err(m(x.to(dev)), OL.linear_mxint_forward(x, qw, qb, w.cfg))
    print(f"config 3 (4096^3) rel err {e:.3e}")
    assert e < 1e-2


def test_config4_mxfp_linear_full_size_slices(dev):
    from mase_amd.quantized import LinearMXFP

    w = bench.MxfpLinear()
    x = w.make_x(torch, w.M)
    wt = w.make_w(torch, w.N)
    m = LinearMXFP(w.K, w.N, bias=False, device=dev, dtype=torch.bfloat16, config=dict(w.cfg))
    m.load_state_dict({"weight": wt})
    assert m._w_packed.valid_for(m.weight)
    y = m(x.to(dev))
    assert y.shape == (w.M, w.N) and bool(torch.isfinite(y).all())
    # slice: rows are independent, so the oracle on the slice is the oracle on the full problem restricted to it
    ms, ns = 256, 2048
    for r0, c0 in ((0, 0), (w.M - ms, w.N - ns)):
        qw, _ = OL.mxfp_prepare_weights(wt[c0:c0 + ns], None, w.cfg)
        ref = OL.linear_mxfp_forward(x[r0:r0 + ms], qw, None, w.cfg)
        e = rel_err(y[r0:r0 + ms, c0:c0 + ns], ref)
        print(f"config 4 slice rows {r0}.. cols {c0}..: rel err {e:.3e}")
        assert e < 1e-2
    # quantized weight slice bit-exact
    assert_bits_equal(m.weight.data[:ns], OL.mxfp_prepare_weights(wt[:ns], None, w.cfg)[0], "config 4 weight slice")
