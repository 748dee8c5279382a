"""Packed MX checkpoints: codes + scales written by the quantizers, dequantized by mase_mx_unpack.  The unpacked
weight must equal the oracle's quantized weight bit for bit, and a model loaded from a packed file must compute
exactly what the model it was written from computes."""
import os

import pytest
import torch

import oracle as O
from helpers import assert_bits_equal

pytestmark = pytest.mark.gpu


def assert_same_but_zero_sign(got, want, what):
    """bit-identical except that a -0.0 of ``want`` may be +0.0 in ``got`` (integer codes have no negative zero)"""
    got, want = got.cpu(), want.cpu()
    assert_bits_equal(torch.where(want == 0, torch.zeros_like(got), got), torch.where(want == 0, torch.zeros_like(want), want), what)
    assert bool((got[want == 0] == 0).all()), what

MXINT = {"weight_block_size": 32, "weight_width": 8, "data_in_block_size": 32, "data_in_width": 8}
MXFP4 = {"weight_block_size": 32, "weight_exponent_width": 2, "weight_frac_width": 1,
         "data_in_block_size": 32, "data_in_exponent_width": 4, "data_in_frac_width": 3}
MXFP8 = {"weight_block_size": 32, "weight_exponent_width": 4, "weight_frac_width": 3,
         "data_in_block_size": 32, "data_in_exponent_width": 4, "data_in_frac_width": 3}


def _weights(dtype, rows=96, cols=256, seed=0):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(rows, cols, generator=g) * 0.05
    w[3, :32] = 0.0                       # an all-zero block
    w[5, 40] = 3.0                        # an outlier
    w[7, 64:96] = torch.linspace(-1, 1, 32) * 2.0 ** -20
    w[9, 0] = 0.5                         # block maximum exactly a power of two
    return w.to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_unpack_reproduces_the_quantized_tensor(dev, dtype):
    from mase_amd.quantized.packed import pack_weight, unpack_weight

    w = _weights(dtype)
    for bits, block in ((8, 32), (8, 16), (4, 32), (6, 64)):
        deq, codes, scales = pack_weight(w.to(dev), "mxint", block, bits)
        assert codes.shape == w.shape and scales.shape == (w.shape[0], w.shape[1] // block) and codes.dtype == torch.int8
        want = O.mxint_quantizer(w, block, bits, block_dim=1)
        assert_bits_equal(deq, want, f"mxint{bits} q-dq")
        assert_same_but_zero_sign(unpack_weight(codes, scales, "mxint", block, bits, 0, dtype), want, f"mxint{bits} unpack {dtype}")
    for e, f in ((4, 3), (5, 2), (2, 1), (2, 3), (3, 2)):
        deq, codes, scales = pack_weight(w.to(dev), "mxfp", 32, e, f)
        want = O.mxfp_quantizer(w, 32, e, f, block_dim=1)
        assert_bits_equal(deq, want, f"mxfp e{e}m{f} q-dq")
        assert_bits_equal(unpack_weight(codes, scales, "mxfp", 32, e, f, dtype), want, f"mxfp e{e}m{f} unpack {dtype}")
    # block sizes that are not multiples of 16 take the element-wise kernel
    deq, codes, scales = pack_weight(w[:, :40].contiguous().to(dev), "mxint", 8, 8)
    assert_same_but_zero_sign(unpack_weight(codes, scales, "mxint", 8, 8, 0, dtype),
                              O.mxint_quantizer(w[:, :40].contiguous(), 8, 8, block_dim=1), "block 8")


class Net(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.a = torch.nn.Linear(256, 384, bias=True)
        self.b = torch.nn.Linear(384, 128, bias=False)
        self.c = torch.nn.Linear(128, 64, bias=False)
        self.norm = torch.nn.LayerNorm(64)

    def forward(self, x):
        return self.norm(self.c(torch.relu(self.b(torch.relu(self.a(x))))))


def _quantized_net(dev, dtype, seed):
    from mase_amd.passes import quantize_module_transform_pass

    torch.manual_seed(seed)
    net = Net().to(device=dev, dtype=dtype)
    float_sd = {k: v.detach().clone() for k, v in net.state_dict().items()}
    args = {"by": "name", "a": {"config": {"name": "mxint", **MXINT}}, "b": {"config": {"name": "mxfp", **MXFP4}},
            "c": {"config": {"name": "mxfp", **MXFP8}}}
    net, _ = quantize_module_transform_pass(net, args)
    return net.eval(), float_sd


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_round_trip_through_a_packed_file(dev, dtype, tmp_path):
    from mase_amd.quantized.packed import load_packed, packed_state_dict, save_packed, unpacked_state_dict

    net, float_sd = _quantized_net(dev, dtype, 1)
    x = torch.randn(4, 32, 256, device=dev, dtype=dtype)
    with torch.no_grad():
        y0 = net(x)
    path = str(tmp_path / "model.packed.pt")
    save_packed(net, path, float_state_dict=float_sd)
    packed = torch.load(path, weights_only=True)
    for name in ("a", "b", "c"):
        assert f"{name}.weight" not in packed and packed[f"{name}.weight.mx_codes"].shape == getattr(net, name).weight.shape
    assert "a.bias" in packed and "norm.weight" in packed
    plain = str(tmp_path / "model.pt")
    torch.save({k: v.cpu() for k, v in net.state_dict().items()}, plain)
    ratio = os.path.getsize(path) / os.path.getsize(plain)
    assert ratio < (0.30 if dtype == torch.float32 else 0.56), ratio  # 8.25 bits against 32 / 16 per weight

    # a fresh model with other weights, same modules: load the packed file, nothing is re-quantized
    net2, _ = _quantized_net(dev, dtype, 2)
    missing, unexpected = load_packed(net2, path)
    assert not missing and not unexpected
    for k, v in net.state_dict().items():
        (assert_same_but_zero_sign if k == "a.weight" else assert_bits_equal)(net2.state_dict()[k], v.cpu(), k)
    assert net2.b._w_packed.valid_for(net2.b.weight) and net2.c._w_packed.valid_for(net2.c.weight)
    with torch.no_grad():
        y1 = net2(x)
    assert torch.equal(y1, y0), "forward after packed load"
    # the unpacked dict is the plain one
    up = unpacked_state_dict(packed_state_dict(net, float_sd))
    assert set(up) == set(net.state_dict())

    # without the original weights the codes come from re-quantizing: whatever is packed still round-trips exactly
    again = unpacked_state_dict(packed_state_dict(net))
    for k, v in net.state_dict().items():
        assert torch.equal(again[k], v), k + " (repacked)"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_mxint_streams_codes_for_decode_sized_batches(dev, dtype, tmp_path):
    """config["packed_decode"]: forwards of at most 128 rows contract against the int8 codes + scale bytes (the same
    bf16 operand values, another summation order); larger batches take the bf16 image as before.  A packed checkpoint
    hands the codes over as well."""
    from mase_amd.quantized import LinearMXInt
    from mase_amd.quantized.packed import load_packed_state_dict, packed_state_dict
    from oracle import linear as OL

    g = torch.Generator().manual_seed(9)
    w = (torch.randn(384, 512, generator=g) * 0.05).to(dtype)
    b = torch.randn(384, generator=g).to(dtype)
    plain = LinearMXInt(512, 384, device=dev, dtype=dtype, config=dict(MXINT))
    plain.load_state_dict({"weight": w, "bias": b})
    packed = LinearMXInt(512, 384, device=dev, dtype=dtype, config={**MXINT, "packed_decode": True})
    packed.load_state_dict({"weight": w, "bias": b})
    assert packed._w_codes.valid_for(packed.weight) and not plain._w_codes.valid_for(plain.weight)
    assert torch.equal(packed.weight, plain.weight)                     # the same quantized weight either way
    qw, qb = OL.mxint_prepare_weights(w, b, MXINT)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    for rows in (1, 5, 128, 129, 300):
        x = torch.randn(rows, 512, generator=g).to(dtype)
        y = packed(x.to(dev))
        ref = OL.linear_mxint_forward(x, qw, qb, MXINT)
        err = float((y.double().cpu() - ref.double()).abs().max() / ref.double().abs().max())
        assert err < tol, (rows, err)
        y0 = plain(x.to(dev))
        assert float((y.double() - y0.double()).abs().max() / y0.double().abs().max()) < (2e-6 if dtype == torch.float32 else 8e-3)
    x3 = torch.randn(2, 3, 512, generator=g).to(dtype)                  # leading dimensions
    assert packed(x3.to(dev)).shape == (2, 3, 384)
    # an edited weight invalidates the codes: the forward goes back to the parameter
    with torch.no_grad():
        packed.weight.mul_(0.0)
    assert not packed._w_codes.valid_for(packed.weight)
    assert float(packed(x3.to(dev)).sub(packed.bias).abs().max()) == 0.0
    # codes arriving through a packed state dict
    class Net(torch.nn.Module):
        def __init__(self, lin):
            super().__init__()
            self.lin = lin
    sd = packed_state_dict(Net(plain), float_state_dict={"lin.weight": w.to(dev), "lin.bias": b.to(dev)})
    assert "lin.weight.mx_codes" in sd
    fresh = Net(LinearMXInt(512, 384, device=dev, dtype=dtype, config=dict(MXINT)))
    load_packed_state_dict(fresh, sd)
    assert fresh.lin._w_codes.valid_for(fresh.lin.weight)
    x = torch.randn(4, 512, generator=g).to(dtype).to(dev)
    again = LinearMXInt(512, 384, device=dev, dtype=dtype, config={**MXINT, "packed_decode": True})
    again.load_state_dict({"weight": w, "bias": b})
    assert torch.equal(fresh.lin._w_codes.codes, again._w_codes.codes)   # the codes of the original weights both ways
    assert torch.equal(fresh.lin(x), again(x))
