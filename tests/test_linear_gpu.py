"""GPU parity of the quantized Linear modules against the CPU oracle.

Error measure everywhere: max|y - y_ref| / max|y_ref|, bound 1e-2 (the north-star tolerance; the measured
values are printed and are orders of magnitude below it for fp32).  Quantized parameters are compared bit-exactly.
"""
import copy

import pytest
import torch
from torch import nn

import oracle as O
from oracle import linear as OL
from helpers import assert_bits_equal

pytestmark = pytest.mark.gpu
TOL = 1e-2


def rel_err(y, ref):
    return float((y.double().cpu() - ref.double()).abs().max() / ref.double().abs().max())


MXINT_CFG = {"weight_block_size": 32, "weight_width": 8, "data_in_block_size": 32, "data_in_width": 8}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,out_f,bias", [((16, 128), 96, True), ((4, 33, 256), 64, False), ((300, 64), 257, True)])
def test_linear_mxint(dev, dtype, shape, out_f, bias):
    from mase_amd.quantized import LinearMXInt

    g = torch.Generator().manual_seed(2)
    x = torch.randn(*shape, generator=g).to(dtype)
    w = (torch.randn(out_f, shape[-1], generator=g) * 0.02).to(dtype)
    b = torch.randn(out_f, generator=g).to(dtype) if bias else None
    cfg = dict(MXINT_CFG)
    m = LinearMXInt(shape[-1], out_f, bias=bias, device=dev, dtype=dtype, config=copy.deepcopy(cfg))
    sd = {"weight": w} if b is None else {"weight": w, "bias": b}
    res = m.load_state_dict(copy.deepcopy(sd))
    missing, unexpected = res
    assert not missing and not unexpected
    qw, qb = OL.mxint_prepare_weights(w, b, cfg)
    assert_bits_equal(m.weight.data, qw, "LinearMXInt weight after load_state_dict")
    y = m(x.to(dev))
    ref = OL.linear_mxint_forward(x, qw, qb, cfg)
    assert y.shape == ref.shape and y.dtype == ref.dtype
    e = rel_err(y, ref)
    print(f"LinearMXInt {dtype} {shape}->{out_f}: rel err {e:.3e}")
    assert e < (TOL if dtype != torch.float32 else 1e-5)
    assert m._w_cache.get(m.weight) is not None  # the matrix-core path was taken


def test_linear_mxint_config3_full_size(dev):
    """Headline configuration 3: activations [4096,4096] N(0,1), weight [4096,4096] N(0,0.02), bias zeros, fp32."""
    from mase_amd.quantized import LinearMXInt

    g = torch.Generator().manual_seed(2)
    x = torch.randn(4096, 4096, generator=g)
    w = torch.randn(4096, 4096, generator=g) * 0.02
    b = torch.zeros(4096)
    cfg = dict(MXINT_CFG)
    m = LinearMXInt(4096, 4096, bias=True, device=dev, config=dict(cfg))
    m.load_state_dict({"weight": w, "bias": b})
    qw, qb = OL.mxint_prepare_weights(w, b, cfg)
    assert_bits_equal(m.weight.data, qw, "config 3 weight")
    y = m(x.to(dev))
    ref = OL.linear_mxint_forward(x, qw, qb, cfg)
    e = rel_err(y, ref)
    print(f"config 3 rel err {e:.3e}")
    assert e < 1e-5 < TOL


def test_linear_mxint_bias_quantization_bypass_and_fallbacks(dev):
    from mase_amd.quantized import LinearMXInt

    g = torch.Generator().manual_seed(3)
    x = torch.randn(8, 64, generator=g)
    w = torch.randn(32, 64, generator=g)
    b = torch.randn(32, generator=g)
    cfg = {**MXINT_CFG, "bias_block_size": 16, "bias_width": 6}
    m = LinearMXInt(64, 32, device=dev, config=dict(cfg))
    m.load_state_dict({"weight": w, "bias": b})
    qw, qb = OL.mxint_prepare_weights(w, b, cfg)
    assert_bits_equal(m.bias.data, qb, "quantized bias")
    assert rel_err(m(x.to(dev)), OL.linear_mxint_forward(x, qw, qb, cfg)) < 1e-5
    # bypass: a plain linear on untouched weights
    mb = LinearMXInt(64, 32, device=dev, config={**cfg, "bypass": True})
    mb.load_state_dict({"weight": w, "bias": b})
    assert_bits_equal(mb.weight.data, w, "bypass keeps the weight")
    assert rel_err(mb(x.to(dev)), torch.nn.functional.linear(x, w, b)) < 1e-5
    # gptq: weights are not quantized at load; they have no exact bf16 image -> library GEMM on q(x)
    mg = LinearMXInt(64, 32, device=dev, config={**cfg, "gptq": True})
    mg.load_state_dict({"weight": w, "bias": b})
    assert mg._w_cache.get(mg.weight) is None
    assert rel_err(mg(x.to(dev)), torch.nn.functional.linear(O.mxint_quantizer(x, 32, 8), w, b)) < 1e-5
    # no activation config: weights only
    mw = LinearMXInt(64, 32, device=dev, config={"weight_block_size": 32, "weight_width": 8})
    mw.load_state_dict({"weight": w, "bias": b})
    assert rel_err(mw(x.to(dev)), torch.nn.functional.linear(x, qw, b)) < 1e-5
    # a weight modified after loading is picked up (version counter), also when it leaves the MXINT grid
    with torch.no_grad():
        m.weight.mul_(2.0)
    assert rel_err(m(x.to(dev)), OL.linear_mxint_forward(x, qw * 2, qb, cfg)) < 1e-5
    with torch.no_grad():
        m.weight.add_(0.001)
    assert rel_err(m(x.to(dev)), OL.linear_mxint_forward(x, qw * 2 + 0.001, qb, cfg)) < 1e-5
    assert m._w_cache.get(m.weight) is None
    m.weight.data.copy_(qw.to(dev))          # an edit through .data needs an explicit invalidation
    m.invalidate_weight_cache()
    assert rel_err(m(x.to(dev)), OL.linear_mxint_forward(x, qw, qb, cfg)) < 1e-5
    with pytest.raises(AssertionError):
        LinearMXInt(64, 32, device=dev)


HW_MXFP = {(4, 3), (5, 2), (2, 1)}


@pytest.mark.parametrize("native", [True, False])
@pytest.mark.parametrize("wfmt,xfmt", [((2, 1), (4, 3)), ((4, 3), (4, 3)), ((5, 2), (5, 2)), ((2, 1), (5, 2)), ((2, 3), (3, 2)),
                                       ((1, 2), (2, 1))])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_mxfp(dev, dtype, wfmt, xfmt, native):
    from mase_amd.quantized import LinearMXFP

    g = torch.Generator().manual_seed(4)
    x = torch.randn(5, 40, 128, generator=g)
    x[..., 7] *= 20
    x = x.to(dtype)
    w = (torch.randn(96, 128, generator=g) * 0.02).to(dtype)
    cfg = {"weight_block_size": 32, "weight_exponent_width": wfmt[0], "weight_frac_width": wfmt[1],
           "data_in_block_size": 32, "data_in_exponent_width": xfmt[0], "data_in_frac_width": xfmt[1]}
    m = LinearMXFP(128, 96, bias=False, device=dev, dtype=dtype, config=dict(cfg, native_mx=native))
    m.load_state_dict({"weight": w})
    qw, _ = OL.mxfp_prepare_weights(w, None, cfg)
    assert_bits_equal(m.weight.data, qw, "LinearMXFP weight")
    on_matrix_instruction = native and wfmt in HW_MXFP and xfmt in HW_MXFP - {(2, 1)}
    assert m._w_packed.valid_for(m.weight) == on_matrix_instruction
    y = m(x.to(dev))
    ref = OL.linear_mxfp_forward(x, qw, None, cfg)
    e = rel_err(y, ref)
    print(f"LinearMXFP {dtype} w=e{wfmt[0]}m{wfmt[1]} x=e{xfmt[0]}m{xfmt[1]} native={native}: rel err {e:.3e}")
    if dtype != torch.float32:
        assert e < TOL
    elif on_matrix_instruction:
        # the instruction truncates inside groups of 8 products (about 2^-12 of the largest) and blocks whose
        # maximum takes the reserved top code are stored one scale up: both far inside the 1e-2 bound
        assert e < 2e-3
    else:
        assert e < 1e-5


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("wfmt", [(2, 1), (4, 3)])
def test_linear_mxfp_native_path_shapes_bias_and_invalidation(dev, dtype, wfmt):
    """the shape of the MXFP8 x MXFP4 configuration, scaled down: [2, 300, 1024] x [1024 -> 768], with bias"""
    from mase_amd.quantized import LinearMXFP

    g = torch.Generator().manual_seed(9)
    x = torch.randn(2, 300, 1024, generator=g)
    x[..., 100] *= 30
    x = x.to(dtype)
    w = (torch.randn(768, 1024, generator=g) * 0.02).to(dtype)
    b = torch.randn(768, generator=g).to(dtype)
    cfg = {"weight_block_size": 32, "weight_exponent_width": wfmt[0], "weight_frac_width": wfmt[1],
           "data_in_block_size": 32, "data_in_exponent_width": 4, "data_in_frac_width": 3}
    m = LinearMXFP(1024, 768, bias=True, device=dev, dtype=dtype, config=dict(cfg))
    m.load_state_dict({"weight": w, "bias": b})
    assert m._w_packed.valid_for(m.weight)
    qw, qb = OL.mxfp_prepare_weights(w, b, cfg)
    ref = OL.linear_mxfp_forward(x, qw, qb, cfg)
    y = m(x.to(dev))
    assert y.shape == (2, 300, 768) and y.dtype == dtype
    e = rel_err(y, ref)
    print(f"LinearMXFP native {dtype} w=e{wfmt[0]}m{wfmt[1]}: rel err {e:.3e}")
    assert e < (TOL if dtype != torch.float32 else 2e-3)
    if wfmt == (2, 1):
        # 600 rows of e2m1 weights take the kernel that reads tile images; same bits as the row-major kernel
        from mase_amd._gemm import gemm_mxfp_scaled, mxfp_pack

        pk = m._w_packed
        assert pk._tiled is not None and pk._tiled[0] is pk.codes
        xc, xs = mxfp_pack(x.to(dev).reshape(-1, 1024), 4, 3)
        y_rm = gemm_mxfp_scaled(xc, xs, (4, 3), pk.codes, pk.scales, pk.fmt, m.bias.data, dtype)
        assert torch.equal(y.reshape(-1, 768), y_rm)
    # same module with the matrix instruction switched off: the two paths agree to the same bound
    m2 = LinearMXFP(1024, 768, bias=True, device=dev, dtype=dtype, config=dict(cfg, native_mx=False))
    m2.load_state_dict({"weight": w, "bias": b})
    assert rel_err(y, m2(x.to(dev)).cpu()) < (TOL if dtype != torch.float32 else 2e-3)
    # a weight edited after loading no longer matches the packed image: the forward must follow the new weight
    with torch.no_grad():
        m.weight.mul_(2.0)
    assert not m._w_packed.valid_for(m.weight)
    ref2 = OL.linear_mxfp_forward(x, qw * 2, qb, cfg)
    assert rel_err(m(x.to(dev)), ref2) < (TOL if dtype != torch.float32 else 1e-5)
    # empty batch
    assert m(torch.zeros(0, 1024, device=dev, dtype=dtype)).shape == (0, 768)


def test_linear_block_fp_integer_minifloat(dev):
    from mase_amd.quantized import LinearBlockFP, LinearInteger, LinearMinifloatDenorm, LinearMinifloatIEEE

    g = torch.Generator().manual_seed(5)
    x3 = torch.randn(2, 24, 64, generator=g)
    x2 = torch.randn(24, 64, generator=g)
    w = torch.randn(48, 64, generator=g) * 0.1
    b = torch.randn(48, generator=g)
    sd = {"weight": w, "bias": b}
    bfp = {f"{k}_{s}": v for k in ("weight", "data_in", "bias")
           for s, v in (("width", 8), ("exponent_width", 8), ("exponent_bias", None), ("block_size", [16]))}
    m = LinearBlockFP(64, 48, device=dev, config=dict(bfp))
    m.load_state_dict(sd)
    for x in (x3, x2):
        assert rel_err(m(x.to(dev)), OL.linear_block_fp(x, w, b, bfp)) < 1e-5      # grad recorded: library GEMM
        with torch.no_grad():
            assert rel_err(m(x.to(dev)), OL.linear_block_fp(x, w, b, bfp)) < 1e-5  # inference: matrix-core kernel
    # training still works: straight-through quantizers + differentiable GEMM
    xg = x2.to(dev).requires_grad_(True)
    m(xg).sum().backward()
    assert xg.grad is not None and m.weight.grad is not None and bool(torch.isfinite(m.weight.grad).all())
    icfg = {"weight_width": 8, "weight_frac_width": 6, "data_in_width": 8, "data_in_frac_width": 4, "bias_width": 8,
            "bias_frac_width": 5}
    mi = LinearInteger(64, 48, device=dev, config=dict(icfg))
    mi.load_state_dict(sd)
    assert rel_err(mi(x3.to(dev)), OL.linear_integer(x3, w, b, icfg)) < 1e-5
    with torch.no_grad():
        assert rel_err(mi(x3.to(dev)), OL.linear_integer(x3, w, b, icfg)) < 1e-5
    mo = LinearInteger(64, 48, device=dev, config={**icfg, "data_out_width": 8, "data_out_frac_width": 3}, floor=True)
    mo.load_state_dict(sd)
    ref = OL.linear_integer(x3, w, b, {**icfg, "data_out_width": 8, "data_out_frac_width": 3, "floor": True})
    got = mo(x3.to(dev)).cpu()
    # the output re-quantization can flip a value sitting on a rounding boundary by one step of 2^-3
    assert float((got - ref).abs().max()) <= 0.125 and float(((got - ref) != 0).float().mean()) < 1e-3
    mcfg = {f"{k}_{s}": v for k in ("weight", "data_in", "bias") for s, v in (("width", 8), ("exponent_width", 4), ("exponent_bias", None))}
    for cls, fn in ((LinearMinifloatDenorm, OL.linear_minifloat_denorm), (LinearMinifloatIEEE, OL.linear_minifloat_ieee)):
        mm = cls(64, 48, device=dev, config=dict(mcfg))
        mm.load_state_dict(sd)
        assert rel_err(mm(x3.to(dev)), fn(x3, w, b, mcfg)) < 1e-5
        with torch.no_grad():
            assert rel_err(mm(x3.to(dev)), fn(x3, w, b, mcfg)) < 1e-5


def test_linear_block_fp_integer_wide_formats_take_the_library_gemm(dev):
    """widths beyond 9 bits are not exact in bf16: the forward must still match (library GEMM in the tensor dtype),
    and the narrow formats must match in bf16 and fp16 tensors too"""
    from mase_amd.quantized import LinearBlockFP, LinearInteger

    g = torch.Generator().manual_seed(6)
    x = torch.randn(3, 40, 128, generator=g)
    w = torch.randn(72, 128, generator=g) * 0.1
    b = torch.randn(72, generator=g)
    for width, tol in ((12, 1e-5), (8, 1e-5)):
        bfp = {f"{k}_{s}": v for k in ("weight", "data_in", "bias")
               for s, v in (("width", width), ("exponent_width", 8), ("exponent_bias", None), ("block_size", [16]))}
        m = LinearBlockFP(128, 72, device=dev, config=dict(bfp)).requires_grad_(False)
        m.load_state_dict({"weight": w, "bias": b})
        assert rel_err(m(x.to(dev)), OL.linear_block_fp(x, w, b, bfp)) < tol
        icfg = {"weight_width": width, "weight_frac_width": width - 2, "data_in_width": width, "data_in_frac_width": width - 4,
                "bias_width": width, "bias_frac_width": width - 3}
        mi = LinearInteger(128, 72, device=dev, config=dict(icfg)).requires_grad_(False)
        mi.load_state_dict({"weight": w, "bias": b})
        assert rel_err(mi(x.to(dev)), OL.linear_integer(x, w, b, icfg)) < tol
    for dtype in (torch.bfloat16, torch.float16):
        bfp = {f"{k}_{s}": v for k in ("weight", "data_in", "bias")
               for s, v in (("width", 8), ("exponent_width", 8), ("exponent_bias", None), ("block_size", [16]))}
        m = LinearBlockFP(128, 72, device=dev, dtype=dtype, config=dict(bfp)).requires_grad_(False)
        m.load_state_dict({"weight": w.to(dtype), "bias": b.to(dtype)})
        e = rel_err(m(x.to(dtype).to(dev)), OL.linear_block_fp(x.to(dtype), w.to(dtype), b.to(dtype), bfp))
        print(f"LinearBlockFP {dtype}: rel err {e:.3e}")
        assert e < TOL


class MLP(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc1 = nn.Linear(64, 128)
        self.act = nn.ReLU()
        self.fc2 = nn.Linear(128, 32, bias=False)
        self.head = nn.ModuleDict({"out": nn.Linear(32, 32)})

    def forward(self, x):
        return self.head["out"](self.fc2(self.act(self.fc1(x))))


def test_quantize_module_transform_pass(dev):
    from mase_amd.passes import quantize_module_transform_pass
    from mase_amd.quantized import LinearInteger, LinearMXInt, quantized_module_map

    torch.manual_seed(0)
    net = MLP().to(dev)
    ref_net = copy.deepcopy(net).cpu()
    x = torch.randn(16, 64)
    pass_args = {"by": "type", "linear": {"config": {"name": "mxint", **MXINT_CFG}}}
    out, info = quantize_module_transform_pass(net, pass_args)
    assert info == {} and out is net
    assert "by" not in pass_args and "name" not in pass_args["linear"]["config"]  # popped like the reference does
    assert all(isinstance(m, LinearMXInt) for m in (net.fc1, net.fc2, net.head["out"]))
    assert net.fc2.bias is None and net.fc1.config is pass_args["linear"]["config"]
    h = x
    for lin, act in ((ref_net.fc1, True), (ref_net.fc2, False), (ref_net.head["out"], False)):
        qw, qb = OL.mxint_prepare_weights(lin.weight.data, lin.bias.data if lin.bias is not None else None, MXINT_CFG)
        h = OL.linear_mxint_forward(h, qw, qb, MXINT_CFG)
        h = torch.relu(h) if act else h
    assert rel_err(net(x.to(dev)), h) < 1e-4
    # by name and by regex
    net2 = MLP().to(dev)
    quantize_module_transform_pass(net2, {"by": "name", "fc1": {"config": {"name": "integer", "weight_width": 8,
        "weight_frac_width": 4, "data_in_width": 8, "data_in_frac_width": 4, "bias_width": 8, "bias_frac_width": 4}}})
    assert isinstance(net2.fc1, LinearInteger) and type(net2.fc2) is nn.Linear
    net3 = MLP().to(dev)
    quantize_module_transform_pass(net3, {"by": "regex_name", r"head\.\w+": {"config": {"name": "mxint", **MXINT_CFG}}})
    assert isinstance(net3.head["out"], LinearMXInt) and type(net3.fc1) is nn.Linear
    with pytest.raises(ValueError):
        quantize_module_transform_pass(MLP().to(dev), {"by": "type", "default": {"config": {"name": None}}})
    with pytest.raises(ValueError):
        quantize_module_transform_pass(MLP().to(dev), {"by": "layer"})
    assert set(quantized_module_map) >= {"linear_mxint", "linear_mxfp", "linear_block_fp", "linear_integer",
                                         "linear_fixed", "linear_minifloat_ieee", "linear_minifloat_denorm"}


def test_quantized_parameter_cache_modes(dev):
    """LinearBlockFP / Integer / Minifloat*.  Default (the reference's behaviour): weight and bias are quantized on
    every forward, so an edit made through ``weight.data`` (which no version counter sees) is picked up.  With
    ``cache_quantized_params=True`` the module keeps the quantized weight and bias (and the weight's bf16 and
    fragment-ordered copies) between forwards under no_grad: the same results, a versioned in-place update is picked
    up, an edit through ``.data`` is served from the old parameters until ``invalidate_weight_cache()``."""
    import mase_amd.quantized.functional.linear as FL
    from mase_amd.quantized import LinearBlockFP, LinearInteger, LinearMinifloatDenorm, LinearMinifloatIEEE

    g = torch.Generator().manual_seed(6)
    bfp = {f"{k}_{s}": v for k in ("weight", "data_in", "bias")
           for s, v in (("width", 8), ("exponent_width", 8), ("exponent_bias", None), ("block_size", [16]))}
    icfg = {"weight_width": 8, "weight_frac_width": 6, "data_in_width": 8, "data_in_frac_width": 4, "bias_width": 8,
            "bias_frac_width": 5}
    mcfg = {f"{k}_{s}": v for k in ("weight", "data_in", "bias") for s, v in (("width", 8), ("exponent_width", 4), ("exponent_bias", None))}
    cases = [(LinearBlockFP, FL.linearBlockFP, bfp), (LinearInteger, FL.linearInteger, icfg),
             (LinearMinifloatDenorm, FL.linearMinifloatDenorm, mcfg), (LinearMinifloatIEEE, FL.linearMinifloatIEEE, mcfg)]
    for dtype in (torch.float32, torch.bfloat16):
        for cls, fn, cfg in cases:
            for cached in (False, True):
                mc = dict(cfg, cache_quantized_params=True) if cached else dict(cfg)
                m = cls(256, 512, device=dev, dtype=dtype, config=mc)
                m.load_state_dict({"weight": (torch.randn(512, 256, generator=g) * 0.1).to(dtype), "bias": torch.randn(512, generator=g).to(dtype)})
                for rows in (8, 300, 4096):  # weight-streaming kernel, K-range form, tiled kernel
                    x = torch.randn(rows, 256, generator=g).to(dtype).to(dev)
                    with torch.no_grad():
                        want = fn(x, m.weight, m.bias, dict(cfg))
                        assert torch.equal(m(x), want) and torch.equal(m(x), want), (cls.__name__, dtype, rows, cached)
                if cached:
                    assert m._param_cache.qw is not None and m._param_cache.packed() is not None
                else:
                    assert m._param_cache.qw is None
                with torch.no_grad():
                    m.weight.mul_(0.5)
                    want = fn(x, m.weight, m.bias, dict(cfg))
                    assert torch.equal(m(x), want), (cls.__name__, "after an in-place update", cached)
                    m.weight.data.add_(0.25)           # an edit the version counter does not see
                    fresh = fn(x, m.weight, m.bias, dict(cfg))
                    assert not torch.equal(fresh, want)
                    if cached:
                        assert torch.equal(m(x), want), "the opt-in cache serves the parameters it was built from"
                        m.invalidate_weight_cache()
                    assert torch.equal(m(x), fresh), (cls.__name__, "after an edit through .data", cached)
                y = m(x[:4].clone().requires_grad_(True))  # gradients recorded: nothing cached is used, autograd works
                y.sum().backward()
                assert m.weight.grad is not None


def test_mx_linears_under_inference_mode(dev):
    """activations (and parameters) made under torch.inference_mode() carry no version counter; the forwards must not
    depend on one: same results as under no_grad"""
    from mase_amd.quantized import LinearMXFP, LinearMXInt
    from mase_amd.workloads import DecoderLayer, DecoderLayerConfig
    from mase_amd.passes import quantize_module_transform_pass

    g = torch.Generator().manual_seed(16)
    fcfg = {"weight_block_size": 32, "weight_exponent_width": 2, "weight_frac_width": 1,
            "data_in_block_size": 32, "data_in_exponent_width": 4, "data_in_frac_width": 3}
    w = torch.randn(512, 256, generator=g) * 0.05
    for cls, cfg in ((LinearMXInt, MXINT_CFG), (LinearMXFP, fcfg), (LinearMXFP, dict(fcfg, native_mx=False))):
        for dtype in (torch.float32, torch.bfloat16):
            m = cls(256, 512, bias=False, device=dev, dtype=dtype, config=dict(cfg))
            m.load_state_dict({"weight": w.to(dtype)})
            for rows in (8, 600):
                x = torch.randn(rows, 256, generator=g).to(dtype).to(dev)
                with torch.no_grad():
                    want = m(x)
                with torch.inference_mode():
                    xi = x * 1.0                   # an inference tensor
                    assert xi.is_inference()
                    got = m(xi)
                    got2 = m(xi)
                assert torch.equal(got, want) and torch.equal(got2, want), (cls.__name__, dtype, rows)
    # a module whose parameters are inference tensors themselves
    with torch.inference_mode():
        mi = LinearMXInt(256, 512, bias=False, device=dev, config=dict(MXINT_CFG))
        mi.load_state_dict({"weight": w})
        assert mi.weight.is_inference()
        x = torch.randn(300, 256, generator=g).to(dev)
        got = mi(x)
    m = LinearMXInt(256, 512, bias=False, device=dev, config=dict(MXINT_CFG))
    m.load_state_dict({"weight": w})
    assert torch.equal(got, m(x))
    # the decoder layer with its shared projections
    cfg = DecoderLayerConfig(hidden_size=256, num_heads=4, head_dim=64, intermediate_size=512)
    layer = DecoderLayer(cfg, device=dev, dtype=torch.bfloat16, seed=3)
    layer, _ = quantize_module_transform_pass(layer, {"by": "type", "linear": {"config": dict(MXINT_CFG, name="mxint")}})
    x = torch.randn(2, 160, 256, generator=g).bfloat16().to(dev)
    with torch.no_grad():
        want = layer(x)
    with torch.inference_mode():
        got = layer(x * 1.0)
    assert torch.equal(got, want)


def test_sibling_projections_share_one_quantized_activation(dev):
    """project_shared(x, modules) == [m(x) for m in modules], bit for bit, for every path an MX Linear can take, for
    modules that quantize differently (each gets its own copy) and for plain nn.Linear; nothing is kept afterwards, so
    an in-place change of x between two calls is seen"""
    from mase_amd.quantized import LinearMXFP, LinearMXInt
    from mase_amd.quantized.functional.mx_linear import project_shared

    g = torch.Generator().manual_seed(17)
    fcfg = {"weight_block_size": 32, "weight_exponent_width": 2, "weight_frac_width": 1,
            "data_in_block_size": 32, "data_in_exponent_width": 4, "data_in_frac_width": 3}

    def make(cls, cfg, n_out, dtype):
        m = cls(256, n_out, bias=False, device=dev, dtype=dtype, config=dict(cfg))
        m.load_state_dict({"weight": (torch.randn(n_out, 256, generator=g) * 0.05).to(dtype)})
        return m

    for dtype in (torch.float32, torch.bfloat16):
        mods = [make(LinearMXInt, MXINT_CFG, 512, dtype), make(LinearMXInt, MXINT_CFG, 128, dtype),
                make(LinearMXInt, dict(MXINT_CFG, data_in_width=6), 256, dtype),
                make(LinearMXInt, dict(MXINT_CFG, packed_decode=True), 256, dtype),
                make(LinearMXFP, fcfg, 512, dtype), make(LinearMXFP, fcfg, 256, dtype),
                make(LinearMXFP, dict(fcfg, native_mx=False), 256, dtype),
                make(LinearMXInt, dict(MXINT_CFG, bypass=True), 64, dtype),
                torch.nn.Linear(256, 64, bias=False, device=dev, dtype=dtype)]
        for rows in (4, 200, 1500):
            x = torch.randn(2, rows // 2, 256, generator=g).to(dtype).to(dev)
            with torch.no_grad():
                want = [m(x) for m in mods]
                got = project_shared(x, mods)
                for a, b, m in zip(got, want, mods):
                    assert torch.equal(a, b), (type(m).__name__, dtype, rows)
                x.data.mul_(1.5)  # unseen by any version counter
                want2 = [m(x) for m in mods]
                for a, b, m in zip(project_shared(x, mods), want2, mods):
                    assert torch.equal(a, b), (type(m).__name__, dtype, rows, "after an edit of x")
                assert not torch.equal(want2[0], want[0])


def test_linear_mxint_from_codes(dev):
    """config["weight_memory"] = "codes": forwards of more than 128 rows run from the fragment-ordered MXINT8 code image
    (widened to bf16 in registers); results are those of the default module bit for bit, neither the bf16 image nor its
    fragment-ordered copy gets built, and a changed weight falls back to the reference's F.linear on the new values"""
    from mase_amd.quantized import LinearMXInt

    g = torch.Generator().manual_seed(21)
    w = torch.randn(512, 256, generator=g) * 0.05
    w[::5] *= torch.exp2(torch.randint(-5, 6, (256,), generator=g).float())
    b = torch.randn(512, generator=g)
    for dtype in (torch.float32, torch.bfloat16):
        for extra in ({}, {"packed_decode": True}):
            ref = LinearMXInt(256, 512, device=dev, dtype=dtype, config=dict(MXINT_CFG))
            m = LinearMXInt(256, 512, device=dev, dtype=dtype, config=dict(MXINT_CFG, weight_memory="codes", **extra))
            for mod in (ref, m):
                mod.load_state_dict({"weight": w.to(dtype), "bias": b.to(dtype)})
            assert torch.equal(m.weight, ref.weight)
            assert m._w_image.valid_for(m.weight) and m._w_codes.valid_for(m.weight) == bool(extra)
            assert m._w_image.codes.numel() == 512 * 256 and m._w_image.scales.numel() == 512 * 8
            for rows in (300, 1500, 4096):
                x = torch.randn(rows, 256, generator=g).to(dtype).to(dev)
                got, want = m(x), ref(x)
                if rows == 300:   # the default module cuts K into ranges for a few hundred rows: another summation order
                    assert rel_err(got, want.cpu()) < (1e-5 if dtype == torch.float32 else 1e-2)
                else:
                    assert torch.equal(got, want), (dtype, rows)
            assert m._w_cache._w is None and m._w_cache._packed is None, "the bf16 images must not have been built"
            x8 = torch.randn(8, 256, generator=g).to(dtype).to(dev)
            assert rel_err(m(x8), ref(x8).cpu()) < (1e-5 if dtype == torch.float32 else 1e-2)
            with torch.no_grad():
                m.weight.mul_(0.5)     # no longer the tensor the codes were made for
                ref.weight.mul_(0.5)
            x = torch.randn(600, 256, generator=g).to(dtype).to(dev)
            assert not m._w_image.valid_for(m.weight)
            assert rel_err(m(x), ref(x).cpu()) < (1e-5 if dtype == torch.float32 else 1e-2)
    # a packed checkpoint hands the codes over: the image is built from them
    from mase_amd.quantized.packed import load_packed_state_dict, packed_state_dict

    src = LinearMXInt(256, 512, device=dev, dtype=torch.bfloat16, config=dict(MXINT_CFG))
    src.load_state_dict({"weight": w.bfloat16(), "bias": b.bfloat16()})
    dst = LinearMXInt(256, 512, device=dev, dtype=torch.bfloat16, config=dict(MXINT_CFG, weight_memory="codes"))
    holder_src, holder_dst = nn.Sequential(src), nn.Sequential(dst)
    packed = packed_state_dict(holder_src, {"0.weight": w.bfloat16()})   # codes of the weights the model was quantized from
    assert "0.weight.mx_codes" in packed
    load_packed_state_dict(holder_dst, packed)
    assert dst._w_image.valid_for(dst.weight)
    x = torch.randn(2048, 256, generator=g).bfloat16().to(dev)
    assert torch.equal(dst(x), src(x))
