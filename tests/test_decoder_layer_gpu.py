"""The decoder-layer workload: every nn.Linear replaced by LinearMXInt through the quantize pass, compared with the
same layer on the CPU whose Linears compute the reference's forward (oracle restatement) and whose attention core is
the reference's (``oracle.llama.eager_causal_attention``: scores in bf16, fp32 softmax, probabilities in bf16).

Error measure: max|y - y_ref| / max|y_ref| on the layer output, bound 1e-2.

What the measure can resolve at the real widths (hidden 4096, FFN 11008).  With the reference's attention result handed
to it, the GPU layer is BIT-IDENTICAL to the CPU layer (comparison (b) below measures 0.0 at every shape): RMSNorm,
rotary embedding, SwiGLU and all seven Linears reproduce the CPU's bits.  What is left is the attention core, and there
the measure is discontinuous: every Linear quantizes its input to MXINT8, so a change of ONE bf16 step in one element of
the attention result flips a code of o_proj's input with probability ~1/4, which moves that token's 4096 o_proj
outputs, hundreds of them across a bf16 rounding boundary, then dozens of gate / up input codes, about half of that
token's 11008 gate / up outputs by one step, a quarter of down_proj's input codes, and its output by ~0.06 of a range
of ~6.  Measured on the CPU alone (``tests/test_layer_sensitivity.py``): flipping the last bit of 0.1 % of the
reference's attention result moves the reference layer's output by 1.1e-2, of 0.02 % by 8e-3; the reference's
attention against the same function evaluated exactly (fp32 throughout) gives 1.8e-2 to 2.0e-2.  No attention kernel
whose fp32 sums run in another order than the CPU's can stay below the bound at these widths: the layer-level error is
either zero or that of a re-drawn quantization noise (1e-2 to 2e-2).  Hence:

 (a) every GPU Linear on the exact input its CPU counterpart saw: bit-identical outputs;
 (b) the GPU layer with the attention core's result computed by the reference's attention (on the CPU) from the GPU's
     q, k, v: everything but the attention core, free running: bound 1e-2, measured 0.0;
 (c) the default path (the attention kernel of this package where the shape allows: a multiple of 128 tokens; the
     library's kernel otherwise): bound 1e-2 where it holds (hidden 1024: 6e-3); at the real widths below 1.5 x the
     distance between the reference's attention and its exact evaluation, with an absolute cap of 2.5e-2 (measured
     1.9e-2 against 1.8e-2 to 2.0e-2).  The attention kernel itself is held to 1e-2 of its output range against fp32
     tensor operations in ``test_layer_ops_gpu.py`` and, at 2048 tokens inside the layer, in
     ``test_headline_configs_gpu.py``.  The numbers are printed."""
import copy

import pytest
import torch
from torch import nn

from oracle import linear as OL
from oracle import llama as OLL

pytestmark = pytest.mark.gpu

MXINT = {"weight_block_size": 32, "weight_width": 8, "data_in_block_size": 32, "data_in_width": 8}


class OracleLinearMXInt(nn.Module):
    """CPU stand-in for the reference's LinearMXInt: weights quantized once, forward = q(x) @ W^T"""

    def __init__(self, linear: nn.Linear, cfg):
        super().__init__()
        self.cfg = dict(cfg)
        self.qw, self.qb = OL.mxint_prepare_weights(linear.weight.data, None if linear.bias is None else linear.bias.data, self.cfg)

    def forward(self, x):
        return OL.linear_mxint_forward(x, self.qw, self.qb, self.cfg)


def swap_in_oracle(layer, cfg):
    for name, m in list(layer.named_children()):
        if isinstance(m, nn.Linear):
            setattr(layer, name, OracleLinearMXInt(m, cfg))
    return layer


def rel_err(y, ref):
    return float((y.double().cpu() - ref.double()).abs().max() / ref.double().abs().max())


def reference_attention_on_cpu(q, k, v):
    """the reference's attention core evaluated on the CPU, whatever device the operands live on"""
    return OLL.eager_causal_attention(q.cpu(), k.cpu(), v.cpu()).to(q.device)


def build_pair(dev, cfg, seed):
    from mase_amd.passes import quantize_module_transform_pass
    from mase_amd.quantized import LinearMXInt
    from mase_amd.workloads import DecoderLayer

    cpu = DecoderLayer(cfg, dtype=torch.bfloat16, seed=seed)
    gpu = DecoderLayer(cfg, device=dev, dtype=torch.bfloat16, seed=seed)
    assert torch.equal(cpu.q_proj.weight, gpu.q_proj.weight.cpu())
    gpu, _ = quantize_module_transform_pass(gpu, {"by": "type", "linear": {"config": dict(MXINT, name="mxint")}})
    assert sum(isinstance(m, LinearMXInt) for m in gpu.modules()) == 7
    cpu = swap_in_oracle(cpu, MXINT)
    cpu.attention_fn = OLL.eager_causal_attention
    return cpu, gpu


REAL = (4096, 32, 11008)
SMALL = (1024, 8, 2752)


@pytest.mark.parametrize("shape,widths", [((2, 128), SMALL), ((1, 320), SMALL), ((1, 64), REAL), ((1, 128), REAL), ((2, 256), REAL)])
def test_decoder_layer_mxint_matches_cpu_reference(dev, shape, widths):
    """REAL = the layer widths of the headline configuration (hidden 4096, 32 x 128 heads, FFN 11008) on short sequences
    so that the CPU side finishes in seconds; its down_proj is the K = 11008 contraction.  (1, 320) and (1, 64) are not
    multiples of 128 tokens: the default path takes the library's attention kernel there."""
    from mase_amd.quantizers import _ops
    from mase_amd.workloads import DecoderLayerConfig
    from mase_amd.workloads.decoder_layer import causal_attention

    cfg = DecoderLayerConfig(hidden_size=widths[0], num_heads=widths[1], head_dim=128, intermediate_size=widths[2])
    B, T = shape
    x = torch.randn(B, T, cfg.hidden_size, generator=torch.Generator().manual_seed(4)).bfloat16()
    cpu, gpu = build_pair(dev, cfg, 40)
    # quantized weights: bit-identical
    for name in ("q_proj", "down_proj"):
        assert torch.equal(getattr(gpu, name).weight.data.cpu().view(torch.int16), getattr(cpu, name).qw.view(torch.int16))
    seen = {}
    hooks = [m.register_forward_hook(lambda mod, inp, out, n=n: seen.__setitem__(n, (inp[0], out)))
             for n, m in cpu.named_children() if isinstance(m, OracleLinearMXInt)]
    with torch.no_grad():
        ref = cpu(x)
        for h in hooks:
            h.remove()
        # (a) every Linear on the input its CPU counterpart saw: bit-identical output
        assert len(seen) == 7
        for n, (inp, out) in seen.items():
            got = getattr(gpu, n)(inp.to(dev))
            assert torch.equal(got.cpu().view(torch.int16), out.view(torch.int16)), f"{n}: Linear output differs"
        # (b) free-running layer, attention core evaluated by the reference's attention on both sides
        gpu.attention_fn = reference_attention_on_cpu
        y = gpu(x.to(dev))
        e_rest = rel_err(y, ref)
        # (c) the default path
        gpu.attention_fn = causal_attention
        own_calls = []
        real_attention = _ops.attention_causal
        _ops.attention_causal = lambda *a, **k: (own_calls.append(k), real_attention(*a, **k))[1]
        try:
            y_own = gpu(x.to(dev))
        finally:
            _ops.attention_causal = real_attention
        e_own = rel_err(y_own, ref)
        own_kernel = T % 128 == 0
        assert len(own_calls) == (1 if own_kernel else 0)
        if own_kernel:  # q rotated on load, output in o_proj's MXINT form
            assert own_calls[0].get("q_rope") is not None and own_calls[0].get("mxint_bits") == 8
        # the reference's attention evaluated exactly: how far the reference's own roundings move the layer output
        cpu.attention_fn = lambda q, k, v: OLL.eager_causal_attention(q, k, v, exact=True)
        spread = rel_err(cpu(x), ref)
    print(f"decoder layer MXINT8 {shape} widths {widths}: rel err {e_rest:.3e} with the reference's attention core, "
          f"{e_own:.3e} on the default path ({'own kernel' if own_kernel else 'library kernel'}); "
          f"reference attention vs its exact evaluation {spread:.3e}")
    assert y.dtype == torch.bfloat16 and y.shape == x.shape
    assert e_rest < 1e-2
    assert e_own < 2.5e-2
    assert e_own < 1e-2 or (widths == REAL and e_own < 1.5 * spread), (e_own, spread)


@pytest.mark.parametrize("T", [300, 256])
def test_decoder_layer_producers_write_the_quantized_form(dev, monkeypatch, T):
    """RMSNorm and the SwiGLU product hand the MXINT Linears their quantized activations directly
    (rmsnorm_mxint / add_rmsnorm_mxint / silu_mul_mxint): the layer's output is bit for bit that of the layer whose Linears quantize the
    stored tensors themselves, and the separate quantizer runs only for o_proj.  With a multiple of 128 tokens the
    attention kernel of this package runs and takes over q's rotation and o_proj's quantizer as well (no separate
    quantizer at all); with 300 tokens the library's attention kernel runs."""
    from mase_amd.quantizers import _ops
    from mase_amd.workloads import DecoderLayerConfig, decoder_layer

    cfg = DecoderLayerConfig(hidden_size=1024, num_heads=8, head_dim=128, intermediate_size=2752)
    _, gpu = build_pair(dev, cfg, 41)
    x = torch.randn(2, T, cfg.hidden_size, generator=torch.Generator().manual_seed(5)).bfloat16().to(dev)
    own = T % 128 == 0
    calls = {"qdq": 0, "norm": 0, "addnorm": 0, "silu": 0}
    real = {"qdq": _ops.mxint_qdq, "norm": _ops.rmsnorm_mxint, "addnorm": _ops.add_rmsnorm_mxint, "silu": _ops.silu_mul_mxint,
            "attn": _ops.attention_causal, "rope": _ops.rope}
    attn_kw, ropes = [], []
    monkeypatch.setattr(_ops, "attention_causal", lambda *a, **k: (attn_kw.append(k), real["attn"](*a, **k))[1])
    monkeypatch.setattr(_ops, "rope", lambda *a, **k: (ropes.append(1), real["rope"](*a, **k))[1])
    monkeypatch.setattr(_ops, "mxint_qdq", lambda *a, **k: (calls.__setitem__("qdq", calls["qdq"] + 1), real["qdq"](*a, **k))[1])
    monkeypatch.setattr(_ops, "rmsnorm_mxint", lambda *a, **k: (calls.__setitem__("norm", calls["norm"] + 1), real["norm"](*a, **k))[1])
    monkeypatch.setattr(_ops, "add_rmsnorm_mxint",
                        lambda *a, **k: (calls.__setitem__("addnorm", calls["addnorm"] + 1), real["addnorm"](*a, **k))[1])
    monkeypatch.setattr(_ops, "silu_mul_mxint", lambda *a, **k: (calls.__setitem__("silu", calls["silu"] + 1), real["silu"](*a, **k))[1])
    with torch.no_grad():
        fused = gpu(x)
    # the second norm also takes the residual addition; o_proj's quantizer runs inside the attention kernel when that runs
    assert calls == {"qdq": 0 if own else 1, "norm": 1, "addnorm": 1, "silu": 1}
    if own:  # one fused call: q rotated on load (only k goes through rope()), result in o_proj's MXINT form
        assert len(attn_kw) == 1 and attn_kw[0]["q_rope"] is not None and attn_kw[0]["mxint_bits"] == 8 and len(ropes) == 1
    else:
        assert attn_kw == [] and len(ropes) == 2
    attn_kw.clear(), ropes.clear()
    monkeypatch.setattr(decoder_layer, "shared_mxint_width", lambda *a, **k: None)
    calls.update(qdq=0, norm=0, addnorm=0, silu=0)
    with torch.no_grad():
        plain = gpu(x)
    assert calls == {"qdq": 4, "norm": 0, "addnorm": 0, "silu": 0}
    if own:  # the same kernel without the output form (o_proj quantizes for itself); q still rotated on load
        assert len(attn_kw) == 1 and attn_kw[0].get("q_rope") is not None and attn_kw[0].get("mxint_bits") is None and len(ropes) == 1
    assert torch.equal(fused.view(torch.int16), plain.view(torch.int16))
