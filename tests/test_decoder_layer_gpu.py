"""The decoder-layer workload: every nn.Linear replaced by LinearMXInt through the quantize pass, compared with the
same layer on the CPU whose Linears compute the reference's forward (oracle restatement).

Error measure: max|y - y_ref| / max|y_ref| <= 1e-2 on the layer output.  Both sides run the non-Linear parts
(RMSNorm, rotary embedding, causal attention, SiLU) with the same torch ops in bf16; only the seven Linears differ
in implementation.  torch's own scaled_dot_product_attention differs between its CPU and GPU kernels by about
3e-3 of the maximum (measured with identical inputs), and the quantizers downstream turn such differences into
whole quantization steps; so the end-to-end comparison that carries the 1e-2 bound evaluates the attention core on
the CPU for both sides, a second one with the GPU attention kernel is held to 3e-2, and a third feeds every GPU
Linear the exact input its CPU counterpart saw and demands bit-identical outputs."""
import copy

import pytest
import torch
from torch import nn

from oracle import linear as OL

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


def cpu_attention(q, k, v):
    """the library's CPU attention, whatever device the operands live on"""
    o = torch.nn.functional.scaled_dot_product_attention(q.cpu(), k.cpu(), v.cpu(), is_causal=True)
    return o.to(q.device)


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
    return cpu, gpu


@pytest.mark.parametrize("shape,widths", [((2, 128), (1024, 8, 2752)), ((1, 320), (1024, 8, 2752)), ((1, 64), (4096, 32, 11008))])
def test_decoder_layer_mxint_matches_cpu_reference(dev, shape, widths):
    """(1, 64) runs the real layer widths (hidden 4096, 32 x 128 heads, FFN 11008) on a short sequence so that the
    CPU side finishes in seconds; its down_proj is the K = 11008 contraction no other test covers"""
    from mase_amd.workloads import DecoderLayerConfig

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
        # (b) free-running layer, attention core evaluated by the same (CPU) library kernel on both sides
        gpu.attention_fn = cpu_attention
        y = gpu(x.to(dev))
        e = rel_err(y, ref)
        # (c) free-running layer with the GPU attention kernel of the library
        del gpu.attention_fn
        gpu.attention_fn = lambda q, k, v: torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
        e_lib = rel_err(gpu(x.to(dev)), ref)
        # (d) free-running layer with its own default attention (the kernel of this package where the shape allows)
        from mase_amd.workloads.decoder_layer import causal_attention
        gpu.attention_fn = causal_attention
        e_own = rel_err(gpu(x.to(dev)), ref)
        assert e_own < 3e-2, e_own
    print(f"decoder layer MXINT8 {shape} widths {widths}: rel err {e:.3e} (same attention kernel), {e_lib:.3e} (GPU attention kernel)")
    assert y.dtype == torch.bfloat16 and y.shape == x.shape
    assert e < 1e-2
    assert e_lib < 3e-2


def test_decoder_layer_producers_write_the_quantized_form(dev, monkeypatch):
    """RMSNorm and the SwiGLU product hand the MXINT Linears their quantized activations directly
    (rmsnorm_mxint / add_rmsnorm_mxint / silu_mul_mxint): the layer's output is bit for bit that of the layer whose Linears quantize the
    stored tensors themselves, and the separate quantizer runs only for o_proj"""
    from mase_amd.quantizers import _ops
    from mase_amd.workloads import DecoderLayerConfig, decoder_layer

    cfg = DecoderLayerConfig(hidden_size=1024, num_heads=8, head_dim=128, intermediate_size=2752)
    _, gpu = build_pair(dev, cfg, 41)
    x = torch.randn(2, 300, cfg.hidden_size, generator=torch.Generator().manual_seed(5)).bfloat16().to(dev)
    calls = {"qdq": 0, "norm": 0, "addnorm": 0, "silu": 0}
    real = {"qdq": _ops.mxint_qdq, "norm": _ops.rmsnorm_mxint, "addnorm": _ops.add_rmsnorm_mxint, "silu": _ops.silu_mul_mxint}
    monkeypatch.setattr(_ops, "mxint_qdq", lambda *a, **k: (calls.__setitem__("qdq", calls["qdq"] + 1), real["qdq"](*a, **k))[1])
    monkeypatch.setattr(_ops, "rmsnorm_mxint", lambda *a, **k: (calls.__setitem__("norm", calls["norm"] + 1), real["norm"](*a, **k))[1])
    monkeypatch.setattr(_ops, "add_rmsnorm_mxint",
                        lambda *a, **k: (calls.__setitem__("addnorm", calls["addnorm"] + 1), real["addnorm"](*a, **k))[1])
    monkeypatch.setattr(_ops, "silu_mul_mxint", lambda *a, **k: (calls.__setitem__("silu", calls["silu"] + 1), real["silu"](*a, **k))[1])
    with torch.no_grad():
        fused = gpu(x)
    assert calls == {"qdq": 1, "norm": 1, "addnorm": 1, "silu": 1}  # the second norm also takes the residual addition
    monkeypatch.setattr(decoder_layer, "shared_mxint_width", lambda *a, **k: None)
    calls.update(qdq=0, norm=0, addnorm=0, silu=0)
    with torch.no_grad():
        plain = gpu(x)
    assert calls == {"qdq": 4, "norm": 0, "addnorm": 0, "silu": 0}
    assert torch.equal(fused.view(torch.int16), plain.view(torch.int16))
