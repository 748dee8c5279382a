"""CPU restatement of the MX-quantized Llama attention / MLP / RMSNorm forwards.  TEST INFRASTRUCTURE ONLY.

Follows the reference op for op: ``chop/nn/quantized/modules/llama/attention.py:147-217`` (projections, quantized
RoPE tables, KV-cache quantization) and ``:334-457`` (``_eager_attention_forward_mxfp/_mxint``: query quantized, scores,
mask, ``softmax_minifloat``, probabilities quantized, value product), ``llama/mlp.py:56-62`` (``silu_minifloat`` on the
gate projection), ``llama/rms_norm.py:72-84``, and the functional helpers ``functional/rope.py:8-27, 78-101``,
``functional/softmax.py:41-57``, ``functional/silu.py:41-57``, ``functional/kvcache.py:8-43``.
Pinned by composition: every quantizer used here is pinned in ``oracle.quantizers``; the remaining operations are
library routines (``F.linear``, ``matmul``, ``softmax``, ``silu``, ``rsqrt``).
"""
import torch
from torch.nn import functional as F

from .quantizers import minifloat_quantizer_sim, mxfp_quantizer, mxint_quantizer


def _cast(config, prefix="data_in"):
    return lambda t: minifloat_quantizer_sim(t, config[f"{prefix}_exponent_width"], config[f"{prefix}_frac_width"],
                                             config.get(f"{prefix}_is_finite", True),
                                             config.get(f"{prefix}_round_mode", "rn"))


def _mx(kind, config):
    if kind == "mxfp":
        return lambda t: mxfp_quantizer(t, config["data_in_block_size"], config["data_in_exponent_width"],
                                        config["data_in_frac_width"], block_dim=-1)
    return lambda t: mxint_quantizer(t, config["data_in_block_size"], config["data_in_width"], block_dim=-1)


def rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def rope(q, k, cos, sin, config=None):
    """config None = unquantized tables (the bypass branch)"""
    if config is not None:
        cos, sin = _cast(config)(cos), _cast(config)(sin)
    cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    if config is not None:
        cos, sin = cos[..., : q.size(-2), :], sin[..., : q.size(-2), :]
    return (q * cos) + (rotate_half(q) * sin), (k * cos) + (rotate_half(k) * sin)


def repeat_kv(x, n_rep):
    b, h, s, d = x.shape
    if n_rep == 1:
        return x
    return x[:, :, None, :, :].expand(b, h, n_rep, s, d).reshape(b, h * n_rep, s, d)


def head_rms_norm(x, weight, eps):
    """RMSNorm over head_dim as the Qwen3 attention applies it to the projected queries and keys
    (qwen3/attention.py:53-59; transformers' Qwen3RMSNorm arithmetic)"""
    dt = x.dtype
    x = x.to(torch.float32)
    x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return weight * x.to(dt)


def eager_causal_attention(q, k, v, exact: bool = False):
    """The attention core of the reference's unquantized Llama block on [batch, heads, tokens, head_dim] operands
    (``chop/models/llama/modeling_llama.py:430-446``): ``matmul(q, k^T) / sqrt(head_dim)`` in the model dtype, the
    additive causal mask, softmax in fp32, the probabilities cast back to the model dtype, ``matmul`` with v.
    ``exact``: the same function evaluated in fp32 throughout with one rounding of the result (what the reference's
    chain of roundings approximates); the distance between the two is the reference's own rounding noise."""
    T, d = q.shape[-2], q.shape[-1]
    dt = q.dtype
    if exact:
        q, k, v = q.float(), k.float(), v.float()
    w = torch.matmul(q, k.transpose(2, 3)) / d ** 0.5
    mask = torch.full((T, T), torch.finfo(w.dtype).min, dtype=w.dtype).triu(1)
    w = w + mask
    w = F.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype)
    return torch.matmul(w, v).to(dt)


def attention_forward(kind, weights, hidden_states, cos, sin, attention_mask, n_heads, n_kv_heads, q_config,
                      past=None, qk_norm_eps=None):
    """weights: dict with q_proj/k_proj/v_proj/o_proj ``.weight`` (and optional ``.bias``) tensors.
    past: optional (key, value) already in the cache; the new (quantized) states are appended along the sequence.
    qk_norm_eps: the Qwen3 form (``q_norm.weight`` / ``k_norm.weight`` in ``weights``), else the Llama form."""
    lin = lambda name, t: F.linear(t, weights[f"{name}.weight"], weights.get(f"{name}.bias"))
    cfg = lambda name: q_config.get(name, {})
    on = lambda name: not cfg(name).get("bypass", False)
    B, S, _ = hidden_states.shape
    head_dim = weights["q_proj.weight"].shape[0] // n_heads
    q = lin("q_proj", hidden_states).view(B, S, -1, head_dim)
    k = lin("k_proj", hidden_states).view(B, S, -1, head_dim)
    if qk_norm_eps is not None:
        q = head_rms_norm(q, weights["q_norm.weight"], qk_norm_eps)
        k = head_rms_norm(k, weights["k_norm.weight"], qk_norm_eps)
    q, k = q.transpose(1, 2), k.transpose(1, 2)
    v = lin("v_proj", hidden_states).view(B, S, -1, head_dim).transpose(1, 2)
    q, k = rope(q, k, cos, sin, cfg("rope") if on("rope") else None)
    if past is not None:
        if on("kv_cache"):
            k, v = _mx(kind, cfg("kv_cache"))(k), _mx(kind, cfg("kv_cache"))(v)
        k, v = torch.cat([past[0], k], dim=2), torch.cat([past[1], v], dim=2)
    ks, vs = repeat_kv(k, n_heads // n_kv_heads), repeat_kv(v, n_heads // n_kv_heads)
    if on("qk_matmul"):
        q = _mx(kind, cfg("qk_matmul"))(q)
    w = torch.matmul(q, ks.transpose(2, 3)) * head_dim ** -0.5
    if attention_mask is not None:
        w = w + attention_mask[:, :, :, : ks.shape[-2]]
    if on("softmax"):
        w = _cast(cfg("softmax"))(w)
    w = F.softmax(w.to(torch.float32), dim=-1).to(w.dtype)
    if on("av_matmul"):
        w = _mx(kind, cfg("av_matmul"))(w)
    o = torch.matmul(w, vs).transpose(1, 2).contiguous().reshape(B, S, -1)
    return lin("o_proj", o), w


def mlp_forward(weights, x, q_config):
    lin = lambda name, t: F.linear(t, weights[f"{name}.weight"], weights.get(f"{name}.bias"))
    g = lin("gate_proj", x)
    if not q_config.get("bypass", False):
        g = _cast(q_config)(g)
    return lin("down_proj", F.silu(g) * lin("up_proj", x))


def rms_norm_forward(weight, x, eps, q_config):
    dt = x.dtype
    bypass = q_config.get("bypass", False)
    if not bypass and not q_config.get("data_in_bypass", False):
        x = _cast(q_config, "data_in")(x)
    x = x.to(torch.float32)
    x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    if not bypass and not q_config.get("weight_bypass", False):
        weight = _cast(q_config, "weight")(weight)
    return weight * x.to(dt)
