"""A Llama-style decoder layer out of plain ``torch.nn`` parts: the workload whose ``nn.Linear`` modules the
quantize pass replaces (RMSNorm -> q/k/v projections -> rotary embedding -> causal attention -> o projection ->
residual; RMSNorm -> SwiGLU MLP -> residual).

Semantics follow the reference's Llama block (``chop/models/llama/modeling_llama.py:79-93`` RMSNorm, ``:99-147,
185-216`` rotary embedding with ``rotate_half``, ``:219-236`` MLP ``down(silu(gate(x)) * up(x))``, ``:362-480``
attention, ``:843-918`` layer with pre-norm residuals); no KV cache, no dropout, no attention bias.
On the CPU everything except the seven Linears is ordinary torch, which is what lets the same class serve as the CPU
reference once its Linears are swapped for reference ones; on the GPU (no gradient recorded) the causal attention
core runs as a one-pass kernel (``mase_attention_causal``: bf16, head dimension 128, sequence a multiple of 128;
otherwise the library's), and RMSNorm, the rotary embedding and the SwiGLU product run as one-pass kernels with the same arithmetic (``mase_rmsnorm_minifloat``,
``mase_rope``, ``mase_silu_mul_minifloat`` with their casts off); where the Linears that consume an RMSNorm or the
SwiGLU product are MXINT Linears on the matrix-core path, those kernels write the quantized form the Linears would
each compute (``mase_rmsnorm_mxint``, ``mase_silu_mul_mxint``), which saves a pass over the tensor.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
from torch import nn
from torch.nn import functional as F

from ..quantizers import _ops
from ..quantized.functional.mx_linear import project_shared, shared_mxint_width


@dataclass
class DecoderLayerConfig:
    hidden_size: int = 4096
    num_heads: int = 32
    head_dim: int = 128
    intermediate_size: int = 11008
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    init_std: float = 0.02


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.eps = eps

    def forward(self, x):
        if x.is_cuda and _ops.rmsnorm_supported(x, self.weight):
            return _ops.rmsnorm_minifloat(x, self.weight, self.eps)  # the same arithmetic in one pass
        dtype = x.dtype
        h = x.to(torch.float32)
        h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.eps)
        return self.weight * h.to(dtype)


def rotate_half(x):
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def rope_tables(seq_len: int, head_dim: int, theta: float, device, dtype):
    """cos / sin tables of the rotary embedding, evaluated on the host whatever ``device`` is: the host's and the
    device's ``cos`` / ``sin`` differ in the last fp32 place for some arguments, which moves about one table entry in
    a thousand to the neighbouring 16-bit value; with the host's tables a GPU layer and a CPU layer rotate with
    identical factors"""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    t = torch.arange(seq_len, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype).to(device), emb.sin().to(dtype).to(device)


def causal_attention(q, k, v, mxint_bits=None, q_rope=None):
    """softmax(q k^T / sqrt(d) + causal mask) v: the one-pass kernel of this package where it applies (bf16, head
    dimension 128, a multiple of 128 tokens, no gradient), the library's scaled_dot_product_attention otherwise.
    Only where the kernel applies: ``mxint_bits``, the result in the MXINT form of the Linear that reads it;
    ``q_rope = (cos, sin)``, q handed over before its rotary embedding, which the kernel applies on load."""
    if q.is_cuda and _ops.attention_causal_supported(q, k, v):
        return _ops.attention_causal(q, k, v, mxint_bits=mxint_bits, q_rope=q_rope)
    assert mxint_bits is None and q_rope is None
    return F.scaled_dot_product_attention(q, k, v, is_causal=True)


class DecoderLayer(nn.Module):
    def __init__(self, cfg: DecoderLayerConfig = DecoderLayerConfig(), device=None, dtype=None, seed: int | None = None):
        super().__init__()
        self.cfg = cfg
        kw = dict(bias=False, device=device, dtype=dtype)
        H, D, I = cfg.hidden_size, cfg.num_heads * cfg.head_dim, cfg.intermediate_size
        self.input_layernorm = RMSNorm(H, cfg.rms_norm_eps).to(device=device, dtype=dtype)
        self.q_proj = nn.Linear(H, D, **kw)
        self.k_proj = nn.Linear(H, D, **kw)
        self.v_proj = nn.Linear(H, D, **kw)
        self.o_proj = nn.Linear(D, H, **kw)
        self.post_attention_layernorm = RMSNorm(H, cfg.rms_norm_eps).to(device=device, dtype=dtype)
        self.gate_proj = nn.Linear(H, I, **kw)
        self.up_proj = nn.Linear(H, I, **kw)
        self.down_proj = nn.Linear(I, H, **kw)
        # the attention core; tests replace it to keep both sides of a comparison on the same implementation (the
        # library's CPU and GPU kernels and the kernel of this package differ by a few bf16 ulps)
        self.attention_fn = causal_attention
        if seed is not None:
            self.reset_parameters_seeded(seed)

    @torch.no_grad()
    def reset_parameters_seeded(self, seed: int):
        """N(0, init_std) weights drawn on the CPU from one generator, so that a CPU and a GPU instance built with
        the same seed hold identical parameters"""
        g = torch.Generator().manual_seed(seed)
        for name in ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"):
            w = getattr(self, name).weight
            w.copy_((torch.randn(w.shape, generator=g) * self.cfg.init_std).to(w.dtype))

    # RMSNorm / the SwiGLU product write the quantized form MXINT Linears after them would compute (see
    # _norm_then_project); False: every Linear receives the plain tensor and quantizes it itself
    fuse_producers = True

    def _norm_then_project(self, norm, x, modules, addend=None):
        """``x, [m(norm(x)) for m in modules]`` with ``x + addend`` for ``x`` when an addend is given (the residual
        addition that precedes the norm).  Sibling projections of one tensor: quantized Linears that treat it alike
        share one quantized copy, and when they are MXINT Linears on the matrix-core path the norm writes that copy
        itself instead of a tensor each of them would read and quantize (same values: the quantizer's arithmetic on
        the norm's rounded output); the addition then happens in the norm's pass as well."""
        if (self.fuse_producers and x.is_cuda and not torch.is_grad_enabled() and x.shape[-1] % 32 == 0
                and _ops.rmsnorm_supported(x, norm.weight)):
            bits = shared_mxint_width(x, modules)
            if bits is not None:
                if addend is not None and addend.shape == x.shape and addend.dtype == x.dtype:
                    x, hq = _ops.add_rmsnorm_mxint(x, addend, norm.weight, norm.eps, bits)
                else:
                    x = x if addend is None else x + addend
                    hq = _ops.rmsnorm_mxint(x, norm.weight, norm.eps, bits)
                return x, [m(hq, prepared=hq.reshape(-1, hq.shape[-1])) for m in modules]
        x = x if addend is None else x + addend
        return x, project_shared(norm(x), modules)

    def _rope_tables(self, T, device, dtype):
        """the cos / sin tables of the rotary embedding depend on (sequence length, device, dtype) only: kept from one
        forward to the next (a model computes them once per forward for all its layers)"""
        key = (T, device, dtype)
        if getattr(self, "_rope_key", None) != key:
            self._rope_key, self._rope_val = key, rope_tables(T, self.cfg.head_dim, self.cfg.rope_theta, device, dtype)
        return self._rope_val

    def forward(self, x):
        cfg = self.cfg
        B, T, _ = x.shape
        q, k, v = (t.view(B, T, cfg.num_heads, cfg.head_dim).transpose(1, 2)
                   for t in self._norm_then_project(self.input_layernorm, x, (self.q_proj, self.k_proj, self.v_proj))[1])
        cos, sin = self._rope_tables(T, x.device, x.dtype)
        own_kernel = (self.fuse_producers and self.attention_fn is causal_attention and q.is_cuda
                      and not torch.is_grad_enabled() and _ops.attention_causal_supported(q, k, v))
        rope_ok = q.is_cuda and _ops.rope_supported(q, cos, sin) and _ops.rope_supported(k, cos, sin)
        q_rope = (cos, sin) if own_kernel and rope_ok else None  # the attention kernel rotates q as it loads it
        if rope_ok:
            k = _ops.rope(k, cos, sin)  # the same products and sum in one pass
            if q_rope is None:
                q = _ops.rope(q, cos, sin)
        else:
            q = q * cos + rotate_half(q) * sin
            k = k * cos + rotate_half(k) * sin
        # o_proj's input has x's dtype and device and a last dimension that is a multiple of 32
        bits = shared_mxint_width(x, (self.o_proj,)) if own_kernel else None
        if own_kernel:
            a = causal_attention(q, k, v, mxint_bits=bits, q_rope=q_rope)
        else:
            a = self.attention_fn(q, k, v)
        a = a.transpose(1, 2).reshape(B, T, cfg.num_heads * cfg.head_dim)
        o = self.o_proj(a, prepared=a.reshape(-1, a.shape[-1])) if bits is not None else self.o_proj(a)
        x, (gate, up) = self._norm_then_project(self.post_attention_layernorm, x, (self.gate_proj, self.up_proj), addend=o)
        if gate.is_cuda and _ops.silu_mul_supported(gate, up):
            bits = shared_mxint_width(gate, (self.down_proj,)) if self.fuse_producers and gate.shape[-1] % 32 == 0 else None
            if bits is not None and not torch.is_grad_enabled():
                actq = _ops.silu_mul_mxint(gate, up, bits)  # the product, already in down_proj's quantized form
                return x + self.down_proj(actq, prepared=actq.reshape(-1, actq.shape[-1]))
            act = _ops.silu_mul_minifloat(gate, up)  # silu(gate) * up in one pass
        else:
            act = F.silu(gate) * up
        return x + self.down_proj(act)

    def linear_flops(self, tokens: int) -> float:
        H, D, I = self.cfg.hidden_size, self.cfg.num_heads * self.cfg.head_dim, self.cfg.intermediate_size
        return 2.0 * tokens * (3 * H * D + D * H + 3 * H * I)
