"""GPU parity of the MX-quantized Llama attention / MLP / RMSNorm modules against the CPU oracle's restatement of
the reference forwards, and of the module pass that swaps them in.

Tolerances (max |y - y_ref| / max |y_ref|): fp32 5e-3, bf16 3e-2.  The quantizers themselves are bit-exact (tested
elsewhere); what differs between the two sides is the library's GEMM / softmax rounding on CPU and GPU, which a
downstream quantizer can turn into one quantization step on an element (2^-7 of its block maximum for MXINT8, 2^-3
for e4m3 probabilities)."""
from types import SimpleNamespace

import pytest
import torch

from oracle import llama as OL

pytestmark = pytest.mark.gpu

CFG = SimpleNamespace(hidden_size=256, num_attention_heads=8, num_key_value_heads=4, head_dim=32, attention_bias=False,
                      attention_dropout=0.0, intermediate_size=512, mlp_bias=False, hidden_act="silu", rms_norm_eps=1e-6)
MINI = {"data_in_exponent_width": 5, "data_in_frac_width": 8}
Q_INT = {"qk_matmul": {"data_in_block_size": 32, "data_in_width": 8}, "av_matmul": {"data_in_block_size": 32, "data_in_width": 8},
         "rope": dict(MINI), "softmax": dict(MINI), "kv_cache": {"data_in_block_size": 32, "data_in_width": 8}}
_FP = {"data_in_block_size": 32, "data_in_exponent_width": 4, "data_in_frac_width": 3}
Q_FP = {"qk_matmul": dict(_FP), "av_matmul": dict(_FP), "rope": dict(MINI), "softmax": dict(MINI), "kv_cache": dict(_FP)}


def rel_err(y, ref):
    return float((y.double().cpu() - ref.double()).abs().max() / ref.double().abs().max())


def rope_tables(batch, seq, dim, dtype, offset=0):
    inv = 1.0 / (10000 ** (torch.arange(0, dim, 2).float() / dim))
    ang = (torch.arange(offset, offset + seq).float()[:, None] * inv[None, :])
    emb = torch.cat([ang, ang], dim=-1)
    return emb.cos()[None].expand(batch, -1, -1).to(dtype).contiguous(), emb.sin()[None].expand(batch, -1, -1).to(dtype).contiguous()


def causal_mask(batch, q_len, kv_len, dtype):
    m = torch.full((q_len, kv_len), torch.finfo(dtype).min, dtype=dtype)
    m = torch.triu(m, diagonal=kv_len - q_len + 1)
    return m[None, None].expand(batch, 1, -1, -1).contiguous()


class ListCache:
    """the part of the cache interface the attention uses: update() appends along the sequence and returns all"""

    def __init__(self, k, v):
        self.k, self.v = k, v

    def update(self, k, v, layer_idx, cache_kwargs=None):
        assert layer_idx == 3 and set(cache_kwargs) == {"sin", "cos", "cache_position"}
        self.k, self.v = torch.cat([self.k, k], dim=2), torch.cat([self.v, v], dim=2)
        return self.k, self.v


def seeded(module, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    sd = {k: (torch.randn(v.shape, generator=g) * (0.06 if v.dim() == 2 else 1.0)).to(dtype)
          for k, v in module.state_dict().items()}
    return sd


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["mxint", "mxfp"])
def test_attention_prefill_and_decode_match_the_oracle(dev, dtype, kind):
    from mase_amd.quantized import LlamaAttentionMXFP, LlamaAttentionMXInt

    cls, qc = (LlamaAttentionMXInt, Q_INT) if kind == "mxint" else (LlamaAttentionMXFP, Q_FP)
    tol = 5e-3 if dtype == torch.float32 else 3e-2
    m = cls(CFG, layer_idx=3, q_config=qc).to(dtype)
    sd = seeded(m, 21, dtype)
    m.load_state_dict(sd, strict=True)
    m = m.to(dev).eval()
    g = torch.Generator().manual_seed(22)
    B, S = 2, 64
    x = torch.randn(B, S, CFG.hidden_size, generator=g).to(dtype)
    cos, sin = rope_tables(B, S, CFG.head_dim, dtype)
    mask = causal_mask(B, S, S, dtype)
    with torch.no_grad():
        y, w = m(x.to(dev), (cos.to(dev), sin.to(dev)), mask.to(dev))
    ref, wref = OL.attention_forward(kind, sd, x, cos, sin, mask, 8, 4, qc)
    assert y.shape == (B, S, CFG.hidden_size) and w.shape == (B, 8, S, S)
    assert rel_err(y, ref) < tol, (kind, dtype, rel_err(y, ref))
    # probabilities: within one quantization step of their block maximum (<= 1), and exactly 0 above the diagonal
    assert float((w.float().cpu() - wref.float()).abs().max()) <= (2 ** -6 if kind == "mxint" else 2 ** -3)
    assert float(w.float().cpu().triu(1).abs().max()) == 0.0

    # decode: one new token against a cache of S - 1 states (S keys in all: the flattened probabilities must be whole
    # blocks, as in the reference); no mask
    past_k = torch.randn(B, 4, S - 1, CFG.head_dim, generator=g).to(dtype)
    past_v = torch.randn(B, 4, S - 1, CFG.head_dim, generator=g).to(dtype)
    x1 = torch.randn(B, 1, CFG.hidden_size, generator=g).to(dtype)
    cos1, sin1 = rope_tables(B, 1, CFG.head_dim, dtype, offset=S - 1)
    cache = ListCache(past_k.to(dev), past_v.to(dev))
    with torch.no_grad():
        y1, w1 = m(x1.to(dev), (cos1.to(dev), sin1.to(dev)), None, past_key_value=cache, cache_position=torch.tensor([S - 1]))
    ref1, _ = OL.attention_forward(kind, sd, x1, cos1, sin1, None, 8, 4, qc, past=(past_k, past_v))
    assert cache.k.shape == (B, 4, S, CFG.head_dim) and w1.shape == (B, 8, 1, S)
    assert rel_err(y1, ref1) < tol, (kind, dtype, rel_err(y1, ref1))


def test_attention_bypass_is_plain_attention_and_from_attention_copies_weights(dev):
    from mase_amd.quantized import LlamaAttentionMXInt

    class LlamaAttention(torch.nn.Module):  # the layout of the module being replaced
        def __init__(self):
            super().__init__()
            self.config, self.layer_idx = CFG, 5
            self.q_proj = torch.nn.Linear(256, 256, bias=False)
            self.k_proj = torch.nn.Linear(256, 128, bias=False)
            self.v_proj = torch.nn.Linear(256, 128, bias=False)
            self.o_proj = torch.nn.Linear(256, 256, bias=False)

    torch.manual_seed(5)
    src = LlamaAttention().to(dev)
    bypass = {k: {"bypass": True} for k in ("qk_matmul", "av_matmul", "rope", "softmax", "kv_cache")}
    m = LlamaAttentionMXInt.from_attention(src, bypass).eval()
    assert m.layer_idx == 5 and m.q_proj.weight.device.type == "cuda"
    assert torch.equal(m.k_proj.weight, src.k_proj.weight)
    B, S = 2, 48
    x = torch.randn(B, S, 256, device=dev)
    cos, sin = (t.to(dev) for t in rope_tables(B, S, 32, torch.float32))
    mask = causal_mask(B, S, S, torch.float32).to(dev)
    with torch.no_grad():
        y, _ = m(x, (cos, sin), mask)
        q = src.q_proj(x).view(B, S, 8, 32).transpose(1, 2)
        k = src.k_proj(x).view(B, S, 4, 32).transpose(1, 2)
        v = src.v_proj(x).view(B, S, 4, 32).transpose(1, 2)
        rot = lambda t: torch.cat((-t[..., 16:], t[..., :16]), -1)
        q, k = q * cos[:, None] + rot(q) * sin[:, None], k * cos[:, None] + rot(k) * sin[:, None]
        k, v = k.repeat_interleave(2, 1), v.repeat_interleave(2, 1)
        p = torch.softmax(q @ k.transpose(2, 3) * 32 ** -0.5 + mask, -1)
        ref = src.o_proj((p @ v).transpose(1, 2).reshape(B, S, 256))
    assert float((y - ref).abs().max() / ref.abs().max()) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mlp_and_rms_norm_match_the_oracle(dev, dtype):
    from mase_amd.quantized import LlamaMLPMXFP, LlamaMLPMXInt, LlamaRMSNormMinifloat

    tol = 1e-4 if dtype == torch.float32 else 2e-2
    g = torch.Generator().manual_seed(31)
    x = torch.randn(3, 40, CFG.hidden_size, generator=g).to(dtype)
    for cls in (LlamaMLPMXInt, LlamaMLPMXFP):
        for qc in ({"data_in_exponent_width": 4, "data_in_frac_width": 3}, {"bypass": True}):
            m = cls(CFG, layer_idx=0, q_config=qc).to(dtype)
            sd = seeded(m, 32, dtype)
            m.load_state_dict(sd, strict=True)
            with torch.no_grad():
                y = m.to(dev)(x.to(dev))
            assert rel_err(y, OL.mlp_forward(sd, x, qc)) < tol, (cls.__name__, qc)
    nq = {"weight_exponent_width": 4, "weight_frac_width": 3, "data_in_exponent_width": 5, "data_in_frac_width": 2,
          "data_in_round_mode": "rz"}
    for qc in (nq, {**nq, "weight_bypass": True}, {**nq, "data_in_bypass": True}, {"bypass": True}):
        n = LlamaRMSNormMinifloat(CFG, layer_idx=1, q_config=qc).to(dtype)
        w = (1.0 + 0.1 * torch.randn(CFG.hidden_size, generator=g)).to(dtype)
        n.load_state_dict({"weight": w})
        with torch.no_grad():
            y = n.to(dev)(x.to(dev))
        assert y.dtype == dtype
        assert rel_err(y, OL.rms_norm_forward(w, x, CFG.rms_norm_eps, qc)) < (1e-5 if dtype == torch.float32 else 1e-2), qc


def test_module_pass_swaps_llama_blocks_by_regex_name(dev):
    """quantize_module_transform_pass with by="regex_name": Llama attention / MLP / RMSNorm and Linear targets in one
    call, weights carried over, network.config handed to the Llama replacements"""
    from mase_amd.passes import quantize_module_transform_pass
    from mase_amd.quantized import LinearMXInt, LlamaAttentionMXInt, LlamaMLPMXInt, LlamaRMSNormMinifloat

    class LlamaRMSNorm(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.ones(256))

    class LlamaMLP(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.gate_proj = torch.nn.Linear(256, 512, bias=False)
            self.up_proj = torch.nn.Linear(256, 512, bias=False)
            self.down_proj = torch.nn.Linear(512, 256, bias=False)

    class LlamaAttention(torch.nn.Module):
        def __init__(self, layer_idx):
            super().__init__()
            self.layer_idx = layer_idx
            self.q_proj = torch.nn.Linear(256, 256, bias=False)
            self.k_proj = torch.nn.Linear(256, 128, bias=False)
            self.v_proj = torch.nn.Linear(256, 128, bias=False)
            self.o_proj = torch.nn.Linear(256, 256, bias=False)

    class Block(torch.nn.Module):
        def __init__(self, i):
            super().__init__()
            self.input_layernorm, self.self_attn, self.mlp = LlamaRMSNorm(), LlamaAttention(i), LlamaMLP()

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.config = CFG
            self.layers = torch.nn.ModuleList([Block(0), Block(1)])
            self.lm_head = torch.nn.Linear(256, 100, bias=False)

    torch.manual_seed(7)
    net = Net().to(dev)
    k_before = net.layers[1].self_attn.k_proj.weight.detach().clone()
    pass_args = {
        "by": "regex_name",
        r"layers\.\d+\.self_attn": {"config": {"name": "mxint", **Q_INT}},
        r"layers\.\d+\.mlp": {"config": {"name": "mxint", "data_in_exponent_width": 4, "data_in_frac_width": 3}},
        r"layers\.\d+\.input_layernorm": {"config": {"name": "minifloat", "weight_exponent_width": 4, "weight_frac_width": 3,
                                                      "data_in_exponent_width": 4, "data_in_frac_width": 3}},
        r"lm_head": {"config": {"name": "mxint", "weight_block_size": 32, "weight_width": 8, "data_in_block_size": 32,
                                "data_in_width": 8}},
    }
    net, info = quantize_module_transform_pass(net, pass_args)
    assert info == {} and "by" not in pass_args
    blk = net.layers[1]
    assert isinstance(blk.self_attn, LlamaAttentionMXInt) and blk.self_attn.layer_idx == 1 and blk.self_attn.config is CFG
    assert isinstance(blk.mlp, LlamaMLPMXInt) and isinstance(blk.input_layernorm, LlamaRMSNormMinifloat)
    assert isinstance(net.lm_head, LinearMXInt)
    assert torch.equal(blk.self_attn.k_proj.weight, k_before) and blk.self_attn.k_proj.weight.device.type == "cuda"
    # the swapped-in blocks run
    x = torch.randn(2, 32, 256, device=dev)
    cos, sin = (t.to(dev) for t in rope_tables(2, 32, 32, torch.float32))
    with torch.no_grad():
        h = blk.input_layernorm(x)
        a, _ = blk.self_attn(h, (cos, sin), causal_mask(2, 32, 32, torch.float32).to(dev))
        out = net.lm_head(blk.mlp(x + a))
    assert out.shape == (2, 32, 100) and bool(torch.isfinite(out).all())


def _oracle_probabilities(scores, mask, scaling, cast, mx):
    """the reference's tensor passes from raw scores to quantized probabilities, on the CPU (attention.py:363-392)"""
    import oracle as O

    w = scores * scaling
    if mask is not None:
        w = w + mask
    if cast is not None:
        w = O.minifloat_quantizer_sim(w, cast[0], cast[1], cast[2], cast[3])
    w = torch.softmax(w.to(torch.float32), dim=-1).to(scores.dtype)
    if mx is not None and mx[0] == "mxint":
        w = O.mxint_quantizer(w, 32, mx[1], block_dim=-1)
    elif mx is not None:
        w = O.mxfp_quantizer(w, 32, mx[1], mx[2], block_dim=-1)
    return w


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kv_len", [32, 544, 2048])
def test_one_pass_probabilities_match_the_separate_passes(dev, dtype, kv_len):
    """mase_attn_softmax_mx against the oracle's separate passes.  The exponentials differ by rounding between the
    two, so a probability may land on the neighbouring code: asserted bound = one quantization step of its block
    (2^-7 of a block maximum <= 1 for MXINT8, 2^-3 for e4m3; 2^-8 relative for the unquantized case), and at least
    99 % of the elements bit-identical."""
    from mase_amd.quantizers._ops import attn_softmax_mx, attn_softmax_mx_supported

    g = torch.Generator().manual_seed(kv_len)
    B, H, S = 2, 3, 40
    scores = (torch.randn(B, H, S, kv_len, generator=g) * 6).to(dtype)
    wide = torch.zeros(B, 1, S, kv_len + 64, dtype=dtype)
    wide[..., :kv_len] = causal_mask(B, S, kv_len, dtype)
    wide[1, 0, 3, : kv_len // 2] = torch.finfo(dtype).min  # a padding-like hole
    for mask in (None, wide):
        m_dev = None if mask is None else mask.to(dev)[:, :, :, :kv_len]
        m_cpu = None if mask is None else mask[:, :, :, :kv_len]
        assert attn_softmax_mx_supported(scores.to(dev), m_dev)
        for cast, mx, step in (((5, 8, True, "rn"), ("mxint", 8), 2 ** -7), ((4, 3, True, "rn"), ("mxfp", 4, 3), 2 ** -3),
                               (None, ("mxfp", 2, 1), 0.5), ((5, 2, False, "rz"), None, 2 ** -8), (None, None, 2 ** -8)):
            got = attn_softmax_mx(scores.to(dev), m_dev, 0.125, cast, mx).cpu()
            want = _oracle_probabilities(scores, m_cpu, 0.125, cast, mx)
            # a fully masked row whose mask value the cast turns into -inf (fp16) is NaN on both sides
            nan = torch.isnan(want)
            assert torch.equal(torch.isnan(got), nan), (cast, mx)
            diff = (got.float() - want.float()).abs()[~nan]
            if mx is None and dtype == torch.float32:  # unquantized fp32: the exponentials differ in the last bits
                assert float((diff / want.float()[~nan].clamp_min(1e-30)).max()) < 1e-5
            else:
                assert float(diff.max()) <= step, (cast, mx, float(diff.max()))
                same = float((got == want)[~nan].float().mean())
                assert same > 0.99, (cast, mx, same)
            if mask is not None:  # in rows that keep a key, the masked positions carry exactly zero probability
                masked = (m_cpu < 0).expand_as(got)
                open_row = (~masked).any(-1, keepdim=True).expand_as(got)
                assert float(got[masked & open_row].abs().max()) == 0.0


def test_attention_module_one_pass_and_separate_passes_agree(dev):
    from mase_amd.quantized import LlamaAttentionMXInt

    m = LlamaAttentionMXInt(CFG, layer_idx=3, q_config=Q_INT).to(torch.bfloat16)
    m.load_state_dict(seeded(m, 41, torch.bfloat16))
    m = m.to(dev).eval()
    g = torch.Generator().manual_seed(42)
    B, S = 2, 256
    x = torch.randn(B, S, CFG.hidden_size, generator=g).bfloat16().to(dev)
    cos, sin = (t.to(dev) for t in rope_tables(B, S, CFG.head_dim, torch.bfloat16))
    mask = causal_mask(B, S, S, torch.bfloat16).to(dev)
    with torch.no_grad():
        m.fused_probabilities = True
        y1, w1 = m(x, (cos, sin), mask)
        m.fused_probabilities = False  # the default
        y0, w0 = m(x, (cos, sin), mask)
    assert float((w1.float() - w0.float()).abs().max()) <= 2 ** -7
    assert float((w1 == w0).float().mean()) > 0.99
    assert float((y1.float() - y0.float()).abs().max() / y0.float().abs().max()) < 1e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["mxint", "mxfp"])
def test_qwen3_attention_matches_the_oracle(dev, dtype, kind):
    """the Qwen3 form: RMSNorm over head_dim on the projected queries and keys before the rotary embedding"""
    from mase_amd.quantized import Qwen3AttentionMXFP, Qwen3AttentionMXInt

    cls, qc = (Qwen3AttentionMXInt, Q_INT) if kind == "mxint" else (Qwen3AttentionMXFP, Q_FP)
    tol = 5e-3 if dtype == torch.float32 else 3e-2
    m = cls(CFG, layer_idx=3, q_config=qc).to(dtype)
    assert {"q_norm.weight", "k_norm.weight"} <= set(m.state_dict())
    sd = seeded(m, 31, dtype)
    m.load_state_dict(sd, strict=True)
    m = m.to(dev).eval()
    g = torch.Generator().manual_seed(32)
    B, S = 2, 64
    x = torch.randn(B, S, CFG.hidden_size, generator=g).to(dtype)
    cos, sin = rope_tables(B, S, CFG.head_dim, dtype)
    mask = causal_mask(B, S, S, dtype)
    with torch.no_grad():
        y, w = m(x.to(dev), (cos.to(dev), sin.to(dev)), mask.to(dev))
    ref, wref = OL.attention_forward(kind, sd, x, cos, sin, mask, 8, 4, qc, qk_norm_eps=CFG.rms_norm_eps)
    plain, _ = OL.attention_forward(kind, sd, x, cos, sin, mask, 8, 4, qc)
    assert rel_err(y, ref) < tol, (kind, dtype, rel_err(y, ref))
    assert rel_err(y, plain) > 10 * tol  # the norms do act
    assert float((w.float().cpu() - wref.float()).abs().max()) <= (2 ** -6 if kind == "mxint" else 2 ** -3)


def test_qwen3_registry_and_pass(dev):
    from mase_amd.passes import quantize_module_transform_pass
    from mase_amd.quantized import Qwen3AttentionMXInt, Qwen3MLPMXInt, Qwen3RMSNormMinifloat, quantized_module_map

    for key in ("qwen3_self_attention_mxfp", "qwen3_self_attention_mxint", "qwen3_rms_norm_minifloat", "qwen3_mlp_mxfp",
                "qwen3_mlp_mxint"):
        assert key in quantized_module_map

    class Qwen3RMSNorm(torch.nn.Module):
        def __init__(self, n):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.ones(n))

    class Qwen3MLP(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.gate_proj = torch.nn.Linear(256, 512, bias=False)
            self.up_proj = torch.nn.Linear(256, 512, bias=False)
            self.down_proj = torch.nn.Linear(512, 256, bias=False)

    class Qwen3Attention(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.layer_idx = 0
            self.q_proj = torch.nn.Linear(256, 256, bias=False)
            self.k_proj = torch.nn.Linear(256, 128, bias=False)
            self.v_proj = torch.nn.Linear(256, 128, bias=False)
            self.o_proj = torch.nn.Linear(256, 256, bias=False)
            self.q_norm, self.k_norm = Qwen3RMSNorm(32), Qwen3RMSNorm(32)

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.config = CFG
            self.self_attn, self.mlp, self.norm = Qwen3Attention(), Qwen3MLP(), Qwen3RMSNorm(256)

    net = Block().to(dev)
    wq = net.self_attn.q_norm.weight.data.normal_().clone()
    args = {"by": "regex_name",
            r"self_attn$": {"config": {"name": "mxint", **Q_INT}},
            r"mlp$": {"config": {"name": "mxint", **MINI}},
            r"^norm$": {"config": {"name": "minifloat", "weight_exponent_width": 5, "weight_frac_width": 8, **MINI}}}
    net, _ = quantize_module_transform_pass(net, args)
    assert isinstance(net.self_attn, Qwen3AttentionMXInt) and isinstance(net.mlp, Qwen3MLPMXInt)
    assert isinstance(net.norm, Qwen3RMSNormMinifloat)
    assert torch.equal(net.self_attn.q_norm.weight.data, wq)


@pytest.mark.parametrize("kind", ["mxint", "mxfp"])
def test_attention_contractions_run_on_the_batched_kernel_of_this_package(dev, monkeypatch, kind):
    """bf16 modules: query x keys and probabilities x values both go through mase_gemm_bf16_tn_batched (prefill, and
    decode against a cache whose length is not a multiple of 64); torch.matmul is not called at all.  fp32 modules keep
    torch.matmul: their keys and values are not bf16 values."""
    from mase_amd import _gemm
    from mase_amd.quantized import LlamaAttentionMXFP, LlamaAttentionMXInt

    cls, q = (LlamaAttentionMXInt, Q_INT) if kind == "mxint" else (LlamaAttentionMXFP, Q_FP)
    calls = []
    real = _gemm.gemm_bf16_tn_batched
    monkeypatch.setattr(_gemm, "gemm_bf16_tn_batched", lambda a, b, **kw: (calls.append((tuple(a.shape), tuple(b.shape))), real(a, b, **kw))[1])
    library = []
    real_matmul = torch.matmul
    monkeypatch.setattr(torch, "matmul", lambda *a, **k: (library.append(1), real_matmul(*a, **k))[1])
    for dtype, own in ((torch.bfloat16, True), (torch.float32, False)):
        m = cls(CFG, layer_idx=0, q_config=q).to(dtype)
        m.load_state_dict(seeded(m, 5, dtype))
        m = m.to(dev).eval()
        B, S = 2, 70
        x = torch.randn(B, S, CFG.hidden_size, generator=torch.Generator().manual_seed(6)).to(dtype).to(dev)
        cos, sin = (t.to(dev) for t in rope_tables(B, S, CFG.head_dim, dtype))
        calls.clear(), library.clear()
        with torch.no_grad():
            m(x, (cos, sin), causal_mask(B, S, S, dtype).to(dev))
        if own:
            # head_dim 32 is padded to one K tile of 64; 70 keys to 128
            assert calls == [((B, 8, S, 64), (B, 8, S, 64)), ((B, 8, S, 128), (B, 8, CFG.head_dim, 128))] and library == []
        else:
            assert calls == [] and len(library) == 2
