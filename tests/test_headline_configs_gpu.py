"""Parity at the headline configurations' full sizes, on the same seeded inputs the benchmark uses.

Configurations 1 and 2 (quantize-dequantize) are compared bit for bit with the CPU oracle over the whole tensor.
Configuration 3 (MXINT8 Linear 4096^3) is compared with the oracle's forward within 1e-2 (measured ~1e-6).
Configuration 4 (MXFP8 x MXFP4 Linear, M=8192 K=8192 N=28672) is too large for the CPU oracle to finish in seconds,
so it is checked on a slice that is: the first 256 activation rows against the first 2048 weight rows, taken from
the full-size operands (rows are independent in both quantizers and in the product), plus size-independent
properties of the full-size result (finite, row slices agree with the sliced computation).
Configuration 5 (decoder layer, batch 8 x seq 2048) runs at full size on the GPU; each of its seven Linears is checked
on the first and the last 256 tokens against the oracle's forward of exactly the rows the GPU Linear was fed; the
attention kernel is checked inside the layer on two (batch, head) pairs against the tensor operations in fp32 at the
full 2048 tokens; and the layer output rows of the first and last 256 tokens are compared with the CPU layer (oracle
Linears) continued from the attention output the GPU produced for those tokens."""
import pytest
import torch

import bench
import oracle as O
from oracle import linear as OL
from oracle import llama as OLL
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


def test_config5_decoder_layer_full_size_linear_slices(dev):
    """The layer the benchmark times, at batch 8 x seq 2048 (16384 tokens): forward hooks record, for each of the seven
    Linears, the first and last 256 rows of its input and output; the oracle's LinearMXInt forward of those input rows
    (rows are independent in the quantizer and in the product) must give the same output rows.  Bound, per Linear:
    max|y - y_ref| / max|y_ref| <= 1e-2; measured: the outputs are bf16 roundings of fp32 sums that differ only in
    summation order, so all but a few per million are bit-identical and the rest are one bf16 step apart, which is
    asserted too.  Every contraction must have taken the tiled kernel on the fragment-ordered weight."""
    from mase_amd._gemm import gemm_bf16_takes_packed_b
    from mase_amd.passes import quantize_module_transform_pass
    from mase_amd.quantized import LinearMXInt

    w = bench.DecoderLayerMxint()
    layer = w.build(torch, dev)
    cpu_weights = {n: m.weight.data.cpu() for n, m in layer.named_children() if isinstance(m, torch.nn.Linear)}
    layer, _ = quantize_module_transform_pass(layer, {"by": "type", "linear": {"config": dict(w.cfg, name="mxint")}})
    names = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")
    assert all(isinstance(getattr(layer, n), LinearMXInt) for n in names)
    tok, S = w.B * w.T, 256
    seen = {}

    def hook(name):
        def fn(mod, inp, out):
            i2, o2 = inp[0].reshape(tok, -1), out.reshape(tok, -1)
            seen[name] = (torch.cat((i2[:S], i2[-S:])).cpu(), torch.cat((o2[:S], o2[-S:])).cpu())
        return fn

    hooks = [getattr(layer, n).register_forward_hook(hook(n)) for n in names]
    x = torch.randn(w.B, w.T, 4096, generator=torch.Generator().manual_seed(4)).bfloat16()
    from mase_amd.quantizers import _ops

    PAIRS = ((0, 0), (w.B - 1, 31))
    attn_seen = []  # per call of the attention kernel: its options and, for PAIRS, operand and result slices
    real_attention = _ops.attention_causal

    def recording_attention(q, k, v, scaling=None, mxint_bits=None, q_rope=None):
        out = real_attention(q, k, v, scaling, mxint_bits=mxint_bits, q_rope=q_rope)
        sl = lambda t: [t[b:b + 1, h:h + 1] for b, h in PAIRS]
        attn_seen.append(dict(mxint_bits=mxint_bits, q_rope=q_rope, q=sl(q), k=sl(k), v=sl(v), out=[t.clone() for t in sl(out)]))
        return out

    _ops.attention_causal = recording_attention
    try:
        with torch.no_grad():
            layer.fuse_producers = False  # every Linear quantizes its own input; q rotated before the attention call
            y = layer(x.to(dev))
            for h in hooks:
                h.remove()
            layer.fuse_producers = True
            y_fused = layer(x.to(dev))
    finally:
        _ops.attention_causal = real_attention
    _check_config5_attention(attn_seen, w.T, dev)
    _check_config5_rows_after_attention(w, x, y_fused, seen["o_proj"][0], S)
    # the Linears are checked on the plain tensors they receive when each quantizes its own input; the layer as the
    # benchmark runs it (RMSNorm, the SwiGLU product and the attention kernel writing the quantized form) must give the
    # same bits
    assert torch.equal(y_fused.view(torch.int16), y.view(torch.int16))
    assert y.shape == x.shape and y.dtype == torch.bfloat16 and bool(torch.isfinite(y).all())
    assert len(seen) == 7
    for n in names:
        m = getattr(layer, n)
        N, K = m.weight.shape
        assert gemm_bf16_takes_packed_b(tok, N, K), n
        assert m._w_cache._packed is not None, f"{n}: the forward did not use the fragment-ordered weight"
        qw, _ = OL.mxint_prepare_weights(cpu_weights[n], None, w.cfg)
        assert_bits_equal(m.weight.data, qw, f"config 5 {n} weight")
        inp, out = seen[n]
        ref = OL.linear_mxint_forward(inp, qw, None, w.cfg)
        e = rel_err(out, ref)
        differ = out.view(torch.int16) != ref.view(torch.int16)
        n_diff = int(differ.sum())
        # the ones that differ sit on a rounding boundary of the fp32 sum: neighbouring bf16 values
        step = (out.view(torch.int16).int() - ref.view(torch.int16).int()).abs()[differ]
        print(f"config 5 {n} [{tok}x{K}]x[{N}x{K}]: rel err {e:.3e}, {n_diff} of {out.numel()} outputs not bit-identical",
              flush=True)
        assert e < 1e-2, n
        assert n_diff <= out.numel() * 1e-4 and (n_diff == 0 or int(step.max()) == 1), n


def _check_config5_attention(attn_seen, T, dev):
    """The two forwards of the layer called the attention kernel once each: plain (q rotated by rope() before the call)
    and fused (q rotated on load, result in o_proj's MXINT8 form).  For each recorded (batch, head) pair, at the full
    2048 tokens: the plain result against softmax(q k^T / sqrt(128) + causal mask) v in fp32 on the same bf16 operands,
    bound 1e-2 of the result's range; the fused result bit for bit equal to the MXINT8 quantizer (CPU oracle) applied to
    the plain kernel's result on the rotated q."""
    from mase_amd.quantizers import _ops

    assert len(attn_seen) == 2
    plain, fused = attn_seen
    assert plain["mxint_bits"] is None and plain["q_rope"] is None
    assert fused["mxint_bits"] == 8 and fused["q_rope"] is not None
    cos, sin = fused["q_rope"]
    for i in range(len(plain["q"])):
        q, k, v = plain["q"][i], plain["k"][i], plain["v"][i]
        s = (q.float() @ k.float().transpose(-1, -2)) * 128 ** -0.5
        s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool, device=dev), 1), float("-inf"))
        ref = torch.softmax(s, -1) @ v.float()
        e = float((plain["out"][i].float() - ref).abs().max() / ref.abs().max())
        print(f"config 5 attention kernel inside the layer, pair {i}, {T} tokens: err {e:.3e} of the range vs fp32", flush=True)
        assert e < 1e-2
        # the fused call received q before its rotation: rope() of it is the q of the plain call
        assert torch.equal(_ops.rope(fused["q"][i], cos, sin), q)
        assert torch.equal(fused["k"][i], k) and torch.equal(fused["v"][i], v)
        want = O.mxint_quantizer(plain["out"][i].transpose(1, 2).reshape(1, T, 128).cpu(), 32, 8, block_dim=-1)
        assert_bits_equal(fused["out"][i].transpose(1, 2).reshape(1, T, 128), want, f"config 5 fused attention output, pair {i}")


def _check_config5_rows_after_attention(w, x, y_gpu, attn_rows, S):
    """Everything after the attention core is row-wise: the CPU layer (oracle Linears, torch's RMSNorm / SiLU
    arithmetic) continued from the attention output the GPU layer produced for the first and last S tokens must give
    the GPU layer's output rows for those tokens: max|y - y_ref| / max|y_ref| <= 1e-2."""
    from test_decoder_layer_gpu import swap_in_oracle

    cpu = swap_in_oracle(w.build(torch, None), w.cfg)
    tok = w.B * w.T
    xr = x.reshape(tok, -1)
    xr = torch.cat((xr[:S], xr[-S:]))
    with torch.no_grad():
        h = xr + cpu.o_proj(attn_rows)
        n = cpu.post_attention_layernorm(h)
        ref = h + cpu.down_proj(torch.nn.functional.silu(cpu.gate_proj(n)) * cpu.up_proj(n))
    yr = y_gpu.reshape(tok, -1)
    got = torch.cat((yr[:S], yr[-S:])).cpu()
    e = rel_err(got, ref)
    n_diff = int((got.view(torch.int16) != ref.view(torch.int16)).sum())
    print(f"config 5 layer output rows (first / last {S} tokens) vs the CPU layer continued from the GPU's attention "
          f"output: rel err {e:.3e}, {n_diff} of {got.numel()} elements not bit-identical", flush=True)
    assert e < 1e-2
