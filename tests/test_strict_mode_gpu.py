"""The two default-on paths whose results are not the reference's bit for bit, and their switches.

LinearMXFP on the block-scaled matrix instruction (``native_mx``, default True) deviates in two modelled ways: blocks
that hold a code the OCP formats reserve are stored one scale up with halved codes, and the instruction truncates
products about 12 bits below the largest of a group of eight.  On inputs whose products and sums are exact in fp32
neither deviation can act, so both the instruction path and the bf16 path (``native_mx=False``) must return the
oracle's bits; on inputs built so that only the re-expression acts, the instruction path must equal an emulation of it
and stay within one element step of the block per term.  The one-pass attention probabilities
(``fused_probabilities``, opt-in) are compared with the separate passes (the default) and both with the oracle.
"""
import pytest
import torch
import torch.nn.functional as F

from oracle import linear as OL
from oracle import quantizers as OQ
from helpers import assert_bits_equal

pytestmark = pytest.mark.gpu

CFG = {"weight_block_size": 32, "weight_exponent_width": 2, "weight_frac_width": 1,
       "data_in_block_size": 32, "data_in_exponent_width": 4, "data_in_frac_width": 3}


def exact_operands(M, N, K, seed, top_code_every=0):
    """x on the e4m3 grid and w on the e2m1 grid of their blocks, spread over so few binades that every product and
    every partial sum of a row is exact in fp32 in any order.  ``top_code_every`` = n puts the largest e4m3 magnitude
    (code S.1111.111, which OCP e4m3 reserves) at the head of every n-th block of x."""
    g = torch.Generator().manual_seed(seed)
    nb = K // 32

    def pick(shape, choices):
        return torch.tensor(choices)[torch.randint(0, len(choices), shape, generator=g)]

    sign = lambda shape: pick(shape, [-1.0, 1.0])
    x = sign((M, nb, 32)) * pick((M, nb, 32), [m / 8 for m in range(8, 15)]) * pick((M, nb, 32), [1.0, 2.0])
    x[:, :, 1] = x[:, :, 1].sign() * 2.5  # the block maximum sits in the upper binade, below the top code
    x = x * pick((M, nb, 1), [0.5, 1.0, 2.0])
    if top_code_every:
        x[:, ::top_code_every, 0] = 3.75 * x[:, ::top_code_every, 1].abs() / 2.5  # 1.875 * 2^(binade of the maximum)
    w = sign((N, nb, 32)) * pick((N, nb, 32), [1.0, 1.5]) * pick((N, nb, 32), [1.0, 2.0])
    w[:, :, 2] = 3.0
    w = w * pick((N, nb, 1), [0.25, 0.5, 1.0])
    return x.reshape(M, K), w.reshape(N, K)


def build(dev, w, native, dtype=torch.float32):
    from mase_amd.quantized import LinearMXFP

    m = LinearMXFP(w.shape[1], w.shape[0], bias=False, device=dev, dtype=dtype, config=dict(CFG, native_mx=native))
    m.load_state_dict({"weight": w.to(dtype)})
    return m


@pytest.mark.parametrize("top_code_every", [0, 2])
def test_linear_mxfp_bit_for_bit_where_the_sums_are_exact(dev, top_code_every):
    M, N, K = 192, 128, 256
    x, w = exact_operands(M, N, K, 5, top_code_every)
    qw, _ = OL.mxfp_prepare_weights(w, None, CFG)
    assert torch.equal(qw, w)  # the operands are on their grids: quantization changes nothing
    sc, el = OQ.mxfp_components(x.reshape(-1, 32), 32, 4, 3)
    has_top = ((el & 0x7F) == 0x7F).any(1)
    assert bool(has_top.any()) == bool(top_code_every)
    ref = OL.linear_mxfp_forward(x, qw, None, CFG)
    assert torch.equal(ref, F.linear(x.double(), w.double()).float())  # exact: no rounding anywhere
    strict = build(dev, w, native=False)
    native = build(dev, w, native=True)
    assert native._w_packed.valid_for(native.weight) and not strict._w_packed.valid_for(strict.weight)
    assert_bits_equal(strict(x.to(dev)), ref, "LinearMXFP native_mx=False")
    # halving a code with exponent field >= 2 is exact, so re-expressed blocks change nothing here either
    assert_bits_equal(native(x.to(dev)), ref, "LinearMXFP on the block-scaled instruction")


def test_linear_mxfp_reserved_code_blocks_follow_the_modelled_re_expression(dev):
    """Every block of x holds the top code at position 0 and values in the subnormal range of its scale elsewhere; the
    weight is zero against position 0..7 (the top code's group of eight products), so the output is made of the small
    elements only and the one-scale-up re-expression (round half to even to twice the step) is what the two paths
    differ by."""
    M, N, K = 128, 128, 512
    g = torch.Generator().manual_seed(11)
    nb = K // 32
    top = 480.0 * torch.exp2(torch.randint(-12, -4, (M, nb, 1), generator=g).float())  # 1.875 * 2^8 * 2^sh
    step = top / 480.0 * 2.0 ** -9                                                     # the block's subnormal step
    # multiples of the step that the reference's cast keeps: it flushes magnitudes up to 4 steps (2^-bias) to zero
    k = torch.tensor([0.0] + [float(v) for v in range(5, 16)])[torch.randint(0, 12, (M, nb, 32), generator=g)]
    x = step * k * (torch.randint(0, 2, (M, nb, 32), generator=g).float() * 2 - 1)
    x[:, :, 0:1] = top
    x = x.reshape(M, K)
    _, w = exact_operands(M, N, K, 12)
    w = w.reshape(N, nb, 32)
    w[:, :, :8] = 0
    w = w.reshape(N, K)
    qw, _ = OL.mxfp_prepare_weights(w, None, CFG)
    qx = OQ.mxfp_quantizer(x, 32, 4, 3)
    assert torch.equal(qx, x) and torch.equal(qw, w)
    ref = OL.linear_mxfp_forward(x, qw, None, CFG)
    # the re-expression: values below the smallest normal of the old scale go to multiples of twice the step
    st = step.expand(M, nb, 32).reshape(M, K)
    small = x.abs() < 16 * st
    x_re = torch.where(small, torch.round(x / (2 * st)) * (2 * st), x)
    expect = F.linear(x_re.double(), w.double()).float()
    y_native = build(dev, w, native=True)(x.to(dev)).cpu()
    y_strict = build(dev, w, native=False)(x.to(dev)).cpu()
    scale = float(ref.abs().max())
    assert float((y_strict - ref).abs().max()) <= 1e-6 * scale
    # the instruction path is the emulation up to the truncation inside groups of eight products ...
    trunc = 7 * 2.0 ** -12 * F.linear(x_re.abs().double(), w.abs().double()).float()
    assert bool(((y_native - expect).abs() <= trunc + 1e-6 * scale).all())
    # ... it does differ from the reference's values, by at most one step of the block per term
    bound = F.linear((small * st).double(), w.abs().double()).float()
    assert bool(((y_native - ref).abs() <= bound + trunc + 1e-6 * scale).all())
    assert float((y_native - ref).abs().max()) > 1e-3 * scale
    print(f"re-expressed blocks: |native - reference| max {float((y_native - ref).abs().max()) / scale:.2e} of the "
          f"output range, |native - emulation| max {float((y_native - expect).abs().max()) / scale:.2e}")


@pytest.mark.parametrize("fused", [False, True])
def test_attention_probabilities_against_the_oracle(dev, fused):
    """fused_probabilities=False (the default) runs cast, fp32 softmax and MX quantization as separate passes, the
    softmax being the library's own on the device: what is left between them and the oracle is the device's exp and GEMM
    summation order against the host's.  The one-pass kernel (opt-in) must meet the same bound."""
    from mase_amd.quantized import LlamaAttentionMXInt
    from oracle import llama as OLL
    from test_llama_modules_gpu import CFG as LCFG, Q_INT, causal_mask, rope_tables, seeded

    m = LlamaAttentionMXInt(LCFG, layer_idx=3, q_config=Q_INT).to(torch.bfloat16)
    sd = seeded(m, 41, torch.bfloat16)
    m.load_state_dict(sd)
    m = m.to(dev).eval()
    m.fused_probabilities = fused
    g = torch.Generator().manual_seed(42)
    B, S = 2, 160
    x = torch.randn(B, S, LCFG.hidden_size, generator=g).bfloat16()
    cos, sin = rope_tables(B, S, LCFG.head_dim, torch.bfloat16)
    mask = causal_mask(B, S, S, torch.bfloat16)
    with torch.no_grad():
        y, w = m(x.to(dev), (cos.to(dev), sin.to(dev)), mask.to(dev))
    ref, wref = OLL.attention_forward("mxint", sd, x, cos, sin, mask, 8, 4, Q_INT)
    w, y = w.cpu().float(), y.cpu().float()
    same = float((w == wref.float()).float().mean())
    print(f"attention probabilities fused={fused}: {same:.4f} of elements equal to the oracle's")
    assert same > 0.98 and float((w - wref.float()).abs().max()) <= 2 ** -6
    assert float((y - ref.float()).abs().max() / ref.float().abs().max()) < 3e-2
