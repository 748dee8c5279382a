"""The hot path under HIP graph capture: a quantized Linear forward and a quantize-dequantize call are recorded once
(after a warm-up call, which sets kernel attributes and builds the cached tables) and replayed with new input
contents; every replay must equal the eager result bit for bit."""
import pytest
import torch

pytestmark = pytest.mark.gpu

MXINT = {"weight_block_size": 32, "weight_width": 8, "data_in_block_size": 32, "data_in_width": 8}
MXFP = {"weight_block_size": 32, "weight_exponent_width": 2, "weight_frac_width": 1,
        "data_in_block_size": 32, "data_in_exponent_width": 4, "data_in_frac_width": 3}


@pytest.mark.parametrize("kind", ["mxint", "mxfp"])
def test_linear_forward_replays_from_a_graph(dev, kind):
    from mase_amd.quantized import LinearMXFP, LinearMXInt
    import mase_amd.quantizers as Q

    g = torch.Generator().manual_seed(21)
    w = torch.randn(512, 1024, generator=g) * 0.02
    m = (LinearMXInt if kind == "mxint" else LinearMXFP)(1024, 512, bias=False, device=dev, dtype=torch.bfloat16,
                                                         config=dict(MXINT if kind == "mxint" else MXFP))
    m.load_state_dict({"weight": w.bfloat16()})
    xs = [torch.randn(300, 1024, generator=g).bfloat16().to(dev) for _ in range(3)]
    static_x = xs[0].clone()
    kw = dict(width=8, exponent_width=8, exponent_bias=None, block_size=[1, 16], skip_first_dim=True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # warm-up on the capture stream
        m(static_x)
        Q.block_fp_quantizer(static_x, **kw)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = m(static_x)
        static_q = Q.block_fp_quantizer(static_x, **kw)
    for x in xs + xs[:1]:
        static_x.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        eager_y = m(x)
        eager_q = Q.block_fp_quantizer(x, **kw)
        torch.cuda.synchronize()
        assert torch.equal(static_y.view(torch.int16), eager_y.view(torch.int16))
        assert torch.equal(static_q.view(torch.int16), eager_q.view(torch.int16))


@pytest.mark.parametrize("kind", ["mxint", "mxint-codes", "mxfp4"])
def test_decode_sized_forward_replays_from_a_graph(dev, kind):
    """16 rows of activations take the weight-streaming kernels (split-K partial sums in a workspace + a reduction):
    the forward is recorded once and replayed with new inputs, with eager work and synchronisation between replays."""
    from mase_amd.quantized import LinearMXFP, LinearMXInt

    g = torch.Generator().manual_seed(22)
    w = torch.randn(1536, 2048, generator=g) * 0.02
    if kind == "mxfp4":
        m = LinearMXFP(2048, 1536, bias=True, device=dev, dtype=torch.bfloat16, config=dict(MXFP))
    else:
        cfg = dict(MXINT, packed_decode=(kind == "mxint-codes"))
        m = LinearMXInt(2048, 1536, bias=True, device=dev, dtype=torch.bfloat16, config=cfg)
    m.load_state_dict({"weight": w.bfloat16(), "bias": (torch.randn(1536, generator=g) * 0.1).bfloat16()})
    xs = [torch.randn(16, 2048, generator=g).bfloat16().to(dev) for _ in range(3)]
    static_x = xs[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        m(static_x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = m(static_x)
    for x in xs + xs[:1]:
        static_x.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        eager_y = m(x)
        torch.cuda.synchronize()
        assert torch.equal(static_y.view(torch.int16), eager_y.view(torch.int16))
