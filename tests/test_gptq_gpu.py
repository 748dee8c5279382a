"""GPU tests of the GPTQ pre-pass: the per-layer algorithm against the CPU oracle, and the driver on a small causal LM."""
import copy

import pytest
import torch

import oracle as O
from oracle import gptq as G

pytestmark = pytest.mark.gpu

MXINT4 = {"weight_block_size": 32, "weight_width": 4}
MXFP4 = {"weight_block_size": 32, "weight_exponent_width": 2, "weight_frac_width": 1}


def correlated_inputs(g, n, tokens, cols):
    mix = torch.randn(cols, cols, generator=g) * 0.3 + torch.eye(cols)
    return [torch.randn(2, tokens, cols, generator=g) @ mix for _ in range(n)]


@pytest.mark.parametrize("fmt,cfg", [("mxint", MXINT4), ("mxfp", MXFP4)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gptq_layer_against_the_oracle(dev, fmt, cfg, dtype):
    """Same Gram matrix on both sides (accumulated on the device, copied to the host; the oracle's Hessian is that
    matrix times 2 / samples, a scale the result does not depend on): the column walk must then agree except where the
    device's blocked fp32 updates and the host's group-by-group updates in the weight dtype round differently and an
    element sits on a rounding boundary; the proxy loss must agree closely and beat plain quantization like the oracle's."""
    from mase_amd.passes.gptq import InputGram, group_quantizer, round_weight

    g = torch.Generator().manual_seed(3)
    lin = torch.nn.Linear(256, 96, bias=False)
    lin.weight.data = (torch.randn(96, 256, generator=g) * 0.05).to(dtype)
    xs = correlated_inputs(g, 4, 64, 256)
    dlin = copy.deepcopy(lin).to(dev)
    gram = InputGram()
    for x in xs:
        gram.update(x.to(dev).to(dtype))
    assert gram.rows_seen == 4 * 2 * 64
    n_batch_items = sum(x.shape[0] for x in xs)
    H = gram.matrix.cpu() * (2.0 / n_batch_items)   # the oracle's normalisation
    Hh = G.hessian([x.to(dtype) for x in xs])
    assert float((H - Hh).abs().max() / Hh.abs().max()) < 1e-4
    q = round_weight(dlin.weight.data, gram.matrix, 32, group_quantizer(fmt, cfg, True)).cpu()
    assert q.dtype == dtype
    want = G.fasterquant(lin.weight.data, H, fmt, cfg)
    same = float((q == want).float().mean())
    lq, lw = G.proxy_loss(lin.weight.data.float(), q.float(), H), G.proxy_loss(lin.weight.data.float(), want.float(), H)
    rtn = G.proxy_loss(lin.weight.data.float(), G.quantize_group(lin.weight.data, fmt, cfg, True).float(), H)
    print(f"gptq {fmt} {dtype}: {same:.4f} of the weights identical; proxy loss {lq:.4e} (oracle {lw:.4e}, plain {rtn:.4e})")
    # bf16 weights: the oracle (like the reference) keeps its working copy in bf16 and rounds every fed-forward
    # correction to it, the pass keeps it in fp32 and rounds each group once when it is quantized: a few per cent of the
    # weights land on the neighbouring code, the loss is the same
    assert same > (0.999 if dtype == torch.float32 else 0.9)
    assert abs(lq - lw) < 0.05 * lw and lq < 0.9 * rtn
    # the first group has seen no feedback: identical bit for bit
    assert torch.equal(q[:, :32], want[:, :32])


def test_gptq_without_search_and_with_a_dead_column(dev):
    from mase_amd.passes.gptq import InputGram, group_quantizer, round_weight

    g = torch.Generator().manual_seed(4)
    lin = torch.nn.Linear(128, 64, bias=False).to(dev)
    xs = correlated_inputs(g, 2, 32, 128)
    for x in xs:
        x[..., 7] = 0.0
    gram = InputGram()
    for x in xs:
        gram.update(x.to(dev))
    H = gram.matrix.cpu().clone()
    w8 = {"weight_block_size": 32, "weight_width": 8}
    q = round_weight(lin.weight.data, gram.matrix, 32, group_quantizer("mxint", w8, False)).cpu()
    # one panel of all groups = the unblocked feed-forward: the same weights up to the rounding of the partial sums
    q1 = round_weight(lin.weight.data, gram.matrix, 32, group_quantizer("mxint", w8, False), panel_groups=1).cpu()
    assert float((q == q1).float().mean()) > 0.999
    want = G.fasterquant(lin.weight.data.cpu(), H, "mxint", {"weight_block_size": 32, "weight_width": 8}, quant_search=False)
    assert bool((q[:, 7] == 0).all())
    assert float((q == want).float().mean()) > 0.97
    # clip_search_y: the search of every column group scored on the layer's calibration inputs
    gram = InputGram(keep_inputs=True)
    for x in xs:
        gram.update(x.reshape(1, -1, x.shape[-1]).to(dev))
    act = torch.stack([x.reshape(-1, x.shape[-1]) for x in xs])
    assert torch.equal(gram.calibration().cpu(), act)
    q_y = round_weight(lin.weight.data, gram.matrix, 32, group_quantizer("mxint", MXINT4, True, cali_batch_size=2),
                       calibration=gram.calibration()).cpu()
    want_y = G.fasterquant(lin.weight.data.cpu(), H, "mxint", MXINT4, activation=act, cali_batch_size=2)
    assert float((q_y[:, :32] == want_y[:, :32]).float().mean()) > 0.97   # the first column group sees identical inputs
    assert float((q_y == want_y).float().mean()) > 0.9
    assert G.proxy_loss(lin.weight.data.cpu(), q_y, H) < 1.1 * G.proxy_loss(lin.weight.data.cpu(), want_y, H)


def test_run_gptq_on_a_small_causal_lm(dev):
    """the driver over a transformers Llama (random weights, synthetic token ids): every nn.Linear of the decoder
    layers is rewritten, and on the calibration data the rewritten model is closer to the original than the same
    model with plainly quantized weights; the quantize pass with a "gptq" entry then swaps the modules in without
    quantizing the weights again"""
    from transformers import LlamaConfig, LlamaForCausalLM

    from mase_amd.passes import quantize_module_transform_pass
    from mase_amd.passes.gptq import group_quantizer, linear_modules, run_gptq
    from mase_amd.quantized.modules.linear import LinearMXInt

    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=128, intermediate_size=256, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, vocab_size=128, max_position_embeddings=128)
    base = LlamaForCausalLM(cfg).to(dev).eval()
    data = torch.randint(0, 128, (6, 48), generator=torch.Generator().manual_seed(1))
    gcfg = {"model_name": "synthetic", "device": str(dev), "format": "mxint", "weight_config": MXINT4,
            "calibration_data": data, "quantile_search": True}

    from mase_amd.passes import gptq as gptq_mod

    updates = []
    real_update = gptq_mod.InputGram.update
    gptq_mod.InputGram.update = lambda self, x: (updates.append(tuple(x.shape)), real_update(self, x))[1]
    try:
        tuned = run_gptq(copy.deepcopy(base), dict(gcfg))
    finally:
        gptq_mod.InputGram.update = real_update
    # q / k / v and gate / up read one tensor each: 4 Gram matrices per layer, each fed once per sample
    assert len(updates) == 2 * 4 * 6, len(updates)
    plain = copy.deepcopy(base)
    plain_quantizer = group_quantizer("mxint", MXINT4, True)
    for layer in plain.model.layers:
        for lin in linear_modules(layer).values():
            lin.weight.data.copy_(plain_quantizer(lin.weight.data))
    changed = 0
    for lt, lb in zip(tuned.model.layers, base.model.layers):
        for (n, mt), mb in zip(linear_modules(lt).items(), linear_modules(lb).values()):
            assert mt.weight.shape == mb.weight.shape and not torch.equal(mt.weight, mb.weight), n
            changed += 1
    assert changed == 14
    assert tuned.config.use_cache == base.config.use_cache

    def hidden(model):
        with torch.no_grad():
            return model.model(data.to(dev)).last_hidden_state.float()

    ref = hidden(base)
    e_tuned = float((hidden(tuned) - ref).pow(2).mean())
    e_plain = float((hidden(plain) - ref).pow(2).mean())
    print(f"hidden-state MSE against the unquantized model: GPTQ {e_tuned:.4e}, plain clip search {e_plain:.4e}")
    assert e_tuned < e_plain

    pass_args = {"gptq": dict(gcfg), "by": "type",
                 "linear": {"config": {"name": "mxint", "gptq": True, "weight_block_size": 32, "weight_width": 4,
                                       "data_in_block_size": 32, "data_in_width": 8}}}
    swapped, _ = quantize_module_transform_pass(copy.deepcopy(base), pass_args)
    mods = [m for m in swapped.model.layers.modules() if isinstance(m, LinearMXInt)]
    assert len(mods) == 14
    want = linear_modules(tuned.model.layers[1])["mlp.down_proj"].weight
    assert torch.equal(swapped.model.layers[1].mlp.down_proj.weight, want)
    with pytest.raises(NotImplementedError):
        run_gptq(copy.deepcopy(base), {**gcfg, "calibration_data": None})
    tuned_y = run_gptq(copy.deepcopy(base), {**gcfg, "clip_search_y": True, "cali_batch_size": 4})
    e_y = float((hidden(tuned_y) - ref).pow(2).mean())
    print(f"hidden-state MSE with clip_search_y: {e_y:.4e}")
    assert e_y < e_plain
