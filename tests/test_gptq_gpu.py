"""GPU tests of the GPTQ pre-pass: the per-layer algorithm against the CPU oracle, and the driver on a small causal LM."""
import copy
import os

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
    """Same Hessian on both sides (accumulated on the device, copied to the host): the column walk must then agree
    except where the device's and the host's rank-32 updates round differently and an element sits on a rounding
    boundary; the proxy loss must agree closely and beat plain quantization like the oracle's."""
    from mase_amd.passes.gptq import GPTQ

    g = torch.Generator().manual_seed(3)
    lin = torch.nn.Linear(256, 96, bias=False)
    lin.weight.data = (torch.randn(96, 256, generator=g) * 0.05).to(dtype)
    xs = correlated_inputs(g, 4, 64, 256)
    dlin = copy.deepcopy(lin).to(dev)
    gp = GPTQ(dlin)
    for x in xs:
        gp.add_batch(x.to(dev).to(dtype))
    H = gp.H.cpu().clone()
    Hh = G.hessian([x.to(dtype) for x in xs])
    assert float((H - Hh).abs().max() / Hh.abs().max()) < 1e-4
    q = gp.fasterquant(None, fmt, cfg).cpu()
    want = G.fasterquant(lin.weight.data, H, fmt, cfg)
    same = float((q == want).float().mean())
    lq, lw = G.proxy_loss(lin.weight.data.float(), q.float(), H), G.proxy_loss(lin.weight.data.float(), want.float(), H)
    rtn = G.proxy_loss(lin.weight.data.float(), G.quantize_group(lin.weight.data, fmt, cfg, True).float(), H)
    print(f"gptq {fmt} {dtype}: {same:.4f} of the weights identical; proxy loss {lq:.4e} (oracle {lw:.4e}, plain {rtn:.4e})")
    assert same > (0.999 if dtype == torch.float32 else 0.99)
    assert abs(lq - lw) < 0.05 * lw and lq < 0.9 * rtn
    # the first group has seen no feedback: identical bit for bit
    assert torch.equal(q[:, :32], want[:, :32])


def test_gptq_without_search_and_with_a_dead_column(dev):
    from mase_amd.passes.gptq import GPTQ

    g = torch.Generator().manual_seed(4)
    lin = torch.nn.Linear(128, 64, bias=False).to(dev)
    xs = correlated_inputs(g, 2, 32, 128)
    for x in xs:
        x[..., 7] = 0.0
    gp = GPTQ(lin)
    for x in xs:
        gp.add_batch(x.to(dev))
    H = gp.H.cpu().clone()
    q = gp.fasterquant(None, "mxint", {"weight_block_size": 32, "weight_width": 8}, quant_search=False).cpu()
    want = G.fasterquant(lin.weight.data.cpu(), H, "mxint", {"weight_block_size": 32, "weight_width": 8}, quant_search=False)
    assert bool((q[:, 7] == 0).all())
    assert float((q == want).float().mean()) > 0.97
    # clip_search_y: the search of every column group scored on the layer's calibration inputs
    gp = GPTQ(lin)
    for x in xs:
        gp.add_batch(x.to(dev))
    act = torch.stack([x.reshape(-1, x.shape[-1]) for x in xs])
    q_y = gp.fasterquant(act.to(dev), "mxint", MXINT4, cali_batch_size=2).cpu()
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
    from mase_amd.passes.gptq import find_qlayers, quantize_tensor, run_gptq
    from mase_amd.quantized.modules.linear import LinearMXInt

    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=128, intermediate_size=256, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, vocab_size=128, max_position_embeddings=128)
    base = LlamaForCausalLM(cfg).to(dev).eval()
    data = torch.randint(0, 128, (6, 48), generator=torch.Generator().manual_seed(1))
    gcfg = {"model_name": "synthetic", "device": str(dev), "format": "mxint", "weight_config": MXINT4,
            "calibration_data": data, "quantile_search": True}

    tuned = run_gptq(copy.deepcopy(base), dict(gcfg))
    plain = copy.deepcopy(base)
    for layer in plain.model.layers:
        for lin in find_qlayers(layer).values():
            lin.weight.data.copy_(quantize_tensor(lin.weight.data, 1, "mxint", MXINT4, True))
    changed = 0
    for lt, lb in zip(tuned.model.layers, base.model.layers):
        for (n, mt), mb in zip(find_qlayers(lt).items(), find_qlayers(lb).values()):
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
    want = find_qlayers(tuned.model.layers[1])["mlp.down_proj"].weight
    assert torch.equal(swapped.model.layers[1].mlp.down_proj.weight, want)
    with pytest.raises(NotImplementedError):
        run_gptq(copy.deepcopy(base), {**gcfg, "calibration_data": None})
    tuned_y = run_gptq(copy.deepcopy(base), {**gcfg, "clip_search_y": True, "cali_batch_size": 4})
    e_y = float((hidden(tuned_y) - ref).pow(2).mean())
    print(f"hidden-state MSE with clip_search_y: {e_y:.4e}")
    assert e_y < e_plain


def test_run_gptq_layer_checkpoints_and_resume(dev, tmp_path):
    """checkpoint_dir: one safetensors file + JSON description per finished layer, named as the reference names them;
    a second run finds them, loads them and quantizes only what is left; when every layer is there it returns at once.
    With resume_propagate the resumed run gives the weights of the uninterrupted run (the reference's driver, and the
    default here, calibrates the first resumed layer on layer 0's inputs instead)."""
    from safetensors.torch import load_file
    from transformers import LlamaConfig, LlamaForCausalLM

    from mase_amd.passes.gptq import detect_quantized_layers, run_gptq

    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=128, intermediate_size=256, num_hidden_layers=3, num_attention_heads=4,
                      num_key_value_heads=2, vocab_size=128, max_position_embeddings=128)
    base = LlamaForCausalLM(cfg).to(dev).eval()
    data = torch.randint(0, 128, (4, 32), generator=torch.Generator().manual_seed(1))
    gcfg = {"model_name": "synthetic", "device": str(dev), "format": "mxint", "weight_config": MXINT4,
            "calibration_data": data, "quantile_search": True}
    full = run_gptq(copy.deepcopy(base), dict(gcfg))

    d = str(tmp_path / "ckpt")
    first = run_gptq(copy.deepcopy(base), {**gcfg, "checkpoint_dir": d, "max_layers": 2})
    assert sorted(detect_quantized_layers(d)) == [0, 1]
    assert sorted(os.listdir(d)) == ["quantized_model_layer_0.safetensors", "quantized_model_layer_0_metadata.json",
                                     "quantized_model_layer_1.safetensors", "quantized_model_layer_1_metadata.json"]
    saved = load_file(os.path.join(d, "quantized_model_layer_1.safetensors"))
    assert set(saved) == {n for n, _ in base.model.layers[1].named_parameters()}
    assert torch.equal(saved["mlp.down_proj.weight"], first.model.layers[1].mlp.down_proj.weight.cpu())
    assert torch.equal(first.model.layers[1].mlp.down_proj.weight, full.model.layers[1].mlp.down_proj.weight)
    assert torch.equal(first.model.layers[2].mlp.down_proj.weight, base.model.layers[2].mlp.down_proj.weight)

    resumed = run_gptq(copy.deepcopy(base), {**gcfg, "checkpoint_dir": d, "resume_propagate": True})
    assert sorted(detect_quantized_layers(d)) == [0, 1, 2]
    for lr, lf in zip(resumed.model.layers, full.model.layers):
        for (n, pr), (_, pf) in zip(lr.named_parameters(), lf.named_parameters()):
            assert torch.equal(pr, pf), n
    # everything is there now: nothing is computed (no calibration data is even looked at)
    again = run_gptq(copy.deepcopy(base), {**gcfg, "checkpoint_dir": d, "calibration_data": None})
    assert torch.equal(again.model.layers[2].mlp.down_proj.weight, full.model.layers[2].mlp.down_proj.weight)
    # the reference's resume: layer 2 calibrated on the embedding outputs, so other weights than the straight run's
    os.remove(os.path.join(d, "quantized_model_layer_2.safetensors"))
    ref_style = run_gptq(copy.deepcopy(base), {**gcfg, "checkpoint_dir": d})
    assert torch.equal(ref_style.model.layers[1].mlp.down_proj.weight, full.model.layers[1].mlp.down_proj.weight)
    assert not torch.equal(ref_style.model.layers[2].mlp.down_proj.weight, full.model.layers[2].mlp.down_proj.weight)
