"""GPTQ weight optimisation in front of the quantize pass, with the contract of the reference's
``chop/passes/module/transforms/gptq/`` (``gptq.py:16-128`` the algorithm, ``quantize_dispatch.py:36-82`` the quantizer
dispatch, ``utils.py:7-18`` the layer search, ``run.py:20-232`` the driver over a causal LM's decoder layers).

The algorithm per ``nn.Linear``: accumulate H = 2/n * sum x x^T over the calibration inputs, damp its diagonal, take
the upper Cholesky factor U of H^-1, then walk the columns in groups of ``weight_block_size``: quantize the group
(``quantile_search`` clip search of the MX quantizers, one MX block per row and group), divide the quantization error
by U's diagonal and subtract its product with U's off-diagonal rows from the columns still to come.  The quantizer
calls are the device kernels of this package (``mase_mxint_clip_search`` / ``mase_mxfp_clip_search`` or the plain
quantize-dequantize kernels); the Hessian, its factorisations and the rank-32 updates are library calls on the same
device.  Weights are written back into the ``nn.Linear`` modules, so that the quantize pass that follows finds them
(its ``LinearMX*`` replacements are configured with ``gptq=True`` and do not quantize again).

Differences from the reference's driver: calibration token ids are passed in (``gptq_config["calibration_data"]``, an
integer tensor ``[nsamples, seqlen]`` or a list of ``[1, seqlen]`` tensors) instead of being downloaded by dataset
name.  ``clip_search_y`` scores the clip search of each column group on the group's calibration inputs
(``mase_mx*_clip_candidates`` plus matrix products).  ``checkpoint_dir`` writes one safetensors file (and a JSON
description) per finished decoder layer and resumes after the last layer found there, with the reference's file names
(``checkpoint.py:9-135``); like the reference's driver, a resumed run calibrates its first layer on the inputs of
layer 0 unless ``resume_propagate`` is set, which first runs those inputs through the layers that were loaded.
"""
from __future__ import annotations

import json
import logging
import math
import os
import re

import torch
from torch import Tensor, nn

from ..quantizers import MXFPMeta, MXIntMeta, mxfp_quantizer_sim, mxint_quantizer_sim


def quantize_tensor(input: Tensor, block_dim: int, fmt: str, config: dict, quantile_search: bool,
                    act_tensor: Tensor | None = None, dtype: torch.dtype | None = None,
                    cali_batch_size: int = 32) -> Tensor:
    """quantize_dispatch.py:36-82"""
    if fmt == "mxfp":
        meta = MXFPMeta(block_size=config["weight_block_size"], scale_exp_bits=8,
                        element_exp_bits=config["weight_exponent_width"], element_frac_bits=config["weight_frac_width"],
                        element_is_finite=True, round_mode="rn")
        return mxfp_quantizer_sim(input, block_dim=block_dim, mxfp_meta=meta, act_tensor=act_tensor, dtype=dtype,
                                  quantile_search=quantile_search, cali_batch_size=cali_batch_size)
    if fmt == "mxint":
        meta = MXIntMeta(block_size=config["weight_block_size"], scale_bits=8, element_bits=config["weight_width"])
        return mxint_quantizer_sim(input, block_dim=block_dim, mxint_meta=meta, act_tensor=act_tensor, dtype=dtype,
                                   quantile_search=quantile_search, cali_batch_size=cali_batch_size)
    raise ValueError(f"Unsupported GPTQ format: {fmt}. Use 'mxfp' or 'mxint'.")


def find_qlayers(module, layers=(nn.Linear,), name=""):
    """utils.py:7-18: {dotted name: module} of the sub-modules whose type is one of ``layers``"""
    if type(module) in tuple(layers):
        return {name: module}
    found = {}
    for child_name, child in module.named_children():
        found.update(find_qlayers(child, layers=layers, name=f"{name}.{child_name}" if name != "" else child_name))
    return found


class GPTQ:
    """gptq.py:16-128"""

    def __init__(self, layer):
        self.layer = layer
        self.dev = layer.weight.device
        self.rows, self.columns = layer.weight.shape
        self.H = torch.zeros((self.columns, self.columns), device=self.dev)
        self.nsamples = 0

    def add_batch(self, inp, out=None):
        """gptq.py:27-37: running mean of 2 * x x^T over the samples seen"""
        if inp.dim() == 2:
            inp = inp.unsqueeze(0)
        n = inp.shape[0]
        if inp.dim() == 3:
            inp = inp.reshape(-1, inp.shape[-1])
        inp = inp.t()
        self.H *= self.nsamples / (self.nsamples + n)
        self.nsamples += n
        inp = math.sqrt(2 / self.nsamples) * inp.float()
        self.H += inp.matmul(inp.t())

    def inverse_factor(self, percdamp: float = 0.01):
        """gptq.py:65-78: columns that never fired are pinned, the diagonal damped by ``percdamp`` of its mean, and the
        upper Cholesky factor of H^-1 returned; consumes ``self.H``"""
        H = self.H
        del self.H
        dead = torch.diag(H) == 0
        H[dead, dead] = 1
        damp = percdamp * torch.mean(torch.diag(H))
        diag = torch.arange(self.columns, device=self.dev)
        H[diag, diag] += damp
        H = torch.linalg.cholesky(H)
        H = torch.cholesky_inverse(H)
        return torch.linalg.cholesky(H, upper=True), dead

    def fasterquant(self, activation, fmt, weight_config, percdamp=0.01, cali_batch_size=32, layer_name=None,
                    quant_search=True):
        """gptq.py:39-122"""
        W = self.layer.weight.data.clone()
        Hinv, dead = self.inverse_factor(percdamp)
        W[:, dead] = 0
        Q = torch.zeros_like(W)
        blocksize = weight_config["weight_block_size"]
        for i1 in range(0, self.columns, blocksize):
            i2 = min(i1 + blocksize, self.columns)
            W1 = W[:, i1:i2].clone()
            # clip_search_y: the group's search is scored on the layer's calibration inputs of these columns
            act1 = None if activation is None else activation[:, :, i1:i2].clone()
            Q1 = quantize_tensor(W1, block_dim=1, fmt=fmt, config=weight_config, quantile_search=quant_search,
                                 act_tensor=act1, cali_batch_size=cali_batch_size)
            Q[:, i1:i2] = Q1
            if i2 < self.columns:
                err = (W1 - Q1) / torch.diag(Hinv[i1:i2, i1:i2]).unsqueeze(0)
                W[:, i2:] -= err.matmul(Hinv[i1:i2, i2:])
        assert Q.shape == W.shape, f"Shape mismatch: {Q.shape} != {W.shape}"
        return Q

    def free(self):
        self.H = None


_SEQUENTIAL = (  # run.py:136-141
    ("self_attn.k_proj", "self_attn.v_proj", "self_attn.q_proj"),
    ("self_attn.o_proj",),
    ("mlp.up_proj", "mlp.gate_proj"),
    ("mlp.down_proj",),
)


@torch.no_grad()
def gptq_decoder_layer(layer, run_layer, nsamples: int, fmt: str, weight_config: dict, quantile_search: bool = True,
                       cali_batch_size: int = 32, sequential=_SEQUENTIAL, layer_name: str = "",
                       clip_search_y: bool = False):
    """The per-layer body of run.py:150-214: for each group of projections in ``sequential``, run the layer over the
    ``nsamples`` calibration samples (``run_layer(j)`` runs sample j through ``layer``) with hooks that feed each
    projection's inputs to its GPTQ object, then quantize those projections and write the weights back.
    ``clip_search_y``: the inputs of the group (its projections share them; recorded at the last one, run.py:173) are
    kept as [nsamples, tokens, columns] and the clip search of every column group is scored on them."""
    full = find_qlayers(layer, layers=[nn.Linear])
    for names in sequential:
        subset = {n: full[n] for n in names if n in full}
        if not subset:
            continue
        gptq = {n: GPTQ(m) for n, m in subset.items()}

        def hook(name):
            def fn(_, inp, out):
                gptq[name].add_batch(inp[0].data, out.data)
            return fn

        handles = [m.register_forward_hook(hook(n)) for n, m in subset.items()]
        pre_act = []
        if clip_search_y:
            last = list(subset.values())[-1]
            handles.append(last.register_forward_pre_hook(lambda _, inp: pre_act.append(inp[0])))
        try:
            for j in range(nsamples):
                run_layer(j)
        finally:
            for h in handles:
                h.remove()
        activation = torch.cat(pre_act, dim=0) if clip_search_y else None
        for n, m in subset.items():
            q = gptq[n].fasterquant(activation=activation, fmt=fmt, weight_config=weight_config, percdamp=0.01,
                                    cali_batch_size=cali_batch_size, layer_name=f"{layer_name}.{n}",
                                    quant_search=quantile_search)
            assert q.shape == m.weight.shape
            m.weight.data.copy_(q)
            gptq[n].free()


def _calibration_batches(gptq_config):
    data = gptq_config.get("calibration_data")
    if data is None:
        raise NotImplementedError(
            "run_gptq: pass the calibration token ids as gptq_config['calibration_data'] ([nsamples, seqlen] or a list "
            "of [1, seqlen] tensors); loading a dataset by name needs a network connection and is not built")
    if isinstance(data, Tensor):
        return [row.unsqueeze(0) for row in data]
    return [d if d.dim() == 2 else d.unsqueeze(0) for d in data]


_CKPT_MODEL_NAME = "quantized_model"


def _layer_file(checkpoint_dir: str, layer_idx: int) -> str:
    return os.path.join(checkpoint_dir, f"{_CKPT_MODEL_NAME}_layer_{layer_idx}.safetensors")


def save_layer_checkpoint(network, layer_idx: int, checkpoint_dir: str | None) -> None:
    """checkpoint.py:9-72: the parameters of decoder layer ``layer_idx`` under their names relative to the layer, in
    ``<dir>/quantized_model_layer_<i>.safetensors``, and a JSON description beside it"""
    if checkpoint_dir is None:
        return
    from safetensors.torch import save_file

    os.makedirs(checkpoint_dir, exist_ok=True)
    prefix = f"model.layers.{layer_idx}."
    tensors = {name[len(prefix):]: p.detach().cpu().contiguous() for name, p in network.named_parameters()
               if name.startswith(prefix)}
    if not tensors:
        logging.warning(f"No parameters found for layer {layer_idx} with prefix {prefix}")
        return
    path = _layer_file(checkpoint_dir, layer_idx)
    save_file(tensors, path)
    meta = {"layer_idx": layer_idx, "total_layers": len(network.model.layers), "checkpoint_file": path,
            "model_name": _CKPT_MODEL_NAME, "num_parameters": len(tensors), "parameter_names": list(tensors)}
    with open(os.path.join(checkpoint_dir, f"{_CKPT_MODEL_NAME}_layer_{layer_idx}_metadata.json"), "w") as f:
        json.dump(meta, f, indent=2)


def detect_quantized_layers(checkpoint_dir: str | None) -> dict:
    """checkpoint.py:75-91: {layer index: file} of the layer files present"""
    found = {}
    if checkpoint_dir is None or not os.path.isdir(checkpoint_dir):
        return found
    pat = re.compile(rf"^{_CKPT_MODEL_NAME}_layer_(\d+)\.safetensors$")
    for fn in os.listdir(checkpoint_dir):
        m = pat.match(fn)
        if m:
            found[int(m.group(1))] = os.path.join(checkpoint_dir, fn)
    return found


def auto_load_quantized_layers(network, checkpoint_dir: str | None) -> int:
    """checkpoint.py:94-135: loads the layer files in ascending order of their index, stops at the first that fails,
    returns the last index loaded (-1: none)"""
    from safetensors.torch import load_file

    last = -1
    for idx, path in sorted(detect_quantized_layers(checkpoint_dir).items()):
        try:
            state = {f"model.layers.{idx}.{k}": v for k, v in load_file(path).items()}
            network.load_state_dict(state, strict=False)
        except Exception as e:  # a damaged file ends the resume, as in the reference
            logging.warning(f"Failed to load layer {idx} ({e}), stopping auto-load")
            break
        last = idx
    return last


@torch.no_grad()
def run_gptq(network, gptq_config):
    """run.py:20-232 for a ``transformers`` causal LM with ``network.model.layers`` / ``embed_tokens`` / ``norm`` /
    ``rotary_emb``: GPTQ over every ``nn.Linear`` of every decoder layer, layer by layer, the inputs of layer i+1 being
    the outputs of the already quantized layer i.  Keys of ``gptq_config`` as in the reference (``device``, ``format``,
    ``weight_config``, ``quantile_search``, ``clip_search_y``, ``cali_batch_size``, ``max_layers``) plus
    ``calibration_data``."""
    clip_search_y = gptq_config.get("clip_search_y", False)
    checkpoint_dir = gptq_config.get("checkpoint_dir", None)
    start_layer = 0
    if checkpoint_dir is not None:  # run.py:64-74
        start_layer = auto_load_quantized_layers(network, checkpoint_dir) + 1
        if start_layer:
            logging.info(f"Resuming GPTQ from layer {start_layer}")
        if start_layer == len(network.model.layers):
            logging.info("All layers already quantized, skipping GPTQ")
            return network
    dev = gptq_config.get("device", "cuda:0")
    fmt = gptq_config["format"]
    weight_config = gptq_config["weight_config"]
    quantile_search = gptq_config.get("quantile_search", True)
    cali_batch_size = gptq_config.get("cali_batch_size", 32)
    max_layers = gptq_config.get("max_layers", None)
    batches = _calibration_batches(gptq_config)
    nsamples = len(batches)
    seqlen = batches[0].shape[-1]

    use_cache = network.config.use_cache
    network.config.use_cache = False
    layers = network.model.layers
    network.model.embed_tokens = network.model.embed_tokens.to(dev)
    network.model.norm = network.model.norm.to(dev)
    rope = network.model.rotary_emb.to(dev)
    layers[0] = layers[0].to(dev)
    dtype = next(iter(network.parameters())).dtype
    inps = torch.zeros((nsamples, seqlen, network.config.hidden_size), dtype=dtype, device=dev)
    cache = {"i": 0, "attention_mask": None, "position_ids": None}

    class Catcher(nn.Module):  # run.py:108-118: records what the first decoder layer receives
        def __init__(self, module):
            super().__init__()
            self.module = module

        def forward(self, inp, **kwargs):
            inps[cache["i"]] = inp
            cache["i"] += 1
            cache["attention_mask"] = kwargs.get("attention_mask")
            cache["position_ids"] = kwargs.get("position_ids")
            raise ValueError

    layers[0] = Catcher(layers[0])
    for batch in batches:
        try:
            network(batch.to(dev))
        except ValueError:
            pass
    layers[0] = layers[0].module
    outs = torch.zeros_like(inps)
    attention_mask, position_ids = cache["attention_mask"], cache["position_ids"]
    if position_ids is None:
        position_ids = torch.arange(seqlen, device=dev).unsqueeze(0)

    end_layer = len(layers) if max_layers is None else min(start_layer + max_layers, len(layers))
    logging.info(f"GPTQ: quantizing layers {start_layer} to {end_layer - 1} (of {len(layers)} total)")
    if start_layer and gptq_config.get("resume_propagate", False):
        for i in range(start_layer):  # the loaded layers' outputs, not layer 0's inputs, feed the first new layer
            layer = layers[i].to(dev)
            for j in range(nsamples):
                x = inps[j].unsqueeze(0)
                cos, sin = rope(x, position_ids)
                out = layer(x, attention_mask=attention_mask, position_embeddings=(cos, sin))
                outs[j] = out[0] if isinstance(out, tuple) else out
            inps, outs = outs, inps
    for i in range(start_layer, end_layer):
        layer = layers[i].to(dev)

        def run_layer(j, layer=layer):
            x = inps[j].unsqueeze(0)
            cos, sin = rope(x, position_ids)
            out = layer(x, attention_mask=attention_mask, position_embeddings=(cos, sin))
            outs[j] = out[0] if isinstance(out, tuple) else out

        gptq_decoder_layer(layer, run_layer, nsamples, fmt, weight_config, quantile_search, cali_batch_size,
                           layer_name=f"layers{i}", clip_search_y=clip_search_y)
        for j in range(nsamples):  # run.py:197-205: the quantized layer's outputs feed the next layer
            run_layer(j)
        inps, outs = outs, inps
        save_layer_checkpoint(network, i, checkpoint_dir)
    network.config.use_cache = use_cache
    return network
