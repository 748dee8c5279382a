"""Module-level quantize pass with the contract of the reference's
``chop/passes/module/transforms/quantize/quantize.py:95-151`` for ``nn.Linear`` targets:

    network, info = quantize_module_transform_pass(network, {"by": "type", "linear": {"config": {"name": "mxint", ...}}})

Like the reference it pops ``"by"`` (and ``"gptq"``) from ``pass_args`` and ``"name"`` from a by-type/by-name config
(:28, :48, :140), instantiates ``quantized_module_map["linear_<name>"]`` with the original module's shape, bias,
device and dtype (``module_modify_helper.py:149-176``), hands the weights over with
``load_state_dict(deepcopy(state_dict), strict=False)`` (:103-114) and swaps the module in by name (:137-141).
``nn.Embedding`` targets (:191-216) and Llama / Qwen3 attention / MLP / RMSNorm targets (:264-275, selected by name or
regex with a ``llama_* / qwen3_*`` ``self_attention_* / mlp_* / rms_norm_*`` entry of the registry) are handled the same
way; the Llama replacements receive ``config=network.config`` like the reference's (quantize.py:52-56, 82-86).  A
module counts as a Llama attention / MLP / RMSNorm when a class of that name is among its bases, so that the
``transformers`` classes match without being imported here.  A ``"gptq"`` entry runs ``mase_amd.passes.gptq.run_gptq``
first (:134-138).  Other model families and conv2d are outside this build.
"""
from __future__ import annotations

import inspect
import logging
import re
from copy import deepcopy

import torch

from ..quantized.modules import quantized_module_map


def _instantiate_linear(module, postfix, module_map, additional_module_args):
    linear_cls = module_map[f"linear_{postfix}"]
    has_bias = module.bias is not None
    kwargs = dict(in_features=module.in_features, out_features=module.out_features, bias=has_bias,
                  device=module.weight.device, dtype=module.weight.dtype)
    if "config" in inspect.signature(linear_cls.__init__).parameters:
        return linear_cls(**kwargs, config=additional_module_args)
    return linear_cls(**kwargs, **additional_module_args)


def _instantiate_embedding(module, postfix, module_map, additional_module_args):
    embedding_cls = module_map[f"embedding_{postfix}"]
    kwargs = dict(num_embeddings=module.num_embeddings, embedding_dim=module.embedding_dim,
                  padding_idx=module.padding_idx, max_norm=module.max_norm, norm_type=module.norm_type,
                  scale_grad_by_freq=module.scale_grad_by_freq, sparse=module.sparse)
    if "config" in inspect.signature(embedding_cls.__init__).parameters:
        return embedding_cls(**kwargs, config=additional_module_args)
    return embedding_cls(**kwargs, **additional_module_args)


_LLAMA_PREFIX = {"LlamaAttention": "llama_self_attention", "LlamaMLP": "llama_mlp", "LlamaRMSNorm": "llama_rms_norm",
                 "Qwen3Attention": "qwen3_self_attention", "Qwen3MLP": "qwen3_mlp", "Qwen3RMSNorm": "qwen3_rms_norm"}


def _llama_prefix(module):
    for cls in type(module).__mro__:
        if cls.__name__ in _LLAMA_PREFIX:
            return _LLAMA_PREFIX[cls.__name__]
    return None


def _instantiate_llama_module(module, postfix, prefix, module_map, module_args, network_args):
    llama_cls = module_map[f"{prefix}_{postfix}"]
    new = llama_cls(config=network_args, layer_idx=getattr(module, "layer_idx", None), q_config=module_args)
    first = next(module.parameters(), None)
    return new if first is None else new.to(device=first.device, dtype=first.dtype)


def _instantiate_module(module, postfix, module_map, additional_module_args):
    module_args = additional_module_args["config"]
    network_args = additional_module_args.get("network_config", None)
    if isinstance(module, torch.nn.Linear):
        return _instantiate_linear(module, postfix, module_map, module_args)
    if isinstance(module, torch.nn.Embedding):
        return _instantiate_embedding(module, postfix, module_map, module_args)
    prefix = _llama_prefix(module)
    if prefix is not None:
        return _instantiate_llama_module(module, postfix, prefix, module_map, module_args, network_args)
    raise ValueError(f"{module} is not supported.")


def _module_args(network, quan_config):
    """``network_config`` travels with the module config when the network carries a model config (the reference
    tests for a ``transformers`` model; any network with a ``config`` attribute is treated the same here)"""
    network_config = getattr(network, "config", None)
    if network_config is not None:
        return {"config": quan_config, "network_config": network_config}
    return {"config": quan_config}


def _weight_replacement(x, y):
    target_state_dict = deepcopy(x.state_dict())
    missing_keys, unexpected_keys = y.load_state_dict(target_state_dict, strict=False)
    if missing_keys:
        logging.warning(f"Missing keys when loading state_dict: {missing_keys} from {x} to {y}")
    if unexpected_keys:
        logging.warning(f"Unexpected keys when loading state_dict: {unexpected_keys} from {x} to {y}")
    return y


def _replace_by_name(network, name, module):
    original = network.get_submodule(name)
    new = _weight_replacement(original, module)
    parent_name, _, child = name.rpartition(".")
    parent = network.get_submodule(parent_name) if parent_name else network
    setattr(parent, child, new)
    return network


def _quantize_by_type(network, pass_args):
    for type_name, config in pass_args.items():
        n_m = dict(network.named_modules())
        if type_name == "linear":
            module = torch.nn.Linear
        elif type_name == "conv2d":
            raise ValueError("conv2d is outside this build (Linear only)")
        else:
            raise ValueError(f"{type_name} is not supported!")
        config = config["config"]
        postfix = config.pop("name")
        for n, m in n_m.items():
            if isinstance(m, module):
                new_m = _instantiate_module(m, postfix, quantized_module_map, {"config": config})
                network = _replace_by_name(network, n, new_m)
    return network


def _quantize_by_name(network, pass_args):
    n_m = dict(network.named_modules())
    for n, m in n_m.items():
        if n in pass_args:
            quan_config = pass_args[n]["config"]
            postfix = quan_config.pop("name")
            new_m = _instantiate_module(m, postfix, quantized_module_map, _module_args(network, quan_config))
            network = _replace_by_name(network, n, new_m)
    return network


def _match_a_pattern(name: str, patterns):
    for pattern in patterns:
        if re.fullmatch(pattern, name):
            return pattern
    return None


def _quantize_by_regex_name(network, pass_args):
    patterns = list(pass_args.keys())
    n_m = dict(network.named_modules())
    for n, m in n_m.items():
        matched = _match_a_pattern(n, patterns)
        if not matched:
            continue
        quan_config = pass_args[matched]["config"]
        postfix = quan_config["name"]
        new_m = _instantiate_module(m, postfix, quantized_module_map, _module_args(network, quan_config))
        network = _replace_by_name(network, n, new_m)
    return network


def quantize_module_transform_pass(network, pass_args):
    gptq_config = pass_args.pop("gptq", None)
    if gptq_config is not None:  # quantize.py:134-138: GPTQ rewrites the nn.Linear weights before the modules are swapped
        from .gptq import run_gptq

        network = run_gptq(network, gptq_config)
    by = pass_args.pop("by")
    if by == "type":
        network = _quantize_by_type(network, pass_args)
    elif by == "name":
        network = _quantize_by_name(network, pass_args)
    elif by == "regex_name":
        network = _quantize_by_regex_name(network, pass_args)
    else:
        raise ValueError(f'Unsupported quantize "by": {by}')
    return network, {}
