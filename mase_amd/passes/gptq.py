"""Second-order weight rounding (GPTQ) in front of the quantize pass.

Contract kept from the reference (``chop/passes/module/transforms/gptq/run.py:20-60``, called from
``passes/module/transforms/quantize/quantize.py:134-138``): ``run_gptq(network, gptq_config)`` takes a causal LM with
``network.model.layers`` and the keys ``device``, ``format`` ("mxint" | "mxfp"), ``weight_config`` (the MASE weight
keys), ``quantile_search``, ``clip_search_y``, ``cali_batch_size``, ``max_layers``; it rewrites the weights of the
``nn.Linear`` modules of the decoder layers in place and returns the network, whose modules the quantize pass then
swaps for ``LinearMX*`` configured with ``gptq=True`` (they do not quantize the weights again).  Calibration token ids
come in as ``gptq_config["calibration_data"]`` (``[samples, tokens]`` integers, or a list of ``[1, tokens]``): there
is no dataset download here.

What is computed (the algorithm of ``gptq/gptq.py:16-128`` for block formats): for a Linear with weight W [out, in] and
calibration inputs X, with G = sum x x^T, damped by 1 % of its mean diagonal, and U the upper Cholesky factor of
G^-1, the input columns are walked in groups of ``weight_block_size``; a group is quantized as a whole (one MX block
per row, optionally with the clip search), its error divided by U's diagonal and fed forward into the columns not yet
quantized through U's rows.  The scale of G does not matter (the damping is relative and U's scale cancels in
``error / diag(U) @ U``), so G is kept as the plain sum.

How it is organised here:

* One Gram matrix per distinct input tensor.  Projections that read the same tensor (q / k / v; gate / up) are hooked
  together, the hook recognises the shared tensor and its Gram matrix is accumulated once, with one ``addmm_`` per
  sample, and factored once.
* The feed-forward of the error is blocked on two levels: inside a panel of ``PANEL_GROUPS`` column groups the update
  reaches the rest of the panel only; the columns behind the panel receive the panel's accumulated errors in one
  ``addmm_`` ([out, panel] x [panel, rest]).  Same sums, fewer and larger products.
* The working copy of W is fp32 whatever the weight dtype; each group is handed to the quantizer in the weight's
  dtype, which is what the modules' own quantizer would see.
* The quantizers are this package's device kernels (``mase_mx*_clip_search``, ``mase_mx*_qdq``, and with
  ``clip_search_y`` the candidate kernels scored on the group's calibration inputs).
* The first decoder layer's inputs are recorded by a forward pre-hook that stops the forward; every later call of a
  layer replays the keyword arguments recorded there (mask, positions, rotary tables), whatever the model passes.
"""
from __future__ import annotations

import logging
from typing import Callable, Sequence

import torch
from torch import Tensor, nn

from ..quantizers import MXFPMeta, MXIntMeta, mxfp_quantizer_sim, mxint_quantizer_sim

log = logging.getLogger(__name__)

PANEL_GROUPS = 4       # column groups per panel of the blocked error feed-forward
RELATIVE_DAMPING = 0.01

# projections of a decoder layer in the order they are rounded; members of one entry read the same tensor, and an
# entry sees the outputs of the already rounded entries before it
PROJECTION_GROUPS = (
    ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj"),
    ("self_attn.o_proj",),
    ("mlp.gate_proj", "mlp.up_proj"),
    ("mlp.down_proj",),
)


def group_quantizer(fmt: str, weight_config: dict, search: bool, cali_batch_size: int = 32) -> Callable:
    """``f(w_group [out, block], calibration [samples, tokens, block] | None) -> quantize-dequantize of the group``, one
    MX block per row (the dispatch of ``gptq/quantize_dispatch.py:36-82`` on the weight keys of the MASE config)"""
    block = weight_config["weight_block_size"]
    if fmt == "mxint":
        meta = MXIntMeta(block_size=block, scale_bits=8, element_bits=weight_config["weight_width"])
        sim = mxint_quantizer_sim
        kw = {"mxint_meta": meta}
    elif fmt == "mxfp":
        meta = MXFPMeta(block_size=block, scale_exp_bits=8, element_exp_bits=weight_config["weight_exponent_width"],
                        element_frac_bits=weight_config["weight_frac_width"], element_is_finite=True, round_mode="rn")
        sim = mxfp_quantizer_sim
        kw = {"mxfp_meta": meta}
    else:
        raise ValueError(f"gptq: format {fmt!r} is not one of 'mxint', 'mxfp'")

    def quantize(w_group: Tensor, calibration: Tensor | None = None) -> Tensor:
        return sim(w_group, block_dim=1, act_tensor=calibration if search else None, quantile_search=search,
                   cali_batch_size=cali_batch_size, **kw)

    return quantize


class InputGram:
    """sum of x x^T over the rows of every tensor handed to ``update`` (fp32, on the tensor's device), and optionally
    the tensors themselves for a clip search scored on calibration inputs"""

    def __init__(self, keep_inputs: bool = False):
        self.matrix: Tensor | None = None
        self.rows_seen = 0
        self.inputs: list[Tensor] | None = [] if keep_inputs else None

    def update(self, x: Tensor) -> None:
        rows = x.detach().reshape(-1, x.shape[-1]).float()
        if self.matrix is None:
            self.matrix = torch.zeros(rows.shape[1], rows.shape[1], dtype=torch.float32, device=rows.device)
        self.matrix.addmm_(rows.t(), rows)
        self.rows_seen += rows.shape[0]
        if self.inputs is not None:
            self.inputs.append(x.detach().reshape(1, -1, x.shape[-1]) if x.dim() <= 2 else x.detach())

    def calibration(self) -> Tensor | None:
        return None if self.inputs is None else torch.cat(self.inputs, dim=0)


def inverse_cholesky_upper(gram: Tensor, relative_damping: float = RELATIVE_DAMPING):
    """(U, dead): U upper triangular with U^T U = (G + damping)^-1 where input columns that never fired (``dead``) are
    given a unit diagonal first"""
    G = gram.clone()
    d = torch.diagonal(G)
    dead = d == 0
    d[dead] = 1.0
    d += relative_damping * d.mean()
    L = torch.linalg.cholesky(G)
    return torch.linalg.cholesky(torch.cholesky_inverse(L), upper=True), dead


def round_weight(weight: Tensor, gram: Tensor, group_size: int, quantize: Callable, calibration: Tensor | None = None,
                 relative_damping: float = RELATIVE_DAMPING, panel_groups: int = PANEL_GROUPS) -> Tensor:
    """The rounded weight, in ``weight``'s dtype.  ``quantize(w_group, calibration_group)`` rounds one column group;
    ``calibration`` [samples, tokens, in] is sliced to the group's columns for it."""
    out_features, in_features = weight.shape
    U, dead = inverse_cholesky_upper(gram, relative_damping)
    W = weight.detach().float().clone()
    W[:, dead] = 0.0
    Q = torch.empty_like(weight)
    inv_diag = 1.0 / torch.diagonal(U)
    panel = group_size * panel_groups
    for p0 in range(0, in_features, panel):
        p1 = min(p0 + panel, in_features)
        scaled_err = torch.empty(out_features, p1 - p0, dtype=torch.float32, device=W.device)
        for c0 in range(p0, p1, group_size):
            c1 = min(c0 + group_size, p1)
            cal = None if calibration is None else calibration[:, :, c0:c1].contiguous()
            q = quantize(W[:, c0:c1].to(weight.dtype).contiguous(), cal)
            Q[:, c0:c1] = q
            e = (W[:, c0:c1] - q.float()) * inv_diag[c0:c1]
            scaled_err[:, c0 - p0:c1 - p0] = e
            if c1 < p1:  # the rest of this panel sees the group's error now
                W[:, c1:p1].addmm_(e, U[c0:c1, c1:p1], alpha=-1.0)
        if p1 < in_features:  # everything behind the panel sees the panel's errors in one product
            W[:, p1:].addmm_(scaled_err, U[p0:p1, p1:], alpha=-1.0)
    return Q


def linear_modules(module: nn.Module) -> dict[str, nn.Linear]:
    """{dotted name: module} of the plain ``nn.Linear`` sub-modules (subclasses, e.g. already swapped ones, excluded)"""
    return {name: m for name, m in module.named_modules() if type(m) is nn.Linear}


@torch.no_grad()
def round_decoder_layer(layer: nn.Module, forward_sample: Callable[[int], object], n_samples: int, quantize: Callable,
                        group_size: int, score_on_inputs: bool = False,
                        projection_groups: Sequence[Sequence[str]] = PROJECTION_GROUPS) -> list[str]:
    """Rounds the Linears of one decoder layer, one entry of ``projection_groups`` after the other: run the layer over
    the calibration samples (``forward_sample(j)``) with pre-hooks collecting the Gram matrix of each distinct input
    tensor of the entry, then rewrite the entry's weights.  Linears not named in ``projection_groups`` are left alone.
    Returns the names rewritten."""
    found = linear_modules(layer)
    done = []
    for entry in projection_groups:
        members = [(n, found[n]) for n in entry if n in found]
        if not members:
            continue
        gram_of: dict[str, InputGram] = {}
        # within one forward: id of an input tensor -> (the tensor, kept alive so that the id stays its own; its Gram)
        accounted: dict[int, tuple[Tensor, InputGram]] = {}

        def collect(name):
            def pre_hook(_module, args):
                x = args[0]
                hit = accounted.get(id(x))
                if hit is None:  # the first member to read this tensor in this forward accumulates it
                    gram = gram_of.setdefault(name, InputGram(keep_inputs=score_on_inputs))
                    gram.update(x)
                    accounted[id(x)] = (x, gram)
                elif gram_of.setdefault(name, hit[1]) is not hit[1]:
                    raise RuntimeError(f"gptq: {name} shares its input with a sibling in some calibration samples only")
            return pre_hook

        handles = [m.register_forward_pre_hook(collect(n)) for n, m in members]
        try:
            for j in range(n_samples):
                accounted.clear()
                forward_sample(j)
        finally:
            for h in handles:
                h.remove()
        accounted.clear()
        for name, m in members:
            gram = gram_of[name]
            cal = gram.calibration() if score_on_inputs else None
            m.weight.data.copy_(round_weight(m.weight.data, gram.matrix, group_size, quantize, cal))
            done.append(name)
    return done


class _StopForward(Exception):
    """raised by the recording hook once the first decoder layer's inputs are known"""


def _samples(gptq_config) -> list[Tensor]:
    data = gptq_config.get("calibration_data")
    if data is None:
        raise NotImplementedError(
            "run_gptq: pass the calibration token ids as gptq_config['calibration_data'] ([samples, tokens] or a list "
            "of [1, tokens] tensors); loading a dataset by name needs a network connection and is not built")
    if isinstance(data, Tensor):
        return [row.reshape(1, -1) for row in data]
    return [d.reshape(1, -1) for d in data]


@torch.no_grad()
def run_gptq(network, gptq_config):
    """See the module docstring.  Decoder layers are processed in order; layer i + 1 is calibrated on the outputs of the
    already rounded layer i."""
    dev = torch.device(gptq_config.get("device", "cuda:0"))
    weight_config = gptq_config["weight_config"]
    score_on_inputs = bool(gptq_config.get("clip_search_y", False))
    quantize = group_quantizer(gptq_config["format"], weight_config, bool(gptq_config.get("quantile_search", True)),
                               gptq_config.get("cali_batch_size", 32))
    samples = _samples(gptq_config)
    decoder = network.model.layers
    n_layers = len(decoder) if gptq_config.get("max_layers") is None else min(len(decoder), gptq_config["max_layers"])

    # what the first decoder layer receives for every sample: positional hidden states + keyword arguments
    hidden, call_kwargs = [], {}

    def record(_module, args, kwargs):
        hidden.append(args[0] if args else kwargs["hidden_states"])
        call_kwargs.clear()
        call_kwargs.update({k: v for k, v in kwargs.items() if k != "hidden_states"})
        raise _StopForward

    cache_setting = getattr(network.config, "use_cache", None)
    if cache_setting is not None:
        network.config.use_cache = False
    network.to(dev)
    handle = decoder[0].register_forward_pre_hook(record, with_kwargs=True)
    try:
        for ids in samples:
            try:
                network(ids.to(dev))
            except _StopForward:
                pass
    finally:
        handle.remove()
    if len(hidden) != len(samples):
        raise RuntimeError("gptq: the first decoder layer was not reached for every calibration sample")
    call_kwargs.pop("past_key_values", None)
    call_kwargs.pop("past_key_value", None)
    if "use_cache" in call_kwargs:
        call_kwargs["use_cache"] = False

    log.info("gptq: %d decoder layers, %d calibration samples of %d tokens, format %s", n_layers, len(samples),
             samples[0].shape[-1], gptq_config["format"])
    for index in range(n_layers):
        layer = decoder[index]
        outputs: list = [None] * len(samples)

        def forward_sample(j, layer=layer, outputs=outputs):
            y = layer(hidden[j], **call_kwargs)
            outputs[j] = y[0] if isinstance(y, (tuple, list)) else y

        names = round_decoder_layer(layer, forward_sample, len(samples), quantize, weight_config["weight_block_size"],
                                    score_on_inputs)
        for j in range(len(samples)):  # the rounded layer's outputs are the next layer's calibration inputs
            forward_sample(j)
        hidden = outputs
        log.info("gptq: layer %d rounded (%s)", index, ", ".join(names))
    if cache_setting is not None:
        network.config.use_cache = cache_setting
    return network
