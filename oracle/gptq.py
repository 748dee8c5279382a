"""CPU restatement of the reference's GPTQ weight optimisation (chop/passes/module/transforms/gptq/gptq.py:16-128).
TEST INFRASTRUCTURE ONLY, like the rest of this package.

Pinned by: the Hessian against a direct double-precision sum; U^T U against the inverse of the damped Hessian; with
groups of one column the walk equals optimal-brain-surgeon rounding column by column evaluated in float64 with an
explicit inverse per column (no factor involved), exactly; with uncorrelated inputs (diagonal H) the result is the
plain clip-search quantization; with correlated inputs the proxy loss tr((W-Q) H (W-Q)^T) is below that of plain
quantization.  What remains source text alone is the reference's simplification inside a group of more than one
column (the error divided by the diagonal of the factor's block, gptq.py:111-117, where the column-by-column walk
would solve with the block); the reference holds no vectors or tests for this path.
"""
from __future__ import annotations

import math

import torch

from .quantizers import mxfp_clip_search, mxfp_quantizer, mxint_clip_search, mxint_quantizer


def hessian(batches):
    """gptq.py:27-37 applied to a sequence of [batch, tokens, columns] or [tokens, columns] inputs"""
    H, n_seen = None, 0
    for inp in batches:
        if inp.dim() == 2:
            inp = inp.unsqueeze(0)
        n = inp.shape[0]
        inp = inp.reshape(-1, inp.shape[-1]).t()
        if H is None:
            H = torch.zeros(inp.shape[0], inp.shape[0])
        H *= n_seen / (n_seen + n)
        n_seen += n
        inp = math.sqrt(2 / n_seen) * inp.float()
        H += inp.matmul(inp.t())
    return H


def inverse_factor(H, percdamp=0.01):
    """gptq.py:65-78"""
    H = H.clone()
    dead = torch.diag(H) == 0
    H[dead, dead] = 1
    damp = percdamp * torch.mean(torch.diag(H))
    idx = torch.arange(H.shape[0])
    H[idx, idx] += damp
    H = torch.linalg.cholesky(H)
    H = torch.cholesky_inverse(H)
    return torch.linalg.cholesky(H, upper=True), dead


def quantize_group(W1, fmt, weight_config, quant_search, act_tensor=None, cali_batch_size=32):
    """quantize_dispatch.py:36-82 with block_dim=1; ``act_tensor``: the calibration inputs of these columns, which
    only the search branch looks at (mxint.py:99, mxfp.py:65)"""
    if act_tensor is not None and quant_search:
        bs = weight_config["weight_block_size"]
        if fmt == "mxint":
            return mxint_clip_search(W1, bs, weight_config["weight_width"], 1, act_tensor=act_tensor,
                                     cali_batch_size=cali_batch_size)[0]
        if fmt == "mxfp":
            return mxfp_clip_search(W1, bs, weight_config["weight_exponent_width"], weight_config["weight_frac_width"], 1,
                                    act_tensor=act_tensor, cali_batch_size=cali_batch_size)[0]
    if fmt == "mxint":
        return mxint_quantizer(W1, weight_config["weight_block_size"], weight_config["weight_width"], 1,
                               quantile_search=quant_search)
    if fmt == "mxfp":
        return mxfp_quantizer(W1, weight_config["weight_block_size"], weight_config["weight_exponent_width"],
                              weight_config["weight_frac_width"], 1, quantile_search=quant_search)
    raise ValueError(fmt)


def fasterquant(weight, H, fmt, weight_config, percdamp=0.01, quant_search=True, activation=None, cali_batch_size=32):
    """gptq.py:39-122; ``activation`` [nsamples, tokens, columns]: the layer's calibration inputs (clip_search_y)"""
    W = weight.clone()
    Hinv, dead = inverse_factor(H, percdamp)
    W[:, dead] = 0
    Q = torch.zeros_like(W)
    bs = weight_config["weight_block_size"]
    cols = W.shape[1]
    for i1 in range(0, cols, bs):
        i2 = min(i1 + bs, cols)
        W1 = W[:, i1:i2].clone()
        act1 = None if activation is None else activation[:, :, i1:i2].clone()
        Q1 = quantize_group(W1, fmt, weight_config, quant_search, act1, cali_batch_size)
        Hinv1 = Hinv[i1:i2, i1:i2]
        err = (W1 - Q1) / torch.diag(Hinv1).unsqueeze(0)
        Q[:, i1:i2] = Q1
        W[:, i2:] -= err.matmul(Hinv[i1:i2, i2:])
    return Q


def proxy_loss(weight, Q, H):
    """tr((W - Q) H (W - Q)^T): the layer's output error on the calibration inputs, up to the factor 2/n"""
    E = (weight - Q).double()
    return float((E @ H.double() * E).sum())
