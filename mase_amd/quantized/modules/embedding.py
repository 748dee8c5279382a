"""``EmbeddingMXInt`` / ``EmbeddingMXFP`` with the constructors, config keys and results of the reference's
``chop/nn/quantized/modules/embedding.py:9-71``: the embedding table is MX-quantized along the embedding dimension
(``block_dim=1``) at forward time and then indexed.

The reference quantizes the whole table on every call.  Quantization blocks lie inside one row, so quantizing only
the rows that are looked up gives bit-identical results at a cost proportional to the number of tokens instead of
the vocabulary size; that is what happens here whenever the row length is a multiple of the block size and the
lookup has no side effect on the table (``max_norm is None``).  Otherwise the reference's order is kept.
"""
from __future__ import annotations

from functools import partial

import torch
from torch import Tensor, nn
from torch.nn import functional as F

from ...quantizers import mxfp_quantizer, mxint_quantizer


class _EmbeddingMX(nn.Embedding):
    def __init__(self, num_embeddings, embedding_dim, config=None, **kwargs):
        super().__init__(num_embeddings, embedding_dim, **kwargs)
        self.config = config or {}
        self.bypass = self.config.get("bypass", False)
        if not self.bypass:
            self.w_quantizer = self._make_quantizer()

    def _make_quantizer(self):
        raise NotImplementedError

    @torch.no_grad()
    def forward(self, input: Tensor) -> Tensor:
        if self.bypass:
            return super().forward(input)
        rows_first = (self.max_norm is None and not self.sparse
                      and self.embedding_dim % self.config["weight_block_size"] == 0)
        if rows_first:
            rows = F.embedding(input, self.weight, self.padding_idx, None, self.norm_type, self.scale_grad_by_freq, False)
            if rows.numel() == 0:
                return rows
            return self.w_quantizer(rows.reshape(-1, self.embedding_dim)).reshape(rows.shape)
        weight = self.w_quantizer(self.weight)
        return F.embedding(input, weight, self.padding_idx, self.max_norm, self.norm_type, self.scale_grad_by_freq,
                           self.sparse)


class EmbeddingMXFP(_EmbeddingMX):
    """MXFP-quantized Embedding. Weight is quantized at forward time."""

    def _make_quantizer(self):
        return partial(mxfp_quantizer, block_size=self.config["weight_block_size"],
                       element_exp_bits=self.config["weight_exponent_width"],
                       element_frac_bits=self.config["weight_frac_width"], block_dim=1)


class EmbeddingMXInt(_EmbeddingMX):
    """MXInt-quantized Embedding. Weight is quantized at forward time."""

    def _make_quantizer(self):
        return partial(mxint_quantizer, block_size=self.config["weight_block_size"],
                       element_bits=self.config["weight_width"], block_dim=1)
