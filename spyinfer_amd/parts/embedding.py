"""Token embedding and output head.  h[t] = E[id[t]] with no scaling
(src/models/qwen3.hpp:114-119); logits = norm(h) . W^T for the asked rows only, W = E when the
model ties them (src/models/qwen3.hpp:46, 283-301)."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part


class TokenEmbedding(Part):
    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.weight = None

    def weight_specs(self, prefix):
        return [WeightSpec(prefix + ".weight", (self.vocab_size, self.hidden_size))]

    def bind(self, prefix, weights):
        self.weight = weights[prefix + ".weight"]

    def forward(self, ids):
        return ops.embedding(ids, self.weight)

    def forward_for(self, ids, norm, act_dtype):
        """(stream, pending) with the input of ``norm`` prepared where few rows and a foldable norm allow it."""
        fold = norm.foldable(act_dtype) if norm is not None else None
        if fold is None or not ops.fused_decode_ok(ids.shape[0], act_dtype):
            return ops.embedding(ids, self.weight), None
        return ops.embedding_scaled(ids, self.weight, fold[0], fold[1], norm)


class LMHead(Part):
    def __init__(self, vocab_size: int, hidden_size: int, tied_to: TokenEmbedding = None):
        self.vocab_size, self.hidden_size, self.tied_to = vocab_size, hidden_size, tied_to
        self.weight = None

    def weight_specs(self, prefix):
        if self.tied_to is not None:
            # a tied checkpoint may store the head again; it is not read (src/models/qwen3.hpp:46)
            return [WeightSpec(prefix + ".weight", (self.vocab_size, self.hidden_size), optional=True)]
        return [WeightSpec(prefix + ".weight", (self.vocab_size, self.hidden_size))]

    def bind(self, prefix, weights):
        self.weight = self.tied_to.weight if self.tied_to is not None else weights[prefix + ".weight"]
        self.weight_tiled = ops.tile_weight(self.weight)

    def can_fold(self, batch):
        # above 32 rows the library's product (after a norm kernel) is faster for a matrix of this size (measured with
        # 151936 x 4096: 229 / 253 us at 24 / 32 rows against the library's 264 / 269, but 323 against 260 at 48)
        return batch.T <= 32 and ops.fused_decode_ok(batch.T, batch.act_dtype, self.weight_tiled)

    def forward(self, normed):
        if isinstance(normed, ops.ScaledInput):
            return ops.decode_linear(normed, self.weight_tiled, torch.float32)
        return ops.linear(normed, self.weight, torch.float32, tiled=self.weight_tiled)
