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

    def capturable(self, batch):
        return True

    def forward(self, ids):
        return ops.embedding(ids, self.weight)

    def forward_for(self, ids, norm, act_dtype):
        """(stream, pending) with the input of ``norm`` prepared where few rows and a foldable norm allow it."""
        fold = norm.foldable(act_dtype) if norm is not None else None
        if fold is None or not ops.fused_decode_ok(ids.shape[0], act_dtype):
            return ops.embedding(ids, self.weight), None
        return ops.embedding_scaled(ids, self.weight, fold[0], fold[1], norm)


class LMHead(Part):
    def __init__(self, vocab_size: int, hidden_size: int, tied_to: TokenEmbedding = None, fold_rows: int = 64):
        """``fold_rows``: most rows for which the head runs as a decode product with the final norm folded in.  Above,
        the library's product after a norm kernel is faster for a large matrix (measured with 151936 x 4096: 235 / 246 /
        253 / 267 us at 24 / 32 / 48 / 64 rows against the library's 263 / 270 / 258 / 268 and a norm kernel of 6, but
        281 / 288 / 367 against 274 / 280 / 293 at 80 / 96 / 128)."""
        self.vocab_size, self.hidden_size, self.tied_to = vocab_size, hidden_size, tied_to
        self.fold_rows = fold_rows
        self.weight = None

    def weight_specs(self, prefix):
        if self.tied_to is not None:
            # a tied checkpoint may store the head again; it is not read (src/models/qwen3.hpp:46)
            return [WeightSpec(prefix + ".weight", (self.vocab_size, self.hidden_size), optional=True)]
        return [WeightSpec(prefix + ".weight", (self.vocab_size, self.hidden_size))]

    def bind(self, prefix, weights):
        if self.tied_to is not None:
            self.weight, self.weight_tiled = ops.weight_forms(self.tied_to.weight, keep_rows=True)   # the table's rows are looked up
        else:
            self.weight, self.weight_tiled = ops.weight_forms(weights.pop(prefix + ".weight"))

    def capturable(self, batch):
        return True

    def can_fold(self, batch):
        # without the matrix's rows the library's product would have them restored first (more bytes than the product
        # itself reads): the folded product stands as far as it is built
        rows = ops.FUSED_DECODE_MAX_ROWS if isinstance(self.weight, ops.TiledOnly) else self.fold_rows
        return ops.fused_decode_ok(batch.T, batch.act_dtype, self.weight_tiled, max_rows=rows)

    def logits(self, resid, pending, final_norm, batch, out=None):
        """The end of a forward pass: ``final_norm`` of the stream (``pending`` as a block leaves it: None, an addend
        or the prepared input of a norm) at the batch's wanted rows, then the head."""
        if isinstance(pending, ops.ScaledInput):
            if pending.norm is final_norm and batch.all_rows_wanted and self.can_fold(batch):
                return self.forward(pending, out)
            pending = None                       # the stream is complete
        return self.forward(final_norm.add_norm(resid, pending, batch.act_dtype, batch.logit_rows), out)

    def forward(self, normed, out=None):
        """float32 logits [rows, vocab]; written into ``out`` if the caller brings a tensor of that shape."""
        if isinstance(normed, ops.ScaledInput):
            return ops.decode_linear(normed, self.weight_tiled, torch.float32, out)
        return ops.linear(normed, self.weight, torch.float32, tiled=self.weight_tiled, out=out)
