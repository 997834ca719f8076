"""Pre-norm block: h += mixer(norm1(h)); h += ffn(norm2(h))  (src/models/qwen3.hpp:122-278).
The sums are carried as a pending addend and folded into the next norm's kernel."""
from __future__ import annotations

from ..kernels import ops
from .base import Block, FeedForward, Mixer, Norm


class PreNormBlock(Block):
    def __init__(self, norm1: Norm, mixer: Mixer, norm2: Norm, ffn: FeedForward,
                 names=("input_layernorm", "self_attn", "post_attention_layernorm", "mlp")):
        self.norm1, self.mixer, self.norm2, self.ffn = norm1, mixer, norm2, ffn
        self.names = names

    def _parts(self, prefix):
        return zip((self.norm1, self.mixer, self.norm2, self.ffn), (prefix + "." + n for n in self.names))

    def weight_specs(self, prefix):
        return [s for part, p in self._parts(prefix) for s in part.weight_specs(p)]

    def bind(self, prefix, weights):
        for part, p in self._parts(prefix):
            part.bind(p, weights)

    def entry_norm(self):
        return self.norm1

    def capturable(self, batch):
        return all(part.capturable(batch) for part in (self.norm1, self.mixer, self.norm2, self.ffn))

    def forward(self, resid, pending, batch, cache, store=True, next_norm=None):
        act = batch.act_dtype
        ready = isinstance(pending, ops.ScaledInput)
        mine = ready and pending.norm is self.norm1
        fold = self.norm2.foldable(act) is not None and self.mixer.can_fold(batch) and self.ffn.can_fold(batch)
        if fold and not ops.folded_products_take(pending if mine else None, batch.T):
            # beyond 64 rows the folded products take an input in operand order only, which only the part before this
            # block can have prepared (another kind of block, a position encoding on the embeddings, parts that fold up
            # to fewer rows may not have): the plain path then
            fold = False
        if fold:
            # few rows: the sums go into the stream inside the products, the norms' scales into the products after them
            if mine:
                n1 = pending
            else:
                n1 = self.norm1.add_norm(resid, None if ready else pending, act)
            n2 = self.mixer.forward_into(n1, batch, cache, store, resid, self.norm2)
            if next_norm is not None and next_norm.foldable(act) is not None:
                return resid, self.ffn.forward_into(n2, batch, resid, next_norm)
            return resid, self.ffn.forward(n2, batch)
        n1 = self.norm1.add_norm(resid, None if ready else pending, act)
        a = self.mixer.forward(n1, batch, cache, store)
        n2 = self.norm2.add_norm(resid, a, act)
        return resid, self.ffn.forward(n2, batch)
