"""A decoder as data: an embedding, a list of layers (blocks of parts), the
order in which they run, a final norm and an output head.

The run order is a list of ``LayerCall``s.  It may name a layer twice (its
weights are used again, each call with a cache of its own) or let a call read
the cache that another call writes (``cache`` = that call's cache id,
``store=False``).  By default layer i runs once with cache i, as in the
reference (src/models/qwen3.hpp:122-278).
"""
from __future__ import annotations

from typing import Dict, List, NamedTuple, Optional, Sequence

import torch

from ..parts.base import Block, Norm, PositionEncoding
from ..parts.embedding import LMHead, TokenEmbedding
from ..weights.loader import WeightSpec


class LayerCall(NamedTuple):
    layer: int
    cache: Optional[int] = None   # cache id; None = the call has no cache of its own kind
    store: bool = True            # False: read cache ``cache`` without writing


class DecoderModel:
    def __init__(self, config, embed: TokenEmbedding, position: Optional[PositionEncoding], layers: Sequence[Block],
                 final_norm: Norm, lm_head: LMHead, schedule: Optional[Sequence[LayerCall]] = None,
                 names: Dict[str, str] = None, max_positions: int = 0):
        self.config = config
        self.embed, self.position, self.layers = embed, position, list(layers)
        self.final_norm, self.lm_head = final_norm, lm_head
        self.schedule = list(schedule) if schedule is not None else [LayerCall(i, i) for i in range(len(self.layers))]
        n = dict(embed="model.embed_tokens", position="model.position", layers="model.layers.%d", final_norm="model.norm",
                 lm_head="lm_head")
        n.update(names or {})
        self.names = n
        self.max_positions = max_positions
        self.vocab_size = lm_head.vocab_size
        for call in self.schedule:
            if not (0 <= call.layer < len(self.layers)):
                raise ValueError("the run order names layer %d of %d" % (call.layer, len(self.layers)))
        self.cache_specs()  # validates the run order

    # ---- weights ---------------------------------------------------------
    def weight_specs(self) -> List[WeightSpec]:
        specs = list(self.embed.weight_specs(self.names["embed"]))
        if self.position is not None:
            specs += self.position.weight_specs(self.names["position"])
        for i, layer in enumerate(self.layers):
            specs += layer.weight_specs(self.names["layers"] % i)
        specs += self.final_norm.weight_specs(self.names["final_norm"])
        specs += self.lm_head.weight_specs(self.names["lm_head"])
        return specs

    def bind(self, weights: Dict[str, torch.Tensor], device) -> None:
        self.embed.bind(self.names["embed"], weights)
        if self.position is not None:
            self.position.bind(self.names["position"], weights)
            self.position.prepare(device, self.max_positions)
        for i, layer in enumerate(self.layers):
            layer.bind(self.names["layers"] % i, weights)
        self.final_norm.bind(self.names["final_norm"], weights)
        self.lm_head.bind(self.names["lm_head"], weights)

    # ---- cache -----------------------------------------------------------
    def cache_specs(self) -> List[Optional[object]]:
        """Need of every cache id, taken from the call that writes it."""
        ids = [c.cache for c in self.schedule if c.cache is not None]
        specs: List[Optional[object]] = [None] * (max(ids) + 1 if ids else 0)
        writers = {}
        for call in self.schedule:
            if call.cache is None or not call.store:
                continue
            if call.cache in writers:
                raise ValueError("cache %d is written by two calls of the run order" % call.cache)
            writers[call.cache] = call
            specs[call.cache] = self.layers[call.layer].mixer.cache_spec()
        for call in self.schedule:
            if call.cache is not None and not call.store:
                if call.cache not in writers:
                    raise ValueError("a call reads cache %d that no call writes" % call.cache)
                if self.layers[call.layer].mixer.cache_spec() != specs[call.cache]:
                    raise ValueError("layer %d reads cache %d of another shape" % (call.layer, call.cache))
        return specs

    # ---- step ------------------------------------------------------------
    def plan(self, batch) -> None:
        for call in self.schedule:
            self.layers[call.layer].mixer.plan(batch)

    def plan_ints(self, entries: int) -> int:
        """Most int32 values that the mixers' plans add to a step of ``entries`` single tokens (``Mixer.plan_arrays``)."""
        arrays = {}
        for call in self.schedule:
            arrays.update(self.layers[call.layer].mixer.plan_arrays(entries))
        return sum(arrays.values()) + 4 * len(arrays)

    def capturable(self, batch) -> bool:
        """Whether this step may be recorded in a HIP graph: every part that runs in it says so (``Part.capturable``)."""
        parts = [self.embed, self.final_norm, self.lm_head] + [self.layers[i] for i in sorted({c.layer for c in self.schedule})]
        if self.position is not None:
            parts.append(self.position)
        return all(p.capturable(batch) for p in parts)

    def forward(self, batch, storage, logits_out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Runs the batch's tokens through all calls of the run order; float32 logits [R, vocab]
        at the batch's wanted rows (in ``logits_out`` if the caller brings a tensor of that shape)."""
        calls = self.schedule
        entry = [self.layers[c.layer].entry_norm() for c in calls] + [self.final_norm]
        if self.position is None or type(self.position).on_embeddings is PositionEncoding.on_embeddings:
            resid, pending = self.embed.forward_for(batch.token_ids, entry[0], batch.act_dtype)
        else:
            resid, pending = self.position.on_embeddings(self.embed.forward(batch.token_ids), batch), None
        for i, call in enumerate(calls):
            cache = storage.layer(call.cache) if call.cache is not None else None
            resid, pending = self.layers[call.layer].forward(resid, pending, batch, cache, call.store, next_norm=entry[i + 1])
        if batch.R == 0:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=resid.device) if logits_out is None else logits_out
        return self.lm_head.logits(resid, pending, self.final_norm, batch, logits_out)
