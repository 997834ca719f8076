"""The step function: runs a batch of (request, its next tokens) from the cache
and returns logits at the wanted places.

It stands where the reference has ``ModelRunner::execute_model``
(src/engine/model_runner.cpp:49-157), but samples nothing and changes no
request: it runs only the tokens it is given, as one batch, prompt portions
beside single decoded tokens, cut anywhere.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..cache.manager import CacheManager
from ..cache.spec import PagedKV
from ..cache.storage import CacheStorage
from ..config.registry import load_model_config
from ..models.base import DecoderModel
from ..weights.loader import load_weights
from .batch import StepBatch, StepEntry

DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32, "bf16": torch.bfloat16, "fp32": torch.float32}


def resolve_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError("dtype must be bfloat16 or float32")
        return name
    if name not in DTYPES:
        raise ValueError("dtype must be 'bfloat16' or 'float32', got %r" % (name,))
    return DTYPES[name]


def load_model(folder: str, dtype, device) -> DecoderModel:
    """config.json -> architecture -> model of parts, weights bound by name."""
    arch, cfg = load_model_config(folder)
    model = arch.build(cfg)
    weights = load_weights(folder, model.weight_specs(), resolve_dtype(dtype), device)
    model.bind(weights, device)
    return model


class ModelRunner:
    def __init__(self, model: DecoderModel, dtype, device, page_size: int, num_pages: int, max_num_seqs: int,
                 max_num_batched_tokens: int = 16384):
        self.model = model
        self.act_dtype = resolve_dtype(dtype)
        self.device = torch.device(device)
        self.max_num_batched_tokens = max_num_batched_tokens
        self.manager = CacheManager(model.cache_specs(), page_size, num_pages, max_num_seqs)
        self.storage = CacheStorage(self.manager, self.act_dtype, self.device)
        self.steps_run = 0

    @staticmethod
    def bytes_per_page(model: DecoderModel, page_size: int, dtype) -> int:
        """Device bytes that one more page in every page group costs."""
        act = 2 if resolve_dtype(dtype) == torch.bfloat16 else 4
        return sum(2 * s.num_kv_heads * s.head_dim * page_size * act for s in model.cache_specs() if isinstance(s, PagedKV))

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Run the entries' tokens as one batch.  Pages for them must have been reserved
        (``manager.reserve``).  Returns float32 logits [wanted rows, vocab] in the order of the
        entries and of their ``want``; afterwards the tokens count as cached."""
        entries = list(entries)
        if not entries:
            return torch.empty((0, self.model.vocab_size), dtype=torch.float32, device=self.device)
        batch = StepBatch(entries, self.manager, self.act_dtype, self.device, self.model.vocab_size)
        if batch.T > self.max_num_batched_tokens:
            raise ValueError("the step holds %d tokens, max_num_batched_tokens is %d" % (batch.T, self.max_num_batched_tokens))
        if self.model.max_positions and batch.max_kv_len > self.model.max_positions:
            raise ValueError("a request would reach %d tokens, the model's positions end at %d"
                             % (batch.max_kv_len, self.model.max_positions))
        self.model.plan(batch)
        batch.upload()
        self._reset_fresh_state(batch)
        logits = self.model.forward(batch, self.storage)
        for e in entries:
            self.manager.commit(e.cache, len(e.tokens))
        self.steps_run += 1
        return logits

    def _reset_fresh_state(self, batch: StepBatch) -> None:
        """State slots of requests that run their first tokens start from zero."""
        if not self.manager.state_groups:
            return
        fresh = [e.cache.slot for e in batch.entries if e.cache.fresh]
        if not fresh:
            return
        idx = torch.tensor(fresh, dtype=torch.long, device=self.device)
        for g in self.manager.state_groups:
            for cid in g.cache_ids:
                self.storage.layer(cid).state.index_fill_(0, idx, 0)
