"""Device memory behind the cache manager's page and slot numbers.

Every group's kind (``cache.spec.CacheKind``) allocates the tensors of its
layers and says what one layer sees of them.  A page number addresses the same
page in every layer of a group, as in the reference
(src/engine/model_runner.cpp:35-40, layout ``[L, NB, P, n_kv*d]`` there).
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .manager import CacheManager
from .spec import PagedKVLayer, StateLayer  # noqa: F401  (the layer views' home was here)


class CacheStorage:
    def __init__(self, manager: CacheManager, act_dtype: torch.dtype, device):
        self.manager = manager
        self.layers: Dict[int, object] = {}
        self.tensors: List[torch.Tensor] = []
        for groups, count_of in ((manager.page_groups, lambda g: g.pool.num_pages),
                                 (manager.state_groups, lambda g: manager.slots.num_slots)):
            for g in groups:
                tensors = g.spec.allocate(len(g.cache_ids), count_of(g), manager.page_size, act_dtype, device)
                self.tensors += tensors
                for i, cid in enumerate(g.cache_ids):
                    self.layers[cid] = g.spec.layer_view(g.index, tensors, i, manager.page_size)

    def layer(self, cache_id: int):
        return self.layers.get(cache_id)

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.tensors)

    def fill(self, value: float) -> None:
        """Every element of every cache tensor := value (tests poison the pool with NaN this way: a slot is
        always written before it is read, so a correct engine never shows it)."""
        for t in self.tensors:
            if t.is_floating_point():
                t.fill_(value)

    @staticmethod
    def bytes_per_page(cache_specs, page_size: int, act_dtype: torch.dtype) -> int:
        """Bytes that one more page in every page group costs, over all layer caches."""
        return sum(s.page_bytes(page_size, act_dtype) for s in cache_specs if s is not None and s.paged)
