"""Device memory behind the cache manager's page and slot numbers.

Per page group, for its ``n`` layer caches:
  keys    ``[n, num_pages, num_kv_heads, page_size, head_dim]``
  values  ``[n, num_pages, num_kv_heads, head_dim, page_size]``  (transposed in the page)
A page number addresses the same page in every layer of the group, as in the
reference (src/engine/model_runner.cpp:35-40, layout ``[L, NB, P, n_kv*d]``
there).  Here one head's part of a page is contiguous, so that a wave reads it
with full-width loads, and values lie with the key index innermost, which is
the operand order of the MFMA product P.V.
Per state group: ``[n, num_slots, *shape]``.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .manager import CacheManager


class PagedKVLayer:
    """The part of a page group's memory that one layer cache owns."""

    def __init__(self, group: int, k: torch.Tensor, v: torch.Tensor, page_size: int):
        self.group = group
        self.k = k
        self.v = v
        self.page_size = page_size
        self.num_pages = k.shape[0]


class StateLayer:
    def __init__(self, group: int, state: torch.Tensor):
        self.group = group
        self.state = state      # [num_slots, *shape]


class CacheStorage:
    def __init__(self, manager: CacheManager, act_dtype: torch.dtype, device):
        self.manager = manager
        self.layers: Dict[int, object] = {}
        self.tensors: List[torch.Tensor] = []
        for g in manager.page_groups:
            n, s = len(g.cache_ids), g.spec
            k = torch.zeros((n, g.pool.num_pages, s.num_kv_heads, g.page_size, s.head_dim), dtype=act_dtype, device=device)
            v = torch.zeros((n, g.pool.num_pages, s.num_kv_heads, s.head_dim, g.page_size), dtype=act_dtype, device=device)
            self.tensors += [k, v]
            for i, cid in enumerate(g.cache_ids):
                self.layers[cid] = PagedKVLayer(g.index, k[i], v[i], g.page_size)
        for g in manager.state_groups:
            dt = torch.float32 if g.spec.dtype == "float32" else act_dtype
            st = torch.zeros((len(g.cache_ids), manager.slots.num_slots) + tuple(g.spec.shape), dtype=dt, device=device)
            self.tensors.append(st)
            for i, cid in enumerate(g.cache_ids):
                self.layers[cid] = StateLayer(g.index, st[i])

    def layer(self, cache_id: int):
        return self.layers.get(cache_id)

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.tensors)

    @staticmethod
    def bytes_per_page(manager_specs, page_size: int, act_bytes: int) -> int:
        """Bytes that one more page costs, summed over all page groups."""
        total = 0
        for spec, n_layers in manager_specs:
            total += 2 * n_layers * spec.num_kv_heads * spec.head_dim * page_size * act_bytes
        return total
