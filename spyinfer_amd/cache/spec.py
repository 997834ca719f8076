"""What a mixer asks of the cache manager, as kinds that describe themselves.

The reference has one implicit kind: every layer's keys and values of all
tokens, ``[L, NB, P, n_kv*d]`` (src/engine/model_runner.cpp:35-40).  Here a
mixer states its need as a ``CacheKind``; layer caches whose kinds are equal
form a group with pages (or slots) and block tables of its own.  A kind says
whether it lives in pages or in per-request slots, how many bytes a page of
it costs, which device tensors back a group of layers, and what one layer of
the group gets handed in ``Mixer.forward``.  The manager and the storage ask
only these questions, so a further kind (another layout, another dtype, one
tensor instead of two) is a subclass and nothing else.
"""
from __future__ import annotations

import dataclasses
from typing import List, Optional, Tuple

import torch


class CacheKind:
    """Base of all cache needs.  Subclasses are frozen dataclasses: equal kinds share a group."""

    #: True: the kind lives in pages that grow with the request's tokens (block table per request);
    #: False: one slot of fixed size per request
    paged: bool = True
    #: paged kinds: only the last ``window`` tokens are ever read again (None = all)
    window: Optional[int] = None

    def page_bytes(self, page_size: int, act_dtype: torch.dtype) -> int:
        """Device bytes of one page (paged) or one slot (not paged) in ONE layer."""
        raise NotImplementedError

    def allocate(self, num_layers: int, count: int, page_size: int, act_dtype: torch.dtype, device) -> List[torch.Tensor]:
        """The tensors behind a group of ``num_layers`` layer caches with ``count`` pages (or slots); zero-filled."""
        raise NotImplementedError

    def layer_view(self, group: int, tensors: List[torch.Tensor], index: int, page_size: int):
        """What layer ``index`` of the group is handed as ``cache`` in ``Mixer.forward``."""
        raise NotImplementedError

    def reset(self, layer, slots: torch.Tensor) -> None:
        """Kinds in slots: the slots ``slots`` (int64 on the device) of this layer view start from their initial
        state; called before the first tokens of a request run."""
        raise NotImplementedError


def _elem(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


class PagedKVLayer:
    """One layer's part of a key/value group: ``k [pages, n_kv, page, d]``, ``v [pages, n_kv, d, page]``."""

    def __init__(self, group: int, k: torch.Tensor, v: torch.Tensor, page_size: int):
        self.group, self.k, self.v, self.page_size = group, k, v, page_size
        self.num_pages = k.shape[0]


class StateLayer:
    def __init__(self, group: int, state: torch.Tensor):
        self.group = group
        self.state = state      # [num_slots, *shape]


@dataclasses.dataclass(frozen=True)
class PagedKV(CacheKind):
    """Keys and values of every token, in pages; ``window`` = only the last
    ``window`` tokens are ever read again (older pages are given back).

    Device layout per group of ``n`` layers: keys ``[n, pages, n_kv, page, d]``, values
    ``[n, pages, n_kv, d, page]`` in the activation dtype.  One head's part of a page is contiguous, so that a wave
    reads it with full-width loads, and values lie with the key index innermost, which is the operand order of the
    MFMA product P.V."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    paged = True

    def page_bytes(self, page_size, act_dtype):
        return 2 * self.num_kv_heads * self.head_dim * page_size * _elem(act_dtype)

    def allocate(self, num_layers, count, page_size, act_dtype, device):
        k = torch.zeros((num_layers, count, self.num_kv_heads, page_size, self.head_dim), dtype=act_dtype, device=device)
        v = torch.zeros((num_layers, count, self.num_kv_heads, self.head_dim, page_size), dtype=act_dtype, device=device)
        return [k, v]

    def layer_view(self, group, tensors, index, page_size):
        return PagedKVLayer(group, tensors[0][index], tensors[1][index], page_size)


@dataclasses.dataclass(frozen=True)
class FixedState(CacheKind):
    """State of fixed size per request, ``shape`` elements of ``dtype``
    ("float32" or "activation") in a slot; zeroed when a request runs its first tokens.
    Device layout per group of ``n`` layers: ``[n, slots, *shape]``."""

    shape: Tuple[int, ...]
    dtype: str = "float32"
    paged = False

    def _dtype(self, act_dtype):
        return torch.float32 if self.dtype == "float32" else act_dtype

    def page_bytes(self, page_size, act_dtype):
        n = 1
        for s in self.shape:
            n *= s
        return n * _elem(self._dtype(act_dtype))

    def allocate(self, num_layers, count, page_size, act_dtype, device):
        return [torch.zeros((num_layers, count) + tuple(self.shape), dtype=self._dtype(act_dtype), device=device)]

    def layer_view(self, group, tensors, index, page_size):
        return StateLayer(group, tensors[0][index])

    def reset(self, layer, slots: torch.Tensor) -> None:
        """Slots of requests that start: their state begins at zero."""
        layer.state.index_fill_(0, slots, 0)
