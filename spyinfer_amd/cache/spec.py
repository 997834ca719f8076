"""What a mixer asks of the cache manager.

The reference has one implicit kind: every layer's keys and values of all
tokens, ``[L, NB, P, n_kv*d]`` (src/engine/model_runner.cpp:35-40).  Here a
mixer states its need and layers with equal needs form a group with pages and
block tables of its own.
"""
from __future__ import annotations

import dataclasses
from typing import Optional, Tuple


@dataclasses.dataclass(frozen=True)
class PagedKV:
    """Keys and values of every token, in pages; ``window`` = only the last
    ``window`` tokens are ever read again (older pages are given back)."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclasses.dataclass(frozen=True)
class FixedState:
    """State of fixed size per request, ``shape`` elements of ``dtype``
    ("float32" or "activation") in a slot; zeroed when a request is admitted."""

    shape: Tuple[int, ...]
    dtype: str = "float32"
