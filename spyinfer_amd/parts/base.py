"""Interfaces of the parts a decoder is put together from.

A part knows its own sizes and constants (given to its constructor), the
safetensors names and shapes of its weights under a prefix, and how to run on
the tokens of a step.  No part knows which model it is in; the model picks the
parts layer by layer from its configuration.

All parts run on a flat batch of tokens ``[T, ...]`` described by a
``StepBatch`` (``spyinfer_amd.engine.batch``).  The residual stream is
float32; activations between parts have the run dtype (bfloat16 or float32).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..weights.loader import WeightSpec


class Part:
    """Common protocol: weights by name."""

    def weight_specs(self, prefix: str) -> List[WeightSpec]:
        """Tensors this part reads, with full names under ``prefix``."""
        return []

    def bind(self, prefix: str, weights: Dict[str, torch.Tensor]) -> None:
        """Take the tensors named by ``weight_specs(prefix)`` (already on the device).  A part that copies tensors into
        a form of its own (fused, reordered) may take them out of ``weights`` (``pop``), so that the originals are freed."""

    def capturable(self, batch) -> bool:
        """May this part's work on ``batch`` (a step of single tokens) be recorded once in a HIP graph and replayed for
        later steps of the same shape?  A replay runs the recorded kernels with the recorded addresses and sizes; only
        the CONTENTS of the batch's device arrays (token ids, positions, ``slot_ids``, block tables, what ``plan``
        added) are those of the new step.  So True needs: everything that differs from step to step is read on the
        device from those arrays (never from ``batch.entries``, ``batch.lens`` or other host values, which a replay
        does not see), no copy to the host and no wait for the device, and launch shapes that depend only on the arrays'
        lengths and on what ``plan`` put into the graph's key (``batch.add_graph_key``).  The default is False: a part
        that does not say otherwise is always run kernel by kernel, and so is every step of a model that has one."""
        return False


class Norm(Part):
    """y = norm(x) over the hidden dimension."""

    def add_norm(self, resid: torch.Tensor, delta: Optional[torch.Tensor], out_dtype: torch.dtype,
                 rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """resid += delta in float32 (in place, unless ``rows`` selects rows), then the norm of
        the sum in ``out_dtype``.  Fusing the residual sum into the norm saves one pass over
        the hidden state."""
        raise NotImplementedError

    def foldable(self, out_dtype: torch.dtype):
        """None, or (weight, eps) if this norm can be folded into the products around it when a step has few rows:
        the product before it adds to the stream and prepares this norm's input, the product after it applies the
        scale (``spyinfer_amd.kernels.ops.ScaledInput``).  Parts that do not know of this are never asked."""
        return None


class PositionEncoding(Part):
    """How positions enter the model.  A rotary encoding hands its tables to the mixer,
    which applies them to queries and keys; an encoding added to the embeddings
    overrides ``on_embeddings``."""

    def prepare(self, device, max_positions: int) -> None:
        pass

    def rotary(self):
        """None, or (cos, sin, rotary_dim): float32 tables [positions, rotary_dim/2]."""
        return None

    def on_embeddings(self, hidden: torch.Tensor, batch) -> torch.Tensor:
        return hidden


class Mixer(Part):
    """Mixes information between the tokens of a request (attention here)."""

    def cache_spec(self):
        """``PagedKV``, ``FixedState`` or None: what one layer of this mixer keeps per request."""
        return None

    def plan(self, batch) -> None:
        """Called once per step and per distinct mixer before the batch goes to the device:
        may add integer arrays to it with ``batch.add_array``."""

    def plan_arrays(self, entries: int) -> dict:
        """{array name: most int32 values} of what ``plan`` adds to a step of ``entries`` single tokens: the runner's
        account of the device memory that a captured step of that size holds.  Arrays that several layers share have
        one name."""
        return {}

    def forward(self, x: torch.Tensor, batch, cache, store: bool = True) -> torch.Tensor:
        """x [T, H] (normed) -> [T, H].  ``cache`` is this call's layer cache
        (``PagedKVLayer``/``StateLayer``/None).  ``store=False``: read the cache of
        another layer without writing to it."""
        raise NotImplementedError

    def can_fold(self, batch) -> bool:
        """True if, for this step, ``forward`` takes a ``ScaledInput`` in place of x and ``forward_into`` exists."""
        return False

    def forward_into(self, x, batch, cache, store, resid: torch.Tensor, next_norm: Norm):
        """Optional: resid += mixer(x) in place; returns the ``ScaledInput`` for ``next_norm`` (which is foldable)."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x: torch.Tensor, batch) -> torch.Tensor:
        """x [T, H] (normed) -> [T, H]."""
        raise NotImplementedError

    def can_fold(self, batch) -> bool:
        """As ``Mixer.can_fold``."""
        return False

    def forward_into(self, x, batch, resid: torch.Tensor, next_norm: Norm):
        """Optional: resid += ffn(x) in place; returns the ``ScaledInput`` for ``next_norm`` (which is foldable)."""
        raise NotImplementedError


class Block(Part):
    """Arrangement of norm, mixer and feed-forward in one layer."""

    mixer: Mixer

    def forward(self, resid: torch.Tensor, delta, batch, cache, store: bool = True, next_norm: Optional[Norm] = None):
        """(residual stream, pending) -> (residual stream, pending).  ``pending`` is None, an addend [T, H] that
        the next norm sums into the stream, or a ``ScaledInput``: then the stream is complete and the input of
        the norm named in it is prepared (a block that cannot use it ignores it).  ``next_norm``: the norm that
        reads the stream after this block, if the caller knows it; only then may a ``ScaledInput`` be returned."""
        raise NotImplementedError

    def entry_norm(self) -> Optional[Norm]:
        """The norm that reads the stream first in this block, if it wants the block before it to prepare its
        input."""
        return None
