"""Gated feed-forward: down( silu(gate(x)) * up(x) ), no biases
(src/models/qwen3.hpp:232-263; src/backends/cpu/x64/kernels.cpp:242-247).
Gate and up run as one product with rows [gate | up]."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import FeedForward


class GatedMLP(FeedForward):
    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu", fold_rows=None):
        """``fold_rows``: most rows of a step whose products here run with the norms and the residual sum folded in
        (None: ``ops.default_fold_rows`` of this part's matrices)."""
        if activation != "silu":
            raise ValueError("GatedMLP: activation %r is not implemented" % activation)
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.fold_rows = fold_rows
        self.w_gate_up = self.w_down = self.w_gate_up_tiled = self.w_down_tiled = None

    def weight_specs(self, prefix):
        H, I = self.hidden_size, self.intermediate_size
        return [WeightSpec(prefix + ".gate_proj.weight", (I, H)), WeightSpec(prefix + ".up_proj.weight", (I, H)),
                WeightSpec(prefix + ".down_proj.weight", (H, I))]

    def bind(self, prefix, weights):
        # (popped: the separate matrices are freed once they are fused, see PagedAttention.bind)
        g, u = weights.pop(prefix + ".gate_proj.weight"), weights.pop(prefix + ".up_proj.weight")
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        self.w_gate_up = torch.cat([g, u], dim=0).contiguous()
        del g, u
        # tiles 0 .. I/16 - 1 of the tiled copy are gate rows, the rest up rows: what the fused SwiGLU kernel expects
        if self.intermediate_size % 16 == 0:
            self.w_gate_up, self.w_gate_up_tiled = ops.weight_forms(self.w_gate_up)
        self.w_down, self.w_down_tiled = ops.weight_forms(weights.pop(prefix + ".down_proj.weight"))

    def capturable(self, batch):
        return True

    def can_fold(self, batch):
        return ops.fused_decode_ok(batch.T, batch.act_dtype, self.w_gate_up_tiled, self.w_down_tiled, max_rows=self.fold_rows)

    def forward(self, x, batch):
        if isinstance(x, ops.ScaledInput):
            return ops.linear(ops.decode_linear_swiglu(x, self.w_gate_up_tiled), self.w_down, tiled=self.w_down_tiled)
        return ops.linear(ops.linear_swiglu(x, self.w_gate_up, self.w_gate_up_tiled), self.w_down, tiled=self.w_down_tiled)

    def forward_into(self, x, batch, resid, next_norm):
        weight, eps = next_norm.foldable(batch.act_dtype)
        return ops.decode_linear_residual(ops.decode_linear_swiglu(x, self.w_gate_up_tiled, for_product=True), self.w_down_tiled,
                                          resid, weight, eps, next_norm)
