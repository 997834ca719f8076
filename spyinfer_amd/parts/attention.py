"""Grouped-query attention over the paged cache.

Per step: fused q/k/v projection; per-head RMS norm of q and k (optional;
before the rotation, src/models/qwen3.hpp:160-194); rotation; keys and values
of all tokens of the step written to their pages before any query reads
(src/backends/cpu/cpu_attention.cpp:61-68); then every query reads its keys
through its request's block table with the causal mask ``key <= position``
(:98-111), scale 1/sqrt(d) after the dot product (:59, :110), kv head
``h * n_kv / n_q`` (:96); output projection.  One meaning for whole prompts,
portions and single tokens.  ``window`` keeps only the last ``window`` keys.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from ..cache.spec import PagedKV
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Mixer, PositionEncoding


class PagedAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: Optional[PositionEncoding], qk_norm_eps: Optional[float] = None,
                 window: Optional[int] = None, scale: Optional[float] = None):
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        self.position = position
        self.qk_norm_eps = qk_norm_eps
        self.window = window
        self.scale = 1.0 / math.sqrt(head_dim) if scale is None else float(scale)
        self.w_qkv = self.w_o = self.q_norm = self.k_norm = self.w_qkv_tiled = self.w_o_tiled = None

    # ---- weights ---------------------------------------------------------
    def weight_specs(self, prefix):
        H, nq, nkv, d = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim
        specs = [WeightSpec(prefix + ".q_proj.weight", (nq * d, H)), WeightSpec(prefix + ".k_proj.weight", (nkv * d, H)),
                 WeightSpec(prefix + ".v_proj.weight", (nkv * d, H)), WeightSpec(prefix + ".o_proj.weight", (H, nq * d))]
        if self.qk_norm_eps is not None:
            specs += [WeightSpec(prefix + ".q_norm.weight", (d,), "norm"), WeightSpec(prefix + ".k_norm.weight", (d,), "norm")]
        return specs

    def bind(self, prefix, weights):
        q, k, v = (weights[prefix + ".%s_proj.weight" % n] for n in "qkv")
        if not (q.dtype == k.dtype == v.dtype):
            q, k, v = q.float(), k.float(), v.float()
        # one product for q, k and v: rows [q heads | k heads | v heads]
        self.w_qkv = torch.cat([q, k, v], dim=0).contiguous()
        self.w_o = weights[prefix + ".o_proj.weight"]
        self.w_qkv_tiled, self.w_o_tiled = ops.tile_weight(self.w_qkv), ops.tile_weight(self.w_o)
        if self.qk_norm_eps is not None:
            self.q_norm, self.k_norm = weights[prefix + ".q_norm.weight"], weights[prefix + ".k_norm.weight"]
            if self.q_norm.dtype != self.k_norm.dtype:
                self.q_norm, self.k_norm = self.q_norm.float(), self.k_norm.float()

    # ---- cache -----------------------------------------------------------
    def cache_spec(self):
        return PagedKV(self.num_kv_heads, self.head_dim, self.window)

    def plan(self, batch) -> None:
        batch.add_attention_tiles(self.num_heads // self.num_kv_heads, ops.prefill_attention_ok(self.head_dim, batch.page_size))

    # ---- step ------------------------------------------------------------
    def can_fold(self, batch):
        return ops.fused_decode_ok(batch.T, batch.act_dtype, self.w_qkv_tiled, self.w_o_tiled)

    def _attend(self, x, batch, cache, store, for_product=False):
        nq, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
        if isinstance(x, ops.ScaledInput):
            qkv = ops.decode_linear(x, self.w_qkv_tiled)
        else:
            qkv = ops.linear(x, self.w_qkv, tiled=self.w_qkv_tiled)
        rot = self.position.rotary() if self.position is not None else None
        cos, sin, rdim = rot if rot is not None else (None, None, 0)
        eps = self.qk_norm_eps if self.qk_norm_eps is not None else 0.0
        meta = batch.attention_meta(cache.group, nq // nkv)
        if ops.fused_attention_ok(qkv.dtype, meta, nq, nkv, d, cache.page_size, rdim, self.q_norm, self.k_norm):
            # single tokens only: the attention kernel norms, rotates and stores by itself
            raw = ops.RawQKV(qkv, self.q_norm, self.k_norm, eps, cos if rdim else None, sin if rdim else None, store)
            return ops.paged_attention(None, cache.k, cache.v, cache.page_size, meta, nq, nkv, d, self.scale, self.window, raw,
                                       for_product=for_product)
        slots = batch.slot_mapping(cache.group) if store else None
        q = ops.qk_norm_rope_store(qkv, nq, nkv, d, self.q_norm, self.k_norm, eps,
                                   cos, sin, rdim, batch.positions, cache.k, cache.v, cache.page_size, slots)
        return ops.paged_attention(q, cache.k, cache.v, cache.page_size, meta, nq, nkv, d, self.scale, self.window,
                                   for_product=for_product)

    def forward(self, x, batch, cache, store=True):
        return ops.linear(self._attend(x, batch, cache, store), self.w_o, tiled=self.w_o_tiled)

    def forward_into(self, x, batch, cache, store, resid, next_norm):
        weight, eps = next_norm.foldable(batch.act_dtype)
        return ops.decode_linear_residual(self._attend(x, batch, cache, store, for_product=True), self.w_o_tiled, resid, weight, eps,
                                          next_norm)
