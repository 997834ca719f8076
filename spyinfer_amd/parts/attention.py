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

import numpy as np
import torch

from ..cache.spec import PagedKV
from ..kernels import key_pieces, ops
from ..weights.loader import WeightSpec
from .base import Mixer, PositionEncoding


ROWS_PER_TILE = 16        # rows of (token, head-in-group) pairs in a small attention tile
BIG_MIN_ROWS = 64         # entries with at least this many rows go to the prefill kernel


def plan_attention_tiles(batch, group_size: int, big_rows: int = 0, key_parts: bool = True) -> None:
    """Adds to the step's arrays the tiles over each entry's rows (token-major, head-in-group minor) for a query-head
    group of ``group_size``: entries with at least BIG_MIN_ROWS rows are cut into tiles of ``big_rows`` rows (the
    LDS-sharing prefill kernel; 0: never), the others into 16-row tiles (one block of waves each).  Once per step,
    group size and tile size.  ``key_parts``: the caller's launches take the number of key parts from the longest
    request (False: its keys are cut another way, ``plan_decode_pieces``)."""
    if key_parts:
        # the 16-row tiles' keys are split into a number of parts that follows the longest request: a launch shape
        batch.add_graph_key("attention_key_parts", ops.key_parts_for(batch.max_kv_len))
    note = ("attention_tiles", group_size, big_rows)
    if note in batch.shared:
        return
    S, lens = batch.S, batch.lens
    rows = lens.astype(np.int64) * group_size
    big = (rows >= BIG_MIN_ROWS) & bool(big_rows)
    counts = {}
    for kind, size, mask in (("small", ROWS_PER_TILE, ~big), ("big", max(big_rows, 1), big)):
        ntiles = np.where(mask, (rows + size - 1) // size, 0)
        tile_entry = np.repeat(np.arange(S, dtype=np.int32), ntiles)
        first = np.zeros(S + 1, dtype=np.int64)
        np.cumsum(ntiles, out=first[1:])
        tile_row0 = ((np.arange(int(first[-1]), dtype=np.int64) - first[:-1][tile_entry]) * size).astype(np.int32)
        if kind == "big" and tile_entry.shape[0] > 2:
            # the prefill kernel gives a block the tiles b and n - 1 - b: sorted by the keys they read, blocks are even
            pos0 = batch.host_array("pos0")[tile_entry].astype(np.int64)
            last_tok = np.minimum(lens[tile_entry].astype(np.int64), (tile_row0.astype(np.int64) + size + group_size - 1) // group_size)
            order = np.argsort(-(pos0 + last_tok), kind="stable")
            tile_entry, tile_row0 = tile_entry[order], tile_row0[order]
        counts[kind] = int(first[-1])
        batch.add_array("tile_entry_%s_%d_%d" % (kind, group_size, big_rows), tile_entry)
        batch.add_array("tile_row0_%s_%d_%d" % (kind, group_size, big_rows), tile_row0)
    batch.shared[note] = counts


def plan_decode_pieces(batch, n_kv: int, window: int, head_dim: int) -> None:
    """Adds to the arrays of a step of single tokens its keys cut into pieces of even size (``key_pieces.decode_pieces``), for
    layers of ``n_kv`` kv heads of ``head_dim`` and this window.  The array's length follows the numbers of entries and
    heads alone."""
    note = ("decode_pieces", n_kv, window, head_dim)
    if note not in batch.shared:
        batch.add_array("decode_pieces_%d_%d_%d" % note[1:], key_pieces.decode_pieces(batch.host_array("kv_len"), n_kv, window, head_dim=head_dim))
        batch.shared[note] = True


def attention_meta(batch, group: int, group_size: int, big_rows: int = 0) -> ops.AttentionMeta:
    """The step's description for the attention kernels, from the batch's arrays on the device (one object per step,
    cache group, group size and tile size)."""
    note = ("attention_meta", group, group_size, big_rows)
    meta = batch.shared.get(note)
    if meta is None:
        tiles = None
        counts = batch.shared.get(("attention_tiles", group_size, big_rows))
        if counts is not None:
            tiles = {kind: (batch.array("tile_entry_%s_%d_%d" % (kind, group_size, big_rows)),
                            batch.array("tile_row0_%s_%d_%d" % (kind, group_size, big_rows)), n) for kind, n in counts.items()}
        pieces = {key[1:]: batch.array("decode_pieces_%d_%d_%d" % key[1:]).view(-1, key_pieces.PIECE_RECORD)
                  for key in batch.shared if isinstance(key, tuple) and key[0] == "decode_pieces"}
        meta = ops.AttentionMeta(batch.array("cu_q"), batch.array("pos0"), batch.array("kv_len"), batch.block_table(group),
                                 batch.array("token_entry"), batch.array("positions"), batch.S, batch.T, batch.max_blocks[group],
                                 batch.max_kv_len, batch.max_q_len, tiles, group_size, fixed_shape=batch.fixed_shape,
                                 big_rows=big_rows or 128, pieces=pieces)
        batch.shared[note] = meta
    return meta


class PagedAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: Optional[PositionEncoding], qk_norm_eps: Optional[float] = None,
                 window: Optional[int] = None, scale: Optional[float] = None, fold_rows: Optional[int] = None):
        """``fold_rows``: most rows of a step whose products here run with the norms and the residual sum folded in
        (None: ``ops.default_fold_rows`` of this part's matrices)."""
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        self.position = position
        self.qk_norm_eps = qk_norm_eps
        self.window = window
        self.scale = 1.0 / math.sqrt(head_dim) if scale is None else float(scale)
        self.fold_rows = fold_rows
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
        # the three matrices leave the caller's dictionary here, so that they are freed once they are fused: binding a
        # model never holds the separate matrices, the fused one and its tiled copy of all layers at once
        q, k, v = (weights.pop(prefix + ".%s_proj.weight" % n) for n in "qkv")
        if not (q.dtype == k.dtype == v.dtype):
            q, k, v = q.float(), k.float(), v.float()
        # one product for q, k and v: rows [q heads | k heads | v heads]
        self.w_qkv = torch.cat([q, k, v], dim=0).contiguous()
        del q, k, v
        self.w_qkv, self.w_qkv_tiled = ops.weight_forms(self.w_qkv)
        self.w_o, self.w_o_tiled = ops.weight_forms(weights.pop(prefix + ".o_proj.weight"))
        if self.qk_norm_eps is not None:
            self.q_norm, self.k_norm = weights[prefix + ".q_norm.weight"], weights[prefix + ".k_norm.weight"]
            if self.q_norm.dtype != self.k_norm.dtype:
                self.q_norm, self.k_norm = self.q_norm.float(), self.k_norm.float()

    # ---- cache -----------------------------------------------------------
    def cache_spec(self):
        return PagedKV(self.num_kv_heads, self.head_dim, self.window)

    def plan(self, batch) -> None:
        # a step of single tokens that the fused kernel will take has its keys cut into even pieces on the host
        pieces = ops.decode_pieces_ok(batch.S, batch.T, batch.act_dtype, self.num_kv_heads, self.head_dim) and self._rotated_whole()
        plan_attention_tiles(batch, self.num_heads // self.num_kv_heads, self._big_rows(batch, batch.page_size), key_parts=not pieces)
        if pieces:
            plan_decode_pieces(batch, self.num_kv_heads, int(self.window or 0), self.head_dim)

    def plan_arrays(self, entries):
        G = self.num_heads // self.num_kv_heads
        out = {"tile_entry_small_%d" % G: entries, "tile_row0_small_%d" % G: entries}
        if ops.decode_pieces_ok(entries, entries, torch.bfloat16, self.num_kv_heads, self.head_dim):
            out["decode_pieces_%d_%d_%d" % (self.num_kv_heads, int(self.window or 0), self.head_dim)] = \
                key_pieces.decode_pieces_capacity(entries, self.num_kv_heads) * key_pieces.PIECE_RECORD
        return out

    def _rotated_whole(self) -> bool:
        """The head is rotated whole or not at all, and the group is one tile: what the fused kernel takes."""
        rot = self.position.rotary() if self.position is not None else None
        return (rot is None or rot[2] in (0, self.head_dim)) and self.num_heads // self.num_kv_heads <= 16

    def _big_rows(self, batch, page_size: int) -> int:
        """Rows of the tiles for this step's entries with many rows; 0 if the prefill kernel does not take this head
        size or page."""
        if not ops.prefill_attention_ok(self.head_dim, page_size):
            return 0
        note = ("attention_big_rows", self.num_heads, self.num_kv_heads, self.head_dim)
        if note not in batch.shared:
            rows = batch.lens.astype(np.int64) * (self.num_heads // self.num_kv_heads)
            batch.shared[note] = ops.prefill_tile_rows(self.head_dim, rows[rows >= BIG_MIN_ROWS], self.num_kv_heads)
        return batch.shared[note]

    # ---- step ------------------------------------------------------------
    def capturable(self, batch):
        # everything a step changes is read from the batch's device arrays; the one launch shape that follows the
        # requests' lengths, the number of key parts, is in the graph's key (plan_attention_tiles)
        return self.position is None or self.position.capturable(batch)

    def can_fold(self, batch):
        # (beyond 64 rows the products take their inputs in operand order only: the attention must hand its result over so)
        if batch.T > 64 and not ops.attention_hands_over_operand_rows(batch.act_dtype, self.num_heads, self.head_dim, batch.page_size):
            return False
        return ops.fused_decode_ok(batch.T, batch.act_dtype, self.w_qkv_tiled, self.w_o_tiled, max_rows=self.fold_rows)

    def _attend(self, x, batch, cache, store, for_product=False):
        nq, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
        if isinstance(x, ops.ScaledInput):
            qkv = ops.decode_linear(x, self.w_qkv_tiled)
        else:
            qkv = ops.linear(x, self.w_qkv, tiled=self.w_qkv_tiled)
        rot = self.position.rotary() if self.position is not None else None
        cos, sin, rdim = rot if rot is not None else (None, None, 0)
        eps = self.qk_norm_eps if self.qk_norm_eps is not None else 0.0
        meta = attention_meta(batch, cache.group, nq // nkv, self._big_rows(batch, cache.page_size))
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
