"""The flat batch of one step: which tokens run, where they sit in their
requests, where their keys and values go, which rows give logits.

The reference builds the same arrays in its scheduler and runner
(src/engine/scheduler.cpp:52-119, src/engine/model_runner.cpp:61-94):
prompt_tokens, positions, slot_mapping, seq_idx_mapping, context_lens,
cu_seqlens, block_tables.  Here they are right for any mix of portions and
single tokens, exist once per cache group, and travel to the device as one
packed int32 buffer.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from ..cache.manager import CacheManager, RequestCache
from ..kernels.ops import AttentionMeta

ROWS_PER_TILE = 16   # rows of (token, head-in-group) pairs that one attention wave works on


class StepEntry:
    """One request's part of a step: its next tokens and the places whose logits are wanted."""

    def __init__(self, cache: RequestCache, tokens: Sequence[int], want: Sequence[int] = ()):
        self.cache = cache
        self.tokens = list(tokens)
        self.want = list(want)
        if not self.tokens:
            raise ValueError("a step entry needs at least one token")
        for w in self.want:
            if not (0 <= w < len(self.tokens)):
                raise ValueError("wanted place %d is outside the entry's %d tokens" % (w, len(self.tokens)))


class StepBatch:
    def __init__(self, entries: Sequence[StepEntry], manager: CacheManager, act_dtype: torch.dtype, device,
                 vocab_size: Optional[int] = None, min_max_blocks: int = 0):
        self.entries = list(entries)
        self.act_dtype = act_dtype
        self.device = torch.device(device)
        self.S = len(self.entries)
        self._arrays: Dict[str, List[int]] = {}
        self._dev: Dict[str, torch.Tensor] = {}
        self._tiles: Dict[int, int] = {}
        seen = set()
        token_ids, positions, token_entry, cu_q, pos0, kv_len, slot_ids, fresh, rows = [], [], [], [0], [], [], [], [], []
        for s, e in enumerate(self.entries):
            rc = e.cache
            if id(rc) in seen:
                raise ValueError("request %r appears twice in one step" % (rc.request_id,))
            seen.add(id(rc))
            if not rc.live:
                raise ValueError("request %r holds no cache any more" % (rc.request_id,))
            n = len(e.tokens)
            if n > rc.reserved:
                raise ValueError("request %r runs %d tokens but pages are reserved for %d" % (rc.request_id, n, rc.reserved))
            if vocab_size is not None:
                for t in e.tokens:
                    if not (0 <= t < vocab_size):
                        raise ValueError("token id %r of request %r is outside the vocabulary of %d" % (t, rc.request_id, vocab_size))
            base = len(token_ids)
            token_ids += e.tokens
            positions += range(rc.num_tokens, rc.num_tokens + n)
            token_entry += [s] * n
            cu_q.append(base + n)
            pos0.append(rc.num_tokens)
            kv_len.append(rc.num_tokens + n)
            slot_ids.append(rc.slot)
            fresh.append(1 if rc.fresh else 0)
            rows += [base + w for w in e.want]
        self.T, self.R = len(token_ids), len(rows)
        self.max_q_len = max((len(e.tokens) for e in self.entries), default=0)
        self.max_kv_len = max(kv_len, default=0)
        self.host = dict(token_ids=token_ids, positions=positions, token_entry=token_entry, cu_q=cu_q, pos0=pos0,
                         kv_len=kv_len, slot_ids=slot_ids, fresh=fresh, logit_rows=rows)
        for k, v in self.host.items():
            self._arrays[k] = v
        # per page group: block tables padded with -1, and the slot of every token of the step
        self.max_blocks = []
        for g in manager.page_groups:
            width = max([len(e.cache.tables[g.index]) for e in self.entries] + [min_max_blocks, 1])
            table, slots = [], []
            for e in self.entries:
                t = e.cache.tables[g.index]
                table += t + [-1] * (width - len(t))
                for p in range(e.cache.num_tokens, e.cache.num_tokens + len(e.tokens)):
                    slots.append(manager.slot_of_token(e.cache, g.index, p))
            self.max_blocks.append(width)
            self._arrays["block_table_%d" % g.index] = table
            self._arrays["slot_mapping_%d" % g.index] = slots
        self.num_groups = len(manager.page_groups)

    # ---- additions by parts, before upload ---------------------------------
    def add_array(self, name: str, values: List[int]) -> None:
        if self._dev:
            raise RuntimeError("the batch is already on the device")
        self._arrays[name] = list(values)

    def add_attention_tiles(self, group_size: int) -> None:
        """16-row tiles over each entry's rows (token-major, head-in-group minor) for a
        query-head group of ``group_size``."""
        if group_size in self._tiles:
            return
        tile_entry, tile_row0 = [], []
        for s, e in enumerate(self.entries):
            nrows = len(e.tokens) * group_size
            for r0 in range(0, nrows, ROWS_PER_TILE):
                tile_entry.append(s)
                tile_row0.append(r0)
        self._tiles[group_size] = len(tile_entry)
        self.add_array("tile_entry_%d" % group_size, tile_entry)
        self.add_array("tile_row0_%d" % group_size, tile_row0)

    # ---- to the device -------------------------------------------------------
    def layout(self):
        """name -> (offset, length) in the packed buffer; every array starts at a multiple of 4 ints."""
        off, out = 0, {}
        for name, vals in self._arrays.items():
            out[name] = (off, len(vals))
            off += (len(vals) + 3) // 4 * 4
        return out, max(off, 4)

    def upload(self, device_buffer: Optional[torch.Tensor] = None, pinned: Optional[torch.Tensor] = None) -> None:
        layout, total = self.layout()
        flat = [0] * total
        for name, (off, n) in layout.items():
            flat[off:off + n] = self._arrays[name]
        host = torch.tensor(flat, dtype=torch.int32)
        if device_buffer is None:
            dev = host.to(self.device)
        else:
            if device_buffer.numel() < total:
                raise ValueError("the step's metadata (%d ints) exceeds the device buffer (%d)" % (total, device_buffer.numel()))
            dev = device_buffer[:total]
            if pinned is not None:
                pinned[:total].copy_(host)
                dev.copy_(pinned[:total], non_blocking=True)
            else:
                dev.copy_(host)
        for name, (off, n) in layout.items():
            self._dev[name] = dev[off:off + n]

    def __getattr__(self, name):
        dev = self.__dict__.get("_dev", {})
        if name in dev:
            return dev[name]
        raise AttributeError(name)

    def array(self, name: str) -> torch.Tensor:
        return self._dev[name]

    def slot_mapping(self, group: int) -> torch.Tensor:
        return self._dev["slot_mapping_%d" % group]

    def block_table(self, group: int) -> torch.Tensor:
        return self._dev["block_table_%d" % group].view(self.S, self.max_blocks[group])

    def attention_meta(self, group: int, group_size: int) -> AttentionMeta:
        tiles, n_tiles = None, 0
        if group_size in self._tiles:
            tiles = (self._dev["tile_entry_%d" % group_size], self._dev["tile_row0_%d" % group_size])
            n_tiles = self._tiles[group_size]
        return AttentionMeta(self._dev["cu_q"], self._dev["pos0"], self._dev["kv_len"], self.block_table(group),
                             self._dev["token_entry"], self._dev["positions"], self.S, self.T, self.max_blocks[group],
                             self.max_kv_len, self.max_q_len, tiles, group_size, n_tiles)
