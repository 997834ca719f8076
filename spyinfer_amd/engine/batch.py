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

import numpy as np
import torch

from ..cache.manager import CacheManager, RequestCache


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


def _table_row(rc: RequestCache, group: int) -> np.ndarray:
    """The request's block table of a group as an int32 array, cached until the table changes."""
    cache = rc.__dict__.setdefault("_rows", {})
    hit = cache.get(group)
    if hit is None or hit[0] != rc.versions[group]:
        hit = (rc.versions[group], np.asarray(rc.tables[group], dtype=np.int32))
        cache[group] = hit
    return hit[1]


class StepBatch:
    def __init__(self, entries: Sequence[StepEntry], manager: CacheManager, act_dtype: torch.dtype, device,
                 vocab_size: Optional[int] = None, fixed_max_blocks: int = 0):
        """``fixed_max_blocks`` > 0: block tables have exactly that width (and attention splits its
        keys into a number of parts that does not depend on the lengths), so that steps with the
        same numbers of entries, tokens and wanted rows have one memory layout: what a captured
        graph needs."""
        self.entries = list(entries)
        self.act_dtype = act_dtype
        self.device = torch.device(device)
        self.S = S = len(self.entries)
        self.fixed_shape = fixed_max_blocks > 0
        self._arrays: Dict[str, np.ndarray] = {}
        self._dev: Dict[str, torch.Tensor] = {}
        #: host-side notes of the parts for this step (what one layer planned, the next need not plan again)
        self.shared: Dict[object, object] = {}
        self._graph_extra: Dict[str, object] = {}
        seen = set()
        lens = np.empty(S, dtype=np.int32)
        pos0 = np.empty(S, dtype=np.int32)
        slot_ids = np.empty(S, dtype=np.int32)
        fresh = np.empty(S, dtype=np.int32)
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
            lens[s], pos0[s], slot_ids[s], fresh[s] = n, rc.num_tokens, rc.slot, 1 if rc.fresh else 0
        cu_q = np.zeros(S + 1, dtype=np.int32)
        np.cumsum(lens, out=cu_q[1:])
        self.T = T = int(cu_q[-1])
        token_ids = np.fromiter((t for e in self.entries for t in e.tokens), dtype=np.int64, count=T)
        if vocab_size is not None and T and (token_ids.min() < 0 or token_ids.max() >= vocab_size):
            bad = token_ids[(token_ids < 0) | (token_ids >= vocab_size)][0]
            raise ValueError("token id %d is outside the vocabulary of %d" % (int(bad), vocab_size))
        token_entry = np.repeat(np.arange(S, dtype=np.int32), lens)
        positions = (np.arange(T, dtype=np.int32) - cu_q[:-1][token_entry] + pos0[token_entry]).astype(np.int32)
        rows = np.fromiter((int(cu_q[s]) + w for s, e in enumerate(self.entries) for w in e.want), dtype=np.int32)
        self.R = int(rows.shape[0])
        #: every token's logits are wanted, in order: the output head may take the step's rows as they are
        self.all_rows_wanted = self.R == T and bool((rows == np.arange(T, dtype=np.int32)).all())
        kv_len = pos0 + lens
        self.max_q_len = int(lens.max()) if S else 0
        self.max_kv_len = int(kv_len.max()) if S else 0
        self.lens = lens
        for name, arr in (("token_ids", token_ids.astype(np.int32)), ("positions", positions), ("token_entry", token_entry),
                          ("cu_q", cu_q), ("pos0", pos0), ("kv_len", kv_len.astype(np.int32)), ("slot_ids", slot_ids),
                          ("fresh", fresh), ("logit_rows", rows)):
            self._arrays[name] = arr
        # per page group: block tables padded with -1, and the slot of every token of the step
        self.max_blocks = []
        for g in manager.page_groups:
            tables = [_table_row(e.cache, g.index) for e in self.entries]
            width = max([len(t) for t in tables] + [1])
            if fixed_max_blocks:
                if width > fixed_max_blocks:
                    raise ValueError("a block table has %d pages, the fixed width is %d" % (width, fixed_max_blocks))
                width = fixed_max_blocks
            table = np.full((S, width), -1, dtype=np.int32)
            for s, t in enumerate(tables):
                table[s, :len(t)] = t
            P = g.page_size
            pages = table[token_entry, positions // P] if T else np.empty(0, dtype=np.int32)
            if T and pages.min() < 0:
                t = int(np.argmin(pages))
                raise ValueError("position %d of request %r has no page in group %d"
                                 % (int(positions[t]), self.entries[int(token_entry[t])].cache.request_id, g.index))
            self.max_blocks.append(width)
            self._arrays["block_table_%d" % g.index] = table.reshape(-1)
            self._arrays["slot_mapping_%d" % g.index] = (pages * P + positions % P).astype(np.int32)
        self.num_groups = len(manager.page_groups)
        self.page_size = manager.page_size
        self._graph_key = None

    # ---- additions by parts, before upload ---------------------------------
    def add_array(self, name: str, values) -> None:
        if self._dev:
            raise RuntimeError("the batch is already on the device")
        self._arrays[name] = np.asarray(values, dtype=np.int32).reshape(-1)

    def has_array(self, name: str) -> bool:
        return name in self._arrays

    def add_graph_key(self, name: str, value) -> None:
        """A part's ``plan`` says what, beside the arrays' lengths, the shape of its launches takes from this step
        (a number of blocks that follows the requests' lengths, say): a captured graph is replayed only for steps
        with the same values."""
        self._graph_extra[name] = value
        self._graph_key = None

    # ---- to the device -------------------------------------------------------
    def layout(self):
        """name -> (offset, length) in the packed buffer; every array starts at a multiple of 4 ints."""
        off, out = 0, {}
        for name, vals in self._arrays.items():
            out[name] = (off, int(vals.shape[0]))
            off += (int(vals.shape[0]) + 3) // 4 * 4
        return out, max(off, 4)

    def layout_key(self):
        return tuple((name, int(v.shape[0])) for name, v in self._arrays.items())

    def graph_key(self):
        """What a captured graph of this step depends on beside the arrays' contents."""
        if self._graph_key is None:
            self._graph_key = (self.layout_key(), self.all_rows_wanted, tuple(sorted(self._graph_extra.items())))
        return self._graph_key

    def host_array(self, name: str) -> np.ndarray:
        return self._arrays[name]

    def pack_into(self, host: torch.Tensor):
        """Write all arrays into the int32 host tensor; returns (layout, total ints)."""
        layout, total = self.layout()
        if host.numel() < total:
            raise ValueError("the step's metadata (%d ints) exceeds the buffer (%d)" % (total, host.numel()))
        flat = host.numpy()
        for name, (off, n) in layout.items():
            flat[off:off + n] = self._arrays[name]
        return layout, total

    def bind_device(self, dev: torch.Tensor, layout) -> None:
        for name, (off, n) in layout.items():
            self._dev[name] = dev[off:off + n]

    def upload(self) -> None:
        """Simple path: a fresh host tensor, one copy to the device."""
        _layout, total = self.layout()
        host = torch.empty(total, dtype=torch.int32)
        layout, total = self.pack_into(host)
        self.bind_device(host.to(self.device), layout)

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
