"""Cache manager: pages with a block table per request and per group of layers,
and slots for per-request state of fixed size.

Host-side bookkeeping only; the device tensors that the page and slot numbers
index are made by ``cache.storage``.  Compared with the reference
(src/engine/block_manager.cpp, src/engine/scheduler.cpp:24-35, 74-87,
src/engine/llm_engine.cpp:149-157): pages are taken for exactly the tokens of
the coming step, are given back as soon as a request ends or a window has
passed them, and running out of pages is reported, never thrown mid-step.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional, Sequence

from .pages import OutOfPages, PagePool
from .spec import CacheKind


class OutOfSlots(RuntimeError):
    pass


class SlotPool:
    """Slots 0..N-1 for per-request state; lowest free slot first."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._held = [False] * num_slots

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise OutOfSlots("no free state slot (pool of %d)" % self.num_slots)
        s = self._free.pop()
        self._held[s] = True
        return s

    def free(self, slot: int) -> None:
        if not (0 <= slot < self.num_slots) or not self._held[slot]:
            raise ValueError("slot %r is freed but not held" % (slot,))
        self._held[slot] = False
        self._free.append(slot)

    def held(self) -> List[int]:
        return [s for s, h in enumerate(self._held) if h]


@dataclasses.dataclass
class PageGroup:
    """Layer caches with one need: they share page numbers and block tables."""

    index: int
    spec: CacheKind
    cache_ids: List[int]
    page_size: int
    pool: PagePool

    def first_needed_page(self, num_tokens: int) -> int:
        """Logical page below which nothing is read once ``num_tokens`` are cached:
        the next query sits at position >= num_tokens and reads keys > position - window."""
        if self.spec.window is None:
            return 0
        return max(0, num_tokens - self.spec.window + 1) // self.page_size


@dataclasses.dataclass
class StateGroup:
    index: int
    spec: CacheKind
    cache_ids: List[int]


class RequestCache:
    """What one live request holds: a slot, and per page group its block table
    (logical page -> physical page, -1 where nothing is held)."""

    def __init__(self, request_id, slot: int, num_groups: int):
        self.request_id = request_id
        self.slot = slot
        self.num_tokens = 0          # tokens whose keys/values/state are in the cache
        self.reserved = 0            # tokens beyond num_tokens that have pages
        self.tables: List[List[int]] = [[] for _ in range(num_groups)]
        self.fresh = True            # no step has run yet: state slots must be reset
        self.live = True
        self.versions = [0] * num_groups   # bumped whenever a table changes (lets callers cache copies)

    def pages_held(self, group: int) -> List[int]:
        return [p for p in self.tables[group] if p >= 0]


def window_pages(window: int, page_size: int, step_tokens: int = 1) -> int:
    """Most pages that one request holds in a group whose layers read the last ``window`` keys only, while it runs
    ``step_tokens`` tokens in a step: the keys that the step's first query reads and the step's own, which begin and
    end anywhere in a page."""
    return -(-(window - 1 + step_tokens) // page_size) + 1


class CacheManager:
    def __init__(self, cache_specs: Sequence[Optional[object]], page_size: int, num_pages: int, max_num_seqs: int,
                 max_step_tokens: Optional[int] = None):
        """``cache_specs[i]`` is the need of layer cache ``i`` (None = nothing).
        Every page group gets a pool of ``num_pages`` pages of ``page_size`` tokens; a group with a window gets no
        more than ``max_num_seqs`` requests can hold at once when none runs more than ``max_step_tokens`` tokens in a
        step (if that is given)."""
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        self.page_size = page_size
        self.max_step_tokens = max_step_tokens
        self.page_groups: List[PageGroup] = []
        self.state_groups: List[StateGroup] = []
        self.location: Dict[int, tuple] = {}   # cache id -> ("paged"|"state", group index, index in group)
        for cid, spec in enumerate(cache_specs):
            if spec is None:
                continue
            if not isinstance(spec, CacheKind):
                raise TypeError("cache need %r of layer cache %d is no CacheKind" % (spec, cid))
            # equal kinds share a group: one pool of pages (or the slots) and one block table per request
            if spec.paged:
                grp = next((g for g in self.page_groups if g.spec == spec), None)
                if grp is None:
                    grp = PageGroup(len(self.page_groups), spec, [], page_size,
                                    PagePool(self.pages_of_group(spec, page_size, num_pages, max_num_seqs, max_step_tokens)))
                    self.page_groups.append(grp)
            else:
                grp = next((g for g in self.state_groups if g.spec == spec), None)
                if grp is None:
                    grp = StateGroup(len(self.state_groups), spec, [])
                    self.state_groups.append(grp)
            self.location[cid] = ("paged" if spec.paged else "state", grp.index, len(grp.cache_ids))
            grp.cache_ids.append(cid)
        self.slots = SlotPool(max_num_seqs)
        self.requests: Dict[object, RequestCache] = {}

    @staticmethod
    def pages_of_group(spec: CacheKind, page_size: int, num_pages: int, max_num_seqs: int, max_step_tokens: Optional[int]) -> int:
        """Pages in the pool of a group of kind ``spec`` when ``num_pages`` are offered to every group."""
        if spec.window is None or max_step_tokens is None:
            return num_pages
        return max(1, min(num_pages, max_num_seqs * window_pages(spec.window, page_size, max_step_tokens)))

    # ---- admission -------------------------------------------------------
    def can_admit(self) -> bool:
        return self.slots.num_free > 0

    def admit(self, request_id) -> RequestCache:
        if request_id in self.requests:
            raise ValueError("request %r is already live" % (request_id,))
        rc = RequestCache(request_id, self.slots.allocate(), len(self.page_groups))
        self.requests[request_id] = rc
        return rc

    # ---- pages -----------------------------------------------------------
    def pages_needed(self, rc: RequestCache, n_tokens: int) -> List[int]:
        """New pages per group so that positions up to num_tokens + n_tokens have pages."""
        end = rc.num_tokens + n_tokens
        need = []
        for g in self.page_groups:
            total = -(-end // g.page_size)
            need.append(max(0, total - len(rc.tables[g.index])))
        return need

    def can_reserve(self, rc: RequestCache, n_tokens: int) -> bool:
        return all(n <= g.pool.num_free for n, g in zip(self.pages_needed(rc, n_tokens), self.page_groups))

    def reserve(self, rc: RequestCache, n_tokens: int) -> None:
        """Take pages for the next ``n_tokens`` tokens of ``rc`` in every group, or none at all."""
        need = self.pages_needed(rc, n_tokens)
        for n, g in zip(need, self.page_groups):
            if n > g.pool.num_free:
                raise OutOfPages("request %r needs %d page(s) of group %d, %d free"
                                 % (rc.request_id, n, g.index, g.pool.num_free))
        for n, g in zip(need, self.page_groups):
            for _ in range(n):
                rc.tables[g.index].append(g.pool.allocate())
            if n:
                rc.versions[g.index] += 1
        rc.reserved = max(rc.reserved, n_tokens)

    def commit(self, rc: RequestCache, n_tokens: int) -> None:
        """``n_tokens`` more tokens are now cached; give back pages that a window has passed."""
        if n_tokens > rc.reserved:
            raise ValueError("commit of %d tokens, only %d reserved" % (n_tokens, rc.reserved))
        rc.num_tokens += n_tokens
        rc.reserved -= n_tokens
        rc.fresh = False
        for g in self.page_groups:
            table = rc.tables[g.index]
            for i in range(min(g.first_needed_page(rc.num_tokens), len(table))):
                if table[i] >= 0:
                    g.pool.free(table[i])
                    table[i] = -1
                    rc.versions[g.index] += 1

    def rewind(self, rc: RequestCache, num_tokens: int) -> bool:
        """Count only the first ``num_tokens`` tokens as cached again, so that the later ones are computed anew into
        the pages they already have (a further turn of a request whose last token was stored by a step run ahead
        needs that token's logits once more).  False, and nothing changed, if that cannot be done: a state of fixed
        size has taken the tokens in for good, or a window has given back a page that a query at ``num_tokens`` reads."""
        if not (0 <= num_tokens <= rc.num_tokens):
            raise ValueError("rewind to %d tokens, %d are cached" % (num_tokens, rc.num_tokens))
        if num_tokens == rc.num_tokens:
            return True
        if self.state_groups:
            return False
        for g in self.page_groups:
            table = rc.tables[g.index]
            last = -(-rc.num_tokens // g.page_size)
            if any(table[i] < 0 for i in range(g.first_needed_page(num_tokens), last)):
                return False
        rc.reserved += rc.num_tokens - num_tokens
        rc.num_tokens = num_tokens
        return True

    def release(self, rc: RequestCache) -> None:
        """The request ends (or is preempted): everything it holds goes back."""
        if not rc.live:
            raise ValueError("request %r was already released" % (rc.request_id,))
        for g in self.page_groups:
            # last page first, so that the LIFO pool hands them out again in ascending logical order
            for p in reversed(rc.tables[g.index]):
                if p >= 0:
                    g.pool.free(p)
            rc.tables[g.index] = []
            rc.versions[g.index] += 1
        self.slots.free(rc.slot)
        rc.live = False
        rc.num_tokens = 0
        rc.reserved = 0
        del self.requests[rc.request_id]

    # ---- queries ---------------------------------------------------------
    def slot_of_token(self, rc: RequestCache, group: int, position: int) -> int:
        g = self.page_groups[group]
        page = rc.tables[group][position // g.page_size]
        if page < 0:
            raise ValueError("position %d of request %r has no page in group %d" % (position, rc.request_id, group))
        return page * g.page_size + position % g.page_size

    def num_free_pages(self) -> List[int]:
        return [g.pool.num_free for g in self.page_groups]

    def max_tokens_per_request(self) -> int:
        """Most tokens one request alone can reach (the smallest group decides).  A group with a window gives back the
        pages that the window has passed, so with room for the window and one token more it sets no limit."""
        limit = 1 << 62
        for g in self.page_groups:
            if g.spec.window is not None and g.pool.num_pages >= window_pages(g.spec.window, g.page_size):
                continue
            limit = min(limit, g.pool.num_pages * g.page_size)
        return limit

    def max_reservable(self, rc: RequestCache, n_tokens: int) -> int:
        """The most tokens up to ``n_tokens`` for which ``rc`` could get pages now."""
        for g in self.page_groups:
            room = (len(rc.tables[g.index]) + g.pool.num_free) * g.page_size - rc.num_tokens
            n_tokens = min(n_tokens, room)
        return max(0, n_tokens)

    def check(self) -> None:
        """Invariant: every page is either free or in exactly one live table; same for slots."""
        for g in self.page_groups:
            seen = {}
            for rc in self.requests.values():
                for p in rc.pages_held(g.index):
                    if p in seen:
                        raise AssertionError("page %d of group %d is held by %r and %r" % (p, g.index, seen[p], rc.request_id))
                    seen[p] = rc.request_id
            if sorted(seen) != g.pool.held():
                raise AssertionError("group %d: held pages %r, tables hold %r" % (g.index, g.pool.held(), sorted(seen)))
            if len(seen) + g.pool.num_free != g.pool.num_pages:
                raise AssertionError("group %d: a page is lost" % g.index)
        slots = sorted(rc.slot for rc in self.requests.values())
        if slots != self.slots.held() or len(set(slots)) != len(slots):
            raise AssertionError("slots held %r, requests hold %r" % (self.slots.held(), slots))
