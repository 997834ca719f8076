"""Continuous batching above the step function.

Like the reference's scheduler (src/engine/scheduler.cpp:17-122) it keeps a waiting and a
running queue, admits in arrival order while pages are free, and lets every running request
take part in every step.  Beyond it: a token budget per step (``max_num_batched_tokens``,
which the reference stores but never consults) under which prompts are cut into portions,
a cap on one request's portion per step (``prefill_chunk``, so that a long prompt does not hold up
the requests that decode beside it), a cap on running requests (``max_num_seqs``), and a decided
answer when pages run out.

One step holds, in this order:
  1. one token for every running request that is decoding;
  2. portions of running requests that still have prompt (or recomputation) left, in admission
     order, each as large as the remaining budget and ``prefill_chunk`` allow;
  3. newly admitted requests from the head of the waiting queue, while a slot, budget and pages
     for their first portion are there.  The first one that does not fit stops admission
     (arrival order is kept, as in the reference, scheduler.cpp:39-42).
When pages run out for a running request, the request admitted last is preempted: its pages
and slot are given back, it keeps all its tokens and goes to the FRONT of the waiting queue,
and recomputes them when it is admitted again.  (The reference skips the token and
desynchronises its batch, scheduler.cpp:79-86.)  A request that could never fit the pool is
refused when it is added.

A finished request may keep what it holds (``finish(..., keep=True)``), as the reference's do until
they are removed (src/engine/llm_engine.cpp:40-73, 149-157), so that a further turn computes its
new tokens only.  Unlike there, such a parked cache is the first thing taken back when a slot or
pages are short, oldest first; the further turn then recomputes its history.
"""
from __future__ import annotations

import collections
from typing import Deque, List, NamedTuple, Optional

from ..cache.manager import CacheManager
from .sequence import Sequence, SequenceStatus


class Scheduled(NamedTuple):
    seq: Sequence
    num_tokens: int        # tokens of seq.tokens[num_computed : num_computed + num_tokens] run in this step
    samples: bool          # the portion reaches the request's last known token: a new token is sampled


class Scheduler:
    def __init__(self, manager: CacheManager, max_num_batched_tokens: int, max_num_seqs: int, max_model_len: int,
                 prefill_chunk: Optional[int] = None):
        self.manager = manager
        self.max_num_batched_tokens = max_num_batched_tokens
        #: most tokens of one request in one step (None: the budget alone decides)
        self.prefill_chunk = prefill_chunk if prefill_chunk else max_num_batched_tokens
        self.parked: List[Sequence] = []       # finished requests that still hold their cache, oldest first
        self.max_num_seqs = max_num_seqs
        self.max_model_len = max_model_len
        self.waiting: Deque[Sequence] = collections.deque()
        self.running: List[Sequence] = []
        self.num_preemptions = 0
        self._admitted = 0

    # ---- queues ----------------------------------------------------------
    def check_admissible(self, num_tokens: int, max_new_tokens: Optional[int]) -> None:
        """Raises ValueError if a request of ``num_tokens`` known tokens could never run here."""
        if num_tokens == 0:
            raise ValueError("a request needs at least one prompt token")
        if num_tokens >= self.max_model_len:
            raise ValueError("the prompt has %d tokens; max_model_len is %d" % (num_tokens, self.max_model_len))
        limit = min(self.max_model_len, num_tokens + (max_new_tokens or self.max_model_len))
        if limit > self.manager.max_tokens_per_request():
            raise ValueError("the request may reach %d tokens; the cache pool holds %d" % (limit, self.manager.max_tokens_per_request()))

    def add_sequence(self, seq: Sequence) -> None:
        self.check_admissible(len(seq), seq.params.max_new_tokens)
        seq.status = SequenceStatus.WAITING
        self.waiting.append(seq)

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    def finish(self, seq: Sequence, reason: str, keep: bool = False) -> None:
        """The request ends: what it holds goes back to the pools at once, unless ``keep`` parks it for a
        further turn (it then goes back when pages or slots are short, or when the request is removed)."""
        seq.status = SequenceStatus.FINISHED
        seq.finish_reason = reason
        if seq in self.running:
            self.running.remove(seq)
        if seq.cache is not None and seq.cache.live:
            if keep:
                if seq not in self.parked:
                    self.parked.append(seq)
                return
            self._unpark(seq)
            self.manager.release(seq.cache)
        seq.cache = None

    def abort(self, seq: Sequence) -> None:
        if seq in self.waiting:
            self.waiting.remove(seq)
        self._unpark(seq)
        self.finish(seq, "removed")

    def _unpark(self, seq: Sequence) -> None:
        if seq in self.parked:
            self.parked.remove(seq)

    def _reclaim_parked(self, spare: Optional[Sequence] = None) -> bool:
        """Take back the oldest parked cache (not ``spare``'s); False if there is none."""
        for seq in self.parked:
            if seq is not spare:
                self.parked.remove(seq)
                self.manager.release(seq.cache)
                seq.cache = None
                return True
        return False

    def _preempt(self, seq: Sequence) -> None:
        self.running.remove(seq)
        self.manager.release(seq.cache)
        seq.cache = None
        seq.status = SequenceStatus.WAITING
        seq.num_preemptions += 1
        self.num_preemptions += 1
        self.waiting.appendleft(seq)

    # ---- one step --------------------------------------------------------
    def schedule(self) -> List[Scheduled]:
        budget = self.max_num_batched_tokens
        out: List[Scheduled] = []
        # 1 and 2: running requests, decoding ones first, each group in admission order
        order = sorted(self.running, key=lambda s: (s.is_prefill, s.admit_order))
        for seq in order:
            if seq.status is not SequenceStatus.RUNNING:
                continue                       # preempted while an earlier request was served
            if budget <= 0:
                break
            left = len(seq) - seq.num_computed
            n = min(left, budget, self.prefill_chunk)
            while not self.manager.can_reserve(seq.cache, n):
                if self._reclaim_parked():
                    continue
                victim = max(self.running, key=lambda s: s.admit_order)
                if victim is seq and len(self.running) == 1:
                    # alone, nobody to take pages from: a smaller portion (a window gives pages back as it moves on)
                    n = self.manager.max_reservable(seq.cache, n)
                    if n == 0:
                        raise RuntimeError("request %d cannot get pages although it runs alone; the pool is too small" % seq.id)
                    break
                for x in out:
                    if x.seq is victim:    # a victim scheduled earlier in this step leaves it and returns its budget
                        budget += x.num_tokens
                out = [x for x in out if x.seq is not victim]
                self._preempt(victim)
                if victim is seq:
                    break
            if seq.status is not SequenceStatus.RUNNING:
                continue
            self.manager.reserve(seq.cache, n)
            out.append(Scheduled(seq, n, n == left))
            budget -= n
        # 3: admission from the head of the waiting queue
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs:
            seq = self.waiting[0]
            kept = seq.cache is not None and seq.cache.live        # a further turn of a request whose cache is parked
            if kept and seq.cache.num_tokens >= len(seq) and not self.manager.rewind(seq.cache, len(seq) - 1):
                # The turn brings no token that is not cached yet (a step run ahead stored the last one, and the turn
                # is empty), but its first new token is sampled from the last token's logits: that token runs again.
                # Where the cache cannot step back, it is given up and the history computed anew.
                self._unpark(seq)
                self.manager.release(seq.cache)
                seq.cache, kept = None, False
            if not kept and not self.manager.can_admit() and not self._reclaim_parked():
                break
            cache = seq.cache if kept else self.manager.admit(seq.id)
            n = min(len(seq) - cache.num_tokens, budget, self.prefill_chunk)
            while not self.manager.can_reserve(cache, n) and self._reclaim_parked(spare=seq):
                pass
            if not self.manager.can_reserve(cache, n) and not self.running and not out:
                n = self.manager.max_reservable(cache, n)     # nothing runs that could end and free pages: a smaller portion
            if n == 0 or not self.manager.can_reserve(cache, n):
                if not kept:
                    self.manager.release(cache)
                break
            self._unpark(seq)
            self.waiting.popleft()
            seq.cache = cache
            seq.status = SequenceStatus.RUNNING
            seq.admit_order = self._admitted
            self._admitted += 1
            self.running.append(seq)
            self.manager.reserve(cache, n)
            out.append(Scheduled(seq, n, cache.num_tokens + n == len(seq)))
            budget -= n
        return out
