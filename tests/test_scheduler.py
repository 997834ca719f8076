"""The scheduler's decisions (CPU): admission order, token budget, portions, the cap on running
requests, finishing, and what happens when pages run out."""
import pytest

from spyinfer_amd.cache import CacheManager, PagedKV
from spyinfer_amd.engine.scheduler import Scheduler
from spyinfer_amd.engine.sequence import Sequence, SequenceStatus
from spyinfer_amd.sampling import SamplingParams


def make(num_pages=16, page=4, budget=64, max_seqs=4, max_len=64):
    m = CacheManager([PagedKV(1, 8)], page, num_pages, max_seqs)
    return m, Scheduler(m, budget, max_seqs, max_len)


def run_step(m, sched, next_token=7):
    """What the engine does around a step, without a model: commit, then append a token where one is sampled."""
    out = sched.schedule()
    for sc in out:
        m.commit(sc.seq.cache, sc.num_tokens)
    for sc in out:
        if sc.samples:
            sc.seq.tokens.append(next_token)
    m.check()
    return out


def seq(i, n, **kw):
    return Sequence(i, list(range(1, n + 1)), SamplingParams(**kw))


def test_fifo_admission_and_budget_cut_prompts():
    m, s = make(budget=10)
    a, b = seq(0, 7), seq(1, 9)
    s.add_sequence(a); s.add_sequence(b)
    out = run_step(m, s)
    # a whole (7), then b's first portion under what is left of the budget (3)
    assert [(x.seq.id, x.num_tokens, x.samples) for x in out] == [(0, 7, True), (1, 3, False)]
    out = run_step(m, s)
    # decoding requests first (1 token), then the rest of b's prompt
    assert [(x.seq.id, x.num_tokens, x.samples) for x in out] == [(0, 1, True), (1, 6, True)]
    out = run_step(m, s)
    assert [(x.seq.id, x.num_tokens) for x in out] == [(0, 1), (1, 1)]
    assert sum(x.num_tokens for x in out) <= 10


def test_cap_on_running_requests_and_slots():
    m, s = make(max_seqs=2, budget=100)
    for i in range(3):
        s.add_sequence(seq(i, 3))
    out = run_step(m, s)
    assert [x.seq.id for x in out] == [0, 1] and len(s.waiting) == 1
    s.finish(out[0].seq, "max_new_tokens")
    out = run_step(m, s)
    assert sorted(x.seq.id for x in out) == [1, 2]


def test_head_of_line_waits_for_pages():
    m, s = make(num_pages=4, page=4, budget=100, max_len=16)      # 16 tokens in all
    a, b, c = seq(0, 10), seq(1, 9), seq(2, 2)
    for x in (a, b, c):
        s.add_sequence(x)
    out = run_step(m, s)
    # a takes 3 pages; b needs 3: it does not fit, and c behind it waits too (arrival order is kept)
    assert [x.seq.id for x in out] == [0] and [x.id for x in s.waiting] == [1, 2]
    s.finish(a, "eos")
    assert m.num_free_pages() == [4]
    assert [x.seq.id for x in run_step(m, s)] == [1, 2]


def test_preemption_when_pages_run_out():
    m, s = make(num_pages=4, page=4, budget=100, max_len=16)
    a, b = seq(0, 7), seq(1, 6)
    s.add_sequence(a); s.add_sequence(b)
    run_step(m, s)                                     # a: 2 pages (7 -> 8 tokens fit), b: 2 pages (6 -> 7, 8)
    run_step(m, s)                                     # a has 8 cached+1 pending: needs a 3rd page next
    out = run_step(m, s)
    # no page is free for a's 9th token: the request admitted last (b) is preempted and keeps its tokens
    assert [x.seq.id for x in out] == [0]
    assert b.status is SequenceStatus.WAITING and b.cache is None and s.waiting[0] is b and b.num_preemptions == 1
    assert len(b.tokens) == 6 + 2 and s.num_preemptions == 1
    # when a ends, b is admitted again and recomputes everything it has, then samples
    s.finish(a, "eos")
    out = run_step(m, s)
    assert [(x.seq.id, x.num_tokens, x.samples) for x in out] == [(1, 8, True)]


def test_every_request_finishes_under_pressure():
    m, s = make(num_pages=6, page=4, budget=8, max_seqs=3, max_len=24)
    seqs = [seq(i, n, max_new_tokens=6) for i, n in enumerate([5, 11, 3, 9, 2, 7])]
    for x in seqs:
        s.add_sequence(x)
    steps = 0
    while s.has_unfinished():
        out = run_step(m, s)
        assert out and sum(x.num_tokens for x in out) <= 8 and len(s.running) <= 3
        for sc in out:
            if sc.samples and sc.seq.num_generated >= 6:
                s.finish(sc.seq, "max_new_tokens")
        steps += 1
        assert steps < 500
    assert all(x.status is SequenceStatus.FINISHED and x.num_generated == 6 for x in seqs)
    assert m.num_free_pages() == [6] and m.slots.num_free == 3


def test_requests_that_can_never_fit_are_refused():
    m, s = make(num_pages=2, page=4, max_len=64)
    with pytest.raises(ValueError, match="pool"):
        s.add_sequence(seq(0, 9))
    with pytest.raises(ValueError, match="max_model_len"):
        s.add_sequence(seq(1, 64))
    with pytest.raises(ValueError):
        s.add_sequence(Sequence(2, [], SamplingParams()))
    s.add_sequence(seq(3, 4, max_new_tokens=4))
