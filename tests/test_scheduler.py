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


def test_prefill_chunk_caps_one_requests_portion():
    """A long prompt beside decoding requests is cut into portions of ``prefill_chunk``: it takes ceil(200 / 32) steps,
    the budget is never exceeded, and every decoding request gets its token in every one of them."""
    m = CacheManager([PagedKV(1, 8)], 8, 64, 8)
    s = Scheduler(m, 64, 8, 512, prefill_chunk=32)
    decoders = [seq(i, 5) for i in range(3)]
    for d in decoders:
        s.add_sequence(d)
    run_step(m, s)
    long = seq(9, 200)
    s.add_sequence(long)
    steps = 0
    while long.num_generated == 0:
        out = run_step(m, s)
        steps += 1
        assert sum(x.num_tokens for x in out) <= 64
        assert [(x.seq.id, x.num_tokens, x.samples) for x in out[:3]] == [(0, 1, True), (1, 1, True), (2, 1, True)]
        mine = [x for x in out if x.seq is long]
        assert len(mine) == 1 and mine[0].num_tokens == (32 if steps < 7 else 8) and mine[0].samples == (steps == 7)
    assert steps == -(-200 // 32) == 7
    # two long prompts share a step's budget, each under the cap
    a, b = seq(20, 100), seq(21, 100)
    s.add_sequence(a); s.add_sequence(b)
    out = run_step(m, s)
    assert [(x.seq.id, x.num_tokens) for x in out[4:]] == [(20, 32), (21, 28)] and sum(x.num_tokens for x in out) == 64


@pytest.mark.parametrize("chunk,page", [(2, 4), (4, 4), (8, 8), (3, 8)])
def test_small_portions_and_portions_that_end_at_a_page_edge(chunk, page):
    """Portions down to two tokens; with chunk == page every portion ends exactly at a page's edge: pages are taken for
    exactly the tokens that run, one page per step and never one ahead."""
    m = CacheManager([PagedKV(1, 8)], page, 16, 2)
    s = Scheduler(m, 100, 2, 64, prefill_chunk=chunk)
    a = seq(0, 19)
    s.add_sequence(a)
    done = 0
    while a.num_generated == 0:
        out = run_step(m, s)
        assert len(out) == 1 and out[0].num_tokens == min(chunk, 19 - done)
        done += out[0].num_tokens
        assert a.cache.num_tokens == done and len(a.cache.tables[0]) == -(-done // page)
        assert out[0].samples == (done == 19)
    assert done == 19


def test_a_parked_cache_serves_the_next_turn_and_goes_first_when_pages_are_short():
    m, s = make(num_pages=6, page=4, budget=100, max_seqs=2, max_len=24)
    a = seq(0, 6)
    s.add_sequence(a)
    run_step(m, s); run_step(m, s)                      # 6 prompt tokens, then one decoded: 7 cached, 8 known
    s.finish(a, "max_new_tokens", keep=True)
    assert a.status is SequenceStatus.FINISHED and a.cache is not None and a.cache.live and s.parked == [a]
    assert m.num_free_pages() == [4] and not s.has_unfinished()
    # a further turn: only what is not cached yet runs (the last sampled token and the new ones)
    a.tokens += [3, 4, 5]
    a.num_prompt_tokens = len(a.tokens)
    s.add_sequence(a)
    out = run_step(m, s)
    assert [(x.seq.id, x.num_tokens, x.samples) for x in out] == [(0, 4, True)] and s.parked == []
    s.finish(a, "eos", keep=True)
    # another request needs the pages: the parked cache is taken back before anything is preempted or made to wait
    b = seq(1, 17)
    s.add_sequence(b)
    out = run_step(m, s)
    assert [(x.seq.id, x.num_tokens) for x in out] == [(1, 17)] and a.cache is None and s.parked == [] and s.num_preemptions == 0
    # the turn after that recomputes the history
    s.finish(b, "eos")
    a.tokens += [6]
    a.num_prompt_tokens = len(a.tokens)
    s.add_sequence(a)
    known = len(a.tokens)
    assert [(x.seq.id, x.num_tokens) for x in run_step(m, s)] == [(0, known)]
    s.finish(a, "eos", keep=True)
    s.abort(a)                                           # removing the request gives the parked cache back
    assert m.num_free_pages() == [6] and m.slots.num_free == 2 and s.parked == []


def test_a_parked_cache_gives_its_slot_to_a_new_request():
    m, s = make(num_pages=16, page=4, budget=100, max_seqs=1, max_len=24)
    a = seq(0, 3)
    s.add_sequence(a)
    run_step(m, s)
    s.finish(a, "eos", keep=True)
    b = seq(1, 3)
    s.add_sequence(b)
    assert [(x.seq.id) for x in run_step(m, s)] == [1] and a.cache is None


def test_a_model_with_windows_only_runs_requests_longer_than_its_pool():
    """Every paged layer reads the last 10 keys only, and the window gives back the pages it has passed: a pool of 6
    pages of 4 tokens (24 tokens) runs a prompt of 60 tokens to 90, in portions as large as the free pages allow, and a
    second request beside it."""
    m = CacheManager([PagedKV(1, 8, window=10), PagedKV(1, 8, window=10)], page_size=4, num_pages=6, max_num_seqs=2)
    assert m.max_tokens_per_request() > 1 << 40
    s = Scheduler(m, 64, 2, 128)
    a = seq(0, 60, max_new_tokens=30, ignore_eos=True)
    s.add_sequence(a)                                        # not refused, though 60 > 24
    portions = []
    while a.num_generated < 30:
        out = run_step(m, s)
        assert out, "the request is stuck"
        portions.append(out[0].num_tokens)
        assert len(a.cache.pages_held(0)) <= 6
    assert len(a) == 90 and max(portions) <= 24 and portions.count(1) >= 29
    s.finish(a, "max_new_tokens")
    assert m.num_free_pages() == [6]
    # two at once: the second waits for pages, then runs; nothing is preempted for good
    b, c = seq(1, 30, max_new_tokens=8, ignore_eos=True), seq(2, 17, max_new_tokens=8, ignore_eos=True)
    s.add_sequence(b); s.add_sequence(c)
    for _ in range(200):
        if not s.has_unfinished():
            break
        for sc in run_step(m, s):
            if sc.seq.num_generated >= 8:
                s.finish(sc.seq, "max_new_tokens")
    assert not s.has_unfinished() and len(b) == 38 and len(c) == 25
    m.check()
    # a window that the pool cannot hold is a limit like any other
    small = CacheManager([PagedKV(1, 8, window=40)], page_size=4, num_pages=6, max_num_seqs=2)
    assert small.max_tokens_per_request() == 24
    with pytest.raises(ValueError, match="cache pool"):
        Scheduler(small, 64, 2, 128).add_sequence(seq(3, 60))
