"""The cache manager (CPU): no page lost, held twice or freed twice, under random orders of
requests; windows give pages back; slots."""
import random

import pytest

from spyinfer_amd.cache import CacheManager, FixedState, OutOfPages, OutOfSlots, PagedKV, PagePool


def test_pool_is_lifo_like_the_reference():
    # src/engine/block_manager.cpp:24-26: the first page handed out is N-1; a freed page comes next
    p = PagePool(4)
    assert [p.allocate(), p.allocate()] == [3, 2]
    p.free(3)
    assert p.allocate() == 3
    assert [p.allocate(), p.allocate()] == [1, 0]
    with pytest.raises(OutOfPages):
        p.allocate()
    p.free(2)
    with pytest.raises(ValueError):
        p.free(2)
    with pytest.raises(ValueError):
        p.free(9)


def test_groups_by_need():
    full, win = PagedKV(2, 16), PagedKV(2, 16, window=20)
    m = CacheManager([full, win, full, None, FixedState((4,)), win], page_size=8, num_pages=10, max_num_seqs=2)
    assert [g.cache_ids for g in m.page_groups] == [[0, 2], [1, 5]] and [g.cache_ids for g in m.state_groups] == [[4]]
    assert m.location[5] == ("paged", 1, 1) and 3 not in m.location


def test_reserve_commit_release_and_window():
    full, win = PagedKV(1, 8), PagedKV(1, 8, window=10)
    m = CacheManager([full, win], page_size=4, num_pages=8, max_num_seqs=2)
    rc = m.admit("a")
    assert m.pages_needed(rc, 9) == [3, 3]
    m.reserve(rc, 9)
    m.commit(rc, 9)
    m.check()
    # window 10: with 9 tokens the next query (position 9) reads keys 0..9: nothing is given back
    assert rc.tables[1].count(-1) == 0
    m.reserve(rc, 8)
    m.commit(rc, 8)
    # 17 tokens: the next query at 17 reads keys 8..17: pages 0 and 1 of the window group are back
    assert rc.tables[1][:2] == [-1, -1] and rc.tables[1][2] >= 0 and rc.tables[0].count(-1) == 0
    assert m.num_free_pages() == [8 - 5, 8 - 3]
    m.check()
    with pytest.raises(ValueError):
        m.commit(rc, 1)                      # nothing reserved
    m.release(rc)
    assert m.num_free_pages() == [8, 8] and m.slots.num_free == 2
    with pytest.raises(ValueError):
        m.release(rc)
    m.check()


def test_reserve_is_all_or_nothing():
    m = CacheManager([PagedKV(1, 8), PagedKV(1, 8, window=4)], page_size=4, num_pages=3, max_num_seqs=4)
    a, b = m.admit("a"), m.admit("b")
    m.reserve(a, 8)
    assert not m.can_reserve(b, 8)
    with pytest.raises(OutOfPages):
        m.reserve(b, 8)
    assert m.num_free_pages() == [1, 1] and b.tables == [[], []]
    m.check()


def test_slots():
    m = CacheManager([PagedKV(1, 8)], 4, 4, max_num_seqs=2)
    a, b = m.admit(1), m.admit(2)
    assert (a.slot, b.slot) == (0, 1) and not m.can_admit()
    with pytest.raises(OutOfSlots):
        m.admit(3)
    with pytest.raises(ValueError):
        m.admit(1)
    m.release(a)
    assert m.admit(3).slot == 0


@pytest.mark.parametrize("seed", range(5))
def test_random_orders_keep_the_invariants(seed):
    rng = random.Random(seed)
    m = CacheManager([PagedKV(2, 16), PagedKV(2, 16, window=24), PagedKV(2, 16)], page_size=8, num_pages=40, max_num_seqs=6)
    live, n = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.can_admit():
            live[n] = m.admit(n)
            n += 1
        elif op < 0.85 and live:
            rc = rng.choice(list(live.values()))
            k = rng.choice([1, 1, 1, 2, 5, 17, 30])
            if m.can_reserve(rc, k):
                m.reserve(rc, k)
                if rng.random() < 0.9:
                    m.commit(rc, rng.randint(1, k))
            else:
                with pytest.raises(OutOfPages):
                    m.reserve(rc, k)
        elif live:
            rid = rng.choice(list(live))
            m.release(live.pop(rid))
        m.check()
    for rc in live.values():
        m.release(rc)
    m.check()
    assert m.num_free_pages() == [40, 40] and m.slots.num_free == 6


def test_a_cache_kind_from_outside_forms_groups_of_its_own():
    """The manager and the storage ask a kind only what ``CacheKind`` defines: a kind defined here (pages of one float32
    tensor) is grouped apart from keys and values, gets its own pool and block tables, and its layers get its view."""
    import dataclasses

    import torch

    from spyinfer_amd.cache import CacheKind
    from spyinfer_amd.cache.storage import CacheStorage

    @dataclasses.dataclass(frozen=True)
    class Latent(CacheKind):
        width: int
        paged = True

        def page_bytes(self, page_size, act_dtype):
            return 4 * self.width * page_size

        def allocate(self, num_layers, count, page_size, act_dtype, device):
            return [torch.zeros((num_layers, count, page_size, self.width), dtype=torch.float32, device=device)]

        def layer_view(self, group, tensors, index, page_size):
            return ("latent", group, tensors[0][index])

    m = CacheManager([Latent(12), PagedKV(2, 16), Latent(12), FixedState((3,)), Latent(5)], page_size=8, num_pages=6, max_num_seqs=2)
    assert [g.cache_ids for g in m.page_groups] == [[0, 2], [1], [4]] and [g.cache_ids for g in m.state_groups] == [[3]]
    st = CacheStorage(m, torch.bfloat16, "cpu")
    assert [tuple(t.shape) for t in st.tensors] == [(2, 6, 8, 12), (1, 6, 2, 8, 16), (1, 6, 2, 16, 8), (1, 6, 8, 5), (1, 2, 3)]
    kind, group, view = st.layer(2)
    assert kind == "latent" and group == 0 and view.data_ptr() == st.tensors[0][1].data_ptr()
    assert CacheStorage.bytes_per_page([s for s in (Latent(12), PagedKV(2, 16), Latent(12), FixedState((3,)), Latent(5), None)], 8,
                                       torch.bfloat16) == 4 * 12 * 8 * 2 + 2 * 2 * 16 * 8 * 2 + 4 * 5 * 8
    rc = m.admit("a")
    m.reserve(rc, 20)
    assert [len(t) for t in rc.tables] == [3, 3, 3] and m.num_free_pages() == [3, 3, 3]
    m.commit(rc, 20)
    m.release(rc)
    m.check()
    with pytest.raises(TypeError, match="CacheKind"):
        CacheManager([object()], 8, 4, 2)


def test_rewind_steps_back_where_the_cache_allows_it():
    m = CacheManager([PagedKV(1, 8)], page_size=4, num_pages=4, max_num_seqs=2)
    rc = m.admit("a")
    m.reserve(rc, 8)
    m.commit(rc, 8)
    table = list(rc.tables[0])
    assert m.rewind(rc, 7) and rc.num_tokens == 7 and rc.reserved == 1 and rc.tables[0] == table
    assert m.pages_needed(rc, 1) == [0]
    m.reserve(rc, 1)
    m.commit(rc, 1)
    assert rc.num_tokens == 8 and rc.reserved == 0
    m.check()
    with pytest.raises(ValueError):
        m.rewind(rc, 9)
    # a window that has given back the page which the earlier position reads: no way back
    w = CacheManager([PagedKV(1, 8, window=4)], page_size=4, num_pages=4, max_num_seqs=2)
    rc = w.admit("a")
    w.reserve(rc, 7)
    w.commit(rc, 7)                 # the next query (position 7) reads keys 4..7: page 0 is back
    assert rc.tables[0][0] == -1
    assert not w.rewind(rc, 6) and rc.num_tokens == 7          # position 6 reads keys 3..6
    w.reserve(rc, 1)
    w.commit(rc, 1)
    assert w.rewind(rc, 7) and rc.num_tokens == 7               # position 7 reads keys 4..7, all there
    # a state of fixed size has taken its tokens in for good
    s = CacheManager([PagedKV(1, 8), FixedState((4,))], page_size=4, num_pages=4, max_num_seqs=2)
    rc = s.admit("a")
    s.reserve(rc, 5)
    s.commit(rc, 5)
    assert not s.rewind(rc, 4) and rc.num_tokens == 5 and s.rewind(rc, 5)
