"""The host's cut of a decode step's keys into pieces (``key_pieces.decode_pieces``): every block of 32 keys of every (entry,
kv head) lies in exactly one piece, whatever the lengths, the window and the numbers of entries and heads are."""
import numpy as np
import pytest

from spyinfer_amd.kernels import key_pieces


def _check(kv_len, n_kv, window):
    rec = key_pieces.decode_pieces(kv_len, n_kv, window)
    assert rec.dtype == np.int32 and rec.shape == (key_pieces.decode_pieces_capacity(len(kv_len), n_kv), key_pieces.PIECE_RECORD)
    live = rec[rec[:, 0] >= 0]
    assert (rec[len(live):] == -1).all(), "unused records come last and say so"
    sizes = live[:, 3] - live[:, 2]
    assert (sizes > 0).all(), "no empty piece"
    # the order of the blocks: the largest 256 pieces, then the next 256 from the smallest up (a unit's second block
    # evens out its first), then what is left, falling
    per = max(1, key_pieces.PIECE_UNITS // n_kv) * n_kv
    assert (np.diff(sizes[:per]) <= 0).all() and (np.diff(sizes[per:2 * per]) >= 0).all() and (np.diff(sizes[2 * per:]) <= 0).all()
    if len(sizes) > per:
        assert sizes[:per].min() >= sizes[per:].max() and (len(sizes) <= 2 * per or sizes[per:2 * per].min() >= sizes[2 * per:].max())
    slots = set()
    for s, kvl in enumerate(kv_len):
        p0 = kvl - 1
        lo = (max(0, p0 - window + 1) if window else 0) & ~31
        nblk = (p0 - lo) // 32 + 1
        for hk in range(n_kv):
            mine = live[(live[:, 0] == s) & (live[:, 1] == hk)]
            mine = mine[np.argsort(mine[:, 4])]
            parts = len(mine)
            assert 1 <= parts <= key_pieces.MAX_PARTS
            assert (mine[:, 4] == np.arange(parts)).all() and (mine[:, 5] == parts).all() and (mine[:, 7] == kvl).all()
            assert mine[0, 2] == 0 and mine[-1, 3] == nblk and (mine[1:, 2] == mine[:-1, 3]).all(), "the parts tile the entry's blocks"
            assert (mine[:, 6] == mine[0, 6]).all(), "one first slot for all parts of an (entry, kv head)"
            mine_slots = set(range(int(mine[0, 6]), int(mine[0, 6]) + parts))
            assert not (slots & mine_slots)
            slots |= mine_slots
    assert slots == set(range(len(live))), "the workspace slots are dense: one per piece"
    return live


@pytest.mark.parametrize("seed", range(12))
def test_every_block_of_keys_lies_in_one_piece(seed):
    rng = np.random.default_rng(seed)
    S = int(rng.integers(1, 70))
    n_kv = int(rng.choice([1, 2, 3, 8]))
    window = int(rng.choice([0, 0, 40, 1000]))
    top = int(rng.choice([40, 700, 5000, 20000]))
    kv_len = rng.integers(1, top, S)
    _check(kv_len, n_kv, window)


def test_requests_of_one_length_that_fill_the_chip_are_not_cut():
    live = _check(np.full(32, 1153), 8, 0)
    assert len(live) == 256 and (live[:, 5] == 1).all()


def test_few_requests_are_cut_to_fill_the_chip():
    live = _check(np.full(8, 1153), 8, 0)
    assert len(live) == 256 and (live[:, 5] == 4).all()


def test_a_few_requests_more_than_fill_the_chip_give_every_unit_a_whole_entry_and_a_part():
    """40 requests of one length and 8 kv heads are 320 (entry, kv head) pairs for 256 units: 32 requests stay whole (a
    unit's first block), 8 are cut in four (a quarter as every unit's second block), 512 blocks in all."""
    live = _check(np.full(40, 1153), 8, 0)
    parts = {s: int(live[live[:, 0] == s][0, 5]) for s in range(40)}
    assert sorted(parts.values()) == [1] * 32 + [4] * 8 and len(live) == 512
    sizes = live[:, 3] - live[:, 2]
    assert (sizes[:256] == 37).all() and sizes[256:].max() <= 10
    # 44 requests: a third part each would make more second blocks than units
    live = _check(np.full(44, 1153), 8, 0)
    assert sorted(int(live[live[:, 0] == s][0, 5]) for s in range(44)) == [1] * 32 + [2] * 12 and len(live) == 448


def test_a_long_request_among_short_ones_is_cut_and_the_short_ones_are_not():
    kv_len = np.array([6000] + [200] * 40)
    live = _check(kv_len, 8, 0)
    assert live[live[:, 0] == 0][0, 5] > 4 and (live[live[:, 0] > 0][:, 5] == 1).all()
    # no piece is far above an even share of the step's blocks
    share = (live[:, 3] - live[:, 2]).sum() / key_pieces.PIECE_UNITS
    assert (live[:, 3] - live[:, 2]).max() <= 1.5 * share + key_pieces.PIECE_MIN_BLOCKS


def test_the_longest_request_never_has_more_parts_than_the_kernel_merges():
    live = _check(np.array([100000, 5]), 1, 0)
    assert live[:, 5].max() <= key_pieces.MAX_PARTS


def test_a_window_counts_the_blocks_it_sees_only():
    live = _check(np.array([5000, 70]), 2, 64)
    assert (live[live[:, 0] == 0][:, 3] <= 3).all()
