"""The keys of a decode step, cut into pieces on the host.

A step of single tokens has one query row per request, and its attention reads every request's keys once: the time of
the step's attention is the time of the compute unit with the most keys.  With one number of key parts for all requests
that is the longest request's part.  Here the host cuts every request's keys by its own length, from an estimate of the
kernel's time, and hands the kernel one record per block (``decode_pieces``); the kernel's grid is then a fixed number
of records whatever the lengths are.  Plain numpy: nothing here touches the device.
"""
from __future__ import annotations

from typing import Optional

import numpy as np

MAX_PARTS = 32              # most parts of an (entry, kv head): what the kernel's merging block takes (8 kv heads of one long
                            # request give every compute unit a block only in 32 parts: 38 000 keys 39.5 us against 53.7 in 16)
PIECE_UNITS = 256           # compute units that the pieces are dealt to; each runs two blocks at a time
PIECE_MIN_BLOCKS = 8        # a part wants this many blocks of 32 keys at least (measured at 1100 keys, 1 to 4 requests: 4-8 parts best)
PIECE_RECORD = 8            # ints per record
# What the estimate of a cut's time is made of, in microseconds (measured with 8 kv heads of 128, 8 to 96 requests of
# even and uneven lengths; the estimates are within 8 % rms of the kernel's times, and the cut they choose was the
# fastest of those measured, to within the timings' noise, in every case):
PIECE_START_US = 7.0        # from the kernel's start to a block's first keys, and its end
PIECE_MERGE_US = 3.0        # the way of the parts through memory, once per step that cuts any entry
PIECE_MERGE_MORE_US = 2.5   # each eight parts beyond sixteen of the entry with the most (the merging block asks for eight at a time)
PIECE_ROUND_US = 4.0        # each further round of blocks on the units beyond the two that are there from the start
PIECE_BLOCK_US = 0.45       # a unit's time for a block of 32 keys (16 KB) while it reads alone
PIECE_SHARED_US = 0.56      # what all units reading at once add to it (the two add as squares)


def decode_pieces_capacity(entries: int, n_kv: int) -> int:
    """Records in the array that ``decode_pieces`` fills for a step of ``entries`` single tokens: a fixed number (a
    launch shape), whatever the requests' lengths are."""
    return 2 * PIECE_UNITS + entries * n_kv


def _piece_sizes(nblk, width, even):
    """How entries of ``nblk`` blocks of 32 keys are cut into parts of at most ``width`` blocks: [entries, MAX_PARTS]
    sizes (0: no such part) and the numbers of parts.  Parts of one size and the rest (the last part, which also prepares
    and stores the new key, is the shortest); a rest shorter than half of what a part may be joins the part before it.
    ``even``: the size is the least that gives the entry no more parts than ``width`` does (37 blocks at width 12: 10,
    10, 10, 7 instead of 12, 12, 13).  ``width``: one for all entries, or one per entry."""
    n = nblk.astype(np.int64)
    idx = np.arange(MAX_PARTS, dtype=np.int64)[None, :]
    w = np.broadcast_to(np.asarray(width, dtype=np.int64), n.shape).copy()      # (one width, or one per entry)
    if even:
        w = np.maximum(1, -(-n // np.maximum(1, -(-n // width))))
    full = n // w
    rest = n - full * w
    joined = (rest > 0) & (2 * rest < np.minimum(PIECE_MIN_BLOCKS, w)) & (full > 0)
    parts = np.maximum(1, full + ((rest > 0) & ~joined))
    sizes = np.where(idx < full[:, None], w[:, None], 0)
    last = (parts - 1)[:, None]
    sizes = np.where((idx == last) & (rest > 0)[:, None], np.where(joined, w + rest, rest)[:, None], sizes)
    return sizes, parts


def _estimated_time(sizes_per_entry, n_kv, d=128) -> float:
    """Microseconds of the attention kernel for a cut.  Unit c takes blocks c and c + 256 of the records' order (the
    largest 256 pieces, then the next 256 from the smallest up, so that a long first piece meets a short second one), and
    later blocks go where least is left; the units share the memory evenly (a unit with one block gets as much as one
    with two), so a step ends with its fullest unit, which reads alone at the end at what a unit can take."""
    s = np.repeat(sizes_per_entry[sizes_per_entry > 0], n_kv).astype(np.float64)
    s = -np.sort(-s)
    U = PIECE_UNITS
    load = np.zeros(U)
    load[:min(U, s.shape[0])] += s[:U]
    second = s[U:2 * U][::-1]                                # (the second round goes out smallest first: decode_pieces)
    load[:second.shape[0]] += second
    for r0 in range(2 * U, s.shape[0], U):
        chunk = s[r0:r0 + U]
        load = np.sort(load)
        load[:chunk.shape[0]] += chunk
    load = np.sort(load)
    steps = np.diff(load, prepend=0.0)
    reading = U - np.arange(U)                              # units still reading while the i-th fullest finishes
    t = float((steps * np.sqrt(PIECE_BLOCK_US ** 2 + (reading * (PIECE_SHARED_US / U)) ** 2)).sum()) * (d / 128.0)
    return t + PIECE_START_US + PIECE_ROUND_US * max(0, -(-int(s.shape[0]) // (2 * U)) - 1)


def _merge_time(parts) -> float:
    """Microseconds that a step's merges add: the last block of the entry with the most parts asks for eight at a time."""
    return PIECE_MERGE_US + PIECE_MERGE_MORE_US * max(0, -(-int(parts.max(initial=1)) // 8) - 2)


def _fill_widths(nblk, n_kv):
    """Widths per entry for the cut that fills the units in two rounds: the longest entries, as many as give the units
    their first blocks (cut only where longer than a unit's even share), and the others cut so finely that they make
    about one second block per unit: 40 requests of one length are 32 whole and 8 in four parts each, and every unit
    has a whole entry and a quarter.  Never more second blocks than units, in coarser parts if need be (44 requests: 32
    whole and 12 in two parts each, not in three: a third round costs more than the uneven second).  None if the first
    round takes all entries."""
    n = nblk.astype(np.int64)
    total = int(n.sum()) * n_kv
    share = max(1, -(-total // PIECE_UNITS))
    floor = -(-n // MAX_PARTS)
    first_parts = -(-n // np.maximum(share, floor))
    order = np.argsort(-n, kind="stable")
    taken = np.cumsum(first_parts[order]) * n_kv
    first = np.zeros(n.shape[0], dtype=bool)
    first[order[:int(np.searchsorted(taken, PIECE_UNITS, side="left")) + 1]] = True
    if first.all():
        return None
    rest = int(n[~first].sum()) * n_kv
    fine = max(PIECE_MIN_BLOCKS, -(-rest // PIECE_UNITS))
    longest = int(n[~first].max())
    for parts in range(MAX_PARTS, 0, -1):
        fine = max(fine, -(-longest // parts))
        if int((-(-n[~first] // fine)).sum()) * n_kv <= PIECE_UNITS:
            break
    return np.where(first, np.maximum(share, floor), np.maximum(fine, floor))


_piece_choices = {}


def _piece_choice(nblk, n_kv, d=128):
    """How a step whose entries have ``nblk`` blocks of keys is cut: None (not at all), (W, even): parts of at most W
    blocks, W being the whole step's blocks over the compute units or over twice as many (and no less than gives the
    longest entry 16 parts, or 32), an entry's parts of one size or W and a rest, or ("fill", True) (``_fill_widths``):
    whichever has the shortest estimated time.
    Decided from the lengths rounded up to 8 blocks, so that a step is always cut the same way and the choice is looked
    up in most steps (a request's rounded length changes once in 256 steps); the last choices are kept."""
    coarse = nblk >> 3
    key = (coarse.tobytes(), n_kv, d, MAX_PARTS, PIECE_UNITS, PIECE_MIN_BLOCKS, PIECE_START_US, PIECE_MERGE_US, PIECE_ROUND_US)
    if key in _piece_choices:
        return _piece_choices[key]
    rounded = (coarse << 3) + 7
    total = int(rounded.sum()) * n_kv
    if 4 * PIECE_UNITS * int(rounded.max(initial=1)) <= total:
        # the longest entry is no more than a quarter of a unit's even share: whole entries, dealt out as blocks end,
        # even the units out by themselves (and the estimates of thousands of pieces would cost the host half a
        # millisecond a step)
        _piece_choices[key] = None
        return None
    longest = int(rounded.max(initial=1))
    whole = rounded[:, None] * (np.arange(MAX_PARTS)[None, :] == 0)
    best = (_estimated_time(whole, n_kv, d), None)
    # (the longest entry in at most 16 parts as well as in at most MAX_PARTS: more than 16 cost the merge further round trips)
    widths = {max(PIECE_MIN_BLOCKS, -(-longest // most), -(-total // (PIECE_UNITS * k))) for k in (1, 2) for most in (16, MAX_PARTS)}
    for width in sorted(widths):
        for even in (True, False):
            sizes, parts = _piece_sizes(rounded, width, even)
            if int(parts.max(initial=1)) > 1:
                t = _estimated_time(sizes, n_kv, d) + _merge_time(parts)
                if t < best[0]:
                    best = (t, (width, even))
    per_entry = _fill_widths(rounded, n_kv)
    if per_entry is not None:
        sizes, parts = _piece_sizes(rounded, per_entry, True)
        if int(parts.max(initial=1)) > 1:
            t = _estimated_time(sizes, n_kv, d) + _merge_time(parts)
            if t < best[0]:
                best = (t, ("fill", True))
    if len(_piece_choices) >= 64:
        _piece_choices.pop(next(iter(_piece_choices)))
    _piece_choices[key] = best[1]
    return best[1]


def _piece_plan(nblk, n_kv, d=128):
    """(sizes [S, 16], parts [S]) for entries of ``nblk`` blocks (``_piece_choice``, ``_piece_sizes``)."""
    choice = _piece_choice(nblk, n_kv, d)
    if choice is not None and choice[0] == "fill":
        widths = _fill_widths(nblk, n_kv)
        choice = None if widths is None else (widths, True)
    if choice is None:
        return nblk[:, None] * (np.arange(MAX_PARTS)[None, :] == 0), np.ones(nblk.shape[0], dtype=np.int64)
    return _piece_sizes(nblk, choice[0], choice[1])


def decode_pieces(kv_len, n_kv: int, window: int = 0, capacity: Optional[int] = None, head_dim: int = 128):
    """Cuts the keys of a step of single tokens into pieces for the fused attention kernel, one block each, so that the
    compute units have even shares whatever the requests' lengths are (with one number of parts for all entries, a step
    takes as long as its longest request's part).  ``kv_len`` [S]: keys of every entry after this step.  Returns int32
    [capacity, 8] records { entry, kv head, first and end block of 32 keys (counted from the first block the entry's
    window sees), number of the part, parts of the (entry, kv head), workspace slot of its first part, kv_len }, the
    largest pieces first (see below for the order), entry -1 in the unused ones.

    Entries are cut into parts of at most W blocks, W being the whole step's blocks over the 256 compute units or over
    twice as many, the parts of an entry even or W and a rest, or the longest entries whole and the others fine
    (``_fill_widths``), or they are not cut at all: whichever gives the shortest estimated time (``_piece_choice``)."""
    kv_len = np.asarray(kv_len, dtype=np.int64)
    S = int(kv_len.shape[0])
    capacity = decode_pieces_capacity(S, n_kv) if capacity is None else capacity
    p0 = kv_len - 1
    lo = (np.maximum(0, p0 - window + 1) if window > 0 else np.zeros_like(p0)) & ~31
    nblk = np.maximum(0, (p0 - lo) // 32 + 1)
    sizes, parts = _piece_plan(nblk, n_kv, head_dim)
    begin = np.cumsum(sizes, axis=1) - sizes
    ent, part = np.nonzero(sizes > 0)
    count = int(ent.shape[0])
    if count * n_kv > capacity:
        raise ValueError("decode_pieces: %d pieces for %d records" % (count * n_kv, capacity))
    order = np.argsort(-sizes[ent, part], kind="stable")
    ent, part = ent[order], part[order]
    # The records' order is the blocks' order, and the first 2 x 256 blocks go to the 256 units in turn: the largest 256
    # pieces first, then the next 256 / n_kv from the smallest up (measured against all in falling order, requests of 128
    # to 2560 keys: 55.2 / 56.8 us at 40 requests, 84.0 / 86.3 at 64, 24.4 / 25.4 at 16; even lengths: no difference).
    per = max(1, PIECE_UNITS // n_kv)
    if count > per:
        second = slice(per, min(count, 2 * per))
        ent[second], part[second] = ent[second][::-1].copy(), part[second][::-1].copy()
    # workspace slots: the parts of an (entry, kv head) lie together, entries and heads in order
    first_slot = (np.cumsum(parts) - parts) * n_kv
    rec = np.full((capacity, PIECE_RECORD), -1, dtype=np.int32)
    hk = np.tile(np.arange(n_kv, dtype=np.int64), count)
    ent, part = np.repeat(ent, n_kv), np.repeat(part, n_kv)
    n = count * n_kv
    rec[:n, 0] = ent
    rec[:n, 1] = hk
    rec[:n, 2] = begin[ent, part]
    rec[:n, 3] = begin[ent, part] + sizes[ent, part]
    rec[:n, 4] = part
    rec[:n, 5] = parts[ent]
    rec[:n, 6] = first_slot[ent] + hk * parts[ent]
    rec[:n, 7] = kv_len[ent]
    return rec
