"""The work list of decode attention (csrc/runtime.cpp, syn_decode_items): which sequence gets how
many of a step's workgroups.  No GPU: the list is laid out on the host."""
import random

import pytest

from synaptix_amd.kernels import runtime as rt

UNIT, MIN_UNITS = 32, 8


def _unpacked(lengths, n_splits, window=None):
    """(sequence, split, splits of the sequence, first) of every item; the length that an item carries and the
    table by sequence behind the items are checked here."""
    flat = rt.decode_items(lengths, n_splits, window)
    T, rows = len(lengths) * n_splits, len(lengths)
    assert len(flat) == 4 * T + 2 * rows
    out = []
    for at in range(T):
        seq, split_and_n, first, length = flat[4 * at:4 * at + 4]
        assert seq < 0 or length == lengths[seq]
        out.append((seq, split_and_n & 0xFFFF, split_and_n >> 16, first))
        if seq >= 0:
            assert flat[4 * T + 2 * seq:4 * T + 2 * seq + 2] == [first, split_and_n >> 16]   # the same by sequence
    return out


def _by_sequence(items):
    seqs = {}
    for at, (seq, split, n, first) in enumerate(items):
        if seq < 0:
            continue
        seqs.setdefault(seq, []).append((at, split, n, first))
    return seqs


def _check(lengths, n_splits, window=None):
    items = _unpacked(lengths, n_splits, window)
    assert len(items) == len(lengths) * n_splits
    seqs = _by_sequence(items)
    assert sorted(seqs) == list(range(len(lengths)))          # every sequence is there
    taken = set()
    for seq, rows in seqs.items():
        n = rows[0][2]
        assert [r[1] for r in rows] == list(range(n)) and all(r[2] == n for r in rows)   # each split once, in order
        first = rows[0][3]
        assert all(r[3] == first for r in rows) and first >= 0                           # one place for the sequence's partial results
        places = set(range(first, first + n))
        assert not (places & taken) and max(places) < len(items)
        taken |= places
        keys = lengths[seq] if window is None else min(lengths[seq], window)
        units = max(1, -(-keys // UNIT))
        assert n == 1 or units >= MIN_UNITS * n                                           # no split shorter than the least
    spare = [at for at, it in enumerate(items) if it[0] < 0]
    assert spare == list(range(len(items) - len(spare), len(items)))                      # spare items last
    return items, {s: rows[0][2] for s, rows in seqs.items()}


def test_sequences_of_one_length_get_equal_shares():
    _, n = _check([2060] * 8, 4)
    assert set(n.values()) == {4}
    _, n = _check([300] * 3, 5)      # 10 units: no second split of 8
    assert set(n.values()) == {1}


def test_longer_sequences_get_more_splits_and_lie_first():
    lengths = [64, 4000, 700, 3900, 1200, 90, 2500, 512]
    items, n = _check(lengths, 4)
    assert n[1] >= n[6] >= n[4] >= n[2] >= n[0] == 1
    assert sum(n.values()) <= 32 and n[1] > 4                 # what short sequences cannot use goes to long ones
    # in rounds: every sequence's first split, then the second of those that have one, ...; in a round the longest pieces first
    rounds = [sp for s, sp, _, _ in items if s >= 0]
    assert rounds == sorted(rounds)
    for r in set(rounds):
        pieces = [-(-(-(-lengths[s] // UNIT)) // k) for s, sp, k, _ in items if s >= 0 and sp == r]
        assert pieces == sorted(pieces, reverse=True)
    pieces = [-(-(-(-lengths[s] // UNIT)) // k) for s, sp, k, _ in items if s >= 0]
    # the longest piece of the uneven batch is shorter than with equal shares
    assert max(pieces) < -(-(-(-4000 // UNIT)) // 4)


def test_a_window_bounds_the_keys_that_count():
    _, n = _check([5000, 600], 4, window=512)
    assert n == {0: 2, 1: 2}                                  # both see 512 keys = 16 units: two splits of 8
    _, n = _check([5000, 600], 4)
    assert n[0] > n[1]


def test_padding_rows_and_random_batches_keep_the_list_whole():
    rnd = random.Random(3)
    for _ in range(200):
        rows = rnd.randint(1, 40)
        lengths = [rnd.choice([1, rnd.randint(1, 300), rnd.randint(1, 40000)]) for _ in range(rows)]
        _check(lengths, rnd.randint(1, 16), rnd.choice([None, None, 128, 4096]))


def test_refuses_an_empty_list():
    with pytest.raises(rt.CacheError):
        rt.decode_items([], 4)
