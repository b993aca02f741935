"""The native host runtime on its own: the integer tables of a step, written from the cache's state."""
import ctypes as C

import numpy as np
import pytest
import torch

from synaptix_amd.cache import SequenceCache, CacheError
from synaptix_amd.engine.batch import StepLayout, fill_host_buffer
from synaptix_amd.kernels import runtime as rt
from synaptix_amd.parts.base import KvNeed


def make_cache():
    return SequenceCache([KvNeed(2, 16), KvNeed(1, 32, window=100)], 64 * 12, 4, torch.float32, "cpu")


def test_layout_puts_the_arrays_one_after_another():
    lay = StepLayout(7, 2, 3, [4, 2])
    assert lay.off == {"tokens": (0, 7), "tok_seq": (7, 7), "tok_pos": (14, 7), "seq_start": (21, 3),
                       "seq_past": (24, 2), "seq_len": (26, 2), "seq_slot": (28, 2), "want": (30, 3)}
    assert lay.table_off == [(33, 8), (41, 4)] and lay.total == 45
    assert StepLayout(0, 0, 0, []).total == 1


def test_step_tables_follow_the_cache():
    c = make_cache()
    a, b = c.acquire(), c.acquire()
    c.reserve(a, 70), c.commit(a, 70)
    c.reserve_step([b, a], [3, 2])
    lay = StepLayout(5, 2, 2, [c.table_width(g, [b, a]) for g in range(2)])
    assert lay.widths == [2, 2]
    host = np.full(lay.total + 3, -7, dtype=np.int32)
    fill_host_buffer(lay, host, c, [b, a], np.array([11, 12, 13, 21, 22]), [3, 2], [2, 4])

    def arr(name):
        o, n = lay.off[name]
        return host[o:o + n].tolist()

    assert arr("tokens") == [11, 12, 13, 21, 22]
    assert arr("tok_seq") == [0, 0, 0, 1, 1]
    assert arr("tok_pos") == [0, 1, 2, 70, 71]
    assert arr("seq_start") == [0, 3, 5] and arr("seq_past") == [0, 70] and arr("seq_len") == [3, 72]
    assert arr("seq_slot") == [b, a] and arr("want") == [2, 4]
    for g in range(2):
        o, n = lay.table_off[g]
        assert host[o:o + n].reshape(2, 2).tolist() == c.page_table(g, [b, a], width=2).tolist()
    assert host[lay.total:].tolist() == [-7, -7, -7]            # nothing written behind the tables
    with pytest.raises(CacheError, match="not live"):
        fill_host_buffer(lay, host, c, [b, 3], np.zeros(5), [3, 2], [2, 4])
    with pytest.raises(ValueError):
        fill_host_buffer(lay, host[:10], c, [b, a], np.zeros(5), [3, 2], [2, 4])


def test_decode_tables_pad_with_a_spare_page():
    c = make_cache()
    a, b = c.acquire(), c.acquire()
    c.reserve(a, 130), c.commit(a, 130)
    c.reserve(b, 5), c.commit(b, 5)
    c.reserve(a, 1), c.reserve(b, 1)
    rows, widths, spare = 4, [4, 4], [12, 12]
    lay = StepLayout(rows, rows, rows, widths)
    item_splits = [0, 3]                       # the second group keeps a work list for its attention: 4 x 3 items
    host = np.zeros(lay.total + 2 * rows + 4 * rows * 3 + 2 * rows, dtype=np.int32)
    temps, unis = (C.c_float * 2)(0.5, 0.0), (C.c_float * 2)(0.25, 0.75)
    rt.check(rt.lib().syn_decode_fill(c._h, rows, 2, rt.ints([a, b]), rt.ints([9, 8]), 2, rt.ints(widths),
                                      rt.ints(spare), temps, unis, rt.ints(item_splits), host.ctypes.data))

    def arr(name):
        o, n = lay.off[name]
        return host[o:o + n].tolist()

    assert arr("tokens") == [9, 8, 0, 0] and arr("tok_pos") == [130, 5, 0, 0]
    assert arr("tok_seq") == [0, 1, 2, 3] and arr("seq_start") == [0, 1, 2, 3, 4]
    assert arr("seq_past") == [130, 5, 0, 0] and arr("seq_len") == [131, 6, 1, 1]
    assert arr("seq_slot") == [a, b, -1, -1] and arr("want") == [0, 1, 2, 3]
    full = host[lay.table_off[0][0]:][:16].reshape(4, 4)
    own = c.page_table(0, [a, b], width=4)
    assert full[0, :3].tolist() == own[0, :3].tolist() and full[1, 0] == own[1, 0]
    assert full[0, 3] == 12 and full[1, 1:].tolist() == [12, 12, 12] and (full[2:] == 12).all()
    f = host[lay.total:lay.total + 2 * rows].view(np.float32)
    assert f.tolist() == [0.5, 0.0, 0.0, 0.0, 0.25, 0.75, 0.0, 0.0]
    flat = host[lay.total + 2 * rows:].tolist()
    assert flat == rt.decode_items([131, 6, 1, 1], 3)                          # from the lengths that the step has
    items = [flat[4 * i:4 * i + 4] for i in range(12)]
    assert sorted(i[0] for i in items[:4]) == [0, 1, 2, 3] and all(i[0] == -1 for i in items[4:])   # too short to split
    assert all(i[1] == 1 << 16 for i in items[:4]) and sorted(i[3] for i in items[:4]) == [1, 1, 6, 131]
    assert flat[48:] == [x for i in range(4) for x in (next(it[2] for it in items if it[0] == i), 1)]   # the same by sequence
    with pytest.raises(CacheError, match="width"):
        rt.check(rt.lib().syn_decode_fill(c._h, rows, 2, rt.ints([a, b]), rt.ints([9, 8]), 2, rt.ints([2, 4]),
                                          rt.ints(spare), None, None, None, host.ctypes.data))
    with pytest.raises(CacheError, match="rows"):
        rt.check(rt.lib().syn_decode_fill(c._h, 1, 2, rt.ints([a, b]), rt.ints([9, 8]), 2, rt.ints(widths),
                                          rt.ints(spare), None, None, None, host.ctypes.data))


def test_host_side_rules_of_the_kernels_stay_within_their_kernels_limits():
    """The numbers of splits and slices that the host picks: pure functions, checked over a grid of sizes."""
    import torch
    from synaptix_amd.kernels import ops
    for n_seqs in (1, 2, 3, 8, 17, 64, 300):
        for n_kv in (1, 2, 8):
            for pages in (1, 2, 8, 9, 33, 96, 128, 512, 4096):
                s = ops.decode_splits(n_seqs, n_kv, pages)
                assert 1 <= s <= 64 and s <= pages
                assert s == 1 or pages // s >= 4          # a split keeps at least four blocks
    assert ops.decode_splits(64, 8, 33) == 1 and ops.decode_splits(1, 8, 33) > 1
    for M in (1, 8, 9, 32, 33, 64, 65, 128, 512, 2048, 8192):
        for N, K in ((4096, 4096), (6144, 4096), (4096, 12288), (151936, 4096), (64, 64), (4096, 1000)):
            s = ops.gemm_slices(M, N, K, torch.bfloat16)
            assert 1 <= s <= 8
            if s > 1:
                step = ((K + s - 1) // s + 127) // 128 * 128
                assert (s - 1) * step < K, "no slice may be empty"
                assert K % 8 == 0 and (M <= 64 or K % 128 == 0)
            assert ops.gemm_slices(M, N, K, torch.float32) == 1
