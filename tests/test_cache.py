"""The cache's bookkeeping (no GPU): no slot or page lost, held twice or freed twice."""
import random

import pytest
import torch

from synaptix_amd.cache import SequenceCache, CacheFull, CacheError, pages_for
from synaptix_amd.parts import KvNeed, StateNeed


def make(max_tokens=640, max_slots=None, needs=None, max_positions=None):
    needs = needs if needs is not None else [KvNeed(2, 16)] * 3
    return SequenceCache(needs, max_tokens, max_slots, torch.float32, "cpu", max_positions=max_positions)


def test_groups_and_storage():
    c = make(needs=[KvNeed(2, 16), KvNeed(1, 32), KvNeed(2, 16), StateNeed((3, 5)), None, KvNeed(2, 16, window=100)])
    assert [g.layers for g in c.groups] == [[0, 2], [1], [5]]
    assert c.groups[0].k.shape == (2, 11, 2, 64, 16) and c.groups[0].v.shape == (2, 11, 2, 16, 64)   # + a spare page
    assert c.groups[1].k.shape == (1, 11, 1, 64, 32) and c.groups[1].spare_page == 10
    v0, v2, v3 = c.layer_view(0), c.layer_view(2), c.layer_view(3)
    assert v0.group == v2.group == 0 and v0.k_pages.data_ptr() != v2.k_pages.data_ptr()
    assert v3.state.shape == (10 + 1, 3, 5) and v3.spare_row == 10 and c.layer_view(4) is None   # a row for padding
    assert c.bytes_per_token() == 2 * 4 * (2 * 2 * 16 + 1 * 32 + 2 * 16)


def test_slot_life_cycle_and_errors():
    c = make(max_tokens=256, max_slots=2)
    a, b = c.acquire(), c.acquire()
    assert {a, b} == {0, 1} and c.free_slots == 0
    with pytest.raises(CacheFull, match="slots"):
        c.acquire()
    c.reserve(a, 70)
    c.commit(a, 70)
    assert c.length(a) == 70 and c.groups[0].pool.free_pages == 2
    c.reserve(a, 1)                                  # 71 tokens still fit two pages
    assert c.groups[0].pool.free_pages == 2
    with pytest.raises(CacheError, match="commit without reserve"):
        c.commit(a, 5)
    c.commit(a, 1)
    c.reserve(b, 128)
    with pytest.raises(CacheFull):
        c.reserve(a, 100)                            # would need a third page; nothing changes
    assert c.groups[0].pool.free_pages == 0 and c.length(a) == 71
    c.check()
    c.release(a)
    with pytest.raises(CacheError, match="not live"):
        c.release(a)                                 # freed twice
    with pytest.raises(CacheError, match="not live"):
        c.length(a)
    with pytest.raises(CacheError):
        c.reserve(7, 1)
    with pytest.raises(CacheError, match="at least one token"):
        c.reserve(b, 0)
    assert c.acquire() == a and c.length(a) == 0     # the slot is used again, empty
    c.check()


def test_position_range():
    c = make(max_tokens=1024, max_positions=100)
    s = c.acquire()
    c.reserve(s, 100)
    c.commit(s, 100)
    with pytest.raises(CacheError, match="KV overflow"):
        c.reserve(s, 1)


def test_page_table_follows_each_sequence():
    c = make(max_tokens=64 * 8)
    a, b = c.acquire(), c.acquire()
    c.reserve(a, 65); c.commit(a, 65)
    c.reserve(b, 10); c.commit(b, 10)
    c.reserve(a, 64); c.commit(a, 64)                # a grows after b took a page: its pages are not adjacent
    t = c.page_table(0, [b, a])
    assert t.shape == (2, 3) and t.dtype.name == "int32"
    assert t[1].tolist() == [0, 1, 3] and t[0].tolist()[0] == 2
    assert c.page_table(0, [a], width=5).shape == (1, 5)
    with pytest.raises(CacheError):
        c.page_table(0, [a], width=2)


def test_window_group_gives_pages_back_early():
    c = make(max_tokens=64 * 6, needs=[KvNeed(1, 16), KvNeed(1, 16, window=70)])
    s = c.acquire()
    c.reserve(s, 200); c.commit(s, 200)
    full, win = c.groups[0].pool, c.groups[1].pool
    assert full.free_pages == 2
    # the next query sits at 200 and sees keys 131..200: pages 0 and 1 (keys 0..127) are out of reach
    assert win.free_pages == 4
    assert c.page_table(1, [s])[0].tolist() == [0, 0, 2, 3] or c.page_table(1, [s])[0].tolist()[2:] == [2, 3]
    c.check()
    c.release(s)
    assert full.free_pages == win.free_pages == 6
    c.check()


def test_window_group_of_its_own_size():
    """With a promise about the longest step a group that keeps a window gets pages for the window and one step of
    every slot, not for all tokens; its pool, its spare page and its storage follow, the other group keeps its size,
    and long sequences still fit because the window gives pages back."""
    c = SequenceCache([KvNeed(1, 16), KvNeed(1, 16, window=70)], 64 * 40, 2, torch.float32, "cpu", max_step_tokens=64)
    full, win = c.groups[0], c.groups[1]
    assert full.n_pages == 40 and win.n_pages == 2 * (3 + 1)           # window 70 + step 64 = 134 tokens: 3 pages, + 1
    assert win.k.shape[1] == win.n_pages + 1 and win.spare_page == win.n_pages and full.k.shape[1] == 41
    a, b = c.acquire(), c.acquire()
    for _ in range(15):                                                # 960 tokens each, far beyond the small pool
        for s in (a, b):
            c.reserve(s, 64); c.commit(s, 64)
        c.check()
    assert c.length(a) == 960 and win.pool.free_pages >= 2 and full.pool.free_pages == 40 - 30
    assert max(c.page_table(1, [a, b]).max(), 0) < win.n_pages
    with pytest.raises(CacheFull):                                     # a step beyond the promise does not fit the small pool
        c.reserve(a, 64 * 9)
    c.check()
    c.release(a); c.release(b)
    assert win.pool.free_pages == win.n_pages and full.pool.free_pages == 40
    c.check()


def test_state_is_zeroed_when_a_slot_is_taken():
    c = make(needs=[StateNeed((4,))], max_slots=2)
    s = c.acquire()
    c.layer_view(0).state[s] += 5
    c.release(s)
    s2 = c.acquire()
    assert s2 == s and float(c.layer_view(0).state[s2].abs().sum()) == 0.0


def test_random_walk_keeps_every_invariant():
    rng = random.Random(0)
    c = make(max_tokens=64 * 40, max_slots=12, needs=[KvNeed(2, 16), KvNeed(2, 16, window=130)])
    live = {}
    for _ in range(3000):
        op = rng.random()
        if op < 0.25 and c.free_slots:
            live[c.acquire()] = 0
        elif op < 0.45 and live:
            s = rng.choice(list(live))
            c.release(s)
            del live[s]
        elif live:
            s = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 5, 64, 100])
            try:
                c.reserve(s, n)
                c.commit(s, n)
                live[s] += n
            except CacheFull:
                pass
        assert sorted(live) == c.live_slots
        for s, n in live.items():
            assert c.length(s) == n
    c.check()
    held = sum(pages_for(n) for n in live.values())
    assert c.groups[0].pool.free_pages <= 40 - held       # reserved pages may exceed the committed ones
    for s in list(live):
        c.release(s)
    c.check()
    assert c.free_slots == 12 and all(g.pool.free_pages == 40 for g in c.groups)


def test_states_of_some_slots_are_copied_and_put_back_and_padding_has_a_row_of_its_own():
    """What a captured step needs of the states: the rows of its slots alone can be saved and put back without a
    touch to lengths or to other slots; and a step's sequences map to rows through the step's own slot array, the
    padding (slot -1) to the spare row behind the slots."""
    from types import SimpleNamespace
    c = make(needs=[StateNeed((3,)), KvNeed(2, 16)], max_slots=3)
    a, b, d = c.acquire(), c.acquire(), c.acquire()
    st = c.layer_view(0).state
    st[a] += 1.0
    st[b] += 2.0
    st[d] += 3.0
    saved = c.states_of([a, d])
    st += 10.0
    c.put_states(saved)
    assert st[a].tolist() == [1.0] * 3 and st[d].tolist() == [3.0] * 3 and st[b].tolist() == [12.0] * 3
    view = c.layer_view(0)
    ctx = SimpleNamespace(seq_slot=torch.tensor([d, -1, a], dtype=torch.int32), tok_seq=torch.tensor([0, 0, 2, 1], dtype=torch.int32))
    assert view.seq_rows(ctx).tolist() == [d, 3, a] and view.spare_row == 3
    assert view.token_rows(ctx).tolist() == [d, d, a, 3]
    with pytest.raises(CacheError):
        c.states_of([7.5])


def test_going_back_to_a_snapshot():
    """A length can be rewound; a running state cannot, so a snapshot keeps a copy of it.  A
    window that has already given a page back refuses to go back behind it."""
    c = make(needs=[KvNeed(2, 16), StateNeed((3,)), KvNeed(2, 16, window=70)], max_slots=2)
    s = c.acquire()
    c.reserve(s, 40), c.commit(s, 40)
    c.layer_view(1).state[s] += 5.0
    snap = c.snapshot(s)
    c.reserve(s, 30), c.commit(s, 30)
    c.layer_view(1).state[s] += 1.0
    held = c.groups[0].pool.free_pages
    c.restore(snap)
    assert c.length(s) == 40 and c.layer_view(1).state[s].tolist() == [5.0, 5.0, 5.0]
    assert c.groups[0].pool.free_pages == held              # the pages stay with the sequence
    c.reserve(s, 30), c.commit(s, 30)                       # and are written again without new ones
    assert c.groups[0].pool.free_pages == held and c.length(s) == 70
    with pytest.raises(CacheError, match="cannot go back"):
        c.truncate(s, 71)
    c.reserve(s, 130), c.commit(s, 130)                     # 200 tokens: the window has let page 0 and 1 go
    with pytest.raises(CacheError, match="window"):
        c.restore(snap)
    c.truncate(s, 199)                                      # within what the window still holds
    c.check()
    c.release(s)
    c.check()
