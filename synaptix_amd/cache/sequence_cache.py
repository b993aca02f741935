"""The cache of the live sequences: a slot for each, keys and values for each layer that keeps
them, each sequence with its own length, and beside it a fixed-size state for each slot.

Layers with the same needs (kv heads, head size, all keys or a window of them) form a group; a
group has storage and a page pool of its own:
    k_pages [layers, pages, kv_heads, 64, head_dim]
    v_pages [layers, pages, kv_heads, head_dim, 64]      (transposed inside the page; a bf16 page in the
                                                          order of its kernels, ops.v_pages_to_kernel_order)
A group that keeps a window gives pages back as soon as every position in them has left the
window.  Layers with a StateNeed get `state[layer] : [slots + 1, *shape]`, zeroed when a slot is
taken (the reference keeps such state in the same per-layer vector as the keys and values,
crates/synaptix-models/llm/common/src/model.rs:359-362,377-492).

A slot is taken for a sequence (`acquire`), grows with `reserve` + `commit`, and is given back
with `release`; released slots and pages are handed out again.  Stale contents are never read:
attention reads positions below the sequence's length only.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np
import torch

from ..kernels import runtime as rt
from ..parts.base import KvNeed, StateNeed
from .pages import PAGE_TOKENS, CacheError, pages_for


@dataclass
class KvLayerView:
    """What a mixer with a KvNeed is handed for its layer."""
    group: int
    k_pages: torch.Tensor
    v_pages: torch.Tensor


@dataclass
class StateLayerView:
    """What a mixer with a StateNeed is handed: state [slots + 1, *shape]; row = slot id, and the last
    row belongs to the padding rows of a captured step (no sequence owns it, as with the spare page).

    A mixer whose steps are to be replayed from graphs reads and writes its state through row indices
    that lie on the device (`seq_rows`, `token_rows`: index_select / index_copy_ with them), because
    a captured step does not know its slots on the host."""
    state: torch.Tensor

    @property
    def spare_row(self) -> int:
        return self.state.shape[0] - 1

    def seq_rows(self, ctx) -> torch.Tensor:
        """int64 [n_seqs] on the device: the state row of each sequence of the step (padding: the spare row)."""
        slot = ctx.seq_slot
        return torch.where(slot < 0, torch.full_like(slot, self.spare_row), slot).long()

    def token_rows(self, ctx) -> torch.Tensor:
        """int64 [n_tokens] on the device: the state row of the sequence that each token of the step is in."""
        return self.seq_rows(ctx).index_select(0, ctx.tok_seq.long())


@dataclass
class Snapshot:
    """A point in a sequence that `SequenceCache.restore` goes back to."""
    slot: int
    length: int
    states: dict                      # cache layer -> copy of the slot's state


class _GroupPool:
    """The page pool of one group, as the native cache keeps it."""

    def __init__(self, cache, group: int, n_pages: int):
        self._cache, self._group, self.n_pages = cache, group, n_pages

    @property
    def free_pages(self) -> int:
        return rt.lib().syn_cache_free_pages(self._cache._h, self._group)


@dataclass
class _Group:
    need: KvNeed
    layers: list                      # cache-layer indices
    pool: _GroupPool = None
    k: torch.Tensor = None
    v: torch.Tensor = None
    spare_page: int = 0               # a page beyond the pool that no sequence owns (padding rows write there)
    n_pages: int = 0                  # pages of the group's pool (a group that keeps a window may have fewer)


class SequenceCache:
    def __init__(self, needs: list, max_tokens: int, max_slots: int | None, dtype, device,
                 max_positions: int | None = None, max_step_tokens: int | None = None):
        """needs[i]: KvNeed, StateNeed or None of cache layer i.  max_tokens: the most tokens that
        live sequences hold together, each sequence's count rounded up to whole pages.
        max_step_tokens: the most tokens that one step brings for one sequence, if the caller can promise
        it: a group of layers that keeps a window then gets pages for the window and one such step of every
        slot only (a step holds the pages of all its new tokens before the window gives old ones back), not
        for max_tokens; None: every group gets pages for max_tokens."""
        if max_tokens <= 0:
            raise CacheError("max_tokens must be positive")
        self.dtype, self.device = dtype, torch.device(device)
        self.n_pages = pages_for(max_tokens)
        self.max_slots = max_slots if max_slots is not None else self.n_pages
        if self.max_slots <= 0:
            raise CacheError("max_slots must be positive")
        self.max_positions = max_positions
        self.groups: list = []
        self._layer_group = {}
        self._layer_index = {}
        self._state = {}
        self._h = None
        for i, need in enumerate(needs):
            if isinstance(need, KvNeed):
                for gi, g in enumerate(self.groups):
                    if g.need == need:
                        break
                else:
                    gi = len(self.groups)
                    self.groups.append(_Group(need, []))
                self._layer_group[i] = gi
                self._layer_index[i] = len(self.groups[gi].layers)
                self.groups[gi].layers.append(i)
            elif isinstance(need, StateNeed):
                # one row more than slots: the padding rows of a captured step keep their state there
                self._state[i] = torch.zeros((self.max_slots + 1,) + tuple(need.shape), dtype=need.dtype,
                                             device=self.device)
            elif need is not None:
                raise CacheError(f"cache layer {i}: unknown need {need!r}")
        if rt.lib().syn_rt_page_tokens() != PAGE_TOKENS:
            raise RuntimeError("the runtime library was built for another page size")
        windows = [-1 if g.need.window is None else int(g.need.window) for g in self.groups]
        for g in self.groups:
            g.n_pages = self.n_pages
            if g.need.window is not None and max_step_tokens is not None:
                # at most window + step tokens of a sequence are held at once, and they may begin anywhere in a page
                g.n_pages = min(self.n_pages, self.max_slots * (pages_for(int(g.need.window) + int(max_step_tokens)) + 1))
        self._h = rt.lib().syn_cache_new(len(self.groups), rt.longs(windows), self.n_pages,
                                         rt.ints([g.n_pages for g in self.groups]), self.max_slots,
                                         -1 if max_positions is None else int(max_positions))
        if not self._h:
            raise CacheError(rt.last_error())
        for gi, g in enumerate(self.groups):
            n, nd = len(g.layers), g.need
            g.pool = _GroupPool(self, gi, g.n_pages)
            # zeros: what a kernel may touch beyond a sequence's end is at least a number
            g.spare_page = g.n_pages
            g.k = torch.zeros((n, g.n_pages + 1, nd.kv_heads, PAGE_TOKENS, nd.head_dim), dtype=dtype, device=self.device)
            g.v = torch.zeros((n, g.n_pages + 1, nd.kv_heads, nd.head_dim, PAGE_TOKENS), dtype=dtype, device=self.device)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            try:
                rt.lib().syn_cache_delete(h)
            except Exception:       # the interpreter is shutting down; the process's memory goes with it
                pass

    @staticmethod
    def _sid(sid) -> int:
        if not isinstance(sid, (int, np.integer)) or isinstance(sid, bool):
            raise CacheError(f"slot {sid!r} is not live")
        return int(sid)

    # ------------------------------------------------------------------ slots
    @property
    def free_slots(self) -> int:
        return rt.lib().syn_cache_free_slots(self._h)

    @property
    def live_slots(self) -> list:
        out = (C.c_int * self.max_slots)()
        n = rt.lib().syn_cache_live_slots(self._h, out)
        return list(out[:n])

    def acquire(self) -> int:
        sid = C.c_int()
        rt.check(rt.lib().syn_cache_acquire(self._h, C.byref(sid)))
        for st in self._state.values():
            st[sid.value].zero_()
        return sid.value

    def release(self, sid: int) -> None:
        rt.check(rt.lib().syn_cache_release(self._h, self._sid(sid)))

    def length(self, sid: int) -> int:
        out = C.c_long()
        rt.check(rt.lib().syn_cache_length(self._h, self._sid(sid), C.byref(out)))
        return out.value

    # ------------------------------------------------------------------ growth
    def pages_needed(self, sid: int, n_new: int) -> int:
        """Pages of the fullest-keeping group that `reserve(sid, n_new)` would take."""
        out = C.c_long()
        rt.check(rt.lib().syn_cache_pages_needed(self._h, self._sid(sid), int(n_new), C.byref(out)))
        return out.value

    def pages_for_sequence(self, total_tokens: int, longest_step: int) -> list:
        """Pages of each group that a sequence of total_tokens can hold at once when no step brings more than
        longest_step of its tokens: all its pages where every key is kept, the window's and one step's where a window
        is (a planner's bound: what `reserve` will ask for at most)."""
        out = []
        for g in self.groups:
            n = pages_for(total_tokens)
            if g.need.window is not None:
                n = min(n, pages_for(int(g.need.window) + int(longest_step)) + 1)
            out.append(n)
        return out

    def reserve(self, sid: int, n_new: int) -> None:
        """Hold pages for n_new more tokens in every group, or raise CacheFull and change nothing."""
        rt.check(rt.lib().syn_cache_reserve(self._h, self._sid(sid), int(n_new)))

    def reserve_step(self, sids: list, counts: list) -> None:
        """All pages that a step's sequences need, or CacheFull and nothing changed."""
        sids = [self._sid(s) for s in sids]
        rt.check(rt.lib().syn_cache_reserve_step(self._h, len(sids), rt.ints(sids), rt.longs([int(c) for c in counts])))

    def commit(self, sid: int, n_new: int) -> None:
        """The step has written n_new tokens; windows give back the pages that fell out of reach."""
        rt.check(rt.lib().syn_cache_commit(self._h, self._sid(sid), int(n_new)))

    # ------------------------------------------------------------------ going back
    def truncate(self, sid: int, length: int) -> None:
        """Go back to an earlier length; the positions behind it are written again by later steps.
        Enough for keys and values; a fixed-size state needs `restore` of a snapshot taken there."""
        rt.check(rt.lib().syn_cache_truncate(self._h, self._sid(sid), int(length)))

    def snapshot(self, sid: int) -> "Snapshot":
        """The sequence's length and a copy of its fixed-size states: a point to come back to.  A
        running state cannot be rewound by a length (the reference snapshots it likewise,
        crates/synaptix-models/llm/common/src/model.rs:377-492)."""
        return Snapshot(self._sid(sid), self.length(sid), {i: st[sid].clone() for i, st in self._state.items()})

    def restore(self, snap: "Snapshot") -> None:
        """Back to the snapshot's point: the length, and the states as they were there."""
        self.truncate(snap.slot, snap.length)
        for i, saved in snap.states.items():
            self._state[i][snap.slot].copy_(saved)

    def states_of(self, sids: list) -> dict:
        """Copies of the fixed-size states of these slots alone (lengths and pages are not touched)."""
        rows = torch.tensor([self._sid(s) for s in sids], dtype=torch.long, device=self.device)
        return {"rows": rows, "states": {i: st.index_select(0, rows) for i, st in self._state.items()}}

    def put_states(self, saved: dict) -> None:
        """The states as `states_of` found them."""
        for i, rows in saved["states"].items():
            self._state[i].index_copy_(0, saved["rows"], rows)

    # ------------------------------------------------------------------ what a step needs
    def table_width(self, gi: int, sids: list) -> int:
        """Logical pages of the longest of the sequences (at least 1)."""
        sids = [self._sid(s) for s in sids]
        out = C.c_int()
        rt.check(rt.lib().syn_cache_table_width(self._h, gi, rt.ints(sids), len(sids), C.byref(out)))
        return out.value

    def page_table(self, gi: int, sids: list, width: int | None = None) -> np.ndarray:
        """int32 [len(sids), width]: page of each logical page of each sequence (0 where none)."""
        w = self.table_width(gi, sids)
        if width is not None:
            if width < w:
                raise CacheError(f"page table width {width} is less than {w}")
            w = width
        out = np.zeros((len(sids), w), dtype=np.int32)
        sids = [self._sid(s) for s in sids]
        rt.check(rt.lib().syn_cache_page_table(self._h, gi, rt.ints(sids), len(sids), w, out.ctypes.data))
        return out

    def layer_view(self, i: int):
        if i in self._layer_group:
            gi = self._layer_group[i]
            g, li = self.groups[gi], self._layer_index[i]
            return KvLayerView(gi, g.k[li], g.v[li])
        if i in self._state:
            return StateLayerView(self._state[i])
        return None

    # ------------------------------------------------------------------ invariants
    def check(self) -> None:
        """No slot or page lost, held twice or free twice."""
        rt.check(rt.lib().syn_cache_check(self._h))

    def bytes_per_token(self) -> int:
        el = torch.empty(0, dtype=self.dtype).element_size()
        return sum(2 * len(g.layers) * g.need.kv_heads * g.need.head_dim * el for g in self.groups)
