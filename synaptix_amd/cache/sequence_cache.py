"""The cache of the live sequences: a slot for each, keys and values for each layer that keeps
them, each sequence with its own length, and beside it a fixed-size state for each slot.

Layers with the same needs (kv heads, head size, all keys or a window of them) form a group; a
group has storage and a page pool of its own:
    k_pages [layers, pages, kv_heads, 64, head_dim]
    v_pages [layers, pages, kv_heads, head_dim, 64]      (transposed inside the page)
A group that keeps a window gives pages back as soon as every position in them has left the
window.  Layers with a StateNeed get `state[layer] : [slots, *shape]`, zeroed when a slot is
taken (the reference keeps such state in the same per-layer vector as the keys and values,
crates/synaptix-models/llm/common/src/model.rs:359-362,377-492).

A slot is taken for a sequence (`acquire`), grows with `reserve` + `commit`, and is given back
with `release`; released slots and pages are handed out again.  Stale contents are never read:
attention reads positions below the sequence's length only.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..parts.base import KvNeed, StateNeed
from .pages import PAGE_TOKENS, PagePool, CacheFull, CacheError, pages_for


@dataclass
class KvLayerView:
    """What a mixer with a KvNeed is handed for its layer."""
    group: int
    k_pages: torch.Tensor
    v_pages: torch.Tensor


@dataclass
class StateLayerView:
    """What a mixer with a StateNeed is handed: state [slots, *shape]; row = slot id."""
    state: torch.Tensor


@dataclass
class _Group:
    need: KvNeed
    layers: list                      # cache-layer indices
    pool: PagePool
    k: torch.Tensor = None
    v: torch.Tensor = None
    spare_page: int = 0               # a page beyond the pool that no sequence owns (padding rows write there)


@dataclass
class _Slot:
    live: bool = False
    length: int = 0
    reserved: int = 0                 # tokens for which pages are held (>= length)
    pages: dict = field(default_factory=dict)     # group -> list of page ids by logical page (-1: given back)


class SequenceCache:
    def __init__(self, needs: list, max_tokens: int, max_slots: int | None, dtype, device,
                 max_positions: int | None = None):
        """needs[i]: KvNeed, StateNeed or None of cache layer i.  max_tokens: the most tokens that
        live sequences hold together, each sequence's count rounded up to whole pages."""
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
        for i, need in enumerate(needs):
            if isinstance(need, KvNeed):
                for gi, g in enumerate(self.groups):
                    if g.need == need:
                        break
                else:
                    gi = len(self.groups)
                    self.groups.append(_Group(need, [], PagePool(self.n_pages)))
                self._layer_group[i] = gi
                self._layer_index[i] = len(self.groups[gi].layers)
                self.groups[gi].layers.append(i)
            elif isinstance(need, StateNeed):
                self._state[i] = torch.zeros((self.max_slots,) + tuple(need.shape), dtype=need.dtype,
                                             device=self.device)
            elif need is not None:
                raise CacheError(f"cache layer {i}: unknown need {need!r}")
        for g in self.groups:
            n, nd = len(g.layers), g.need
            # zeros: what a kernel may touch beyond a sequence's end is at least a number
            g.spare_page = self.n_pages
            g.k = torch.zeros((n, self.n_pages + 1, nd.kv_heads, PAGE_TOKENS, nd.head_dim), dtype=dtype, device=self.device)
            g.v = torch.zeros((n, self.n_pages + 1, nd.kv_heads, nd.head_dim, PAGE_TOKENS), dtype=dtype, device=self.device)
        self._slots = [_Slot() for _ in range(self.max_slots)]
        self._free_slots = list(range(self.max_slots - 1, -1, -1))

    # ------------------------------------------------------------------ slots
    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    @property
    def live_slots(self) -> list:
        return [i for i, s in enumerate(self._slots) if s.live]

    def acquire(self) -> int:
        if not self._free_slots:
            raise CacheFull(f"all {self.max_slots} slots are taken")
        sid = self._free_slots.pop()
        s = self._slots[sid]
        s.live, s.length, s.reserved = True, 0, 0
        s.pages = {gi: [] for gi in range(len(self.groups))}
        for st in self._state.values():
            st[sid].zero_()
        return sid

    def release(self, sid: int) -> None:
        s = self._slot(sid)
        for gi, pages in s.pages.items():
            self.groups[gi].pool.give_back([p for p in pages if p >= 0])
        s.live, s.length, s.reserved, s.pages = False, 0, 0, {}
        self._free_slots.append(sid)

    def _slot(self, sid: int) -> _Slot:
        if not isinstance(sid, (int, np.integer)) or not (0 <= sid < self.max_slots) or not self._slots[sid].live:
            raise CacheError(f"slot {sid!r} is not live")
        return self._slots[sid]

    def length(self, sid: int) -> int:
        return self._slot(sid).length

    # ------------------------------------------------------------------ growth
    def pages_needed(self, sid: int, n_new: int) -> int:
        """Pages of the fullest-keeping group that `reserve(sid, n_new)` would take."""
        s = self._slot(sid)
        return max(0, pages_for(s.length + n_new) - pages_for(s.reserved))

    def reserve(self, sid: int, n_new: int) -> None:
        """Hold pages for n_new more tokens in every group, or raise CacheFull and change nothing."""
        s = self._slot(sid)
        if n_new <= 0:
            raise CacheError("a step brings at least one token for each of its sequences")
        total = s.length + n_new
        if self.max_positions is not None and total > self.max_positions:
            raise CacheError(f"KV overflow: {s.length} + {n_new} tokens exceed the position range {self.max_positions}")
        want = pages_for(total) - pages_for(s.reserved)
        if want > 0:
            for g in self.groups:
                if g.pool.free_pages < want:
                    raise CacheFull(f"{want} pages wanted, {g.pool.free_pages} of {g.pool.n_pages} free")
            for gi, g in enumerate(self.groups):
                s.pages[gi].extend(g.pool.take(want))
        s.reserved = max(s.reserved, total)

    def commit(self, sid: int, n_new: int) -> None:
        """The step has written n_new tokens; windows give back the pages that fell out of reach."""
        s = self._slot(sid)
        if s.length + n_new > s.reserved:
            raise CacheError("commit without reserve")
        s.length += n_new
        for gi, g in enumerate(self.groups):
            w = g.need.window
            if w is None:
                continue
            # the next query sits at position `length`; it sees keys > length - w
            first_needed = max(0, s.length - w + 1) // PAGE_TOKENS
            pages = s.pages[gi]
            gone = [p for p in pages[:first_needed] if p >= 0]
            if gone:
                g.pool.give_back(gone)
                for i in range(first_needed):
                    pages[i] = -1

    # ------------------------------------------------------------------ what a step needs
    def page_table(self, gi: int, sids: list, width: int | None = None) -> np.ndarray:
        """int32 [len(sids), width]: page of each logical page of each sequence (0 where none)."""
        rows = [self._slot(sid).pages[gi] for sid in sids]
        w = max([len(r) for r in rows] + [1])
        if width is not None:
            if width < w:
                raise CacheError(f"page table width {width} is less than {w}")
            w = width
        out = np.zeros((len(sids), w), dtype=np.int32)
        for i, r in enumerate(rows):
            out[i, :len(r)] = [max(p, 0) for p in r]
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
        free = set(self._free_slots)
        if len(free) != len(self._free_slots):
            raise CacheError("a slot is in the free list twice")
        for i, s in enumerate(self._slots):
            if s.live == (i in free):
                raise CacheError(f"slot {i} is {'both live and free' if s.live else 'lost'}")
        for gi, g in enumerate(self.groups):
            g.pool.check()
            held = [p for s in self._slots if s.live for p in s.pages[gi] if p >= 0]
            if len(held) != len(set(held)):
                raise CacheError(f"group {gi}: a page is held by two sequences")
            if len(held) + g.pool.free_pages != g.pool.n_pages:
                raise CacheError(f"group {gi}: {g.pool.n_pages - len(held) - g.pool.free_pages} pages lost")

    def bytes_per_token(self) -> int:
        el = torch.empty(0, dtype=self.dtype).element_size()
        return sum(2 * len(g.layers) * g.need.kv_heads * g.need.head_dim * el for g in self.groups)
