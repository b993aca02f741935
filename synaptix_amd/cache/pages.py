"""A pool of fixed-size cache pages: host-side bookkeeping only.

The reference preallocates [batch, kv_heads, capacity, head_dim] for each layer and keeps one
length for the whole batch (crates/synaptix-models/llm/common/src/model.rs:349-368,998-1050).
Here sequences have lengths of their own, so storage is cut into pages of 64 tokens that
sequences take as they grow and give back when they end.
"""
from __future__ import annotations

PAGE_TOKENS = 64


class CacheFull(RuntimeError):
    """No free page (or slot) is left; nothing was taken."""


class CacheError(RuntimeError):
    """A misuse of the cache: unknown slot, double release, overflow of the position range."""


def pages_for(n_tokens: int) -> int:
    return (n_tokens + PAGE_TOKENS - 1) // PAGE_TOKENS


class PagePool:
    def __init__(self, n_pages: int):
        if n_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.n_pages = n_pages
        self._free = list(range(n_pages - 1, -1, -1))   # pop() hands out 0, 1, 2, ... first
        self._held = [False] * n_pages

    @property
    def free_pages(self) -> int:
        return len(self._free)

    def take(self, n: int) -> list:
        """n pages, or CacheFull and nothing taken."""
        if n > len(self._free):
            raise CacheFull(f"{n} pages wanted, {len(self._free)} of {self.n_pages} free")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._held[p] = True
        return out

    def give_back(self, pages) -> None:
        for p in pages:
            if not (0 <= p < self.n_pages) or not self._held[p]:
                raise CacheError(f"page {p} is not held")
            self._held[p] = False
            self._free.append(p)

    def check(self) -> None:
        """Every page is either free once or held: none lost, none twice."""
        seen = set(self._free)
        if len(seen) != len(self._free):
            raise CacheError("a page is in the free list twice")
        for p in range(self.n_pages):
            if self._held[p] == (p in seen):
                raise CacheError(f"page {p} is {'both held and free' if self._held[p] else 'lost'}")
