"""A pool of fixed-size cache pages: bookkeeping only, kept by the native runtime.

The reference preallocates [batch, kv_heads, capacity, head_dim] for each layer and keeps one
length for the whole batch (crates/synaptix-models/llm/common/src/model.rs:349-368,998-1050).
Here sequences have lengths of their own, so storage is cut into pages of 64 tokens that
sequences take as they grow and give back when they end.
"""
from __future__ import annotations

import ctypes as C

from ..kernels import runtime as rt
from ..kernels.runtime import CacheFull, CacheError

PAGE_TOKENS = 64


def pages_for(n_tokens: int) -> int:
    return (n_tokens + PAGE_TOKENS - 1) // PAGE_TOKENS


class PagePool:
    """A pool on its own (the cache keeps one for each of its groups inside its native state)."""

    def __init__(self, n_pages: int):
        if n_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        if rt.lib().syn_rt_page_tokens() != PAGE_TOKENS:
            raise RuntimeError("the runtime library was built for another page size")
        self.n_pages = n_pages
        self._h = rt.lib().syn_pool_new(n_pages)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            try:
                rt.lib().syn_pool_delete(h)
            except Exception:       # the interpreter is shutting down; the process's memory goes with it
                pass

    @property
    def free_pages(self) -> int:
        return rt.lib().syn_pool_free_pages(self._h)

    def take(self, n: int) -> list:
        """n pages, or CacheFull and nothing taken."""
        out = (C.c_int * max(n, 1))()
        rt.check(rt.lib().syn_pool_take(self._h, n, out))
        return list(out[:n])

    def give_back(self, pages) -> None:
        pages = [int(p) for p in pages]
        rt.check(rt.lib().syn_pool_give_back(self._h, rt.ints(pages), len(pages)))

    def check(self) -> None:
        """Every page is either free once or held: none lost, none twice."""
        rt.check(rt.lib().syn_pool_check(self._h))
