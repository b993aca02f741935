"""Cache pages of a fixed size; the pools themselves are kept by the native runtime, one for each group of the cache.

The reference preallocates [batch, kv_heads, capacity, head_dim] for each layer and keeps one
length for the whole batch (crates/synaptix-models/llm/common/src/model.rs:349-368,998-1050).
Here sequences have lengths of their own, so storage is cut into pages of 64 tokens that
sequences take as they grow and give back when they end.
"""
from __future__ import annotations

from ..kernels.runtime import CacheFull, CacheError

PAGE_TOKENS = 64


def pages_for(n_tokens: int) -> int:
    return (n_tokens + PAGE_TOKENS - 1) // PAGE_TOKENS
