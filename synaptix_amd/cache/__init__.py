from .pages import PAGE_TOKENS, CacheFull, CacheError, pages_for
from .sequence_cache import SequenceCache, KvLayerView, StateLayerView, Snapshot

__all__ = ["PAGE_TOKENS", "CacheFull", "CacheError", "pages_for", "SequenceCache", "Snapshot", "KvLayerView",
           "StateLayerView"]
