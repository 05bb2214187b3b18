from .pages import PAGE_TOKENS, CacheFull, PagePool, pages_for
from .sequence_cache import KVGroup, KVNeed, SequenceCache, StateNeed

__all__ = ["PAGE_TOKENS", "CacheFull", "PagePool", "pages_for", "KVGroup", "KVNeed", "SequenceCache", "StateNeed"]
