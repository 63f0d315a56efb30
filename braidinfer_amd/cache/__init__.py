from .allocator import PagePool, SlotAllocator
from .kv_cache import CacheNeed, StateNeed, CacheGroup, SequenceCache, PAGE_TOKENS

__all__ = ["PagePool", "SlotAllocator", "CacheNeed", "StateNeed", "CacheGroup", "SequenceCache", "PAGE_TOKENS"]
