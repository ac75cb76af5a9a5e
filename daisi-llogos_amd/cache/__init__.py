from .pages import PAGE_TOKENS, CacheError, CacheFull, GroupPages, PagePool, SlotAllocator, pages_for
from .kv_cache import Cache, KVGroup
