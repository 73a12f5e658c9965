from .manager import CacheManager, KVCacheView, OutOfPages, OutOfSlots, RequestCache
from .needs import KVNeed, StateNeed
from .pool import PagePool, PoolStats, chain_hash
