from .manager import CacheGroup, CacheManager, RequestCache
from .page_pool import NULL_PAGE, OutOfPages, PagePool, chain_hash
from .state_slots import OutOfSlots, StateSlotPool

__all__ = ["CacheGroup", "CacheManager", "RequestCache", "NULL_PAGE", "OutOfPages", "PagePool", "chain_hash",
           "OutOfSlots", "StateSlotPool"]
