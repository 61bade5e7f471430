from .pages import OutOfPages, PageError, PagePool, SlotPool
from .manager import CacheGroup, CacheManager, RequestCache, chain_hash, plan_groups

__all__ = ["OutOfPages", "PageError", "PagePool", "SlotPool", "CacheGroup", "CacheManager", "RequestCache",
           "chain_hash", "plan_groups"]
