from .manager import CacheError, CacheManager, GroupConfig, OutOfPages, PagePool, RELEASED, RequestCache
from .storage import CacheStorage, GroupLayout, bytes_per_token, plan_groups

__all__ = ["CacheError", "CacheManager", "GroupConfig", "OutOfPages", "PagePool", "RELEASED", "RequestCache",
           "CacheStorage", "GroupLayout", "bytes_per_token", "plan_groups"]
