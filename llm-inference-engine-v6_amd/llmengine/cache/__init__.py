from .manager import CacheError, CacheManager, GroupSpec, PagePool
from .storage import CacheStorage, group_name, plan_groups

__all__ = ["CacheError", "CacheManager", "GroupSpec", "PagePool", "CacheStorage", "group_name", "plan_groups"]
