from .manager import (RESERVE_NEVER_FITS, RESERVE_NO_PAGES, RESERVE_NO_SLOT, RESERVE_OK, CacheGroupSpec,
                      CacheManager)
from .storage import CacheStorage, PagedKV, cache_bytes, group_keys, group_position_bytes, plan_groups

__all__ = ["RESERVE_NEVER_FITS", "RESERVE_NO_PAGES", "RESERVE_NO_SLOT", "RESERVE_OK", "CacheGroupSpec",
           "CacheManager", "CacheStorage", "PagedKV", "cache_bytes", "group_keys", "group_position_bytes", "plan_groups"]
