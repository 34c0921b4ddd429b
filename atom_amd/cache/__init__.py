from .kinds import (CacheKind, KVBinding, StateBinding, kind_of, register_cache_kind, unregister_cache_kind)
from .manager import CacheManager, GroupSpec, OutOfPages, OutOfSlots, PagePool, StateSlots
from .storage import CachePlan, CacheStorage, group_runs, plan_cache

__all__ = ["CacheManager", "GroupSpec", "OutOfPages", "OutOfSlots", "PagePool", "StateSlots", "CachePlan",
           "CacheStorage", "group_runs", "plan_cache", "CacheKind", "KVBinding", "StateBinding", "kind_of",
           "register_cache_kind", "unregister_cache_kind"]
