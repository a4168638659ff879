"""The paged cache: page tables and state slots (manager) and their device memory (pool)."""
from .manager import CacheError, CacheManager, GroupGeometry, OutOfPages
from .pool import CachePlan, CachePool, GroupPlan, LayerCache, pages_for_memory, pages_for_tokens, plan_cache

__all__ = ["CacheError", "CacheManager", "GroupGeometry", "OutOfPages", "CachePlan", "CachePool", "GroupPlan",
           "LayerCache", "pages_for_memory", "pages_for_tokens", "plan_cache"]
