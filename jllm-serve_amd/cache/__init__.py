"""Pages, block tables and state slots."""
from .pages import OutOfPages, PagePool
from .manager import CacheEntryPlan, CacheManager, CacheRow, KvSpec, LayerSlot, PageSpec, StateSpec

__all__ = ["OutOfPages", "PagePool", "CacheEntryPlan", "CacheManager", "CacheRow", "KvSpec", "LayerSlot", "PageSpec", "StateSpec"]
