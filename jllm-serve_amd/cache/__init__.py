"""Pages, block tables and state slots."""
from .pages import OutOfPages, PagePool
from .manager import CacheEntryPlan, CacheManager, KvSpec, LayerSlot, StateSpec

__all__ = ["OutOfPages", "PagePool", "CacheEntryPlan", "CacheManager", "KvSpec", "LayerSlot", "StateSpec"]
