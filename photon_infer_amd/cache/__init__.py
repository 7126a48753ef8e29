from .manager import CacheManager
from .pages import PagePool
from .state_slots import StateSlots

__all__ = ["CacheManager", "PagePool", "StateSlots"]
