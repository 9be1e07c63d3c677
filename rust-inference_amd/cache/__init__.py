from .cache import PAGE_SIZE, UNMAPPED, Cache, KVGroup, KVNeed, KVView, StateNeed
from .pages import PagePool
from .slots import SlotAllocator

__all__ = ["Cache", "KVGroup", "KVNeed", "KVView", "StateNeed", "PagePool", "SlotAllocator", "PAGE_SIZE", "UNMAPPED"]
