from .cache import Cache, CacheLineView, KVGroup, PAGE_SIZE, SlotAllocator, StateGroup, pages_for

__all__ = ["Cache", "CacheLineView", "KVGroup", "PAGE_SIZE", "SlotAllocator", "StateGroup", "pages_for"]
