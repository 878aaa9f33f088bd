from .cache import (Cache, CacheGroup, CacheLineView, Geometry, KVGroup, PAGE_SIZE, PagedGroup, SlotAllocator,
                    StateGroup, pages_for, register_cache_group)
