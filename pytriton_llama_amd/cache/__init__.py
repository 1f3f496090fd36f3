from .manager import RELEASED, CacheManager, OutOfPages, OutOfSlots, PagedGroup, PagePool, StateGroup
from .storage import CacheStorage, PagedLayerView, StateLayerView
