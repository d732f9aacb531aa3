from .manager import CacheManager, LayerCache, PageGroup, RequestPages
from .pages import OutOfPages, OutOfSlots, PagePool, SlotPool
