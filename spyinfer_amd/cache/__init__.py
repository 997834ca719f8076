from .manager import CacheManager, OutOfSlots, PageGroup, RequestCache, SlotPool, StateGroup
from .pages import OutOfPages, PagePool
from .spec import CacheKind, FixedState, PagedKV, PagedKVLayer, StateLayer
