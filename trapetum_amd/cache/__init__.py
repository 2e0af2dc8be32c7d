from .slots import CacheError, FreeList, GroupPages, SlotBook   # noqa: F401
from .store import CacheSite, KVSpec, ModelCache, StateSpec   # noqa: F401
