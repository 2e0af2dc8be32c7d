from .slots import CacheError, FreeList, GroupPages, SlotBook   # noqa: F401
from .store import CacheSite, ModelCache, StateSpec, TokenSpec   # noqa: F401
