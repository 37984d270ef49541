from .pages import KVNeed, StateNeed, OutOfPages, PagePool, CacheGroup
from .state import StateSlots
from .manager import CacheManager, Appended, pages_that_fit
