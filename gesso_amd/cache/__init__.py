from .manager import RELEASED, CacheLayout, CacheManager, PagedGroup, RequestCache, SlotMember
from .pages import PagePool, Pool, SlotPool
