from tokasaurus_amd.cache.manager import RELEASED, CacheGroup, CacheManager, RequestCache, plan_groups  # noqa: F401
from tokasaurus_amd.cache.pages import NoSpaceException, PagePool, SlotAllocator  # noqa: F401
