from .manager import NO_PAGE, CacheManager, KVGroup, LayerCacheView
from .pages import PageAllocator
