"""Cache manager: pages, block tables, cache groups and fixed-size state slots."""
from .device import DeviceCache, LayerCache
from .manager import NO_PAGE, CacheManager
from .needs import CacheNeed, StateNeed
from .pages import PageError, PagePool
