"""Cache manager: pages, block tables, cache groups and fixed-size state slots."""
from .device import DeviceCache, LayerCache
from .manager import NO_PAGE, CacheManager, PageError
from .needs import CacheNeed, StateNeed
