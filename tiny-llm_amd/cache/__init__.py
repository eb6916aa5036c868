from .block_pool import BlockPool, CacheError, OutOfBlocks
from .manager import CacheManager, CacheGroup, RequestCache, NoFreeSlot, RELEASED
