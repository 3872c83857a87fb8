from .manager import (RELEASED, CacheError, CacheManager, GroupInfo, OutOfPages, PagePool,
                      SequenceCache, SlotPool, group_layers)
from .storage import CacheStorage, LayerCache
