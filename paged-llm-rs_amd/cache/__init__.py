from .layout import CacheGroupLayout, CacheLayout, KVCacheSpec, StateSpec
from .manager import BlockPool, CacheManager, GroupGeometry, block_hash
from .pools import LayerKV, PagedCache

__all__ = ["CacheGroupLayout", "CacheLayout", "KVCacheSpec", "StateSpec", "BlockPool", "CacheManager",
           "GroupGeometry", "block_hash", "LayerKV", "PagedCache"]
