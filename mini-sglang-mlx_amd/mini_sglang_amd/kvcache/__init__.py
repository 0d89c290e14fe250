from .base import BaseCacheHandle, BaseCacheManager, BaseKVCache, SizeInfo
from .mha_pool import MHAKVCache
from .radix_manager import (HybridCacheHandle, HybridRadixCacheManager, RadixCacheHandle,
                            RadixCacheManager, RadixTreeNode)

__all__ = ["BaseKVCache", "MHAKVCache", "BaseCacheHandle", "BaseCacheManager", "SizeInfo",
           "RadixTreeNode", "RadixCacheHandle", "RadixCacheManager", "HybridCacheHandle",
           "HybridRadixCacheManager"]
