"""Pools and prefix caches either side of the attention path, plus the reference's factory
functions (mini_sglang_mlx/kvcache/__init__.py:28-83)."""
from __future__ import annotations

from typing import Callable, Dict, Tuple

import torch

from .base import BaseCacheHandle, BaseCacheManager, BaseKVCache, SizeInfo
from .mamba_pool import MambaStateConfig, MambaStatePool, MambaStateShape
from .mha_pool import MHAKVCache
from .radix_manager import (HybridCacheHandle, HybridRadixCacheManager, RadixCacheHandle,
                            RadixCacheManager, RadixTreeNode)


class NaiveCacheHandle(BaseCacheHandle):
    pass


class NaiveCacheManager(BaseCacheManager):
    """The manager for "no prefix caching" (reference: mini_sglang_mlx/kvcache/naive_manager.py:14-44).
    Nothing is ever remembered, so nothing matches, nothing is locked and there is nothing to
    evict: asking for more than zero evicted tokens is an error, as in the reference."""

    _NOTHING = torch.empty(0, dtype=torch.int32)
    size_info = property(lambda self: SizeInfo(evictable_size=0, protected_size=0))

    def __init__(self, device=None):
        del device

    def match_prefix(self, input_ids: torch.Tensor) -> Tuple[NaiveCacheHandle, torch.Tensor]:
        return NaiveCacheHandle(cached_len=0), self._NOTHING

    def insert_prefix(self, input_ids: torch.Tensor, indices: torch.Tensor) -> int:
        n = len(indices)
        assert n == len(input_ids)
        return n  # "already cached": the caller keeps ownership of none of the pages

    def evict(self, size: int) -> torch.Tensor:
        if size != 0:
            raise NotImplementedError("NaiveCacheManager does not support eviction.")
        return self._NOTHING

    def lock_handle(self, handle: BaseCacheHandle, unlock: bool = False) -> None:
        return None

    def reset(self) -> None:
        return None

    def check_integrity(self) -> None:
        return None


def create_kvcache(model_config, num_pages: int, dtype: torch.dtype, device="cuda") -> BaseKVCache:
    """K/V pools for a model described by ``num_kv_heads`` / ``num_layers`` / ``head_dim``."""
    return MHAKVCache(num_kv_heads=model_config.num_kv_heads, num_layers=model_config.num_layers,
                      head_dim=model_config.head_dim, num_pages=num_pages, dtype=dtype, device=device)


SUPPORTED_CACHE_MANAGER: Dict[str, Callable[..., BaseCacheManager]] = {
    "naive": lambda device=None: NaiveCacheManager(device=device),
    "radix": lambda device=None: RadixCacheManager(device=device),
}


def create_cache_manager(device=None, type: str = "naive") -> BaseCacheManager:
    if type not in SUPPORTED_CACHE_MANAGER:
        raise KeyError(f"Unsupported Cache Manager: {type!r}; known: {sorted(SUPPORTED_CACHE_MANAGER)}")
    return SUPPORTED_CACHE_MANAGER[type](device)


def create_hybrid_radix_cache_manager(mamba_pool: MambaStatePool, device=None) -> BaseCacheManager:
    return HybridRadixCacheManager(mamba_pool=mamba_pool, device=device)


__all__ = ["BaseKVCache", "MHAKVCache", "BaseCacheHandle", "BaseCacheManager", "SizeInfo",
           "RadixTreeNode", "RadixCacheHandle", "RadixCacheManager", "HybridCacheHandle",
           "HybridRadixCacheManager", "NaiveCacheHandle", "NaiveCacheManager", "MambaStateShape",
           "MambaStateConfig", "MambaStatePool", "create_kvcache", "create_cache_manager",
           "create_hybrid_radix_cache_manager", "SUPPORTED_CACHE_MANAGER"]
