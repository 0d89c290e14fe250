"""KV-cache and prefix-cache interfaces of the path (reference: mini_sglang_mlx/kvcache/base.py)."""
from __future__ import annotations

from abc import ABC, abstractmethod
from dataclasses import dataclass
from typing import NamedTuple, Tuple

import torch


class BaseKVCache(ABC):
    @abstractmethod
    def k_cache(self, index: int) -> torch.Tensor: ...

    @abstractmethod
    def v_cache(self, index: int) -> torch.Tensor: ...

    @abstractmethod
    def store_kv(self, k: torch.Tensor, v: torch.Tensor, out_loc: torch.Tensor,
                 layer_id: int) -> None: ...

    @property
    @abstractmethod
    def dtype(self) -> torch.dtype: ...

    @property
    @abstractmethod
    def num_layers(self) -> int: ...


@dataclass(frozen=True)
class BaseCacheHandle(ABC):
    """Reference: mini_sglang_mlx/kvcache/base.py:37-39."""
    cached_len: int


class SizeInfo(NamedTuple):
    """Reference: mini_sglang_mlx/kvcache/base.py:42-48."""
    evictable_size: int
    protected_size: int

    @property
    def total_size(self) -> int:
        return self.evictable_size + self.protected_size


class BaseCacheManager(ABC):
    """Prefix-cache interface (mini_sglang_mlx/kvcache/base.py:51-121).  ``input_ids`` and
    ``indices`` are 1-D int32 tensors; what comes back lives in host memory.

    The life of a request against a manager: ``match_prefix`` finds the longest cached prefix
    (nothing is pinned yet), ``lock_handle`` pins it while the request runs, ``insert_prefix``
    hands the finished request's tokens and pages to the cache, ``lock_handle(unlock=True)``
    releases the pin, and ``evict`` gives unpinned pages back when the allocator runs dry."""

    @abstractmethod
    def match_prefix(self, input_ids: torch.Tensor) -> Tuple[BaseCacheHandle, torch.Tensor]:
        """``(handle, pages)`` of the longest cached prefix of ``input_ids``; ``pages`` has
        ``handle.cached_len`` entries.  Does not change what is evictable."""

    @abstractmethod
    def insert_prefix(self, input_ids: torch.Tensor, indices: torch.Tensor) -> int:
        """Cache ``input_ids`` with the pages ``indices``; returns how many leading tokens were
        cached already (their pages in ``indices`` stay with the caller, who frees them)."""

    @abstractmethod
    def lock_handle(self, handle: BaseCacheHandle, unlock: bool = False) -> None:
        """Pin (or release) the prefix behind ``handle``: pinned pages are never evicted."""

    @abstractmethod
    def evict(self, size: int) -> torch.Tensor:
        """Give up at least ``size`` unpinned cached tokens, coldest first; returns their pages.
        Asking for more than ``size_info.evictable_size`` is an error."""

    @property
    @abstractmethod
    def size_info(self) -> SizeInfo:
        """Cached tokens that could be evicted now, and cached tokens that are pinned."""

    @abstractmethod
    def check_integrity(self) -> None:
        """Raise if the bookkeeping is inconsistent (meant for idle moments)."""

    @abstractmethod
    def reset(self) -> None:
        """Forget everything."""
