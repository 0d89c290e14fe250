"""Per-layer slot-indexed K and V pools (reference: mini_sglang_mlx/kvcache/mha_pool.py:10-56).

Each layer owns two ``(num_pages, num_kv_heads, head_dim)`` tensors in HBM; "page" here is the
reference's word for a token slot.  ``store_kv`` is the only writer and goes through the
``store_kv_cache`` kernel.  Unlike the reference there is no host synchronisation before the
store (mha_pool.py:47 forces its lazy inputs): launches are stream-ordered.
"""
from __future__ import annotations

import torch

from mini_sglang_amd_kernel import store_kv_cache

from .base import BaseKVCache


class MHAKVCache(BaseKVCache):
    def __init__(self, num_kv_heads: int, num_layers: int, head_dim: int, num_pages: int,
                 dtype: torch.dtype, device="cuda"):
        self._num_layers = num_layers
        shape = (num_pages, num_kv_heads, head_dim)
        self._k_buffer = [torch.zeros(shape, dtype=dtype, device=device) for _ in range(num_layers)]
        self._v_buffer = [torch.zeros(shape, dtype=dtype, device=device) for _ in range(num_layers)]
        self._storage_shape = shape
        self._dtype = dtype

    def k_cache(self, index: int) -> torch.Tensor:
        return self._k_buffer[index]

    def v_cache(self, index: int) -> torch.Tensor:
        return self._v_buffer[index]

    def store_kv(self, k: torch.Tensor, v: torch.Tensor, out_loc: torch.Tensor,
                 layer_id: int) -> None:
        assert out_loc.dtype == torch.int32, "out_loc must be int32"
        k_cache = self._k_buffer[layer_id]
        v_cache = self._v_buffer[layer_id]
        if len(out_loc) != k.shape[0] or len(out_loc) != v.shape[0]:
            raise ValueError(
                f"store_kv shape mismatch: len(out_loc)={len(out_loc)}, "
                f"k.shape={tuple(k.shape)}, v.shape={tuple(v.shape)}"
            )
        store_kv_cache(k_cache=k_cache, v_cache=v_cache, indices=out_loc, k=k, v=v)

    @property
    def dtype(self) -> torch.dtype:
        # the reference's property reads a nonexistent attribute (mha_pool.py:50-52);
        # this one answers
        return self._dtype

    @property
    def num_layers(self) -> int:
        return self._num_layers
