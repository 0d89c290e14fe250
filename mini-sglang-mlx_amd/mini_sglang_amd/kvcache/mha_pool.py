"""Slot-indexed K and V pools of all layers, laid out for one large HBM allocation each.

Counterpart of ``MHAKVCache`` (mini_sglang_mlx/kvcache/mha_pool.py:10-56): same constructor
arguments, ``k_cache(i)`` / ``v_cache(i)`` / ``store_kv`` / ``dtype`` / ``num_layers``.  "Page" is the
reference's word for a token slot.

Layout: K of every layer lives in one ``(num_layers, num_pages, num_kv_heads, head_dim)`` slab and
V in another (the reference keeps ``2 * num_layers`` separate arrays); a layer's pool is the view
``slab[i]``, whose slot stride is ``num_kv_heads * head_dim`` elements, the contiguous layout the
kernels take at full speed.  The slabs are zero-filled once at construction, as the reference's are.
``store_kv`` is the only writer and goes through the ``store_kv_cache`` kernel; there is no host
synchronisation before it (the reference forces its lazy inputs there, mha_pool.py:47): launches
are ordered by the stream.
"""
from __future__ import annotations

from typing import Tuple

import torch

from mini_sglang_amd_kernel import store_kv_cache

from .base import BaseKVCache


class MHAKVCache(BaseKVCache):
    def __init__(self, num_kv_heads: int, num_layers: int, head_dim: int, num_pages: int,
                 dtype: torch.dtype, device="cuda"):
        if min(num_kv_heads, num_layers, head_dim, num_pages) <= 0:
            raise ValueError("MHAKVCache: every dimension must be positive")
        slab = (num_layers, num_pages, num_kv_heads, head_dim)
        self._k_slab = torch.zeros(slab, dtype=dtype, device=device)
        self._v_slab = torch.zeros(slab, dtype=dtype, device=device)

    # ---- the reference's surface -----------------------------------------------------------
    def k_cache(self, index: int) -> torch.Tensor:
        return self._k_slab[index]

    def v_cache(self, index: int) -> torch.Tensor:
        return self._v_slab[index]

    def store_kv(self, k: torch.Tensor, v: torch.Tensor, out_loc: torch.Tensor,
                 layer_id: int) -> None:
        """``pool[layer_id][out_loc[r]] = k[r]`` (and v): one kernel launch, bit copy."""
        assert out_loc.dtype == torch.int32, "out_loc must be int32"
        rows = out_loc.shape[0]
        if k.shape[0] != rows or v.shape[0] != rows:
            raise ValueError(f"store_kv: {rows} slot ids for k of shape {tuple(k.shape)} and v of "
                             f"shape {tuple(v.shape)}")
        store_kv_cache(self._k_slab[layer_id], self._v_slab[layer_id], out_loc, k, v)

    @property
    def dtype(self) -> torch.dtype:
        # the reference's property reads an attribute that does not exist (mha_pool.py:50-52)
        return self._k_slab.dtype

    @property
    def num_layers(self) -> int:
        return self._k_slab.shape[0]

    # ---- extras ----------------------------------------------------------------------------
    @property
    def pool_shape(self) -> Tuple[int, int, int]:
        """``(num_pages, num_kv_heads, head_dim)`` of one layer's pool."""
        return tuple(self._k_slab.shape[1:])

    @property
    def nbytes(self) -> int:
        """HBM held by both slabs."""
        return 2 * self._k_slab.numel() * self._k_slab.element_size()
