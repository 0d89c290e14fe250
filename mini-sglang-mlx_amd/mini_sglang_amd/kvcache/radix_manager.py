"""Radix prefix cache: the producer of the prefix lengths and slot ids the attention path reads.

Mirror of ``mini_sglang_mlx/kvcache/radix_manager.py`` (``RadixTreeNode``, ``RadixCacheHandle``,
``RadixCacheManager``, ``HybridCacheHandle``, ``HybridRadixCacheManager``): same names, argument
meaning, return values and assertion texts.  The tree itself lives in the native library (C ABI
in ``include/msgl_radix_cache.h``); the classes here are views over it.  Token ids and slot ids
are int32 tensors; a tensor on a GPU is copied to the host on the way in (a synchronising
copy) and results are host tensors, which the caller moves where the page table lives.

The mamba pool of the hybrid manager is whatever object the caller brings: it needs
``free(slot)`` and ``check_ownership(slots)`` (mamba_pool.py:107-162).
"""
from __future__ import annotations

import ctypes
import time
from dataclasses import dataclass
from typing import Dict, Iterator, List, Optional, Tuple

import torch

from mini_sglang_amd_kernel import _lib

from .base import BaseCacheHandle, BaseCacheManager, SizeInfo

_ROOT = 0
_NO_SLOT = -1
_ERR_NODE = -1
_ERR_SNAPSHOT_ON_ROOT = -3
_ERR_REF_COUNT = -4
_ERR_CANNOT_EVICT = -5


def _host_i32(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dtype != torch.int32:
        raise TypeError(f"{name} must be int32, got {t.dtype}")
    t = t.reshape(-1)
    if t.device.type != "cpu":
        t = t.cpu()
    return t if t.is_contiguous() else t.contiguous()


def _ptr(t: torch.Tensor):
    return t.data_ptr() if t.numel() else None


class _Children:
    """``node.children``: first token of a child's key -> child, in insertion order."""

    def __init__(self, owner: "RadixTreeNode") -> None:
        self._owner = owner

    def _pairs(self) -> List[Tuple[int, int]]:
        tree = self._owner._tree
        n = tree._lib.msgl_radix_node_children(tree._handle, self._owner._id, None, None, 0)
        tree._check_node(n)
        toks = (ctypes.c_int32 * max(n, 1))()
        ids = (ctypes.c_int64 * max(n, 1))()
        tree._lib.msgl_radix_node_children(tree._handle, self._owner._id, toks, ids, n)
        return [(int(toks[i]), int(ids[i])) for i in range(n)]

    def __len__(self) -> int:
        return self._owner._info()[5]

    def __contains__(self, token: int) -> bool:
        tree = self._owner._tree
        return tree._lib.msgl_radix_node_child(tree._handle, self._owner._id, int(token)) >= 0

    def __getitem__(self, token: int) -> "RadixTreeNode":
        tree = self._owner._tree
        cid = tree._lib.msgl_radix_node_child(tree._handle, self._owner._id, int(token))
        if cid < 0:
            raise KeyError(token)
        return tree._node(cid)

    def __iter__(self) -> Iterator[int]:
        return iter(t for t, _ in self._pairs())

    def keys(self):
        return [t for t, _ in self._pairs()]

    def values(self) -> List["RadixTreeNode"]:
        return [self._owner._tree._node(i) for _, i in self._pairs()]

    def items(self):
        return [(t, self._owner._tree._node(i)) for t, i in self._pairs()]


class RadixTreeNode:
    """View of one node of the native tree (reference: radix_manager.py:18-90).  The manager
    hands out one object per node, so ``is`` compares nodes."""

    def __init__(self, tree: "_NativeTree", node_id: int) -> None:
        self._tree = tree
        self._id = node_id
        self.children = _Children(self)

    def _info(self) -> Tuple[int, int, int, int, int, int]:
        parent, length, ts, nch = (ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64(),
                                   ctypes.c_int64())
        ref, slot = ctypes.c_int32(), ctypes.c_int32()
        rc = self._tree._lib.msgl_radix_node_info(
            self._tree._handle, self._id, ctypes.byref(parent), ctypes.byref(length),
            ctypes.byref(ref), ctypes.byref(ts), ctypes.byref(slot), ctypes.byref(nch))
        self._tree._check_node(rc)
        return parent.value, length.value, ref.value, ts.value, slot.value, nch.value

    @property
    def uuid(self) -> int:
        return self._id

    @property
    def length(self) -> int:
        return self._info()[1]

    @property
    def parent(self) -> "RadixTreeNode":
        p = self._info()[0]
        assert p >= 0
        return self._tree._node(p)

    @property
    def ref_count(self) -> int:
        return self._info()[2]

    @property
    def timestamp(self) -> int:
        return self._info()[3]

    @timestamp.setter
    def timestamp(self, value: int) -> None:
        self._tree._check_node(self._tree._lib.msgl_radix_node_set(self._tree._handle, self._id, 0,
                                                                   int(value)))

    @property
    def mamba_slot(self) -> Optional[int]:
        s = self._info()[4]
        return None if s == _NO_SLOT else s

    @mamba_slot.setter
    def mamba_slot(self, value: Optional[int]) -> None:
        self._tree._check_node(self._tree._lib.msgl_radix_node_set(
            self._tree._handle, self._id, 1, _NO_SLOT if value is None else int(value)))

    def _key_value(self) -> Tuple[torch.Tensor, torch.Tensor]:
        n = self.length
        key = torch.empty(n, dtype=torch.int32)
        value = torch.empty(n, dtype=torch.int32)
        self._tree._lib.msgl_radix_node_key_value(self._tree._handle, self._id, _ptr(key),
                                                  _ptr(value), n)
        return key, value

    @property
    def _key(self) -> torch.Tensor:
        return self._key_value()[0]

    @property
    def value(self) -> torch.Tensor:
        return self._key_value()[1]

    def is_root(self) -> bool:
        return self._id == _ROOT

    def is_leaf(self) -> bool:
        return self._info()[5] == 0

    def get_match_len(self, input_ids: torch.Tensor) -> int:
        from mini_sglang_amd_kernel import fast_compare_key

        return fast_compare_key(self._key, _host_i32(input_ids, "input_ids"))

    def __lt__(self, other: "RadixTreeNode") -> bool:
        return self.timestamp < other.timestamp

    def __repr__(self) -> str:
        return f"RadixTreeNode(uuid={self._id})"


class _NativeTree:
    """Owner of one ``msgl_radix_*`` tree handle and of the node views handed out for it."""

    def __init__(self) -> None:
        self._lib = _lib.load()
        self._handle = self._lib.msgl_radix_create()
        if not self._handle:
            raise MemoryError("msgl_radix_create failed")
        self._views: Dict[int, RadixTreeNode] = {}

    def __del__(self) -> None:
        handle, self._handle = getattr(self, "_handle", None), None
        if handle:
            self._lib.msgl_radix_destroy(handle)

    def _check_node(self, rc: int) -> None:
        if rc == _ERR_NODE:
            raise KeyError("the node is no longer part of the tree")
        if rc < 0:
            raise RuntimeError(f"radix tree call failed with code {rc}")

    def _node(self, node_id: int) -> RadixTreeNode:
        view = self._views.get(node_id)
        if view is None:
            view = self._views[node_id] = RadixTreeNode(self, node_id)
        return view

    def _forget_dead_views(self) -> None:
        dead = [i for i in self._views
                if self._lib.msgl_radix_node_info(self._handle, i, None, None, None, None, None,
                                                  None) < 0]
        for i in dead:
            del self._views[i]


@dataclass(frozen=True)
class RadixCacheHandle(BaseCacheHandle):
    node: RadixTreeNode


class RadixCacheManager(BaseCacheManager):
    """Reference: radix_manager.py:98-275."""

    def __init__(self, device=None):
        del device  # the tree is host-side whatever device the pools live on
        self.empty_tensor = torch.empty(0, dtype=torch.int32)
        super().__init__()
        self._tree = _NativeTree()
        self.root_node = self._tree._node(_ROOT)
        self.clock = time.monotonic_ns  # timestamps of the LRU order; replaceable for replay

    # sizes live in the native tree; these read through
    @property
    def evictable_size(self) -> int:
        return self.size_info.evictable_size

    @property
    def protected_size(self) -> int:
        return self.size_info.protected_size

    def lock_handle(self, handle: BaseCacheHandle, unlock: bool = False) -> None:
        assert isinstance(handle, (RadixCacheHandle, HybridCacheHandle))
        rc = self._tree._lib.msgl_radix_lock(self._tree._handle, handle.node._id, int(bool(unlock)))
        assert rc != _ERR_REF_COUNT, "unlock of a handle that is not locked"
        self._tree._check_node(rc)

    def _walk(self, input_ids: torch.Tensor) -> Tuple[RadixTreeNode, int]:
        ids = _host_i32(input_ids, "input_ids")
        node = ctypes.c_int64()
        prefix_len = self._tree._lib.msgl_radix_walk(self._tree._handle, _ptr(ids), ids.numel(),
                                                     self.clock(), ctypes.byref(node))
        self._tree._check_node(prefix_len)
        return self._tree._node(node.value), int(prefix_len)

    def _path_values(self, node: RadixTreeNode) -> torch.Tensor:
        n = self._tree._lib.msgl_radix_path_values(self._tree._handle, node._id, None, 0)
        self._tree._check_node(n)
        out = torch.empty(n, dtype=torch.int32)
        self._tree._lib.msgl_radix_path_values(self._tree._handle, node._id, _ptr(out), n)
        return out

    def match_prefix(self, input_ids: torch.Tensor) -> Tuple[RadixCacheHandle, torch.Tensor]:
        node, prefix_len = self._walk(input_ids)
        if prefix_len == 0:
            assert node.is_root() and node is self.root_node and prefix_len == 0
            return RadixCacheHandle(prefix_len, node), self.empty_tensor
        return RadixCacheHandle(prefix_len, node), self._path_values(node)

    def _insert(self, input_ids: torch.Tensor, indices: torch.Tensor,
                mamba_slot: Optional[int]) -> Tuple[int, Optional[int]]:
        ids = _host_i32(input_ids, "input_ids")
        idx = _host_i32(indices, "indices")
        assert idx.numel() >= ids.numel(), "indices must cover input_ids"
        to_free = ctypes.c_int32(_NO_SLOT)
        rc = self._tree._lib.msgl_radix_insert(
            self._tree._handle, _ptr(ids), _ptr(idx), ids.numel(),
            _NO_SLOT if mamba_slot is None else int(mamba_slot), self.clock(),
            ctypes.byref(to_free))
        assert rc != _ERR_SNAPSHOT_ON_ROOT, "cannot store a snapshot on the root"
        self._tree._check_node(rc)
        return int(rc), (None if to_free.value == _NO_SLOT else to_free.value)

    def insert_prefix(self, input_ids: torch.Tensor, indices: torch.Tensor) -> int:
        return self._insert(input_ids, indices, None)[0]

    def _release_node_state(self, node: RadixTreeNode) -> int:
        """What a node holds besides its pages: nothing in the plain tree
        (radix_manager.py:181-189)."""
        del node
        return 0

    def _release_slots(self, slots: List[int]) -> None:
        assert not slots, "a plain radix tree holds no snapshots"

    def _evict_leaves(self, size: int = 0, num_slots: int = 0) -> Tuple[torch.Tensor, int]:
        n_slots = ctypes.c_int64()
        n = self._tree._lib.msgl_radix_evict(self._tree._handle, int(size), int(num_slots),
                                             ctypes.byref(n_slots))
        assert n != _ERR_CANNOT_EVICT, (
            f"Cannot evict enough cache, need {size}, only {self.evictable_size} evictable")
        self._tree._check_node(n)
        indices = torch.empty(n, dtype=torch.int32) if n else self.empty_tensor
        slots = (ctypes.c_int32 * max(n_slots.value, 1))()
        self._tree._check_node(self._tree._lib.msgl_radix_evicted(
            self._tree._handle, _ptr(indices), n, slots, n_slots.value))
        self._release_slots([int(slots[i]) for i in range(n_slots.value)])
        self._tree._forget_dead_views()
        return indices, n_slots.value

    def evict(self, size: int) -> torch.Tensor:
        if size == 0:
            return self.empty_tensor
        assert (
            size <= self.evictable_size
        ), f"Cannot evict {size}, only {self.evictable_size} is evictable"
        indices, _ = self._evict_leaves(size=size)
        return indices

    def reset(self) -> None:
        raise NotImplementedError("RadixManager.reset is not implemented")

    @property
    def size_info(self) -> SizeInfo:
        ev, pr = ctypes.c_int64(), ctypes.c_int64()
        self._tree._lib.msgl_radix_sizes(self._tree._handle, ctypes.byref(ev), ctypes.byref(pr))
        return SizeInfo(evictable_size=ev.value, protected_size=pr.value)

    def check_integrity(self) -> None:
        pass


@dataclass(frozen=True)
class HybridCacheHandle(BaseCacheHandle):
    """``node`` is the deepest matched node that carries a mamba snapshot; ``cached_len > 0`` iff
    there is one (reference: radix_manager.py:281-296)."""

    node: RadixTreeNode


class HybridRadixCacheManager(RadixCacheManager):
    """Radix cache that also keeps, per node, the slot of the recurrent state at that node's end
    (reference: radix_manager.py:299-452)."""

    def __init__(self, mamba_pool, device=None) -> None:
        super().__init__(device=device)
        self.mamba_pool = mamba_pool

    def match_prefix(self, input_ids: torch.Tensor) -> Tuple[HybridCacheHandle, torch.Tensor]:
        node, prefix_len = self._walk(input_ids)
        mamba_node, mamba_depth = self._find_mamba_ancestor(node, prefix_len)
        if mamba_node.mamba_slot is None or mamba_depth == 0:
            return HybridCacheHandle(0, self.root_node), self.empty_tensor
        return HybridCacheHandle(mamba_depth, mamba_node), self._path_values(mamba_node)

    def _find_mamba_ancestor(self, node: RadixTreeNode, depth: int) -> Tuple[RadixTreeNode, int]:
        out = ctypes.c_int64()
        nid = self._tree._lib.msgl_radix_find_mamba_ancestor(self._tree._handle, node._id,
                                                             int(depth), ctypes.byref(out))
        self._tree._check_node(nid)
        return self._tree._node(nid), out.value

    def insert_prefix(self, input_ids: torch.Tensor, indices: torch.Tensor,
                      mamba_slot: Optional[int] = None) -> int:
        prefix_len, to_free = self._insert(input_ids, indices, mamba_slot)
        if to_free is not None:
            # the whole sequence was cached and its node already had a snapshot
            self.mamba_pool.free(to_free)
        return prefix_len

    def _release_node_state(self, node: RadixTreeNode) -> int:
        if node.mamba_slot is None:
            return 0
        self.mamba_pool.free(node.mamba_slot)
        node.mamba_slot = None
        return 1

    def _release_slots(self, slots: List[int]) -> None:
        for slot in slots:
            self.mamba_pool.free(slot)

    def evict_for_mamba(self, count: int) -> Tuple[torch.Tensor, int]:
        """Evict least-recently-used prefixes until ``count`` snapshots come back; returns the
        evicted slot ids and how many snapshots were freed (fewer once nothing is left)."""
        return self._evict_leaves(num_slots=count)

    def collect_mamba_slots(self) -> List[int]:
        n = self._tree._lib.msgl_radix_collect_mamba_slots(self._tree._handle, None, 0)
        out = (ctypes.c_int32 * max(n, 1))()
        self._tree._lib.msgl_radix_collect_mamba_slots(self._tree._handle, out, n)
        return [int(out[i]) for i in range(n)]

    def coldest_snapshot_node(self, exclude: Optional[RadixTreeNode] = None) -> Optional[RadixTreeNode]:
        nid = self._tree._lib.msgl_radix_coldest_snapshot(
            self._tree._handle, _ERR_NODE if exclude is None else exclude._id)
        return None if nid < 0 else self._tree._node(nid)

    def check_integrity(self) -> None:
        super().check_integrity()
        self.mamba_pool.check_ownership(self.collect_mamba_slots())
