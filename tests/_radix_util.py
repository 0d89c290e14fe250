"""Harness shared by the radix-cache tests.

One set of scenarios -- the reference's own (mini_sglang_mlx/tests/test_radix_prefix_cache.py,
cited per scenario) -- runs against two implementations through a small adapter: the pure-Python
oracle and the native tree behind ``mini_sglang_amd.kvcache``.  The adapter plays the part of the
reference's scheduler-side ``CacheManager`` (scheduler/cache.py:19-76, 169-181): a free list of
pages around the tree, eviction on demand, and the page accounting the reference checks after
every scenario.
"""
from __future__ import annotations

import itertools
from typing import List, Optional, Sequence

import pytest
import torch

from oracle.radix_oracle import RadixOracle

PREFIX = [1, 2, 3, 4, 5, 6]
NUM_PAGES = 64


class SlotPool:
    """Slots 1..num_slots with the ownership rules of MambaStatePool (mamba_pool.py:107-162);
    the state buffers themselves play no part in the tree's behaviour."""

    def __init__(self, num_slots: int) -> None:
        self.num_slots = num_slots
        self._free_slots = list(range(1, num_slots + 1))

    @property
    def available_size(self) -> int:
        return len(self._free_slots)

    def alloc(self) -> Optional[int]:
        return self._free_slots.pop() if self._free_slots else None

    def free(self, slot: int) -> None:
        assert 1 <= slot <= self.num_slots, f"Invalid slot {slot}"
        assert slot not in self._free_slots, f"Slot {slot} is already free"
        self._free_slots.append(slot)

    def check_ownership(self, tree_slots) -> None:
        owned = set(self._free_slots)
        assert len(owned) == len(self._free_slots), "free list contains duplicates"
        for slot in tree_slots:
            assert 1 <= slot <= self.num_slots, f"tree holds invalid slot {slot}"
            assert slot not in owned, f"Slot {slot} is owned twice"
            owned.add(slot)
        leaked = set(range(1, self.num_slots + 1)) - owned
        if leaked:
            raise RuntimeError(f"{len(leaked)} mamba slot(s) leaked: {sorted(leaked)} are "
                               "neither free nor held by a cached prefix")


class _Harness:
    hybrid = False

    def __init__(self, num_pages: int = NUM_PAGES, num_slots: int = 4) -> None:
        self.num_pages = num_pages
        self.free_pages: List[int] = list(range(num_pages))
        self.pool = SlotPool(num_slots)
        self._tick = itertools.count(1)

    def clock(self) -> int:
        return next(self._tick)

    # -- the scheduler-side wrapper --------------------------------------------------------
    def free(self, pages: Sequence[int]) -> None:
        self.free_pages.extend(pages)

    def allocate(self, n: int) -> List[int]:
        if n > len(self.free_pages):
            self.free(self.evict(n - len(self.free_pages)))
            assert len(self.free_pages) >= n, "Eviction did not free enough space."
        out, self.free_pages = self.free_pages[:n], self.free_pages[n:]
        return out

    def cache_prefix(self, tokens: Sequence[int], mamba_slot: Optional[int] = None) -> List[int]:
        pages = self.allocate(len(tokens))
        in_cache = self.insert_prefix(tokens, pages, mamba_slot)
        self.free(pages[:in_cache])
        return pages

    @property
    def available_size(self) -> int:
        return self.sizes()[0] + len(self.free_pages)

    def evict_for_mamba(self, count: int) -> int:
        pages, freed = self.evict_leaves(num_slots=count)
        self.free(pages)
        return freed

    def page_balance(self):
        held = sum(self.sizes())
        assert len(self.free_pages) + held == self.num_pages, (
            f"page accounting broken: {len(self.free_pages)} free + {held} held != {self.num_pages}")
        assert len(set(self.free_pages)) == len(self.free_pages), "a page is free twice"
        return len(self.free_pages), held

    def check_integrity(self) -> None:
        if self.hybrid:
            self.pool.check_ownership(self.collect_mamba_slots())
        self.page_balance()

    def set_lru_order(self, paths) -> None:
        """Rewrite timestamps so that these nodes are the coldest, in the order given (the
        reference writes 1000 + order, far below its nanosecond clock)."""
        for order, path in enumerate(paths):
            self.set_timestamp(self.node_of(path), -10 ** 6 + order)


class _OracleHarness(_Harness):
    def __init__(self, *a, **kw) -> None:
        super().__init__(*a, **kw)
        self.tree = RadixOracle(self.clock, self.pool)

    def insert_prefix(self, tokens, pages, mamba_slot=None):
        return self.tree.insert_prefix(list(tokens), list(pages), mamba_slot)

    def match_prefix(self, tokens):
        f = self.tree.match_prefix_hybrid if self.hybrid else self.tree.match_prefix
        return f(list(tokens))

    def lock(self, node):
        self.tree.lock(node)

    def unlock(self, node):
        self.tree.lock(node, unlock=True)

    def evict(self, size):
        return self.tree.evict(size)

    def evict_leaves(self, size=0, num_slots=0):
        return self.tree.evict_leaves(size, num_slots)

    def sizes(self):
        return self.tree.evictable_size, self.tree.protected_size

    def node_of(self, tokens):
        return self.tree.node_of(tokens)

    def set_timestamp(self, node, value):
        node.timestamp = value

    def collect_mamba_slots(self):
        return self.tree.collect_mamba_slots()

    def coldest_snapshot_node(self, exclude=None):
        return self.tree.coldest_snapshot_node(exclude)

    def root_is_leaf(self):
        return self.tree.root.is_leaf()

    def release_node_state_of_root(self):
        return 0  # the plain tree holds nothing but pages (radix_manager.py:181-189)

    def dump(self):
        return self.tree.dump()


class OraclePlain(_OracleHarness):
    hybrid = False


class OracleHybrid(_OracleHarness):
    hybrid = True


def _t(values) -> torch.Tensor:
    return torch.tensor(list(values), dtype=torch.int32)


class _NativeHarness(_Harness):
    def __init__(self, *a, **kw) -> None:
        super().__init__(*a, **kw)
        from mini_sglang_amd.kvcache import HybridRadixCacheManager, RadixCacheManager

        self.manager = HybridRadixCacheManager(self.pool) if self.hybrid else RadixCacheManager()
        self.manager.clock = self.clock

    def insert_prefix(self, tokens, pages, mamba_slot=None):
        if self.hybrid:
            return self.manager.insert_prefix(_t(tokens), _t(pages), mamba_slot=mamba_slot)
        assert mamba_slot is None
        return self.manager.insert_prefix(_t(tokens), _t(pages))

    def match_prefix(self, tokens):
        handle, indices = self.manager.match_prefix(_t(tokens))
        assert indices.dtype == torch.int32 and indices.dim() == 1
        return handle.cached_len, handle.node, indices.tolist()

    def _handle(self, node):
        from mini_sglang_amd.kvcache import RadixCacheHandle

        return RadixCacheHandle(0, node)

    def lock(self, node):
        self.manager.lock_handle(self._handle(node))

    def unlock(self, node):
        self.manager.lock_handle(self._handle(node), unlock=True)

    def evict(self, size):
        return self.manager.evict(size).tolist()

    def evict_leaves(self, size=0, num_slots=0):
        indices, freed = self.manager._evict_leaves(size=size, num_slots=num_slots)
        return indices.tolist(), freed

    def sizes(self):
        s = self.manager.size_info
        return s.evictable_size, s.protected_size

    def node_of(self, tokens):
        node, offset = self.manager.root_node, 0
        while offset < len(tokens):
            node = node.children[tokens[offset]]
            assert node._key.tolist() == list(tokens[offset:offset + node.length])
            offset += node.length
        return node

    def set_timestamp(self, node, value):
        node.timestamp = value

    def collect_mamba_slots(self):
        return self.manager.collect_mamba_slots()

    def coldest_snapshot_node(self, exclude=None):
        return self.manager.coldest_snapshot_node(exclude)

    def root_is_leaf(self):
        return self.manager.root_node.is_leaf()

    def release_node_state_of_root(self):
        return self.manager._release_node_state(self.manager.root_node)

    def dump(self):
        rows = []

        def visit(node, path):
            for tok, child in sorted(node.children.items()):
                p = path + tuple(child._key.tolist())
                rows.append((p, tuple(child.value.tolist()), child.ref_count, child.mamba_slot,
                             child.timestamp))
                visit(child, p)

        visit(self.manager.root_node, ())
        return rows


class NativePlain(_NativeHarness):
    hybrid = False


class NativeHybrid(_NativeHarness):
    hybrid = True


# ---- the reference's scenarios (test_radix_prefix_cache.py, line of each test given) ----------

def match_is_a_pure_query(make):  # :28-44
    m = make(num_slots=4)
    m.cache_prefix(PREFIX, mamba_slot=m.pool.alloc())
    before = (m.pool.available_size, m.sizes(), m.available_size)
    for _ in range(3):
        cached, _, indices = m.match_prefix(PREFIX)
        assert cached == len(PREFIX) and len(indices) == len(PREFIX)
        assert (m.pool.available_size, m.sizes(), m.available_size) == before


def hit_reports_snapshot_and_pages(make):  # :47-55 (match_req drops the last token: cache.py:30-33)
    m = make(num_slots=4)
    slot = m.pool.alloc()
    pages = m.cache_prefix(PREFIX, mamba_slot=slot)
    cached, node, indices = m.match_prefix(PREFIX)
    assert cached == len(PREFIX) and node.mamba_slot == slot and indices == pages


def split_leaves_snapshot_on_deeper_node(make):  # :58-82
    m = make(num_slots=4)
    a, b = m.pool.alloc(), m.pool.alloc()
    m.cache_prefix(PREFIX, mamba_slot=a)
    m.cache_prefix([1, 2, 3, 9], mamba_slot=b)
    assert m.node_of([1, 2, 3]).mamba_slot is None  # the split point is a tombstone
    assert m.node_of(PREFIX).mamba_slot == a
    assert m.node_of([1, 2, 3, 9]).mamba_slot == b
    assert sorted(m.collect_mamba_slots()) == sorted([a, b])
    assert m.match_prefix([1, 2, 3])[0] == 0  # no state at that boundary: no reuse at all
    cached, node, indices = m.match_prefix(PREFIX)
    assert cached == len(PREFIX) and node.mamba_slot == a and len(indices) == len(PREFIX)


def locking_moves_prefix_out_of_evictable(make):  # :85-99
    m = make(num_slots=4)
    m.cache_prefix(PREFIX, mamba_slot=m.pool.alloc())
    _, node, _ = m.match_prefix(PREFIX)
    before = m.available_size
    m.lock(node)
    assert m.available_size == before - len(PREFIX)
    assert m.sizes()[1] == len(PREFIX)
    m.unlock(node)
    assert m.available_size == before
    m.page_balance()


def eviction_frees_snapshot_and_returns_pages(make):  # :102-117
    m = make(num_slots=4)
    m.cache_prefix(PREFIX, mamba_slot=m.pool.alloc())
    free_before, held_before = m.page_balance()
    assert held_before == len(PREFIX)
    handed_out = m.allocate(free_before + 2)  # more than is free: the only evictable leaf goes
    assert m.pool.available_size == 4
    assert m.collect_mamba_slots() == []
    assert m.root_is_leaf()
    m.free(handed_out)
    m.page_balance()


def evict_for_mamba_in_lru_order(make):  # :120-138
    m = make(num_slots=4)
    for path in ([1, 2], [10, 11], [20, 21]):
        m.cache_prefix(path, mamba_slot=m.pool.alloc())
    assert m.pool.available_size == 1
    m.set_lru_order([[1, 2], [10, 11], [20, 21]])
    assert m.evict_for_mamba(1) == 1
    assert m.pool.available_size == 2
    with pytest.raises(KeyError):
        m.node_of([1, 2])
    assert m.node_of([10, 11]).mamba_slot is not None
    m.page_balance()
    assert m.evict_for_mamba(1) == 1
    with pytest.raises(KeyError):
        m.node_of([10, 11])
    m.page_balance()


def evict_for_mamba_walks_through_slot_less_leaves(make):  # :141-163
    m = make(num_slots=4)
    m.cache_prefix(PREFIX, mamba_slot=m.pool.alloc())
    m.cache_prefix([1, 2, 3, 9], mamba_slot=m.pool.alloc())
    m.free(m.evict(4))  # the tombstone's children (3 + 1 pages); 7 would take the tombstone too
    tomb = m.node_of([1, 2, 3])
    assert tomb.mamba_slot is None and tomb.is_leaf()
    assert m.pool.available_size == 4
    m.cache_prefix([9], mamba_slot=m.pool.alloc())
    m.set_lru_order([[1, 2, 3]])  # colder than the [9] leaf
    _, held_before = m.page_balance()
    assert m.evict_for_mamba(1) == 1  # the coldest leaf owns no snapshot and still goes first
    _, held_after = m.page_balance()
    assert held_before - held_after == 4  # 3 tombstone pages + 1 leaf page
    assert m.collect_mamba_slots() == []


def evict_for_mamba_drains_gracefully(make):  # :166-174
    m = make(num_slots=4)
    assert m.evict_for_mamba(2) == 0
    m.page_balance()
    m.cache_prefix([1, 2], mamba_slot=m.pool.alloc())
    assert m.evict_for_mamba(5) == 1  # more than exists
    assert m.evict_for_mamba(1) == 0
    m.page_balance()


def coldest_snapshot_skips_only_the_node_itself(make):  # :177-196
    m = make(num_slots=4)
    slots = [m.pool.alloc() for _ in range(3)]
    m.cache_prefix([1, 2], mamba_slot=slots[0])
    m.cache_prefix([1, 2, 3, 4], mamba_slot=slots[1])
    m.cache_prefix(PREFIX, mamba_slot=slots[2])
    coldest = m.coldest_snapshot_node()
    assert coldest is m.node_of([1, 2])
    assert m.coldest_snapshot_node(exclude=coldest) is m.node_of([1, 2, 3, 4])
    assert m.coldest_snapshot_node(exclude=m.node_of(PREFIX)) is coldest


def integrity_detects_escaped_slot(make):  # :199-210
    m = make(num_slots=3)
    m.cache_prefix(PREFIX, mamba_slot=m.pool.alloc())
    m.check_integrity()
    leaked = m.pool.alloc()  # nothing records it
    with pytest.raises(RuntimeError, match="leaked"):
        m.check_integrity()
    m.pool.free(leaked)
    m.check_integrity()


def plain_manager_keeps_the_evict_contract(make):  # :213-227
    m = make(num_pages=32)
    pages = m.allocate(6)
    assert m.insert_prefix(PREFIX, pages) == 0
    assert m.evict(0) == []
    assert m.release_node_state_of_root() == 0
    with pytest.raises(AssertionError, match="Cannot evict"):
        m.evict(7)
    m.free(m.evict(6))
    m.page_balance()


def insert_refuses_snapshot_on_root(make):  # :230-234
    m = make(num_slots=2)
    with pytest.raises(AssertionError, match="snapshot on the root"):
        m.insert_prefix([], [], mamba_slot=m.pool.alloc())


# name -> (scenario, needs the hybrid manager)
SCENARIOS = {
    "match_is_a_pure_query": (match_is_a_pure_query, True),
    "hit_reports_snapshot_and_pages": (hit_reports_snapshot_and_pages, True),
    "split_leaves_snapshot_on_deeper_node": (split_leaves_snapshot_on_deeper_node, True),
    "locking_moves_prefix_out_of_evictable": (locking_moves_prefix_out_of_evictable, True),
    "eviction_frees_snapshot_and_returns_pages": (eviction_frees_snapshot_and_returns_pages, True),
    "evict_for_mamba_in_lru_order": (evict_for_mamba_in_lru_order, True),
    "evict_for_mamba_walks_through_slot_less_leaves": (evict_for_mamba_walks_through_slot_less_leaves, True),
    "evict_for_mamba_drains_gracefully": (evict_for_mamba_drains_gracefully, True),
    "coldest_snapshot_skips_only_the_node_itself": (coldest_snapshot_skips_only_the_node_itself, True),
    "integrity_detects_escaped_slot": (integrity_detects_escaped_slot, True),
    "plain_manager_keeps_the_evict_contract": (plain_manager_keeps_the_evict_contract, False),
    "insert_refuses_snapshot_on_root": (insert_refuses_snapshot_on_root, True),
}


def run_scenario(name: str, harness_cls) -> None:
    SCENARIOS[name][0](harness_cls)
