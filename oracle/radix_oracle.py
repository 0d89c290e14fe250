"""TEST INFRASTRUCTURE ONLY -- not part of the product path.

Pure-Python restatement of the reference's radix prefix cache on plain lists, used by the
tests as the checker of the native tree (and by bench.py as the CPU baseline of that leg).

Follows mini_sglang_mlx/kvcache/radix_manager.py:
  RadixTreeNode / _split_at            :18-90
  RadixCacheManager                    :98-275   (lock_handle :108-125, match_prefix :127-138,
                                                  insert_prefix :140-150, _walk :152-179,
                                                  _evict_leaves :191-237, evict :239-247)
  HybridRadixCacheManager              :299-452  (match_prefix :319-345, _find_mamba_ancestor
                                                  :347-358, insert_prefix :362-392,
                                                  coldest_snapshot_node :429-446)
and fast_compare_key (mini-sglang-mlx-kernel/csrc/fast_compare_key.cpp:9-45).

Three things the reference leaves open are fixed here the way the native tree fixes them: nodes
with equal timestamps are evicted (and ranked "coldest") in creation order; asking
``_evict_leaves`` for more pages than are evictable fails before anything is evicted; an insert
reads the clock once (the reference stamps the new leaf with a second, later reading, which
only orders it after its own ancestors).

Pinned by tests/test_oracle_radix.py against the scenarios and expected values of the
reference's own mini_sglang_mlx/tests/test_radix_prefix_cache.py.
"""
from __future__ import annotations

import heapq
import itertools
from typing import Callable, Dict, List, Optional, Sequence, Tuple


def fast_compare_key(a: Sequence[int], b: Sequence[int]) -> int:
    n = min(len(a), len(b))
    for i in range(n):
        if a[i] != b[i]:
            return i
    return n


class Node:
    def __init__(self, uuid: int, timestamp: int) -> None:
        self.children: Dict[int, "Node"] = {}
        self.parent: Optional["Node"] = None
        self.ref_count = 0
        self.uuid = uuid
        self.timestamp = timestamp
        self.mamba_slot: Optional[int] = None
        self.key: List[int] = []
        self.value: List[int] = []

    @property
    def length(self) -> int:
        return len(self.key)

    def is_root(self) -> bool:
        return self.parent is None

    def is_leaf(self) -> bool:
        return not self.children

    def set_parent(self, parent: "Node") -> None:
        self.parent = parent
        parent.children[self.key[0]] = self


class RadixOracle:
    """Plain and hybrid manager in one: ``pool`` (an object with ``free(slot)``) is only
    touched when snapshots are involved."""

    def __init__(self, clock: Callable[[], int], pool=None) -> None:
        self._ids = itertools.count()
        self.clock = clock
        self.pool = pool
        self.root = Node(next(self._ids), 0)  # never compared: the root is never a candidate
        self.root.ref_count = 1
        self.evictable_size = 0
        self.protected_size = 0

    def _new(self, timestamp: int) -> Node:
        return Node(next(self._ids), timestamp)

    def _split_at(self, node: Node, pos: int) -> Node:
        assert 0 < pos < node.length
        upper = self._new(node.timestamp)
        upper.key, upper.value = node.key[:pos], node.value[:pos]
        upper.set_parent(node.parent)
        upper.ref_count = node.ref_count
        node.key, node.value = node.key[pos:], node.value[pos:]
        node.set_parent(upper)
        return upper

    def walk(self, ids: Sequence[int], tic: Optional[int] = None) -> Tuple[Node, int]:
        prefix, node = 0, self.root
        tic = self.clock() if tic is None else tic
        while prefix < len(ids):
            child = node.children.get(ids[prefix])
            if child is None:
                return node, prefix
            node = child
            match = fast_compare_key(node.key, ids[prefix:])
            prefix += match
            if match != node.length:
                return self._split_at(node, match), prefix
            node.timestamp = tic
        return node, prefix

    @staticmethod
    def path_values(node: Node) -> List[int]:
        parts = []
        while not node.is_root():
            parts.append(node.value)
            node = node.parent
        return [v for part in reversed(parts) for v in part]

    def match_prefix(self, ids: Sequence[int]) -> Tuple[int, Node, List[int]]:
        node, prefix = self.walk(ids)
        return prefix, node, self.path_values(node) if prefix else []

    def find_mamba_ancestor(self, node: Node, depth: int) -> Tuple[Node, int]:
        while not node.is_root():
            if node.mamba_slot is not None:
                return node, depth
            depth -= node.length
            node = node.parent
        return self.root, 0

    def match_prefix_hybrid(self, ids: Sequence[int]) -> Tuple[int, Node, List[int]]:
        node, prefix = self.walk(ids)
        mnode, depth = self.find_mamba_ancestor(node, prefix)
        if mnode.mamba_slot is None or depth == 0:
            return 0, self.root, []
        return depth, mnode, self.path_values(mnode)

    def insert_prefix(self, ids: Sequence[int], indices: Sequence[int],
                      mamba_slot: Optional[int] = None) -> int:
        # one stamp per call: the reference reads its clock a second time for the new leaf, which
        # orders that leaf after the nodes the walk touched -- all of them its own ancestors
        tic = self.clock()
        node, prefix = self.walk(ids, tic)
        if prefix < len(ids):
            leaf = self._new(tic)
            leaf.key, leaf.value = list(ids[prefix:]), list(indices[prefix:len(ids)])
            leaf.set_parent(node)
            leaf.mamba_slot = mamba_slot
            self.evictable_size += leaf.length
        elif mamba_slot is not None:
            assert not node.is_root(), "cannot store a snapshot on the root"
            if node.mamba_slot is None:
                node.mamba_slot = mamba_slot
            else:
                self.pool.free(mamba_slot)
        return prefix

    def lock(self, node: Node, unlock: bool = False) -> None:
        while not node.is_root():
            if unlock:
                node.ref_count -= 1
                assert node.ref_count >= 0
                if node.ref_count == 0:
                    self.evictable_size += node.length
                    self.protected_size -= node.length
            else:
                if node.ref_count == 0:
                    self.evictable_size -= node.length
                    self.protected_size += node.length
                node.ref_count += 1
            node = node.parent

    def _nodes(self):
        stack = [self.root]
        while stack:
            node = stack.pop()
            yield node
            stack.extend(node.children.values())

    def evict_leaves(self, size: int = 0, num_slots: int = 0) -> Tuple[List[int], int]:
        assert size <= self.evictable_size, f"Cannot evict {size}, only {self.evictable_size} is evictable"
        heap = [(n.timestamp, n.uuid, n) for n in self._nodes() if n.is_leaf() and n.ref_count == 0]
        heapq.heapify(heap)
        out: List[int] = []
        freed = 0
        while len(out) < size or freed < num_slots:
            if not heap:
                break
            node = heapq.heappop(heap)[2]
            assert node.ref_count == 0 and node.is_leaf() and not node.is_root()
            out.extend(node.value)
            self.evictable_size -= node.length
            if node.mamba_slot is not None:
                self.pool.free(node.mamba_slot)
                node.mamba_slot = None
                freed += 1
            parent = node.parent
            del parent.children[node.key[0]]
            if parent.is_leaf() and parent.ref_count == 0:
                heapq.heappush(heap, (parent.timestamp, parent.uuid, parent))
        return out, freed

    def evict(self, size: int) -> List[int]:
        return self.evict_leaves(size=size)[0] if size else []

    def collect_mamba_slots(self) -> List[int]:
        return [n.mamba_slot for n in self._nodes() if n.mamba_slot is not None]

    def coldest_snapshot_node(self, exclude: Optional[Node] = None) -> Optional[Node]:
        best = None
        for n in self._nodes():
            if n.mamba_slot is not None and n is not exclude:
                if best is None or (n.timestamp, n.uuid) < (best.timestamp, best.uuid):
                    best = n
        return best

    def node_of(self, tokens: Sequence[int]) -> Node:
        """The node whose key path ends exactly at ``tokens`` (KeyError if there is none)."""
        node, offset = self.root, 0
        while offset < len(tokens):
            node = node.children[tokens[offset]]
            assert node.key == list(tokens[offset:offset + node.length])
            offset += node.length
        return node

    def dump(self) -> list:
        """Canonical picture of the tree: one tuple per node in key order."""
        rows = []

        def visit(node: Node, path: Tuple[int, ...]) -> None:
            for tok in sorted(node.children):
                child = node.children[tok]
                p = path + tuple(child.key)
                rows.append((p, tuple(child.value), child.ref_count, child.mamba_slot, child.timestamp))
                visit(child, p)

        visit(self.root, ())
        return rows
