"""CPU restatement of the reference's recurrent-state slot pool -- TEST INFRASTRUCTURE ONLY.

Follows mini_sglang_mlx/kvcache/mamba_pool.py:36-215 on numpy arrays, one array per layer and
buffer as there: LIFO free list over slots 1..num_slots (slot 0 is the padding slot, :85),
``alloc`` zeroes the slot it hands out (:137-142), ``alloc_many`` does not and takes nothing
when it cannot serve the request (:144-158), ``free`` rejects slots outside the pool and slots
already free (:160-168), ``check_ownership`` (:107-135), ``copy`` / ``copy_batched`` as
``buf[dst] = buf[src]`` with every source read before any write (:170-189).

Pinned by the twelve scenarios of the reference's mini_sglang_mlx/tests/test_mamba_slots.py
(expected values held as data in tests/golden/mamba_slot_scenarios.json).  bfloat16 buffers are kept as uint16 bit
patterns: nothing here does arithmetic on them.
"""
from __future__ import annotations

from typing import Iterable, List, Optional, Sequence

import numpy as np


class MambaPoolOracle:
    def __init__(self, num_slots: int, num_layers: int, conv_shapes: List[List[tuple]],
                 temporal_shapes: List[tuple], verify_width: int = 0):
        self.num_slots = num_slots
        self.num_layers = num_layers
        self.verify_width = verify_width
        rows = num_slots + 1
        self.conv = [[np.zeros((rows, *s), dtype=np.uint16) for s in conv_shapes[l]]
                     for l in range(num_layers)]
        self.temporal = [np.zeros((rows, *temporal_shapes[l]), dtype=np.float32)
                         for l in range(num_layers)]
        self.windows = [[np.zeros((rows, verify_width, *s), dtype=np.uint16) for s in conv_shapes[l]]
                        if verify_width > 0 else [] for l in range(num_layers)]
        self.free_slots = list(range(1, num_slots + 1))

    @property
    def available_size(self) -> int:
        return len(self.free_slots)

    def _state_buffers(self):
        for layer in self.conv:
            yield from layer
        yield from self.temporal

    def alloc(self) -> Optional[int]:
        if not self.free_slots:
            return None
        slot = self.free_slots.pop()
        for buf in self._state_buffers():
            buf[slot] = 0
        return slot

    def alloc_many(self, n: int) -> Optional[List[int]]:
        if n == 0:
            return []
        if len(self.free_slots) < n:
            return None
        slots = self.free_slots[-n:]
        del self.free_slots[-n:]
        return slots

    def free(self, slot: int) -> None:
        assert 1 <= slot <= self.num_slots, f"Invalid slot {slot}"
        assert slot not in self.free_slots, f"Slot {slot} is already free"
        self.free_slots.append(slot)

    def free_many(self, slots: Sequence[int]) -> None:
        for slot in slots:
            self.free(slot)

    def check_ownership(self, tree_slots: Iterable[int]) -> None:
        owned = set(self.free_slots)
        assert len(owned) == len(self.free_slots), "free list contains duplicates"
        for slot in tree_slots:
            assert 1 <= slot <= self.num_slots, f"tree holds invalid slot {slot}"
            assert slot not in owned, f"Slot {slot} is owned twice"
            owned.add(slot)
        leaked = set(range(1, self.num_slots + 1)) - owned
        if leaked:
            raise RuntimeError(f"{len(leaked)} mamba slot(s) leaked: {sorted(leaked)}")

    def copy(self, src: int, dst: int) -> None:
        self.copy_batched([src], [dst])

    def copy_batched(self, src: Sequence[int], dst: Sequence[int]) -> None:
        src, dst = np.asarray(src, dtype=np.int64), np.asarray(dst, dtype=np.int64)
        assert src.shape == dst.shape
        for buf in self._state_buffers():
            buf[dst] = buf[src]  # fancy indexing gathers the sources first

    def conv_window(self, layer: int, group: int = 0) -> np.ndarray:
        assert self.verify_width > 0, "conv windows not allocated"
        return self.windows[layer][group]
