"""Slot pool of recurrent (conv + temporal) state for the linear-attention layers, laid out for
whole-pool device operations.

Counterpart of ``MambaStatePool`` (mini_sglang_mlx/kvcache/mamba_pool.py:36-215): same
configuration object, slot lifecycle (``alloc`` / ``alloc_many`` / ``free`` / ``free_many`` /
``check_ownership``, LIFO free list, slot 0 reserved as the padding slot), accessors
(``temporal_state`` / ``conv_state`` / ``conv_window``) and copies (``copy`` / ``copy_batched``).
It is the ``state`` argument of ``gdn_state_inplace`` and the pool whose slots the hybrid radix
cache hands out as prefix snapshots.

Layout: layers whose buffers have the same shape share one ``(layers, slots + 1, ...)`` slab (the
reference keeps one array per layer and buffer), so a copy or a zero fill of some slots is one
``msgl_copy_state_slots`` launch per slab instead of one array update per layer and buffer.  A
layer's buffer is the view ``slab[i]``.  Temporal state has the configured dtype (float32 by
default), conv state and conv windows are bfloat16, as in the reference (mamba_pool.py:57-83).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Iterable, List, NamedTuple, Optional, Sequence, Tuple, Union

import torch

from mini_sglang_amd_kernel import _lib


class MambaStateShape(NamedTuple):
    """Shapes of one layer's state buffers (mamba_pool.py:13-17)."""
    conv: List[tuple]
    temporal: tuple


@dataclass(frozen=True)
class MambaStateConfig:
    """What the pool allocates (mamba_pool.py:20-33).  ``verify_width`` > 0 adds, per conv
    buffer, ``verify_width`` sliding windows per slot for replay-style speculative verify."""
    num_slots: int
    num_layers: int
    conv_shapes: List[List[tuple]]
    temporal_shapes: List[tuple]
    dtype: torch.dtype = torch.float32
    verify_width: int = 0


class _Slab:
    """Buffers of equal shape from several layers in one allocation."""

    def __init__(self, rows: int, shape: Sequence[int], dtype: torch.dtype, device) -> None:
        self.shape = tuple(int(x) for x in shape)
        self.members = 0  # layers (or layer/group entries) placed so far
        self.rows = rows
        self.dtype = dtype
        self.device = device
        self.data: Optional[torch.Tensor] = None

    def reserve(self) -> int:
        self.members += 1
        return self.members - 1

    def allocate(self) -> None:
        self.data = torch.zeros((self.members, self.rows, *self.shape), dtype=self.dtype,
                                device=self.device)


class MambaStatePool:
    def __init__(self, config: MambaStateConfig, device="cuda") -> None:
        if config.num_slots < 0 or config.num_layers < 0:
            raise ValueError("MambaStatePool: negative size")
        if len(config.conv_shapes) != config.num_layers or len(config.temporal_shapes) != config.num_layers:
            raise ValueError("MambaStatePool: one conv shape list and one temporal shape per layer")
        self.num_slots = config.num_slots
        self.num_layers = config.num_layers
        self.dtype = config.dtype
        self.verify_width = config.verify_width
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise ValueError("MambaStatePool lives in GPU memory (its copies and zero fills are "
                             "device kernels); there is no host implementation")
        rows = config.num_slots + 1  # slot 0 is the padding slot

        slabs: Dict[tuple, _Slab] = {}

        def place(kind: str, shape: Sequence[int], dtype: torch.dtype) -> Tuple[_Slab, int]:
            key = (kind, tuple(shape), dtype)
            if key not in slabs:
                slabs[key] = _Slab(rows, shape, dtype, self.device)
            return slabs[key], slabs[key].reserve()

        self._temporal: List[Tuple[_Slab, int]] = []
        self._conv: List[List[Tuple[_Slab, int]]] = []
        self._windows: List[List[Tuple[_Slab, int]]] = []
        for layer in range(config.num_layers):
            self._temporal.append(place("temporal", config.temporal_shapes[layer], config.dtype))
            self._conv.append([place("conv", s, torch.bfloat16) for s in config.conv_shapes[layer]])
            self._windows.append(
                [place("window", (config.verify_width, *s), torch.bfloat16)
                 for s in config.conv_shapes[layer]] if config.verify_width > 0 else [])
        self._slabs = list(slabs.values())
        for slab in self._slabs:
            slab.allocate()
        # copies and zero fills move the slot state, not the verify windows (mamba_pool.py:170-189)
        self._state_slabs = [s for (kind, _, _), s in slabs.items() if kind != "window"]
        self._free_slots: List[int] = list(range(1, config.num_slots + 1))

    # ---- slot lifecycle (host) -------------------------------------------------------------
    @property
    def available_size(self) -> int:
        return len(self._free_slots)

    def alloc(self) -> Optional[int]:
        """Most recently freed slot, zeroed; ``None`` when the pool is exhausted."""
        if not self._free_slots:
            return None
        slot = self._free_slots.pop()
        self._zero_slot(slot)
        return slot

    def alloc_many(self, n: int) -> Optional[List[int]]:
        """``n`` slots at once, not zeroed (verify scratch slots are overwritten by a copy
        first); ``None``, and nothing taken, when fewer are free."""
        if n == 0:
            return []
        if len(self._free_slots) < n:
            return None
        slots = self._free_slots[-n:]
        del self._free_slots[-n:]
        return slots

    def free(self, slot: int) -> None:
        assert 1 <= slot <= self.num_slots, f"Invalid slot {slot}"
        # a slot in the free list twice would be handed to two sequences at once
        assert slot not in self._free_slots, f"Slot {slot} is already free"
        self._free_slots.append(slot)

    def free_many(self, slots: List[int]) -> None:
        for slot in slots:
            self.free(slot)

    def check_ownership(self, tree_slots: Iterable[int]) -> None:
        """Every slot is in the free list or held by a cached prefix, never both, never neither
        (meaningful when no request is running; mamba_pool.py:107-135)."""
        owned = set(self._free_slots)
        assert len(owned) == len(self._free_slots), "free list contains duplicates"
        for slot in tree_slots:
            assert 1 <= slot <= self.num_slots, f"tree holds invalid slot {slot}"
            assert slot not in owned, f"Slot {slot} is owned twice"
            owned.add(slot)
        leaked = set(range(1, self.num_slots + 1)) - owned
        if leaked:
            raise RuntimeError(f"{len(leaked)} mamba slot(s) leaked: {sorted(leaked)} are neither "
                               "free nor held by a cached prefix")

    # ---- device operations -----------------------------------------------------------------
    def _ids(self, ids: Union[torch.Tensor, Sequence[int]]) -> torch.Tensor:
        if isinstance(ids, torch.Tensor):
            if ids.dtype != torch.int32:
                raise TypeError("slot ids must be int32")
            return ids.to(self.device).contiguous().view(-1)
        return torch.tensor(list(ids), dtype=torch.int32, device=self.device)

    def _launch(self, src: Optional[torch.Tensor], dst: torch.Tensor) -> None:
        n = dst.numel()
        if n == 0:
            return
        lib = _lib.load()
        with torch.cuda.device(self.device):
            stream = torch.cuda.current_stream(self.device).cuda_stream
            for slab in self._state_slabs:
                data = slab.data
                esz = data.element_size()
                rc = lib.msgl_copy_state_slots(
                    data.data_ptr(), data.stride(0) * esz, data.stride(1) * esz,
                    data.stride(1) * esz, data.shape[0], data.shape[1],
                    src.data_ptr() if src is not None else None, dst.data_ptr(), n, stream)
                if rc != 0:
                    raise RuntimeError(f"msgl_copy_state_slots: {_lib.strerror(rc)}")

    def copy(self, src: int, dst: int) -> None:
        """All state of slot ``src`` into slot ``dst``, every layer."""
        self.copy_batched([src], [dst])

    def copy_batched(self, src, dst) -> None:
        """``slot dst[i] <- slot src[i]`` for every ``i``, every layer, one launch per slab.
        ``src`` / ``dst``: int32 tensors of one shape, or sequences of ints.  The destinations
        must be distinct and disjoint from the sources (checked when given on the host)."""
        if not isinstance(src, torch.Tensor) and not isinstance(dst, torch.Tensor):
            src, dst = list(src), list(dst)
            assert len(src) == len(dst)
            moved = [(s, d) for s, d in zip(src, dst) if s != d]
            targets = [d for _, d in moved]
            if len(set(targets)) != len(targets) or set(targets) & {s for s, _ in moved}:
                raise ValueError("copy_batched: destination slots must be distinct and must not "
                                 "also be sources")
        s, d = self._ids(src), self._ids(dst)
        assert s.shape == d.shape
        self._launch(s, d)

    def _zero_slot(self, slot: int) -> None:
        self._launch(None, self._ids([slot]))

    # ---- accessors -------------------------------------------------------------------------
    def temporal_state(self, layer_idx: int) -> torch.Tensor:
        slab, at = self._temporal[layer_idx]
        return slab.data[at]

    def conv_state(self, layer_idx: int, group: int = 0) -> torch.Tensor:
        slab, at = self._conv[layer_idx][group]
        return slab.data[at]

    def conv_window(self, layer_idx: int, group: int = 0) -> torch.Tensor:
        """Row ``[slot, j]``: the conv window after ``j + 1`` verify tokens (mamba_pool.py:194-203)."""
        assert self.verify_width > 0, "conv windows not allocated"
        slab, at = self._windows[layer_idx][group]
        return slab.data[at]

    def mem_usage_bytes(self) -> int:
        return sum(s.data.numel() * s.data.element_size() for s in self._slabs)
