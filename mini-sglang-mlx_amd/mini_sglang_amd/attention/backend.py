"""Attention backend of the path on torch-ROCm
(reference: mini_sglang_mlx/attention/backend.py:15-307).

``AttnBackend.forward`` stores the new K/V rows first and then attends through the slot
lists, so the new tokens are read back from the pool exactly like cached ones
(backend.py:139-141).  Metadata are int32 CSR arrays; ``kv_indices`` holds one pool slot
per token.  The builders keep the reference's formulas and keyword overrides (virtual
extend windows for speculative verify, backend.py:205-293).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch

from mini_sglang_amd_kernel import (build_attention_metadata, paged_decode_attention,
                                    paged_prefill_attention, qk_norm_rope_store)

MAX_KV_SPLITS = 32


@dataclass
class BaseAttnMetadata:
    positions: torch.Tensor

    def get_last_indices(self, bs: int) -> torch.Tensor:
        raise NotImplementedError


@dataclass
class PrefillMetadata(BaseAttnMetadata):
    """Several new query tokens per sequence on top of a cached prefix (backend.py:26-41)."""

    qo_indptr: torch.Tensor  # (batch + 1,) int32
    kv_indptr: torch.Tensor  # (batch + 1,) int32
    kv_indices: torch.Tensor  # (total_kv,) int32 pool slots
    prefix_lens: torch.Tensor  # (batch,) int32
    max_len_extend: int

    def get_last_indices(self, bs: int) -> torch.Tensor:
        return self.qo_indptr[1 : 1 + bs] - 1


@dataclass
class DecodeMetadata(BaseAttnMetadata):
    """One new query token per sequence (backend.py:44-58)."""

    kv_indptr: torch.Tensor  # (batch + 1,) int32
    kv_indices: torch.Tensor  # (total_kv,) int32 pool slots
    num_kv_splits: torch.Tensor  # (batch,) int32
    max_kv_splits: int

    def get_last_indices(self, bs: int) -> torch.Tensor:
        return torch.arange(bs, dtype=torch.int32, device=self.kv_indptr.device)


AttnMetadata = PrefillMetadata | DecodeMetadata


class AttnBackend:
    """Paged attention backend for MI355X using the msgl HIP kernels.

    ``config`` needs ``head_dim``; ``kvcache`` is a ``BaseKVCache``; ``page_table`` is the
    ``(max_running_req + 1, max_seq_len)`` int32 slot table the scheduler fills.
    """

    def __init__(self, config, kvcache, page_table: torch.Tensor) -> None:
        self.config = config
        self.kvcache = kvcache
        self.page_table = page_table
        self.sm_scale = 1.0 / math.sqrt(config.head_dim)

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, layer_id: int, batch, *,
                is_cross_attention: bool = False, sliding_window_size: int = 0) -> torch.Tensor:
        """Write the new K/V rows at ``batch.out_loc`` and run paged attention.

        The two flags select one of four masks on the prefill path (backend.py:112-127):
        causal, full, causal + window, bidirectional + window.  Decode rejects both.
        """
        assert sliding_window_size >= 0, (
            f"sliding_window_size must be >= 0, got {sliding_window_size}"
        )
        metadata = batch.attn_metadata
        self.kvcache.store_kv(k, v, batch.out_loc, layer_id)
        k_cache = self.kvcache.k_cache(layer_id)
        v_cache = self.kvcache.v_cache(layer_id)
        return self._attend(q, k_cache, v_cache, metadata, is_cross_attention, sliding_window_size)

    def _attend(self, q, k_cache, v_cache, metadata, is_cross_attention: bool,
                sliding_window_size: int) -> torch.Tensor:
        if isinstance(metadata, PrefillMetadata):
            return paged_prefill_attention(
                q, k_cache, v_cache, metadata.qo_indptr, metadata.kv_indptr, metadata.kv_indices,
                metadata.prefix_lens, sm_scale=self.sm_scale,
                max_len_extend=metadata.max_len_extend,
                is_cross_attention=is_cross_attention, sliding_window_size=sliding_window_size)
        assert isinstance(metadata, DecodeMetadata)
        assert not is_cross_attention and sliding_window_size == 0, (
            "is_cross_attention / sliding_window_size are only "
            "supported on the prefill path."
        )
        return paged_decode_attention(
            q, k_cache, v_cache, metadata.kv_indptr, metadata.kv_indices, metadata.num_kv_splits,
            sm_scale=self.sm_scale, max_kv_splits=metadata.max_kv_splits)

    def forward_fused_norm_rope(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                                q_norm_weight: torch.Tensor, k_norm_weight: torch.Tensor,
                                layer_id: int, batch, *, rms_norm_eps: float, rope_base: float,
                                is_cross_attention: bool = False,
                                sliding_window_size: int = 0) -> torch.Tensor:
        """``forward`` for a Qwen3-style layer that hands over the raw projections: q/k RMSNorm,
        rotary embedding at ``batch.attn_metadata.positions`` and the KV-store run as one kernel
        (the reference does them as four array ops plus the store, models/qwen3.py:60-68 and
        backend.py:139), then attention runs on the pool without storing again."""
        assert sliding_window_size >= 0, (
            f"sliding_window_size must be >= 0, got {sliding_window_size}"
        )
        metadata = batch.attn_metadata
        k_cache = self.kvcache.k_cache(layer_id)
        v_cache = self.kvcache.v_cache(layer_id)
        q = qk_norm_rope_store(q, k, v, q_norm_weight, k_norm_weight, metadata.positions,
                               batch.out_loc, k_cache, v_cache, eps=rms_norm_eps,
                               rope_base=rope_base)
        return self._attend(q, k_cache, v_cache, metadata, is_cross_attention, sliding_window_size)

    def store_kv_only(self, k: torch.Tensor, v: torch.Tensor, out_loc: torch.Tensor,
                      layer_id: int) -> None:
        """Write K/V without attending (draft calibration, backend.py:174-196)."""
        self.kvcache.store_kv(k, v, out_loc, layer_id)

    def prepare_metadata(self, batch) -> None:
        reqs = batch.padded_reqs
        if batch.is_prefill:
            batch.attn_metadata = self.build_prefill_metadata(reqs)
        else:
            batch.attn_metadata = self.build_decode_metadata(reqs)

    def _gather_indices(self, reqs, kv_lens: Sequence[int]) -> torch.Tensor:
        return torch.cat([self.page_table[reqs[i].table_idx, : kv_lens[i]]
                          for i in range(len(reqs))]).to(torch.int32)

    def _device_metadata(self, reqs, kv_lens: Sequence[int],
                         extend_lens: Optional[Sequence[int]]) -> dict:
        """One upload of the per-request integers, one kernel for every array (slot table on
        the GPU).  The host lists are the reference's own inputs (backend.py:228-238)."""
        device = self.page_table.device
        host = [[req.table_idx for req in reqs], list(kv_lens)]
        if extend_lens is not None:
            host.append(list(extend_lens))
        packed = torch.tensor(host, dtype=torch.int32).to(device, non_blocking=True)
        return build_attention_metadata(
            self.page_table, packed[0], packed[1], packed[2] if extend_lens is not None else None,
            total_kv=int(sum(kv_lens)),
            total_q=int(sum(extend_lens)) if extend_lens is not None else len(reqs),
            max_kv_splits=MAX_KV_SPLITS)

    def build_prefill_metadata(self, reqs: List, *, extend_lens: Optional[List[int]] = None,
                               kv_lens: Optional[List[int]] = None,
                               positions: Optional[torch.Tensor] = None) -> PrefillMetadata:
        device = self.page_table.device
        if extend_lens is None:
            extend_lens = [req.extend_len for req in reqs]
        if kv_lens is None:
            kv_lens = [req.device_len for req in reqs]
        if device.type == "cuda":
            m = self._device_metadata(reqs, kv_lens, extend_lens)
            return PrefillMetadata(
                positions=m["positions"] if positions is None else positions,
                qo_indptr=m["qo_indptr"], kv_indptr=m["kv_indptr"], kv_indices=m["kv_indices"],
                prefix_lens=m["prefix_lens"], max_len_extend=max(extend_lens))
        # slot table in host memory (host-side tests): the same arrays with torch ops
        cached_lens = [kv_lens[i] - extend_lens[i] for i in range(len(reqs))]
        if positions is None:
            positions = torch.cat([
                torch.arange(cached_lens[i], kv_lens[i], dtype=torch.int32, device=device)
                for i in range(len(reqs))
            ])
        return PrefillMetadata(
            positions=positions,
            qo_indptr=_build_indptr(extend_lens, device),
            kv_indptr=_build_indptr(kv_lens, device),
            kv_indices=self._gather_indices(reqs, kv_lens),
            prefix_lens=torch.tensor(cached_lens, dtype=torch.int32, device=device),
            max_len_extend=max(extend_lens),
        )

    def build_decode_metadata(self, reqs: List, *, kv_lens: Optional[List[int]] = None,
                              positions: Optional[torch.Tensor] = None) -> DecodeMetadata:
        device = self.page_table.device
        if kv_lens is None:
            kv_lens = [req.device_len for req in reqs]
        if positions is None:
            positions = torch.tensor([req.cached_len for req in reqs], dtype=torch.int32,
                                     device=device)
        if device.type == "cuda":
            m = self._device_metadata(reqs, kv_lens, None)
            return DecodeMetadata(positions=positions, kv_indptr=m["kv_indptr"],
                                  kv_indices=m["kv_indices"], num_kv_splits=m["num_kv_splits"],
                                  max_kv_splits=MAX_KV_SPLITS)
        return DecodeMetadata(
            positions=positions,
            kv_indptr=_build_indptr(kv_lens, device),
            kv_indices=self._gather_indices(reqs, kv_lens),
            num_kv_splits=_compute_num_kv_splits(kv_lens, device),
            max_kv_splits=MAX_KV_SPLITS,
        )


def _build_indptr(lens: Sequence[int], device=None) -> torch.Tensor:
    """CSR row pointers ``cumsum([0] + lens)`` as int32 (backend.py:299-301)."""
    return torch.cumsum(torch.tensor([0] + list(lens), dtype=torch.int32), 0).to(
        dtype=torch.int32, device=device)


def _compute_num_kv_splits(kv_lens: Sequence[int], device=None) -> torch.Tensor:
    """The reference's split hint ``min(32, max(1, ceil(L / 128)))`` (backend.py:304-307)."""
    splits = [min(MAX_KV_SPLITS, max(1, (l + 127) // 128)) for l in kv_lens]
    return torch.tensor(splits, dtype=torch.int32, device=device)
