"""Recurrence backend of the gated delta-rule (linear attention) layers.

Counterpart of ``GDNBackend`` (mini_sglang_mlx/attention/gdn_backend.py:37-221): the caller of
``gdn_state_inplace``, holding the ``MambaStatePool`` whose temporal state the kernel updates in
place.  Prefill, decode, and the replay-style handling of a speculative verify window:

* ``forward_verify`` runs the whole ``W = K + 1`` window of every request from its *scratch* slot
  (a copy of the main slot, made with ``MambaStatePool.copy_batched`` before the verify forward)
  and keeps the layer's inputs on the batch;
* ``commit_verify`` replays, per request, the accepted prefix of those inputs into the *main*
  slot and restores the conv window that belongs to that prefix.  A rollback is a replay length;
  no per-token snapshots of the state exist.

The backend covers the recurrence only; norm and output projection stay with the model layer.
Everything runs on the current stream; nothing here synchronises (the reference forces an
``mx.eval`` per call because its arrays are lazy, gdn_backend.py:56,67,216).
"""
from __future__ import annotations

from typing import List

import torch

from mini_sglang_amd_kernel import gdn_state_inplace


class GDNBackend:
    def __init__(self, mamba_pool) -> None:
        self.mamba_pool = mamba_pool

    # ---- per-batch metadata shared by all linear layers (gdn_backend.py:50-67) ----------------
    def prepare_batch(self, batch) -> None:
        device = self.mamba_pool.device
        if batch.mamba_slot_ids is None:
            slots = [req.mamba_slot for req in batch.reqs]
            assert all(slot is not None for slot in slots), "Missing mamba slot"
            batch.mamba_slot_ids = torch.tensor(slots, dtype=torch.int32, device=device)
        # one field for both phases: ragged token offsets in prefill, 0..batch in decode
        if batch.mamba_prefill_indptr is None:
            lens = torch.tensor([0] + [req.extend_len for req in batch.reqs], dtype=torch.int64)
            batch.mamba_prefill_indptr = torch.cumsum(lens, 0).to(torch.int32).to(device)

    # ---- one layer's recurrence over the batch (gdn_backend.py:69-98) --------------------------
    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor,
                beta: torch.Tensor, linear_layer_idx: int, batch) -> torch.Tensor:
        """``y`` of shape ``(tokens, hv, dv)``; the state of every request's slot is advanced."""
        assert batch.mamba_slot_ids is not None
        assert batch.mamba_prefill_indptr is not None
        return gdn_state_inplace(q, k, v, g, beta, self.mamba_pool.temporal_state(linear_layer_idx),
                                 batch.mamba_slot_ids, batch.mamba_prefill_indptr,
                                 single_token_mode=batch.is_decode)

    # ---- speculative verify (gdn_backend.py:100-135) ---------------------------------------------
    def forward_verify(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor,
                       beta: torch.Tensor, linear_layer_idx: int, batch) -> torch.Tensor:
        """The verify window of every request, run on its scratch slot; main slots untouched."""
        assert batch.mamba_scratch_slots is not None
        assert batch.mamba_verify_indptr is not None
        if batch.gdn_verify_captured is None:
            batch.gdn_verify_captured = {}
        batch.gdn_verify_captured[linear_layer_idx] = (q, k, v, g, beta)
        return gdn_state_inplace(q, k, v, g, beta, self.mamba_pool.temporal_state(linear_layer_idx),
                                 batch.mamba_scratch_slots, batch.mamba_verify_indptr,
                                 single_token_mode=False)

    def commit_verify(self, batch, num_accepted_host: List[int]) -> None:
        """Request ``i`` accepted ``j_i`` drafts: its main slot advances by the first ``j_i + 1``
        tokens of the window (gdn_backend.py:137-221).  ``window_width`` is read from the host
        copy of the geometry when the batch carries one, else from ``mamba_verify_indptr``."""
        captured = batch.gdn_verify_captured
        if not captured:
            return
        assert batch.mamba_slot_ids is not None
        assert batch.mamba_scratch_slots is not None
        assert batch.mamba_verify_indptr is not None
        device = self.mamba_pool.device
        width = getattr(batch, "mamba_verify_width", None)
        if width is None:
            width = int(batch.mamba_verify_indptr[1].item())  # uniform window: K + 1 tokens
        accepted = torch.tensor(list(num_accepted_host), dtype=torch.int64)
        lengths = accepted + 1
        if int(lengths.max()) > width or int(accepted.min()) < 0:
            raise ValueError("commit_verify: accepted counts must lie in [0, window width)")
        # flat positions of every request's accepted prefix in the (batch * width) verify tensors
        starts = torch.arange(len(lengths), dtype=torch.int64) * width
        idx = torch.cat([torch.arange(s, s + n) for s, n in zip(starts.tolist(), lengths.tolist())])
        idx = idx.to(device)
        indptr = torch.cat([torch.zeros(1, dtype=torch.int64), torch.cumsum(lengths, 0)])
        indptr = indptr.to(torch.int32).to(device)
        main = batch.mamba_slot_ids
        scratch = batch.mamba_scratch_slots.long()
        row = accepted.to(device)  # the conv window after j + 1 tokens is row j of the scratch slot
        for layer, (q, k, v, g, beta) in captured.items():
            gdn_state_inplace(q.index_select(0, idx), k.index_select(0, idx), v.index_select(0, idx),
                              g.index_select(0, idx), beta.index_select(0, idx),
                              self.mamba_pool.temporal_state(layer), main, indptr,
                              single_token_mode=False)
            conv = self.mamba_pool.conv_state(layer, 0)
            conv[main.long()] = self.mamba_pool.conv_window(layer, 0)[scratch, row]
        batch.gdn_verify_captured = None  # the verify inputs may be freed now
