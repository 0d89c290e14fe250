"""CPU restatement (numpy) of the reference's attention-metadata builders.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; the product path never touches it.

Follows mini_sglang_mlx/attention/backend.py:
  * ``build_indptr``            ``_build_indptr``                 :299-301
  * ``compute_num_kv_splits``   ``_compute_num_kv_splits``        :304-307
  * ``build_prefill_metadata``  ``build_prefill_metadata``        :205-257
  * ``build_decode_metadata``   ``build_decode_metadata``         :259-293

Pinned by closed forms that do not retype these formulas (tests/test_oracle_metadata.py):
an identity slot table turns ``kv_indices`` into ``row * max_seq_len + arange(kv_len)``;
``kv_indptr`` differences give back the lengths; positions of a request are consecutive,
start at ``prefix`` and end at ``kv_len - 1``; the split hint is checked against the
step function ``L in (128 (s-1), 128 s] -> s`` up to the cap.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import numpy as np

MAX_KV_SPLITS = 32  # backend.py:15


def build_indptr(lens: Sequence[int]) -> np.ndarray:
    out = np.zeros(len(lens) + 1, dtype=np.int64)
    for i, n in enumerate(lens):  # running sum of [0] + lens
        out[i + 1] = out[i] + int(n)
    return out.astype(np.int32)


def compute_num_kv_splits(kv_lens: Sequence[int], max_kv_splits: int = MAX_KV_SPLITS) -> np.ndarray:
    return np.array([min(max_kv_splits, max(1, (int(n) + 127) // 128)) for n in kv_lens],
                    dtype=np.int32)


def _gather(page_table: np.ndarray, table_rows: Sequence[int], kv_lens: Sequence[int]) -> np.ndarray:
    parts = [page_table[int(r), : int(n)] for r, n in zip(table_rows, kv_lens)]
    return (np.concatenate(parts) if parts else np.zeros(0, np.int32)).astype(np.int32)


def build_prefill_metadata(page_table: np.ndarray, table_rows: Sequence[int],
                           kv_lens: Sequence[int], extend_lens: Sequence[int]) -> Dict[str, np.ndarray]:
    cached = [int(k) - int(e) for k, e in zip(kv_lens, extend_lens)]
    pos = [np.arange(c, int(k), dtype=np.int32) for c, k in zip(cached, kv_lens)]
    return {
        "positions": np.concatenate(pos) if pos else np.zeros(0, np.int32),
        "qo_indptr": build_indptr(extend_lens),
        "kv_indptr": build_indptr(kv_lens),
        "kv_indices": _gather(page_table, table_rows, kv_lens),
        "prefix_lens": np.array(cached, dtype=np.int32),
        "num_kv_splits": compute_num_kv_splits(kv_lens),
        "max_len_extend": max([int(e) for e in extend_lens], default=0),
    }


def build_decode_metadata(page_table: np.ndarray, table_rows: Sequence[int],
                          kv_lens: Sequence[int],
                          positions: Optional[Sequence[int]] = None) -> Dict[str, np.ndarray]:
    if positions is None:  # req.cached_len = device_len - 1 while decoding (core.py:74-76)
        positions = [int(k) - 1 for k in kv_lens]
    return {
        "positions": np.array(positions, dtype=np.int32),
        "kv_indptr": build_indptr(kv_lens),
        "kv_indices": _gather(page_table, table_rows, kv_lens),
        "num_kv_splits": compute_num_kv_splits(kv_lens),
        "max_kv_splits": MAX_KV_SPLITS,
    }
