"""Algorithmic work of the paged-attention path and the MI355X peaks it is priced against.

Algorithmic bytes count every visible K row and V row once per kv head, 4 bytes per
``kv_indices`` entry of a visible token, and q and o once; workspace traffic and re-reads are
not counted.  Algorithmic flops count ``4 * head_dim`` per visible (query, key) pair and q
head (QK^T and PV), softmax excluded.
"""
from __future__ import annotations

from typing import Sequence

HBM_PEAK_BYTES_PER_S = 8.0e12  # MI355X HBM3E
MFMA_BF16_PEAK_FLOPS = 2.5e15  # MI355X dense bf16
ELEM_BYTES = 2  # bf16


def visible_range(prefix: int, q_len: int, kv_len: int, is_cross: bool, window: int):
    """Keys ``[lo, hi)`` visible to at least one of the ``q_len`` queries of a request."""
    if q_len <= 0:
        return 0, 0
    hi = kv_len if is_cross else min(kv_len, prefix + q_len)
    lo = max(0, prefix - window + 1) if window > 0 else 0
    return (lo, hi) if hi > lo else (0, 0)


def visible_pairs(prefix: int, q_len: int, kv_len: int, is_cross: bool, window: int) -> int:
    """Number of visible (query, key) pairs of a request (closed form of the mask predicate)."""
    total = 0
    for i in range(q_len):
        pos = prefix + i
        hi = kv_len - 1 if is_cross else min(pos, kv_len - 1)
        lo = max(0, pos - window + 1) if window > 0 else 0
        total += max(0, hi - lo + 1)
    return total


def attention_bytes(prefixes: Sequence[int], q_lens: Sequence[int], kv_lens: Sequence[int],
                    n_q: int, n_kv: int, d: int, is_cross: bool = False, window: int = 0) -> int:
    tokens = 0
    for p, ql, kl in zip(prefixes, q_lens, kv_lens):
        lo, hi = visible_range(p, ql, kl, is_cross, window)
        tokens += hi - lo
    qo = 2 * sum(q_lens) * n_q * d * ELEM_BYTES
    return tokens * (2 * n_kv * d * ELEM_BYTES + 4) + qo


def decode_bytes(kv_lens: Sequence[int], n_q: int, n_kv: int, d: int) -> int:
    return attention_bytes([l - 1 for l in kv_lens], [1] * len(kv_lens), kv_lens, n_q, n_kv, d)


def attention_flops(prefixes: Sequence[int], q_lens: Sequence[int], kv_lens: Sequence[int],
                    n_q: int, d: int, is_cross: bool = False, window: int = 0) -> int:
    pairs = sum(visible_pairs(p, ql, kl, is_cross, window)
                for p, ql, kl in zip(prefixes, q_lens, kv_lens))
    return 4 * d * n_q * pairs


def store_bytes(n_tokens: int, n_kv: int, d: int) -> int:
    row = n_kv * d * ELEM_BYTES
    return n_tokens * (2 * row + 2 * row + 4)
