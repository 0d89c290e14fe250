"""CPU restatement (numpy, float64) of the reference's gated delta-rule state kernel.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; the product path never touches it.

Follows mini-sglang-mlx-kernel/csrc/gdn_state.metal:14-99 (one state row per simdgroup,
the token loop :72-95) and the host side gdn_state.cpp:87-183 (shapes, decode mode :107-111,
grid :176-178).  Per request b, S = state[slot_ids[b]] (hv, dv, dk), per token t in order:
    S *= g[t, h]                                             (:78)
    kv = S[h] @ k[t, h // (hv // hk)]                         (:79)
    delta = (v[t, h] - kv) * beta[t, h]                       (:80-81)
    S[h] += outer(delta, k)                                   (:83)
    y[t, h] = S[h] @ q[t, h // (hv // hk)], rounded to bf16   (:84-87)

Pinned (tests/test_oracle_gdn_state.py) by facts that do not retype the update: one-hot keys
with g = beta = 1 from a zero state store v_t in column t and read it back exactly; beta = 0
leaves pure decay, S_T = prod(g) S_0; g = 0 forgets everything before the token; after a token
with beta = 1 and a unit-norm key the state returns that token's v for that key (associative
recall); one call over T tokens equals T single-token calls and any split into two calls; y is
linear in (v, S_0) jointly.
"""
from __future__ import annotations

from typing import Optional, Tuple

import numpy as np


def _bf16_round(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(x))


def gdn_state_inplace(q: np.ndarray, k: np.ndarray, v: np.ndarray, g: np.ndarray,
                      beta: np.ndarray, state: np.ndarray, slot_ids: np.ndarray,
                      qo_indptr: Optional[np.ndarray], single_token_mode: bool = False,
                      round_output: bool = True) -> Tuple[np.ndarray, np.ndarray]:
    """q, k: (T, hk, dk); v: (T, hv, dv); g, beta: (T, hv); state: (slots, hv, dv, dk).
    Inputs hold the bf16 values as floats; returns (y (T, hv, dv), new state float32)."""
    T, hk, dk = q.shape
    hv, dv = v.shape[1], v.shape[2]
    rep = hv // hk
    st = state.astype(np.float64).copy()
    y = np.zeros((T, hv, dv), dtype=np.float64)
    for b, slot in enumerate(np.asarray(slot_ids).tolist()):
        lo, hi = (b, b + 1) if single_token_mode else (int(qo_indptr[b]), int(qo_indptr[b + 1]))
        S = st[slot]
        for t in range(lo, hi):
            kk = np.repeat(k[t].astype(np.float64), rep, axis=0)  # (hv, dk)
            qq = np.repeat(q[t].astype(np.float64), rep, axis=0)
            S = S * g[t].astype(np.float64)[:, None, None]
            kv = np.einsum("hvk,hk->hv", S, kk)
            delta = (v[t].astype(np.float64) - kv) * beta[t].astype(np.float64)[:, None]
            S = S + delta[:, :, None] * kk[:, None, :]
            y[t] = np.einsum("hvk,hk->hv", S, qq)
        st[slot] = S
    yf = y.astype(np.float32)
    return (_bf16_round(yf) if round_output else yf), st.astype(np.float32)
