"""Closed-form mask-edge workloads: q = 0 and V[key] = one-hot(key % head_dim) make the output of a
query count(visible keys congruent to d) / count(visible keys) in dimension d, so one key wrongly
seen or dropped shows as a change of 1 / n_visible.  Expected values follow the mask predicate
(mini-sglang-mlx-kernel/csrc/paged_prefill_attention.metal:339-347), not the oracle."""
import numpy as np
import torch


def one_hot_values(wl):
    """q := 0, V row of key k of every request := one-hot(k % head_dim) on every kv head."""
    d = wl.head_dim
    wl.q.zero_()
    indptr = wl.kv_indptr.tolist()
    eye = torch.eye(d, dtype=torch.bfloat16)
    for b in range(len(indptr) - 1):
        n = indptr[b + 1] - indptr[b]
        slots = wl.kv_indices[indptr[b]:indptr[b + 1]].long()
        rows = eye[torch.arange(n) % d]                      # (n, d)
        wl.v_cache[slots] = rows[:, None, :].expand(n, wl.n_kv, d).to(wl.v_cache.device)
    return wl


def expected(wl, decode):
    d = wl.head_dim
    rows = []
    for b, kn in enumerate(wl.kv_lens):
        q_len = 1 if decode else wl.extend_lens[b]
        prefix = kn - 1 if decode else kn - q_len
        for i in range(q_len):
            pos = prefix + i
            lo = max(0, pos - wl.sliding_window_size + 1) if wl.sliding_window_size > 0 else 0
            hi = kn - 1 if (wl.is_cross_attention and not decode) else min(pos, kn - 1)
            e = np.zeros(d)
            n = hi - lo + 1
            if n > 0:
                k = np.arange(lo, hi + 1)
                e = np.bincount(k % d, minlength=d) / n
            rows.append((e, max(n, 1)))
    return rows



def assert_edges(got, wl, what, decode=False):
    """got: (rows, n_q, d) float array."""
    for r, (e, n) in enumerate(expected(wl, decode)):
        tol = 0.35 / n + e * 2.0 ** -8             # under half a key's weight, over bf16 rounding
        err = np.abs(got[r] - e[None, :])
        assert (err <= tol[None, :]).all(), (
            f"{what}: row {r} off by {err.max():.3e} where one key weighs {1.0 / n:.3e}")
