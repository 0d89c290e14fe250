"""Helpers shared by the test modules."""
from __future__ import annotations

import math

import numpy as np
import torch

MAX_ABS_TOL = 2e-2   # tolerance of the path on bf16 outputs vs the oracle
MEAN_ABS_TOL = 2e-3


def bf16_randn(shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float32).to(torch.bfloat16)


def indptr(lens):
    return torch.cumsum(torch.tensor([0] + list(lens), dtype=torch.int64), 0).to(torch.int32)


def assert_close_bf16(actual: torch.Tensor, expected: torch.Tensor, what: str = "",
                      max_tol: float = MAX_ABS_TOL, mean_tol: float = MEAN_ABS_TOL):
    a = actual.detach().float().cpu()
    e = expected.detach().float().cpu()
    assert a.shape == e.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(e.shape)}"
    assert torch.isfinite(a).all(), f"{what}: non-finite values in the result"
    diff = (a - e).abs()
    mx = float(diff.max()) if diff.numel() else 0.0
    mean = float(diff.mean()) if diff.numel() else 0.0
    assert mx <= max_tol and mean <= mean_tol, (
        f"{what}: max-abs {mx:.3e} (tol {max_tol}), mean-abs {mean:.3e} (tol {mean_tol})")
    return mx, mean


def dense_attention_f64(q, k_cache, v_cache, qo_indptr, kv_indptr, kv_indices, prefix_lens,
                        sm_scale, is_cross=False, window=0):
    """Textbook softmax(scale * Q K^T + mask) V in numpy float64, written independently of
    the C oracle (matrix form, explicit mask matrix, numpy softmax)."""
    qf = q.float().numpy().astype(np.float64)
    kf = k_cache.float().numpy().astype(np.float64)
    vf = v_cache.float().numpy().astype(np.float64)
    total_q, n_q, d = qf.shape
    n_kv = kf.shape[1]
    group = n_q // n_kv
    out = np.zeros((total_q, n_q, d))
    qo, kv = qo_indptr.tolist(), kv_indptr.tolist()
    idx = kv_indices.numpy()
    for b in range(len(qo) - 1):
        qn, kn = qo[b + 1] - qo[b], kv[b + 1] - kv[b]
        if qn == 0:
            continue
        slots = idx[kv[b]:kv[b + 1]]
        pos = int(prefix_lens[b]) + np.arange(qn)[:, None]
        j = np.arange(kn)[None, :]
        vis = np.ones((qn, kn), dtype=bool)
        if not is_cross:
            vis &= j <= pos
        if window > 0:
            vis &= j >= pos - window + 1
        for h in range(n_q):
            kk = kf[slots, h // group, :]
            vv = vf[slots, h // group, :]
            s = (qf[qo[b]:qo[b + 1], h, :] @ kk.T) * sm_scale
            s = np.where(vis, s, -np.inf)
            with np.errstate(invalid="ignore"):
                m = np.max(s, axis=1, keepdims=True) if kn else np.zeros((qn, 1))
                m = np.where(np.isfinite(m), m, 0.0)
                p = np.exp(s - m)
                den = p.sum(axis=1, keepdims=True)
                w = np.where(den > 0, p / np.where(den > 0, den, 1.0), 0.0)
            out[qo[b]:qo[b + 1], h, :] = w @ vv
    return torch.from_numpy(out)
