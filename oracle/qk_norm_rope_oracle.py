"""CPU restatement (numpy) of what the reference's Qwen3 attention layer does to q, k and v
between the projections and the attention call.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; the product path never touches it.

Follows
  * mini_sglang_mlx/models/qwen3.py:60-68        q_norm / k_norm on (L, heads, head_dim), rope on both
  * mini_sglang_mlx/layers/rotary_embedding.py:17-21   nn.RoPE(rotary_dim, base=...) with the
    positions as per-token offsets, sequence axis of length one
  * mini_sglang_mlx/attention/backend.py:139     the store of k, v at out_loc before attention
  * mini_sglang_mlx/kvcache/mha_pool.py:36-49    k_cache[out_loc] = k, v_cache[out_loc] = v

``nn.RMSNorm`` and ``nn.RoPE`` live in MLX (mlx >= 0.31.2, requirements.txt:13), which is not
part of the reference tree and not installed here.  Their published definitions are restated:
  RMSNorm (mx.fast.rms_norm):  y = w * (x * rsqrt(mean(x^2, axis=-1) + eps)), statistics in
      float32, result in the input dtype.  The normalised value is rounded to the input dtype
      before the multiplication by w, whose product is rounded again.
  RoPE (mx.fast.rope, traditional=False, scale=1):  with h = dims / 2 and
      theta_i = float32(position) * exp2(-(i / h) * log2(base)) in float32,
      out[i] = x[i] cos(theta_i) - x[i + h] sin(theta_i),
      out[i + h] = x[i] sin(theta_i) + x[i + h] cos(theta_i), result in the input dtype.
PARITY UNPINNED at the bit level of those two MLX kernels (where exactly they round, how they
evaluate exp2 / sin / cos): nothing in the reference tree holds their outputs.  What the
mathematics fixes is pinned in tests/test_oracle_qk_norm_rope.py without retyping these
formulas: position 0 is the identity rotation; a rotation keeps the norm of every pair; the
dot product of a rotated q and k depends only on the difference of their positions; against
numpy's complex multiplication; the norm of a constant vector; scale invariance of the norm;
torch.nn.functional.rms_norm as an independent library routine.
"""
from __future__ import annotations

from typing import Tuple

import numpy as np


def bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest bfloat16 (ties to even), returned as float32."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(x))


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """x: (..., d) float32 holding bf16 values; weight (d,) likewise.  Returns bf16 values."""
    x64 = x.astype(np.float64)
    norm = 1.0 / np.sqrt(np.mean(x64 * x64, axis=-1, keepdims=True) + eps)
    y = bf16_round((x64 * norm).astype(np.float32))
    return bf16_round(weight.astype(np.float32) * y)


def rope_angles(positions: np.ndarray, dims: int, base: float) -> np.ndarray:
    """theta[t, i] in float32, computed in float32 as the kernel that is restated does."""
    h = dims // 2
    d = (np.arange(h, dtype=np.float32) / np.float32(h)).astype(np.float32)
    inv_freq = np.exp2((-d * np.float32(np.log2(base))).astype(np.float32)).astype(np.float32)
    return (positions.astype(np.float32)[:, None] * inv_freq[None, :]).astype(np.float32)


def rope(x: np.ndarray, positions: np.ndarray, base: float) -> np.ndarray:
    """x: (L, heads, d) float32 holding bf16 values; rotate-half form over the whole head."""
    L, H, D = x.shape
    h = D // 2
    theta = rope_angles(positions, D, base).astype(np.float64)
    c, s = np.cos(theta)[:, None, :], np.sin(theta)[:, None, :]
    x1, x2 = x[..., :h].astype(np.float64), x[..., h:].astype(np.float64)
    out = np.concatenate([x1 * c - x2 * s, x1 * s + x2 * c], axis=-1)
    return bf16_round(out.astype(np.float32))


def qk_norm_rope_store(q: np.ndarray, k: np.ndarray, v: np.ndarray, q_weight: np.ndarray,
                       k_weight: np.ndarray, positions: np.ndarray, out_loc: np.ndarray,
                       k_cache: np.ndarray, v_cache: np.ndarray, eps: float,
                       base: float) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """Returns (q_out, k_cache, v_cache); the pools are copies with rows out_loc replaced."""
    q_out = rope(rms_norm(q, q_weight, eps), positions, base)
    k_out = rope(rms_norm(k, k_weight, eps), positions, base)
    kc, vc = k_cache.copy(), v_cache.copy()
    for r, slot in enumerate(out_loc):
        kc[int(slot)] = k_out[r]
        vc[int(slot)] = v[r]
    return q_out, kc, vc
