"""Writes the committed fixtures of this directory.  Run from the repository root:

    python tests/golden/make_fixtures.py

* ``reference_mask_cases.json`` -- the known-answer cases of the reference's own test
  (mini-sglang-mlx-kernel/test_and_bench/test_paged_prefill_attention_masks.py:97-158) as
  data: case parameters and the expected attention-weight matrix of every case, as exact
  fractions.  With q = k = 0 every visible key gets the same weight, so the expected row is
  1/|visible| on the visible keys; visibility is enumerated here from the mask definition
  (paged_prefill_attention.metal:339-347), not taken from any implementation.
* ``small_random_cases.npz`` -- three small seeded workloads (decode, causal extend with
  prefix, bidirectional window extend) with their inputs and the float64 oracle's outputs,
  so the HIP path is also compared with vectors that do not move when the oracle's code does.
  The oracle that wrote them is the one pinned by tests/test_oracle_known_answers.py and
  tests/test_oracle_math.py.
"""
from __future__ import annotations

import json
import os
import sys
from fractions import Fraction

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "mini-sglang-mlx_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

MASK_CASES = [  # (q_len, prefix_len, is_cross_attention, sliding_window_size)
    (4, 0, False, 0), (4, 0, True, 0), (4, 0, False, 2), (4, 4, False, 5), (4, 4, True, 5),
    (2, 6, True, 3),
]


def visible(q_pos: int, kv_pos: int, is_cross: bool, window: int) -> bool:
    upper = is_cross or kv_pos <= q_pos
    lower = window == 0 or kv_pos >= q_pos - window + 1
    return upper and lower


def mask_fixture():
    cases = []
    for q_len, prefix, cross, window in MASK_CASES:
        kv_len = prefix + q_len
        rows = []
        for p in range(q_len):
            vis = [j for j in range(kv_len) if visible(prefix + p, j, cross, window)]
            rows.append([str(Fraction(1, len(vis))) if j in vis else "0" for j in range(kv_len)])
        cases.append({"q_len": q_len, "prefix_len": prefix, "is_cross_attention": cross,
                      "sliding_window_size": window, "kv_len": kv_len, "weights": rows})
    store_case = {"slots": [3, 1, 4, 2], "pool_slots": 5, "q_len": 4,
                  "weights": [[str(Fraction(1, p + 1)) if j <= p else "0" for j in range(4)]
                              for p in range(4)]}
    return {"source": "test_paged_prefill_attention_masks.py:97-158", "head_dim": 128,
            "construction": "q = k = 0, V row j is the one-hot vector e_j, one kv head, one q head",
            "mask_cases": cases, "store_then_prefill": store_case}


def random_fixture():
    import oracle
    from mini_sglang_amd.workloads import build_workload

    out = {}
    specs = {
        "decode": dict(kind="decode", seed=9001, n_q=8, n_kv=1, kv_lens=[1, 37, 150]),
        "extend_causal": dict(kind="prefill", seed=9002, n_q=4, n_kv=2, kv_lens=[5, 40, 75],
                              extend_lens=[5, 9, 40], store_new=True),
        "extend_window_cross": dict(kind="prefill", seed=9003, n_q=4, n_kv=1, kv_lens=[40, 90],
                                    extend_lens=[7, 33], store_new=True, is_cross_attention=True,
                                    sliding_window_size=16),
    }
    for name, spec in specs.items():
        kind = spec.pop("kind")
        wl = build_workload(name, kind, pool_factor=1.1, **spec)
        if wl.out_loc is not None:
            oracle.store_kv_cache(wl.k_cache, wl.v_cache, wl.out_loc, wl.new_k, wl.new_v)
        if kind == "decode":
            ref = oracle.paged_decode_attention(wl.q, wl.k_cache, wl.v_cache, wl.kv_indptr,
                                                wl.kv_indices, wl.num_kv_splits, wl.sm_scale,
                                                wl.max_kv_splits, return_f32=True)
        else:
            ref = oracle.paged_prefill_attention(
                wl.q, wl.k_cache, wl.v_cache, wl.qo_indptr, wl.kv_indptr, wl.kv_indices,
                wl.prefix_lens, wl.sm_scale, wl.max_len_extend,
                is_cross_attention=wl.is_cross_attention,
                sliding_window_size=wl.sliding_window_size, return_f32=True)
        bits = lambda t: t.view(torch.int16).numpy()
        out[f"{name}.q"] = bits(wl.q)
        out[f"{name}.k_cache"] = bits(wl.k_cache)  # after the store
        out[f"{name}.v_cache"] = bits(wl.v_cache)
        out[f"{name}.kv_indptr"] = wl.kv_indptr.numpy()
        out[f"{name}.kv_indices"] = wl.kv_indices.numpy()
        if kind != "decode":
            out[f"{name}.qo_indptr"] = wl.qo_indptr.numpy()
            out[f"{name}.prefix_lens"] = wl.prefix_lens.numpy()
            out[f"{name}.flags"] = np.array([wl.max_len_extend, int(wl.is_cross_attention),
                                             wl.sliding_window_size], dtype=np.int32)
        out[f"{name}.sm_scale"] = np.array([wl.sm_scale], dtype=np.float64)
        out[f"{name}.expected_f32"] = ref[1].numpy().astype(np.float32)  # (bf16, f32) pair
    return out


if __name__ == "__main__":
    with open(os.path.join(HERE, "reference_mask_cases.json"), "w") as f:
        json.dump(mask_fixture(), f, indent=1)
    np.savez_compressed(os.path.join(HERE, "small_random_cases.npz"), **random_fixture())
    print("wrote", sorted(os.listdir(HERE)))
