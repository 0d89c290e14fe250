"""The committed fixtures of tests/golden/ against the CPU oracle (always) and the HIP path
(GPU): the reference's known-answer mask cases as data, and small seeded workloads whose
expected outputs were written once by the float64 oracle."""
import json
import math
import os
from fractions import Fraction

import numpy as np
import pytest
import torch

import oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _mask_cases():
    with open(os.path.join(GOLDEN, "reference_mask_cases.json")) as f:
        return json.load(f)


def _uniform_inputs(q_len, kv_len, d):
    q = torch.zeros((q_len, 1, d), dtype=torch.bfloat16)
    k = torch.zeros((kv_len, 1, d), dtype=torch.bfloat16)
    v = torch.zeros((kv_len, 1, d), dtype=torch.float32)
    for j in range(kv_len):
        v[j, 0, j] = 1.0
    return q, k, v.to(torch.bfloat16)


def _run_mask_case(case, d, fn, device):
    q_len, kv_len = case["q_len"], case["kv_len"]
    q, k, v = _uniform_inputs(q_len, kv_len, d)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=device)
    out = fn(q.to(device), k.to(device), v.to(device), i32([0, q_len]), i32([0, kv_len]),
             torch.arange(kv_len, dtype=torch.int32, device=device), i32([case["prefix_len"]]),
             1.0 / math.sqrt(d), q_len, is_cross_attention=case["is_cross_attention"],
             sliding_window_size=case["sliding_window_size"])
    want = np.array([[float(Fraction(x)) for x in row] for row in case["weights"]], dtype=np.float32)
    got = out.float().cpu().numpy()[:, 0, :]
    np.testing.assert_allclose(got[:, :kv_len], want, rtol=1e-3, atol=1e-3)
    assert np.all(got[:, kv_len:] == 0)


@pytest.mark.parametrize("idx", range(6))
def test_reference_mask_cases_on_the_oracle(idx):
    fx = _mask_cases()
    _run_mask_case(fx["mask_cases"][idx], fx["head_dim"], oracle.paged_prefill_attention, "cpu")


@pytest.mark.gpu
@pytest.mark.parametrize("idx", range(6))
def test_reference_mask_cases_on_the_gpu(gpu, idx):
    from mini_sglang_amd_kernel import paged_prefill_attention

    fx = _mask_cases()
    print(f"golden mask case {idx}", flush=True)
    _run_mask_case(fx["mask_cases"][idx], fx["head_dim"], paged_prefill_attention, gpu)
    torch.cuda.synchronize()


def _load_random(name):
    z = np.load(os.path.join(GOLDEN, "small_random_cases.npz"))  # allow_pickle stays False
    g = {k.split(".", 1)[1]: z[k] for k in z.files if k.startswith(name + ".")}
    bf = lambda a: torch.from_numpy(a.copy()).view(torch.bfloat16)
    return g, bf


def _run_random(name, dev, decode_fn, prefill_fn):
    g, bf = _load_random(name)
    t = lambda a: torch.from_numpy(a.copy()).to(dev)
    q, kc, vc = bf(g["q"]).to(dev), bf(g["k_cache"]).to(dev), bf(g["v_cache"]).to(dev)
    scale = float(g["sm_scale"][0])
    if name == "decode":
        b = g["kv_indptr"].size - 1
        out = decode_fn(q, kc, vc, t(g["kv_indptr"]), t(g["kv_indices"]),
                        torch.ones(b, dtype=torch.int32, device=dev), scale, 32)
    else:
        mle, cross, window = (int(x) for x in g["flags"])
        out = prefill_fn(q, kc, vc, t(g["qo_indptr"]), t(g["kv_indptr"]), t(g["kv_indices"]),
                         t(g["prefix_lens"]), scale, mle, is_cross_attention=bool(cross),
                         sliding_window_size=window)
    diff = np.abs(out.float().cpu().numpy() - g["expected_f32"])
    assert diff.max() <= 2e-2 and diff.mean() <= 2e-3, (name, float(diff.max()), float(diff.mean()))


@pytest.mark.parametrize("name", ["decode", "extend_causal", "extend_window_cross"])
def test_small_random_cases_on_the_oracle(name):
    _run_random(name, "cpu", oracle.paged_decode_attention, oracle.paged_prefill_attention)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["decode", "extend_causal", "extend_window_cross"])
def test_small_random_cases_on_the_gpu(gpu, name):
    from mini_sglang_amd_kernel import paged_decode_attention, paged_prefill_attention

    print(f"golden random case {name}", flush=True)
    _run_random(name, gpu, paged_decode_attention, paged_prefill_attention)
    torch.cuda.synchronize()
