"""Pins the CPU oracle against the reference's own known-answer tests.

* the six closed-form mask cases and the store -> prefill reachability case of
  mini-sglang-mlx-kernel/test_and_bench/test_paged_prefill_attention_masks.py:97-158
  (q = k = 0 gives uniform weights over the visible keys; V rows are one-hot, so output
  row p, column j is 1/|visible(p)| iff key j is visible) -- expected values come from the
  closed form, not from the oracle;
* the row-loop equality of test_and_bench/store_kv_cache.py:43-120 on its five shapes.
"""
import math

import numpy as np
import pytest
import torch

import oracle

HEAD_DIM = 128

# (q_len, prefix_len, is_cross_attention, sliding_window_size), masks test :97-122
MASK_CASES = [
    (4, 0, False, 0),
    (4, 0, True, 0),
    (4, 0, False, 2),
    (4, 4, False, 5),
    (4, 4, True, 5),
    (2, 6, True, 3),
]


def uniform_case(q_len, prefix_len):
    kv_len = prefix_len + q_len
    q = torch.zeros((q_len, 1, HEAD_DIM), dtype=torch.bfloat16)
    k_cache = torch.zeros((kv_len, 1, HEAD_DIM), dtype=torch.bfloat16)
    v = torch.zeros((kv_len, 1, HEAD_DIM), dtype=torch.float32)
    for pos in range(kv_len):
        v[pos, 0, pos] = 1.0
    return dict(
        q=q, k_cache=k_cache, v_cache=v.to(torch.bfloat16),
        qo_indptr=torch.tensor([0, q_len], dtype=torch.int32),
        kv_indptr=torch.tensor([0, kv_len], dtype=torch.int32),
        kv_indices=torch.arange(kv_len, dtype=torch.int32),
        prefix_lens=torch.tensor([prefix_len], dtype=torch.int32))


def expected_weights(q_len, prefix_len, is_cross, window):
    """Closed form: 1/|visible| on visible keys (masks test :60-72)."""
    kv_len = prefix_len + q_len
    w = np.zeros((q_len, kv_len), dtype=np.float32)
    for p in range(q_len):
        pos = prefix_len + p
        attend = [k for k in range(kv_len)
                  if (window == 0 or k >= pos - window + 1) and (is_cross or k <= pos)]
        w[p, attend] = 1.0 / len(attend)
    return w


@pytest.mark.parametrize("q_len,prefix_len,is_cross,window", MASK_CASES)
def test_mask_cases_closed_form(q_len, prefix_len, is_cross, window):
    d = uniform_case(q_len, prefix_len)
    out = oracle.paged_prefill_attention(
        d["q"], d["k_cache"], d["v_cache"], d["qo_indptr"], d["kv_indptr"], d["kv_indices"],
        d["prefix_lens"], 1.0 / math.sqrt(HEAD_DIM), q_len, is_cross_attention=is_cross,
        sliding_window_size=window)
    actual = out.float().numpy()[:, 0, : prefix_len + q_len]
    np.testing.assert_allclose(actual, expected_weights(q_len, prefix_len, is_cross, window),
                               rtol=1e-3, atol=1e-3)
    # dims beyond kv_len see only zero V entries
    assert np.all(out.float().numpy()[:, 0, prefix_len + q_len:] == 0)


def test_store_then_prefill_reaches_written_slots():
    # masks test :125-158: slots [3,1,4,2] of a 5-slot pool
    q_len = 4
    page_ids = torch.tensor([3, 1, 4, 2], dtype=torch.int32)
    q = torch.zeros((q_len, 1, HEAD_DIM), dtype=torch.bfloat16)
    k = torch.zeros((q_len, 1, HEAD_DIM), dtype=torch.bfloat16)
    v = torch.zeros((q_len, 1, HEAD_DIM), dtype=torch.float32)
    for pos in range(q_len):
        v[pos, 0, pos] = 1.0
    v = v.to(torch.bfloat16)
    k_cache = torch.zeros((5, 1, HEAD_DIM), dtype=torch.bfloat16)
    v_cache = torch.zeros((5, 1, HEAD_DIM), dtype=torch.bfloat16)
    oracle.store_kv_cache(k_cache, v_cache, page_ids, k, v)
    out = oracle.paged_prefill_attention(
        q, k_cache, v_cache, torch.tensor([0, q_len], dtype=torch.int32),
        torch.tensor([0, q_len], dtype=torch.int32), page_ids,
        torch.tensor([0], dtype=torch.int32), 1.0 / math.sqrt(HEAD_DIM), q_len)
    np.testing.assert_allclose(out.float().numpy()[:, 0, :q_len],
                               expected_weights(q_len, 0, False, 0), rtol=1e-3, atol=1e-3)
    assert torch.all(v_cache[0] == 0), "slot 0 was not listed and must stay untouched"


# (length, num_pages, num_kv_heads, head_dim), store_kv_cache.py:113-120
STORE_SHAPES = [(1, 128, 4, 128), (3, 128, 4, 128), (32, 128, 4, 128), (67, 256, 8, 128),
                (129, 512, 16, 128)]


@pytest.mark.parametrize("length,num_pages,n_kv,d", STORE_SHAPES)
def test_store_matches_row_loop(length, num_pages, n_kv, d):
    g = torch.Generator().manual_seed(1025)
    k = torch.randn((length, n_kv, d), generator=g).to(torch.bfloat16)
    v = torch.randn((length, n_kv, d), generator=g).to(torch.bfloat16)
    out_loc = torch.randperm(num_pages, generator=g)[:length].to(torch.int32)
    k_cache = torch.zeros((num_pages, n_kv, d), dtype=torch.bfloat16)
    v_cache = torch.zeros((num_pages, n_kv, d), dtype=torch.bfloat16)
    oracle.store_kv_cache(k_cache, v_cache, out_loc, k, v)
    # naive row loop of store_kv_cache.py:43-58, on bit patterns
    k_ref = torch.zeros_like(k_cache)
    v_ref = torch.zeros_like(v_cache)
    for r in range(length):
        k_ref[int(out_loc[r])] = k[r]
        v_ref[int(out_loc[r])] = v[r]
    assert torch.equal(k_cache.view(torch.int16), k_ref.view(torch.int16))
    assert torch.equal(v_cache.view(torch.int16), v_ref.view(torch.int16))


def test_store_honours_all_four_strides_and_overwrites():
    g = torch.Generator().manual_seed(7)
    n_kv, d = 2, 8
    kbig = torch.randn((6, 3, n_kv, d), generator=g).to(torch.bfloat16)
    k = kbig[:, 1]  # stride0 = 3 rows
    v = torch.randn((6, n_kv, d), generator=g).to(torch.bfloat16)
    kc_big = torch.randn((10, 2, n_kv, d), generator=g).to(torch.bfloat16)
    k_cache = kc_big[:, 0]
    v_cache = torch.randn((10, n_kv, d), generator=g).to(torch.bfloat16)
    before_v = v_cache.clone()
    idx = torch.tensor([9, 0, 4, 5, 2, 7], dtype=torch.int32)
    oracle.store_kv_cache(k_cache, v_cache, idx, k, v)
    for r in range(6):
        assert torch.equal(k_cache[int(idx[r])], k[r])
        assert torch.equal(v_cache[int(idx[r])], v[r])
    for s in (1, 3, 6, 8):
        assert torch.equal(v_cache[s], before_v[s])
    assert torch.equal(kc_big[:, 1], kc_big[:, 1])  # neighbouring plane untouched by stride
    # second store to the same slots replaces the rows
    oracle.store_kv_cache(k_cache, v_cache, idx, v, k.contiguous())
    assert torch.equal(k_cache[9], v[0]) and torch.equal(v_cache[9], k[0])
