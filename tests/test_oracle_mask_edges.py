"""The oracle's masks at realistic lengths against the closed form of tests/_mask_edges.py, and the
proof that the closed form notices a single key: the same check must fail when the oracle is run
with a window that is one key too wide, or without the causal limit."""
import pytest

import oracle
from _mask_edges import assert_edges, one_hot_values
from mini_sglang_amd.workloads import build_workload


def _oracle_prefill(wl, window=None, cross=None):
    return oracle.paged_prefill_attention(
        wl.q, wl.k_cache, wl.v_cache, wl.qo_indptr, wl.kv_indptr, wl.kv_indices, wl.prefix_lens,
        wl.sm_scale, wl.max_len_extend,
        is_cross_attention=wl.is_cross_attention if cross is None else cross,
        sliding_window_size=wl.sliding_window_size if window is None else window,
        precision="f64", return_f32=True)[1].numpy()


@pytest.mark.parametrize("is_cross,window", [(False, 0), (False, 1024), (False, 100), (True, 0)])
def test_oracle_prefill_matches_the_closed_form(is_cross, window):
    wl = one_hot_values(build_workload(
        "e", "prefill", seed=9, n_q=4, n_kv=2, kv_lens=[2000 + 20, 130, 1024 + 9],
        extend_lens=[20, 130, 9], is_cross_attention=is_cross, sliding_window_size=window))
    assert_edges(_oracle_prefill(wl), wl, f"oracle cross={is_cross} W={window}")


def test_oracle_decode_matches_the_closed_form():
    wl = one_hot_values(build_workload("e", "decode", seed=9, n_q=4, n_kv=2, kv_lens=[37, 2500, 5001]))
    out = oracle.paged_decode_attention(wl.q, wl.k_cache, wl.v_cache, wl.kv_indptr, wl.kv_indices,
                                        wl.num_kv_splits, wl.sm_scale, wl.max_kv_splits,
                                        precision="f64", return_f32=True)[1].numpy()
    assert_edges(out, wl, "oracle decode", decode=True)


def test_the_closed_form_notices_one_key():
    wl = one_hot_values(build_workload(
        "e", "prefill", seed=10, n_q=4, n_kv=2, kv_lens=[3000 + 12], extend_lens=[12],
        sliding_window_size=1024))
    assert_edges(_oracle_prefill(wl), wl, "as specified")
    with pytest.raises(AssertionError, match="one key weighs"):
        assert_edges(_oracle_prefill(wl, window=1025), wl, "window one key too wide")
    with pytest.raises(AssertionError, match="one key weighs"):
        assert_edges(_oracle_prefill(wl, window=1023), wl, "window one key too narrow")
    wl.sliding_window_size = 0
    assert_edges(_oracle_prefill(wl), wl, "causal")
    with pytest.raises(AssertionError, match="one key weighs"):
        assert_edges(_oracle_prefill(wl, cross=True), wl, "causal limit dropped")
