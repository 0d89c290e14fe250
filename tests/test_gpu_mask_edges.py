"""Mask edges at realistic lengths, pinned by a closed form on every route.

With q = 0 every visible key gets the same weight, and with V[key] = one-hot(key % head_dim) the
output of a query is count(visible keys congruent to d) / count(visible keys) in dimension d.  One
key wrongly seen or wrongly dropped (an off-by-one in a window floor, a causal limit, a key-split
share or a segment cut) moves some dimension by about 1 / n_visible, which at these lengths is far
below the absolute tolerance of the random-data tests and far above bf16 rounding of the result.
The expected values come from the mask predicate
(mini-sglang-mlx-kernel/csrc/paged_prefill_attention.metal:339-347), not from the oracle."""
import pytest

from _mask_edges import assert_edges, one_hot_values
from mini_sglang_amd.workloads import build_workload

pytestmark = pytest.mark.gpu


def _check(wl, gpu, what, decode=False):
    from _gpu_util import run_gpu

    out, _ = run_gpu(wl, gpu, store=False)
    assert_edges(out.float().numpy(), wl, what, decode)


MASKS = [(False, 0), (False, 1024), (False, 100), (True, 0)]


@pytest.mark.parametrize("kv_lens", [[37, 2500, 9001], [4096] * 5 + [1, 64, 65]])
def test_decode_sees_every_key_once(gpu, kv_lens):
    wl = one_hot_values(build_workload("e", "decode", seed=5, n_q=16, n_kv=4, kv_lens=kv_lens,
                                        pool_factor=1.1))
    _check(wl, gpu, f"decode {kv_lens}", decode=True)


@pytest.mark.parametrize("is_cross,window", MASKS)
@pytest.mark.parametrize("q_len", [1, 8, 12, 16])
def test_split_k_route_mask_edges(gpu, tuning, q_len, is_cross, window):
    from mini_sglang_amd_kernel import _lib

    tuning(_lib.TUNE_SMALLQ_MAXCOLS, 64)  # 64 columns would go to the tile kernel by default
    wl = one_hot_values(build_workload(
        "e", "prefill", seed=6, n_q=16, n_kv=4, kv_lens=[q_len + 3000, q_len + 1023, q_len + 1024, q_len + 7777],
        extend_lens=[q_len] * 4, pool_factor=1.1, is_cross_attention=is_cross,
        sliding_window_size=window))
    _check(wl, gpu, f"split-K q_len={q_len} cross={is_cross} W={window}")


@pytest.mark.parametrize("is_cross,window", MASKS)
@pytest.mark.parametrize("head_dim,q_len", [(128, 16), (128, 50), (256, 8), (256, 30)])
def test_tile_route_ragged_shares_mask_edges(gpu, head_dim, q_len, is_cross, window):
    # one query block per (request, kv head) on the tile kernels: requests of 1 to 8 key shares
    wl = one_hot_values(build_workload(
        "e", "prefill", seed=8, n_q=16, n_kv=4, head_dim=head_dim, kv_lens=[q_len + 9000, q_len + 1023, q_len + 1024, q_len + 4100],
        extend_lens=[q_len] * 4, pool_factor=1.1, is_cross_attention=is_cross,
        sliding_window_size=window))
    _check(wl, gpu, f"tile route, ragged shares q_len={q_len} cross={is_cross} W={window}")


@pytest.fixture(params=[0, 1], ids=["pingpong", "fused"])
def tile_variant(request):
    from mini_sglang_amd_kernel import _lib

    _lib.set_tuning(_lib.TUNE_PREFILL_VARIANT, request.param)
    yield request.param
    _lib.set_tuning(_lib.TUNE_PREFILL_VARIANT, 0)


@pytest.mark.parametrize("is_cross,window", MASKS)
@pytest.mark.parametrize("key_splits", [0, 1, 3, 8])
def test_tile_route_mask_edges(gpu, tile_variant, key_splits, is_cross, window):
    from mini_sglang_amd_kernel import _lib

    wl = one_hot_values(build_workload(
        "e", "prefill", seed=7, n_q=8, n_kv=2, kv_lens=[5000 + 300, 130, 1024 + 65, 2047 + 257],
        extend_lens=[300, 130, 65, 257], pool_factor=1.1, is_cross_attention=is_cross,
        sliding_window_size=window))
    _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, key_splits)
    try:
        _check(wl, gpu, f"tile variant={tile_variant} splits={key_splits} cross={is_cross} W={window}")
    finally:
        _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, 0)


@pytest.mark.parametrize("is_cross,window", MASKS)
@pytest.mark.parametrize("key_splits", [0, 4])
def test_head_dim_256_mask_edges(gpu, key_splits, is_cross, window):
    from mini_sglang_amd_kernel import _lib

    wl = one_hot_values(build_workload(
        "e", "prefill", seed=8, n_q=8, n_kv=2, head_dim=256, kv_lens=[3000 + 150, 70, 1025 + 8],
        extend_lens=[150, 70, 8], pool_factor=1.1, is_cross_attention=is_cross,
        sliding_window_size=window))
    _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, key_splits)
    try:
        _check(wl, gpu, f"head_dim 256 splits={key_splits} cross={is_cross} W={window}")
    finally:
        _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, 0)
