"""Gang ranges of the head_dim 128 extend kernel (several query blocks per (request, kv head);
one workgroup per compute unit for the whole launch, the units' keys shared out by length and
the parts of a unit merged by the workgroup that finishes last).

Checked against the oracle, against the same launch without gang ranges, and by the closed-form
mask edges; sizes are forced into the route with MSGL_TUNE_PREFILL_GANGS = 1 where the launch
would be too small to choose it."""
import numpy as np
import pytest
import torch

from _gpu_util import run_gpu, run_oracle
from _mask_edges import assert_edges, one_hot_values
from _util import assert_close_bf16
from mini_sglang_amd.workloads import build_workload

pytestmark = pytest.mark.gpu


@pytest.fixture
def gangs():
    from mini_sglang_amd_kernel import _lib

    def set_(v):
        _lib.set_tuning(_lib.TUNE_PREFILL_GANGS, v)

    yield set_
    _lib.set_tuning(_lib.TUNE_PREFILL_GANGS, 0)


# (n_q, n_kv, extend, prefixes): 2, 4, 8 and 16 query blocks of 256 rows; units of very unequal
# length (a unit is cut into up to all of an XCD's gangs), units shorter than the margin that no
# cut may enter, fewer units than gangs, requests with fewer query blocks than the launch
SHAPES = [
    (32, 8, 128, [3000, 40, 700, 1500]),
    (32, 8, 256, [5000, 0, 90, 2048, 33, 900]),
    (32, 8, 512, [4100, 300]),
    (8, 8, 512, [2500, 0, 1200, 64, 6000, 10, 800, 3333]),
    (16, 8, 2048, [1000, 5000]),
    (64, 8, 300, [2000, 150, 4000]),
]


@pytest.mark.parametrize("is_cross", [False, True])
@pytest.mark.parametrize("n_q,n_kv,extend,prefixes", SHAPES)
def test_forced_gang_ranges_against_oracle(gpu, gangs, n_q, n_kv, extend, prefixes, is_cross):
    ext = [extend if i % 3 != 2 else max(1, extend - 70) for i in range(len(prefixes))]  # ragged extends
    wl = build_workload("g", "prefill", seed=900 + extend, n_q=n_q, n_kv=n_kv,
                        kv_lens=[p + e for p, e in zip(prefixes, ext)], extend_lens=ext,
                        pool_factor=1.2, store_new=True, is_cross_attention=is_cross)
    gangs(1)
    print(f"gang ranges n_q={n_q} extend={extend} cross={is_cross}", flush=True)
    got, _ = run_gpu(wl, gpu)
    gangs(-1)
    plain, _ = run_gpu(wl, gpu)
    want, _ = run_oracle(wl)
    assert_close_bf16(got, want, "gang ranges vs oracle")
    assert_close_bf16(got, plain.float(), "gang ranges vs one pass per unit", max_tol=8e-3, mean_tol=4e-4)


@pytest.mark.parametrize("is_cross", [False, True])
def test_forced_gang_ranges_mask_edges(gpu, gangs, is_cross):
    wl = one_hot_values(build_workload(
        "e", "prefill", seed=17, n_q=32, n_kv=8, kv_lens=[5000 + 300, 130 + 130, 1024 + 265, 2047 + 257],
        extend_lens=[300, 130, 265, 257], pool_factor=1.1, is_cross_attention=is_cross))
    gangs(1)
    got, _ = run_gpu(wl, gpu)
    assert_edges(got.float().numpy()[:, 0], wl, f"gang ranges mask edges cross={is_cross}")
    assert_edges(got.float().numpy()[:, -1], wl, f"gang ranges mask edges cross={is_cross}, last head")


def test_gang_ranges_repeat_bit_identical_and_reuse_a_workspace(gpu, gangs):
    """The count words are left as the launch found them: the same workspace serves launch
    after launch, and which part of a unit finishes last does not change a bit of the result
    beyond the order of two additions per row."""
    from mini_sglang_amd_kernel import paged_prefill_attention, store_kv_cache

    wl = build_workload("g", "prefill", seed=77, n_q=32, n_kv=8, kv_lens=[6000 + 512, 100 + 512, 2500 + 512],
                        extend_lens=[512] * 3, pool_factor=1.1, store_new=True)
    gangs(1)
    g = wl.to(gpu)
    store_kv_cache(g.k_cache, g.v_cache, g.out_loc, g.new_k, g.new_v)
    outs = []
    for _ in range(12):
        outs.append(paged_prefill_attention(g.q, g.k_cache, g.v_cache, g.qo_indptr, g.kv_indptr,
                                            g.kv_indices, g.prefix_lens, g.sm_scale, g.max_len_extend))
    torch.cuda.synchronize()
    want, _ = run_oracle(wl)
    for o in outs:
        assert_close_bf16(o.cpu(), want, "gang ranges, repeated launch")
    worst = max(float((o.float() - outs[0].float()).abs().max()) for o in outs[1:])
    assert worst <= 2e-3, worst


def test_skewed_extend_chooses_gang_ranges_by_itself(gpu, gangs):
    """One long request among short ones, 512-token extends: large enough to take the route
    without being forced; every row against the closed form."""
    wl = one_hot_values(build_workload(
        "s", "prefill", seed=5, n_q=32, n_kv=8, kv_lens=[40000 + 512] + [1500 + 512] * 7,
        extend_lens=[512] * 8, pool_factor=1.05))
    got, _ = run_gpu(wl, gpu, store=False)
    assert_edges(got.float().numpy()[:, 3], wl, "skewed extend")
    gangs(-1)
    plain, _ = run_gpu(wl, gpu, store=False)
    assert_close_bf16(got, plain.float(), "skewed extend vs one pass per unit", max_tol=8e-3, mean_tol=4e-4)
