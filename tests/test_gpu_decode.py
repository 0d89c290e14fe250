"""Paged GQA decode on the GPU vs the oracle (tolerance: max-abs 2e-2, mean-abs 2e-3)."""
import pytest
import torch

from _gpu_util import run_gpu, run_oracle
from _util import assert_close_bf16
from mini_sglang_amd.workloads import build_workload

pytestmark = pytest.mark.gpu


def _check(wl, gpu, what):
    print(what, flush=True)
    got, _ = run_gpu(wl, gpu)
    want, _ = run_oracle(wl)
    return assert_close_bf16(got, want, what)


@pytest.mark.parametrize("n_q,n_kv", [(8, 8), (16, 8), (32, 8), (64, 8), (16, 1), (6, 3)])
def test_decode_group_sizes(gpu, n_q, n_kv):
    wl = build_workload("t", "decode", seed=100 + n_q, n_q=n_q, n_kv=n_kv,
                        kv_lens=[1, 15, 16, 17, 31, 32, 33, 63, 64, 65, 200, 777], pool_factor=1.3)
    _check(wl, gpu, f"decode n_q={n_q} n_kv={n_kv}")


@pytest.mark.parametrize("segments,min_seg", [(1, 64), (2, 64), (3, 128), (7, 64), (55, 64),
                                              (4000, 64), (0, 0)])
def test_decode_result_independent_of_the_split(gpu, segments, min_seg):
    """Segment boundaries fall inside requests, on request boundaries, and (with one
    segment) nowhere; the merged result must not depend on them."""
    from mini_sglang_amd_kernel import _lib

    wl = build_workload("t", "decode", seed=7, n_q=32, n_kv=8,
                        kv_lens=[5, 100, 257, 1000, 2049, 31, 64, 0, 640], pool_factor=1.2)
    _lib.set_tuning(_lib.TUNE_SEGMENTS, segments)
    _lib.set_tuning(_lib.TUNE_MIN_SEGMENT, min_seg)
    _check(wl, gpu, f"decode segments={segments} min_seg={min_seg}")
    _lib.set_tuning(_lib.TUNE_SEGMENTS, 0)
    _lib.set_tuning(_lib.TUNE_MIN_SEGMENT, 0)


def test_decode_empty_request_gives_zeros_and_page_size_one(gpu):
    wl = build_workload("t", "decode", seed=8, n_q=16, n_kv=8, page_size=1,
                        kv_lens=[40, 0, 129, 0], pool_factor=2.0)
    got, _ = run_gpu(wl, gpu)
    want, _ = run_oracle(wl)
    assert_close_bf16(got, want, "decode with empty requests")
    assert torch.count_nonzero(got[1]) == 0 and torch.count_nonzero(got[3]) == 0


def test_decode_head_dim_256(gpu):
    wl = build_workload("t", "decode", seed=9, n_q=8, n_kv=2, head_dim=256,
                        kv_lens=[3, 64, 130, 515], pool_factor=1.5)
    _check(wl, gpu, "decode d=256")


def test_decode_large_batch_many_requests(gpu):
    g = torch.Generator().manual_seed(3)
    lens = torch.randint(1, 300, (150,), generator=g).tolist()
    wl = build_workload("t", "decode", seed=10, n_q=16, n_kv=4, kv_lens=lens, pool_factor=1.1)
    _check(wl, gpu, "decode batch=150")


def test_decode_strided_pool_views(gpu):
    """Pools that are planes of a larger (slots, 2, n_kv, d) allocation: stride0 != n_kv*d."""
    from mini_sglang_amd_kernel import paged_decode_attention

    wl = build_workload("t", "decode", seed=11, n_q=8, n_kv=2, kv_lens=[70, 200], pool_factor=1.0)
    want, _ = run_oracle(wl)
    big = torch.stack([wl.k_cache, wl.v_cache], dim=1).to(gpu)  # (slots, 2, n_kv, d)
    g = wl.to(gpu)
    out = paged_decode_attention(g.q, big[:, 0], big[:, 1], g.kv_indptr, g.kv_indices,
                                 g.num_kv_splits, g.sm_scale, g.max_kv_splits)
    torch.cuda.synchronize()
    assert_close_bf16(out.cpu(), want, "decode strided pools")


@pytest.mark.parametrize("scale", [0.0, -0.3, 1.5])
def test_decode_unusual_softmax_scales(gpu, scale):
    import dataclasses

    wl = build_workload("t", "decode", seed=77, n_q=8, n_kv=2, kv_lens=[1, 90, 700, 2100],
                        pool_factor=1.2)
    _check(dataclasses.replace(wl, sm_scale=scale), gpu, f"decode scale={scale}")


def _as_half(wl):
    """The same workload in IEEE half.  bf16 values are half values too unless they are below
    half's normal range; those few are zeroed on both sides so that both see equal numbers."""
    from dataclasses import replace

    def conv(t):
        t = torch.where(t.float().abs() < 2.0 ** -14, torch.zeros_like(t), t)
        h = t.to(torch.float16)
        assert torch.equal(h.float(), t.float())
        return t, h

    (qb, qh), (kb, kh), (vb, vh) = conv(wl.q), conv(wl.k_cache), conv(wl.v_cache)
    return replace(wl, q=qb, k_cache=kb, v_cache=vb), replace(wl, q=qh, k_cache=kh, v_cache=vh)


@pytest.mark.parametrize("n_q,n_kv,head_dim", [(32, 8, 128), (16, 1, 128), (6, 3, 128), (8, 2, 256)])
def test_decode_in_ieee_half_matches_the_oracle(gpu, n_q, n_kv, head_dim):
    """The reference instantiates decode for float16 as well
    (paged_decode_attention.metal:596-604).  Half keeps three more mantissa bits than bf16,
    so the result is held to a tighter bound than the bf16 one."""
    wl = build_workload("t", "decode", seed=300 + n_q, n_q=n_q, n_kv=n_kv, head_dim=head_dim,
                        kv_lens=[1, 16, 17, 33, 64, 65, 0, 200, 777, 3000], pool_factor=1.3)
    as_bf16, as_half = _as_half(wl)
    print(f"decode float16 n_q={n_q} n_kv={n_kv} d={head_dim}", flush=True)
    got, _ = run_gpu(as_half, gpu)
    assert got.dtype == torch.float16
    want, _ = run_oracle(as_bf16)
    assert_close_bf16(got, want, "decode float16", max_tol=5e-3, mean_tol=4e-4)


def test_decode_in_ieee_half_full_mantissa_inputs_and_split_invariance(gpu):
    """Inputs with all ten mantissa bits in use, against textbook attention in float64;
    the merged result must not depend on the number of segments."""
    from _util import dense_attention_f64, indptr
    from mini_sglang_amd_kernel import _lib, paged_decode_attention

    g = torch.Generator().manual_seed(41)
    n_q, n_kv, d, slots = 16, 4, 128, 6000
    kv_lens = [700, 5, 2049, 64, 1500]
    rnd = lambda *s: torch.randn(s, generator=g, dtype=torch.float32).to(torch.float16)
    q, kc, vc = rnd(len(kv_lens), n_q, d), rnd(slots, n_kv, d), rnd(slots, n_kv, d)
    kv_indptr = indptr(kv_lens)
    kv_indices = torch.randperm(slots, generator=g)[: sum(kv_lens)].to(torch.int32)
    splits = torch.ones(len(kv_lens), dtype=torch.int32)
    qo = indptr([1] * len(kv_lens))
    prefix = torch.tensor([l - 1 for l in kv_lens], dtype=torch.int32)
    want = dense_attention_f64(q, kc, vc, qo, kv_indptr, kv_indices, prefix, d ** -0.5)
    outs = []
    for segments in (0, 1, 13):
        _lib.set_tuning(_lib.TUNE_SEGMENTS, segments)
        print(f"decode float16 dense, segments={segments}", flush=True)
        out = paged_decode_attention(q.to(gpu), kc.to(gpu), vc.to(gpu), kv_indptr.to(gpu),
                                     kv_indices.to(gpu), splits.to(gpu), d ** -0.5, 32)
        torch.cuda.synchronize()
        _lib.set_tuning(_lib.TUNE_SEGMENTS, 0)
        assert_close_bf16(out, want, f"decode float16 dense segments={segments}",
                          max_tol=5e-3, mean_tol=4e-4)
        outs.append(out.float().cpu())
    assert_close_bf16(outs[1], outs[0], "float16 split invariance", max_tol=2e-3, mean_tol=1e-4)
    assert_close_bf16(outs[2], outs[0], "float16 split invariance", max_tol=2e-3, mean_tol=1e-4)


def test_prefill_rejects_ieee_half_as_the_reference_does(gpu):
    from mini_sglang_amd_kernel import paged_prefill_attention

    z = lambda *s: torch.zeros(s, dtype=torch.float16, device=gpu)
    i = lambda *v: torch.tensor(v, dtype=torch.int32, device=gpu)
    with pytest.raises(RuntimeError, match="unsupported dtype"):
        paged_prefill_attention(z(4, 8, 128), z(16, 2, 128), z(16, 2, 128), i(0, 4), i(0, 4),
                                i(0, 1, 2, 3), i(0), 0.1, 4)
