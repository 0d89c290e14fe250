"""Paged prefill / extend on the GPU vs the oracle, both routes (MFMA tile kernel for long
extends, split-K kernel for short query blocks) and all four masks."""
import math

import numpy as np
import pytest
import torch

from _gpu_util import run_gpu, run_oracle
from _util import assert_close_bf16
from mini_sglang_amd.workloads import build_workload
from test_oracle_known_answers import MASK_CASES, expected_weights, uniform_case

pytestmark = pytest.mark.gpu

MASKS = [(False, 0), (True, 0), (False, 100), (True, 100), (False, 1), (False, 17)]


def _check(wl, gpu, what):
    print(what, flush=True)
    got, _ = run_gpu(wl, gpu)
    want, _ = run_oracle(wl)
    return assert_close_bf16(got, want, what)


@pytest.mark.parametrize("q_len,prefix_len,is_cross,window", MASK_CASES)
def test_reference_mask_cases_closed_form(gpu, q_len, prefix_len, is_cross, window):
    """The reference's own known-answer cases, run through the GPU operator."""
    from mini_sglang_amd_kernel import paged_prefill_attention

    d = {k: v.to(gpu) for k, v in uniform_case(q_len, prefix_len).items()}
    out = paged_prefill_attention(d["q"], d["k_cache"], d["v_cache"], d["qo_indptr"],
                                  d["kv_indptr"], d["kv_indices"], d["prefix_lens"],
                                  sm_scale=1.0 / math.sqrt(128), max_len_extend=q_len,
                                  is_cross_attention=is_cross, sliding_window_size=window)
    torch.cuda.synchronize()
    actual = out.float().cpu().numpy()[:, 0, : prefix_len + q_len]
    np.testing.assert_allclose(actual, expected_weights(q_len, prefix_len, is_cross, window),
                               rtol=1e-3, atol=1e-3)


def test_store_then_prefill_reaches_written_slots(gpu):
    from mini_sglang_amd_kernel import paged_prefill_attention, store_kv_cache

    q_len = 4
    page_ids = torch.tensor([3, 1, 4, 2], dtype=torch.int32, device=gpu)
    q = torch.zeros((q_len, 1, 128), dtype=torch.bfloat16, device=gpu)
    k = torch.zeros((q_len, 1, 128), dtype=torch.bfloat16, device=gpu)
    v = torch.zeros((q_len, 1, 128), dtype=torch.float32)
    for pos in range(q_len):
        v[pos, 0, pos] = 1.0
    v = v.to(torch.bfloat16).to(gpu)
    k_cache = torch.zeros((5, 1, 128), dtype=torch.bfloat16, device=gpu)
    v_cache = torch.zeros((5, 1, 128), dtype=torch.bfloat16, device=gpu)
    store_kv_cache(k_cache, v_cache, page_ids, k, v)
    ip = torch.tensor([0, q_len], dtype=torch.int32, device=gpu)
    out = paged_prefill_attention(q, k_cache, v_cache, ip, ip, page_ids,
                                  torch.tensor([0], dtype=torch.int32, device=gpu),
                                  sm_scale=1.0 / math.sqrt(128), max_len_extend=q_len)
    torch.cuda.synchronize()
    np.testing.assert_allclose(out.float().cpu().numpy()[:, 0, :q_len],
                               expected_weights(q_len, 0, False, 0), rtol=1e-3, atol=1e-3)


@pytest.fixture(params=[0, 1], ids=["pingpong", "fused"])
def tile_variant(request):
    """The ping-pong kernel (default) and the fused kernel kept as its comparison partner; each is checked."""
    from mini_sglang_amd_kernel import _lib

    _lib.set_tuning(_lib.TUNE_PREFILL_VARIANT, request.param)
    yield request.param
    _lib.set_tuning(_lib.TUNE_PREFILL_VARIANT, 0)


@pytest.mark.parametrize("is_cross,window", MASKS)
def test_tile_route_masks(gpu, tile_variant, is_cross, window):
    # extends long enough for the MFMA tile kernel, ragged, with and without prefix
    wl = build_workload("t", "prefill", seed=200, n_q=8, n_kv=2,
                        kv_lens=[70, 300, 64 + 130, 33, 513 + 65],
                        extend_lens=[70, 100, 130, 33, 65], pool_factor=1.3, store_new=True,
                        is_cross_attention=is_cross, sliding_window_size=window)
    _check(wl, gpu, f"tile route variant={tile_variant} cross={is_cross} W={window}")


@pytest.mark.parametrize("n_q,n_kv", [(8, 8), (32, 8), (12, 4), (16, 1)])
def test_tile_route_group_sizes(gpu, tile_variant, n_q, n_kv):
    wl = build_workload("t", "prefill", seed=210 + n_q, n_q=n_q, n_kv=n_kv,
                        kv_lens=[200 + 96, 129, 1000 + 257], extend_lens=[96, 129, 257],
                        pool_factor=1.2, store_new=True)
    _check(wl, gpu, f"tile route n_q={n_q} n_kv={n_kv}")


@pytest.mark.parametrize("is_cross,window", MASKS)
@pytest.mark.parametrize("q_len", [1, 3, 8, 11, 16])
def test_splitk_route_masks(gpu, tuning, q_len, is_cross, window):
    # short query blocks (verify / draft proposal): q_len * group <= 64; one, two and three
    # tiles of 16 columns in a wave (q_len 3, 8, 11), four on two waves (16: by default these go
    # to the tile kernel, so the split-K kernel is asked for)
    from mini_sglang_amd_kernel import _lib

    tuning(_lib.TUNE_SMALLQ_MAXCOLS, 64)
    wl = build_workload("t", "prefill", seed=300 + q_len, n_q=16, n_kv=4,
                        kv_lens=[q_len, 40 + q_len, 333 + q_len, 1500 + q_len],
                        extend_lens=[q_len] * 4, pool_factor=1.3, store_new=True,
                        is_cross_attention=is_cross, sliding_window_size=window)
    _check(wl, gpu, f"split-K route q_len={q_len} cross={is_cross} W={window}")


@pytest.mark.parametrize("is_cross,window", MASKS)
def test_head_dim_256_short_and_long_queries(gpu, is_cross, window):
    # extends of 5, 16, 40 and 70 at group 4: the first two are short query blocks (split-K
    # route in one launch), the others go to the tile kernel
    wl = build_workload("t", "prefill", seed=330, n_q=8, n_kv=2, head_dim=256,
                        kv_lens=[5, 100 + 16, 300 + 40, 70], extend_lens=[5, 16, 40, 70],
                        pool_factor=1.2, store_new=True,
                        is_cross_attention=is_cross, sliding_window_size=window)
    _check(wl, gpu, f"head_dim 256 cross={is_cross} W={window}")
    short = build_workload("t", "prefill", seed=331, n_q=8, n_kv=2, head_dim=256,
                           kv_lens=[7, 200 + 7, 64 + 3], extend_lens=[7, 7, 3], pool_factor=1.2,
                           store_new=True, is_cross_attention=is_cross,
                           sliding_window_size=window)
    _check(short, gpu, f"head_dim 256 short cross={is_cross} W={window}")


@pytest.mark.parametrize("is_cross,window", MASKS)
def test_head_dim_256_tile_kernel_masks(gpu, is_cross, window):
    # ragged extends with and without prefix: lengths around the 32-key step (31, 32, 33, 65),
    # an odd and an even number of steps, several q blocks of 128 rows per (request, kv head)
    wl = build_workload("t", "prefill", seed=340, n_q=8, n_kv=2, head_dim=256,
                        kv_lens=[70, 300, 64 + 130, 33, 513 + 65, 31, 32, 1000 + 97],
                        extend_lens=[70, 100, 130, 33, 65, 31, 32, 97], pool_factor=1.3,
                        store_new=True, is_cross_attention=is_cross, sliding_window_size=window)
    _check(wl, gpu, f"head_dim 256 tile kernel cross={is_cross} W={window}")


@pytest.mark.parametrize("n_q,n_kv", [(8, 8), (32, 8), (12, 4), (16, 1), (24, 1)])
def test_head_dim_256_tile_kernel_group_sizes(gpu, n_q, n_kv):
    wl = build_workload("t", "prefill", seed=350 + n_q, n_q=n_q, n_kv=n_kv, head_dim=256,
                        kv_lens=[200 + 96, 129, 1000 + 257, 2100 + 70], extend_lens=[96, 129, 257, 70],
                        pool_factor=1.2, store_new=True)
    _check(wl, gpu, f"head_dim 256 tile kernel n_q={n_q} n_kv={n_kv}")


def test_head_dim_256_tile_kernel_long_prefix_and_chunked_extend(gpu):
    """A long cached prefix (hundreds of pipeline steps through the stage rings), and one
    extend computed in two chunks against the same extend in one piece."""
    import dataclasses

    wl = build_workload("t", "prefill", seed=360, n_q=8, n_kv=2, head_dim=256,
                        kv_lens=[9000 + 300, 4097 + 200], extend_lens=[300, 200],
                        pool_factor=1.1, store_new=True)
    print("head_dim 256 long prefix", flush=True)
    got, g = run_gpu(wl, gpu)
    want, _ = run_oracle(wl)
    assert_close_bf16(got, want, "head_dim 256 long prefix")
    # the second 150 queries of request 0 as an extend of their own on top of prefix + 150
    from mini_sglang_amd_kernel import paged_prefill_attention
    from _util import indptr

    kv0 = 9000 + 300
    rows = slice(150, 300)
    out = paged_prefill_attention(
        g.q[rows], g.k_cache, g.v_cache, indptr([150]).to(gpu), indptr([kv0]).to(gpu),
        g.kv_indices[:kv0], torch.tensor([9000 + 150], dtype=torch.int32, device=gpu),
        wl.sm_scale, 150)
    torch.cuda.synchronize()
    assert_close_bf16(out.cpu(), got[rows].float(), "head_dim 256 chunked extend", max_tol=8e-3,
                      mean_tol=4e-4)


@pytest.mark.parametrize("scale", [0.0, -0.3, 1.5])
def test_head_dim_256_tile_kernel_unusual_scales_and_magnitudes(gpu, scale):
    import dataclasses

    wl = build_workload("t", "prefill", seed=370, n_q=8, n_kv=2, head_dim=256,
                        kv_lens=[70 + 70, 300 + 130, 65], extend_lens=[70, 130, 65],
                        pool_factor=1.2, store_new=True)
    _check(dataclasses.replace(wl, sm_scale=scale), gpu, f"head_dim 256 scale={scale}")
    big = dataclasses.replace(wl, q=(wl.q.float() * 6).to(torch.bfloat16),
                              k_cache=(wl.k_cache.float() * 6).to(torch.bfloat16),
                              new_k=(wl.new_k.float() * 6).to(torch.bfloat16))
    _check(big, gpu, "head_dim 256 large magnitude")


@pytest.mark.parametrize("head_dim", [128, 256])
@pytest.mark.parametrize("n_q,n_kv,q_len", [(8, 8, 36), (8, 8, 48), (8, 4, 20), (4, 4, 64), (6, 2, 11),
                                            (8, 8, 17), (16, 1, 3)])
def test_splitk_route_every_column_tile_count(gpu, tuning, head_dim, n_q, n_kv, q_len):
    # q_len * group = 36, 48, 40, 64, 33, 17, 48 columns: two, three and four tiles of 16, the
    # three-tile ones with an idle fourth wave per kv head at head_dim 256 (by default most of
    # these column counts go to the tile kernels, so the split-K kernel is asked for)
    from mini_sglang_amd_kernel import _lib

    tuning(_lib.TUNE_SMALLQ_MAXCOLS, 64)
    wl = build_workload("t", "prefill", seed=390 + q_len, n_q=n_q, n_kv=n_kv, head_dim=head_dim,
                        kv_lens=[q_len + 32, 500 + q_len, q_len], extend_lens=[q_len] * 3,
                        pool_factor=1.2, store_new=True, sliding_window_size=0)
    _check(wl, gpu, f"split-K columns d={head_dim} heads={n_q}/{n_kv} q_len={q_len}")
    _check(wl.with_mask(is_cross_attention=False, sliding_window_size=2), gpu, "same, window 2")


@pytest.mark.parametrize("head_dim", [128, 256])
def test_tile_route_many_requests(gpu, head_dim):
    # more requests than the kernels rank by length (they then go in batch order): 150 and 129
    # ragged extends, with one batch exactly at the limit
    for batch in (128, 129, 150):
        g = torch.Generator().manual_seed(batch)
        ext = torch.randint(17, 90, (batch,), generator=g).tolist()
        pre = torch.randint(0, 60, (batch,), generator=g).tolist()
        wl = build_workload("t", "prefill", seed=500 + batch, n_q=8, n_kv=2, head_dim=head_dim,
                            kv_lens=[p + e for p, e in zip(pre, ext)], extend_lens=ext,
                            pool_factor=1.1, store_new=True)
        _check(wl, gpu, f"tile route d={head_dim} batch={batch}")


@pytest.mark.parametrize("scale", [0.0, -0.3, 1.5, 0.01])
def test_unusual_softmax_scales_on_both_routes(gpu, tile_variant, scale):
    # zero (uniform weights), negative (the smallest score wins), large (peaky rows: the running
    # max jumps by more than the lazy threshold again and again), tiny
    import dataclasses

    for extend in ([70, 130, 65], [3, 8, 5]):  # MFMA tile route, split-K route
        wl = build_workload("t", "prefill", seed=400, n_q=8, n_kv=2,
                            kv_lens=[70 + extend[0], 300 + extend[1], extend[2]],
                            extend_lens=extend, pool_factor=1.2, store_new=True)
        wl = dataclasses.replace(wl, sm_scale=scale)
        _check(wl, gpu, f"scale={scale} extend={extend} variant={tile_variant}")


def test_large_magnitude_inputs_do_not_overflow(gpu, tile_variant):
    # q and k eight times larger: scores of several hundred (base-2 exponents far beyond what
    # fp32 exp2 can take without the running max), one key dominating most rows
    import dataclasses

    for extend in ([70, 130, 65], [3, 8, 5]):
        wl = build_workload("t", "prefill", seed=410, n_q=8, n_kv=2,
                            kv_lens=[70 + extend[0], 300 + extend[1], extend[2]],
                            extend_lens=extend, pool_factor=1.2, store_new=True)
        wl = dataclasses.replace(wl, q=(wl.q.float() * 8).to(torch.bfloat16),
                                 k_cache=(wl.k_cache.float() * 8).to(torch.bfloat16),
                                 new_k=(wl.new_k.float() * 8).to(torch.bfloat16))
        got = _check(wl, gpu, f"large magnitude extend={extend} variant={tile_variant}")


def test_splitk_route_ragged_q_and_chunking(gpu):
    from mini_sglang_amd_kernel import _lib

    wl = build_workload("t", "prefill", seed=310, n_q=8, n_kv=2,
                        kv_lens=[5, 100 + 8, 700 + 3, 64 + 16], extend_lens=[5, 8, 3, 16],
                        pool_factor=1.1, store_new=True, sliding_window_size=50)
    for segments in (1, 5, 64, 0):
        _lib.set_tuning(_lib.TUNE_SEGMENTS, segments)
        _lib.set_tuning(_lib.TUNE_MIN_SEGMENT, 64)
        _check(wl, gpu, f"split-K route ragged segments={segments}")
        _lib.set_tuning(_lib.TUNE_SEGMENTS, 0)
        _lib.set_tuning(_lib.TUNE_MIN_SEGMENT, 0)


def test_both_routes_agree_and_decode_equals_prefill_qlen1(gpu):
    from mini_sglang_amd_kernel import _lib, paged_decode_attention

    wl = build_workload("t", "prefill", seed=320, n_q=8, n_kv=2, kv_lens=[90 + 8, 8, 400 + 8],
                        extend_lens=[8, 8, 8], pool_factor=1.0)
    a, _ = run_gpu(wl, gpu)
    _lib.set_tuning(_lib.TUNE_SMALLQ_MAXCOLS, -1)  # force the tile kernel
    b, _ = run_gpu(wl, gpu)
    _lib.set_tuning(_lib.TUNE_SMALLQ_MAXCOLS, 0)
    want, _ = run_oracle(wl)
    assert_close_bf16(a, want, "split-K route")
    assert_close_bf16(b, want, "tile route")
    # decode(L) == prefill(q_len=1, prefix=L-1)
    w1 = build_workload("t", "prefill", seed=321, n_q=8, n_kv=2, kv_lens=[77, 1, 300],
                        extend_lens=[1, 1, 1], pool_factor=1.0)
    p, g = run_gpu(w1, gpu)
    splits = torch.ones(3, dtype=torch.int32, device=gpu)
    dcd = paged_decode_attention(g.q, g.k_cache, g.v_cache, g.kv_indptr, g.kv_indices, splits,
                                 g.sm_scale, 32)
    torch.cuda.synchronize()
    assert_close_bf16(dcd.cpu(), p.float(), "decode vs prefill q_len=1", max_tol=4e-3, mean_tol=2e-4)


def test_rows_without_visible_keys_are_zero(gpu):
    from mini_sglang_amd_kernel import paged_prefill_attention

    wl = build_workload("t", "prefill", seed=330, n_q=4, n_kv=2, kv_lens=[3, 80],
                        extend_lens=[2, 70], pool_factor=1.0)
    g = wl.to(gpu)
    # request 0: kv stream (3 keys) far below the claimed prefix, window 2 => nothing visible
    prefix = torch.tensor([50, 10], dtype=torch.int32, device=gpu)
    for max_ext in (70,):
        out = paged_prefill_attention(g.q, g.k_cache, g.v_cache, g.qo_indptr, g.kv_indptr,
                                      g.kv_indices, prefix, g.sm_scale, max_ext,
                                      sliding_window_size=2)
        torch.cuda.synchronize()
        assert torch.count_nonzero(out[:2]) == 0
        assert torch.isfinite(out.float()).all()


def test_max_len_extend_smaller_than_a_request_leaves_tail_rows_alone(gpu):
    from mini_sglang_amd_kernel import paged_prefill_attention

    wl = build_workload("t", "prefill", seed=340, n_q=4, n_kv=2, kv_lens=[20, 30],
                        extend_lens=[10, 12], pool_factor=1.0)
    want, _ = run_oracle(wl)
    g = wl.to(gpu)
    out = paged_prefill_attention(g.q, g.k_cache, g.v_cache, g.qo_indptr, g.kv_indptr,
                                  g.kv_indices, g.prefix_lens, g.sm_scale, 12)
    torch.cuda.synchronize()
    assert_close_bf16(out.cpu(), want, "reference")


# ---- key splits of the tile kernels: a launch with fewer query blocks than compute units shares
# ---- the keys of every block out over several workgroups and merges fp32 partials ----------------
@pytest.fixture(params=[2, 3, 7, 32], ids=lambda k: f"{k}splits")
def key_splits(request):
    from mini_sglang_amd_kernel import _lib

    _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, request.param)
    yield request.param
    _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, 0)


@pytest.mark.parametrize("head_dim", [128, 256])
@pytest.mark.parametrize("is_cross,window", MASKS)
def test_key_split_masks(gpu, key_splits, head_dim, is_cross, window):
    # ragged requests, some with fewer tiles than shares (empty shares), prefix lengths that put
    # the causal diagonal inside a middle share, windows that start past the first shares
    wl = build_workload("t", "prefill", seed=700 + head_dim, n_q=8, n_kv=2, head_dim=head_dim,
                        kv_lens=[70, 300, 64 + 130, 33, 513 + 65, 31, 1000 + 97, 2049 + 300],
                        extend_lens=[70, 100, 130, 33, 65, 31, 97, 300], pool_factor=1.3,
                        store_new=True, is_cross_attention=is_cross, sliding_window_size=window)
    _check(wl, gpu, f"key splits={key_splits} head_dim={head_dim} cross={is_cross} W={window}")


@pytest.mark.parametrize("head_dim", [128, 256])
@pytest.mark.parametrize("n_q,n_kv", [(8, 8), (32, 8), (12, 4), (16, 1)])
def test_key_split_group_sizes(gpu, key_splits, head_dim, n_q, n_kv):
    wl = build_workload("t", "prefill", seed=720 + n_q, n_q=n_q, n_kv=n_kv, head_dim=head_dim,
                        kv_lens=[200 + 96, 129, 1000 + 257, 2100 + 70], extend_lens=[96, 129, 257, 70],
                        pool_factor=1.2, store_new=True)
    _check(wl, gpu, f"key splits={key_splits} head_dim={head_dim} n_q={n_q} n_kv={n_kv}")


@pytest.mark.parametrize("head_dim", [128, 256])
def test_key_split_equals_one_pass_and_leaves_capped_rows_alone(gpu, head_dim):
    """The split result is the one-pass result up to the fp32 merge; rows past max_len_extend
    keep what `out` held (the merge kernel must not touch them either)."""
    from mini_sglang_amd_kernel import _lib

    lib = _lib.load()
    wl = build_workload("t", "prefill", seed=740, n_q=8, n_kv=4, head_dim=head_dim,
                        kv_lens=[3000 + 90, 5000 + 120, 77], extend_lens=[90, 120, 77],
                        pool_factor=1.1)
    g = wl.to(gpu)
    cap = 100  # request 1 has 120 queries: its last 20 rows stay untouched
    outs = []
    for k in (1, 5):
        print(f"key splits {k} head_dim {head_dim} cap {cap}", flush=True)
        _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, k)
        out = torch.full_like(g.q, 7.0)
        total_q, n_q, d = g.q.shape
        batch, total_kv = g.qo_indptr.shape[0] - 1, g.kv_indices.shape[0]
        ws_bytes = lib.msgl_paged_prefill_workspace_bytes(batch, total_q, total_kv, n_q,
                                                          g.k_cache.shape[1], d, cap)
        assert (ws_bytes > 0) == (k > 1)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=gpu)
        rc = lib.msgl_paged_prefill_attention(
            g.q.data_ptr(), g.k_cache.data_ptr(), g.v_cache.data_ptr(), g.qo_indptr.data_ptr(),
            g.kv_indptr.data_ptr(), g.kv_indices.data_ptr(), g.prefix_lens.data_ptr(),
            out.data_ptr(), ws.data_ptr(), ws_bytes, batch, total_q, total_kv, n_q,
            g.k_cache.shape[1], d, g.k_cache.shape[0], g.k_cache.stride(0), g.v_cache.stride(0),
            float(g.sm_scale), cap, 0, 0, 0, None)
        assert rc == 0, _lib.strerror(rc)
        torch.cuda.synchronize()
        if k > 1:  # too small a workspace is not overrun: the keys go in one pass
            again = torch.full_like(g.q, 7.0)
            ws.fill_(0x7f)
            assert lib.msgl_paged_prefill_attention(
                g.q.data_ptr(), g.k_cache.data_ptr(), g.v_cache.data_ptr(), g.qo_indptr.data_ptr(),
                g.kv_indptr.data_ptr(), g.kv_indices.data_ptr(), g.prefix_lens.data_ptr(),
                again.data_ptr(), ws.data_ptr(), ws_bytes - 1, batch, total_q, total_kv, n_q,
                g.k_cache.shape[1], d, g.k_cache.shape[0], g.k_cache.stride(0),
                g.v_cache.stride(0), float(g.sm_scale), cap, 0, 0, 0, None) == 0
            torch.cuda.synchronize()
            assert torch.equal(again.cpu().view(torch.int16), outs[0].view(torch.int16))
            assert (ws == 0x7f).all()
        _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, 0)
        outs.append(out.cpu())
    tail = slice(90 + cap, 90 + 120)
    for out in outs:
        assert (out[tail].float() == 7.0).all()
    assert_close_bf16(outs[1], outs[0].float(), "split vs one pass", max_tol=8e-3, mean_tol=4e-4)
    want, _ = run_oracle(wl)
    keep = torch.ones(want.shape[0], dtype=torch.bool)
    keep[tail] = False
    assert_close_bf16(outs[1][keep], want[keep], "split vs oracle")


@pytest.mark.parametrize("head_dim", [128, 256])
@pytest.mark.parametrize("extend", [70, 300])
def test_one_long_request_splits_its_keys_by_itself(gpu, head_dim, extend):
    """No knob: one request with a long prefix has too few query blocks for the chip, so the
    library asks for a workspace and splits."""
    from mini_sglang_amd_kernel import _lib

    lib = _lib.load()
    n_q, n_kv, prefix = 8, 2, 20000
    assert lib.msgl_paged_prefill_workspace_bytes(1, extend, prefix + extend, n_q, n_kv, head_dim, extend) > 0
    # the benchmark's extend shape fills the chip: no key split (at head_dim 128 it asks for the
    # slots of its gang ranges instead, which do not depend on the number of queries)
    need = lib.msgl_paged_prefill_workspace_bytes(8, 8 * 512, 8 * 8704, 32, 8, head_dim, 512)
    assert need == (0 if head_dim == 256 else lib.msgl_paged_prefill_workspace_bytes(8, 8 * 300, 8 * 8704, 32, 8, head_dim, 512))
    wl = build_workload("t", "prefill", seed=760 + extend, n_q=n_q, n_kv=n_kv, head_dim=head_dim,
                        kv_lens=[prefix + extend], extend_lens=[extend], pool_factor=1.1, store_new=True)
    _check(wl, gpu, f"one long request head_dim={head_dim} extend={extend}")


@pytest.mark.parametrize("head_dim", [128, 256])
def test_partially_filled_query_blocks_idle_waves(gpu, head_dim):
    """Last query blocks with 1 .. 7 of the eight waves' row ranges empty (head_dim 128: such waves
    move tiles and pass barriers but compute nothing), next to full blocks, on prefixes long enough
    for many tiles; the smallest-query route is kept off so that every request takes a tile kernel."""
    from mini_sglang_amd_kernel import _lib

    # group 4: an extend of e tokens has 4 e rows; blocks hold 256 (head_dim 128) or 128 rows
    ext = [17, 24, 33, 41, 49, 57, 64, 65, 72, 100, 121]
    wl = build_workload("t", "prefill", seed=960, n_q=8, n_kv=2, head_dim=head_dim,
                        kv_lens=[700 + 37 * i + e for i, e in enumerate(ext)], extend_lens=ext,
                        pool_factor=1.2, store_new=True)
    _lib.set_tuning(_lib.TUNE_SMALLQ_MAXCOLS, -1)
    _check(wl, gpu, f"partially filled query blocks head_dim={head_dim}")
    _lib.set_tuning(_lib.TUNE_SMALLQ_MAXCOLS, 0)


@pytest.mark.parametrize("is_cross,window", MASKS)
@pytest.mark.parametrize("head_dim,q_len", [(128, 13), (128, 16), (128, 40), (128, 64), (256, 5),
                                            (256, 13), (256, 32)])
def test_tile_route_ragged_key_shares(gpu, head_dim, q_len, is_cross, window):
    """One query block per (request, kv head) on the tile kernels (52-256 rows at group 4, up to
    128 at head_dim 256): the keys of a request go in as many equal shares as its length asks
    for, so one request here has dozens of shares, others one, one has no prefix and one no rows
    at all."""
    wl = build_workload("t", "prefill", seed=350 + q_len, n_q=16, n_kv=4, head_dim=head_dim,
                        kv_lens=[q_len + 70000, q_len + 300, q_len + 5000, q_len, 0, q_len + 1300],
                        extend_lens=[q_len, q_len, q_len, q_len, 0, q_len], pool_factor=1.1,
                        store_new=True, is_cross_attention=is_cross, sliding_window_size=window)
    _check(wl, gpu, f"tile route, ragged shares, q_len={q_len} cross={is_cross} W={window}")


@pytest.mark.parametrize("head_dim,q_len", [(128, 16), (128, 50), (256, 8)])
def test_tile_route_ragged_shares_many_requests(gpu, head_dim, q_len):
    """More than 128 requests keep ragged key shares when they are long on average: 150 requests,
    one of them twenty times the others, so its shares are spread over three 64-request chunks of
    the share-count scan; and the same batch with short requests, which the tile kernels take
    without shares (or, for the short query blocks, the split-K kernel)."""
    for lens in ([20000] + [1100] * 149, [1100] * 70 + [20000] + [1100] * 79, [3000] + [90] * 149):
        wl = build_workload("t", "prefill", seed=370 + q_len, n_q=16, n_kv=4, head_dim=head_dim,
                            kv_lens=[n + q_len for n in lens], extend_lens=[q_len] * len(lens),
                            pool_factor=1.1, store_new=True)
        _check(wl, gpu, f"tile route, {len(lens)} requests, d={head_dim} q_len={q_len} first={lens[0]}")
