"""Seeded random shapes through both attention operators against the oracle: head counts,
head sizes, page sizes, ragged lengths (empty requests, single tokens, lengths around the 16-,
32- and 64-key tile edges), every mask, with and without a store first.  The fixed cases of the
other modules aim at known edges; this one looks for the ones nobody thought of."""
import os
import random

import pytest
import torch

from _gpu_util import run_gpu, run_oracle
from _util import assert_close_bf16
from mini_sglang_amd.workloads import build_workload

pytestmark = pytest.mark.gpu

# more seeds on request: MSGL_FUZZ_SCALE=10 runs ten times as many cases
_SCALE = max(1, int(os.environ.get("MSGL_FUZZ_SCALE", "1")))
HEADS = [(1, 1), (2, 1), (4, 4), (6, 3), (8, 2), (8, 8), (12, 4), (16, 1), (16, 8), (20, 4), (32, 8)]
EDGES = [0, 1, 2, 15, 16, 17, 31, 32, 33, 47, 63, 64, 65, 95, 96, 97, 127, 128, 129, 255, 257]


def _length(rng, hi):
    return rng.choice(EDGES) if rng.random() < 0.5 else rng.randrange(0, hi)


@pytest.mark.parametrize("seed", range(80 * _SCALE))
def test_random_prefill_shapes(gpu, seed):
    rng = random.Random(1000 + seed)
    n_q, n_kv = rng.choice(HEADS)
    d = rng.choice([128, 128, 256])
    batch = rng.randrange(1, 6)
    # short query blocks (split-K route), long ones (tile kernels), and mixtures of both
    style = rng.choice(["short", "long", "mixed"])
    ext, kv = [], []
    for _ in range(batch):
        if style == "short" or (style == "mixed" and rng.random() < 0.5):
            e = rng.randrange(0, 9)
        else:
            e = max(1, _length(rng, 300))
        prefix = _length(rng, 700) if rng.random() < 0.8 else 0
        ext.append(e)
        kv.append(prefix + e)
    if sum(ext) == 0:
        ext[0], kv[0] = 1, kv[0] + 1
    is_cross = rng.random() < 0.3
    window = rng.choice([0, 0, 1, 2, 17, 64, 100, 1000])
    page = rng.choice([1, 4, 16])
    wl = build_workload("fuzz", "prefill", seed=seed, n_q=n_q, n_kv=n_kv, head_dim=d, page_size=page,
                        kv_lens=kv, extend_lens=ext, pool_factor=rng.choice([1.0, 1.7]),
                        store_new=rng.random() < 0.7, is_cross_attention=is_cross,
                        sliding_window_size=window)
    # half of the cases force a key split of the tile kernels (the split-K route ignores it)
    splits = rng.choice([2, 3, 4, 5, 8, 13, 32]) if rng.random() < 0.5 else 0
    what = (f"fuzz prefill seed={seed} heads={n_q}/{n_kv} d={d} page={page} ext={ext} kv={kv} "
            f"cross={is_cross} W={window} key_splits={splits}")
    print(what, flush=True)
    from mini_sglang_amd_kernel import _lib

    _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, splits)
    got, g = run_gpu(wl, gpu)
    _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, 0)
    want, ref = run_oracle(wl)
    assert_close_bf16(got, want, what)
    if wl.out_loc is not None:
        assert torch.equal(g.k_cache.cpu().view(torch.int16), ref.k_cache.view(torch.int16)), what
        assert torch.equal(g.v_cache.cpu().view(torch.int16), ref.v_cache.view(torch.int16)), what


@pytest.mark.parametrize("seed", range(40 * _SCALE))
def test_random_decode_shapes(gpu, seed):
    rng = random.Random(2000 + seed)
    n_q, n_kv = rng.choice([h for h in HEADS if h[0] // h[1] <= 16])
    d = rng.choice([128, 128, 256])
    batch = rng.randrange(1, 40)
    kv = [_length(rng, 2500) for _ in range(batch)]
    page = rng.choice([1, 16])
    wl = build_workload("fuzz", "decode", seed=seed, n_q=n_q, n_kv=n_kv, head_dim=d, page_size=page,
                        kv_lens=kv, pool_factor=rng.choice([1.0, 1.4]))
    what = f"fuzz decode seed={seed} heads={n_q}/{n_kv} d={d} page={page} batch={batch} total={sum(kv)}"
    print(what, flush=True)
    got, _ = run_gpu(wl, gpu)
    want, _ = run_oracle(wl)
    assert_close_bf16(got, want, what)
    for b, l in enumerate(kv):
        if l == 0:
            assert torch.count_nonzero(got[b]) == 0, what


@pytest.mark.parametrize("seed", range(30 * _SCALE))
def test_random_metadata_builds(gpu, seed):
    import numpy as np

    from oracle import metadata_oracle as mo
    from test_gpu_metadata import _case, _run

    rng = np.random.default_rng(3000 + seed)
    batch = int(rng.choice([1, 2, 3, 17, 63, 64, 65, 200, 1000]))
    rows = int(rng.integers(1, 70))
    max_seq = int(rng.choice([1, 2, 31, 32, 33, 255, 257, 1000, 4100]))
    table, trows, kv, ext = _case(rng, batch, rows, max_seq, zero_frac=float(rng.choice([0.0, 0.1, 0.6])))
    decode = rng.random() < 0.3
    print(f"fuzz metadata seed={seed} batch={batch} rows={rows} max_seq={max_seq} decode={decode}", flush=True)
    if decode:
        kv = np.maximum(kv, 1)
        got = _run(gpu, table, trows, kv, None, total_kv=int(kv.sum()))
        want = mo.build_decode_metadata(table, trows, kv)
        keys = ("kv_indptr", "kv_indices", "num_kv_splits", "positions")
    else:
        got = _run(gpu, table, trows, kv, ext, total_kv=int(kv.sum()), total_q=int(ext.sum()))
        want = mo.build_prefill_metadata(table, trows, kv, ext)
        keys = ("kv_indptr", "kv_indices", "qo_indptr", "prefix_lens", "positions", "num_kv_splits")
    for k in keys:
        np.testing.assert_array_equal(got[k], want[k], err_msg=f"{k} seed={seed}")


@pytest.mark.parametrize("seed", range(20 * _SCALE))
def test_random_norm_rope_store_shapes(gpu, seed):
    from test_gpu_qk_norm_rope import _run_case

    rng = random.Random(4000 + seed)
    n_q, n_kv = rng.choice(HEADS)
    d = rng.choice([128, 128, 256])
    L = rng.choice([1, 2, 7, 63, 64, 65, 300, 1025])
    _run_case(gpu, L, n_q, n_kv, d, slots=L + rng.randrange(0, 50), max_pos=rng.choice([0, 100, 9000, 100000]),
              base=rng.choice([1e4, 1e6]), seed=seed, fused_view=rng.random() < 0.4)


@pytest.mark.parametrize("seed", range(16 * _SCALE))
def test_random_gdn_state_shapes(gpu, seed):
    import numpy as np

    from oracle import gdn_state_oracle as go
    from test_gpu_gdn_state import _check, _gpu, _inputs

    rng = np.random.default_rng(5000 + seed)
    hk = int(rng.choice([1, 2, 4, 16]))
    hv = hk * int(rng.choice([1, 2, 3]))
    single = rng.random() < 0.4
    if single:
        batch = int(rng.choice([1, 3, 8, 33, 100]))
        lengths = [1] * batch
    else:
        batch = int(rng.integers(1, 7))
        lengths = [int(rng.choice([0, 1, 2, 9, 40, 130])) for _ in range(batch)]
        if sum(lengths) == 0:
            lengths[0] = 5
    total = sum(lengths)
    d, state = _inputs(rng, total, hk, hv, batch + 4)
    slots = rng.permutation(batch + 4)[:batch]
    indptr = np.concatenate([[0], np.cumsum(lengths)])
    print(f"fuzz gdn seed={seed} hk={hk} hv={hv} single={single} lengths={lengths[:8]}", flush=True)
    got_y, got_st = _gpu(gpu, d, state, slots, indptr, single)
    want_y, want_st = go.gdn_state_inplace(d["q"], d["k"], d["v"], d["g"], d["beta"], state, slots,
                                           None if single else indptr, single_token_mode=single)
    _check(got_y, got_st, want_y, want_st, f"fuzz gdn seed={seed}")
    other = np.setdiff1d(np.arange(state.shape[0]), slots)
    np.testing.assert_array_equal(got_st[other], state[other])


MORE_HEADS = HEADS + [(7, 1), (10, 2), (32, 1), (48, 2), (40, 8), (64, 8), (3, 3)]


def _strided(pool, pad_elems):
    """The same pool values in a buffer whose slots are `pad_elems` further apart."""
    slots, n_kv, d = pool.shape
    buf = torch.zeros((slots, n_kv * d + pad_elems), dtype=pool.dtype, device=pool.device)
    view = buf[:, : n_kv * d].view(slots, n_kv, d)
    view.copy_(pool)
    return view


@pytest.mark.parametrize("seed", range(40 * _SCALE))
def test_random_prefill_strides_heads_and_query_caps(gpu, seed):
    """More of the argument space: odd head counts and large groups, pools with padded slots,
    a `max_len_extend` below the longest extend (rows past it are not computed, as in the
    reference's grid, paged_prefill_attention.cpp:152-159), a caller-owned stream."""
    import dataclasses

    from mini_sglang_amd_kernel import paged_prefill_attention, store_kv_cache

    rng = random.Random(6000 + seed)
    n_q, n_kv = rng.choice(MORE_HEADS)
    d = rng.choice([128, 256])
    batch = rng.randrange(1, 5)
    ext = [rng.choice([1, 2, 5, 16, 17, 40, 70, 129, 200]) for _ in range(batch)]
    kv = [e + (_length(rng, 400) if rng.random() < 0.8 else 0) for e in ext]
    wl = build_workload("fuzz", "prefill", seed=seed, n_q=n_q, n_kv=n_kv, head_dim=d,
                        page_size=rng.choice([1, 16]), kv_lens=kv, extend_lens=ext, pool_factor=1.3,
                        store_new=True, is_cross_attention=rng.random() < 0.3,
                        sliding_window_size=rng.choice([0, 0, 3, 50, 300]))
    cap = max(ext) if rng.random() < 0.6 else rng.randrange(1, max(ext) + 1)
    wl = dataclasses.replace(wl, max_len_extend=cap)
    pad = rng.choice([0, 8, 64, 1000 * 8])
    what = (f"fuzz prefill+ seed={seed} heads={n_q}/{n_kv} d={d} ext={ext} kv={kv} cap={cap} pad={pad} "
            f"cross={wl.is_cross_attention} W={wl.sliding_window_size}")
    print(what, flush=True)
    g = wl.to(gpu)
    kc, vc = _strided(g.k_cache, pad), _strided(g.v_cache, pad)
    side = torch.cuda.Stream(device=gpu)
    side.wait_stream(torch.cuda.current_stream(gpu))
    with torch.cuda.stream(side):
        store_kv_cache(kc, vc, g.out_loc, g.new_k, g.new_v, stream=side)
        got = paged_prefill_attention(g.q, kc, vc, g.qo_indptr, g.kv_indptr, g.kv_indices,
                                      g.prefix_lens, g.sm_scale, cap,
                                      is_cross_attention=g.is_cross_attention,
                                      sliding_window_size=g.sliding_window_size, stream=side)
    side.synchronize()
    want, ref = run_oracle(wl)
    qo = wl.qo_indptr.tolist()
    rows = torch.cat([torch.arange(qo[b], qo[b] + min(ext[b], cap)) for b in range(batch)])
    assert_close_bf16(got.cpu()[rows], want[rows], what)
    assert torch.equal(kc.cpu().view(torch.int16), ref.k_cache.view(torch.int16)), what
    assert torch.equal(vc.cpu().view(torch.int16), ref.v_cache.view(torch.int16)), what


@pytest.mark.parametrize("seed", range(30 * _SCALE))
def test_random_decode_half_precision_and_strides(gpu, seed):
    from mini_sglang_amd_kernel import paged_decode_attention
    from test_gpu_decode import _as_half

    rng = random.Random(7000 + seed)
    n_q, n_kv = rng.choice([h for h in MORE_HEADS if h[0] // h[1] <= 16])
    d = rng.choice([128, 256])
    batch = rng.randrange(1, 20)
    kv = [_length(rng, 1500) for _ in range(batch)]
    wl = build_workload("fuzz", "decode", seed=seed, n_q=n_q, n_kv=n_kv, head_dim=d,
                        page_size=rng.choice([1, 16]), kv_lens=kv, pool_factor=1.2)
    half = rng.random() < 0.5
    pad = rng.choice([0, 8, 264])
    what = f"fuzz decode+ seed={seed} heads={n_q}/{n_kv} d={d} batch={batch} half={half} pad={pad}"
    print(what, flush=True)
    as_bf16, as_half = _as_half(wl)
    src = (as_half if half else as_bf16).to(gpu)
    got = paged_decode_attention(src.q, _strided(src.k_cache, pad), _strided(src.v_cache, pad),
                                 src.kv_indptr, src.kv_indices, src.num_kv_splits, src.sm_scale,
                                 src.max_kv_splits)
    torch.cuda.synchronize()
    assert got.dtype == (torch.float16 if half else torch.bfloat16)
    want, _ = run_oracle(as_bf16)
    if half:
        assert_close_bf16(got, want, what, max_tol=5e-3, mean_tol=4e-4)
    else:
        assert_close_bf16(got, want, what)


@pytest.mark.parametrize("seed", range(24 * _SCALE))
def test_random_forced_gang_ranges(gpu, seed):
    """Extends of 2, 4, 8 or 16 query blocks per (request, kv head) forced into gang ranges
    (head_dim 128): random unit lengths, ragged extends, requests with fewer query blocks than the
    launch, causal and cross masks; against the oracle and against one workgroup per query block."""
    from mini_sglang_amd_kernel import _lib

    rng = random.Random(7000 + seed)
    n_kv = rng.choice([8, 8, 4])
    group = rng.choice([1, 2, 4, 8])
    batch = rng.randrange(1, 7)
    if (batch * n_kv) % 8:
        batch += 1  # whole (request, kv head) units per XCD
    n_qblk = rng.choice([2, 2, 4, 4, 8, 16])
    rows = rng.randrange((n_qblk - 1) * 256 + 1, n_qblk * 256 + 1)
    extend = max(1, (rows + group - 1) // group)
    while (extend * group + 255) // 256 != n_qblk:
        extend -= 1
    ext = [extend] + [extend if rng.random() < 0.6 else rng.randrange(1, extend + 1) for _ in range(batch - 1)]
    rng.shuffle(ext)
    kv = [(rng.choice([0, 1, 63, 64, 65, 700, 2048]) if rng.random() < 0.4 else rng.randrange(0, 5000)) + e
          for e in ext]
    is_cross = rng.random() < 0.3
    wl = build_workload("fuzz", "prefill", seed=seed, n_q=n_kv * group, n_kv=n_kv, head_dim=128,
                        page_size=rng.choice([1, 16]), kv_lens=kv, extend_lens=ext,
                        pool_factor=rng.choice([1.0, 1.5]), store_new=rng.random() < 0.5,
                        is_cross_attention=is_cross)
    what = f"fuzz gang ranges seed={seed} heads={n_kv * group}/{n_kv} ext={ext} kv={kv} cross={is_cross}"
    print(what, flush=True)
    lib = _lib.load()
    try:
        _lib.set_tuning(_lib.TUNE_PREFILL_GANGS, 1)
        need = lib.msgl_paged_prefill_workspace_bytes(batch, sum(ext), sum(kv), n_kv * group, n_kv, 128, max(ext))
        assert need > 0, "the shape was meant to take gang ranges: " + what
        got, _ = run_gpu(wl, gpu)
        _lib.set_tuning(_lib.TUNE_PREFILL_GANGS, -1)
        plain, _ = run_gpu(wl, gpu)
    finally:
        _lib.set_tuning(_lib.TUNE_PREFILL_GANGS, 0)
    want, _ = run_oracle(wl)
    assert_close_bf16(got, want, what)
    assert_close_bf16(got, plain.float(), what + " (against one workgroup per query block)", max_tol=8e-3,
                      mean_tol=4e-4)
