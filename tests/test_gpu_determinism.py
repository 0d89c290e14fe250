"""Same inputs, same bits: every attention route is launched many times on one workload and each
result must equal the first bit for bit.  The kernels use no atomics and merge partials in a fixed
order, so any difference is a race between waves (a stage refilled while another wave still reads
it, a wait that does not cover a load), which the parity tests only see when it happens to strike
on their single run."""
import pytest
import torch

from mini_sglang_amd.workloads import build_workload
from mini_sglang_amd_kernel import _lib, paged_decode_attention, paged_prefill_attention

pytestmark = pytest.mark.gpu

RUNS = 40


def _prefill(g, cap, **kw):
    return paged_prefill_attention(g.q, g.k_cache, g.v_cache, g.qo_indptr, g.kv_indptr, g.kv_indices,
                                   g.prefix_lens, g.sm_scale, cap, **kw)


@pytest.mark.parametrize("head_dim", [128, 256])
@pytest.mark.parametrize("splits", [1, 4, 32])
@pytest.mark.parametrize("n_q,n_kv", [(32, 8), (16, 1)])
def test_tile_kernels_repeat_bit_identical(gpu, head_dim, splits, n_q, n_kv):
    # many workgroups with few pipeline steps each: start-up and wind-down of the stage rings
    # are most of what runs
    wl = build_workload("t", "prefill", seed=900 + n_q, n_q=n_q, n_kv=n_kv, head_dim=head_dim,
                        kv_lens=[200 + 96, 129, 1000 + 257, 2100 + 70, 33, 64 + 65],
                        extend_lens=[96, 129, 257, 70, 33, 65], pool_factor=1.2)
    g = wl.to(gpu)
    print(f"repeat tile head_dim={head_dim} splits={splits} heads={n_q}/{n_kv}", flush=True)
    _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, splits)
    outs = [_prefill(g, 257) for _ in range(RUNS)]
    torch.cuda.synchronize()
    _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, 0)
    for i, out in enumerate(outs[1:], 1):
        assert torch.equal(out.view(torch.int16), outs[0].view(torch.int16)), f"run {i} differs from run 0"


@pytest.mark.parametrize("head_dim", [128, 256])
@pytest.mark.parametrize("is_cross,window", [(False, 0), (False, 100), (True, 0)])
def test_tile_kernels_repeat_bit_identical_long_rows(gpu, head_dim, is_cross, window):
    wl = build_workload("t", "prefill", seed=910, n_q=8, n_kv=2, head_dim=head_dim,
                        kv_lens=[3000 + 300, 31, 700 + 513], extend_lens=[300, 31, 513],
                        pool_factor=1.1, is_cross_attention=is_cross, sliding_window_size=window)
    g = wl.to(gpu)
    print(f"repeat tile long head_dim={head_dim} cross={is_cross} W={window}", flush=True)
    outs = [_prefill(g, 513, is_cross_attention=is_cross, sliding_window_size=window) for _ in range(RUNS)]
    torch.cuda.synchronize()
    for i, out in enumerate(outs[1:], 1):
        assert torch.equal(out.view(torch.int16), outs[0].view(torch.int16)), f"run {i} differs from run 0"


@pytest.mark.parametrize("head_dim", [128, 256])
@pytest.mark.parametrize("q_len", [1, 4, 8])
def test_splitk_kernel_repeat_bit_identical(gpu, head_dim, q_len):
    lens = [1, 17, 900, 4000, 64, 2500, 129, 33]
    wl = build_workload("t", "prefill", seed=920, n_q=16, n_kv=4, head_dim=head_dim,
                        kv_lens=[n + q_len for n in lens], extend_lens=[q_len] * len(lens), pool_factor=1.1)
    g = wl.to(gpu)
    print(f"repeat split-K head_dim={head_dim} q_len={q_len}", flush=True)
    outs = [_prefill(g, q_len) for _ in range(RUNS)]
    torch.cuda.synchronize()
    for i, out in enumerate(outs[1:], 1):
        assert torch.equal(out.view(torch.int16), outs[0].view(torch.int16)), f"run {i} differs from run 0"


@pytest.mark.parametrize("head_dim", [128, 256])
def test_decode_repeat_bit_identical(gpu, head_dim):
    wl = build_workload("t", "decode", seed=930, n_q=32, n_kv=8, head_dim=head_dim,
                        kv_lens=[1, 17, 900, 4000, 64, 2500, 129, 33, 7000, 2, 640], pool_factor=1.1)
    g = wl.to(gpu)
    print(f"repeat decode head_dim={head_dim}", flush=True)
    outs = [paged_decode_attention(g.q, g.k_cache, g.v_cache, g.kv_indptr, g.kv_indices,
                                   g.num_kv_splits, g.sm_scale, g.max_kv_splits) for _ in range(RUNS)]
    torch.cuda.synchronize()
    for i, out in enumerate(outs[1:], 1):
        assert torch.equal(out.view(torch.int16), outs[0].view(torch.int16)), f"run {i} differs from run 0"


@pytest.mark.parametrize("cfg,variant,head_dim", [(2, "", 128), (3, "", 128), (3, "", 256), (5, "", 128),
                                                  (5, "window", 128)])
def test_benchmark_shapes_repeat_bit_identical(gpu, cfg, variant, head_dim):
    """The same demand at full size, where every compute unit is busy and waves drift apart."""
    from _gpu_util import run_gpu
    from mini_sglang_amd.workloads import config_workload

    wl = config_workload(cfg, variant=variant, pool_device=gpu, head_dim=head_dim)
    print(f"repeat shape {cfg} {variant} head_dim={head_dim}", flush=True)
    first, g = run_gpu(wl, gpu)
    first = first.view(torch.int16)
    for i in range(1, 16):
        if wl.kind == "decode":
            out = paged_decode_attention(g.q, g.k_cache, g.v_cache, g.kv_indptr, g.kv_indices,
                                         g.num_kv_splits, g.sm_scale, g.max_kv_splits)
        else:
            out = _prefill(g, g.max_len_extend, is_cross_attention=g.is_cross_attention,
                           sliding_window_size=g.sliding_window_size)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu().view(torch.int16), first), f"run {i} differs from run 0"


@pytest.mark.parametrize("seed", range(40))
def test_random_extend_shapes_repeat_bit_identical(gpu, seed):
    """Random ragged extends (both head sizes, every mask, forced key splits on half of them), each
    launched 12 times: a race that needs an unusual shape still has to show as a changed bit."""
    import random

    from test_gpu_fuzz import HEADS, _length

    rng = random.Random(7000 + seed)
    n_q, n_kv = rng.choice(HEADS)
    d = rng.choice([128, 256])
    batch = rng.randrange(1, 7)
    ext = [max(1, _length(rng, 400)) for _ in range(batch)]
    kv = [e + (_length(rng, 3000) if rng.random() < 0.8 else 0) for e in ext]
    is_cross = rng.random() < 0.3
    window = rng.choice([0, 0, 17, 100, 1000])
    splits = rng.choice([0, 0, 2, 5, 32])
    wl = build_workload("t", "prefill", seed=seed, n_q=n_q, n_kv=n_kv, head_dim=d, kv_lens=kv,
                        extend_lens=ext, pool_factor=1.2, is_cross_attention=is_cross,
                        sliding_window_size=window)
    g = wl.to(gpu)
    print(f"repeat random seed={seed} heads={n_q}/{n_kv} d={d} ext={ext} kv={kv} cross={is_cross} "
          f"W={window} key_splits={splits}", flush=True)
    _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, splits)
    outs = [_prefill(g, max(ext), is_cross_attention=is_cross, sliding_window_size=window)
            for _ in range(12)]
    torch.cuda.synchronize()
    _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, 0)
    for i, out in enumerate(outs[1:], 1):
        assert torch.equal(out.view(torch.int16), outs[0].view(torch.int16)), f"run {i} differs from run 0"


@pytest.mark.parametrize("seed", range(30))
def test_random_decode_and_verify_shapes_repeat_bit_identical(gpu, seed):
    """The split-K kernel and its merge on random batches (empty and one-token requests, several
    requests per segment, one request over many segments), decode and short query blocks."""
    import random

    from test_gpu_fuzz import HEADS, _length

    rng = random.Random(8000 + seed)
    n_q, n_kv = rng.choice([h for h in HEADS if h[0] // h[1] <= 16])
    d = rng.choice([128, 256])
    batch = rng.randrange(1, 40)
    q_len = rng.choice([0, 0, 1, 2, 3, 8])  # 0: decode
    q_len = min(q_len, 64 // (n_q // n_kv))
    hi = rng.choice([40, 300, 5000])
    lens = [_length(rng, hi) for _ in range(batch)]
    if q_len == 0:
        lens = [max(n, 1) if i == 0 else n for i, n in enumerate(lens)]
        wl = build_workload("t", "decode", seed=seed, n_q=n_q, n_kv=n_kv, head_dim=d, kv_lens=lens,
                            pool_factor=1.2)
        g = wl.to(gpu)
        run = lambda: paged_decode_attention(g.q, g.k_cache, g.v_cache, g.kv_indptr, g.kv_indices,
                                             g.num_kv_splits, g.sm_scale, g.max_kv_splits)
    else:
        window = rng.choice([0, 0, 64, 1000])
        wl = build_workload("t", "prefill", seed=seed, n_q=n_q, n_kv=n_kv, head_dim=d,
                            kv_lens=[n + q_len for n in lens], extend_lens=[q_len] * batch,
                            pool_factor=1.2, sliding_window_size=window)
        g = wl.to(gpu)
        run = lambda: _prefill(g, q_len, sliding_window_size=window)
    print(f"repeat random split-K seed={seed} heads={n_q}/{n_kv} d={d} q_len={q_len} lens={lens}", flush=True)
    outs = [run() for _ in range(12)]
    torch.cuda.synchronize()
    for i, out in enumerate(outs[1:], 1):
        assert torch.equal(out.view(torch.int16), outs[0].view(torch.int16)), f"run {i} differs from run 0"


@pytest.mark.parametrize("head_dim", [128, 256])
@pytest.mark.parametrize("kind", ["extend", "extend_split", "verify", "decode"])
def test_repeat_bit_identical_while_another_stream_saturates_memory(gpu, head_dim, kind):
    """Large device copies on a second stream change when loads return and how far waves drift
    apart; the results must not notice."""
    if kind == "decode":
        wl = build_workload("t", "decode", seed=940, n_q=32, n_kv=8, head_dim=head_dim,
                            kv_lens=[3000, 17, 900, 4000, 64, 2500, 129, 7000], pool_factor=1.1)
        g = wl.to(gpu)
        run = lambda: paged_decode_attention(g.q, g.k_cache, g.v_cache, g.kv_indptr, g.kv_indices,
                                             g.num_kv_splits, g.sm_scale, g.max_kv_splits)
    else:
        ext = {"extend": [300, 70, 513], "extend_split": [300], "verify": [6, 6, 6, 6]}[kind]
        pre = {"extend": [3000, 0, 700], "extend_split": [20000], "verify": [3000, 17, 900, 4000]}[kind]
        wl = build_workload("t", "prefill", seed=941, n_q=16, n_kv=4, head_dim=head_dim,
                            kv_lens=[p + e for p, e in zip(pre, ext)], extend_lens=ext, pool_factor=1.1)
        g = wl.to(gpu)
        run = lambda: _prefill(g, max(ext))
    print(f"repeat under contention head_dim={head_dim} {kind}", flush=True)
    quiet = run()
    torch.cuda.synchronize()
    src = torch.empty(256 << 20, dtype=torch.uint8, device=gpu)
    dst = torch.empty_like(src)
    side = torch.cuda.Stream(device=gpu)
    side.wait_stream(torch.cuda.current_stream(gpu))
    with torch.cuda.stream(side):
        for _ in range(40):
            dst.copy_(src, non_blocking=True)
    outs = [run() for _ in range(25)]
    torch.cuda.synchronize()
    for i, out in enumerate(outs):
        assert torch.equal(out.view(torch.int16), quiet.view(torch.int16)), f"run {i} differs"
