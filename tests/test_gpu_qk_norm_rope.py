"""Fused q/k RMSNorm + rotary embedding + KV-store (msgl_qk_norm_rope_store) against the numpy
oracle.  v and untouched pool rows bit-exact; q and k within one bf16 step of the oracle (the
two sides evaluate exp2 / sin / cos with different routines) and inside the path's stated
tolerance (max-abs 2e-2, mean-abs 2e-3 on unit-scale data)."""
import numpy as np
import pytest
import torch

from oracle import qk_norm_rope_oracle as qo

pytestmark = pytest.mark.gpu


def _bf16_t(a, dev):
    return torch.from_numpy(a).to(torch.bfloat16).to(dev)


def _run_case(gpu, L, n_q, n_kv, d, slots, max_pos, base, seed, fused_view=False):
    from mini_sglang_amd_kernel import qk_norm_rope_store

    rng = np.random.default_rng(seed)
    r = lambda *s: qo.bf16_round(rng.standard_normal(s).astype(np.float32))
    q, k, v = r(L, n_q, d), r(L, n_kv, d), r(L, n_kv, d)
    qw = qo.bf16_round((1 + 0.2 * rng.standard_normal(d)).astype(np.float32))
    kw = qo.bf16_round((1 + 0.2 * rng.standard_normal(d)).astype(np.float32))
    pos = rng.integers(0, max_pos + 1, size=L).astype(np.int32)
    loc = rng.permutation(slots)[:L].astype(np.int32)
    kc, vc = r(slots, n_kv, d), r(slots, n_kv, d)
    want_q, want_kc, want_vc = qo.qk_norm_rope_store(q, k, v, qw, kw, pos, loc, kc, vc, 1e-6, base)
    tq, tk, tv = _bf16_t(q, gpu), _bf16_t(k, gpu), _bf16_t(v, gpu)
    if fused_view:  # q, k, v as views of one (L, (n_q + 2 n_kv) d) projection output
        fused = torch.cat([tq.reshape(L, -1), tk.reshape(L, -1), tv.reshape(L, -1)], dim=1)
        tq = fused[:, : n_q * d].view(L, n_q, d)
        tk = fused[:, n_q * d: (n_q + n_kv) * d].view(L, n_kv, d)
        tv = fused[:, (n_q + n_kv) * d:].view(L, n_kv, d)
    tkc, tvc = _bf16_t(kc, gpu), _bf16_t(vc, gpu)
    print(f"qk_norm_rope_store L={L} n_q={n_q} n_kv={n_kv} d={d} max_pos={max_pos} view={fused_view}",
          flush=True)
    got_q = qk_norm_rope_store(tq, tk, tv, _bf16_t(qw, gpu), _bf16_t(kw, gpu),
                               torch.from_numpy(pos).to(gpu), torch.from_numpy(loc).to(gpu),
                               tkc, tvc, eps=1e-6, rope_base=base)
    torch.cuda.synchronize()
    got_q = got_q.float().cpu().numpy()
    got_kc, got_vc = tkc.float().cpu().numpy(), tvc.float().cpu().numpy()
    np.testing.assert_array_equal(got_vc, want_vc)  # v is a bit copy, other rows untouched
    untouched = np.setdiff1d(np.arange(slots), loc)
    np.testing.assert_array_equal(got_kc[untouched], want_kc[untouched])
    for got, want, name in ((got_q, want_q, "q"), (got_kc[loc], want_kc[loc], "k")):
        diff = np.abs(got - want)
        # one bf16 step of the larger magnitude, plus the angle's float32 granularity at long positions
        h = want.shape[-1] // 2
        pair = np.hypot(want[..., :h], want[..., h:])  # an angle error moves a value by angle * pair norm
        pair = np.concatenate([pair, pair], axis=-1)
        # (a value is x cos - y sin of a pair of norm `pair`: an intermediate rounding of x or y
        # moves it by a step of THEIR size, however small the difference comes out)
        step = 2.0 ** -7 * np.maximum(np.maximum(np.abs(want), pair), 2.0 ** -6) + 2e-7 * max_pos * pair
        # An intermediate rounding (normalised value, weighted value) that sits on a tie can fall
        # the other way with float32 statistics; that moves a result by up to two more steps
        # and is rare.
        assert np.all(diff <= 3 * step), (name, float(diff.max()), float((diff / step).max()))
        assert np.mean(diff > step) < 5e-3, (name, float(np.mean(diff > step)))
        # the path's stated tolerance, plus what float32 angles cost at this position range
        # (pos * inv_freq carries 2^-24 of pos radians: 6e-3 rad at position 100000)
        angle_slack = 2e-7 * max_pos * float(pair.max())
        # (2e-2 on unit-scale values; one bf16 step of the largest value where that is more)
        assert diff.max() <= max(2e-2, 2.0 ** -7 * float(np.abs(want).max())) + angle_slack, name
        assert diff.mean() <= 2e-3 + 2e-7 * max_pos * float(pair.mean()), name
    return got_q


@pytest.mark.parametrize("L,n_q,n_kv,d", [(1, 16, 8, 128), (64, 32, 8, 128), (333, 8, 2, 128),
                                          (4096, 32, 8, 128), (50, 4, 4, 256), (7, 64, 8, 128)])
def test_matches_the_oracle(gpu, L, n_q, n_kv, d):
    _run_case(gpu, L, n_q, n_kv, d, slots=L + 37, max_pos=8192, base=1e6, seed=L + n_q)


def test_long_positions_small_base_and_fused_projection_views(gpu):
    _run_case(gpu, 40, 16, 8, 128, slots=64, max_pos=131071, base=1e6, seed=1)
    _run_case(gpu, 40, 16, 8, 128, slots=64, max_pos=4000, base=1e4, seed=2)
    _run_case(gpu, 130, 32, 8, 128, slots=200, max_pos=9000, base=1e6, seed=3, fused_view=True)


def test_position_zero_is_the_plain_norm_and_empty_input_is_a_no_op(gpu):
    from mini_sglang_amd_kernel import qk_norm_rope_store

    rng = np.random.default_rng(9)
    q = qo.bf16_round(rng.standard_normal((5, 8, 128)).astype(np.float32))
    k = qo.bf16_round(rng.standard_normal((5, 2, 128)).astype(np.float32))
    w = np.ones(128, dtype=np.float32)
    tkc = torch.zeros((8, 2, 128), dtype=torch.bfloat16, device=gpu)
    tvc = torch.zeros_like(tkc)
    print("qk_norm_rope_store position 0", flush=True)
    got = qk_norm_rope_store(_bf16_t(q, gpu), _bf16_t(k, gpu), _bf16_t(k, gpu), _bf16_t(w, gpu),
                             _bf16_t(w, gpu), torch.zeros(5, dtype=torch.int32, device=gpu),
                             torch.arange(5, dtype=torch.int32, device=gpu), tkc, tvc,
                             eps=1e-6, rope_base=1e6)
    torch.cuda.synchronize()
    want = torch.nn.functional.rms_norm(torch.from_numpy(q).double(), (128,), None, 1e-6).numpy()
    np.testing.assert_allclose(got.float().cpu().numpy(), want, rtol=2 ** -7, atol=1e-6)
    print("qk_norm_rope_store empty", flush=True)
    e = torch.zeros((0, 8, 128), dtype=torch.bfloat16, device=gpu)
    ek = torch.zeros((0, 2, 128), dtype=torch.bfloat16, device=gpu)
    out = qk_norm_rope_store(e, ek, ek, _bf16_t(w, gpu), _bf16_t(w, gpu),
                             torch.zeros(0, dtype=torch.int32, device=gpu),
                             torch.zeros(0, dtype=torch.int32, device=gpu), tkc, tvc,
                             eps=1e-6, rope_base=1e6)
    assert out.shape == (0, 8, 128)


def test_backend_fused_forward_equals_norm_rope_then_forward(gpu):
    """The fused layer entry gives what the unfused chain gives when q, k are prepared by the
    oracle: same attention output (both run the same attention kernels on the same pool)."""
    from mini_sglang_amd.attention.backend import AttnBackend
    from mini_sglang_amd.kvcache import MHAKVCache
    from test_oracle_metadata import _Req

    rng = np.random.default_rng(21)
    n_q, n_kv, d, slots = 16, 4, 128, 256
    table = rng.permutation(slots).astype(np.int32).reshape(4, 64)
    reqs = [_Req(0, 20, 30), _Req(2, 0, 17), _Req(3, 63, 64)]

    class Cfg:
        head_dim = d

    def make():
        kv = MHAKVCache(num_kv_heads=n_kv, num_layers=1, head_dim=d, num_pages=slots,
                        dtype=torch.bfloat16, device=gpu)
        pre = torch.from_numpy(qo.bf16_round(rng2.standard_normal((slots, n_kv, d)).astype(np.float32)))
        kv.k_cache(0).copy_(pre.to(torch.bfloat16))
        kv.v_cache(0).copy_(pre.flip(0).to(torch.bfloat16))
        return kv, AttnBackend(Cfg(), kv, torch.from_numpy(table).to(gpu))

    L = sum(r.extend_len for r in reqs)
    q = qo.bf16_round(rng.standard_normal((L, n_q, d)).astype(np.float32))
    k = qo.bf16_round(rng.standard_normal((L, n_kv, d)).astype(np.float32))
    v = qo.bf16_round(rng.standard_normal((L, n_kv, d)).astype(np.float32))
    w = qo.bf16_round((1 + 0.1 * rng.standard_normal(d)).astype(np.float32))

    class Batch:
        pass

    outs = []
    for fused in (True, False):
        rng2 = np.random.default_rng(5)
        kv, be = make()
        b = Batch()
        b.attn_metadata = be.build_prefill_metadata(reqs)
        b.out_loc = torch.cat([torch.from_numpy(table[r.table_idx, r.cached_len:r.device_len])
                               for r in reqs]).to(gpu)
        pos = b.attn_metadata.positions.cpu().numpy()
        print(f"backend fused={fused}", flush=True)
        if fused:
            o = be.forward_fused_norm_rope(_bf16_t(q, gpu), _bf16_t(k, gpu), _bf16_t(v, gpu),
                                           _bf16_t(w, gpu), _bf16_t(w, gpu), 0, b,
                                           rms_norm_eps=1e-6, rope_base=1e6)
        else:
            qn = qo.rope(qo.rms_norm(q, w, 1e-6), pos, 1e6)
            kn = qo.rope(qo.rms_norm(k, w, 1e-6), pos, 1e6)
            o = be.forward(_bf16_t(qn, gpu), _bf16_t(kn, gpu), _bf16_t(v, gpu), 0, b)
        torch.cuda.synchronize()
        outs.append(o.float().cpu().numpy())
    diff = np.abs(outs[0] - outs[1])
    assert diff.max() <= 2e-2 and diff.mean() <= 2e-3, (diff.max(), diff.mean())
