"""The five benchmark shapes at FULL size on the GPU.

Parity against the CPU oracle on the same seeded inputs (all requests where the oracle
finishes in seconds, the shortest requests otherwise), KV-pool bit-exactness after the
store, and size-independent properties at full size: independence of the split, one extend
== two chunked extends, decode(L) == extend(q_len 1)."""
import pytest
import torch

import oracle
from _gpu_util import run_gpu, run_oracle
from _util import assert_close_bf16
from mini_sglang_amd.workloads import config_workload

pytestmark = pytest.mark.gpu


def _shortest(wl, n):
    order = sorted(range(wl.batch), key=lambda b: wl.kv_lens[b])
    return sorted(order[:n])


def test_cfg1_small_decode_full_oracle(gpu):
    wl = config_workload(1)
    assert wl.kv_lens == [37, 128, 500, 1023] and wl.k_cache.shape[0] == 512 * 16
    got, _ = run_gpu(wl, gpu)
    want, _ = run_oracle(wl)
    assert_close_bf16(got, want, "cfg1")


def test_cfg2_decode_batch64_full_oracle(gpu):
    print("cfg2 build", flush=True)
    wl = config_workload(2)
    assert wl.batch == 64 and min(wl.kv_lens) >= 1024 and max(wl.kv_lens) <= 8192
    got, _ = run_gpu(wl, gpu)
    print("cfg2 oracle", flush=True)
    want, _ = run_oracle(wl, precision="f32")
    assert_close_bf16(got, want, "cfg2")


def test_cfg3_chunked_extend_with_store(gpu):
    from mini_sglang_amd_kernel import paged_prefill_attention, store_kv_cache

    print("cfg3 build", flush=True)
    wl = config_workload(3)
    assert wl.batch == 8 and wl.extend_lens == [512] * 8
    got, g = run_gpu(wl, gpu)
    assert torch.isfinite(got.float()).all()
    # pools after the store: bit-exact against the oracle's row scatter
    ref = wl.clone_pools()
    oracle.store_kv_cache(ref.k_cache, ref.v_cache, ref.out_loc, ref.new_k, ref.new_v)
    assert torch.equal(g.k_cache.cpu().view(torch.int16), ref.k_cache.view(torch.int16))
    assert torch.equal(g.v_cache.cpu().view(torch.int16), ref.v_cache.view(torch.int16))
    # oracle on the two shortest requests (all 512 rows, all heads)
    reqs = _shortest(wl, 2)
    print(f"cfg3 oracle on requests {reqs}", flush=True)
    sub = wl.select(reqs)
    want, _ = run_oracle(sub, precision="f32")
    qo = wl.qo_indptr.tolist()
    rows = torch.cat([torch.arange(qo[b], qo[b + 1]) for b in reqs])
    assert_close_bf16(got[rows], want, "cfg3 sampled requests")
    # full size, no oracle: one 512-token extend == a 256-token extend then another on
    # prefix + 256 (the stored pool already holds all 512 new rows)
    print("cfg3 chunked-extend property", flush=True)
    halves = []
    for part in (0, 1):
        ext = [256] * wl.batch
        kv_lens = [p + 256 * (part + 1) for p in wl.prefixes]
        ip = wl.kv_indptr.tolist()
        idx = torch.cat([wl.kv_indices[ip[b]:ip[b] + kv_lens[b]] for b in range(wl.batch)])
        qrows = torch.cat([torch.arange(qo[b] + 256 * part, qo[b] + 256 * (part + 1))
                           for b in range(wl.batch)])
        kvp = torch.cumsum(torch.tensor([0] + kv_lens), 0).to(torch.int32)
        qop = torch.cumsum(torch.tensor([0] + ext), 0).to(torch.int32)
        pre = torch.tensor([p + 256 * part for p in wl.prefixes], dtype=torch.int32)
        out = paged_prefill_attention(g.q[qrows.to(gpu)], g.k_cache, g.v_cache, qop.to(gpu),
                                      kvp.to(gpu), idx.to(gpu), pre.to(gpu), g.sm_scale, 256)
        halves.append((qrows, out.cpu()))
    torch.cuda.synchronize()
    for qrows, out in halves:
        assert_close_bf16(out, got[qrows].float(), "cfg3 chunked extend", max_tol=8e-3, mean_tol=4e-4)


def test_cfg4_long_context_decode_split_and_sampled_oracle(gpu):
    from mini_sglang_amd_kernel import _lib

    print("cfg4 build", flush=True)
    wl = config_workload(4, pool_device=gpu)
    assert wl.batch == 16 and min(wl.kv_lens) >= 32768 and max(wl.kv_lens) <= 131072
    got, g = run_gpu(wl, gpu)
    assert torch.isfinite(got.float()).all()
    # the merged result must not depend on where the stream is cut
    for segments in (16, 509):
        print(f"cfg4 segments={segments}", flush=True)
        _lib.set_tuning(_lib.TUNE_SEGMENTS, segments)
        other, _ = run_gpu(wl, gpu)
        _lib.set_tuning(_lib.TUNE_SEGMENTS, 0)
        assert_close_bf16(other, got.float(), f"cfg4 split invariance ({segments})",
                          max_tol=4e-3, mean_tol=2e-4)
    reqs = _shortest(wl, 2)
    print(f"cfg4 oracle on requests {reqs}", flush=True)
    sub = wl.select(reqs).to("cpu")
    want, _ = run_oracle(sub, precision="f32")
    assert_close_bf16(got[reqs], want, "cfg4 sampled requests")


@pytest.mark.parametrize("variant", ["", "window"])
def test_cfg5_speculative_verify_full_oracle(gpu, variant):
    print(f"cfg5 {variant} build", flush=True)
    wl = config_workload(5, variant=variant)
    assert wl.batch == 32 and wl.extend_lens == [8] * 32
    assert wl.sliding_window_size == (1024 if variant else 0)
    got, _ = run_gpu(wl, gpu)
    print("cfg5 oracle", flush=True)
    want, _ = run_oracle(wl, precision="f32")
    assert_close_bf16(got, want, f"cfg5 {variant}")


_FULL_SIZE_SHAPES = [(2, ""), (3, ""), (3, "head_dim_256"), (4, ""), (5, ""), (5, "window")]


def _full_size_workload(cfg, variant, gpu):
    if variant == "head_dim_256":
        return config_workload(cfg, head_dim=256)
    return config_workload(cfg, variant=variant, **({"pool_device": gpu} if cfg == 4 else {}))


def _uniform_attention_expected(g):
    """With q = 0 every visible key weighs the same, so a row's output is the plain mean of the
    V rows it may see: sums in float64 (torch on the GPU as the adding machine), no oracle."""
    group = g.n_q // g.n_kv
    ip = g.kv_indptr.tolist()
    window, cross = g.sliding_window_size, g.is_cross_attention
    outs = []
    for b in range(g.batch):
        rows = g.v_cache[g.kv_indices[ip[b]:ip[b + 1]].long()].double()  # (kv_len, n_kv, d)
        kv_len = rows.shape[0]
        if g.kind == "decode":
            mean = rows.sum(0, keepdim=True) / kv_len
        else:
            ext = g.extend_lens[b]
            before = torch.cat([torch.zeros_like(rows[:1]), rows.cumsum(0)])  # sum of keys < t
            pos = (kv_len - ext) + torch.arange(ext, device=rows.device)
            hi = torch.full_like(pos, kv_len - 1) if cross else pos
            lo = torch.clamp(pos - window + 1, min=0) if window > 0 else torch.zeros_like(pos)
            mean = (before[hi + 1] - before[lo]) / (hi + 1 - lo).double()[:, None, None]
        outs.append(mean.repeat_interleave(group, dim=1))
        del rows
    return torch.cat(outs)


@pytest.mark.parametrize("cfg,variant", _FULL_SIZE_SHAPES)
def test_uniform_attention_closed_form_every_row_full_size(gpu, cfg, variant):
    """Full size, every request, every row and head, against a closed form: q = 0 makes the
    weights exactly 1 / (visible keys), so a dropped, doubled or wrongly gathered key, a
    wrong causal limit or window floor, or a mis-merged segment moves the result by about
    |v| / keys, which the bound below (bf16 rounding of the result plus 4e-5) does not cover
    for a v of ordinary size.  (4e-5: where the partials of a request's shares are much larger
    than their mean, which is what q = 0 on random V produces, their rounding to IEEE half,
    2^-12 of a partial of 0.05 .. 0.1, is what is left of the error.)"""
    print(f"cfg{cfg} {variant} uniform attention: build", flush=True)
    wl = _full_size_workload(cfg, variant, gpu)
    wl.q.zero_()
    got, g = run_gpu(wl, gpu)
    print(f"cfg{cfg} {variant} uniform attention: closed form", flush=True)
    want = _uniform_attention_expected(g)
    diff = (got.to(gpu).double() - want).abs()
    bound = want.abs() * 2.0 ** -8 + 4e-5
    worst = float((diff - bound).max())
    assert worst <= 0.0, (f"cfg{cfg} {variant}: a row is {worst:.3e} beyond its bound; "
                          f"max-abs diff {float(diff.max()):.3e}")


def _needle_queries(g, gap_nats=28.0):
    """A query per (row, q head) that points at ONE visible key of its own: q = c k* / |k*|^2,
    with c large enough that the softmax weight of every other key is below e^-gap.  Targets
    cycle through the last visible key (the causal limit / the diagonal tile), the first visible
    key (position 0 or the window floor) and one in between.  Returns (q, expected output):
    the expected row is the target's V row, bit for bit."""
    group = g.n_q // g.n_kv
    ip = g.kv_indptr.tolist()
    window, cross = g.sliding_window_size, g.is_cross_attention
    dev = g.k_cache.device
    head = torch.arange(g.n_q, device=dev)
    qs, wants = [], []
    row0 = 0
    for b in range(g.batch):
        idx = g.kv_indices[ip[b]:ip[b + 1]].long()
        kv_len, ext = idx.numel(), g.extend_lens[b]
        pos = (kv_len - ext) + torch.arange(ext, device=dev)
        hi = torch.full_like(pos, kv_len - 1) if (cross or g.kind == "decode") else pos
        lo = torch.clamp(pos - window + 1, min=0) if window > 0 else torch.zeros_like(pos)
        pick = (row0 + torch.arange(ext, device=dev))[:, None] + head[None, :]  # (ext, n_q)
        mid = lo[:, None] + (pick * 7919) % (hi - lo + 1)[:, None]
        target = torch.where(pick % 3 == 0, hi[:, None], torch.where(pick % 3 == 1, lo[:, None], mid))
        slot = idx[target]                                         # (ext, n_q)
        kvh = (head // group)[None, :].expand_as(slot)
        k_star = g.k_cache[slot, kvh].double()                     # (ext, n_q, d)
        norm2 = (k_star * k_star).sum(-1)                          # (ext, n_q)
        u = k_star / norm2[..., None]
        # other keys' logits relative to the target's: k_j . k* / |k*|^2, largest over the request
        # (keys the row cannot see included: that only makes c larger than needed)
        k_heads = g.k_cache[idx][:, head // group].float()         # (kv_len, n_q, d)
        ratio = torch.einsum("thd,ehd->eht", k_heads, u.float())   # (ext, n_q, kv_len)
        ratio.scatter_(2, target[..., None], float("-inf"))
        worst = ratio.max(dim=2).values.double().clamp(min=0.0)
        assert float(worst.max()) < 0.9, "another key is nearly parallel to a target"
        c = gap_nats / (g.sm_scale * (1.0 - worst))
        del k_heads, ratio
        qs.append((u * c[..., None]).to(torch.bfloat16))
        wants.append(g.v_cache[slot, kvh])
        row0 += ext
    return torch.cat(qs), torch.cat(wants)


@pytest.mark.parametrize("cfg,variant", _FULL_SIZE_SHAPES)
def test_needle_queries_return_their_key_every_row_full_size(gpu, cfg, variant):
    """Full size, every request, row and head, no oracle: each query points at one visible key
    (its last, its first, or one in between), every other key's weight is below e^-28, so the
    row must be that key's V row.  Pins what the uniform-attention check leaves open: the QK
    product, K and V gathered by the same slot id, and the score path at the mask edges (a
    target wrongly masked, or a key beyond the edge wrongly seen, changes the whole row)."""
    from mini_sglang_amd_kernel import store_kv_cache

    print(f"cfg{cfg} {variant} needle queries: build", flush=True)
    wl = _full_size_workload(cfg, variant, gpu)
    g = wl.to(gpu)
    if g.out_loc is not None:
        store_kv_cache(g.k_cache, g.v_cache, g.out_loc, g.new_k, g.new_v)
    q, want = _needle_queries(g)
    g.q = q.reshape(g.q.shape)
    print(f"cfg{cfg} {variant} needle queries: run", flush=True)
    got, _ = run_gpu(g, gpu, store=False)
    got = got.to(gpu).reshape(want.shape)
    exact = (got.view(torch.int16) == want.view(torch.int16)).all(dim=-1)
    diff = (got.double() - want.double()).abs()
    bound = want.double().abs() * 2.0 ** -8 + 1e-6
    assert bool((diff <= bound).all()), (
        f"cfg{cfg} {variant}: {int((~(diff <= bound).all(dim=-1)).sum())} rows are not their "
        f"target's V row; max-abs diff {float(diff.max()):.3e}")
    assert float(exact.double().mean()) > 0.99, "fewer than 99 % of the rows are bit-exact copies"


@pytest.mark.parametrize("head_dim", [128, 256])
@pytest.mark.parametrize("lens,ext", [([40000], 1), ([70000, 300, 5000], 1), ([30000], 8),
                                      ([20000, 900], 3)])
def test_few_long_requests_merge_of_many_partials(gpu, lens, ext, head_dim):
    """One long request alone (or beside short ones) is cut into as many segments as the chip
    has workgroups, so the merge sees up to a hundred partials per row: both closed forms
    (uniform weights, needle queries), every row and head, decode and short query blocks."""
    from mini_sglang_amd.workloads import build_workload

    kind = "decode" if ext == 1 else "prefill"
    wl = build_workload(f"long_{lens}_{ext}", kind, seed=7, n_q=16, n_kv=4, head_dim=head_dim,
                        kv_lens=lens, extend_lens=[ext] * len(lens), pool_device=gpu)
    g = wl.to(gpu)
    q_rand = g.q.clone()
    g.q = torch.zeros_like(q_rand)
    got, _ = run_gpu(g, gpu, store=False)
    want = _uniform_attention_expected(g)
    diff = (got.to(gpu).double().reshape(want.shape) - want).abs()
    assert float((diff - (want.abs() * 2.0 ** -8 + 4e-5)).max()) <= 0.0, (
        f"uniform attention: max-abs diff {float(diff.max()):.3e}")
    q, want = _needle_queries(g)
    g.q = q.reshape(q_rand.shape)
    got, _ = run_gpu(g, gpu, store=False)
    got = got.to(gpu).reshape(want.shape)
    diff = (got.double() - want.double()).abs()
    assert bool((diff <= want.double().abs() * 2.0 ** -8 + 1e-6).all()), (
        f"needle queries: max-abs diff {float(diff.max()):.3e}")
