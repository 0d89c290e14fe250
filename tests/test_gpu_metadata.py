"""On-device metadata build (msgl_build_attention_metadata) against the numpy oracle:
integer work, compared exactly."""
import numpy as np
import pytest
import torch

from oracle import metadata_oracle as mo

pytestmark = pytest.mark.gpu


def _case(rng, batch, rows, max_seq, zero_frac=0.1):
    table = rng.integers(0, 2 ** 31 - 1, size=(rows, max_seq), dtype=np.int64).astype(np.int32)
    trows = rng.integers(0, rows, size=batch).astype(np.int32)
    kv = rng.integers(1, max_seq + 1, size=batch).astype(np.int32)
    kv[rng.random(batch) < zero_frac] = 0
    ext = np.array([rng.integers(0, k + 1) for k in kv], dtype=np.int32)
    return table, trows, kv, ext


def _run(gpu, table, trows, kv, ext, **kw):
    from mini_sglang_amd_kernel import build_attention_metadata

    t = lambda a: torch.from_numpy(a).to(gpu)
    out = build_attention_metadata(t(table) if isinstance(table, np.ndarray) else table, t(trows),
                                   t(kv), None if ext is None else t(ext), **kw)
    torch.cuda.synchronize()
    return {k: v.cpu().numpy() for k, v in out.items()}


@pytest.mark.parametrize("batch,rows,max_seq", [(1, 1, 1), (1, 3, 700), (7, 9, 333), (64, 65, 8192),
                                                (150, 40, 257), (3000, 64, 40)])
def test_prefill_metadata_matches_the_oracle(gpu, batch, rows, max_seq):
    rng = np.random.default_rng(batch * 7 + rows)
    table, trows, kv, ext = _case(rng, batch, rows, max_seq)
    print(f"metadata prefill batch={batch} rows={rows} max_seq={max_seq}", flush=True)
    got = _run(gpu, table, trows, kv, ext, total_kv=int(kv.sum()), total_q=int(ext.sum()))
    want = mo.build_prefill_metadata(table, trows, kv, ext)
    for k in ("kv_indptr", "kv_indices", "qo_indptr", "prefix_lens", "positions", "num_kv_splits"):
        np.testing.assert_array_equal(got[k], want[k], err_msg=k)


@pytest.mark.parametrize("batch", [1, 64, 500])
def test_decode_metadata_matches_the_oracle(gpu, batch):
    rng = np.random.default_rng(batch)
    table, trows, kv, _ = _case(rng, batch, 80, 5000, zero_frac=0.0)
    print(f"metadata decode batch={batch}", flush=True)
    got = _run(gpu, table, trows, kv, None, total_kv=int(kv.sum()))
    want = mo.build_decode_metadata(table, trows, kv)
    for k in ("kv_indptr", "kv_indices", "num_kv_splits", "positions"):
        np.testing.assert_array_equal(got[k], want[k], err_msg=k)
    np.testing.assert_array_equal(got["qo_indptr"], np.arange(batch + 1))
    np.testing.assert_array_equal(got["prefix_lens"], kv - 1)


def test_strided_table_empty_batch_and_short_capacity(gpu):
    rng = np.random.default_rng(5)
    table, trows, kv, ext = _case(rng, 12, 10, 300)
    wide = torch.zeros((10, 512), dtype=torch.int32, device=gpu)
    wide[:, :300] = torch.from_numpy(table).to(gpu)
    print("metadata strided table", flush=True)
    got = _run(gpu, wide[:, :300], trows, kv, ext, total_kv=int(kv.sum()), total_q=int(ext.sum()))
    want = mo.build_prefill_metadata(table, trows, kv, ext)
    np.testing.assert_array_equal(got["kv_indices"], want["kv_indices"])
    # outputs sized too small: nothing is written past them, the indptr still tells the truth
    short = int(kv.sum()) // 2
    print("metadata short capacity", flush=True)
    got = _run(gpu, table, trows, kv, ext, total_kv=short, total_q=3)
    np.testing.assert_array_equal(got["kv_indices"], want["kv_indices"][:short])
    np.testing.assert_array_equal(got["positions"], want["positions"][:3])
    assert got["kv_indptr"][-1] == kv.sum() and got["qo_indptr"][-1] == ext.sum()
    print("metadata empty batch", flush=True)
    e = np.zeros(0, np.int32)
    got = _run(gpu, table, e, e, e, total_kv=0, total_q=0)
    assert got["kv_indptr"].tolist() == [0] and got["kv_indices"].size == 0


def test_backend_builds_the_same_metadata_on_the_gpu_as_on_the_host(gpu):
    from mini_sglang_amd.attention.backend import AttnBackend
    from test_oracle_metadata import _Req

    rng = np.random.default_rng(11)
    table = rng.permutation(20 * 600).astype(np.int32).reshape(20, 600)
    reqs = []
    for r in rng.permutation(20)[:13]:
        dl = int(rng.integers(1, 601))
        reqs.append(_Req(int(r), int(rng.integers(0, dl)), dl))

    class Cfg:
        head_dim = 128

    host = AttnBackend(Cfg(), None, torch.from_numpy(table))
    dev = AttnBackend(Cfg(), None, torch.from_numpy(table).to(gpu))
    print("metadata backend prefill", flush=True)
    a, b = host.build_prefill_metadata(reqs), dev.build_prefill_metadata(reqs)
    for k in ("positions", "qo_indptr", "kv_indptr", "kv_indices", "prefix_lens"):
        assert torch.equal(getattr(a, k), getattr(b, k).cpu()), k
    assert a.max_len_extend == b.max_len_extend
    print("metadata backend decode", flush=True)
    a, b = host.build_decode_metadata(reqs), dev.build_decode_metadata(reqs)
    for k in ("positions", "kv_indptr", "kv_indices", "num_kv_splits"):
        assert torch.equal(getattr(a, k), getattr(b, k).cpu()), k
    # verify-style override: K+1 virtual positions per request (backend.py:213-221)
    ext = [min(4, q.device_len) for q in reqs]
    kvl = [q.device_len for q in reqs]
    a = host.build_prefill_metadata(reqs, extend_lens=ext, kv_lens=kvl)
    b = dev.build_prefill_metadata(reqs, extend_lens=ext, kv_lens=kvl)
    for k in ("positions", "qo_indptr", "kv_indptr", "kv_indices", "prefix_lens"):
        assert torch.equal(getattr(a, k), getattr(b, k).cpu()), k
