"""Pins ``oracle/metadata_oracle.py`` (numpy restatement of
mini_sglang_mlx/attention/backend.py:205-307) with closed forms that do not retype its
formulas, and checks the torch builders of the host-side backend against it."""
import numpy as np
import pytest
import torch

from oracle import metadata_oracle as mo


def _identity_table(rows, max_seq_len):
    # slot of token t in row r is r * max_seq_len + t: a gather is then visible in the values
    return (np.arange(rows, dtype=np.int32)[:, None] * max_seq_len
            + np.arange(max_seq_len, dtype=np.int32)[None, :])


def test_indptr_is_a_running_sum_and_differences_give_back_the_lengths():
    lens = [5, 0, 17, 1, 300]
    ip = mo.build_indptr(lens)
    assert ip.dtype == np.int32 and ip[0] == 0 and ip[-1] == 323
    assert np.diff(ip).tolist() == lens
    assert mo.build_indptr([]).tolist() == [0]


def test_split_hint_is_a_step_function_of_128_tokens_capped_at_32():
    # L in (128 (s-1), 128 s] -> s, at least 1, at most 32 (backend.py:304-307)
    for s in range(1, 33):
        assert mo.compute_num_kv_splits([128 * (s - 1) + 1, 128 * s]).tolist() == [s, s]
    assert mo.compute_num_kv_splits([0, 1, 128 * 32 + 1, 10 ** 6]).tolist() == [1, 1, 32, 32]


def test_prefill_metadata_on_an_identity_table():
    table = _identity_table(6, 50)
    rows, kv, ext = [4, 0, 5], [10, 50, 7], [3, 50, 1]
    m = mo.build_prefill_metadata(table, rows, kv, ext)
    want = np.concatenate([r * 50 + np.arange(k) for r, k in zip(rows, kv)])
    assert m["kv_indices"].tolist() == want.tolist()
    assert m["kv_indptr"].tolist() == [0, 10, 60, 67]
    assert m["qo_indptr"].tolist() == [0, 3, 53, 54]
    assert m["prefix_lens"].tolist() == [7, 0, 6]
    assert m["max_len_extend"] == 50
    # positions of a request are consecutive and end at its last token
    pos, qo = m["positions"], m["qo_indptr"]
    for b in range(3):
        seg = pos[qo[b]:qo[b + 1]]
        assert seg[-1] == kv[b] - 1 and np.all(np.diff(seg) == 1) and len(seg) == ext[b]


def test_decode_metadata_on_an_identity_table():
    table = _identity_table(4, 300)
    m = mo.build_decode_metadata(table, [3, 1], [200, 1])
    assert m["kv_indptr"].tolist() == [0, 200, 201]
    assert m["kv_indices"][:3].tolist() == [900, 901, 902] and m["kv_indices"][-1] == 300
    assert m["positions"].tolist() == [199, 0]
    assert m["num_kv_splits"].tolist() == [2, 1] and m["max_kv_splits"] == 32


class _Req:
    def __init__(self, table_idx, cached_len, device_len):
        self.table_idx, self.cached_len, self.device_len = table_idx, cached_len, device_len

    @property
    def extend_len(self):
        return self.device_len - self.cached_len


@pytest.mark.parametrize("seed", [0, 1])
def test_host_backend_builders_agree_with_the_oracle(seed):
    from mini_sglang_amd.attention.backend import AttnBackend

    rng = np.random.default_rng(seed)
    rows, max_seq = 9, 400
    table = rng.permutation(rows * max_seq).astype(np.int32).reshape(rows, max_seq)
    reqs = []
    for r in rng.permutation(rows)[:6]:
        dl = int(rng.integers(1, max_seq + 1))
        reqs.append(_Req(int(r), int(rng.integers(0, dl)), dl))

    class Cfg:
        head_dim = 128

    be = AttnBackend(Cfg(), None, torch.from_numpy(table))
    pm = be.build_prefill_metadata(reqs)
    want = mo.build_prefill_metadata(table, [q.table_idx for q in reqs],
                                     [q.device_len for q in reqs], [q.extend_len for q in reqs])
    for k in ("positions", "qo_indptr", "kv_indptr", "kv_indices", "prefix_lens"):
        assert getattr(pm, k).numpy().tolist() == want[k].tolist(), k
    assert pm.max_len_extend == want["max_len_extend"]
    dm = be.build_decode_metadata(reqs, kv_lens=[q.device_len for q in reqs])
    wd = mo.build_decode_metadata(table, [q.table_idx for q in reqs], [q.device_len for q in reqs],
                                  positions=[q.cached_len for q in reqs])
    for k in ("positions", "kv_indptr", "kv_indices", "num_kv_splits"):
        assert getattr(dm, k).numpy().tolist() == wd[k].tolist(), k
