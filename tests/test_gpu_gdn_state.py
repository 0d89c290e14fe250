"""gdn_state_inplace on the GPU against the numpy oracle, on the reference's own case list
(test_and_bench/gdn_state.py:33-48, 309-335: hk 16, hv 32 / 48, decode batches 1 / 4 / 8,
prefill lengths [1] [7] [128] [33, 65] [17, 129, 257], inputs scaled by 0.05, gates through a
sigmoid) and its tolerance (max-abs 5e-4 on y and on the state)."""
import numpy as np
import pytest
import torch

from oracle import gdn_state_oracle as go

pytestmark = pytest.mark.gpu
SCALE = 0.05


def _inputs(rng, tokens, hk, hv, slots):
    f = lambda *s: go._bf16_round((SCALE * rng.standard_normal(s)).astype(np.float32))
    sig = lambda *s: go._bf16_round((1 / (1 + np.exp(-rng.standard_normal(s)))).astype(np.float32))
    d = dict(q=f(tokens, hk, 128), k=f(tokens, hk, 128), v=f(tokens, hv, 128), g=sig(tokens, hv),
             beta=sig(tokens, hv))
    state = (SCALE * rng.standard_normal((slots, hv, 128, 128))).astype(np.float32)
    return d, state


def _gpu(gpu, d, state, slot_ids, indptr, single):
    from mini_sglang_amd_kernel import gdn_state_inplace

    bf = lambda a: torch.from_numpy(a).to(torch.bfloat16).to(gpu)
    st = torch.from_numpy(state.copy()).to(gpu)
    ip = torch.from_numpy(np.asarray(indptr, np.int32)).to(gpu)
    y = gdn_state_inplace(bf(d["q"]), bf(d["k"]), bf(d["v"]), bf(d["g"]), bf(d["beta"]), st,
                          torch.from_numpy(np.asarray(slot_ids, np.int32)).to(gpu), ip,
                          single_token_mode=single)
    torch.cuda.synchronize()
    return y.float().cpu().numpy(), st.cpu().numpy()


def _check(got_y, got_st, want_y, want_st, what):
    dy, ds = np.abs(got_y - want_y).max(), np.abs(got_st - want_st).max()
    assert dy <= 5e-4 and ds <= 5e-4, (what, float(dy), float(ds))


@pytest.mark.parametrize("hv", [32, 48])
@pytest.mark.parametrize("batch", [1, 4, 8])
def test_decode_cases_of_the_reference(gpu, hv, batch):
    rng = np.random.default_rng(100 + hv + batch)
    d, state = _inputs(rng, batch, 16, hv, batch + 1)
    slots = np.arange(batch)
    print(f"gdn decode hv={hv} batch={batch}", flush=True)
    got_y, got_st = _gpu(gpu, d, state, slots, np.arange(batch + 1), True)
    want_y, want_st = go.gdn_state_inplace(d["q"], d["k"], d["v"], d["g"], d["beta"], state, slots,
                                           None, single_token_mode=True)
    _check(got_y, got_st, want_y, want_st, f"decode hv={hv} batch={batch}")


@pytest.mark.parametrize("hv", [32, 48])
@pytest.mark.parametrize("lengths", [[1], [7], [128], [33, 65], [17, 129, 257]])
def test_prefill_cases_of_the_reference(gpu, hv, lengths):
    rng = np.random.default_rng(200 + hv + sum(lengths))
    batch, total = len(lengths), sum(lengths)
    d, state = _inputs(rng, total, 16, hv, batch + 6)
    slots = np.arange(1, batch + 1)
    indptr = np.concatenate([[0], np.cumsum(lengths)])
    print(f"gdn prefill hv={hv} lengths={lengths}", flush=True)
    got_y, got_st = _gpu(gpu, d, state, slots, indptr, False)
    want_y, want_st = go.gdn_state_inplace(d["q"], d["k"], d["v"], d["g"], d["beta"], state, slots,
                                           indptr)
    _check(got_y, got_st, want_y, want_st, f"prefill hv={hv} lengths={lengths}")
    # slots no request names keep their bits
    other = np.setdiff1d(np.arange(state.shape[0]), slots)
    np.testing.assert_array_equal(got_st[other], state[other])


def test_many_requests_empty_request_permuted_slots_and_ungrouped_heads(gpu):
    # enough (request, head) pairs for the multi-row variants of the kernel; one request
    # without tokens; slots in scrambled order; hk == hv
    rng = np.random.default_rng(7)
    lengths = [3, 0, 5, 1] * 16
    batch, total = len(lengths), sum(lengths)
    d, state = _inputs(rng, total, 16, 16, batch + 3)
    slots = rng.permutation(batch + 3)[:batch]
    indptr = np.concatenate([[0], np.cumsum(lengths)])
    print("gdn many requests", flush=True)
    got_y, got_st = _gpu(gpu, d, state, slots, indptr, False)
    want_y, want_st = go.gdn_state_inplace(d["q"], d["k"], d["v"], d["g"], d["beta"], state, slots,
                                           indptr)
    _check(got_y, got_st, want_y, want_st, "many requests")
    for b, n in enumerate(lengths):
        if n == 0:
            np.testing.assert_array_equal(got_st[slots[b]], state[slots[b]])
    print("gdn decode batch 256", flush=True)
    d, state = _inputs(rng, 256, 16, 32, 257)
    slots = rng.permutation(257)[:256]
    got_y, got_st = _gpu(gpu, d, state, slots, np.arange(257), True)
    want_y, want_st = go.gdn_state_inplace(d["q"], d["k"], d["v"], d["g"], d["beta"], state, slots,
                                           None, single_token_mode=True)
    _check(got_y, got_st, want_y, want_st, "decode batch 256")


def test_argument_errors_carry_the_reference_texts(gpu):
    from mini_sglang_amd_kernel import gdn_state_inplace

    z = lambda *s, dt=torch.bfloat16: torch.zeros(*s, dtype=dt, device=gpu)
    q, k, v, g, beta = z(2, 2, 128), z(2, 2, 128), z(2, 4, 128), z(2, 4), z(2, 4)
    st = z(3, 4, 128, 128, dt=torch.float32)
    ids, ip = z(2, dt=torch.int32), torch.tensor([0, 1, 2], dtype=torch.int32, device=gpu)
    with pytest.raises(RuntimeError, match="state must be float32"):
        gdn_state_inplace(q, k, v, g, beta, st.to(torch.bfloat16), ids, ip)
    with pytest.raises(RuntimeError, match="requires dk=dv=128"):
        gdn_state_inplace(z(2, 2, 64), z(2, 2, 64), v, g, beta, z(3, 4, 128, 64, dt=torch.float32), ids, ip)
    with pytest.raises(RuntimeError, match="hv must be a multiple of hk"):
        gdn_state_inplace(z(2, 3, 128), z(2, 3, 128), v, g, beta, st, ids, ip)
    with pytest.raises(RuntimeError, match="decode mode expects one token per request"):
        gdn_state_inplace(q, k, v, g, beta, st, z(1, dt=torch.int32), ip, single_token_mode=True)
    with pytest.raises(RuntimeError, match=r"qo_indptr must have shape \(batch \+ 1,\)"):
        gdn_state_inplace(q, k, v, g, beta, st, ids, ip[:2])
