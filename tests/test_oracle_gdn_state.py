"""Pins ``oracle/gdn_state_oracle.py`` (restatement of gdn_state.metal:14-99) with closed forms
and invariants that do not retype its update rule."""
import numpy as np

from oracle import gdn_state_oracle as go

HK, HV, DK, DV = 2, 4, 128, 128


def _rand(rng, T, scale=0.05):
    f = lambda *s: go._bf16_round((scale * rng.standard_normal(s)).astype(np.float32))
    sig = lambda *s: go._bf16_round((1 / (1 + np.exp(-rng.standard_normal(s)))).astype(np.float32))
    return dict(q=f(T, HK, DK), k=f(T, HK, DK), v=f(T, HV, DV), g=sig(T, HV), beta=sig(T, HV))


def _call(d, state, slots, indptr, **kw):
    return go.gdn_state_inplace(d["q"], d["k"], d["v"], d["g"], d["beta"], state,
                                np.asarray(slots, np.int32), np.asarray(indptr, np.int32), **kw)


def test_one_hot_keys_store_and_recall_exactly():
    rng = np.random.default_rng(0)
    T = 6
    d = _rand(rng, T, scale=1.0)
    d["g"][:] = 1.0
    d["beta"][:] = 1.0
    d["k"][:] = 0
    d["q"][:] = 0
    for t in range(T):
        d["k"][t, :, t] = 1.0          # key t is e_t
        d["q"][t, :, max(t - 1, 0)] = 1.0  # ask for what token t-1 stored
    y, st = _call(d, np.zeros((1, HV, DV, DK), np.float32), [0], [0, T], round_output=False)
    for t in range(T):
        np.testing.assert_array_equal(st[0][:, :, t], d["v"][t])  # column t holds v_t
        np.testing.assert_array_equal(y[t], d["v"][max(t - 1, 0)])
    assert np.all(st[0][:, :, T:] == 0)


def test_beta_zero_is_pure_decay_and_g_zero_forgets():
    rng = np.random.default_rng(1)
    T = 5
    d = _rand(rng, T)
    s0 = (0.05 * rng.standard_normal((1, HV, DV, DK))).astype(np.float32)
    d0 = dict(d, beta=np.zeros_like(d["beta"]))
    y, st = _call(d0, s0, [0], [0, T], round_output=False)
    decay = np.prod(d["g"].astype(np.float64), axis=0)  # (HV,)
    np.testing.assert_allclose(st[0], s0[0] * decay[:, None, None], rtol=1e-6)
    # g = 0 at the last token: only that token's outer product survives
    dz = {k: v.copy() for k, v in d.items()}
    dz["g"][T - 1] = 0.0
    y, st = _call(dz, s0, [0], [0, T], round_output=False)
    kk = np.repeat(d["k"][T - 1], HV // HK, axis=0).astype(np.float64)
    want = (d["v"][T - 1].astype(np.float64) * d["beta"][T - 1].astype(np.float64)[:, None])[:, :, None] * kk[:, None, :]
    np.testing.assert_allclose(st[0], want, rtol=1e-6, atol=1e-12)


def test_unit_key_with_beta_one_is_recalled():
    rng = np.random.default_rng(2)
    d = _rand(rng, 3, scale=1.0)
    d["beta"][-1] = 1.0
    kk = d["k"][-1].astype(np.float64)
    kk /= np.linalg.norm(kk, axis=-1, keepdims=True)
    d["k"][-1] = kk  # float64 -> float32, close enough to unit norm
    s0 = rng.standard_normal((2, HV, DV, DK)).astype(np.float32)
    _, st = _call(d, s0, [1], [0, 3], round_output=False)
    k_exp = np.repeat(d["k"][-1].astype(np.float64), HV // HK, axis=0)
    recalled = np.einsum("hvk,hk->hv", st[1].astype(np.float64), k_exp)
    np.testing.assert_allclose(recalled, d["v"][-1], rtol=1e-4, atol=1e-4)
    np.testing.assert_array_equal(st[0], s0[0])  # the other slot is untouched


def test_chunking_and_single_token_mode_are_consistent():
    rng = np.random.default_rng(3)
    T = 9
    d = _rand(rng, T)
    s0 = (0.05 * rng.standard_normal((3, HV, DV, DK))).astype(np.float32)
    y_all, st_all = _call(d, s0, [2], [0, T], round_output=False)
    cut = 4
    head = {k: v[:cut] for k, v in d.items()}
    tail = {k: v[cut:] for k, v in d.items()}
    y1, st1 = _call(head, s0, [2], [0, cut], round_output=False)
    y2, st2 = _call(tail, st1, [2], [0, T - cut], round_output=False)
    np.testing.assert_allclose(np.concatenate([y1, y2]), y_all, rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(st2, st_all, rtol=1e-5, atol=1e-7)
    # token by token in decode mode
    st = s0
    for t in range(T):
        one = {k: v[t:t + 1] for k, v in d.items()}
        yt, st = go.gdn_state_inplace(one["q"], one["k"], one["v"], one["g"], one["beta"], st,
                                      np.array([2], np.int32), None, single_token_mode=True,
                                      round_output=False)
        np.testing.assert_allclose(yt[0], y_all[t], rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(st, st_all, rtol=1e-5, atol=1e-7)


def test_output_is_jointly_linear_in_v_and_initial_state():
    rng = np.random.default_rng(4)
    T = 4
    d = _rand(rng, T)
    s0 = (0.05 * rng.standard_normal((1, HV, DV, DK))).astype(np.float32)
    y1, _ = _call(d, s0, [0], [0, T], round_output=False)
    d2 = dict(d, v=d["v"] * 2)
    y2, _ = _call(d2, s0 * 2, [0], [0, T], round_output=False)
    np.testing.assert_allclose(y2, 2 * y1, rtol=1e-5, atol=1e-8)
