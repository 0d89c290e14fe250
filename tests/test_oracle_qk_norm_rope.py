"""Pins ``oracle/qk_norm_rope_oracle.py`` with facts the mathematics fixes and with library
routines, none of which retypes the oracle's formulas (MLX, whose RMSNorm and RoPE the
reference calls, is not available: bit-level parity with it stays unpinned)."""
import numpy as np
import torch

from oracle import qk_norm_rope_oracle as qo


def _bf16(x):
    return qo.bf16_round(np.asarray(x, dtype=np.float32))


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(5000) * np.exp(rng.uniform(-20, 20, 5000))).astype(np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    np.testing.assert_array_equal(qo.bf16_round(x), want)


def test_rms_norm_against_torch_and_closed_forms():
    rng = np.random.default_rng(1)
    x = _bf16(rng.standard_normal((7, 3, 128)))
    w = _bf16(1 + 0.1 * rng.standard_normal(128))
    got = qo.rms_norm(x, w, 1e-6)
    want = torch.nn.functional.rms_norm(torch.from_numpy(x).double(), (128,),
                                        torch.from_numpy(w).double(), 1e-6).numpy()
    # two bf16 roundings (normalised value, then the product with w): 2^-8 relative each
    np.testing.assert_allclose(got, want, rtol=2 ** -7, atol=1e-30)
    # a constant vector has rms |c|: the result is sign(c) * w up to rounding
    c = np.full((1, 1, 128), -3.0, dtype=np.float32)
    np.testing.assert_allclose(qo.rms_norm(c, w, 0.0)[0, 0], -w, rtol=2 ** -7)
    # scale invariance (power-of-two scale is exact in bf16) when eps is 0
    np.testing.assert_array_equal(qo.rms_norm(x * 4, w, 0.0), qo.rms_norm(x, w, 0.0))


def test_rope_is_a_rotation_with_relative_phase():
    rng = np.random.default_rng(2)
    L, H, D = 9, 2, 128
    x = _bf16(rng.standard_normal((L, H, D)))
    pos = np.array([0, 1, 2, 3, 100, 1000, 5000, 70000, 131071], dtype=np.int32)
    y = qo.rope(x, pos, 1e6)
    # position 0: identity
    np.testing.assert_array_equal(y[0], x[0])
    # every (i, i + D/2) pair keeps its norm (up to the bf16 rounding of the result)
    n_in = np.hypot(x[..., :64], x[..., 64:])
    n_out = np.hypot(y[..., :64], y[..., 64:])
    np.testing.assert_allclose(n_out, n_in, rtol=2 ** -7, atol=2 ** -9)
    # the same thing as complex multiplication by exp(i theta), theta = pos * base^(-i/(D/2))
    i = np.arange(64)
    theta = pos[:, None].astype(np.float64) * (1e6 ** (-i / 64.0))[None, :]
    z = (x[..., :64] + 1j * x[..., 64:]) * np.exp(1j * theta)[:, None, :]
    # float32 angles (as the restated kernel computes them) differ from these float64 ones by up
    # to half an ulp of the angle: 131071 rad -> 4e-3 rad
    np.testing.assert_allclose(y[..., :64], z.real, atol=3e-2, rtol=2 ** -7)
    np.testing.assert_allclose(y[..., 64:], z.imag, atol=3e-2, rtol=2 ** -7)
    np.testing.assert_allclose(y[:6, :, :64], z.real[:6], atol=2e-3, rtol=2 ** -7)


def test_rotated_dot_product_depends_on_the_position_difference_only():
    rng = np.random.default_rng(3)
    q = _bf16(rng.standard_normal((1, 1, 128)))
    k = _bf16(rng.standard_normal((1, 1, 128)))
    dots = []
    for m, n in ((5, 2), (105, 102), (2003, 2000)):
        qr = qo.rope(q, np.array([m], np.int32), 1e4)
        kr = qo.rope(k, np.array([n], np.int32), 1e4)
        dots.append(float((qr.astype(np.float64) * kr.astype(np.float64)).sum()))
    assert abs(dots[0] - dots[1]) < 0.15 and abs(dots[0] - dots[2]) < 0.15, dots


def test_store_part_replaces_exactly_the_addressed_rows():
    rng = np.random.default_rng(4)
    q = _bf16(rng.standard_normal((3, 4, 128)))
    k = _bf16(rng.standard_normal((3, 2, 128)))
    v = _bf16(rng.standard_normal((3, 2, 128)))
    w = np.ones(128, dtype=np.float32)
    kc = _bf16(rng.standard_normal((6, 2, 128)))
    vc = _bf16(rng.standard_normal((6, 2, 128)))
    loc = np.array([4, 0, 3], dtype=np.int32)
    q_out, kc2, vc2 = qo.qk_norm_rope_store(q, k, v, w, w, np.zeros(3, np.int32), loc, kc, vc, 1e-6, 1e6)
    for slot in (1, 2, 5):
        np.testing.assert_array_equal(kc2[slot], kc[slot])
        np.testing.assert_array_equal(vc2[slot], vc[slot])
    np.testing.assert_array_equal(vc2[loc], v)
    # position 0, unit weights: the stored k is the normalised k
    np.testing.assert_array_equal(kc2[loc], qo.rms_norm(k, w, 1e-6))
    np.testing.assert_array_equal(q_out, qo.rms_norm(q, w, 1e-6))
