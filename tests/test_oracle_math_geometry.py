"""Pins the oracle's elementary functions and ray/ellipsoid geometry against libm and closed forms.

None of these tests retypes the oracle's formulas: the references are numpy's float64 routines,
analytic special cases (identity rotation, ray through the centre) and invariances (rigid motion).
"""
import numpy as np
import pytest

from helpers import ulp_diff


def test_exp_matches_libm_within_two_ulp(oracle_mod):
    x = np.concatenate([np.linspace(-86.9, 87.9, 400001), np.linspace(-1, 1, 100001)]).astype(np.float32)
    got = oracle_mod.math("exp", x)
    ref = np.exp(x.astype(np.float64)).astype(np.float32)
    assert ulp_diff(got, ref).max() <= 2


def test_exp_range_rules(oracle_mod):
    x = np.array([-87.5, -1000.0, 88.5, 1e9, 0.0, -0.0], np.float32)
    got = oracle_mod.math("exp", x)
    assert got[0] == 0 and got[1] == 0 and np.isinf(got[2]) and np.isinf(got[3]) and got[4] == 1 and got[5] == 1
    assert np.isnan(oracle_mod.math("exp", np.array([np.nan], np.float32))[0])


def test_sincos_matches_libm_on_the_phase_range(oracle_mod):
    # phases reach |x| * 32 pi * 0.6 ~ 61 rad for unit directions; test well past that
    x = np.linspace(-400.0, 400.0, 1600001).astype(np.float32)
    s, c = oracle_mod.math("sincos", x)
    xd = x.astype(np.float64)
    assert np.abs(s - np.sin(xd)).max() < 2.5e-7
    assert np.abs(c - np.cos(xd)).max() < 2.5e-7
    # a wrong quadrant, a swapped pair or a sign slip breaks the Pythagorean identity or these anchors
    assert np.abs(s.astype(np.float64) ** 2 + c.astype(np.float64) ** 2 - 1).max() < 5e-7
    s0, c0 = oracle_mod.math("sincos", np.array([0.0, np.pi / 2, np.pi, -np.pi / 2], np.float32))
    np.testing.assert_allclose(s0, [0, 1, 0, -1], atol=1e-6)
    np.testing.assert_allclose(c0, [1, 0, -1, 0], atol=1e-6)


def test_sincos_out_of_range_is_nan(oracle_mod):
    s, c = oracle_mod.math("sincos", np.array([1e6, np.inf, np.nan], np.float32))
    assert np.isnan(s).all() and np.isnan(c).all()


def test_log1p_softplus_sigmoid_match_libm(oracle_mod):
    x = np.exp(np.linspace(-25, 21, 200001)).astype(np.float32)
    got = oracle_mod.math("log1p", x)
    ref = np.log1p(x.astype(np.float64))
    assert (np.abs(got - ref) / ref).max() < 3e-7
    z = np.linspace(-30, 30, 120001).astype(np.float32)
    sp = oracle_mod.math("softplus", z)
    ref_sp = np.where(z > 20, z, np.log1p(np.exp(z.astype(np.float64))))
    assert (np.abs(sp - ref_sp) / ref_sp).max() < 4e-7
    sg = oracle_mod.math("sigmoid", z)
    assert np.abs(sg - 1 / (1 + np.exp(-z.astype(np.float64)))).max() < 2e-7


def test_softplus_cutoffs(oracle_mod):
    # np_tile_kernels.cu:79-83: identity above 20, bare exp below -20
    sp = oracle_mod.math("softplus", np.array([20.5, 35.0, -20.5], np.float32))
    assert sp[0] == np.float32(20.5) and sp[1] == np.float32(35.0)
    assert sp[2] == oracle_mod.math("exp", np.array([-20.5], np.float32))[0]


def test_bf16_and_f16_rounding(oracle_mod):
    import torch
    x = np.random.default_rng(1).standard_normal(100000).astype(np.float32) * 3
    x[:4] = [1.0, 1.00390625, 1.01171875, 65520.0]  # exact, tie to even (down), tie to even (up), f16 overflow
    b = oracle_mod.math("round_bf16", x)
    h = oracle_mod.math("round_f16", x)
    np.testing.assert_array_equal(b, torch.from_numpy(x).bfloat16().float().numpy())
    np.testing.assert_array_equal(h, torch.from_numpy(x).half().float().numpy())


# ---------------------------------------------------------------------------------------------
def _rand_unit_quat(rng):
    q = rng.standard_normal(4)
    return (q / np.linalg.norm(q)).astype(np.float32)


def _rotmat(q):
    w, x, y, z = q.astype(np.float64)
    return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)],
                     [2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)],
                     [2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)]])


def test_hit_identity_rotation_isotropic_closed_form(oracle_mod):
    # identity quaternion + one scale s: t = v.d, decay = exp(-|v - t d|^2 / (2 s^2))
    rng = np.random.default_rng(0)
    for _ in range(200):
        o = rng.uniform(-1, 1, 3).astype(np.float32)
        d = rng.standard_normal(3)
        d = (d / np.linalg.norm(d)).astype(np.float32)
        c = (o + d * rng.uniform(0.5, 3) + rng.standard_normal(3) * 0.05).astype(np.float32)
        ls = np.float32(rng.uniform(-3.5, -1.5))
        hit, h = oracle_mod.hit(o, d, c, [ls, ls, ls], [1, 0, 0, 0], 1e-3)
        v = c.astype(np.float64) - o
        t = v @ d.astype(np.float64)
        perp = v - t * d
        decay = np.exp(-(perp @ perp) / (2 * np.exp(2 * float(ls))))
        assert abs(h["t"] - t) < 1e-5 * max(1, abs(t))
        assert abs(h["decay"] - decay) < 2e-5 + 1e-3 * decay  # the f32 perpendicular offset carries ~1e-7 absolute error
        assert hit == (h["decay"] > np.float32(1e-3))
        np.testing.assert_allclose(h["d"], perp, atol=2e-6)
        np.testing.assert_allclose(h["q"], perp, atol=2e-6)  # local frame == world frame


def test_hit_through_the_centre(oracle_mod):
    # the reference tests' scene (tests/test_cuda_renderer.py:111-141): t = depth, d = q = 0, decay = 1
    hit, h = oracle_mod.hit([0, 0, 0], [0, 0, 1], [0, 0, 1], [0, 0, 0], [1, 0, 0, 0], 1e-3)
    assert hit and h["t"] == 1 and h["decay"] == 1 and not h["d"].any() and not h["q"].any()


def test_hit_anisotropic_matches_float64_mahalanobis(oracle_mod):
    # general case against a float64 evaluation with the rotation MATRIX (not the quaternion product)
    rng = np.random.default_rng(3)
    for _ in range(300):
        q = _rand_unit_quat(rng)
        R = _rotmat(q)
        ls = rng.normal(-2.5, 0.5, 3).astype(np.float32)
        o = rng.uniform(-1, 1, 3).astype(np.float32)
        d = rng.standard_normal(3)
        d = (d / np.linalg.norm(d)).astype(np.float32)
        c = (o + d * rng.uniform(0.5, 3) + rng.standard_normal(3) * 0.1).astype(np.float32)
        hit, h = oracle_mod.hit(o, d, c, ls, q, 1e-3)
        M = R @ np.diag(np.exp(-2 * ls.astype(np.float64))) @ R.T
        v = c.astype(np.float64) - o
        dd = d.astype(np.float64)
        t = (dd @ M @ v) / (dd @ M @ dd)
        off = v - t * dd
        decay = np.exp(-0.5 * off @ M @ off)
        assert abs(h["t"] - t) < 2e-5 * max(1.0, abs(t))
        assert abs(h["decay"] - decay) < 1e-4
        np.testing.assert_allclose(h["q"], R.T @ off, atol=5e-6)
        if abs(decay - 1e-3) > 1e-4:
            assert hit == (t > 0 and decay > 1e-3)


def test_hit_is_invariant_under_a_common_rigid_motion(oracle_mod):
    rng = np.random.default_rng(5)
    q = _rand_unit_quat(rng)
    ls = np.array([-2.0, -2.6, -3.1], np.float32)
    o = np.array([0.1, -0.3, 0.2], np.float32)
    d = np.array([0.2, 0.1, 0.97], np.float32)
    d /= np.linalg.norm(d)
    c = np.array([0.35, -0.1, 1.2], np.float32)
    _, h0 = oracle_mod.hit(o, d, c, ls, q, 1e-4)
    g = _rand_unit_quat(rng)
    G = _rotmat(g)
    shift = np.array([0.5, -1.0, 2.0])
    # compose rotations: q' = g * q
    w1, x1, y1, z1 = g.astype(np.float64)
    w2, x2, y2, z2 = q.astype(np.float64)
    qq = np.array([w1 * w2 - x1 * x2 - y1 * y2 - z1 * z2, w1 * x2 + x1 * w2 + y1 * z2 - z1 * y2,
                   w1 * y2 - x1 * z2 + y1 * w2 + z1 * x2, w1 * z2 + x1 * y2 - y1 * x2 + z1 * w2], np.float32)
    _, h1 = oracle_mod.hit((G @ o + shift).astype(np.float32), (G @ d).astype(np.float32),
                           (G @ c + shift).astype(np.float32), ls, qq, 1e-4)
    assert abs(h0["t"] - h1["t"]) < 1e-5
    assert abs(h0["decay"] - h1["decay"]) < 1e-4
    np.testing.assert_allclose(h0["q"], h1["q"], atol=1e-5)  # the local offset does not see the motion


def test_hit_rejects_behind_and_degenerate(oracle_mod):
    hit, _ = oracle_mod.hit([0, 0, 0], [0, 0, 1], [0, 0, -1], [0, 0, 0], [1, 0, 0, 0], 1e-3)
    assert not hit  # t <= 0
    hit, _ = oracle_mod.hit([0, 0, 0], [0, 0, 0], [0, 0, 1], [0, 0, 0], [1, 0, 0, 0], 1e-3)
    assert not hit  # denom <= 1e-20


def test_sort_keys(oracle_mod):
    rng = np.random.default_rng(7)
    q = _rand_unit_quat(rng)
    ls = np.array([-2.0, -2.5, -3.0], np.float32)
    o = np.zeros(3, np.float32)
    d = np.array([0, 0, 1], np.float32)
    c = np.array([0.1, 0.05, 2.0], np.float32)
    # family 1 equals the hit's t for the same ray; family 2 is the plain projection
    _, h = oracle_mod.hit(o, d, c, ls, q, 1e-9)
    assert oracle_mod.key(1, o, d, c, ls, q) == h["t"]
    assert abs(oracle_mod.key(2, o, d, c, ls, q) - 2.0) < 1e-6
    behind = np.array([0.0, 0.0, -2.0], np.float32)
    assert oracle_mod.key(1, o, d, behind, ls, q) == np.float32(1e30)
    assert oracle_mod.key(2, o, d, behind, ls, q) == np.float32(1e30)


def test_gates_closed_form(oracle_mod):
    # at the centre every gate is 1/4; in general a softmax of tau * (+-ux +-uy +-uz), u clamped to +-1
    np.testing.assert_allclose(oracle_mod.gates([0, 0, 0], [-2, -2, -2], 1.5, 2.0), [0.25] * 4, atol=1e-7)
    rng = np.random.default_rng(11)
    for _ in range(100):
        ql = rng.standard_normal(3) * 0.2
        ls = rng.normal(-2.5, 0.4, 3)
        beta, tau = rng.uniform(0.5, 2.5), rng.uniform(0.5, 3.0)
        g = oracle_mod.gates(ql.astype(np.float32), ls.astype(np.float32), beta, tau)
        u = np.clip(ql.astype(np.float32).astype(np.float64) / (beta * np.exp(ls.astype(np.float32).astype(np.float64)) + 1e-6), -1, 1)
        logits = tau * np.array([u[0] + u[1] + u[2], u[0] - u[1] - u[2], -u[0] + u[1] - u[2], -u[0] - u[1] + u[2]])
        e = np.exp(logits - logits.max())
        np.testing.assert_allclose(g, e / e.sum(), atol=3e-6)
        assert abs(g.sum() - 1) < 1e-6
    far = oracle_mod.gates([10, 10, 10], [-2, -2, -2], 1.5, 2.0)   # clamps: u = (1,1,1)
    e = np.exp(2.0 * np.array([3, -1, -1, -1.0]) - 6.0)
    np.testing.assert_allclose(far, e / e.sum(), atol=1e-6)
