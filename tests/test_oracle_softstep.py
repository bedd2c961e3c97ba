"""Pins the CPU oracle of the soft-step family (oracle/tmq_oracle.c, oracle/torch_path.py).

The reference holds no tests or golden vectors for this path, so the oracle is pinned by what the
mathematics fixes: exact rational values of the closed forms (derived by hand from
y = sig(d*frac - d/2)/(2 sig(d/2)) + 1/2 + floor(w), sig(x) = x(x^2+27)/(27+9x^2)), fp64 finite
differences for the two derivative formulas, fixed points and symmetries, and bit-equality of two
independently written restatements (C scalar loop vs chain of torch ops).
"""
from fractions import Fraction as Fr

import numpy as np
import pytest
import torch

from oracle import torch_path as tp

HARDNESS = [0.1, 1.1684210526315788, 3.0004, 4.72, 6.0]


# ---- exact rational model, written independently of the fp32 code (piecewise cubic over cubic) ----
def r_sig(x):
    x = max(Fr(-3), min(Fr(3), x))
    return x * (x * x + 27) / (27 + 9 * x * x)


def r_S(w, d):
    import math
    fw = math.floor(w)
    return r_sig(d * (w - fw) - d / 2) / (2 * r_sig(d / 2)) + Fr(1, 2) + fw


# Hand-derived known answers (value, slope) -- see the module docstring.
KAT = [
    # d, w, S(w), S'(w)
    (6, Fr(1, 4), Fr(1, 28), Fr(27, 49)),
    (6, Fr(9, 10), Fr(729, 730), Fr(243, 5329)),
    (6, Fr(1, 2), Fr(1, 2), Fr(3)),
    (6, Fr(0), Fr(0), Fr(0)),
    (6, Fr(1), Fr(1), Fr(0)),
    (6, Fr(-1), Fr(-1), Fr(0)),
    (2, Fr(1, 4), Fr(73, 364), Fr(175, 169)),
    (2, Fr(0), Fr(0), Fr(4, 7)),
    (2, Fr(1, 2), Fr(1, 2), Fr(9, 7)),
    (2, Fr(9, 10), Fr(5949, 6370), None),
    (8, Fr(1, 4), Fr(1, 126), Fr(100, 441)),
    (8, Fr(9, 10), Fr(1), Fr(0)),
]


def test_rational_model_matches_hand_answers():
    for d, w, s, _ in KAT:
        assert r_S(w, Fr(d)) == s, (d, w)


def test_oracle_matches_hand_answers(oracle):
    for d, w, s, ds in KAT:
        wv = np.array([float(w)], dtype=np.float32)
        y = oracle.softstep_fwd(wv, float(d))[0]
        assert abs(float(y) - float(s)) <= 3e-7, (d, w, y, float(s))
        if ds is not None:
            g = oracle.softstep_bwd(wv, np.ones(1, np.float32), float(d))[0]
            assert abs(float(g) - float(ds)) <= 2e-6 * max(1.0, float(ds)), (d, w, g, float(ds))


def test_oracle_scalars(oracle):
    d32, h32, c32 = oracle.consts(5.0)
    assert d32 == np.float32(5.0) and h32 == np.float32(2.5)
    assert c32 == np.float32(665.0 / 333.0)          # 2*sig(2.5) = 665/333
    _, _, c = oracle.consts(0.1)
    assert abs(float(c) - 0.0999259876) < 1e-9        # 2*sig(0.05)
    _, _, c6 = oracle.consts(6.0)
    assert c6 == np.float32(2.0)                      # 2*sig(3) = 2


def test_qloss_known_values(oracle):
    # integrand at sharpness 5, strength 1: q(w) = 5*dsig(5 frac - 2.5)/(665/333)
    cases = {0.0: 0.024588498, 1.0: 0.024588498, 0.25: 0.739261834, -0.25: 0.739261834, -0.75: 0.739261834,
             0.5: 2.503759398, 0.9: 0.141936474}
    for w, q in cases.items():
        got = oracle.deriv_fwd(np.array([w], np.float32), 5.0, 1.0)[0]
        assert abs(float(got) - q) < 5e-7, (w, got, q)
    grads = {0.25: 6.535663507, -0.25: -6.535663507, 0.5: 0.0, 0.9: -1.946557355}
    for w, g in grads.items():
        got = oracle.deriv_bwd(np.array([w], np.float32), np.ones(1, np.float32), 5.0, 1.0)[0]
        assert abs(float(got) - g) < 5e-6, (w, got, g)


def _f64_S(w, d):
    fw = np.floor(w)
    x = np.clip(d * (w - fw) - d / 2, -3, 3)
    sig = x * (x * x + 27) / (27 + 9 * x * x)
    xs = min(3.0, d / 2)
    c = 2 * (xs * (xs * xs + 27) / (27 + 9 * xs * xs))
    return sig / c + 0.5 + fw


@pytest.mark.parametrize("d", HARDNESS + [8.0, 20.0])
def test_derivatives_by_finite_differences(oracle, d):
    rng = np.random.default_rng(7)
    w = rng.uniform(-0.98, 0.98, 4000)
    w = w[np.abs(w - np.round(w * 2) / 2) > 1e-3]          # stay off the kinks of floor/clamp
    h = 1e-6
    fd1 = (_f64_S(w + h, d) - _f64_S(w - h, d)) / (2 * h)
    s1 = oracle.softstep_bwd(w.astype(np.float32), np.ones(w.size, np.float32), d).astype(np.float64)
    # slope of fp32(w) vs slope at w: compare at the rounded abscissa
    w32 = w.astype(np.float32).astype(np.float64)
    fd1 = (_f64_S(w32 + h, d) - _f64_S(w32 - h, d)) / (2 * h)
    assert np.max(np.abs(fd1 - s1)) < 2e-5 * max(1.0, d)
    # second derivative: Q(w) = strength*S'(w); Q' by central differences of the fp64 slope
    def slope(v):
        return (_f64_S(v + h, d) - _f64_S(v - h, d)) / (2 * h)
    h2 = 1e-4
    fd2 = (slope(w32 + h2) - slope(w32 - h2)) / (2 * h2)
    keep = np.abs(d * (w32 - np.floor(w32)) - d / 2) < 2.99   # away from the clamp knee
    s2 = oracle.deriv_bwd(w.astype(np.float32), np.ones(w.size, np.float32), d, 1.0).astype(np.float64)
    assert np.max(np.abs(fd2[keep] - s2[keep])) < 2e-3 * max(1.0, d * d)


@pytest.mark.parametrize("d", HARDNESS)
def test_fixed_points_and_symmetry(oracle, d):
    k = np.array([-2, -1, 0, 1, 2], np.float32)
    assert np.max(np.abs(oracle.softstep_fwd(k, d) - k)) <= 1.2e-7            # S(k) = k up to one rounding
    if d == 6.0:
        assert np.array_equal(oracle.softstep_fwd(k, d), k)                   # exact: sig(-3)/2 = -1/2
    assert np.array_equal(oracle.softstep_fwd(k + 0.5, d), k + np.float32(0.5))  # S(k+1/2) = k+1/2 exactly
    f = np.linspace(0.01, 0.49, 97).astype(np.float32)
    a = oracle.softstep_fwd(f, d).astype(np.float64)
    b = oracle.softstep_fwd((1 - f.astype(np.float64)).astype(np.float32), d).astype(np.float64)
    assert np.max(np.abs(a + b - 1.0)) < 1e-6                                  # S(f) + S(1-f) = 1
    w = np.sort(np.random.default_rng(3).uniform(-1.02, 1.02, 20000)).astype(np.float32)
    y = oracle.softstep_fwd(w, d)
    assert np.all(np.diff(y.astype(np.float64)) >= -3e-7)                      # monotone up to rounding
    assert np.all(oracle.softstep_bwd(w, np.ones_like(w), d) >= 0)


def test_small_hardness_is_identity_like(oracle):
    w = np.linspace(-0.99, 0.99, 199).astype(np.float32)
    assert np.max(np.abs(oracle.softstep_fwd(w, 0.05) - w)) < 2e-4


def _special_values():
    v = [0.0, -0.0, 0.5, -0.5, 1.0, -1.0, 1.02, -1.02, 0.25, 0.9, 1e-40, -1e-40, 1e-8, -1e-8, 0.99999994,
         -0.99999994, 1.5, -1.5, 2.0, -2.0, 3.7, np.nan, np.inf, -np.inf, 123456.0, 0.49999997, 0.50000006]
    return np.array(v, dtype=np.float32)


def _bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def _same_bits(a, b):
    a = np.asarray(a, np.float32).reshape(-1)
    b = np.asarray(b, np.float32).reshape(-1)
    nan = np.isnan(a) & np.isnan(b)
    return np.array_equal(_bits(a)[~nan], _bits(b)[~nan]) and np.array_equal(np.isnan(a), np.isnan(b))


@pytest.mark.parametrize("d", HARDNESS + [0.05, 7.3, 20.0])
def test_c_oracle_is_bit_identical_to_torch_chain(oracle, d):
    rng = np.random.default_rng(11)
    w = np.concatenate([rng.uniform(-1.02, 1.02, 50000).astype(np.float32), _special_values(),
                        (rng.integers(-1, 2, 5000) + rng.uniform(-0.02, 0.02, 5000)).astype(np.float32)])
    g = rng.standard_normal(w.size).astype(np.float32)
    tw, tg = torch.from_numpy(w), torch.from_numpy(g)
    assert _same_bits(oracle.softstep_fwd(w, d), tp.softstep_fwd(tw, d).numpy())
    assert _same_bits(oracle.softstep_bwd(w, g, d, 1.0), tp.softstep_bwd(tw, d, 1.0, tg).numpy())
    assert _same_bits(oracle.softstep_bwd(w, g, d, 0.37), tp.softstep_bwd(tw, d, 0.37, tg).numpy())
    assert _same_bits(oracle.deriv_fwd(w, d, 5e-4), tp.deriv_fwd(tw, d, 5e-4).numpy())
    assert _same_bits(oracle.deriv_bwd(w, g, d, 5e-4), tp.deriv_bwd(tw, d, 5e-4, tg).numpy())
    assert _same_bits(oracle.softstep_map(w, d), tp.softstep_map(tw, d).numpy())
    assert _same_bits(oracle.softstep_dmap(w, d), tp.softstep_dmap(tw, d).numpy())
    assert _same_bits(oracle.ternarize(w, d), tp.ternarize(tw, d).numpy())
    assert _same_bits(oracle.clamp(w, -1.0, 1.0), tp.clamp(tw, -1.0, 1.0).numpy())


def test_fused_oracle_is_the_composition(oracle):
    rng = np.random.default_rng(5)
    w = rng.uniform(-1.02, 1.02, 30000).astype(np.float32)
    g = rng.standard_normal(w.size).astype(np.float32)
    d, sharp, p, gl = 3.0004, 5.0, 5e-4, np.float32(1.0 / w.size)
    y, dw, wc, qsum = oracle.fused(w, g, d, sharp, p, float(gl), -1.0, 1.0)
    ty, tdw, twc, tloss = tp.fused_step(torch.from_numpy(w), torch.from_numpy(g), d, sharp, p, float(gl), -1.0, 1.0)
    assert _same_bits(y, ty.numpy()) and _same_bits(dw, tdw.numpy()) and _same_bits(wc, twc.numpy())
    assert abs(qsum / w.size - float(tloss)) < 1e-6 * abs(float(tloss))
    assert abs(qsum - oracle.sum64(oracle.deriv_fwd(w, sharp, p))) == 0.0


@pytest.mark.parametrize("d", HARDNESS + [20.0])
def test_ternarize_equals_round_half_even_on_clamp_range(oracle, d):
    rng = np.random.default_rng(13)
    w = np.concatenate([rng.uniform(-1, 1, 200000).astype(np.float32),
                        np.array([0.5, -0.5, 0.49999997, 0.50000006, -0.49999997, -0.50000006, 1.0, -1.0, 0.0],
                                 np.float32)])
    t = oracle.ternarize(w, d)
    assert set(np.unique(t).tolist()) <= {-1.0, 0.0, 1.0}
    assert np.array_equal(t, np.rint(w))
    assert np.array_equal(oracle.ternarize(t, d), t)            # idempotent


def test_clamp_semantics(oracle):
    w = np.array([-3, -1.0000001, -1, -0.0, 0.0, 1, 1.0000001, 3, np.nan, np.inf, -np.inf], np.float32)
    c = oracle.clamp(w, -1.0, 1.0)
    assert np.array_equal(c[:8], np.array([-1, -1, -1, -0.0, 0.0, 1, 1, 1], np.float32))
    assert np.signbit(c[3]) and not np.signbit(c[4])
    assert np.isnan(c[8]) and c[9] == 1 and c[10] == -1
    assert np.array_equal(oracle.clamp(c[:8], -1.0, 1.0), c[:8])     # idempotent
    assert np.array_equal(oracle.clamp(w[:8], -1.25, 1.25)[[0, 1, 6, 7]], np.array([-1.25, -1.0000001, 1.0000001, 1.25],
                                                                                 np.float32))
