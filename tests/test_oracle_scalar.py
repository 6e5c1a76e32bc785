"""Pins the scalar pieces of the CPU oracle against libm / closed forms (CPU only)."""
import math

import numpy as np
import pytest

from tests import ref_model


def test_softplus_matches_libm(oracle):
    # _softplus (RenderForward.cu:154-159): log(1+exp(x)) below the threshold 20, identity above
    # the sum 1 + exp(x) is rounded to float before the logarithm, as logf(1.f + expf(x)) does
    for x in np.linspace(-30, 19.99, 400):
        e = np.float32(math.exp(float(np.float32(x))))
        want = math.log(float(np.float32(1.0) + e))
        got = oracle.softplus(np.float32(x))
        assert got == pytest.approx(want, rel=3e-7, abs=1e-37)
    # and it is softplus to float accuracy where 1 + exp(x) is well conditioned
    for x in np.linspace(-5, 19.99, 100):
        assert oracle.softplus(np.float32(x)) == pytest.approx(math.log1p(math.exp(float(np.float32(x)))), rel=1e-5)
    assert oracle.softplus(20.5) == 20.5
    assert oracle.softplus(100.0) == 100.0
    # continuity at the threshold
    assert oracle.softplus(20.0) == pytest.approx(20.0, rel=1e-6)


def test_softplus_backward_is_sigmoid(oracle):
    # _softplus_backwards (RenderBackward.cu:71-83)
    for x in np.linspace(-20, 19.9, 200):
        xf = float(np.float32(x))
        assert oracle.softplus_backward(xf) == pytest.approx(1.0 / (1.0 + math.exp(-xf)), rel=3e-7)
    assert oracle.softplus_backward(25.0) == 1.0
    # derivative of softplus by central differences in f64
    for x in (-3.0, -0.5, 0.0, 1.25, 7.0):
        h = 1e-6
        fd = (math.log1p(math.exp(x + h)) - math.log1p(math.exp(x - h))) / (2 * h)
        assert oracle.softplus_backward(x) == pytest.approx(fd, rel=1e-5)


def test_log2_floor_ceil_exact(oracle):
    for k in range(0, 12):
        p = float(2 ** k)
        assert oracle.log2_floor_ceil(p) == (k, k)
        up = float(np.nextafter(np.float32(p), np.float32(1e9)))
        dn = float(np.nextafter(np.float32(p), np.float32(0)))
        assert oracle.log2_floor_ceil(up) == (k, k + 1)
        assert oracle.log2_floor_ceil(dn) == (k - 1, k)
    rng = np.random.default_rng(0)
    for s in np.exp(rng.uniform(0.001, 8, 500)).astype(np.float32):
        lo, hi = oracle.log2_floor_ceil(float(s))
        assert lo == math.floor(math.log2(float(s))) and hi == math.ceil(math.log2(float(s)))


@pytest.mark.parametrize("L", [1, 2, 4, 8])
def test_layer_factor_cases(oracle, L):
    # compute_point_size_fac (PointBlending.h:81-149)
    # small points: 0.75 exp(s-1) + 0.25, gradient constant-slope 0.27591 s
    for s in (0.01, 0.5, 1.0):
        f, g = oracle.layer_factor(s, 0, L)
        assert f == pytest.approx(0.75 * math.exp(s - 1) + 0.25, rel=1e-6)
        assert g == pytest.approx(0.27591 * s, rel=1e-6)
    if L == 1:
        # every size falls in the "small point" branch when there is one layer
        f, g = oracle.layer_factor(5.0, 0, L)
        assert f == pytest.approx(0.75 * math.exp(4.0) + 0.25, rel=1e-6)
        return
    # interpolation: factors of the two adjacent layers sum to 1, slopes are +-1/(2^hi-2^lo)
    for s in (1.5, 3.0, 5.0, 11.0, 100.0):
        lo, hi = math.floor(math.log2(s)), math.ceil(math.log2(s))
        if hi > L - 1:
            continue
        f_lo, g_lo = oracle.layer_factor(s, lo, L)
        f_hi, g_hi = oracle.layer_factor(s, hi, L)
        if lo == L - 1:
            continue
        assert f_lo + f_hi == pytest.approx(1.0, abs=1e-6)
        assert f_hi == pytest.approx((s - 2 ** lo) / (2 ** hi - 2 ** lo), rel=1e-6)
        assert g_hi == pytest.approx(1.0 / (2 ** hi - 2 ** lo), rel=1e-6)
        assert g_lo == pytest.approx(-1.0 / (2 ** hi - 2 ** lo), rel=1e-6)
        # layers below floor(log2 s) render the point at full weight
        for below in range(0, lo):
            assert oracle.layer_factor(s, below, L) == (1.0, 0.0)
    # exact power of two: lo == hi -> factor 1, gradient 1
    assert oracle.layer_factor(2.0, 1, L) == (1.0, 1.0)
    # beyond the coarsest layer: factor 1 (gradient 1 as written)
    big = float(2 ** (L - 1)) * 1.7
    assert oracle.layer_factor(big, L - 1, L) == (1.0, 1.0)


def test_layer_factor_agrees_with_restatement(oracle):
    rng = np.random.default_rng(3)
    s = np.exp(rng.uniform(-3, 6, 2000)).astype(np.float32)
    for L in (1, 3, 8):
        if L == 1:
            s = np.minimum(s, np.float32(40.0))  # exp(s-1) overflows float beyond ~89
        layers = rng.integers(0, L, s.shape[0])
        want = ref_model.layer_factor_np(s, layers, L)
        got = np.array([oracle.layer_factor(float(a), int(l), L)[0] for a, l in zip(s, layers)])
        np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-7)
