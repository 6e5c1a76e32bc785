"""Pins the oracle's Adam (MyAdam.cu:41-88) and pose update (PointRenderer.cu:1428-1447). CPU only."""
import numpy as np
import pytest
import torch
from scipy.linalg import expm
from scipy.spatial.transform import Rotation

from trips_amd import abi


def _tensor(n, rng, dtype=np.float32, **hyper):
    t = dict(w=rng.normal(0, 1, n).astype(dtype), g=rng.normal(0, 1, n).astype(dtype),
             m=np.zeros(n, np.float32), v=np.zeros(n, np.float32), steps=np.zeros(n, np.int64), n=n,
             dtype=abi.TRIPS_DTYPE_F64 if dtype == np.float64 else abi.TRIPS_DTYPE_F32)
    t.update(hyper)
    return t


def test_adam_matches_hand_derived_three_steps(oracle):
    # one element, gradients 1, -2, 0.5; lr=0.1, beta=(0.9, 0.999), eps=1e-8; bias-corrected step
    # lr_t = lr*sqrt(1-b2^t)/(1-b1^t); w -= lr_t * m / (sqrt(v) + eps)     (MyAdam.cu:63-79)
    t = dict(w=np.array([1.0], np.float32), g=np.array([0.0], np.float32), m=np.zeros(1, np.float32),
             v=np.zeros(1, np.float32), steps=np.zeros(1, np.int64), n=1, lr=0.1)
    # the kernel's constants are floats: 1 - 0.999f is 0.00099998713, not 0.001
    b1, b2, lr = float(np.float32(0.9)), float(np.float32(0.999)), float(np.float32(0.1))
    omb1, omb2 = float(np.float32(1) - np.float32(0.9)), float(np.float32(1) - np.float32(0.999))
    w, m, v = 1.0, 0.0, 0.0
    for step, g in enumerate([1.0, -2.0, 0.5], start=1):
        t["g"][0] = g
        oracle.adam_step([t])
        m = b1 * m + omb1 * g
        v = b2 * v + omb2 * g * g
        lr_t = lr * np.sqrt(1 - b2 ** step) / (1 - b1 ** step)
        w = w - lr_t / (np.sqrt(v) + 1e-8) * m
        assert t["w"][0] == pytest.approx(w, rel=2e-6)
        assert t["m"][0] == pytest.approx(m, rel=2e-6)
        assert t["v"][0] == pytest.approx(v, rel=2e-6)
        assert t["steps"][0] == step


def test_adam_equals_torch_adam_at_eps_zero(oracle):
    # with eps = 0 the two placements of the bias correction coincide: compare 5 steps with torch.optim.Adam
    rng = np.random.default_rng(0)
    n = 257
    t = _tensor(n, rng, lr=1e-2, eps=0.0)
    p = torch.tensor(t["w"].copy(), requires_grad=True)
    opt = torch.optim.Adam([p], lr=1e-2, betas=(0.9, 0.999), eps=0.0)
    for _ in range(5):
        g = rng.normal(0, 1, n).astype(np.float32)
        g[g == 0] = 1.0
        t["g"][:] = g
        p.grad = torch.tensor(g)
        opt.step()
        oracle.adam_step([t])
        np.testing.assert_allclose(t["w"], p.detach().numpy(), rtol=2e-5, atol=2e-6)


def test_adam_skips_zero_gradient_and_counts_steps_per_element(oracle):
    # gradient == 0 means "not seen": nothing changes for that element, not even its step counter (MyAdam.cu:57-61)
    t = dict(w=np.array([1.0, 2.0, 3.0], np.float32), g=np.array([0.5, 0.0, -0.5], np.float32),
             m=np.zeros(3, np.float32), v=np.zeros(3, np.float32), steps=np.zeros(3, np.int64), n=3, lr=0.1)
    oracle.adam_step([t])
    assert t["w"][1] == 2.0 and t["m"][1] == 0 and t["v"][1] == 0 and t["steps"][1] == 0
    assert list(t["steps"]) == [1, 0, 1]
    # first step of an element moves it by lr * sign(g) (bias correction cancels), whenever that step happens
    assert t["w"][0] == pytest.approx(1.0 - 0.1, rel=1e-5) and t["w"][2] == pytest.approx(3.0 + 0.1, rel=1e-5)
    t["g"][:] = [0.0, 0.25, 0.0]
    oracle.adam_step([t])
    assert list(t["steps"]) == [1, 1, 1]
    assert t["w"][1] == pytest.approx(2.0 - 0.1, rel=1e-5)


def test_adam_weight_decay_clipping_bounds_and_f64(oracle):
    rng = np.random.default_rng(4)
    n = 64
    base = _tensor(n, rng, lr=0.05)
    ref = {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in base.items()}
    t = {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in base.items()}
    t.update(relative_weight_decay=0.1, absolute_weight_decay=0.02, weight_clipping_magnitude=0.9)
    oracle.adam_step([t])
    oracle.adam_step([ref])
    lr_t = 0.05 * np.sqrt(1 - 0.999) / (1 - 0.9)
    w0 = base["w"].astype(np.float64)
    step = ref["w"].astype(np.float64) - w0  # plain adam displacement
    want = (1 - 0.1 * lr_t) * w0 - np.copysign(0.02 * lr_t, w0) + step
    want = np.clip(want, -0.9, 0.9)
    np.testing.assert_allclose(t["w"], want, rtol=1e-5, atol=1e-6)
    # AdaBound-style clamp of the effective learning rate
    t2 = {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in base.items()}
    t2.update(lower_lr_bound=0.0, upper_lr_bound=0.01)
    oracle.adam_step([t2])
    m = 0.1 * base["g"].astype(np.float64)
    np.testing.assert_allclose(t2["w"], w0 - np.minimum(lr_t / (np.sqrt(0.001 * base["g"].astype(np.float64) ** 2) + 1e-8), 0.01) * m,
                               rtol=1e-5, atol=1e-6)
    # f64 master weights (pose tangents): arithmetic in float, storage in double
    t64 = _tensor(n, rng, dtype=np.float64, lr=0.05)
    t32 = {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in t64.items()}
    t32["w"] = t64["w"].astype(np.float32)
    t32["g"] = t64["g"].astype(np.float32)
    t32["dtype"] = abi.TRIPS_DTYPE_F32
    oracle.adam_step([t64, t32])
    np.testing.assert_array_equal(t64["w"].astype(np.float32), t32["w"])
    assert t64["w"].dtype == np.float64


def test_apply_tangent_matches_matrix_exponential(oracle):
    rng = np.random.default_rng(9)
    n = 6
    poses = np.zeros((n, 8))
    tang = rng.normal(0, 0.3, (n, 6))
    tang[0] = 0  # identity update
    tang[1, 3:] = 1e-13  # small-angle branch
    mats = []
    for i in range(n):
        q = rng.normal(0, 1, 4)
        q /= np.linalg.norm(q)
        poses[i, :4] = q
        poses[i, 4:7] = rng.normal(0, 1, 3)
        T = np.eye(4)
        T[:3, :3] = Rotation.from_quat(q).as_matrix()
        T[:3, 3] = poses[i, 4:7]
        ups, om = tang[i, :3], tang[i, 3:] * 0.1  # rotation part scaled by 0.1 (PointRenderer.cu:1437)
        X = np.zeros((4, 4))
        X[:3, :3] = [[0, -om[2], om[1]], [om[2], 0, -om[0]], [-om[1], om[0], 0]]
        X[:3, 3] = ups
        mats.append(expm(X) @ T)
    oracle.apply_tangent(tang, poses)
    assert np.all(tang == 0)
    for i in range(n):
        R = Rotation.from_quat(poses[i, :4]).as_matrix()
        np.testing.assert_allclose(R, mats[i][:3, :3], atol=1e-12)
        np.testing.assert_allclose(poses[i, 4:7], mats[i][:3, 3], atol=1e-12)
        assert np.linalg.norm(poses[i, :4]) == pytest.approx(1.0, abs=1e-12)
