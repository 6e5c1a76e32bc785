"""Pins the oracle's backward against torch autograd of the independent f64 restatement (tests/ref_model.py)
and its projection Jacobians against finite differences. CPU only."""
import numpy as np
import pytest
import torch

from tests import ref_model
from trips_amd import abi, scenes


def _rand_grads(rng, sizes, B, C):
    return [rng.normal(0, 1, (B, C, h, w)).astype(np.float32) for (w, h) in sizes]


def _autograd(sc, d, lists, grads, view, **kw):
    model = ref_model.Differentiable(sc, d, view, lists, **kw)
    img = model.forward()
    g = torch.cat([torch.from_numpy(x[view].astype(np.float64)).reshape(x.shape[1], -1) for x in grads], dim=1)
    (img * g).sum().backward()
    return model


def _close(got, want, rel, name):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    scale = np.abs(want).max() + 1e-30
    err = np.abs(got - want).max() / scale
    assert err < rel, f"{name}: max error {err:.3e} relative to max |value| {scale:.3e}"


@pytest.mark.parametrize("seed,L,K", [(5, 3, 8), (9, 4, 16), (13, 1, 16)])
def test_backward_matches_autograd(oracle, seed, L, K):
    # with a single layer every size takes the "small point" branch 0.75 exp(s-1)+0.25, which exceeds 1 for
    # s > 1; keep sizes below one pixel there so that alpha stays a valid opacity
    radius = (0.005, 0.5) if L > 1 else (0.005, 0.05)
    sc = scenes.tiny(n=900, w=36, h=26, f=36.0, num_layers=L, list_depth=K, seed=seed, radius=radius)
    sc.confidence = (sc.confidence ** 0.3).astype(np.float32)  # push opacities up so transmittance matters
    sc.intrinsics[0, 4] = 0.7  # non-zero skew so that its gradient is exercised
    d = abi.desc_for_scene(sc, background_mode=abi.TRIPS_BG_CONSISTENT)
    fwd = oracle.forward(sc, d)
    rng = np.random.default_rng(seed)
    grads = _rand_grads(rng, fwd["sizes"], 1, sc.num_channels)
    g = oracle.backward(sc, d, fwd, grads)
    m = _autograd(sc, d, fwd["lists"][0], grads, 0)
    _close(g["d_texture"], m.texture.grad.numpy(), 2e-5, "d_texture")
    _close(g["d_background"], m.background.grad.numpy(), 2e-5, "d_background")
    _close(g["d_confidence"], m.confidence.grad.numpy(), 1e-4, "d_confidence")
    _close(g["d_position"][:, :3], m.xyz.grad.numpy(), 1e-4, "d_position")
    assert np.all(g["d_position"][:, 3] == 0)
    _close(g["d_point_size"], m.raw_size.grad.numpy(), 1e-4, "d_point_size")
    _close(g["d_pose"][0], m.tau.grad.numpy(), 1e-4, "d_pose")
    _close(g["d_intrinsics"][0, :5], m.K.grad.numpy(), 1e-4, "d_K")
    assert np.abs(g["d_pose"]).max() > 0 and np.abs(g["d_point_size"]).max() > 0


def test_backward_without_point_size_gradient_drops_layer_factor(oracle):
    # RenderBackward.cu:366-372: without out_gradient_layer the layer factor is 1 in the backward formulas
    sc = scenes.tiny(n=900, w=36, h=26, f=36.0, num_layers=3, list_depth=8, seed=17, radius=(0.005, 0.5))
    d = abi.desc_for_scene(sc, background_mode=abi.TRIPS_BG_CONSISTENT)
    fwd = oracle.forward(sc, d)
    rng = np.random.default_rng(1)
    grads = _rand_grads(rng, fwd["sizes"], 1, sc.num_channels)
    g = oracle.backward(sc, d, fwd, grads, want_point_size=False)
    m = _autograd(sc, d, fwd["lists"][0], grads, 0, layer_factor_in_backward=False)
    assert g["d_point_size"] is None
    _close(g["d_texture"], m.texture.grad.numpy(), 2e-5, "d_texture")
    _close(g["d_confidence"], m.confidence.grad.numpy(), 1e-4, "d_confidence")
    _close(g["d_position"][:, :3], m.xyz.grad.numpy(), 1e-4, "d_position")
    _close(g["d_pose"][0], m.tau.grad.numpy(), 1e-4, "d_pose")
    # and it does differ from the full version
    g_full = oracle.backward(sc, d, fwd, grads)
    assert np.abs(g_full["d_confidence"] - g["d_confidence"]).max() > 1e-3 * np.abs(g["d_confidence"]).max()


def test_backward_accumulates_over_views_and_optional_outputs(oracle):
    sc = scenes.tiny(n=700, w=30, h=22, f=30.0, num_layers=2, list_depth=8, seed=23, views=2, radius=(0.005, 0.4))
    d = abi.desc_for_scene(sc, background_mode=abi.TRIPS_BG_CONSISTENT)
    fwd = oracle.forward(sc, d)
    rng = np.random.default_rng(2)
    grads = _rand_grads(rng, fwd["sizes"], 2, sc.num_channels)
    g = oracle.backward(sc, d, fwd, grads)
    ms = [_autograd(sc, d, fwd["lists"][b], grads, b) for b in range(2)]
    _close(g["d_texture"], sum(m.texture.grad.numpy() for m in ms), 2e-5, "d_texture")
    _close(g["d_position"][:, :3], sum(m.xyz.grad.numpy() for m in ms), 1e-4, "d_position")
    _close(g["d_intrinsics"][0, :5], sum(m.K.grad.numpy() for m in ms), 1e-4, "d_K")
    for b in range(2):
        _close(g["d_pose"][b], ms[b].tau.grad.numpy(), 1e-4, f"d_pose[{b}]")
    # optional outputs can be left out without changing the others
    g2 = oracle.backward(sc, d, fwd, grads, want_position=False, want_pose=False, want_intrinsics=False)
    np.testing.assert_allclose(g2["d_texture"], g["d_texture"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(g2["d_point_size"], g["d_point_size"], rtol=1e-4, atol=1e-6)


def test_reference_background_mode_backward_uses_transmittance_after_last(oracle):
    # the backward is the same in both background modes: it always weights the background with the
    # transmittance after the last entry (RenderBackward.cu:302-308)
    sc = scenes.tiny(n=500, w=30, h=22, f=30.0, num_layers=2, list_depth=8, seed=29)
    rng = np.random.default_rng(3)
    out = []
    for mode in (abi.TRIPS_BG_REFERENCE, abi.TRIPS_BG_CONSISTENT):
        d = abi.desc_for_scene(sc, background_mode=mode)
        fwd = oracle.forward(sc, d)
        if not out:
            grads = _rand_grads(rng, fwd["sizes"], 1, sc.num_channels)
        out.append(oracle.backward(sc, d, fwd, grads))
    for k in ("d_texture", "d_confidence", "d_background", "d_position"):
        np.testing.assert_allclose(out[0][k], out[1][k], rtol=1e-5, atol=1e-6)


def test_zero_gradient_in_zero_gradient_out(oracle):
    sc = scenes.tiny(n=300, w=20, h=16, f=20.0, num_layers=2, seed=31)
    d = abi.desc_for_scene(sc)
    fwd = oracle.forward(sc, d)
    grads = [np.zeros((1, 4, h, w), np.float32) for (w, h) in fwd["sizes"]]
    g = oracle.backward(sc, d, fwd, grads)
    for k, v in g.items():
        assert np.all(v == 0), k


# ---- projection chain ----

def _view(w=64, h=48, crop=(1.0, 1.0, 0.0, 0.0, 0.0), rot=(1.0, 0.0, 0.0, 1.0)):
    v = abi.TripsView()
    v.w, v.h, v.image_index, v.camera_index, v.camera_model_type = w, h, 0, 0, 0
    for i in range(5):
        v.crop_transform[i] = crop[i]
    for i in range(4):
        v.crop_rotation[i] = rot[i]
    return v


def _project64(pose, K, dist, view, xyz, tau=np.zeros(6)):
    """f64 projection with the 8-parameter distortion model and a left pose perturbation exp(tau)."""
    from scipy.linalg import expm
    R, t = ref_model.rotation_from_pose(pose)
    T = np.eye(4)
    T[:3, :3], T[:3, 3] = R, t
    ups, om = tau[:3], tau[3:]
    X = np.zeros((4, 4))
    X[:3, :3] = [[0, -om[2], om[1]], [om[2], 0, -om[0]], [-om[1], om[0], 0]]
    X[:3, 3] = ups
    T = expm(X) @ T
    v = T[:3, :3] @ xyz + T[:3, 3]
    x, y = v[0] / v[2], v[1] / v[2]
    k1, k2, k3, k4, k5, k6, p1, p2 = dist
    r2 = x * x + y * y
    rad = (1 + k1 * r2 + k2 * r2 ** 2 + k3 * r2 ** 3) / (1 + k4 * r2 + k5 * r2 ** 2 + k6 * r2 ** 3)
    xd = x * rad + 2 * p1 * x * y + p2 * (r2 + 2 * x * x)
    yd = y * rad + p1 * (r2 + 2 * y * y) + 2 * p2 * x * y
    fx, fy, cx, cy, s = K
    ix, iy = fx * xd + s * yd + cx, fy * yd + cy
    c = list(view.crop_transform)
    jx, jy = c[0] * ix + c[4] * iy + c[2], c[1] * iy + c[3]
    cr = list(view.crop_rotation)
    ccx, ccy = float(view.w // 2), float(view.h // 2)
    return np.array([cr[0] * (jx - ccx) + cr[1] * (jy - ccy) + ccx, cr[2] * (jx - ccx) + cr[3] * (jy - ccy) + ccy])


@pytest.mark.parametrize("distorted", [False, True])
def test_projection_jacobians_by_finite_differences(oracle, distorted):
    rng = np.random.default_rng(7)
    th = 0.4
    view = _view(crop=(1.3, 0.9, -3.0, 2.0, 0.0), rot=(np.cos(th), -np.sin(th), np.sin(th), np.cos(th)))
    pose = scenes.look_at_pose((0.4, -0.3, -3.0), (0.1, 0.0, 0.2))
    intr = np.zeros(13, dtype=np.float32)
    intr[:5] = [70.0, 65.0, 32.0, 24.0, 0.8]
    if distorted:
        # parity with Saiga's distortNormalizedPoint is unpinned; this checks the model against its own Jacobian
        intr[5:] = [0.1, -0.05, 0.01, 0.02, 0.01, -0.005, 0.003, -0.002]
    K, dist = intr[:5].astype(np.float64), intr[5:].astype(np.float64)
    for _ in range(10):
        xyz = rng.uniform(-0.8, 0.8, 3)
        grad = rng.normal(0, 1, 2)
        got_ip = oracle.project_point(pose, intr, view, 20.0, xyz)
        want_ip = _project64(pose, K, dist, view, xyz)
        np.testing.assert_allclose(got_ip[:2], want_ip, atol=2e-4)
        gp, gpose, gk, gd = oracle.project_point_backward(pose, intr, view, 20.0, xyz, grad)
        f = lambda **kw: float(grad @ _project64(kw.get("pose", pose), kw.get("K", K), kw.get("dist", dist), view,
                                                  kw.get("xyz", xyz), kw.get("tau", np.zeros(6))))
        h = 1e-6

        def fd(key, base, i):
            e = np.zeros_like(base)
            e[i] = h
            return (f(**{key: base + e}) - f(**{key: base - e})) / (2 * h)

        np.testing.assert_allclose(gp, [fd("xyz", xyz, i) for i in range(3)], rtol=2e-4, atol=1e-4)
        np.testing.assert_allclose(gpose, [fd("tau", np.zeros(6), i) for i in range(6)], rtol=2e-4, atol=1e-4)
        np.testing.assert_allclose(gk, [fd("K", K, i) for i in range(5)], rtol=2e-4, atol=1e-4)
        np.testing.assert_allclose(gd, [fd("dist", dist, i) for i in range(8)], rtol=5e-4, atol=2e-4)


def test_zero_distortion_is_identity_and_cutoff_culls(oracle):
    view = _view()
    pose = scenes.look_at_pose((0, 0, -3.0), (0, 0, 0))
    intr = np.zeros(13, dtype=np.float32)
    intr[:5] = [70.0, 70.0, 32.0, 24.0, 0.0]
    out = oracle.project_point(pose, intr, view, 20.0, [0.3, -0.2, 0.0])
    np.testing.assert_allclose(out[:3], [70 * 0.1 + 32, 70 * (-0.2 / 3) + 24, 3.0], rtol=1e-6)
    assert out[3] == pytest.approx(70.0 / 3.0, rel=1e-6)
    # beyond the cut-off radius (normalised coordinates) the point gets depth 0 and is culled
    out = oracle.project_point(pose, intr, view, 0.05, [0.3, -0.2, 0.0])
    assert out[2] == 0.0
