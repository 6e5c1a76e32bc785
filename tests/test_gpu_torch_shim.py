"""The C++ libtorch host side (trips_amd/csrc/torch_shim): BlendPointCloud / PointRender / MyAdam / ApplyTangent
driven through its pybind11 test module, against the CPU oracle."""
import numpy as np
import pytest
import torch

from trips_amd import abi, scenes


def _load():
    from trips_amd import _trips_torch  # noqa: built by trips_amd.build.build_torch_shim
    return _trips_torch


def test_shim_module_imports_without_gpu():
    m = _load()
    assert hasattr(m, "Session")
    s = m.Session()
    assert hasattr(s, "blend_point_cloud") and hasattr(s, "adam_step") and hasattr(s, "apply_tangent")


def _session(sc, requires_grad=True):
    m = _load()
    f = lambda a, dt=torch.float32: torch.as_tensor(np.ascontiguousarray(a), dtype=dt).cuda().contiguous()
    t = dict(texture=f(sc.texture), background=f(sc.background), confidence=f(sc.confidence).reshape(1, -1),
             position=f(sc.position), point_size=f(sc.point_size).reshape(-1, 1),
             index=f(sc.index, torch.int32).reshape(-1, 1), poses_se3=f(sc.poses_se3, torch.float64),
             tangent_poses=torch.zeros((sc.poses_se3.shape[0], 6), dtype=torch.float64, device="cuda"),
             intrinsics=f(sc.intrinsics))
    if requires_grad:
        for k in ("texture", "background", "confidence", "position", "point_size", "tangent_poses", "intrinsics"):
            t[k].requires_grad_(True)
    s = m.Session()
    s.set_scene(t["texture"], t["background"], t["confidence"], t["position"], t["point_size"], t["index"],
                t["poses_se3"], t["tangent_poses"], t["intrinsics"])
    return s, t


@pytest.mark.gpu
def test_cpp_blend_point_cloud_forward_backward(oracle):
    from tests.gpu_util import assert_grad_close
    sc = scenes.tiny(n=5000, w=80, h=60, f=70.0, num_layers=4, list_depth=16, seed=51, views=2, radius=(0.004, 0.4))
    s, t = _session(sc)
    views = [[v["w"], v["h"], v["image_index"], v["camera_index"]] for v in sc.views]
    outs = s.blend_point_cloud(views, sc.num_layers, True, 0.0, 0, 16)
    d = abi.desc_for_scene(sc)
    ref = oracle.forward(sc, d)
    assert len(outs) == 4
    for a, b in zip(outs, ref["images"]):
        np.testing.assert_allclose(a.detach().cpu().numpy(), b, rtol=1e-5, atol=1e-6)
    rng = np.random.default_rng(0)
    grads = [rng.normal(0, 1, o.shape).astype(np.float32) for o in outs]
    sum((o * torch.as_tensor(g).cuda()).sum() for o, g in zip(outs, grads)).backward()
    g_ref = oracle.backward(sc, d, ref, grads)
    pairs = [("d_texture", t["texture"].grad), ("d_background", t["background"].grad),
             ("d_position", t["position"].grad), ("d_pose", t["tangent_poses"].grad),
             ("d_intrinsics", t["intrinsics"].grad), ("d_confidence", t["confidence"].grad.reshape(-1)),
             ("d_point_size", t["point_size"].grad.reshape(-1))]
    for key, got in pairs:
        assert_grad_close(key, got.cpu().numpy(), g_ref[key])


@pytest.mark.gpu
def test_cpp_eval_mode_and_crop(oracle):
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=3, list_depth=16, seed=52)
    sc.views[0]["crop_transform"] = (1.5, 1.25, -10.0, 4.0, 0.0)
    s, t = _session(sc, requires_grad=False)
    v = sc.views[0]
    views = [[v["w"], v["h"], 0, 0, *v["crop_transform"], 1.0, 0.0, 0.0, 1.0]]
    with torch.no_grad():
        outs = s.blend_point_cloud(views, sc.num_layers, False, 0.0, 0, 16)
    assert outs[0].shape == (1, 4, 48, 64)
    ref = oracle.forward(sc, abi.desc_for_scene(sc, train=False))
    for a, b in zip(outs, ref["images"]):
        np.testing.assert_allclose(a.permute(0, 2, 3, 1).cpu().numpy(), b, rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
def test_cpp_myadam_and_apply_tangent(oracle):
    sc = scenes.tiny(n=2000, w=48, h=40, f=45.0, num_layers=2, list_depth=16, seed=53)
    s, t = _session(sc)
    rng = np.random.default_rng(3)
    gpos = rng.normal(0, 1, sc.position.shape).astype(np.float32)
    gpos[::3] = 0
    gtan = rng.normal(0, 1, (1, 6))
    w0 = t["position"].detach().cpu().numpy().copy()
    p0 = t["tangent_poses"].detach().cpu().numpy().copy()
    s.make_adam([t["position"], t["tangent_poses"]], 1e-2)
    ref_w = dict(w=w0.reshape(-1).copy(), g=gpos.reshape(-1), m=np.zeros(w0.size, np.float32),
                 v=np.zeros(w0.size, np.float32), steps=np.zeros(w0.size, np.int64), n=w0.size, lr=1e-2)
    ref_p = dict(w=p0.reshape(-1).copy(), g=gtan.reshape(-1), m=np.zeros(6, np.float32), v=np.zeros(6, np.float32),
                 steps=np.zeros(6, np.int64), n=6, lr=1e-2, dtype=abi.TRIPS_DTYPE_F64)
    for _ in range(2):
        t["position"].grad = torch.as_tensor(gpos).cuda()
        t["tangent_poses"].grad = torch.as_tensor(gtan).cuda()
        s.adam_step()
        oracle.adam_step([ref_w, ref_p])
    torch.cuda.synchronize()
    np.testing.assert_allclose(t["position"].detach().cpu().numpy().reshape(-1), ref_w["w"], rtol=2e-6, atol=1e-7)
    np.testing.assert_allclose(t["tangent_poses"].detach().cpu().numpy().reshape(-1), ref_p["w"], rtol=2e-6, atol=1e-9)
    # pose <- exp(tangent) * pose, tangent <- 0
    poses = sc.poses_se3.copy()
    tang = t["tangent_poses"].detach().cpu().numpy().copy()
    with torch.no_grad():
        s.apply_tangent()
    torch.cuda.synchronize()
    oracle.apply_tangent(tang, poses)
    np.testing.assert_allclose(t["poses_se3"].cpu().numpy(), poses, atol=1e-13)
    assert float(t["tangent_poses"].detach().abs().max()) == 0.0


@pytest.mark.gpu
def test_cpp_myadam_points_equals_per_tensor_myadam():
    """torch::optim::MyAdamPoints (C++ shim, state packed per point) against the Python MyAdam with the reference's
    per-tensor state: the same groups and options, points without gradient, a step in which the sizes have no
    gradient, and the pose tangents as a parameter outside the packed four. Bit for bit."""
    from trips_amd.adam import MyAdam
    sc = scenes.tiny(n=3001, w=48, h=40, f=45.0, num_layers=2, list_depth=16, seed=57)
    s, t = _session(sc)
    names = ("position", "point_size", "texture", "confidence", "tangent_poses")
    twin = {k: torch.nn.Parameter(t[k].detach().clone()) for k in names}
    lr = 1e-2
    plain = MyAdam([{"params": [twin["position"]]}, {"params": [twin["point_size"]]},
                    {"params": [twin["texture"]], "lr": 2 * lr}, {"params": [twin["confidence"]]},
                    {"params": [twin["tangent_poses"]]}], lr=lr)
    s.make_adam_points([t["tangent_poses"]], lr)
    rng = np.random.default_rng(4)
    n = sc.num_points
    for step in range(3):
        dead = torch.as_tensor(rng.random(n) < 0.4).cuda()
        for k in names:
            g = torch.as_tensor(rng.normal(0, 1, tuple(t[k].shape))).to(t[k].dtype).cuda()
            if k in ("position", "point_size"):
                g[dead] = 0
            elif k in ("texture", "confidence"):
                g[:, dead] = 0
            if k == "point_size" and step == 1:
                g = None
            t[k].grad = g
            twin[k].grad = None if g is None else g.clone()
        s.adam_step()
        plain.step()
    torch.cuda.synchronize()
    for k in names:
        assert torch.equal(t[k].detach(), twin[k].detach()), k


@pytest.mark.gpu
def test_cpp_myadam_points_save_load_resumes_bit_for_bit(tmp_path):
    """torch::optim::MyAdamPoints::save / load (the reference leaves MyAdam's unimplemented, MyAdam.cu:417-425): an
    optimiser restored from the archive continues like the one that never stopped."""
    sc = scenes.tiny(n=2001, w=48, h=40, f=45.0, num_layers=2, list_depth=16, seed=58)
    names = ("position", "point_size", "texture", "confidence", "tangent_poses")
    rng = np.random.default_rng(5)
    grads = [{k: None for k in names} for _ in range(4)]
    sa, ta = _session(sc)
    for step in range(4):
        for k in names:
            grads[step][k] = torch.as_tensor(rng.normal(0, 1, tuple(ta[k].shape))).to(ta[k].dtype).cuda()
    lr = 1e-2
    sa.make_adam_points([ta["tangent_poses"]], lr)

    def run(s, t, steps):
        for step in steps:
            for k in names:
                t[k].grad = grads[step][k].clone()
            s.adam_step()
    run(sa, ta, (0, 1))
    path = str(tmp_path / "adam.pt")
    sa.adam_save(path)
    sb, tb = _session(sc)
    with torch.no_grad():
        for k in names:
            tb[k].copy_(ta[k])
    sb.make_adam_points([tb["tangent_poses"]], lr)
    sb.adam_load(path)
    run(sa, ta, (2, 3))
    run(sb, tb, (2, 3))
    torch.cuda.synchronize()
    for k in names:
        assert torch.equal(ta[k].detach(), tb[k].detach()), k


@pytest.mark.gpu
def test_cpp_unet_forward_backward_matches_python_mirror():
    """The C++ module (trips_unet_torch.cpp) and the Python mirror drive the same kernels: same weights -> same
    output and gradients; torch autograd through the C++ autograd node reaches inputs and parameters."""
    from trips_amd.unet import MultiScaleUnet2dDecOnlySmallFixed, MultiScaleUnet2dParams
    m = _load()
    filters, L = [16, 32, 64, 64], 4
    cpp = m.UnetSession(filters, L, L)
    py = MultiScaleUnet2dDecOnlySmallFixed(MultiScaleUnet2dParams(num_input_layers=L, num_layers=L,
                                                                  filters_network=filters))
    py.he_normal_(torch.Generator().manual_seed(3))
    cpp_params = dict(cpp.named_parameters())
    with torch.no_grad():
        for n, q in py.named_parameters():
            cpp_params[n].copy_(q)
    cpp.cuda()
    py = py.cuda()
    cpp_params = dict(cpp.named_parameters())
    g = torch.Generator().manual_seed(4)
    sizes = abi.layer_sizes(96, 72, L)
    ins = [torch.rand((2, 4, h, w), generator=g) for (w, h) in sizes]
    up = torch.randn((2, 3, 72, 96), generator=g).cuda() * 1e-3
    a = [t.cuda().requires_grad_(True) for t in ins]
    b = [t.cuda().requires_grad_(True) for t in ins]
    out_cpp = cpp.forward(a)
    out_py = py.forward(b)
    assert torch.equal(out_cpp, out_py)
    (out_cpp * up).sum().backward()
    (out_py * up).sum().backward()
    for x, y in zip(a, b):
        assert torch.equal(x.grad, y.grad)
    for n, q in py.named_parameters():
        assert cpp_params[n].grad is not None, n
        # bias and 1x1 gradients are summed with float atomics: same values up to summation order
        assert torch.allclose(cpp_params[n].grad, q.grad, rtol=1e-4, atol=1e-7 * float(q.grad.abs().max())), n
    # without gradients nothing is kept for a backward; a viewer's frames reuse the packed weights on request
    plain = [t.cuda() for t in ins]
    frame = cpp.forward_no_grad(plain)
    assert torch.equal(frame, out_cpp.detach())
    cpp.set_reuse_packed_weights(True)
    assert torch.equal(cpp.forward_no_grad(plain), frame) and torch.equal(cpp.forward_no_grad(plain), frame)
    name = next(n for n, _ in py.named_parameters() if n.endswith("feature_transform.0.weight"))
    with torch.no_grad():
        cpp_params[name].mul_(1.5)
        dict(py.named_parameters())[name].mul_(1.5)
        cpp.invalidate_packed_weights()
        changed = cpp.forward_no_grad(plain)
        assert not torch.equal(changed, frame) and torch.equal(changed, py.forward(plain))


@pytest.mark.gpu
def test_cpp_unused_layers_and_extra_outputs(oracle):
    from tests.gpu_util import assert_grad_close
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=4, list_depth=16, seed=9)
    s, t = _session(sc)
    views = [[v["w"], v["h"], v["image_index"], v["camera_index"]] for v in sc.views]
    outs = s.blend_point_cloud(views, sc.num_layers, True, 0.0, 0, 16, True, True)
    assert len(outs) == 12 and all(float(o.abs().max()) == 0.0 and o.shape[1] == 1 for o in outs[4:])
    rng = np.random.default_rng(1)
    g0 = rng.normal(0, 1, outs[0].shape).astype(np.float32)
    (outs[0] * torch.as_tensor(g0).cuda()).sum().backward()  # layers 1..3 get no gradient
    d = abi.desc_for_scene(sc)
    ref = oracle.forward(sc, d)
    g_ref = oracle.backward(sc, d, ref, [g0] + [np.zeros_like(ref["images"][l]) for l in (1, 2, 3)])
    assert_grad_close("d_texture", t["texture"].grad.cpu().numpy(), g_ref["d_texture"])
    assert_grad_close("d_position", t["position"].grad.cpu().numpy(), g_ref["d_position"])


@pytest.mark.gpu
def test_cpp_dynamic_refinement(oracle):
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=3, list_depth=16, seed=44, views=2)
    sc.displacement = np.random.default_rng(7).normal(0, 0.05, (2, 3000, 3)).astype(np.float32)
    s, t = _session(sc, requires_grad=False)
    s.set_dynamic_refinement(torch.as_tensor(sc.displacement).cuda())
    views = [[v["w"], v["h"], v["image_index"], v["camera_index"]] for v in sc.views]
    with torch.no_grad():
        outs = s.blend_point_cloud(views, sc.num_layers, True, 0.0, 0, 16)
    ref = oracle.forward(sc, abi.desc_for_scene(sc))
    for a, b in zip(outs, ref["images"]):
        np.testing.assert_allclose(a.cpu().numpy(), b, rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
def test_cpp_backward_refuses_inputs_modified_in_place_after_the_forward():
    sc = scenes.tiny(n=2000, w=64, h=48, f=60.0, num_layers=3, list_depth=16, seed=46)
    s, t = _session(sc)
    views = [[v["w"], v["h"], v["image_index"], v["camera_index"]] for v in sc.views]
    outs = s.blend_point_cloud(views, sc.num_layers, True, 0.0, 0, 16)
    with torch.no_grad():
        t["position"].add_(0.0)
    with pytest.raises(RuntimeError, match="modified in place"):
        sum(o.sum() for o in outs).backward()
