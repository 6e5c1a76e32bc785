"""The reference-shaped operator surface (BlendPointCloud / PointRender autograd function) on the GPU."""
import numpy as np
import pytest
import torch

from trips_amd import abi, scenes

pytestmark = pytest.mark.gpu


def _info(sc, ns, train=True, **params):
    from trips_amd.renderer import NeuralRenderInfo, PointRendererCache, ReducedImageInfo, RenderParams
    p = RenderParams(dropout=0.0, drop_out_points_by_radius=False, max_pixels_per_list=sc.list_depth, **params)
    images = [ReducedImageInfo(w=v["w"], h=v["h"], image_index=v["image_index"], camera_index=v["camera_index"])
              for v in sc.views]
    return NeuralRenderInfo(scene=ns, images=images, params=p, num_layers=sc.num_layers, train=train,
                            cache=PointRendererCache())


def test_blend_point_cloud_forward_backward_matches_oracle(oracle):
    from tests.gpu_util import assert_grad_close
    from trips_amd.renderer import BlendPointCloud, NeuralScene
    sc = scenes.tiny(n=5000, w=80, h=60, f=70.0, num_layers=4, list_depth=16, seed=41, views=2, radius=(0.004, 0.4))
    ns = NeuralScene.from_arrays(sc, requires_grad=True)
    info = _info(sc, ns)
    outs = BlendPointCloud(info)
    assert len(outs) == 4 and outs[0].shape == (2, 4, 60, 80) and outs[3].shape == (2, 4, 8, 10)
    d = abi.desc_for_scene(sc)
    ref = oracle.forward(sc, d)
    for a, b in zip(outs, ref["images"]):
        np.testing.assert_allclose(a.detach().cpu().numpy(), b, rtol=1e-5, atol=1e-6)
    rng = np.random.default_rng(0)
    grads = [rng.normal(0, 1, o.shape).astype(np.float32) for o in outs]
    loss = sum((o * torch.as_tensor(g).cuda()).sum() for o, g in zip(outs, grads))
    loss.backward()
    g_ref = oracle.backward(sc, d, ref, grads)
    pairs = [("d_texture", ns.texture.texture.grad), ("d_background", ns.texture.background_color.grad),
             ("d_position", ns.point_cloud_cuda.t_position.grad), ("d_pose", ns.poses.tangent_poses.grad),
             ("d_intrinsics", ns.intrinsics.intrinsics.grad),
             ("d_confidence", ns.texture.confidence_value_of_point.grad.reshape(-1)),
             ("d_point_size", ns.point_cloud_cuda.t_point_size.grad.reshape(-1))]
    for key, got in pairs:
        assert_grad_close(key, got.cpu().numpy(), g_ref[key])
    assert ns.texture.confidence_value_of_point.grad.shape == (1, 5000)
    assert ns.point_cloud_cuda.t_point_size.grad.shape == (5000, 1)
    assert ns.poses.tangent_poses.grad.dtype == torch.float64


def test_eval_mode_returns_permuted_views_and_no_graph(oracle):
    from trips_amd.renderer import BlendPointCloud, NeuralScene
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=3, list_depth=16, seed=42)
    ns = NeuralScene.from_arrays(sc)
    info = _info(sc, ns, train=False)
    with torch.no_grad():
        outs = BlendPointCloud(info)
    assert outs[0].shape == (1, 4, 48, 64) and not outs[0].is_contiguous()  # [B,H,W,C] storage, permuted view
    d = abi.desc_for_scene(sc, train=False)
    ref = oracle.forward(sc, d)
    for a, b in zip(outs, ref["images"]):
        np.testing.assert_allclose(a.permute(0, 2, 3, 1).cpu().numpy(), b, rtol=1e-5, atol=1e-6)


def test_only_requested_gradients_are_produced(oracle):
    from tests.gpu_util import assert_grad_close
    from trips_amd.renderer import BlendPointCloud, NeuralScene
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=3, list_depth=16, seed=43)
    ns = NeuralScene.from_arrays(sc)
    ns.texture.texture.requires_grad_(True)
    ns.texture.confidence_value_of_point.requires_grad_(True)
    info = _info(sc, ns)
    outs = BlendPointCloud(info)
    sum(o.sum() for o in outs).backward()
    assert ns.point_cloud_cuda.t_position.grad is None and ns.point_cloud_cuda.t_point_size.grad is None
    d = abi.desc_for_scene(sc)
    ref = oracle.forward(sc, d)
    ones = [np.ones(o.shape, np.float32) for o in outs]
    g_ref = oracle.backward(sc, d, ref, ones, want_position=False, want_point_size=False, want_pose=False,
                            want_intrinsics=False)
    assert_grad_close("d_texture", ns.texture.texture.grad.cpu().numpy(), g_ref["d_texture"])
    assert_grad_close("d_confidence", ns.texture.confidence_value_of_point.grad.cpu().numpy().reshape(-1), g_ref["d_confidence"])


def test_dropout_is_drawn_per_forward_in_train_mode():
    from trips_amd.renderer import BlendPointCloud, NeuralScene
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=2, list_depth=16, seed=44)
    ns = NeuralScene.from_arrays(sc)
    info = _info(sc, ns)
    info.params.dropout = 0.5
    torch.manual_seed(0)
    a = BlendPointCloud(info)[0].clone()
    b = BlendPointCloud(info)[0].clone()
    assert not torch.equal(a, b)
    assert info.cache.dropout_points.shape == (1, 3000)
    frac = float(info.cache.dropout_points.mean())
    assert 0.4 < frac < 0.6


def test_unsupported_render_modes_raise():
    from trips_amd.renderer import BlendPointCloud, NeuralScene
    sc = scenes.tiny(n=100)
    ns = NeuralScene.from_arrays(sc)
    info = _info(sc, ns)
    info.params.render_mode = 1
    with pytest.raises(NotImplementedError):
        BlendPointCloud(info)


def test_unused_layers_and_extra_outputs(oracle):
    """A consumer that reads only some pyramid layers leaves the others without a gradient; add_depth_to_network /
    output_background_mask append L zero tensors each, as the reference's path does (PointRenderer.cu:482-505)."""
    from trips_amd.renderer import BlendPointCloud, NeuralScene
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=4, list_depth=16, seed=9)
    ns = NeuralScene.from_arrays(sc, requires_grad=True)
    info = _info(sc, ns, add_depth_to_network=True, output_background_mask=True)
    outs = BlendPointCloud(info)
    assert len(outs) == 12
    for l in range(4):
        assert outs[4 + l].shape == (1, 1) + outs[l].shape[2:] and float(outs[4 + l].detach().abs().max()) == 0.0
        assert outs[8 + l].shape == outs[4 + l].shape and float(outs[8 + l].detach().abs().max()) == 0.0
    rng = np.random.default_rng(1)
    g0, g1 = [torch.as_tensor(rng.normal(0, 1, outs[l].shape).astype(np.float32)).cuda() for l in range(2)]
    ((outs[0] * g0).sum() + (outs[1] * g1).sum()).backward()
    d = abi.desc_for_scene(sc)
    ref = oracle.forward(sc, d)
    grads = [g0.cpu().numpy(), g1.cpu().numpy()] + [np.zeros_like(ref["images"][l]) for l in (2, 3)]
    g_ref = oracle.backward(sc, d, ref, grads)
    from tests.gpu_util import assert_grad_close
    assert_grad_close("d_texture", ns.texture.texture.grad.cpu().numpy(), g_ref["d_texture"])
    assert_grad_close("d_position", ns.point_cloud_cuda.t_position.grad.cpu().numpy(), g_ref["d_position"])


def test_dynamic_refinement_displaces_points_per_view(oracle):
    """A [B,N,3] dynamic_refinement_t moves the points of view b; the [1] dummy does nothing; no gradient comes back
    for it (the reference never allocates one, PointRenderer.cu:243-252)."""
    from tests.gpu_util import assert_grad_close
    from trips_amd.renderer import BlendPointCloud, NeuralScene
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=3, list_depth=16, seed=43, views=2)
    sc.displacement = np.random.default_rng(6).normal(0, 0.05, (2, 3000, 3)).astype(np.float32)
    ns = NeuralScene.from_arrays(sc, requires_grad=True)
    ns.dynamic_refinement_t = torch.as_tensor(sc.displacement).cuda().requires_grad_(True)
    outs = BlendPointCloud(_info(sc, ns))
    d = abi.desc_for_scene(sc)
    ref = oracle.forward(sc, d)
    for a, b in zip(outs, ref["images"]):
        np.testing.assert_allclose(a.detach().cpu().numpy(), b, rtol=1e-5, atol=1e-6)
    rng = np.random.default_rng(0)
    grads = [rng.normal(0, 1, o.shape).astype(np.float32) for o in outs]
    sum((o * torch.as_tensor(g).cuda()).sum() for o, g in zip(outs, grads)).backward()
    g_ref = oracle.backward(sc, d, ref, grads)
    assert_grad_close("d_position", ns.point_cloud_cuda.t_position.grad.cpu().numpy(), g_ref["d_position"])
    assert_grad_close("d_pose", ns.poses.tangent_poses.grad.cpu().numpy(), g_ref["d_pose"])
    assert ns.dynamic_refinement_t.grad is None
    ns.dynamic_refinement_t = torch.zeros((2, 5, 3), device="cuda")
    with pytest.raises(ValueError):
        BlendPointCloud(_info(sc, ns))


def test_step_replays_from_a_hip_graph(oracle):
    """The C ABI is stream-ordered and allocates nothing, so a caller can capture forward + backward + fused Adam
    once and replay it. Every replay is checked against the eager step it stands for, with eager work between the
    replays."""
    from trips_amd.adam import MyAdam
    from trips_amd.renderer import SplatContext, get_context
    sc = scenes.tiny(n=6000, w=96, h=64, f=80.0, num_layers=4, list_depth=16, seed=61, views=2, radius=(0.004, 0.4))
    d = abi.desc_for_scene(sc)
    ctx = get_context(0)
    dev = ctx.device
    f = lambda a, dt=torch.float32: torch.as_tensor(np.ascontiguousarray(a), dtype=dt).to(dev).contiguous()

    def make():
        t = dict(position=f(sc.position), point_size=f(sc.point_size), index=f(sc.index, torch.int32),
                 texture=f(sc.texture), confidence=f(sc.confidence), background=f(sc.background),
                 poses_se3=f(sc.poses_se3, torch.float64), intrinsics=f(sc.intrinsics), dropout=None)
        N, C = d.num_points, d.num_channels
        grads = dict(d_texture=torch.zeros((C, N), device=dev), d_confidence=torch.zeros(N, device=dev),
                     d_background=torch.zeros(C, device=dev), d_position=torch.zeros((N, 4), device=dev),
                     d_point_size=torch.zeros(N, device=dev), d_pose=torch.zeros((d.num_images, 6), dtype=torch.float64, device=dev),
                     d_intrinsics=torch.zeros((d.num_cameras, 13), device=dev))
        params = [torch.nn.Parameter(t[k]) for k in ("position", "point_size", "texture", "confidence")]
        for p, k in zip(params, ("d_position", "d_point_size", "d_texture", "d_confidence")):
            p.grad = grads[k]
        state = dict(t=t, grads=grads, tin=SplatContext.make_in(**t), opt=MyAdam(params, lr=1e-2),
                     ws=ctx.alloc_bytes(ctx.workspace_size(d)), saved=ctx.alloc_bytes(ctx.saved_size(d)),
                     images=ctx.alloc_images(d))
        gen = torch.Generator(device=dev)
        gen.manual_seed(7)
        state["gi"] = [torch.randn(im.shape, generator=gen, device=dev) for im in state["images"]]
        return state

    def step(s):
        for g in s["grads"].values():
            g.zero_()
        ctx.forward(d, s["tin"], s["images"], s["saved"], s["ws"])
        ctx.backward(d, s["tin"], s["saved"], s["gi"], s["grads"], s["ws"])
        s["opt"].step()

    eager, graphed = make(), make()
    step(eager)
    step(graphed)  # the optimiser's state tensors exist before the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step(graphed)
    torch.cuda.synchronize()
    step(eager)  # the capture itself does not run the step; the first replay does
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        for k in ("position", "texture", "confidence", "point_size"):
            assert torch.equal(graphed["t"][k], eager["t"][k]), k
        for a, b in zip(graphed["images"], eager["images"]):
            assert torch.equal(a, b)
        # summed with double atomics over workgroups: equal up to the order of the additions
        assert torch.allclose(graphed["grads"]["d_pose"], eager["grads"]["d_pose"], rtol=1e-9, atol=1e-12)
        (eager["images"][0].sum() + graphed["images"][0].sum()).item()  # eager work and a synchronisation in between
        step(eager)


def test_normalize_grads_changes_nothing_on_this_path():
    """RenderParams.normalize_grads divides the point gradients by per-point counts (PointRenderer.cu:1193-1230,
    1348-1411), but the backward of this path never increments those counts (RenderBackward.cu has no count
    atomics), so `c > 0` at PointRenderer.cu:1202,1223 is never true and the flag leaves the gradients as they are."""
    from trips_amd.renderer import BlendPointCloud, NeuralScene
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=3, list_depth=16, seed=45)
    rng = np.random.default_rng(2)
    grads = None
    results = []
    for flag in (False, True):
        ns = NeuralScene.from_arrays(sc, requires_grad=True)
        outs = BlendPointCloud(_info(sc, ns, normalize_grads=flag))
        if grads is None:
            grads = [torch.as_tensor(rng.normal(0, 1, o.shape).astype(np.float32)).cuda() for o in outs]
        sum((o * g).sum() for o, g in zip(outs, grads)).backward()
        results.append([t.grad.clone() for t in (ns.texture.texture, ns.texture.confidence_value_of_point,
                                                  ns.point_cloud_cuda.t_position, ns.point_cloud_cuda.t_point_size)])
    for a, b in zip(*results):
        assert float(a.abs().max()) > 0 and torch.equal(a, b)


def test_backward_refuses_inputs_modified_in_place_after_the_forward():
    """The backward reads position, size, index, poses and intrinsics again; an optimiser step between forward and
    backward would silently give the gradients of another scene."""
    from trips_amd.renderer import BlendPointCloud, NeuralScene
    sc = scenes.tiny(n=2000, w=64, h=48, f=60.0, num_layers=3, list_depth=16, seed=46)
    ns = NeuralScene.from_arrays(sc, requires_grad=True)
    outs = BlendPointCloud(_info(sc, ns))
    with torch.no_grad():
        ns.point_cloud_cuda.t_position.add_(0.0)
    with pytest.raises(RuntimeError, match="modified in place"):
        sum(o.sum() for o in outs).backward()
