"""The full training step as one chain: splat forward -> reconstruction net forward -> L1 loss -> net backward ->
splat backward (fed with the net's input gradients, the unused coarse layers without a gradient) -> fused Adam over
the point parameters and the net weights. Reference shape of the step: src/lib/models/Pipeline.cpp:317,583-587 and
src/apps/train.cpp:1089-1110.

Every stage of the HIP chain is held against its own checker, fed with what the HIP chain produced upstream of it, so
that each bar is the stage's own (splat: tests/gpu_util.py; net: fp16 operands, 2e-3 forward / 2e-2 gradients of the
largest magnitude; Adam 2e-6); on top of that the point gradients are compared end to end at the net's bar."""
import copy

import numpy as np
import pytest
import torch

from trips_amd import abi, scenes

pytestmark = pytest.mark.gpu

NET_FWD_TOL = 2e-3
NET_GRAD_TOL = 2e-2
ADAM_TOL = 2e-6


def _make_net(num_input_layers, seed, channels=4, filters=(16, 32, 64, 64)):
    from trips_amd.unet import MultiScaleUnet2dDecOnlySmallFixed, MultiScaleUnet2dParams
    p = MultiScaleUnet2dParams(num_input_layers=num_input_layers, num_layers=4, num_input_channels=channels,
                               filters_network=list(filters))
    g = torch.Generator().manual_seed(seed)
    net = MultiScaleUnet2dDecOnlySmallFixed(p).he_normal_(g)
    with torch.no_grad():
        for m in net.modules():
            if isinstance(m, torch.nn.Conv2d):
                m.bias.normal_(0.0, 0.1, generator=g)
    return net


def _point_params(ns):
    return dict(d_position=ns.point_cloud_cuda.t_position, d_point_size=ns.point_cloud_cuda.t_point_size,
                d_texture=ns.texture.texture, d_confidence=ns.texture.confidence_value_of_point)


def _max_norm(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.abs(got - want).max() / (np.abs(want).max() + 1e-30))


def _oracle_adam(oracle, w, g, lr=1e-3):
    """One oracle Adam step from zero state on copies; returns the new weights and the step counters."""
    w = np.ascontiguousarray(w, dtype=np.float32).reshape(-1).copy()
    g = np.ascontiguousarray(g, dtype=np.float32).reshape(-1)
    m, v = np.zeros_like(w), np.zeros_like(w)
    steps = np.zeros(w.shape, dtype=np.int64)
    oracle.adam_step([dict(w=w, g=g, m=m, v=v, steps=steps, n=w.size, lr=lr)])
    return w, steps


@pytest.mark.parametrize("channels,filters", [(4, (16, 32, 64, 64)), (8, (32, 48, 64, 64))])
def test_config5_chain_small(oracle, channels, filters):
    from tests.gpu_util import assert_grads_close
    from tests.ref_unet import unet_forward
    from tests.test_gpu_operator import _info
    from trips_amd.adam import MyAdam
    from trips_amd.renderer import BlendPointCloud, NeuralScene

    sc = scenes.tiny(n=20000, w=160, h=120, f=120.0, num_layers=8, list_depth=16, seed=55, radius=(0.004, 0.3),
                     channels=channels)
    d = abi.desc_for_scene(sc)
    ns = NeuralScene.from_arrays(sc, requires_grad=True)
    net_cpu = _make_net(8, seed=11, channels=channels, filters=filters)
    net = copy.deepcopy(net_cpu).cuda()
    target = torch.rand((1, 3, sc.height, sc.width), generator=torch.Generator().manual_seed(12))

    # ---- the HIP chain through the reference-shaped operator surface ----
    outs = BlendPointCloud(_info(sc, ns))
    assert len(outs) == 8
    for o in outs:
        o.retain_grad()
    rgb = net.forward(list(outs))
    loss = (rgb - target.cuda()).abs().mean()
    loss.backward()
    torch.cuda.synchronize()

    # ---- splat forward against the oracle ----
    ref = oracle.forward(sc, d)
    for l, (a, b) in enumerate(zip(outs, ref["images"])):
        np.testing.assert_allclose(a.detach().cpu().numpy(), b, rtol=1e-5, atol=1e-6, err_msg=f"layer {l}")

    # ---- net forward and loss against the torch restatement, fed with the HIP pyramid ----
    ins_ref = [o.detach().cpu().clone().requires_grad_(True) for o in outs]
    rgb_ref = unet_forward(net_cpu, ins_ref, half_rounding=True)
    assert _max_norm(rgb.detach().cpu().numpy(), rgb_ref.detach().numpy()) < NET_FWD_TOL
    loss_ref = float((rgb_ref.detach() - target).abs().mean())
    assert abs(float(loss.detach()) - loss_ref) < NET_FWD_TOL * max(1.0, loss_ref)

    # ---- net backward: the L1 gradient is evaluated on the HIP output (a sign flip of |rgb - target| where the two
    # outputs straddle the target is the loss's own discontinuity, not an error of either net) ----
    upstream = torch.sign(rgb.detach().cpu() - target) / rgb.numel()
    (rgb_ref * upstream).sum().backward()
    for i in range(4):
        assert outs[i].grad is not None
        assert _max_norm(outs[i].grad.cpu().numpy(), ins_ref[i].grad.numpy()) < NET_GRAD_TOL, f"d inputs[{i}]"
    for i in range(4, 8):
        assert outs[i].grad is None  # the net consumes four of the eight layers
    net_grads = {}
    for (n1, p1), (n2, p2) in zip(net.named_parameters(), net_cpu.named_parameters()):
        assert n1 == n2 and p1.grad is not None
        assert _max_norm(p1.grad.cpu().numpy(), p2.grad.numpy()) < NET_GRAD_TOL, n1
        net_grads[n1] = p1.grad.cpu().numpy().copy()

    # ---- splat backward against the oracle, fed with the HIP net's input gradients (zeros for the unused layers) ----
    gi_hip = [outs[i].grad.cpu().numpy() for i in range(4)] + [np.zeros_like(ref["images"][i]) for i in range(4, 8)]
    g_ref = oracle.backward(sc, d, ref, gi_hip)
    pp = _point_params(ns)
    got = {k: p.grad.detach().cpu().numpy().reshape(g_ref[k].shape) for k, p in pp.items()}
    got["d_background"] = ns.texture.background_color.grad.cpu().numpy()
    got["d_pose"] = ns.poses.tangent_poses.grad.cpu().numpy()
    got["d_intrinsics"] = ns.intrinsics.intrinsics.grad.cpu().numpy()
    assert_grads_close(got, g_ref, what="chain: ")
    assert np.abs(got["d_position"]).max() > 0 and np.abs(got["d_texture"]).max() > 0
    # end to end (oracle forward -> torch net -> torch autograd -> oracle backward) at the net's bar
    gi_ref = [ins_ref[i].grad.numpy() for i in range(4)] + gi_hip[4:]
    g_e2e = oracle.backward(sc, d, ref, gi_ref)
    for k in ("d_position", "d_point_size", "d_texture", "d_confidence"):
        assert _max_norm(got[k], g_e2e[k]) < NET_GRAD_TOL, f"end to end {k}"

    # ---- fused Adam over the point parameters and over the net weights ----
    before = {k: p.detach().cpu().numpy().copy() for k, p in pp.items()}
    net_before = {n: p.detach().cpu().numpy().copy() for n, p in net.named_parameters()}
    opt = MyAdam(list(pp.values()), lr=1e-3)
    net_opt = MyAdam(list(net.parameters()), lr=1e-3)
    opt.step()
    net_opt.step()
    torch.cuda.synchronize()
    for k, p in pp.items():
        want, steps = _oracle_adam(oracle, before[k], got[k])
        np.testing.assert_allclose(p.detach().cpu().numpy().reshape(-1), want, rtol=ADAM_TOL, atol=1e-7, err_msg=k)
        np.testing.assert_array_equal(opt.state[p]["param_steps"].cpu().numpy().reshape(-1), steps)
        assert 0 < int(steps.sum()) < steps.size  # culled points keep their counters (MyAdam.cu:57-61)
    for n, p in net.named_parameters():
        want, steps = _oracle_adam(oracle, net_before[n], net_grads[n])
        np.testing.assert_allclose(p.detach().cpu().numpy().reshape(-1), want, rtol=ADAM_TOL, atol=1e-7, err_msg=n)


def test_config5_full_size_steps():
    """6M points, 1920x1080, eight splat layers, the net on four of them: outputs finite, the forward and the
    per-point gradients repeat bit for bit, and the L1 loss falls over five optimiser steps."""
    from trips_amd.adam import MyAdam
    from trips_amd.renderer import (BlendPointCloud, NeuralRenderInfo, NeuralScene, PointRendererCache, ReducedImageInfo,
                                    RenderParams)
    sc = scenes.config3()
    ns = NeuralScene.from_arrays(sc, requires_grad=True)
    p = RenderParams(dropout=0.0, drop_out_points_by_radius=False, max_pixels_per_list=16)
    views = [ReducedImageInfo(w=v["w"], h=v["h"], image_index=v["image_index"], camera_index=v["camera_index"])
             for v in sc.views]
    info = NeuralRenderInfo(scene=ns, images=views, params=p, num_layers=8, train=True, cache=PointRendererCache())
    net = _make_net(8, seed=21).cuda()
    target = torch.rand((1, 3, sc.height, sc.width), generator=torch.Generator().manual_seed(22)).cuda()
    pp = _point_params(ns)
    everything = list(pp.values()) + list(net.parameters()) + [ns.texture.background_color, ns.poses.tangent_poses,
                                                               ns.intrinsics.intrinsics]

    def step():
        for q in everything:
            q.grad = None
        outs = BlendPointCloud(info)
        rgb = net.forward(list(outs))
        loss = (rgb - target).abs().mean()
        loss.backward()
        return rgb.detach(), float(loss.detach())

    rgb_a, loss_a = step()
    grads_a = {k: q.grad.clone() for k, q in pp.items()}
    rgb_b, loss_b = step()
    assert torch.isfinite(rgb_a).all()
    assert torch.equal(rgb_a, rgb_b) and loss_a == loss_b
    for k, q in pp.items():
        assert torch.isfinite(q.grad).all(), k
        assert float(q.grad.abs().max()) > 0, k
        # the net's input gradients are plain sums in a fixed order and the splat backward has no float atomics on
        # the per-point outputs
        assert torch.equal(q.grad, grads_a[k]), k
    for n, q in net.named_parameters():
        assert torch.isfinite(q.grad).all(), n

    opt = MyAdam(list(pp.values()), lr=1e-3)
    net_opt = MyAdam(list(net.parameters()), lr=1e-3)
    losses = [loss_b]
    for _ in range(5):
        opt.step()
        net_opt.step()
        losses.append(step()[1])
    assert all(np.isfinite(losses))
    assert losses[-1] < losses[0], losses
