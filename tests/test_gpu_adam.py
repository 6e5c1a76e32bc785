"""Fused Adam and pose update on the GPU against the CPU oracle."""
import numpy as np
import pytest
import torch

from trips_amd import abi

pytestmark = pytest.mark.gpu


def _mk(n, rng, dtype=np.float32, zero_frac=0.3, **hyper):
    g = rng.normal(0, 1, n).astype(dtype)
    g[rng.random(n) < zero_frac] = 0
    t = dict(w=rng.normal(0, 1, n).astype(dtype), g=g, m=np.zeros(n, np.float32), v=np.zeros(n, np.float32),
             steps=np.zeros(n, np.int64), n=n, dtype=abi.TRIPS_DTYPE_F64 if dtype == np.float64 else abi.TRIPS_DTYPE_F32)
    t.update(hyper)
    return t


def test_fused_adam_matches_oracle(oracle):
    from tests.oracle_lib import fill_adam_tensor
    from trips_amd.renderer import get_context
    ctx = get_context(0)
    rng = np.random.default_rng(0)
    specs = [_mk(6001 * 4, rng, lr=1e-3), _mk(6001, rng, lr=5e-3, relative_weight_decay=0.05),
             _mk(4 * 6001 + 3, rng, lr=1e-2, absolute_weight_decay=0.01, weight_clipping_magnitude=1.5),
             _mk(6001, rng, lr=1e-3, lower_lr_bound=0.0, upper_lr_bound=0.02),
             _mk(37 * 6, rng, dtype=np.float64, lr=1e-4, zero_frac=0.0), _mk(1, rng), _mk(0, rng)]
    # the same with 32-bit step counters
    for extra in (_mk(6001 * 4, rng, lr=1e-3), _mk(4 * 6001 + 3, rng, lr=2e-3), _mk(50, rng, dtype=np.float64)):
        extra["steps"] = np.zeros(extra["n"], np.int32)
        extra["steps_dtype"] = abi.TRIPS_STEPS_I32
        specs.append(extra)
    dev = ctx.device
    gpu = []
    for s in specs:
        gpu.append({k: (torch.as_tensor(v).to(dev) if isinstance(v, np.ndarray) else v) for k, v in s.items()})
    for step in range(3):
        for s, gt in zip(specs, gpu):
            g = rng.normal(0, 1, s["n"]).astype(s["g"].dtype)
            g[rng.random(s["n"]) < 0.3] = 0
            s["g"][:] = g
            gt["g"].copy_(torch.as_tensor(g))
        descs = []
        for gt in gpu:
            d = abi.TripsAdamTensor()
            fill_adam_tensor(d, gt, lambda a: a.data_ptr())
            descs.append(d)
        ctx.adam_step(descs)
        torch.cuda.synchronize()
        oracle.adam_step(specs)
        for i, (s, gt) in enumerate(zip(specs, gpu)):
            np.testing.assert_array_equal(gt["steps"].cpu().numpy(), s["steps"], err_msg=f"tensor {i}")
            np.testing.assert_allclose(gt["m"].cpu().numpy(), s["m"], rtol=1e-6, atol=1e-9, err_msg=f"tensor {i}")
            np.testing.assert_allclose(gt["v"].cpu().numpy(), s["v"], rtol=1e-6, atol=1e-12, err_msg=f"tensor {i}")
            np.testing.assert_allclose(gt["w"].cpu().numpy(), s["w"], rtol=2e-6, atol=1e-7, err_msg=f"tensor {i}")


def test_myadam_optimizer_matches_oracle(oracle):
    from trips_amd.adam import MyAdam
    rng = np.random.default_rng(1)
    n = 5000
    w0 = rng.normal(0, 1, (4, n)).astype(np.float32)
    p0 = rng.normal(0, 1, (7, 6))
    w = torch.nn.Parameter(torch.as_tensor(w0).cuda())
    pose = torch.nn.Parameter(torch.as_tensor(p0).cuda())
    opt = MyAdam([{"params": [w], "lr": 1e-2}, {"params": [pose], "lr": 1e-3}])
    ref_w = dict(w=w0.copy().reshape(-1), g=None, m=np.zeros(4 * n, np.float32), v=np.zeros(4 * n, np.float32),
                 steps=np.zeros(4 * n, np.int64), n=4 * n, lr=1e-2)
    ref_p = dict(w=p0.copy().reshape(-1), g=None, m=np.zeros(42, np.float32), v=np.zeros(42, np.float32),
                 steps=np.zeros(42, np.int64), n=42, lr=1e-3, dtype=abi.TRIPS_DTYPE_F64)
    for _ in range(3):
        gw = rng.normal(0, 1, (4, n)).astype(np.float32)
        gw[:, rng.random(n) < 0.5] = 0
        gp = rng.normal(0, 1, (7, 6))
        w.grad = torch.as_tensor(gw).cuda()
        pose.grad = torch.as_tensor(gp).cuda()
        opt.step()
        ref_w["g"], ref_p["g"] = gw.reshape(-1), gp.reshape(-1)
        oracle.adam_step([ref_w, ref_p])
    torch.cuda.synchronize()
    np.testing.assert_allclose(w.detach().cpu().numpy().reshape(-1), ref_w["w"], rtol=2e-6, atol=1e-7)
    np.testing.assert_allclose(pose.detach().cpu().numpy().reshape(-1), ref_p["w"], rtol=2e-6, atol=1e-9)
    # state shrink / append follow the last dimension (MyAdam.cu:346-415)
    keep = torch.arange(0, n, 2)
    opt.shrinkInternalState(0, keep)
    assert opt.state[w]["first_moments"].shape == (4, n // 2)
    opt.appendToInternalState(0, n)
    assert opt.state[w]["param_steps"].shape == (4, n) and int(opt.state[w]["param_steps"][:, n // 2:].sum()) == 0


def _point_params(n, c, rng, dev="cuda"):
    shapes = [(n, 4), (n, 1), (c, n), (1, n)]
    return [rng.normal(0, 1, s).astype(np.float32) for s in shapes]


def _point_grads(n, c, rng, dead_frac):
    g = _point_params(n, c, rng)
    dead = rng.random(n) < dead_frac
    g[0][:, 3] = 0            # the drop-out radius in position.w is never trained
    g[0][dead] = 0
    g[1][dead] = 0
    g[2][:, dead] = 0
    g[3][:, dead] = 0
    g[2][0, ::7] = 0          # single elements of live points that are not seen
    g[0][::11, 1] = 0
    return g


@pytest.mark.parametrize("n,c", [(1000, 4), (70001, 3), (5003, 6), (3000, 8), (2000, 16), (63, 4), (1, 4), (6_000_000, 4)])
def test_packed_point_adam_equals_per_tensor_adam(oracle, n, c):
    """MyAdamPoints (state packed per point, trips_adam_step_points) against MyAdam (trips_adam_step_fused) with
    different options per tensor, points without gradient, single elements without gradient, a step in which one of
    the four tensors has no gradient at all, and one further parameter outside the packed four: weights, moments and
    counters bit for bit; and, through the per-tensor optimiser, against the oracle."""
    from trips_amd.adam import MyAdam, MyAdamPoints
    rng = np.random.default_rng(n + c)
    w0 = _point_params(n, c, rng)
    extra0 = rng.normal(0, 1, (7, 6))
    groups = lambda ps, ex: [{"params": [ps[0]], "lr": 1e-3}, {"params": [ps[1]], "lr": 2e-3, "adabound": True},
                             {"params": [ps[2]], "lr": 5e-3, "weight_clipping_magnitude": 1.5},
                             {"params": [ps[3]], "lr": 1e-2, "relative_weight_decay": 0.01, "absolute_weight_decay": 1e-4},
                             {"params": [ex], "lr": 1e-3}]
    pa = [torch.nn.Parameter(torch.as_tensor(x).cuda()) for x in w0]
    pb = [torch.nn.Parameter(torch.as_tensor(x).cuda()) for x in w0]
    ea, eb = (torch.nn.Parameter(torch.as_tensor(extra0).cuda()) for _ in range(2))
    plain = MyAdam(groups(pa, ea))
    packed = MyAdamPoints(groups(pb, eb), *pb)
    ref = [dict(w=x.copy().reshape(-1), g=None, m=np.zeros(x.size, np.float32), v=np.zeros(x.size, np.float32),
                steps=np.zeros(x.size, np.int64), n=x.size) for x in w0]
    ref[0].update(lr=1e-3)
    ref[2].update(lr=5e-3, weight_clipping_magnitude=1.5)
    ref[3].update(lr=1e-2, relative_weight_decay=0.01, absolute_weight_decay=1e-4)
    for step in range(4):
        g = _point_grads(n, c, rng, 0.4)
        ge = rng.normal(0, 1, (7, 6))
        for ps, ex in ((pa, ea), (pb, eb)):
            for p, gi in zip(ps, g):
                p.grad = torch.as_tensor(gi).cuda()
            ex.grad = torch.as_tensor(ge).cuda()
            if step == 2:
                ps[1].grad = None  # the sizes are not optimised in this step
        plain.step()
        packed.step()
        if n <= 100_000:  # (the scalar oracle: small sizes only; the per-tensor kernel is pinned by it at any size)
            for i in (0, 2, 3):  # (the sizes, with their AdaBound bounds and the step they sit out, are pinned by `plain`)
                ref[i]["g"] = g[i].reshape(-1)
            oracle.adam_step([ref[0], ref[2], ref[3]])
    torch.cuda.synchronize()
    for a, b in zip(pa + [ea], pb + [eb]):
        assert torch.equal(a.data, b.data)
    for a, b in zip(pa, pb):
        sa, sb = plain.state[a], packed.unpacked_state(b)
        for k in ("first_moments", "second_moments"):
            assert torch.equal(sa[k], sb[k]), k
        assert torch.equal(sa["param_steps"].to(torch.int32), sb["param_steps"])
    if n <= 100_000:
        for i in (0, 2, 3):
            np.testing.assert_allclose(pb[i].detach().cpu().numpy().reshape(-1), ref[i]["w"], rtol=2e-6, atol=1e-7)
    if n < 4:
        return
    # point removal / addition: the rows follow the group of the descriptors; one more step must agree again
    # (the per-tensor state of positions and sizes, whose last dimension is not the point, is cut by hand)
    keep = torch.arange(0, n, 2)
    m = int(keep.numel())
    for p in pa[:2]:
        for k in ("first_moments", "second_moments", "param_steps"):
            plain.state[p][k] = plain.state[p][k][keep.cuda()].contiguous()
    for opt, ps in ((plain, pa), (packed, pb)):
        for gi in (2, 3):
            opt.shrinkInternalState(gi, keep)
        ps[0].data = ps[0].data[keep.cuda()].contiguous()
        ps[1].data = ps[1].data[keep.cuda()].contiguous()
        ps[2].data = ps[2].data[:, keep.cuda()].contiguous()
        ps[3].data = ps[3].data[:, keep.cuda()].contiguous()
    assert packed.packed_state.shape[0] == m
    g = _point_grads(m, c, rng, 0.4)
    for opt, ps in ((plain, pa), (packed, pb)):
        for p, gi in zip(ps, g):
            p.grad = torch.as_tensor(gi).cuda()
        opt.step()
    for a, b in zip(pa, pb):
        assert torch.equal(a.data, b.data)
        assert torch.equal(plain.state[a]["second_moments"], packed.unpacked_state(b)["second_moments"])
    for opt in (plain, packed):
        for gi in (2, 3):
            opt.appendToInternalState(gi, m + 5)
    assert packed.packed_state.shape[0] == m + 5 and int(packed.packed_state[m:].abs().sum()) == 0


def test_packed_point_adam_state_dict_round_trip():
    """A checkpoint of MyAdamPoints carries the rows of the four point parameters: an optimiser restored from
    state_dict() continues bit for bit like the one that never stopped."""
    from trips_amd.adam import MyAdamPoints
    n, c = 4001, 4
    rng = np.random.default_rng(12)
    w0 = _point_params(n, c, rng)
    mk = lambda: [torch.nn.Parameter(torch.as_tensor(x).cuda()) for x in w0]
    groups = lambda ps: [{"params": [ps[0]], "lr": 1e-3}, {"params": [ps[1]], "lr": 2e-3, "adabound": True},
                         {"params": [ps[2]], "lr": 5e-3}, {"params": [ps[3]], "lr": 1e-2}]
    pa = mk()
    a = MyAdamPoints(groups(pa), *pa)
    grads = [_point_grads(n, c, rng, 0.4) for _ in range(4)]
    for step in range(2):
        for p, g in zip(pa, grads[step]):
            p.grad = torch.as_tensor(g).cuda()
        a.step()
    sd = a.state_dict()
    assert sd["packed_state"] is not None and sd["packed_state"].shape[0] == n
    pb = [torch.nn.Parameter(p.detach().clone()) for p in pa]
    b = MyAdamPoints(groups(pb), *pb)
    b.load_state_dict(sd)
    for step in range(2, 4):
        for opt, ps in ((a, pa), (b, pb)):
            for p, g in zip(ps, grads[step]):
                p.grad = torch.as_tensor(g).cuda()
            opt.step()
    torch.cuda.synchronize()
    for x, y in zip(pa, pb):
        assert torch.equal(x.data, y.data)
    assert torch.equal(a.packed_state, b.packed_state)


def test_packed_point_adam_argument_checks():
    from trips_amd import _lib
    from trips_amd.renderer import get_context
    ctx = get_context(0)
    nbytes, row = ctx.adam_points_state_size(1000, 4)
    assert row == 128 and nbytes == 1000 * 128
    assert ctx.adam_points_state_size(10, 16)[1] == 384
    with pytest.raises(_lib.TripsError):
        ctx.adam_points_state_size(10, 5)
    w = [torch.zeros(s, device="cuda") for s in ((8, 4), (8,), (4, 8), (8,))]
    state = torch.zeros(8 * 32, dtype=torch.int32, device="cuda")

    def descs(n_pos=32):
        out = []
        for i, x in enumerate(w):
            t = abi.TripsAdamTensor()
            t.weights, t.grads, t.n, t.dtype = x.data_ptr(), x.data_ptr(), (n_pos if i == 0 else x.numel()), abi.TRIPS_DTYPE_F32
            t.lr, t.beta1, t.beta2, t.eps, t.loss_scale, t.upper_lr_bound = 1e-3, 0.9, 0.999, 1e-8, 1.0, abi.FLT_MAX
            out.append(t)
        return out
    ctx.adam_step_points(descs(), 8, 4, state)  # zero gradients: nothing happens
    torch.cuda.synchronize()
    assert int(state.abs().sum()) == 0
    with pytest.raises(_lib.TripsError):
        ctx.adam_step_points(descs(n_pos=31), 8, 4, state)  # position must have 4 N elements


def test_apply_tangent_matches_oracle(oracle):
    from trips_amd.renderer import get_context
    ctx = get_context(0)
    rng = np.random.default_rng(9)
    n = 300
    q = rng.normal(0, 1, (n, 4))
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    poses = np.zeros((n, 8))
    poses[:, :4] = q
    poses[:, 4:7] = rng.normal(0, 1, (n, 3))
    tang = rng.normal(0, 0.3, (n, 6))
    tang[0] = 0
    tang[1, 3:] = 1e-13
    tp, tt = torch.as_tensor(poses).cuda(), torch.as_tensor(tang).cuda()
    ctx.apply_tangent(tt, tp)
    torch.cuda.synchronize()
    oracle.apply_tangent(tang, poses)
    np.testing.assert_allclose(tp.cpu().numpy(), poses, rtol=0, atol=1e-13)
    assert float(tt.abs().max()) == 0.0
