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
