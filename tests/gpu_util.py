"""Helpers shared by the GPU parity tests: upload a scene, run the HIP path through the C ABI."""
import numpy as np
import torch

from trips_amd import abi
from trips_amd.renderer import SplatContext, get_context


class GpuRun:
    def __init__(self, scene, desc, dropout=None):
        self.ctx = get_context(0)
        dev = self.ctx.device
        f = lambda a, dt=torch.float32: torch.as_tensor(np.ascontiguousarray(a), dtype=dt).to(dev).contiguous()
        self.desc = desc
        self.t = dict(position=f(scene.position), point_size=f(scene.point_size), index=f(scene.index, torch.int32),
                      texture=f(scene.texture), confidence=f(scene.confidence), background=f(scene.background),
                      poses_se3=f(scene.poses_se3, torch.float64), intrinsics=f(scene.intrinsics),
                      dropout=None if dropout is None else f(dropout),
                      displacement=None if getattr(scene, "displacement", None) is None else f(scene.displacement))
        self.tin = SplatContext.make_in(**self.t)
        self.workspace = self.ctx.alloc_bytes(self.ctx.workspace_size(desc))
        self.saved = self.ctx.alloc_bytes(self.ctx.saved_size(desc)) if desc.train else None
        self.images = None

    def forward(self):
        self.images = self.ctx.alloc_images(self.desc, fill=float("nan"))
        self.ctx.forward(self.desc, self.tin, self.images, self.saved, self.workspace)
        torch.cuda.synchronize()
        return [im.cpu().numpy() for im in self.images]

    def lists(self, view=0):
        l, r, n = self.ctx.export_lists(self.desc, self.saved, view)
        torch.cuda.synchronize()
        return l.cpu().numpy(), r.cpu().numpy(), n.cpu().numpy()

    def points(self, view=0):
        out = self.ctx.export_points(self.desc, self.saved, view)
        torch.cuda.synchronize()
        return [x.cpu().numpy() for x in out]

    def backward(self, grad_images, want_position=True, want_point_size=True, want_pose=True, want_intrinsics=True,
                 overwrite=False):
        """overwrite: the per-point outputs start as NaN and the call runs with overwrite_point_grads."""
        d, dev = self.desc, self.ctx.device
        z = lambda shape, dt=torch.float32: torch.zeros(shape, dtype=dt, device=dev)
        big = (lambda shape: torch.full(shape, float("nan"), dtype=torch.float32, device=dev)) if overwrite else z
        grads = dict(d_texture=big((d.num_channels, d.num_texels)), d_confidence=big((d.num_texels,)),
                     d_background=z(d.num_channels),
                     d_position=big((d.num_points, 4)) if want_position else None,
                     d_point_size=big((d.num_points,)) if want_point_size else None,
                     d_pose=z((d.num_images, 6), torch.float64) if want_pose else None,
                     d_intrinsics=z((d.num_cameras, 13)) if want_intrinsics else None)
        gi = [torch.as_tensor(np.ascontiguousarray(g), dtype=torch.float32).to(dev) for g in grad_images]
        self.ctx.backward(d, self.tin, self.saved, gi, grads, self.workspace, overwrite_point_grads=overwrite)
        torch.cuda.synchronize()
        return {k: (None if v is None else v.cpu().numpy()) for k, v in grads.items()}


def rel_err(got, want):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    return float(np.abs(got - want).max() / (np.abs(want).max() + 1e-30))
