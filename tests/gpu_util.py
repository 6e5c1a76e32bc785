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
                 overwrite=False, clear=False):
        """overwrite: the per-point outputs start as NaN and the call runs with overwrite_point_grads;
        clear: the block sums start as NaN and the call runs with clear_block_sums."""
        d, dev = self.desc, self.ctx.device
        z = lambda shape, dt=torch.float32: torch.zeros(shape, dtype=dt, device=dev)
        big = (lambda shape: torch.full(shape, float("nan"), dtype=torch.float32, device=dev)) if overwrite else z
        zs = (lambda shape, dt=torch.float32: torch.full(shape, float("nan"), dtype=dt, device=dev)) if clear else z
        grads = dict(d_texture=big((d.num_channels, d.num_texels)), d_confidence=big((d.num_texels,)),
                     d_background=zs((d.num_channels,)),
                     d_position=big((d.num_points, 4)) if want_position else None,
                     d_point_size=big((d.num_points,)) if want_point_size else None,
                     d_pose=zs((d.num_images, 6), torch.float64) if want_pose else None,
                     d_intrinsics=zs((d.num_cameras, 13)) if want_intrinsics else None)
        gi = [torch.as_tensor(np.ascontiguousarray(g), dtype=torch.float32).to(dev) for g in grad_images]
        self.ctx.backward(d, self.tin, self.saved, gi, grads, self.workspace, overwrite_point_grads=overwrite,
                          clear_block_sums=clear)
        torch.cuda.synchronize()
        return {k: (None if v is None else v.cpu().numpy()) for k, v in grads.items()}


def rel_err(got, want):
    """Largest difference over the largest magnitude of `want`: the bar for the few block sums that are reduced
    in double and rounded once (pose, intrinsics, background), where no single element is small by cancellation
    of few terms."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    return float(np.abs(got - want).max() / (np.abs(want).max() + 1e-30))


# The per-point gradients are held to a per-element bound: |got - want| <= GRAD_RTOL |want| + GRAD_FLOOR max|want|.
# The floor covers elements that are the difference of much larger terms summed in another order in float.
GRAD_RTOL = 1e-4   # the bar the path is held to: gradients within 1e-4 relative
GRAD_FLOOR = 3e-7  # measured on the full-size configurations: the worst element sits at a tenth of this bound
PER_POINT = ("d_position", "d_point_size", "d_confidence", "d_texture")
REDUCED = ("d_pose", "d_intrinsics", "d_background")


def elementwise_excess(got, want, rtol=GRAD_RTOL, floor=GRAD_FLOOR):
    """max over elements of |got - want| / (rtol |want| + floor max|want|); <= 1 passes."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    if want.size == 0:
        return 0.0
    bound = rtol * np.abs(want) + floor * np.abs(want).max()
    diff = np.abs(got - want)
    if not np.isfinite(got).all():
        return float("inf")
    return float((diff / np.maximum(bound, 1e-300)).max()) if diff.max() > 0 else 0.0


def assert_grad_close(key, got, want, what=""):
    """One gradient tensor, `key` = its name in TripsSplatGrads (decides which bar applies)."""
    assert_grads_close({key: got}, {key: want}, what)


def assert_grads_close(got, want, what=""):
    """Gradient bar of the parity tests: per element for the per-point outputs, largest-magnitude for the block sums."""
    for k, v in want.items():
        if v is None:
            assert got[k] is None, f"{what}{k}: expected no output"
            continue
        if k in PER_POINT:
            ex = elementwise_excess(got[k], v)
            if ex > 1.0:
                g, w = np.asarray(got[k], np.float64), np.asarray(v, np.float64)
                bound = GRAD_RTOL * np.abs(w) + GRAD_FLOOR * np.abs(w).max()
                i = np.unravel_index(np.argmax(np.abs(g - w) / np.maximum(bound, 1e-300)), w.shape)
                n_bad = int((np.abs(g - w) > bound).sum())
                raise AssertionError(f"{what}{k}: {n_bad} of {w.size} elements outside {GRAD_RTOL:g}|want| + "
                                     f"{GRAD_FLOOR:g} max|want|; worst at {i}: got {g[i]:.9g}, want {w[i]:.9g}, "
                                     f"max|want| {np.abs(w).max():.4g}")
        else:
            e = rel_err(got[k], v)
            assert e < GRAD_RTOL, f"{what}{k}: {e:.3e} of the largest magnitude"
