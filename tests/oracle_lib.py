"""ctypes front-end of oracle/liboracle.so (the CPU oracle). Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

from trips_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(ROOT, "oracle", "liboracle.so")


class OracleForwardOut(C.Structure):
    _fields_ = [
        ("image", C.c_void_p * abi.TRIPS_MAX_LAYERS),
        ("ip", C.c_void_p),
        ("depth", C.c_void_p),
        ("size_px", C.c_void_p),
        ("max_layer", C.c_void_p),
        ("lengths", C.c_void_p),
        ("lists", C.c_void_p),
        ("retained", C.c_void_p),
        ("alpha", C.c_void_p),
        ("counters", C.c_void_p),
    ]


def build():
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "-s"])


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


class Oracle:
    def __init__(self, lib):
        self.lib = lib
        lib.oracle_softplus.restype = C.c_float
        lib.oracle_softplus.argtypes = [C.c_float]
        lib.oracle_softplus_backward.restype = C.c_float
        lib.oracle_softplus_backward.argtypes = [C.c_float]
        lib.oracle_layer_factor.restype = C.c_float
        lib.oracle_layer_factor.argtypes = [C.c_float, C.c_int, C.c_int, C.POINTER(C.c_float)]
        lib.oracle_log2_floor_ceil.restype = None
        lib.oracle_log2_floor_ceil.argtypes = [C.c_float, C.POINTER(C.c_int), C.POINTER(C.c_int)]
        lib.oracle_num_threads.restype = C.c_int
        lib.oracle_set_num_threads.argtypes = [C.c_int]
        lib.oracle_splat_forward.restype = C.c_int
        lib.oracle_splat_backward.restype = C.c_int
        lib.oracle_adam_step.restype = C.c_int
        lib.oracle_apply_tangent.restype = C.c_int

    # ---- scalar pieces ----
    def softplus(self, x):
        return float(self.lib.oracle_softplus(float(x)))

    def softplus_backward(self, x):
        return float(self.lib.oracle_softplus_backward(float(x)))

    def layer_factor(self, s, layer, num_layers):
        g = C.c_float(0)
        f = self.lib.oracle_layer_factor(float(s), int(layer), int(num_layers), C.byref(g))
        return float(f), float(g.value)

    def log2_floor_ceil(self, s):
        lo, hi = C.c_int(0), C.c_int(0)
        self.lib.oracle_log2_floor_ceil(float(s), C.byref(lo), C.byref(hi))
        return lo.value, hi.value

    def num_threads(self):
        return int(self.lib.oracle_num_threads())

    def set_num_threads(self, n):
        self.lib.oracle_set_num_threads(int(n))

    def project_point(self, pose, intr, view, dist_cutoff, xyz):
        pose = np.ascontiguousarray(pose, dtype=np.float64)
        intr = np.ascontiguousarray(intr, dtype=np.float32)
        xyz = np.ascontiguousarray(xyz, dtype=np.float32)
        out = np.zeros(4, dtype=np.float32)
        self.lib.oracle_project_point(_ptr(pose), _ptr(intr), C.byref(view), C.c_float(dist_cutoff), _ptr(xyz),
                                      _ptr(out))
        return out

    def project_point_backward(self, pose, intr, view, dist_cutoff, xyz, grad2):
        pose = np.ascontiguousarray(pose, dtype=np.float64)
        intr = np.ascontiguousarray(intr, dtype=np.float32)
        xyz = np.ascontiguousarray(xyz, dtype=np.float32)
        grad2 = np.ascontiguousarray(grad2, dtype=np.float32)
        gp, gpose, gk, gd = (np.zeros(n, dtype=np.float32) for n in (3, 6, 5, 8))
        self.lib.oracle_project_point_backward(_ptr(pose), _ptr(intr), C.byref(view), C.c_float(dist_cutoff),
                                               _ptr(xyz), _ptr(grad2), _ptr(gp), _ptr(gpose), _ptr(gk), _ptr(gd))
        return gp, gpose, gk, gd

    # ---- full passes ----
    @staticmethod
    def _inputs(scene, dropout=None):
        disp = getattr(scene, "displacement", None)
        arrs = dict(
            position=np.ascontiguousarray(scene.position, dtype=np.float32),
            point_size=np.ascontiguousarray(scene.point_size, dtype=np.float32),
            index=np.ascontiguousarray(scene.index, dtype=np.int32),
            texture=np.ascontiguousarray(scene.texture, dtype=np.float32),
            confidence=np.ascontiguousarray(scene.confidence, dtype=np.float32),
            background=np.ascontiguousarray(scene.background, dtype=np.float32),
            poses_se3=np.ascontiguousarray(scene.poses_se3, dtype=np.float64),
            intrinsics=np.ascontiguousarray(scene.intrinsics, dtype=np.float32),
            dropout=None if dropout is None else np.ascontiguousarray(dropout, dtype=np.float32),
            displacement=None if disp is None else np.ascontiguousarray(disp, dtype=np.float32),
        )
        tin = abi.TripsSplatIn()
        for k, v in arrs.items():
            setattr(tin, k, _ptr(v))
        return tin, arrs

    def forward(self, scene, desc, dropout=None, want_points=True):
        """Returns a dict: images (list per layer), ip, depth, size_px, max_layer, lengths, lists, retained,
        alpha, counters. Arrays are view-major."""
        tin, keep = self._inputs(scene, dropout)
        sizes, offs, P = abi.pyramid_pixels(desc)
        B, N, K, Cn = desc.num_views, desc.num_points, desc.list_depth, desc.num_channels
        res = {}
        imgs = []
        for (w, h) in sizes:
            shape = (B, Cn, h, w) if desc.layout == abi.TRIPS_LAYOUT_CHW else (B, h, w, Cn)
            imgs.append(np.full(shape, np.nan, dtype=np.float32))
        res["images"] = imgs
        if want_points:
            res["ip"] = np.zeros((B, N, 2), dtype=np.float32)
            res["depth"] = np.zeros((B, N), dtype=np.float32)
            res["size_px"] = np.zeros((B, N), dtype=np.float32)
            res["max_layer"] = np.zeros((B, N), dtype=np.int32)
        res["lengths"] = np.zeros((B, P), dtype=np.int32)
        res["lists"] = np.zeros((B, P, K), dtype=np.int32)
        res["retained"] = np.zeros((B, P), dtype=np.int32)
        res["alpha"] = np.zeros((B, P, K), dtype=np.float32)
        res["counters"] = np.zeros((B, 4), dtype=np.int64)
        out = OracleForwardOut()
        for l, im in enumerate(imgs):
            out.image[l] = im.ctypes.data
        for k in ("ip", "depth", "size_px", "max_layer", "lengths", "lists", "retained", "alpha", "counters"):
            if k in res:
                setattr(out, k, _ptr(res[k]))
        rc = self.lib.oracle_splat_forward(C.byref(desc), C.byref(tin), C.byref(out))
        if rc != 0:
            raise RuntimeError(f"oracle_splat_forward failed: {rc}")
        res["_out"] = out
        res["sizes"], res["offsets"], res["P"] = sizes, offs, P
        return res

    def backward(self, scene, desc, fwd, grad_images, *, want_position=True, want_point_size=True, want_pose=True,
                 want_intrinsics=True, dropout=None):
        tin, keep = self._inputs(scene, dropout)
        N, Cn, T = desc.num_points, desc.num_channels, desc.num_texels
        F, Cam = desc.num_images, desc.num_cameras
        g = dict(
            d_texture=np.zeros((Cn, T), dtype=np.float32),
            d_confidence=np.zeros(T, dtype=np.float32),
            d_background=np.zeros(Cn, dtype=np.float32),
            d_position=np.zeros((N, 4), dtype=np.float32) if want_position else None,
            d_point_size=np.zeros(N, dtype=np.float32) if want_point_size else None,
            d_pose=np.zeros((F, 6), dtype=np.float64) if want_pose else None,
            d_intrinsics=np.zeros((Cam, 13), dtype=np.float32) if want_intrinsics else None,
        )
        tg = abi.TripsSplatGrads()
        for k, v in g.items():
            setattr(tg, k, _ptr(v))
        gi = [np.ascontiguousarray(x, dtype=np.float32) for x in grad_images]
        arr = (C.c_void_p * abi.TRIPS_MAX_LAYERS)()
        for l, x in enumerate(gi):
            arr[l] = x.ctypes.data
        rc = self.lib.oracle_splat_backward(C.byref(desc), C.byref(tin), C.byref(fwd["_out"]), arr, C.byref(tg))
        if rc != 0:
            raise RuntimeError(f"oracle_splat_backward failed: {rc}")
        return g

    def adam_step(self, tensors):
        """tensors: list of dicts with numpy arrays w, g, m, v, steps and hyper-parameters (see make_adam_tensor)."""
        arr = (abi.TripsAdamTensor * len(tensors))()
        for i, t in enumerate(tensors):
            fill_adam_tensor(arr[i], t, lambda a: a.ctypes.data)
        rc = self.lib.oracle_adam_step(arr, len(tensors))
        if rc != 0:
            raise RuntimeError(f"oracle_adam_step failed: {rc}")

    def apply_tangent(self, tangent, poses):
        assert tangent.dtype == np.float64 and poses.dtype == np.float64
        rc = self.lib.oracle_apply_tangent(_ptr(tangent), _ptr(poses), int(tangent.shape[0]))
        if rc != 0:
            raise RuntimeError("oracle_apply_tangent failed")


def fill_adam_tensor(dst, t, addr):
    """Fill a TripsAdamTensor from a dict; `addr` maps an array/tensor to its address."""
    dst.weights = addr(t["w"])
    dst.grads = addr(t["g"])
    dst.first_moment = addr(t["m"])
    dst.second_moment = addr(t["v"])
    dst.steps = addr(t["steps"])
    dst.n = int(t["n"])
    dst.dtype = int(t.get("dtype", abi.TRIPS_DTYPE_F32))
    dst.lr = t.get("lr", 1e-3)
    dst.beta1 = t.get("beta1", 0.9)
    dst.beta2 = t.get("beta2", 0.999)
    dst.eps = t.get("eps", 1e-8)
    dst.relative_weight_decay = t.get("relative_weight_decay", 0.0)
    dst.absolute_weight_decay = t.get("absolute_weight_decay", 0.0)
    dst.weight_clipping_magnitude = t.get("weight_clipping_magnitude", 0.0)
    dst.lower_lr_bound = t.get("lower_lr_bound", 0.0)
    dst.upper_lr_bound = t.get("upper_lr_bound", abi.FLT_MAX)
    dst.loss_scale = t.get("loss_scale", 1.0)
    dst.steps_dtype = int(t.get("steps_dtype", abi.TRIPS_STEPS_I64))


_cached = None


def load():
    global _cached
    if _cached is None:
        if not os.path.exists(LIB_PATH):
            build()
        _cached = Oracle(C.CDLL(LIB_PATH))
    return _cached
