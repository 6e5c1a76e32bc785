"""Seeded synthetic scenes for tests and bench.py.

All inputs come from numpy's counter-based Philox generator, so a CPU check and the GPU path
consume bit-identical host arrays. Layouts follow the reference's tensors:
  position   [N,4] f32  xyz + drop-out radius        (src/lib/rendering/NeuralPointCloudCuda.cpp:62)
  point_size [N]   f32  raw, softplus applied inside (NeuralPointCloudCuda.cpp:19-24,50)
  index      [N]   i32  descriptor column            (NeuralPointCloudCuda.cpp:43,86)
  texture    [C,N] f32, confidence [N] f32 in (0,1), background [C] f32
  poses_se3  [F,8] f64  quaternion xyzw, translation, pad; world->camera (src/lib/data/NeuralStructure.cpp:20-35)
  intrinsics [Cam,13] f32 fx fy cx cy s + 8 distortion coefficients     (NeuralStructure.cpp:104-117)
"""
from dataclasses import dataclass, field
from typing import List

import numpy as np


def _rng(seed):
    return np.random.Generator(np.random.Philox(seed))


def inverse_softplus(x):
    """raw value whose softplus is x (NeuralPointCloudCuda.cpp:19-24)."""
    x = np.asarray(x, dtype=np.float64)
    return np.where(x > 20.0, x, np.log(np.expm1(x)))


def rotmat_to_quat_xyzw(R):
    """Unit quaternion (x, y, z, w) of a proper rotation matrix."""
    R = np.asarray(R, dtype=np.float64)
    t = np.trace(R)
    if t > 0:
        s = np.sqrt(t + 1.0) * 2
        w = 0.25 * s
        x = (R[2, 1] - R[1, 2]) / s
        y = (R[0, 2] - R[2, 0]) / s
        z = (R[1, 0] - R[0, 1]) / s
    elif R[0, 0] > R[1, 1] and R[0, 0] > R[2, 2]:
        s = np.sqrt(1.0 + R[0, 0] - R[1, 1] - R[2, 2]) * 2
        w = (R[2, 1] - R[1, 2]) / s
        x = 0.25 * s
        y = (R[0, 1] + R[1, 0]) / s
        z = (R[0, 2] + R[2, 0]) / s
    elif R[1, 1] > R[2, 2]:
        s = np.sqrt(1.0 + R[1, 1] - R[0, 0] - R[2, 2]) * 2
        w = (R[0, 2] - R[2, 0]) / s
        x = (R[0, 1] + R[1, 0]) / s
        y = 0.25 * s
        z = (R[1, 2] + R[2, 1]) / s
    else:
        s = np.sqrt(1.0 + R[2, 2] - R[0, 0] - R[1, 1]) * 2
        w = (R[1, 0] - R[0, 1]) / s
        x = (R[0, 2] + R[2, 0]) / s
        y = (R[1, 2] + R[2, 1]) / s
        z = 0.25 * s
    q = np.array([x, y, z, w])
    return q / np.linalg.norm(q)


def look_at_pose(eye, target, up=(0.0, -1.0, 0.0)):
    """World->camera pose row (8 doubles) of a camera at `eye` looking at `target`;
    camera axes: +z forward, +x right, +y down (image rows grow downwards)."""
    eye = np.asarray(eye, dtype=np.float64)
    fwd = np.asarray(target, dtype=np.float64) - eye
    fwd /= np.linalg.norm(fwd)
    upv = np.asarray(up, dtype=np.float64)
    right = np.cross(fwd, upv)
    if np.linalg.norm(right) < 1e-9:
        right = np.cross(fwd, np.array([1.0, 0.0, 0.0]))
    right /= np.linalg.norm(right)
    down = np.cross(fwd, right)
    R = np.stack([right, down, fwd], axis=0)  # rows = camera axes in world coordinates
    t = -R @ eye
    q = rotmat_to_quat_xyzw(R)
    return np.array([q[0], q[1], q[2], q[3], t[0], t[1], t[2], 0.0])


@dataclass
class Scene:
    name: str
    position: np.ndarray
    point_size: np.ndarray
    index: np.ndarray
    texture: np.ndarray
    confidence: np.ndarray
    background: np.ndarray
    poses_se3: np.ndarray
    intrinsics: np.ndarray
    views: List[dict]
    num_layers: int
    list_depth: int
    seed: int = 0
    extra: dict = field(default_factory=dict)

    @property
    def num_points(self):
        return int(self.position.shape[0])

    @property
    def num_channels(self):
        return int(self.texture.shape[0])

    @property
    def width(self):
        return self.views[0]["w"]

    @property
    def height(self):
        return self.views[0]["h"]


def _intrinsics(w, h, f):
    k = np.zeros((1, 13), dtype=np.float32)
    k[0, :5] = [f, f, w / 2.0, h / 2.0, 0.0]
    return k


def _finish(name, xyz, radius, rng, *, w, h, f, poses, num_layers, list_depth, channels=4, background=0.25, seed=0):
    n = xyz.shape[0]
    position = np.empty((n, 4), dtype=np.float32)
    position[:, :3] = xyz
    position[:, 3] = radius
    point_size = inverse_softplus(radius).astype(np.float32)
    texture = rng.random((channels, n), dtype=np.float32)
    confidence = rng.random(n, dtype=np.float32)
    confidence = np.clip(confidence, 1e-6, 1.0 - 1e-6).astype(np.float32)
    poses = np.asarray(poses, dtype=np.float64).reshape(-1, 8)
    views = [dict(w=w, h=h, image_index=i, camera_index=0) for i in range(poses.shape[0])]
    return Scene(name=name, position=position, point_size=point_size, index=np.arange(n, dtype=np.int32),
                 texture=texture, confidence=confidence, background=np.full(channels, background, dtype=np.float32),
                 poses_se3=poses, intrinsics=_intrinsics(w, h, f), views=views, num_layers=num_layers,
                 list_depth=list_depth, seed=seed)


def _log_uniform(rng, lo, hi, n):
    return np.exp(rng.uniform(np.log(lo), np.log(hi), n))


def config1(n=100_000, seed=1, w=512, h=512):
    """100k points U[-1,1]^3, 512x512, f=500, camera at z=-3 looking at the origin, radius log-U[1e-3,3e-2],
    4 layers, K=8 (forward only)."""
    rng = _rng(seed)
    xyz = rng.uniform(-1.0, 1.0, (n, 3))
    radius = _log_uniform(rng, 1e-3, 3e-2, n)
    pose = look_at_pose((0, 0, -3), (0, 0, 0))
    return _finish("config1", xyz, radius, rng, w=w, h=h, f=500.0, poses=[pose], num_layers=4, list_depth=8,
                   seed=seed)


def config2(n=1_000_000, seed=2, w=1920, h=1080, f=1400.0):
    """1M points N(0,0.5^2), 1920x1080, f=1400, camera at z=-3, radius log-U[5e-4,5e-2], 8 layers, K=16."""
    rng = _rng(seed)
    xyz = rng.normal(0.0, 0.5, (n, 3))
    radius = _log_uniform(rng, 5e-4, 5e-2, n)
    pose = look_at_pose((0, 0, -3), (0, 0, 0))
    return _finish("config2", xyz, radius, rng, w=w, h=h, f=f, poses=[pose], num_layers=8, list_depth=16,
                   background=0.0, seed=seed)


def _morton_blocks(xyz, rng, block=256):
    """Order of a point cloud after the reference's one-time preprocessing (SceneData.cpp:115-116): sorted along a
    3D Morton curve (21 bits per axis), then blocks of `block` consecutive points shuffled."""
    lo, hi = xyz.min(axis=0), xyz.max(axis=0)
    q = ((xyz - lo) / np.maximum(hi - lo, 1e-30) * (2 ** 21 - 1)).astype(np.uint64)

    def spread(v):  # 21 bits -> every third bit
        v = (v | (v << np.uint64(32))) & np.uint64(0x1F00000000FFFF)
        v = (v | (v << np.uint64(16))) & np.uint64(0x1F0000FF0000FF)
        v = (v | (v << np.uint64(8))) & np.uint64(0x100F00F00F00F00F)
        v = (v | (v << np.uint64(4))) & np.uint64(0x10C30C30C30C30C3)
        v = (v | (v << np.uint64(2))) & np.uint64(0x1249249249249249)
        return v

    code = spread(q[:, 0]) | (spread(q[:, 1]) << np.uint64(1)) | (spread(q[:, 2]) << np.uint64(2))
    order = np.argsort(code, kind="stable")
    nb = (len(order) + block - 1) // block
    blocks = rng.permutation(nb)
    idx = (blocks[:, None] * block + np.arange(block)[None, :]).reshape(-1)
    return order[idx[idx < len(order)]]


def config3(n=6_000_000, seed=3, w=1920, h=1080, f=1400.0, order="random"):
    """6M points: 80% on a noisy ground plane (y ~ N(0,0.02^2), x,z uniform over 20x20), 20% uniform in a
    20x20x5 box above it; camera 1.5 above the plane at its edge, looking at the centre; 8 layers, K=16.
    order: "random" (points in no spatial order) or "morton_blocks" (the order the reference's scene
    preprocessing leaves a cloud in)."""
    rng = _rng(seed)
    n_ground = int(round(0.8 * n))
    n_box = n - n_ground
    ground = np.empty((n_ground, 3))
    ground[:, 0] = rng.uniform(-10.0, 10.0, n_ground)
    ground[:, 1] = rng.normal(0.0, 0.02, n_ground)
    ground[:, 2] = rng.uniform(-10.0, 10.0, n_ground)
    box = np.empty((n_box, 3))
    box[:, 0] = rng.uniform(-10.0, 10.0, n_box)
    box[:, 1] = rng.uniform(-5.0, 0.0, n_box)  # "up" is -y
    box[:, 2] = rng.uniform(-10.0, 10.0, n_box)
    xyz = np.concatenate([ground, box], axis=0)
    perm = rng.permutation(n)
    xyz = xyz[perm]
    if order == "morton_blocks":
        xyz = xyz[_morton_blocks(xyz, _rng(seed + 1000))]
    elif order != "random":
        raise ValueError(f"order {order!r}")
    radius = _log_uniform(rng, 5e-4, 5e-2, n)
    pose = look_at_pose((0.0, -1.5, -10.0), (0.0, 0.0, 0.0))
    return _finish("config3", xyz, radius, rng, w=w, h=h, f=f, poses=[pose], num_layers=8, list_depth=16, seed=seed)


def config4(n=4_000_000, seed=4, w=1245, h=825, f=1000.0, views=4, clusters=64):
    """Contention stress: n points in 64 Gaussian clusters (sigma 0.01), `views` random cameras on a sphere of
    radius 3 around the origin, 1245x825, K=16."""
    rng = _rng(seed)
    centres = rng.uniform(-1.0, 1.0, (clusters, 3))
    which = rng.integers(0, clusters, n)
    xyz = centres[which] + rng.normal(0.0, 0.01, (n, 3))
    radius = _log_uniform(rng, 5e-4, 5e-2, n)
    poses = []
    for _ in range(views):
        d = rng.normal(0.0, 1.0, 3)
        d /= np.linalg.norm(d)
        poses.append(look_at_pose(3.0 * d, (0, 0, 0)))
    return _finish("config4", xyz, radius, rng, w=w, h=h, f=f, poses=poses, num_layers=8, list_depth=16, seed=seed)


def tiny(n=200, seed=7, w=32, h=24, f=30.0, num_layers=3, list_depth=8, views=1, channels=4, background=0.25,
         radius=(0.01, 0.3)):
    """Small scene with dense overlap, for brute-force and finite-difference checks."""
    rng = _rng(seed)
    xyz = rng.uniform(-1.0, 1.0, (n, 3))
    rad = _log_uniform(rng, radius[0], radius[1], n)
    poses = [look_at_pose((0.3 * i, 0.1 * i, -3.0), (0, 0, 0)) for i in range(views)]
    return _finish("tiny", xyz, rad, rng, w=w, h=h, f=f, poses=poses, num_layers=num_layers,
                   list_depth=list_depth, channels=channels, background=background, seed=seed)
