"""Writes tests/golden/splat_small.npz: inputs of a small seeded scene and the CPU oracle's outputs for it
(forward in both background modes, backward, one Adam step). The inputs are stored, not regenerated, because
numpy's exp/log differ in the last bit between CPU generations.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from tests import oracle_lib  # noqa: E402
from trips_amd import abi, scenes  # noqa: E402


def build_scene():
    sc = scenes.tiny(n=2000, w=48, h=40, f=45.0, num_layers=3, list_depth=16, seed=4242, views=2, radius=(0.004, 0.4))
    sc.confidence = (sc.confidence ** 0.3).astype(np.float32)
    sc.intrinsics[0, 4] = 0.25
    sc.views[1]["crop_transform"] = (1.25, 1.5, -6.0, 3.0, 0.0)
    return sc


def main():
    oracle = oracle_lib.load()
    sc = build_scene()
    out = dict(position=sc.position, point_size=sc.point_size, index=sc.index, texture=sc.texture,
               confidence=sc.confidence, background=sc.background, poses_se3=sc.poses_se3, intrinsics=sc.intrinsics,
               crop_transform_1=np.array(sc.views[1]["crop_transform"], dtype=np.float32))
    rng = np.random.default_rng(99)
    for mode, tag in ((abi.TRIPS_BG_REFERENCE, "ref"), (abi.TRIPS_BG_CONSISTENT, "con")):
        d = abi.desc_for_scene(sc, background_mode=mode)
        fwd = oracle.forward(sc, d)
        for l, im in enumerate(fwd["images"]):
            out[f"image_{tag}_{l}"] = im
        if mode == abi.TRIPS_BG_REFERENCE:
            for k in ("ip", "depth", "size_px", "max_layer", "lengths", "lists", "retained", "counters"):
                out[k] = fwd[k]
            grads = [rng.normal(0, 1, im.shape).astype(np.float32) for im in fwd["images"]]
            for l, g in enumerate(grads):
                out[f"grad_image_{l}"] = g
            g = oracle.backward(sc, d, fwd, grads)
            for k, v in g.items():
                out[k] = v
            t = dict(w=sc.position.reshape(-1).copy(), g=g["d_position"].reshape(-1), m=np.zeros(sc.position.size, np.float32),
                     v=np.zeros(sc.position.size, np.float32), steps=np.zeros(sc.position.size, np.int64),
                     n=sc.position.size, lr=1e-3)
            oracle.adam_step([t])
            out["adam_position"] = t["w"]
            out["adam_steps"] = t["steps"]
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "splat_small.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
