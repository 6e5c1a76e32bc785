"""On-disk formats (C++ host side, trips_amd/csrc/torch_shim/trips_scene_io.cpp): checkpoint archives with the
reference's registered tensor names, poses.txt, camera ini files, PLY point clouds, the scene directory. CPU only."""
import os
import struct
import zipfile

import numpy as np
import pytest
import torch


def _m():
    from trips_amd import _trips_torch
    return _trips_torch


def _scene_tensors(n=50, c=4, frames=3, cams=2, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(frames, 4, generator=g, dtype=torch.float64)
    q = q / q.norm(dim=1, keepdim=True)
    poses = torch.zeros(frames, 8, dtype=torch.float64)
    poses[:, :4] = q
    poses[:, 4:7] = torch.randn(frames, 3, generator=g, dtype=torch.float64)
    return dict(position=torch.randn(n, 4, generator=g), point_size=torch.randn(n, 1, generator=g),
                index=torch.arange(n, dtype=torch.int32).reshape(n, 1), color=torch.rand(n, 4, generator=g),
                texture=torch.randn(c, n, generator=g), background=torch.rand(c, generator=g),
                confidence=torch.randn(1, n, generator=g), poses_se3=poses, intrinsics=torch.rand(cams, 13, generator=g))


def test_checkpoint_round_trip_and_archive_names(tmp_path):
    m = _m()
    t = _scene_tensors()
    m.save_checkpoint(str(tmp_path), "garden", t["position"], t["point_size"], t["index"], t["color"], t["texture"],
                      t["background"], t["confidence"], t["poses_se3"], t["intrinsics"], False)
    files = sorted(os.listdir(tmp_path))
    # NeuralScene::SaveCheckpoint, src/lib/data/NeuralScene.cpp:602-628
    assert files == ["scene_garden_intrinsics.pth", "scene_garden_points.pth", "scene_garden_poses.pth",
                     "scene_garden_poses.txt", "scene_garden_texture.pth"]
    d = m.load_checkpoint(str(tmp_path), "garden", 50, 4, 3, 2)
    assert d["archives_loaded"] == 4
    # registered names: NeuralPointCloudCuda.cpp:103-108, NeuralTexture.cpp:53-55, NeuralStructure.cpp:34-35,142
    want = {"points.t_position": t["position"], "points.t_point_size": t["point_size"], "points.t_index": t["index"],
            "points.t_original_color": t["color"], "texture.texture": t["texture"],
            "texture.background_color": t["background"], "texture.confidence_value_of_point": t["confidence"],
            "poses.poses_se3": t["poses_se3"], "poses.tangent_poses": torch.zeros(3, 6, dtype=torch.float64),
            "intrinsics.intrinsics": t["intrinsics"]}
    for k, v in want.items():
        assert torch.equal(d[k], v), k
    # what the operator reads: sigmoid(10 * raw), NeuralTexture.h:40-43
    assert torch.allclose(d["texture.prepared_confidence"], torch.sigmoid(10 * t["confidence"]))
    # the archive is libtorch's zip container and names the tensors as registered
    with zipfile.ZipFile(tmp_path / "scene_garden_points.pth") as z:
        blob = b"".join(z.read(n) for n in z.namelist() if n.endswith(".pkl"))
    for name in (b"t_position", b"t_index", b"t_original_color", b"t_point_size"):
        assert name in blob


def test_reduced_checkpoint_skips_the_large_archives(tmp_path):
    m = _m()
    t = _scene_tensors()
    m.save_checkpoint(str(tmp_path), "s", t["position"], t["point_size"], t["index"], t["color"], t["texture"],
                      t["background"], t["confidence"], t["poses_se3"], t["intrinsics"], True)
    assert sorted(os.listdir(tmp_path)) == ["scene_s_intrinsics.pth", "scene_s_poses.pth", "scene_s_poses.txt"]
    d = m.load_checkpoint(str(tmp_path), "s", 50, 4, 3, 2)
    assert d["archives_loaded"] == 2 and torch.equal(d["points.t_position"], torch.zeros(50, 4))


def _quat_to_mat(q):
    x, y, z, w = q
    return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - z * w), 2 * (x * z + y * w)],
                     [2 * (x * y + z * w), 1 - 2 * (x * x + z * z), 2 * (y * z - x * w)],
                     [2 * (x * z - y * w), 2 * (y * z + x * w), 1 - 2 * (x * x + y * y)]])


def test_poses_txt_is_the_inverse_of_the_pose_buffer(tmp_path):
    """poses.txt holds camera -> world (scenes/README.md:92-94), the module world -> camera
    (NeuralStructure.cpp:20-35): composing the two must give the identity."""
    m = _m()
    t = _scene_tensors(frames=4, seed=3)
    m.save_checkpoint(str(tmp_path), "p", t["position"], t["point_size"], t["index"], t["color"], t["texture"],
                      t["background"], t["confidence"], t["poses_se3"], t["intrinsics"], True)
    c2w = np.array(m.load_poses(str(tmp_path / "scene_p_poses.txt")))
    assert c2w.shape == (4, 7)
    for i in range(4):
        Rw, tw = _quat_to_mat(t["poses_se3"][i, :4].numpy()), t["poses_se3"][i, 4:7].numpy()
        Rc, tc = _quat_to_mat(c2w[i, :4]), c2w[i, 4:7]
        np.testing.assert_allclose(Rw @ Rc, np.eye(3), atol=1e-12)
        np.testing.assert_allclose(Rw @ tc + tw, 0, atol=1e-12)


def _write_ply(path, xyz, normals, colors, binary):
    n = xyz.shape[0]
    head = ["ply", "format " + ("binary_little_endian" if binary else "ascii") + " 1.0", f"element vertex {n}",
            "property float x", "property float y", "property float z"]
    if normals is not None:
        head += ["property float nx", "property float ny", "property float nz"]
    if colors is not None:
        head += ["property uchar red", "property uchar green", "property uchar blue"]
    head += ["element face 0", "property list uchar int vertex_indices", "end_header"]
    with open(path, "wb") as f:
        f.write(("\n".join(head) + "\n").encode())
        for i in range(n):
            vals = list(xyz[i]) + (list(normals[i]) if normals is not None else [])
            if binary:
                f.write(struct.pack("<%df" % len(vals), *vals))
                if colors is not None:
                    f.write(struct.pack("<3B", *colors[i]))
            else:
                row = " ".join(repr(float(v)) for v in vals)
                if colors is not None:
                    row += " " + " ".join(str(int(c)) for c in colors[i])
                f.write((row + "\n").encode())


@pytest.mark.parametrize("binary", [False, True])
def test_scene_directory(tmp_path, binary):
    m = _m()
    rng = np.random.default_rng(1)
    scene = tmp_path / "my_dataset"
    scene.mkdir()
    xyz = rng.normal(size=(20, 3)).astype(np.float32)
    nrm = rng.normal(size=(20, 3)).astype(np.float32)
    col = rng.integers(0, 256, size=(20, 3))
    _write_ply(scene / "point_cloud.ply", xyz, nrm, col, binary)
    (scene / "dataset.ini").write_text("[SceneDatasetParams]\nfile_point_cloud = point_cloud.ply\n"
                                       "camera_files = camera0.ini camera1.ini   # two cameras\n")
    K0, K1 = [500.0, 501.0, 320.0, 240.0, 0.0], [1400.0, 1400.0, 960.0, 540.0, 0.5]
    dist = [0.1, -0.05, 0.01, 0.02, 0.01, -0.005, 0.003, -0.002]
    m.save_camera(str(scene / "camera0.ini"), 640, 480, K0, [0.0] * 8)
    m.save_camera(str(scene / "camera1.ini"), 1920, 1080, K1, dist)
    q = rng.normal(size=(3, 4))
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    tr = rng.normal(size=(3, 3))
    m.save_poses(str(scene / "poses.txt"), [list(q[i]) + list(tr[i]) for i in range(3)])
    (scene / "images.txt").write_text("0000.jpg\n0001.jpg\n0002.jpg\n")
    (scene / "camera_indices.txt").write_text("0\n1\n0\n")

    d = m.load_scene(str(scene))
    assert d["scene_name"] == "my_dataset" and d["image_names"] == ["0000.jpg", "0001.jpg", "0002.jpg"]
    assert d["camera_indices"] == [0, 1, 0] and d["camera_sizes"] == [(640, 480), (1920, 1080)]
    want_k = np.array([K0 + [0.0] * 8, K1 + dist], dtype=np.float32)
    np.testing.assert_array_equal(d["intrinsics"].numpy(), want_k)
    np.testing.assert_array_equal(d["point_position"].numpy(), xyz)
    np.testing.assert_array_equal(d["point_normal"].numpy(), nrm)
    np.testing.assert_allclose(d["point_color"].numpy()[:, :3], col / 255.0, atol=1e-7)
    assert (d["point_color"].numpy()[:, 3] == 1).all()
    # world -> camera rows: inverse of the camera -> world poses of the file
    se3 = d["poses_se3"].numpy()
    assert se3.shape == (3, 8) and (se3[:, 7] == 0).all()
    for i in range(3):
        Rc, Rw = _quat_to_mat(q[i]), _quat_to_mat(se3[i, :4])
        np.testing.assert_allclose(Rw @ Rc, np.eye(3), atol=1e-12)
        np.testing.assert_allclose(Rw @ tr[i] + se3[i, 4:7], 0, atol=1e-12)


def test_scene_directory_errors(tmp_path):
    m = _m()
    with pytest.raises(RuntimeError):
        m.load_scene(str(tmp_path))  # no dataset.ini
    (tmp_path / "dataset.ini").write_text("camera_files = camera.ini\n")
    (tmp_path / "camera.ini").write_text("w = 10\nh = 10\n")  # K missing
    with pytest.raises(RuntimeError):
        m.load_scene(str(tmp_path))


def test_network_archive_names(tmp_path):
    """torch::save of the C++ net keeps the reference's module hierarchy (Networks.h:751-787, 999-1118)."""
    m = _m()
    s = m.UnetSession([16, 32, 64, 64], 4, 4)
    names = [n for n, _ in s.named_parameters()]
    assert names[:4] == ["start.conv.feature_transform.0.weight", "start.conv.feature_transform.0.bias",
                         "start.conv.mask_transform.0.weight", "start.conv.mask_transform.0.bias"]
    assert "up1.convolution.feature_transform.0.weight" in names and "up3.convolution.mask_transform.0.bias" in names
    assert names[-2:] == ["final.0.weight", "final.0.bias"]
    shapes = {n: tuple(t.shape) for n, t in s.named_parameters()}
    assert shapes["start.conv.feature_transform.0.weight"] == (56, 4, 3, 3)
    assert shapes["up3.convolution.feature_transform.0.weight"] == (56, 64, 3, 3)
    assert shapes["up2.convolution.feature_transform.0.weight"] == (24, 64, 3, 3)
    assert shapes["up1.convolution.feature_transform.0.weight"] == (12, 32, 3, 3)
    assert shapes["final.0.weight"] == (3, 16, 1, 1)
    # same names as the Python mirror
    from trips_amd.unet import MultiScaleUnet2dDecOnlySmallFixed, MultiScaleUnet2dParams
    py = MultiScaleUnet2dDecOnlySmallFixed(MultiScaleUnet2dParams(num_input_layers=4, num_layers=4,
                                                                  filters_network=[16, 32, 64, 64]))
    assert sorted(n for n, _ in py.named_parameters()) == sorted(names)
    s.save(str(tmp_path / "net.pth"))
    s2 = m.UnetSession([16, 32, 64, 64], 4, 4)
    s2.load(str(tmp_path / "net.pth"))
    for (n1, a), (n2, b) in zip(s.named_parameters(), s2.named_parameters()):
        assert n1 == n2 and torch.equal(a, b)
