"""Pins the oracle's forward (projection, layer selection, per-pixel lists, blend) without the reference:
textbook pinhole in f64 with scipy's rotation, a global-sort brute force for the lists, an f64 dense
restatement for the blend, closed forms for single points. CPU only."""
import numpy as np
import pytest

from tests import ref_model
from trips_amd import abi, scenes


def _fwd(oracle, sc, **kw):
    d = abi.desc_for_scene(sc, **kw)
    return d, oracle.forward(sc, d)


@pytest.mark.parametrize("views", [1, 3])
def test_projection_matches_textbook_pinhole(oracle, views):
    sc = scenes.tiny(n=3000, w=96, h=64, f=80.0, views=views, seed=11)
    # non-trivial crop transform on the second view
    if views > 1:
        sc.views[1]["crop_transform"] = (1.5, 1.25, -10.0, 4.0, 0.0)
        th = 0.3
        sc.views[2]["crop_rotation"] = (np.cos(th), -np.sin(th), np.sin(th), np.cos(th))
    d, r = _fwd(oracle, sc)
    for b in range(views):
        ip, z, scale = ref_model.project_numpy(sc, d, b)
        valid = r["depth"][b] > 0
        assert valid.sum() > 200
        np.testing.assert_allclose(r["ip"][b][valid], ip[valid], rtol=0, atol=2e-4)
        np.testing.assert_allclose(r["depth"][b][valid], z[valid], rtol=2e-6)
        size = scale * ref_model.softplus64(sc.point_size)
        np.testing.assert_allclose(r["size_px"][b][valid], size[valid], rtol=1e-5)
        # validity: z > 0 and 0 <= ip < size-1 at layer 0 (RenderForward.cu:212-218); leave a margin for rounding
        w, h = sc.width, sc.height
        inside = (z > 1e-6) & (ip[:, 0] > 1e-3) & (ip[:, 0] < w - 1 - 1e-3) & (ip[:, 1] > 1e-3) & (ip[:, 1] < h - 1 - 1e-3)
        outside = (z < -1e-6) | (ip[:, 0] < -1e-3) | (ip[:, 0] > w - 1 + 1e-3) | (ip[:, 1] < -1e-3) | (ip[:, 1] > h - 1 + 1e-3)
        assert np.all(valid[inside])
        assert not np.any(valid[outside])
        assert np.all(r["depth"][b][~valid] == -1)


def test_points_behind_camera_and_borders_are_culled(oracle):
    sc = scenes.tiny(n=8, w=32, h=32, f=30.0, num_layers=2, seed=1)
    # camera at z=-3 looking +z; image centre (16,16)
    sc.position[:, :3] = [[0, 0, -4], [0, 0, -3], [0, 0, 0], [100, 0, 0], [0, -100, 0], [1.5, 0, 0], [1.45, 0, 0],
                          [-1.6, -1.6, 0]]
    d, r = _fwd(oracle, sc)
    depth = r["depth"][0]
    assert depth[0] == -1 and depth[1] == -1  # behind / at the camera plane
    assert depth[2] == pytest.approx(3.0)
    assert depth[3] == -1 and depth[4] == -1
    # x = 1.5 -> ip.x = 30*1.5/3 + 16 = 31 = w-1 -> rejected (ip.x >= w-1); 1.45 -> 30.5 accepted
    assert depth[5] == -1 and depth[6] > 0
    assert r["ip"][0][6, 0] == pytest.approx(30.5, abs=1e-4)
    # ip = (0,0) exactly is accepted (ip.x < 0 is the rejection)
    assert depth[7] > 0 and abs(r["ip"][0][7, 0]) < 1e-4


@pytest.mark.parametrize("seed,L,K", [(5, 3, 8), (6, 4, 16), (7, 1, 16)])
def test_lists_match_global_sort_brute_force(oracle, seed, L, K):
    sc = scenes.tiny(n=1500, w=40, h=28, f=40.0, num_layers=L, list_depth=K, seed=seed, radius=(0.005, 0.6))
    d, r = _fwd(oracle, sc)
    lengths, lists, max_layer = ref_model.build_lists(r["ip"][0], r["depth"][0], r["size_px"][0], d)
    np.testing.assert_array_equal(r["max_layer"][0], max_layer)
    np.testing.assert_array_equal(r["lengths"][0], lengths)
    np.testing.assert_array_equal(r["lists"][0], lists)
    # invariants: 4 entries per point per layer it lands in; counters
    assert lengths.sum() == 4 * max_layer.sum()
    assert r["counters"][0, 1] == lengths.sum()
    assert r["counters"][0, 0] == (r["depth"][0] > 0).sum()
    assert r["counters"][0, 3] == r["P"]
    assert lengths.max() > K  # the top-K cut is exercised
    # lists are sorted by (depth, id)
    dep = r["depth"][0]
    for row in r["lists"][0][::17]:
        ids = row[row >= 0]
        keys = [(dep[i], i) for i in ids]
        assert keys == sorted(keys)


def test_lists_invariant_under_point_permutation(oracle):
    sc = scenes.tiny(n=800, w=36, h=30, f=36.0, num_layers=3, list_depth=8, seed=21)
    d, r = _fwd(oracle, sc)
    rng = np.random.default_rng(5)
    perm = rng.permutation(sc.num_points)
    sc2 = scenes.tiny(n=800, w=36, h=30, f=36.0, num_layers=3, list_depth=8, seed=21)
    sc2.position = sc.position[perm]
    sc2.point_size = sc.point_size[perm]
    sc2.texture = sc.texture[:, perm]
    sc2.confidence = sc.confidence[perm]
    d2, r2 = _fwd(oracle, sc2)
    # depths are unique here, so the sorted lists map onto each other through the permutation
    assert len(np.unique(r["depth"][0][r["depth"][0] > 0])) == (r["depth"][0] > 0).sum()
    mapped = np.where(r2["lists"][0] >= 0, perm[np.clip(r2["lists"][0], 0, None)], -1)
    np.testing.assert_array_equal(mapped, r["lists"][0])
    for a, b in zip(r["images"], r2["images"]):
        np.testing.assert_allclose(a, b, rtol=1e-6, atol=1e-7)


def test_tie_break_is_by_point_id(oracle):
    sc = scenes.tiny(n=6, w=16, h=16, f=30.0, num_layers=1, list_depth=8, seed=2)
    sc.position[:, :3] = [[0.01, 0.01, 0.0]] * 6  # identical depth, same pixel
    d, r = _fwd(oracle, sc)
    px = 8 + 16 * 8
    np.testing.assert_array_equal(r["lists"][0][px][:6], np.arange(6))


@pytest.mark.parametrize("bg_mode", [abi.TRIPS_BG_REFERENCE, abi.TRIPS_BG_CONSISTENT])
@pytest.mark.parametrize("seed,L,K", [(5, 3, 8), (9, 4, 16)])
def test_blend_matches_f64_restatement(oracle, bg_mode, seed, L, K):
    sc = scenes.tiny(n=1500, w=40, h=28, f=40.0, num_layers=L, list_depth=K, seed=seed, radius=(0.005, 0.6))
    d, r = _fwd(oracle, sc, background_mode=bg_mode)
    model = ref_model.Differentiable(sc, d, 0, r["lists"][0], reference_gradient_convention=False)
    img = model.forward().detach().numpy()
    layers = [x.numpy() for x in model.split_layers(__import__("torch").from_numpy(img))]
    for l in range(L):
        np.testing.assert_allclose(r["images"][l][0], layers[l], rtol=1e-5, atol=2e-6)
    np.testing.assert_array_equal(r["retained"][0], model.retained.numpy())
    keep = model.keep.numpy()
    np.testing.assert_allclose(r["alpha"][0][keep], model.alpha.detach().numpy()[keep], rtol=1e-5, atol=1e-5)  # weights inherit ~1e-6 px of float ip rounding
    assert np.all(r["alpha"][0][~keep] == -1)


def test_hwc_layout_is_a_permutation_of_chw(oracle):
    sc = scenes.tiny(n=600, w=24, h=20, f=24.0, num_layers=3, seed=4)
    d1, r1 = _fwd(oracle, sc, train=True)
    d2, r2 = _fwd(oracle, sc, train=False)
    assert d2.layout == abi.TRIPS_LAYOUT_HWC
    for a, b in zip(r1["images"], r2["images"]):
        np.testing.assert_array_equal(a, np.transpose(b, (0, 3, 1, 2)))


def test_single_point_closed_forms(oracle):
    # one point exactly on a pixel centre of layer 0: alpha = conf * layer_factor, colour = alpha*desc + bg*(...)
    sc = scenes.tiny(n=1, w=16, h=16, f=30.0, num_layers=1, list_depth=8, seed=3)
    sc.position[0] = [0.1, -0.2, 0.0, 0.01]  # ip = 30*(0.1,-0.2)/3 + 8 = (9, 6)
    sc.confidence[0] = 0.6
    sc.point_size[0] = scenes.inverse_softplus(0.05)  # size_px = 30*0.05/3 = 0.5
    for mode in (abi.TRIPS_BG_REFERENCE, abi.TRIPS_BG_CONSISTENT):
        d, r = _fwd(oracle, sc, background_mode=mode)
        assert r["ip"][0][0] == pytest.approx([9.0, 6.0], abs=1e-5)
        lf = 0.75 * np.exp(0.5 - 1.0) + 0.25
        # the rounding of ip decides which of the 4 footprint pixels carries the weight; sum over them
        img = r["images"][0][0]
        alpha = 0.6 * lf
        foot = img[:, 5:8, 8:11]
        bgw = 1.0 if mode == abi.TRIPS_BG_REFERENCE else (1 - alpha)
        want = alpha * sc.texture[:, 0] + 0.25 * bgw
        got = img[:, 6, 9]
        np.testing.assert_allclose(got, want, rtol=2e-4)
        # everything outside the 2x2 footprint is pure background
        mask = np.ones((16, 16), bool)
        mask[5:8, 8:11] = False
        assert np.all(img[:, mask] == 0.25)
        del foot


def test_four_corner_weights_sum_to_one(oracle):
    sc = scenes.tiny(n=1, w=16, h=16, f=30.0, num_layers=1, list_depth=8, seed=3, background=0.0)
    sc.position[0] = [0.137, -0.211, 0.0, 0.01]
    sc.confidence[0] = 0.5
    sc.texture[:, 0] = 1.0
    sc.point_size[0] = scenes.inverse_softplus(0.05)
    d, r = _fwd(oracle, sc)
    lf = 0.75 * np.exp(0.5 - 1.0) + 0.25
    img = r["images"][0][0, 0]
    assert (img > 0).sum() == 4
    assert img.sum() == pytest.approx(0.5 * lf, rel=1e-5)
    ipx, ipy = 30 * 0.137 / 3 + 8, 30 * -0.211 / 3 + 8
    fx, fy = ipx - np.floor(ipx), ipy - np.floor(ipy)
    x0, y0 = int(np.floor(ipx)), int(np.floor(ipy))
    np.testing.assert_allclose(img[y0, x0], 0.5 * lf * (1 - fx) * (1 - fy), rtol=1e-4)
    np.testing.assert_allclose(img[y0 + 1, x0 + 1], 0.5 * lf * fx * fy, rtol=1e-4)


def test_two_points_over_compositing(oracle):
    # two points on the same pixel centre, different depth: textbook "over"
    sc = scenes.tiny(n=2, w=16, h=16, f=30.0, num_layers=1, list_depth=8, seed=3, background=0.5)
    sc.position[0] = [0.0, 0.0, 0.5, 0.01]  # farther
    sc.position[1] = [0.0, 0.0, 0.0, 0.01]  # nearer; both project to (8,8)
    sc.confidence[:] = [0.8, 0.4]
    sc.point_size[:] = scenes.inverse_softplus(1e-4)
    lf_near = 0.75 * np.exp(30 * 1e-4 / 3.0 - 1.0) + 0.25
    lf_far = 0.75 * np.exp(30 * 1e-4 / 3.5 - 1.0) + 0.25
    for mode in (abi.TRIPS_BG_REFERENCE, abi.TRIPS_BG_CONSISTENT):
        d, r = _fwd(oracle, sc, background_mode=mode)
        np.testing.assert_array_equal(r["lists"][0][8 * 16 + 8][:3], [1, 0, -1])
        a_near, a_far = 0.4 * lf_near, 0.8 * lf_far
        bgw = (1 - a_near) if mode == abi.TRIPS_BG_REFERENCE else (1 - a_near) * (1 - a_far)
        want = a_near * sc.texture[:, 1] + (1 - a_near) * a_far * sc.texture[:, 0] + 0.5 * bgw
        np.testing.assert_allclose(r["images"][0][0, :, 8, 8], want, rtol=2e-5)


def test_transmittance_cutoff(oracle):
    # 12 points stacked on one pixel centre, alpha = 0.95 each: T = 1, .05, .0025, .000125 -> 3 retained
    # (entries whose exclusive transmittance drops below 0.001 contribute nothing, RenderForward.cu:940-949,959)
    n = 12
    sc = scenes.tiny(n=n, w=16, h=16, f=30.0, num_layers=1, list_depth=16, seed=3, background=0.5)
    sc.position[:, :3] = [[0.0, 0.0, 0.1 * i] for i in range(n)]
    sc.confidence[:] = 0.95
    sc.point_size[:] = scenes.inverse_softplus((3.0 + 0.1 * np.arange(n)) / 30.0)  # size_px = 30*r/z = 1 -> lf = 1
    for mode in (abi.TRIPS_BG_REFERENCE, abi.TRIPS_BG_CONSISTENT):
        d, r = _fwd(oracle, sc, background_mode=mode)
        px = 8 * 16 + 8
        np.testing.assert_allclose(r["size_px"][0], 1.0, rtol=1e-5)
        assert r["lengths"][0][px] == n
        np.testing.assert_array_equal(r["lists"][0][px][:n], np.arange(n))
        assert r["retained"][0][px] == 3
        a = r["alpha"][0][px]
        np.testing.assert_allclose(a[:3], 0.95, rtol=1e-5)
        assert np.all(a[3:] == -1)
        want = sum(0.95 * (0.05 ** j) * sc.texture[:, j] for j in range(3))  # no background: T < 0.001 at the end
        np.testing.assert_allclose(r["images"][0][0, :, 8, 8], want, rtol=1e-5)
    # with 3 points only, the background shows through: reference mode weights it with T before the last entry
    sc3 = scenes.tiny(n=3, w=16, h=16, f=30.0, num_layers=1, list_depth=16, seed=3, background=0.5)
    sc3.position[:, :3] = [[0.0, 0.0, 0.1 * i] for i in range(3)]
    sc3.confidence[:] = 0.5
    sc3.point_size[:] = scenes.inverse_softplus((3.0 + 0.1 * np.arange(3)) / 30.0)
    base = sum(0.5 * (0.5 ** j) * sc3.texture[:, j] for j in range(3))
    d, r = _fwd(oracle, sc3, background_mode=abi.TRIPS_BG_REFERENCE)
    np.testing.assert_allclose(r["images"][0][0, :, 8, 8], base + 0.5 * 0.25, rtol=1e-5)
    d, r = _fwd(oracle, sc3, background_mode=abi.TRIPS_BG_CONSISTENT)
    np.testing.assert_allclose(r["images"][0][0, :, 8, 8], base + 0.5 * 0.125, rtol=1e-5)


def test_dropout_and_viewer_cull(oracle):
    sc = scenes.tiny(n=500, w=32, h=24, f=30.0, num_layers=2, seed=8)
    d = abi.desc_for_scene(sc)
    drop = np.zeros((1, 500), dtype=np.float32)
    drop[0, ::2] = 1
    r = oracle.forward(sc, d, dropout=drop)
    assert np.all(r["depth"][0][::2] == -1)
    r0 = oracle.forward(sc, d)
    np.testing.assert_array_equal(r["depth"][0][1::2], r0["depth"][0][1::2])
    # dropout is only honoured in train mode (RenderForward.cu:233,240)
    d_eval = abi.desc_for_scene(sc, train=False)
    r_eval = oracle.forward(sc, d_eval, dropout=drop)
    np.testing.assert_array_equal(r_eval["depth"][0], r0["depth"][0])
    # viewer_only culls low-confidence points (RenderForward.cu:122-130)
    d_view = abi.desc_for_scene(sc, train=False, viewer_only=True, stability_cutoff_value=0.5)
    r_view = oracle.forward(sc, d_view)
    assert np.all(r_view["depth"][0][sc.confidence < 0.5] == -1)
    np.testing.assert_array_equal(r_view["depth"][0][sc.confidence >= 0.5], r0["depth"][0][sc.confidence >= 0.5])


def test_displacement_equals_moved_points_per_view(oracle):
    """View b renders xyz + displacement[b] (NeuralPointCloudCuda.h:260-270): the same bits as a single-view render
    of a cloud whose positions were moved beforehand, forward and backward."""
    import copy
    sc = scenes.tiny(n=600, w=40, h=30, f=38.0, num_layers=3, list_depth=16, seed=21, views=2)
    rng = np.random.default_rng(2)
    sc.displacement = rng.normal(0, 0.05, (2, 600, 3)).astype(np.float32)
    d = abi.desc_for_scene(sc)
    r = oracle.forward(sc, d)
    grads = [rng.normal(0, 1, im.shape).astype(np.float32) for im in r["images"]]
    g = oracle.backward(sc, d, r, grads)
    d_pos = np.zeros_like(g["d_position"])
    for b in range(2):
        one = copy.copy(sc)
        one.displacement = None
        one.position = sc.position.copy()
        one.position[:, :3] = sc.position[:, :3] + sc.displacement[b]
        one.views = [sc.views[b]]
        d1 = abi.desc_for_scene(one)
        r1 = oracle.forward(one, d1)
        for l in range(3):
            np.testing.assert_array_equal(r["images"][l][b], r1["images"][l][0])
        np.testing.assert_array_equal(r["lists"][b], r1["lists"][0])
        g1 = oracle.backward(one, d1, r1, [x[b:b + 1] for x in grads])
        d_pos += g1["d_position"]
    assert np.abs(r["images"][0][0] - oracle.forward(_without_displacement(sc), d)["images"][0][0]).max() > 1e-3
    np.testing.assert_allclose(g["d_position"], d_pos, rtol=1e-5, atol=1e-6 * np.abs(d_pos).max())


def _without_displacement(sc):
    import copy
    out = copy.copy(sc)
    out.displacement = None
    return out


def test_empty_scene_is_background(oracle):
    sc = scenes.tiny(n=4, w=16, h=12, f=30.0, num_layers=3, seed=8)
    sc.position[:, 2] = -100.0  # everything behind the camera
    d, r = _fwd(oracle, sc)
    for im in r["images"]:
        assert np.all(im == 0.25)
    assert r["lengths"].sum() == 0 and np.all(r["lists"] == -1)


def test_layer_sizes_ceil_and_floor(oracle):
    assert abi.layer_sizes(1920, 1080, 8) == [(1920, 1080), (960, 540), (480, 270), (240, 135), (120, 68), (60, 34),
                                              (30, 17), (15, 9)]
    assert abi.layer_sizes(1920, 1080, 8, True)[4:] == [(120, 67), (60, 33), (30, 16), (15, 8)]
    assert abi.layer_sizes(1245, 825, 4) == [(1245, 825), (623, 413), (312, 207), (156, 104)]
    import ctypes as C
    sc = scenes.tiny(n=4, w=1245, h=825, num_layers=8)
    for fl in (False, True):
        d = abi.desc_for_scene(sc, floor_layer_sizes=fl)
        w = (C.c_int32 * 8)()
        h = (C.c_int32 * 8)()
        assert oracle.lib.oracle_layer_sizes(C.byref(d), w, h) == 0
        assert list(zip(w, h)) == abi.layer_sizes(1245, 825, 8, fl)
