"""Parity of the HIP path (called through the C ABI) with the CPU oracle on the same seeded inputs.

Bars: per-point records and per-pixel index lists bit-exact; forward images within 1e-5 relative; per-point
gradients within 1e-4 relative per element (plus a floor of 3e-7 of the tensor's largest magnitude for elements that
are differences of larger terms); the block sums (pose, intrinsics, background) within 1e-4 of their largest
magnitude (tests/gpu_util.py)."""
import numpy as np
import pytest

from trips_amd import abi, scenes

pytestmark = pytest.mark.gpu

IMG_RTOL = 1e-5


def _check_forward(oracle, sc, desc, dropout=None, views=None):
    from tests.gpu_util import GpuRun
    ref = oracle.forward(sc, desc, dropout=dropout)
    run = GpuRun(sc, desc, dropout=dropout)
    imgs = run.forward()
    for l, (a, b) in enumerate(zip(imgs, ref["images"])):
        assert not np.isnan(a).any(), f"layer {l}: unwritten pixels"
        np.testing.assert_allclose(a, b, rtol=IMG_RTOL, atol=1e-6, err_msg=f"layer {l}")
    if desc.train:
        for b in range(desc.num_views):
            lists, retained, lengths = run.lists(b)
            np.testing.assert_array_equal(lengths, ref["lengths"][b])
            np.testing.assert_array_equal(lists, ref["lists"][b])
            np.testing.assert_array_equal(retained, ref["retained"][b])
            ip, depth, size_px, max_layer = run.points(b)
            np.testing.assert_array_equal(depth, ref["depth"][b])
            np.testing.assert_array_equal(ip, ref["ip"][b])
            np.testing.assert_array_equal(size_px, ref["size_px"][b])
            np.testing.assert_array_equal(max_layer, ref["max_layer"][b])
            c = run.ctx.counters(desc, run.saved, b)
            assert [c["valid"], c["E"], c["R"], c["P"]] == list(ref["counters"][b])
    return run, ref, imgs


@pytest.mark.parametrize("L,K,bg", [(1, 16, 0), (3, 8, 0), (4, 16, 1), (8, 16, 0)])
def test_forward_small(oracle, L, K, bg):
    sc = scenes.tiny(n=4000, w=70, h=50, f=60.0, num_layers=L, list_depth=K, seed=100 + L, radius=(0.004, 0.5))
    d = abi.desc_for_scene(sc, background_mode=bg)
    run, ref, _ = _check_forward(oracle, sc, d)
    assert ref["lengths"].max() > 16


def test_forward_views_crop_dropout(oracle):
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=3, list_depth=16, seed=7, views=3)
    sc.views[1]["crop_transform"] = (1.5, 1.25, -10.0, 4.0, 0.0)
    th = 0.3
    sc.views[2]["crop_rotation"] = (float(np.cos(th)), float(-np.sin(th)), float(np.sin(th)), float(np.cos(th)))
    sc.intrinsics[0, 4] = 0.5
    d = abi.desc_for_scene(sc)
    drop = (np.random.default_rng(0).random((3, 3000)) < 0.3).astype(np.float32)
    _check_forward(oracle, sc, d, dropout=drop)


def test_forward_eval_layout_and_viewer_cull(oracle):
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=3, list_depth=16, seed=8)
    d = abi.desc_for_scene(sc, train=False, viewer_only=True, stability_cutoff_value=0.4)
    assert d.layout == abi.TRIPS_LAYOUT_HWC
    _check_forward(oracle, sc, d)


def test_forward_radius_dropout_and_floor_layers(oracle):
    sc = scenes.tiny(n=3000, w=63, h=47, f=60.0, num_layers=4, list_depth=16, seed=9, radius=(0.004, 0.3))
    d = abi.desc_for_scene(sc, drop_out_points_by_radius=True, drop_out_radius_threshold=2.0, floor_layer_sizes=True)
    run, ref, _ = _check_forward(oracle, sc, d)
    assert 0 < ref["counters"][0, 0] < 3000


def test_forward_distortion(oracle):
    # non-zero distortion: parity with Saiga's model is unpinned; this checks HIP == oracle for the restated model
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=3, list_depth=16, seed=10)
    sc.intrinsics[0, 5:] = [0.1, -0.05, 0.01, 0.02, 0.01, -0.005, 0.003, -0.002]
    d = abi.desc_for_scene(sc, dist_cutoff=0.45)
    run, ref, _ = _check_forward(oracle, sc, d)
    assert 0 < ref["counters"][0, 0] < 3000


@pytest.mark.parametrize("channels", [3, 6, 8, 16])
def test_forward_other_channel_counts(oracle, channels):
    sc = scenes.tiny(n=2000, w=48, h=40, f=45.0, num_layers=3, list_depth=16, seed=20 + channels, channels=channels)
    d = abi.desc_for_scene(sc)
    _check_forward(oracle, sc, d)


def test_forward_edge_cases(oracle):
    # all points behind the camera -> pure background; a single point; ties in depth
    sc = scenes.tiny(n=5, w=16, h=12, f=30.0, num_layers=3, seed=8)
    sc.position[:, 2] = -100.0
    _check_forward(oracle, sc, abi.desc_for_scene(sc))
    sc = scenes.tiny(n=40, w=16, h=16, f=30.0, num_layers=1, list_depth=16, seed=2)
    sc.position[:, :3] = [0.01, 0.01, 0.0]  # 40 coincident points: tie-break by id, top-16 of 40
    run, ref, _ = _check_forward(oracle, sc, abi.desc_for_scene(sc))
    lists, _, _ = run.lists(0)
    np.testing.assert_array_equal(lists[8 * 16 + 8], np.arange(16))


@pytest.mark.parametrize("seed", range(10))
def test_random_shapes_forward_backward(oracle, seed):
    """Image sizes that are not multiples of the 32-pixel tiles (down to a few pixels, where the coarse layers are one
    pixel wide), every layer count, both list depths, both layouts and layer-size rules, several views."""
    rng = np.random.default_rng(1000 + seed)
    w, h = int(rng.integers(3, 150)), int(rng.integers(3, 110))
    L = int(rng.integers(1, 9))
    K = int(rng.choice([8, 16]))
    C = int(rng.choice([3, 4, 4, 6, 8, 16]))
    views = int(rng.integers(1, 4))
    floor = bool(rng.integers(0, 2))
    if floor:
        L = min(L, int(np.floor(np.log2(min(w, h)))) + 1)  # no empty layers
    sc = scenes.tiny(n=int(rng.integers(200, 3000)), w=w, h=h, f=float(0.9 * max(w, h)), num_layers=L, list_depth=K,
                     seed=300 + seed, views=views, channels=C, radius=(0.004, 0.5))
    sc.confidence = (sc.confidence ** 0.3).astype(np.float32)
    layout = int(rng.choice([abi.TRIPS_LAYOUT_CHW, abi.TRIPS_LAYOUT_HWC]))
    d = abi.desc_for_scene(sc, layout=layout, floor_layer_sizes=floor, background_mode=int(rng.integers(0, 2)))
    _check_forward(oracle, sc, d)
    _check_backward(oracle, sc, d, seed=seed)


@pytest.mark.parametrize("channels,K,layout,views", [(3, 16, abi.TRIPS_LAYOUT_HWC, 1), (6, 8, abi.TRIPS_LAYOUT_CHW, 2),
                                                     (8, 16, abi.TRIPS_LAYOUT_CHW, 1), (16, 8, abi.TRIPS_LAYOUT_HWC, 2),
                                                     (16, 16, abi.TRIPS_LAYOUT_CHW, 1)])
def test_medium_views_other_channel_counts(oracle, channels, K, layout, views):
    """300 000 points on 640 x 480 and 8 layers (hundreds of tiles, every chunk of the binning populated, lists up to a
    few hundred entries) for the kernel variants that the full-size configurations, all 4-channel, do not reach."""
    sc = scenes.tiny(n=300_000, w=640, h=480, f=520.0, num_layers=8, list_depth=K, seed=40 + channels + K, views=views,
                     channels=channels, radius=(0.0005, 0.05))
    sc.confidence = (sc.confidence ** 0.3).astype(np.float32)
    d = abi.desc_for_scene(sc, layout=layout, background_mode=views % 2)
    run, ref, _ = _check_forward(oracle, sc, d)
    assert ref["lengths"].max() > 64 and ref["counters"][0][0] > 100_000
    _check_backward(oracle, sc, d, seed=channels)


@pytest.mark.parametrize("order", ["random", "by_screen_tile"])
def test_medium_view_memory_order_of_the_points(oracle, order):
    """The same view with its points in random order and sorted by screen tile (neighbouring points in the same tile:
    neighbouring lanes of the point pass then share their rows' lines, and the chunks' compact numbers follow the screen)."""
    sc = scenes.tiny(n=200_000, w=640, h=480, f=520.0, num_layers=6, list_depth=16, seed=61, radius=(0.0005, 0.05))
    if order == "by_screen_tile":
        d0 = abi.desc_for_scene(sc)
        ip = oracle.forward(sc, d0)["ip"][0]
        key = (np.floor(ip[:, 1] / 32).astype(np.int64) * 64 + np.floor(ip[:, 0] / 32).astype(np.int64))
        perm = np.argsort(key, kind="stable")
        sc.position = np.ascontiguousarray(sc.position[perm])
        sc.point_size = np.ascontiguousarray(sc.point_size[perm])
        sc.texture = np.ascontiguousarray(sc.texture[:, perm])
        sc.confidence = np.ascontiguousarray(sc.confidence[perm])
    d = abi.desc_for_scene(sc)
    _check_forward(oracle, sc, d)
    _check_backward(oracle, sc, d, seed=3)


@pytest.mark.parametrize("w,h,L,n", [(4000, 40, 8, 20000), (37, 3000, 6, 20000), (1, 1, 1, 10), (2, 2, 2, 50), (33, 33, 6, 500)])
def test_extreme_image_shapes(oracle, w, h, L, n):
    """Very wide and very tall images (many tile columns / rows, coarse layers one pixel high) and images smaller than
    one tile."""
    sc = scenes.tiny(n=n, w=w, h=h, f=float(0.8 * max(w, h)), num_layers=L, list_depth=16, seed=w + h, radius=(0.002, 0.3))
    d = abi.desc_for_scene(sc)
    _check_forward(oracle, sc, d)
    _check_backward(oracle, sc, d, seed=1)


def test_transmittance_cutoff_matches(oracle):
    n = 12
    sc = scenes.tiny(n=n, w=16, h=16, f=30.0, num_layers=1, list_depth=16, seed=3, background=0.5)
    sc.position[:, :3] = [[0.0, 0.0, 0.1 * i] for i in range(n)]
    sc.confidence[:] = 0.95
    sc.point_size[:] = scenes.inverse_softplus((3.0 + 0.1 * np.arange(n)) / 30.0)
    for mode in (0, 1):
        run, ref, _ = _check_forward(oracle, sc, abi.desc_for_scene(sc, background_mode=mode))
        assert ref["retained"][0][8 * 16 + 8] == 3


def _check_backward(oracle, sc, desc, seed=0, **want):
    from tests.gpu_util import GpuRun, assert_grads_close
    ref = oracle.forward(sc, desc)
    rng = np.random.default_rng(seed)
    shape = (lambda w, h: (desc.num_views, desc.num_channels, h, w)) if desc.layout == abi.TRIPS_LAYOUT_CHW else \
        (lambda w, h: (desc.num_views, h, w, desc.num_channels))
    grads = [rng.normal(0, 1, shape(w, h)).astype(np.float32) for (w, h) in ref["sizes"]]
    g_ref = oracle.backward(sc, desc, ref, grads, **want)
    run = GpuRun(sc, desc)
    run.forward()
    g = run.backward(grads, **want)
    assert_grads_close(g, g_ref)
    return None, g, g_ref


@pytest.mark.parametrize("L,K,bg", [(1, 16, 1), (3, 8, 0), (4, 16, 1), (8, 16, 0)])
def test_backward_small(oracle, L, K, bg):
    radius = (0.004, 0.5) if L > 1 else (0.004, 0.03)
    sc = scenes.tiny(n=4000, w=70, h=50, f=60.0, num_layers=L, list_depth=K, seed=200 + L, radius=radius)
    sc.confidence = (sc.confidence ** 0.3).astype(np.float32)
    sc.intrinsics[0, 4] = 0.7
    d = abi.desc_for_scene(sc, background_mode=bg)
    errs, g, _ = _check_backward(oracle, sc, d)
    assert np.abs(g["d_pose"]).max() > 0 and np.abs(g["d_intrinsics"]).max() > 0


@pytest.mark.parametrize("scene", ["ordinary", "tight_cluster", "many_layers_two_views"])
def test_backward_pair_row_forms_agree(oracle, scene):
    """Between its two passes the backward keeps a row per (point, layer) pair, either all rows cleared beforehand or a
    flag byte per row (chosen per view on the device from the share of retained entries). Forced either way and left
    to choose, the gradients are the same bits, and they are the oracle's."""
    from tests.gpu_util import GpuRun, assert_grads_close
    if scene == "ordinary":
        sc = scenes.tiny(n=6000, w=90, h=70, f=70.0, num_layers=4, list_depth=16, seed=301, radius=(0.004, 0.3))
    elif scene == "tight_cluster":
        sc = scenes.tiny(n=20000, w=96, h=64, f=80.0, num_layers=4, list_depth=16, seed=302, radius=(0.004, 0.2))
        rng = np.random.default_rng(5)
        sc.position[:, :3] = (rng.normal(0, 0.01, (20000, 3)) + np.array([0.05, -0.02, 0.0])).astype(np.float32)
    else:
        sc = scenes.tiny(n=3000, w=128, h=96, f=110.0, num_layers=8, list_depth=16, seed=303, views=2, radius=(0.05, 0.6))
    d = abi.desc_for_scene(sc)
    ref = oracle.forward(sc, d)
    rng = np.random.default_rng(9)
    grads = [rng.normal(0, 1, (d.num_views, d.num_channels, h, w)).astype(np.float32) for (w, h) in ref["sizes"]]
    g_ref = oracle.backward(sc, d, ref, grads)
    run = GpuRun(sc, d)
    run.forward()
    got = {}
    try:
        for mode in (1, 2, 0):
            run.ctx.pair_rows_mode(mode)
            got[mode] = {k: np.array(v, copy=True) for k, v in run.backward(grads).items()}
    finally:
        run.ctx.pair_rows_mode(0)
    assert_grads_close(got[1], g_ref)
    from tests.gpu_util import rel_err
    for k in got[1]:
        if k in ("d_texture", "d_confidence", "d_position", "d_point_size"):
            np.testing.assert_array_equal(got[2][k], got[1][k], err_msg=f"{k}: flagged rows against rows of all pairs")
            np.testing.assert_array_equal(got[0][k], got[1][k], err_msg=f"{k}: the device's own choice")
        else:  # sums over workgroups, added with atomics: the same terms in an order that varies from launch to launch
            assert rel_err(got[2][k], got[1][k]) < 1e-6 and rel_err(got[0][k], got[1][k]) < 1e-6, k


@pytest.mark.parametrize("channels", [4, 16])
def test_backward_points_written_to_many_layers(oracle, channels):
    """Every point is large enough for four to eight layers: a wavefront of the point pass then has several hundred
    (point, layer) items for its 64 points, which it works off in several rounds."""
    sc = scenes.tiny(n=3000, w=128, h=96, f=110.0, num_layers=8, list_depth=16, seed=77, channels=channels,
                     radius=(0.08, 1.2))
    d = abi.desc_for_scene(sc)
    ref = oracle.forward(sc, d)
    layers = ref["max_layer"][0][ref["depth"][0] > 0]
    assert np.median(layers) >= 4 and layers.max() >= 7
    _check_backward(oracle, sc, d, seed=9)


@pytest.mark.parametrize("channels,K", [(3, 16), (8, 8), (16, 16)])
def test_backward_other_channel_counts(oracle, channels, K):
    sc = scenes.tiny(n=2500, w=56, h=40, f=50.0, num_layers=3, list_depth=K, seed=60 + channels, channels=channels,
                     radius=(0.004, 0.4))
    sc.confidence = (sc.confidence ** 0.3).astype(np.float32)
    _check_backward(oracle, sc, abi.desc_for_scene(sc))


def test_backward_views_crop_distortion_optional_outputs(oracle):
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=3, list_depth=16, seed=31, views=2)
    sc.views[1]["crop_transform"] = (1.5, 1.25, -10.0, 4.0, 0.0)
    th = 0.3
    sc.views[1]["crop_rotation"] = (float(np.cos(th)), float(-np.sin(th)), float(np.sin(th)), float(np.cos(th)))
    sc.intrinsics[0, 5:] = [0.1, -0.05, 0.01, 0.02, 0.01, -0.005, 0.003, -0.002]
    d = abi.desc_for_scene(sc)
    _check_backward(oracle, sc, d)
    _check_backward(oracle, sc, d, want_point_size=False)
    _check_backward(oracle, sc, d, want_position=False, want_pose=False, want_intrinsics=False)


@pytest.mark.parametrize("case", ["two_views", "shared_columns", "spare_columns", "bad_index", "no_size_no_position"])
def test_backward_overwrite_mode_equals_adding_into_zeros(case):
    """overwrite_point_grads: the per-point outputs start as NaN and must come out bit-equal to what adding into
    zeroed outputs gives (second view added on top of the first; descriptor columns shared between points, columns
    no point uses and skipped points all end up defined)."""
    from tests.gpu_util import GpuRun
    views = 2 if case == "two_views" else 1
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=3, list_depth=16, seed=41, views=views, radius=(0.004, 0.4))
    if case == "shared_columns":
        sc.index = (np.arange(3000) // 2).astype(np.int32)  # two points per column, the upper half unused
    if case == "spare_columns":
        extra = 100
        sc.texture = np.concatenate([sc.texture, np.ones((sc.texture.shape[0], extra), np.float32)], axis=1)
        sc.confidence = np.concatenate([sc.confidence, np.full(extra, 0.5, np.float32)])
    if case == "bad_index":
        sc.index = sc.index.copy()
        sc.index[::5] = sc.texture.shape[1] + 7
    d = abi.desc_for_scene(sc)
    want = dict(want_point_size=False, want_position=False) if case == "no_size_no_position" else {}
    rng = np.random.default_rng(8)
    run = GpuRun(sc, d)
    images = run.forward()
    grads = [rng.normal(0, 1, im.shape).astype(np.float32) for im in images]
    added = run.backward(grads, **want)
    written = run.backward(grads, overwrite=True, **want)
    for k, v in added.items():
        if v is None:
            assert written[k] is None
            continue
        assert np.isfinite(written[k]).all(), k
        if k in ("d_background", "d_pose", "d_intrinsics"):
            np.testing.assert_allclose(written[k], v, rtol=1e-4, atol=1e-6)  # float atomics across workgroups
        else:
            assert np.array_equal(written[k], v), k
    assert np.abs(added["d_texture"]).max() > 0


@pytest.mark.parametrize("views", [1, 2])
@pytest.mark.parametrize("overwrite", [False, True])
def test_backward_clearing_the_block_sums_equals_adding_into_zeros(views, overwrite):
    """clear_block_sums: d_background, every row of d_pose and every row of d_intrinsics start as NaN and must come out
    as what adding into zeroed buffers gives: cleared once, before the first view of the batch, and added to by every
    view after it; rows of images and cameras no view of the batch touches come out as zero."""
    from tests.gpu_util import GpuRun
    sc = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=3, list_depth=16, seed=43, views=views, radius=(0.004, 0.4))
    sc.poses_se3 = np.concatenate([sc.poses_se3, sc.poses_se3[:1]])  # one image and one camera no view refers to
    sc.intrinsics = np.concatenate([sc.intrinsics, sc.intrinsics[:1]])
    d = abi.desc_for_scene(sc)
    rng = np.random.default_rng(9)
    run = GpuRun(sc, d)
    images = run.forward()
    grads = [rng.normal(0, 1, im.shape).astype(np.float32) for im in images]
    added = run.backward(grads, overwrite=overwrite)
    cleared = run.backward(grads, overwrite=overwrite, clear=True)
    for k, v in added.items():
        assert np.isfinite(cleared[k]).all(), k
        if k in ("d_background", "d_pose", "d_intrinsics"):
            np.testing.assert_allclose(cleared[k], v, rtol=1e-4, atol=1e-6)  # float atomics across workgroups
        else:
            assert np.array_equal(cleared[k], v), k
    assert np.abs(added["d_pose"]).max() > 0 and np.abs(added["d_background"]).max() > 0
    assert not cleared["d_pose"][-1].any() and not cleared["d_intrinsics"][-1].any()


def test_displacement_forward_backward(oracle):
    """Per-view displacements of the point positions (dynamic_refinement_t, PointRenderer.cu:703-713)."""
    sc = scenes.tiny(n=4000, w=70, h=50, f=60.0, num_layers=4, list_depth=16, seed=77, views=3, radius=(0.004, 0.4))
    sc.displacement = np.random.default_rng(5).normal(0, 0.05, (3, 4000, 3)).astype(np.float32)
    d = abi.desc_for_scene(sc)
    _check_forward(oracle, sc, d)
    _check_backward(oracle, sc, d)


def test_index_outside_the_descriptor_table_is_left_out_and_reported(oracle):
    import ctypes as C
    from tests.gpu_util import GpuRun
    from trips_amd import _lib
    sc = scenes.tiny(n=2000, w=48, h=40, f=45.0, num_layers=3, list_depth=16, seed=12)
    sc.index = sc.index.copy()
    sc.index[::7] = -1
    sc.index[3::11] = sc.texture.shape[1]
    d = abi.desc_for_scene(sc)
    run, ref, _ = _check_forward(oracle, sc, d)
    bad = (sc.index < 0) | (sc.index >= sc.texture.shape[1])
    assert np.all(ref["depth"][0][bad] == -1)
    rc = run.ctx.lib.trips_splat_check(run.ctx.ctx, C.c_void_p(run.workspace.data_ptr()), None)
    assert rc == abi.TRIPS_ERR_INVALID_ARG and b"index" in _lib.load().trips_last_error_string()
    with pytest.raises(RuntimeError):
        run.ctx.check(run.workspace)


def test_tight_cluster_long_lists_and_split_tiles(oracle):
    """Thousands of points on a handful of pixels: lists far longer than the segment length of the long-list
    reduction (512 / 256 keys) and tiles with more bin entries than a slice (8192), with exact depth ties."""
    sc = scenes.tiny(n=30000, w=96, h=64, f=80.0, num_layers=4, list_depth=16, seed=91, radius=(0.004, 0.2))
    rng = np.random.default_rng(3)
    sc.position[:, :3] = (rng.normal(0, 0.004, (30000, 3)) + np.array([0.05, -0.02, 0.0])).astype(np.float32)
    sc.position[:2000, 2] = sc.position[0, 2]  # equal depths: the tie-break by point id decides
    sc.position[5000:5600, :3] = rng.uniform(-1, 1, (600, 3)).astype(np.float32)  # some ordinary pixels too
    d = abi.desc_for_scene(sc)
    run, ref, _ = _check_forward(oracle, sc, d)
    assert ref["lengths"].max() > 3000
    c = run.ctx.counters(d, run.saved, 0)
    assert c["E"] > 4 * 8192
    _check_backward(oracle, sc, d)
    # the same with a list storage that is too small: no fault, the overflow is reported
    d_small = abi.desc_for_scene(sc, max_list_entries=20000)
    from tests.gpu_util import GpuRun
    small = GpuRun(sc, d_small)
    small.forward()
    with pytest.raises(RuntimeError):
        small.ctx.check(small.workspace)


def test_footprints_on_tile_and_image_borders_with_equal_depths(oracle):
    """A dense grid of points in a plane that faces the camera: footprints start at every pixel, also at the last
    column and row of a 32-pixel tile (their other pixels belong to the neighbouring tiles) and at the last pixels of
    every layer (a footprint that would leave the image is culled), and all depths are equal, so the order of every
    list is decided by the point ids alone, whichever of a pixel's four cells an entry was filed under."""
    w, h, gx, gy = 100, 70, 230, 170
    sc = scenes.tiny(n=gx * gy, w=w, h=h, f=90.0, num_layers=4, list_depth=16, seed=17, radius=(0.004, 0.12))
    xr, yr = 1.15 * 3.0 * (w / 2) / 90.0, 1.15 * 3.0 * (h / 2) / 90.0  # a little more than the view covers at depth 3
    X, Y = np.meshgrid(np.linspace(-xr, xr, gx), np.linspace(-yr, yr, gy))
    order = np.random.default_rng(5).permutation(gx * gy)  # ids unrelated to the screen position
    sc.position[:, 0] = X.reshape(-1)[order]
    sc.position[:, 1] = Y.reshape(-1)[order]
    sc.position[:, 2] = 0.0
    d = abi.desc_for_scene(sc)
    run, ref, _ = _check_forward(oracle, sc, d)
    depth = ref["depth"][0]
    assert len(np.unique(depth[depth > 0])) == 1  # every visible point at the same depth
    ip = ref["ip"][0][depth > 0]
    px = np.floor(ip[:, 0]).astype(int)
    assert {31, 32, 63, 64, w - 2} <= set(px.tolist()) and px.max() == w - 2
    assert ref["lengths"][0].max() > 16
    _check_backward(oracle, sc, d, seed=4)


def test_more_than_2_to_the_23_points(oracle):
    """Clouds above 2^23 points take the 16-byte form of the tile entries (the 8-byte form has 23 bits for a point's
    number). Most points lie behind the camera; the visible ones sit at both ends of the cloud, enough of them at the
    end that their numbers pass 2^23."""
    n = (1 << 23) + 6000
    sc = scenes.tiny(n=n, w=96, h=64, f=80.0, num_layers=4, list_depth=16, seed=23, radius=(0.004, 0.2))
    sc.position[:, 2] = -10.0  # behind the camera, which looks along +z from z = -3
    rng = np.random.default_rng(8)
    for sl in (slice(0, 3000), slice(n - 40000, n)):
        sc.position[sl, 2] = rng.uniform(-1, 1, sc.position[sl].shape[0]).astype(np.float32)
    d = abi.desc_for_scene(sc)
    run, ref, _ = _check_forward(oracle, sc, d)
    lists = ref["lists"][0]
    assert lists.max() >= 1 << 23 and 0 <= lists[lists >= 0].min() < 3000
    _check_backward(oracle, sc, d, seed=5)


def test_config1_forward_full(oracle):
    sc = scenes.config1()
    _check_forward(oracle, sc, abi.desc_for_scene(sc, train=True))
    _check_forward(oracle, sc, abi.desc_for_scene(sc, train=False))


def test_config2_forward_backward_full(oracle):
    sc = scenes.config2()
    d = abi.desc_for_scene(sc)
    _check_forward(oracle, sc, d)
    _check_backward(oracle, sc, d, seed=2)


def test_config4_contention_reduced(oracle):
    # same shape as the contention config (64 tight clusters, 4 views, K = 16) at a tenth of the points
    sc = scenes.config4(n=400_000)
    d = abi.desc_for_scene(sc)
    run, ref, _ = _check_forward(oracle, sc, d)
    assert ref["lengths"].max() > 200
    _check_backward(oracle, sc, d, seed=4)


def test_config3_forward_backward_full(oracle):
    # the configuration the benchmark is quoted on: 6M points, 1920x1080, 8 layers, K = 16
    sc = scenes.config3()
    d = abi.desc_for_scene(sc)
    run, ref, _ = _check_forward(oracle, sc, d)
    assert int(ref["counters"][0, 1]) > 20_000_000
    _check_backward(oracle, sc, d, seed=3)


def test_config4_contention_full(oracle):
    # 4M points in 64 tight clusters, 4 views, 1245x825 (odd sizes: ceil halving), K = 16
    sc = scenes.config4()
    d = abi.desc_for_scene(sc)
    run, ref, _ = _check_forward(oracle, sc, d)
    assert ref["lengths"].max() > 2000
    _check_backward(oracle, sc, d, seed=5)


def test_point_order_does_not_matter_at_full_size():
    """Size-independent property at the benchmark's size: shuffling the point order permutes the per-point
    gradients and leaves the images unchanged, except where two entries of a pixel list have the same depth: the
    tie breaks by point id, so a shuffle may swap them. The run counts those pixels itself (adjacent equal depths
    among the sorted entries of a list) and allows only that many pixels, and that many times K points, to differ."""
    import dataclasses
    from tests.gpu_util import GRAD_FLOOR, GRAD_RTOL, GpuRun, rel_err
    sc = scenes.config3()
    rng = np.random.Generator(np.random.Philox(99))
    perm = rng.permutation(sc.num_points)
    sc2 = dataclasses.replace(sc, position=sc.position[perm], point_size=sc.point_size[perm],
                              texture=np.ascontiguousarray(sc.texture[:, perm]), confidence=sc.confidence[perm])
    d = abi.desc_for_scene(sc)
    grad_rng = np.random.Generator(np.random.Philox(100))
    sizes, _, _ = abi.pyramid_pixels(d)
    gi = [grad_rng.normal(0, 1, (1, d.num_channels, h, w)).astype(np.float32) for (w, h) in sizes]
    a = GpuRun(sc, d)
    ia = a.forward()
    ga = a.backward(gi)
    ca = a.ctx.counters(d, a.saved, 0)
    lists, retained, _ = a.lists(0)
    _, depth, _, _ = a.points(0)
    del a
    # pixels with a depth tie among their sorted entries, and the points on such pixels
    K = lists.shape[1]
    dl = np.where(lists >= 0, depth[np.clip(lists, 0, None)], np.inf)
    tied = ((dl[:, 1:] == dl[:, :-1]) & np.isfinite(dl[:, 1:])).any(axis=1)
    n_tied = int(tied.sum())
    assert n_tied < 1000  # config 3 has 173 of them among 2.76 M pixels
    b = GpuRun(sc2, d)
    ib = b.forward()
    gb = b.backward(gi)
    cb = b.ctx.counters(d, b.saved, 0)
    assert ca == cb
    differing_pixels = 0
    for x, y in zip(ia, ib):
        differing_pixels += int((np.abs(x - y) > 1e-5 * np.abs(y) + 1e-6).any(axis=1).sum())
    assert differing_pixels <= n_tied, (differing_pixels, n_tied)

    def differing_points(got, want, axis):
        got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
        bad = np.abs(got - want) > GRAD_RTOL * np.abs(want) + GRAD_FLOOR * np.abs(want).max()
        return int(bad.any(axis=axis).sum()) if bad.ndim > 1 else int(bad.sum())

    allowed = n_tied * K  # every entry of a tied pixel's list may see another transmittance
    assert differing_points(gb["d_position"], ga["d_position"][perm], 1) <= allowed
    assert differing_points(gb["d_point_size"], ga["d_point_size"][perm], None) <= allowed
    assert differing_points(gb["d_confidence"], ga["d_confidence"][perm], None) <= allowed
    assert differing_points(gb["d_texture"], ga["d_texture"][:, perm], 0) <= allowed
    assert rel_err(gb["d_pose"], ga["d_pose"]) < 1e-3
    assert rel_err(gb["d_background"], ga["d_background"]) < 1e-3


def test_list_overflow_is_reported(oracle):
    from tests.gpu_util import GpuRun
    from trips_amd._lib import TripsError
    sc = scenes.tiny(n=4000, w=70, h=50, f=60.0, num_layers=3, list_depth=16, seed=103)
    d_ok = abi.desc_for_scene(sc)
    ref = oracle.forward(sc, d_ok)
    E = int(ref["counters"][0, 1])
    run = GpuRun(sc, abi.desc_for_scene(sc, max_list_entries=E))
    run.forward()
    run.ctx.check(run.workspace)  # exactly enough: fine
    run = GpuRun(sc, abi.desc_for_scene(sc, max_list_entries=E // 2))
    run.forward()
    with pytest.raises(TripsError) as ei:
        run.ctx.check(run.workspace)
    assert ei.value.code == abi.TRIPS_ERR_LIST_OVERFLOW


def test_forward_is_deterministic_and_repeatable(oracle):
    from tests.gpu_util import GpuRun
    sc = scenes.tiny(n=20000, w=160, h=120, f=120.0, num_layers=5, list_depth=16, seed=77)
    run = GpuRun(sc, abi.desc_for_scene(sc))
    a = run.forward()
    la = run.lists(0)
    b = run.forward()
    lb = run.lists(0)
    for x, y in zip(a, b):
        np.testing.assert_array_equal(x, y)
    for x, y in zip(la, lb):
        np.testing.assert_array_equal(x, y)
