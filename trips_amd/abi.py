"""ctypes mirror of include/trips_splat.h (structs, enums, constants).

Field order and types must match the header exactly; tests/test_abi.py checks the sizes
against what the compiled library reports.
"""
import ctypes as C

TRIPS_MAX_LAYERS = 8
TRIPS_MAX_VIEWS = 16
TRIPS_ABI_VERSION = 2
TRIPS_STATIC_WORKSPACE_BYTES = 64 << 20  # workspace inside the library, trips_splat_forward_static
TRIPS_STEPS_I64, TRIPS_STEPS_I32 = 0, 1
TRIPS_PROFILE_MAX_KERNELS = 32
TRIPS_UNET_MAX_LEVELS = 8

TRIPS_OK = 0
TRIPS_ERR_INVALID_ARG = 1
TRIPS_ERR_UNSUPPORTED = 2
TRIPS_ERR_WORKSPACE_SMALL = 3
TRIPS_ERR_HIP = 4
TRIPS_ERR_LIST_OVERFLOW = 5

TRIPS_BG_REFERENCE = 0
TRIPS_BG_CONSISTENT = 1
TRIPS_LAYOUT_CHW = 0
TRIPS_LAYOUT_HWC = 1
TRIPS_DTYPE_F32 = 0
TRIPS_DTYPE_F64 = 1


class TripsView(C.Structure):
    _fields_ = [
        ("w", C.c_int32),
        ("h", C.c_int32),
        ("image_index", C.c_int32),
        ("camera_index", C.c_int32),
        ("camera_model_type", C.c_int32),
        ("crop_transform", C.c_float * 5),
        ("crop_rotation", C.c_float * 4),
    ]


class TripsSplatDesc(C.Structure):
    _fields_ = [
        ("abi_version", C.c_int32),
        ("num_points", C.c_int32),
        ("num_texels", C.c_int32),
        ("num_channels", C.c_int32),
        ("num_layers", C.c_int32),
        ("list_depth", C.c_int32),
        ("num_views", C.c_int32),
        ("num_images", C.c_int32),
        ("num_cameras", C.c_int32),
        ("train", C.c_int32),
        ("layout", C.c_int32),
        ("floor_layer_sizes", C.c_int32),
        ("background_mode", C.c_int32),
        ("drop_out_points_by_radius", C.c_int32),
        ("drop_out_radius_threshold", C.c_float),
        ("dist_cutoff", C.c_float),
        ("viewer_only", C.c_int32),
        ("stability_cutoff_value", C.c_float),
        ("max_list_entries", C.c_int64),
        ("views", TripsView * TRIPS_MAX_VIEWS),
    ]


class TripsSplatIn(C.Structure):
    _fields_ = [
        ("position", C.c_void_p),
        ("point_size", C.c_void_p),
        ("index", C.c_void_p),
        ("texture", C.c_void_p),
        ("confidence", C.c_void_p),
        ("background", C.c_void_p),
        ("poses_se3", C.c_void_p),
        ("intrinsics", C.c_void_p),
        ("dropout", C.c_void_p),
        ("displacement", C.c_void_p),
    ]


class TripsSplatOut(C.Structure):
    _fields_ = [
        ("image", C.c_void_p * TRIPS_MAX_LAYERS),
        ("saved", C.c_void_p),
    ]


class TripsSplatGrads(C.Structure):
    _fields_ = [
        ("d_texture", C.c_void_p),
        ("d_confidence", C.c_void_p),
        ("d_background", C.c_void_p),
        ("d_position", C.c_void_p),
        ("d_point_size", C.c_void_p),
        ("d_pose", C.c_void_p),
        ("d_intrinsics", C.c_void_p),
        ("overwrite_point_grads", C.c_int32),
        ("clear_block_sums", C.c_int32),
    ]


class TripsAdamTensor(C.Structure):
    _fields_ = [
        ("weights", C.c_void_p),
        ("grads", C.c_void_p),
        ("first_moment", C.c_void_p),
        ("second_moment", C.c_void_p),
        ("steps", C.c_void_p),
        ("n", C.c_int64),
        ("dtype", C.c_int32),
        ("lr", C.c_float),
        ("beta1", C.c_float),
        ("beta2", C.c_float),
        ("eps", C.c_float),
        ("relative_weight_decay", C.c_float),
        ("absolute_weight_decay", C.c_float),
        ("weight_clipping_magnitude", C.c_float),
        ("lower_lr_bound", C.c_float),
        ("upper_lr_bound", C.c_float),
        ("loss_scale", C.c_float),
        ("steps_dtype", C.c_int32),
    ]


class TripsUnetDesc(C.Structure):
    """include/trips_unet.h"""
    _fields_ = [
        ("abi_version", C.c_int32),
        ("num_levels", C.c_int32),
        ("num_input_channels", C.c_int32),
        ("num_output_channels", C.c_int32),
        ("batch", C.c_int32),
        ("filters", C.c_int32 * TRIPS_UNET_MAX_LEVELS),
        ("level_w", C.c_int32 * TRIPS_UNET_MAX_LEVELS),
        ("level_h", C.c_int32 * TRIPS_UNET_MAX_LEVELS),
        ("weights_packed", C.c_int32),
    ]


class TripsUnetWeights(C.Structure):
    _fields_ = [
        ("feature_weight", C.c_void_p * TRIPS_UNET_MAX_LEVELS),
        ("feature_bias", C.c_void_p * TRIPS_UNET_MAX_LEVELS),
        ("mask_weight", C.c_void_p * TRIPS_UNET_MAX_LEVELS),
        ("mask_bias", C.c_void_p * TRIPS_UNET_MAX_LEVELS),
        ("final_weight", C.c_void_p),
        ("final_bias", C.c_void_p),
    ]


class TripsUnetGrads(C.Structure):
    _fields_ = [
        ("feature_weight", C.c_void_p * TRIPS_UNET_MAX_LEVELS),
        ("feature_bias", C.c_void_p * TRIPS_UNET_MAX_LEVELS),
        ("mask_weight", C.c_void_p * TRIPS_UNET_MAX_LEVELS),
        ("mask_bias", C.c_void_p * TRIPS_UNET_MAX_LEVELS),
        ("final_weight", C.c_void_p),
        ("final_bias", C.c_void_p),
        ("inputs", C.c_void_p * TRIPS_UNET_MAX_LEVELS),
    ]


def make_unet_desc(filters, level_sizes, num_input_channels=4, num_output_channels=3, batch=1):
    """level_sizes: [(w, h)] of the pyramid levels the net consumes, finest first."""
    d = TripsUnetDesc()
    d.abi_version = TRIPS_ABI_VERSION
    d.num_levels = len(level_sizes)
    d.num_input_channels = num_input_channels
    d.num_output_channels = num_output_channels
    d.batch = batch
    for i, (w, h) in enumerate(level_sizes):
        d.filters[i] = int(filters[i])
        d.level_w[i] = int(w)
        d.level_h[i] = int(h)
    return d


FLT_MAX = 3.4028234663852886e38


def layer_sizes(w, h, num_layers, floor_layer_sizes=False):
    """Pyramid layer sizes: ceil halving unless floor_layer_sizes
    (reference: src/lib/rendering/PointRenderer.cu:385-394)."""
    out = []
    for _ in range(num_layers):
        out.append((w, h))
        if floor_layer_sizes:
            w, h = w // 2, h // 2
        else:
            w, h = (w + 1) // 2, (h + 1) // 2
    return out


def make_desc(*, num_points, num_texels, num_channels=4, num_layers, list_depth=16, views, num_images, num_cameras,
              train=True, layout=None, floor_layer_sizes=False, background_mode=TRIPS_BG_REFERENCE,
              drop_out_points_by_radius=False, drop_out_radius_threshold=0.6, dist_cutoff=20.0, viewer_only=False,
              stability_cutoff_value=10000.0, max_list_entries=0):
    """Fill a TripsSplatDesc. `views` is a list of dicts with keys w, h, image_index, camera_index and optional
    crop_transform (fx fy cx cy s; default identity 1 1 0 0 0), crop_rotation (row-major 2x2; default identity)."""
    d = TripsSplatDesc()
    d.abi_version = TRIPS_ABI_VERSION
    d.num_points = num_points
    d.num_texels = num_texels
    d.num_channels = num_channels
    d.num_layers = num_layers
    d.list_depth = list_depth
    d.num_views = len(views)
    d.num_images = num_images
    d.num_cameras = num_cameras
    d.train = int(bool(train))
    if layout is None:
        layout = TRIPS_LAYOUT_CHW if train else TRIPS_LAYOUT_HWC
    d.layout = layout
    d.floor_layer_sizes = int(bool(floor_layer_sizes))
    d.background_mode = background_mode
    d.drop_out_points_by_radius = int(bool(drop_out_points_by_radius))
    d.drop_out_radius_threshold = drop_out_radius_threshold
    d.dist_cutoff = dist_cutoff
    d.viewer_only = int(bool(viewer_only))
    d.stability_cutoff_value = stability_cutoff_value
    d.max_list_entries = max_list_entries
    if len(views) > TRIPS_MAX_VIEWS:
        raise ValueError("too many views")
    for i, v in enumerate(views):
        tv = d.views[i]
        tv.w, tv.h = int(v["w"]), int(v["h"])
        tv.image_index = int(v.get("image_index", 0))
        tv.camera_index = int(v.get("camera_index", 0))
        tv.camera_model_type = int(v.get("camera_model_type", 0))
        ct = v.get("crop_transform", (1.0, 1.0, 0.0, 0.0, 0.0))
        cr = v.get("crop_rotation", (1.0, 0.0, 0.0, 1.0))
        for k in range(5):
            tv.crop_transform[k] = ct[k]
        for k in range(4):
            tv.crop_rotation[k] = cr[k]
    return d


def desc_for_scene(scene, **overrides):
    """TripsSplatDesc for a trips_amd.scenes.Scene; keyword overrides go to make_desc."""
    kw = dict(num_points=scene.num_points, num_texels=int(scene.texture.shape[1]),
              num_channels=scene.num_channels, num_layers=scene.num_layers, list_depth=scene.list_depth,
              views=scene.views, num_images=int(scene.poses_se3.shape[0]),
              num_cameras=int(scene.intrinsics.shape[0]))
    kw.update(overrides)
    return make_desc(**kw)


def pyramid_pixels(desc):
    """(sizes, offsets, P): per-layer (w, h), first pixel number of each layer, total pixel count."""
    sizes = layer_sizes(desc.views[0].w, desc.views[0].h, desc.num_layers, bool(desc.floor_layer_sizes))
    offs = [0]
    for (w, h) in sizes:
        offs.append(offs[-1] + w * h)
    return sizes, offs[:-1], offs[-1]
