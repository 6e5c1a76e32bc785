"""Host-side mirror of the reference's render operator over the C ABI.

Same names and argument meaning as the reference (paths relative to the reference checkout):
  ReducedImageInfo     src/lib/data/SceneData.h:40-61
  RenderParams         src/lib/data/Settings.h:19-83 (the fields the splat path reads)
  NeuralRenderInfo     src/lib/rendering/PointRenderer.h:23-34
  PointRendererCache   src/lib/rendering/PointRenderer.h:120-232 (size-keyed buffers, PointRenderer.cu:276-416)
  PointRender          src/lib/rendering/PointRenderer.h:39-47, RenderInfo.cpp:44-80 (autograd function)
  BlendPointCloud      src/lib/rendering/PointRenderer.h:53, RenderInfo.cpp:27-40

torch is used for device memory, streams and the autograd graph only; all computation happens in
libtrips_splat.so. There is no fallback path: without the library (or without a GPU) these calls raise.
"""
import ctypes as C
from dataclasses import dataclass, field
from typing import List, Optional

import torch

from . import _lib, abi


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream_ptr(device):
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class SplatContext:
    """Thin object wrapper of the C entry points; one per device."""

    def __init__(self, device=0):
        self.lib = _lib.load()
        if not torch.cuda.is_available():
            raise RuntimeError("trips_amd needs a GPU: the splat path has no CPU implementation")
        self.device = torch.device("cuda", device if isinstance(device, int) else torch.device(device).index or 0)
        self.ctx = C.c_void_p()
        _lib.check(self.lib.trips_ctx_create(C.byref(self.ctx), self.device.index))

    def __del__(self):
        try:
            if getattr(self, "ctx", None):
                self.lib.trips_ctx_destroy(self.ctx)
        except Exception:
            pass

    # ---- sizes ----
    def workspace_size(self, desc):
        b = C.c_size_t(0)
        _lib.check(self.lib.trips_splat_workspace_size(C.byref(desc), C.byref(b)))
        return int(b.value)

    def saved_size(self, desc):
        b = C.c_size_t(0)
        _lib.check(self.lib.trips_splat_saved_size(C.byref(desc), C.byref(b)))
        return int(b.value)

    def alloc_bytes(self, n):
        # torch's allocator returns 512-byte aligned blocks; the ABI asks for 256
        return torch.empty(max(int(n), 256), dtype=torch.uint8, device=self.device)

    def alloc_images(self, desc, fill=None):
        sizes, _, _ = abi.pyramid_pixels(desc)
        B, Cn = desc.num_views, desc.num_channels
        out = []
        for (w, h) in sizes:
            shape = (B, Cn, h, w) if desc.layout == abi.TRIPS_LAYOUT_CHW else (B, h, w, Cn)
            t = torch.empty(shape, dtype=torch.float32, device=self.device)
            if fill is not None:
                t.fill_(fill)
            out.append(t)
        return out

    # ---- forward / backward ----
    @staticmethod
    def make_in(position, point_size, index, texture, confidence, background, poses_se3, intrinsics, dropout=None,
                displacement=None):
        tin = abi.TripsSplatIn()
        tin.position = _ptr(position)
        tin.point_size = _ptr(point_size)
        tin.index = _ptr(index)
        tin.texture = _ptr(texture)
        tin.confidence = _ptr(confidence)
        tin.background = _ptr(background)
        tin.poses_se3 = _ptr(poses_se3)
        tin.intrinsics = _ptr(intrinsics)
        tin.dropout = _ptr(dropout)
        tin.displacement = _ptr(displacement)
        return tin

    def forward(self, desc, tin, images, saved, workspace):
        out = abi.TripsSplatOut()
        for l, im in enumerate(images):
            out.image[l] = im.data_ptr()
        out.saved = _ptr(saved)
        _lib.check(self.lib.trips_splat_forward(self.ctx, C.byref(desc), C.byref(tin), C.byref(out), _ptr(workspace),
                                                workspace.numel(), _stream_ptr(self.device)))

    def forward_static(self, desc, tin, images, saved):
        """The forward on the library's own static workspace (abi.TRIPS_STATIC_WORKSPACE_BYTES per GPU): allocates
        nothing; raises TripsError(TRIPS_ERR_WORKSPACE_SMALL) for scenes that need more. Calls on one GPU must not
        overlap."""
        out = abi.TripsSplatOut()
        for l, im in enumerate(images):
            out.image[l] = im.data_ptr()
        out.saved = _ptr(saved)
        _lib.check(self.lib.trips_splat_forward_static(self.ctx, C.byref(desc), C.byref(tin), C.byref(out),
                                                       _stream_ptr(self.device)))

    def backward(self, desc, tin, saved, grad_images, grads, workspace=None, overwrite_point_grads=False,
                 clear_block_sums=False):
        """Adds into `grads` (zeroed by the caller); with overwrite_point_grads the four per-point outputs
        (d_texture, d_confidence, d_position, d_point_size) are written instead and may be uninitialised; with
        clear_block_sums the call clears d_background, d_pose and d_intrinsics itself before it adds to them."""
        arr = (C.c_void_p * abi.TRIPS_MAX_LAYERS)()
        for l, g in enumerate(grad_images):
            arr[l] = g.data_ptr()
        tg = abi.TripsSplatGrads()
        for k in ("d_texture", "d_confidence", "d_background", "d_position", "d_point_size", "d_pose",
                  "d_intrinsics"):
            setattr(tg, k, _ptr(grads.get(k)))
        tg.overwrite_point_grads = int(bool(overwrite_point_grads))
        tg.clear_block_sums = int(bool(clear_block_sums))
        _lib.check(self.lib.trips_splat_backward(self.ctx, C.byref(desc), C.byref(tin), _ptr(saved), arr,
                                                 C.byref(tg), _ptr(workspace),
                                                 0 if workspace is None else workspace.numel(),
                                                 _stream_ptr(self.device)))

    def check(self, workspace):
        """What the last forward on `workspace` found on the device (list overflow, bad descriptor columns); raises."""
        if workspace is None:
            raise ValueError("check(None): pass the workspace of the forward, or call check_static() after forward_static")
        _lib.check(self.lib.trips_splat_check(self.ctx, _ptr(workspace), _stream_ptr(self.device)))

    def check_static(self):
        """The same for the last forward_static on this GPU."""
        _lib.check(self.lib.trips_splat_check_static(self.ctx, _stream_ptr(self.device)))

    def counters(self, desc, saved, view=0):
        c = (C.c_int64 * 4)()
        _lib.check(self.lib.trips_splat_counters(self.ctx, C.byref(desc), _ptr(saved), view, c,
                                                 _stream_ptr(self.device)))
        return dict(valid=int(c[0]), E=int(c[1]), R=int(c[2]), P=int(c[3]))

    def export_lists(self, desc, saved, view=0):
        _, _, P = abi.pyramid_pixels(desc)
        lists = torch.empty((P, desc.list_depth), dtype=torch.int32, device=self.device)
        retained = torch.empty(P, dtype=torch.int32, device=self.device)
        lengths = torch.empty(P, dtype=torch.int32, device=self.device)
        _lib.check(self.lib.trips_splat_export_lists(self.ctx, C.byref(desc), _ptr(saved), view, _ptr(lists),
                                                     _ptr(retained), _ptr(lengths), _stream_ptr(self.device)))
        return lists, retained, lengths

    def export_points(self, desc, saved, view=0):
        N = desc.num_points
        ip = torch.empty((N, 2), dtype=torch.float32, device=self.device)
        depth = torch.empty(N, dtype=torch.float32, device=self.device)
        size_px = torch.empty(N, dtype=torch.float32, device=self.device)
        max_layer = torch.empty(N, dtype=torch.int32, device=self.device)
        _lib.check(self.lib.trips_splat_export_points(self.ctx, C.byref(desc), _ptr(saved), view, _ptr(ip),
                                                      _ptr(depth), _ptr(size_px), _ptr(max_layer),
                                                      _stream_ptr(self.device)))
        return ip, depth, size_px, max_layer

    def pair_rows_mode(self, mode):
        """For tests: 0 = the backward chooses per view how it keeps its (point, layer) rows, 1 = rows of all pairs
        cleared beforehand, 2 = a flag byte per row. Same gradients either way."""
        _lib.check(self.lib.trips_splat_pair_rows_mode(self.ctx, int(mode)))

    # ---- per-kernel timing ----
    def profile_enable(self, on=True):
        _lib.check(self.lib.trips_profile_enable(self.ctx, int(bool(on))))

    def profile_read(self):
        """{kernel name: (milliseconds summed over launches, launches)} since the last read."""
        n = C.c_int(0)
        names = (C.c_char_p * abi.TRIPS_PROFILE_MAX_KERNELS)()
        ms = (C.c_float * abi.TRIPS_PROFILE_MAX_KERNELS)()
        launches = (C.c_int * abi.TRIPS_PROFILE_MAX_KERNELS)()
        _lib.check(self.lib.trips_profile_read(self.ctx, C.byref(n), names, ms, launches))
        return {names[i].decode(): (float(ms[i]), int(launches[i])) for i in range(n.value)}

    # ---- optimiser pieces ----
    def adam_step(self, tensor_descs):
        """tensor_descs: sequence of abi.TripsAdamTensor (device pointers)."""
        n = len(tensor_descs)
        arr = (abi.TripsAdamTensor * n)(*tensor_descs)
        _lib.check(self.lib.trips_adam_step_fused(self.ctx, arr, n, _stream_ptr(self.device)))

    def adam_points_state_size(self, num_points, num_channels):
        """(bytes, bytes per row) of the packed optimiser state of a point cloud."""
        b, row = C.c_size_t(0), C.c_int(0)
        _lib.check(self.lib.trips_adam_points_state_size(int(num_points), int(num_channels), C.byref(b), C.byref(row)))
        return b.value, row.value

    def adam_step_points(self, tensor_descs, num_points, num_channels, state):
        """tensor_descs: four abi.TripsAdamTensor (position, point size, descriptors, confidence); state: the packed
        rows (a device tensor of adam_points_state_size bytes, zero before the first step)."""
        arr = (abi.TripsAdamTensor * 4)(*tensor_descs)
        _lib.check(self.lib.trips_adam_step_points(self.ctx, arr, int(num_points), int(num_channels), _ptr(state),
                                                   _stream_ptr(self.device)))

    def apply_tangent(self, tangent, poses_se3):
        assert tangent.dtype == torch.float64 and poses_se3.dtype == torch.float64
        assert tangent.is_contiguous() and poses_se3.is_contiguous()
        _lib.check(self.lib.trips_apply_tangent(self.ctx, _ptr(tangent), _ptr(poses_se3), int(tangent.shape[0]),
                                                _stream_ptr(self.device)))


_contexts = {}


def get_context(device=0):
    idx = device if isinstance(device, int) else (torch.device(device).index or 0)
    if idx not in _contexts:
        _contexts[idx] = SplatContext(idx)
    return _contexts[idx]


# ----------------------------------------------------------------------------------------------------------------
# reference-shaped operator surface

@dataclass
class ReducedImageInfo:
    w: int = 0
    h: int = 0
    image_index: int = -1
    camera_index: int = -1
    camera_model_type: int = 0  # CameraModel::PINHOLE_DISTORTION
    crop_transform: tuple = (1.0, 1.0, 0.0, 0.0, 0.0)  # fx fy cx cy s
    crop_rotation: tuple = (1.0, 0.0, 0.0, 1.0)  # row-major 2x2

    def as_view(self):
        return dict(w=self.w, h=self.h, image_index=self.image_index, camera_index=self.camera_index,
                    camera_model_type=self.camera_model_type, crop_transform=self.crop_transform,
                    crop_rotation=self.crop_rotation)


@dataclass
class RenderParams:
    """Defaults as in the reference (Settings.h:27-83) for the fields the splat path reads; render_mode 4 with
    use_layer_point_size and render_points_in_all_lower_resolutions is the only path implemented."""
    dropout: float = 0.25
    drop_out_radius_threshold: float = 0.6
    drop_out_points_by_radius: bool = True
    num_texture_channels: int = 4
    dist_cutoff: float = 20.0
    stability_cutoff_value: float = 10000.0
    viewer_only: bool = False
    render_mode: int = 4  # TILED_BILINEAR_BLEND
    use_layer_point_size: bool = True
    combine_lists: bool = False
    render_points_in_all_lower_resolutions: bool = True
    normalize_grads: bool = False
    # never written by the reference's kernels on this path either (RenderForward.cu:43): returned as zeros after
    # the L images so that the output arity matches (PointRenderer.cu:482-505,1183-1190)
    add_depth_to_network: bool = False
    output_background_mask: bool = False
    # not in the reference: see TRIPS_BG_* in include/trips_splat.h; list depth is fixed to 16 there
    background_mode: int = abi.TRIPS_BG_REFERENCE
    max_pixels_per_list: int = 16
    floor_layer_sizes: bool = False  # network_version == "MultiScaleUnet2d" (PointRenderer.cu:385-394)


class PointRendererCache:
    """Workspace kept between calls, re-allocated when the size key changes (PointRenderer.cu:285-309)."""

    def __init__(self):
        self.cache_size = None
        self.workspace = None
        self.dropout_points = None

    def build(self, ctx, desc, train, dropout):
        key = (desc.num_channels, desc.num_points, desc.num_layers, desc.num_views, desc.views[0].h, desc.views[0].w,
               desc.list_depth, int(train))
        need = ctx.workspace_size(desc)
        if key != self.cache_size or self.workspace is None or self.workspace.numel() < need:
            self.workspace = ctx.alloc_bytes(need)
            self.cache_size = key
            self.dropout_points = None
        if train and dropout > 0:
            if self.dropout_points is None:
                self.dropout_points = torch.empty((desc.num_views, desc.num_points), dtype=torch.float32,
                                                  device=ctx.device)
            self.dropout_points.bernoulli_(dropout)  # PointRenderer.cu:516-521
        else:
            self.dropout_points = None


class NeuralRenderInfo:
    def __init__(self, scene=None, images: Optional[List[ReducedImageInfo]] = None, params: RenderParams = None,
                 num_layers=1, train=True, current_epoch=0, timer_system=None, cache: PointRendererCache = None):
        self.scene = scene
        self.images = images if images is not None else []
        self.params = params if params is not None else RenderParams()
        self.num_layers = num_layers
        self.train = train
        self.current_epoch = current_epoch
        self.timer_system = timer_system  # accepted for interface parity; timing is done with HIP events
        self.cache = cache


def _desc_from_info(info, texture):
    sc, p = info.scene, info.params
    if p.render_mode != 4 or not p.use_layer_point_size or not p.render_points_in_all_lower_resolutions \
            or p.combine_lists:
        raise NotImplementedError("only render_mode 4 (TILED_BILINEAR_BLEND) with use_layer_point_size, "
                                  "render_points_in_all_lower_resolutions and !combine_lists is implemented")
    return abi.make_desc(
        num_points=int(sc.point_cloud_cuda.t_position.shape[0]), num_texels=int(texture.shape[1]),
        num_channels=int(texture.shape[0]), num_layers=info.num_layers, list_depth=p.max_pixels_per_list,
        views=[im.as_view() for im in info.images], num_images=int(sc.poses.poses_se3.shape[0]),
        num_cameras=int(sc.intrinsics.intrinsics.shape[0]), train=info.train, floor_layer_sizes=p.floor_layer_sizes,
        background_mode=p.background_mode, drop_out_points_by_radius=p.drop_out_points_by_radius,
        drop_out_radius_threshold=p.drop_out_radius_threshold, dist_cutoff=p.dist_cutoff, viewer_only=p.viewer_only,
        stability_cutoff_value=p.stability_cutoff_value)


class PointRender(torch.autograd.Function):
    """forward(texture [C,N], background_color [C], points [N,4], pose_tangents [F,6] f64, intrinsics [Cam,13],
    confidence [1,N], dynamic_refinement, layer_value_of_point [N,1], info) -> one tensor [B,C,H_l,W_l] per layer;
    backward returns the 8 gradients in that order plus None for info."""

    @staticmethod
    def forward(ctx, texture, background_color, points, pose_tangents, intrinsics, confidence, dynamic_refinement,
                layer_value_of_point, info):
        sc = info.scene
        sctx = get_context(texture.device)
        desc = _desc_from_info(info, texture)
        if info.cache is None:
            info.cache = PointRendererCache()
        cache = info.cache
        cache.build(sctx, desc, info.train, info.params.dropout if info.train else 0.0)
        displacement = None
        if dynamic_refinement is not None and dynamic_refinement.dim() > 1:  # a [1] dummy otherwise, PointRenderer.cu:705-706
            if tuple(dynamic_refinement.shape) != (desc.num_views, desc.num_points, 3):
                raise ValueError(f"dynamic_refinement: expected [{desc.num_views}, {desc.num_points}, 3], "
                                 f"got {tuple(dynamic_refinement.shape)}")
            displacement = dynamic_refinement.detach().to(torch.float32).contiguous()
        tensors = dict(position=points.contiguous(), point_size=layer_value_of_point.contiguous(),
                       index=sc.point_cloud_cuda.t_index.contiguous(), texture=texture.contiguous(),
                       confidence=confidence.contiguous(), background=background_color.contiguous(),
                       poses_se3=sc.poses.poses_se3.contiguous(), intrinsics=intrinsics.contiguous(),
                       dropout=cache.dropout_points, displacement=displacement)
        tin = SplatContext.make_in(**tensors)
        images = sctx.alloc_images(desc)
        saved = sctx.alloc_bytes(sctx.saved_size(desc)) if info.train else None
        sctx.forward(desc, tin, images, saved, cache.workspace)
        ctx.render_info = info
        ctx.desc = desc
        ctx.tensors = tensors
        # the backward reads these again through their pointers: remember their version counters
        ctx.versions = {k: tensors[k]._version for k in ("position", "point_size", "index", "poses_se3", "intrinsics",
                                                          "displacement") if tensors[k] is not None}
        ctx.saved_state = saved
        ctx.shapes = dict(points=points.shape, layer=layer_value_of_point.shape, confidence=confidence.shape,
                          pose=pose_tangents.shape)
        ctx.image_shapes = [tuple(im.shape) for im in images]
        if not info.train:
            images = [im.permute(0, 3, 1, 2) for im in images]  # PointRenderer.cu:747-749
        extra = []
        for flag in (info.params.add_depth_to_network, info.params.output_background_mask):
            if flag:
                extra += [torch.zeros((im.shape[0], 1, im.shape[2], im.shape[3]), dtype=torch.float32, device=im.device)
                          for im in images]
        return tuple(images) + tuple(extra)

    @staticmethod
    def backward(ctx, *grad_output):
        info, desc, t = ctx.render_info, ctx.desc, ctx.tensors
        if ctx.saved_state is None:
            raise RuntimeError("backward needs a forward with info.train = True")
        for k, v in ctx.versions.items():
            if t[k]._version != v:
                raise RuntimeError(f"PointRender.backward: {k} was modified in place after the forward that this "
                                   "backward belongs to (the backward reads it again)")
        sctx = get_context(t["texture"].device)
        need = ctx.needs_input_grad
        dev = t["texture"].device
        # the four per-point outputs are written by the kernels (every element), the small ones are added to
        grads = dict(
            d_texture=torch.empty_like(t["texture"]),
            d_confidence=torch.empty(desc.num_texels, dtype=torch.float32, device=dev),
            d_background=torch.empty_like(t["background"]),
            d_position=torch.empty_like(t["position"]) if need[2] else None,
            d_point_size=torch.empty(desc.num_points, dtype=torch.float32, device=dev) if need[7] else None,
            d_pose=torch.empty((desc.num_images, 6), dtype=torch.float64, device=dev) if need[3] else None,
            d_intrinsics=torch.empty_like(t["intrinsics"]) if need[4] else None,
        )
        # a layer nobody consumed (a net with fewer levels than the pyramid) arrives without a gradient
        gi = [g.contiguous() if g is not None else torch.zeros(shape, dtype=torch.float32, device=dev)
              for g, shape in zip(grad_output[:desc.num_layers], ctx.image_shapes)]
        tin = SplatContext.make_in(**t)
        sctx.backward(desc, tin, ctx.saved_state, gi, grads, info.cache.workspace if info.cache else None,
                      overwrite_point_grads=True, clear_block_sums=True)
        d_layer = grads["d_point_size"].reshape(ctx.shapes["layer"]) if need[7] else None
        d_conf = grads["d_confidence"].reshape(ctx.shapes["confidence"])
        # order of PointRenderer.cu:1423-1426, then None for `info`
        return (grads["d_texture"], grads["d_background"], grads["d_position"], grads["d_pose"],
                grads["d_intrinsics"], d_conf, None, d_layer, None)


def BlendPointCloud(info: NeuralRenderInfo):
    """Render the scene into a batch of image pyramids (RenderInfo.cpp:27-40)."""
    sc = info.scene
    return list(PointRender.apply(sc.texture.texture, sc.texture.background_color, sc.point_cloud_cuda.t_position,
                                  sc.poses.tangent_poses, sc.intrinsics.intrinsics,
                                  sc.texture.confidence_value_of_point, sc.dynamic_refinement_t,
                                  sc.point_cloud_cuda.t_point_size, info))


# ---- minimal scene containers with the reference's member names ----

class _Namespace:
    def __init__(self, **kw):
        self.__dict__.update(kw)


class NeuralScene:
    """Holds the tensors the operator reads, under the reference's names
    (texture.texture / .background_color / .confidence_value_of_point, point_cloud_cuda.t_position / .t_point_size /
    .t_index, poses.poses_se3 / .tangent_poses, intrinsics.intrinsics, dynamic_refinement_t)."""

    def __init__(self, *, texture, background_color, confidence, position, point_size, index, poses_se3, intrinsics,
                 tangent_poses=None):
        dev = texture.device
        if tangent_poses is None:
            tangent_poses = torch.zeros((poses_se3.shape[0], 6), dtype=torch.float64, device=dev)
        self.texture = _Namespace(texture=texture, background_color=background_color,
                                  confidence_value_of_point=confidence)
        self.point_cloud_cuda = _Namespace(t_position=position, t_point_size=point_size, t_index=index)
        self.poses = _Namespace(poses_se3=poses_se3, tangent_poses=tangent_poses)
        self.intrinsics = _Namespace(intrinsics=intrinsics)
        self.dynamic_refinement_t = torch.zeros(1, device=dev)

    @staticmethod
    def from_arrays(scene, device="cuda", requires_grad=False):
        """Upload a trips_amd.scenes.Scene."""
        f = lambda a, dt=torch.float32: torch.as_tensor(a, dtype=dt).to(device).contiguous()
        ns = NeuralScene(texture=f(scene.texture), background_color=f(scene.background),
                         confidence=f(scene.confidence).reshape(1, -1), position=f(scene.position),
                         point_size=f(scene.point_size).reshape(-1, 1), index=f(scene.index, torch.int32).reshape(-1, 1),
                         poses_se3=f(scene.poses_se3, torch.float64), intrinsics=f(scene.intrinsics))
        if requires_grad:
            for t in (ns.texture.texture, ns.texture.background_color, ns.texture.confidence_value_of_point,
                      ns.point_cloud_cuda.t_position, ns.point_cloud_cuda.t_point_size, ns.poses.tangent_poses,
                      ns.intrinsics.intrinsics):
                t.requires_grad_(True)
        return ns
