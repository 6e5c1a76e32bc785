/*
 * trips_splat.h -- C ABI of the MI355X-native TRIPS point-splat rasterizer.
 *
 * Plain pointers and sizes only; no torch / C++ types cross this boundary.
 * Every pointer named "device" is a HIP device pointer; every entry point
 * enqueues its work on the hipStream_t passed as `stream` (given as void* so
 * that this header needs no HIP include) and returns without synchronising.
 * Nothing here allocates device memory: the caller passes outputs, a saved-
 * state buffer and a workspace whose sizes come from the *_size queries.
 *
 * The entry points replace, for the pinhole / TILED_BILINEAR_BLEND "new impl"
 * path of the reference, the following reference interfaces:
 *
 *   trips_splat_forward   <- BlendPointCloudForward   (src/lib/rendering/PointRenderer.cu:676-750,1139-1190)
 *                            + PointRendererCache::RenderFast16 (src/lib/rendering/RenderForward.cu:1065-1394)
 *   trips_splat_backward  <- BlendPointCloudBackward  (src/lib/rendering/PointRenderer.cu:1232-1427)
 *                            + PointRendererCache::BlendBackwardsBilinearFast (src/lib/rendering/RenderBackward.cu:621-693)
 *   trips_adam_step_fused <- torch::optim::MyAdam::step (src/lib/models/MyAdam.cu:164-345)
 *   trips_apply_tangent   <- ApplyTangentToPose       (src/lib/rendering/PointRenderer.cu:1428-1456)
 *   TripsView             <- ReducedImageInfo         (src/lib/data/SceneData.h:40-61)
 *   TripsSplatDesc flags  <- RenderParams             (src/lib/data/Settings.h:19-83)
 */
#ifndef TRIPS_SPLAT_H
#define TRIPS_SPLAT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TRIPS_MAX_LAYERS 8 /* max_layers, src/lib/rendering/RenderConstants.h:38 */
#define TRIPS_MAX_VIEWS 16
/* 2: TripsSplatGrads gained clear_block_sums, TripsUnetDesc gained weights_packed, and the layouts of the saved state
 * and the workspace changed (a saved state or workspace sized by a version-1 library does not fit). A caller built
 * against another version is refused by every entry point that takes a descriptor. */
#define TRIPS_ABI_VERSION 2

/* status codes (the reference aborts through SAIGA_ASSERT instead) */
enum {
    TRIPS_OK                  = 0,
    TRIPS_ERR_INVALID_ARG     = 1,
    TRIPS_ERR_UNSUPPORTED     = 2,
    TRIPS_ERR_WORKSPACE_SMALL = 3,
    TRIPS_ERR_HIP             = 4,
    TRIPS_ERR_LIST_OVERFLOW   = 5 /* reported by trips_splat_check only */
};

/* How the background is weighted in the forward pass.
 * REFERENCE : transmittance *before* the last retained entry, as the forward kernel is
 *             written (src/lib/rendering/RenderForward.cu:1002-1022).
 * CONSISTENT: transmittance *after* the last retained entry, which is what the
 *             reference's own backward differentiates (src/lib/rendering/RenderBackward.cu:302-308)
 *             and what its older kernel computes (src/lib/rendering/RenderForward.cu:2955-2989). */
enum { TRIPS_BG_REFERENCE = 0, TRIPS_BG_CONSISTENT = 1 };

/* Output image layout. CHW: [B,C,H,W] (reference train==true). HWC: [B,H,W,C] (train==false,
 * src/lib/rendering/PointRenderer.cu:458-475). */
enum { TRIPS_LAYOUT_CHW = 0, TRIPS_LAYOUT_HWC = 1 };

/* One rendered view; mirrors ReducedImageInfo (src/lib/data/SceneData.h:40-61).
 * Only camera_model_type == 0 (PINHOLE_DISTORTION) is supported. */
typedef struct TripsView {
    int32_t w, h;
    int32_t image_index;       /* row of poses_se3 / pose gradient */
    int32_t camera_index;      /* row of intrinsics */
    int32_t camera_model_type; /* must be 0 */
    float crop_transform[5];   /* fx fy cx cy s */
    float crop_rotation[4];    /* row-major 2x2: r00 r01 r10 r11 */
} TripsView;

typedef struct TripsSplatDesc {
    int32_t abi_version;  /* TRIPS_ABI_VERSION */
    int32_t num_points;   /* N */
    int32_t num_texels;   /* columns of texture / confidence */
    int32_t num_channels; /* C: 3, 4, 6, 8 or 16 (RenderForward.cu:1281-1331) */
    int32_t num_layers;   /* L in 1..8 */
    int32_t list_depth;   /* K: 8 or 16 (reference fixes 16, PointRenderer.h:178) */
    int32_t num_views;    /* B in 1..TRIPS_MAX_VIEWS; all views share w,h */
    int32_t num_images;   /* rows of poses_se3 */
    int32_t num_cameras;  /* rows of intrinsics */
    int32_t train;        /* 1: write saved state for backward, honour dropout */
    int32_t layout;       /* TRIPS_LAYOUT_* of the output images */
    int32_t floor_layer_sizes; /* 1: h/2 per level ("MultiScaleUnet2d"), 0: ceil (PointRenderer.cu:385-394) */
    int32_t background_mode;   /* TRIPS_BG_* */
    int32_t drop_out_points_by_radius;
    float drop_out_radius_threshold;
    float dist_cutoff;
    int32_t viewer_only; /* 1: cull points whose confidence < stability_cutoff_value (RenderForward.cu:122-130,226-230) */
    float stability_cutoff_value;
    /* capacity, in list entries (a point covers four pixels per layer it is written to), of the list storage of ONE
     * view; 0 = worst case 4*N*L. The storage itself keeps one key per four entries. */
    int64_t max_list_entries;
    TripsView views[TRIPS_MAX_VIEWS];
} TripsSplatDesc;

/* Scene tensors; device pointers, same layouts as the reference's tensors. */
typedef struct TripsSplatIn {
    const float* position;    /* [N,4]  xyz + drop-out radius (NeuralPointCloudCuda.cpp:62) */
    const float* point_size;  /* [N]    raw value; softplus applied inside (RenderForward.cu:248) */
    const int32_t* index;     /* [N]    column of texture / confidence */
    const float* texture;     /* [C,T] */
    const float* confidence;  /* [T]    already sigmoid(10 x) (NeuralTexture.h:40-43) */
    const float* background;  /* [C] */
    const double* poses_se3;  /* [F,8]  qx qy qz qw tx ty tz pad, world->camera (NeuralStructure.cpp:20-35) */
    const float* intrinsics;  /* [Cam,13] fx fy cx cy s + 8 distortion (NeuralStructure.cpp:104-117) */
    const float* dropout;     /* [B,N] or NULL; a point with value 1 is skipped (RenderForward.cu:240-244) */
    const float* displacement; /* [B,N,3] or NULL; view b renders xyz + displacement[b] (dynamic_refinement_t,
                                  PointRenderer.cu:703-713, NeuralPointCloudCuda.h:260-270); no gradient is
                                  returned for it, as in the reference (PointRenderer.cu:243-252 is compiled out) */
} TripsSplatIn;

typedef struct TripsSplatOut {
    float* image[TRIPS_MAX_LAYERS]; /* per layer [B,C,H_l,W_l] or [B,H_l,W_l,C] */
    void* saved;                    /* trips_splat_saved_size bytes; may be NULL when train == 0 */
} TripsSplatOut;

/* Gradient outputs; the kernels ADD into these, the caller zeroes them first
 * (PointRendererCache::Build(info,false), PointRenderer.cu:226-272). NULL = not requested, where allowed.
 * With overwrite_point_grads != 0 the four per-point outputs (d_texture, d_confidence, d_position, d_point_size) are
 * WRITTEN instead: every element receives its value, zero where no gradient arrives (.w of d_position too), so the
 * caller may pass uninitialised memory and skips four fills and the kernel the reads of a read-modify-write;
 * d_background, d_pose and d_intrinsics are added to in either mode; with clear_block_sums != 0 the call clears them
 * itself first (all of d_background, every row of d_pose [num_images, 6] and of d_intrinsics [num_cameras, 13]), which
 * spares the caller three fill launches per step. */
typedef struct TripsSplatGrads {
    float* d_texture;     /* [C,T]   required */
    float* d_confidence;  /* [T]     required */
    float* d_background;  /* [C]     required */
    float* d_position;    /* [N,4]   or NULL (xyz; .w untouched when adding) */
    float* d_point_size;  /* [N]     or NULL; NULL also drops the layer factor from d_confidence and
                                      d_position exactly as RenderBackward.cu:366-372 does */
    double* d_pose;       /* [F,6]   or NULL; translation first, rotation last */
    float* d_intrinsics;  /* [Cam,13] or NULL */
    int32_t overwrite_point_grads; /* 0 = add into everything (the reference's contract); 1 = see above */
    int32_t clear_block_sums;      /* 1 = d_background, d_pose, d_intrinsics are cleared by the call before it adds */
} TripsSplatGrads;

typedef struct TripsCtx TripsCtx;

const char* trips_version(void);
/* message of the last error raised on the calling thread */
const char* trips_last_error_string(void);

int trips_ctx_create(TripsCtx** out_ctx, int device);
int trips_ctx_destroy(TripsCtx* ctx);

/* Layer sizes of the pyramid for desc->width/height rules; w[l], h[l] for l < num_layers. Host only. */
int trips_splat_layer_sizes(const TripsSplatDesc* desc, int32_t* w, int32_t* h);
/* Bytes of workspace / saved-state the caller must provide. Host only. */
int trips_splat_workspace_size(const TripsSplatDesc* desc, size_t* bytes);
int trips_splat_saved_size(const TripsSplatDesc* desc, size_t* bytes);

int trips_splat_forward(TripsCtx* ctx, const TripsSplatDesc* desc, const TripsSplatIn* in, const TripsSplatOut* out,
                        void* workspace, size_t workspace_bytes, void* stream);

/* `in` must hold what the forward saw: besides background, poses and intrinsics the backward reads position, index,
 * point_size and displacement again (the reference's backward likewise reads the points again, RenderBackward.cu:410,424). */
int trips_splat_backward(TripsCtx* ctx, const TripsSplatDesc* desc, const TripsSplatIn* in, const void* saved,
                         const float* const grad_image[TRIPS_MAX_LAYERS], const TripsSplatGrads* grads,
                         void* workspace, size_t workspace_bytes, void* stream);

/* The forward for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc) and have no workspace to hand over. It has no counterpart in the reference, whose
 * forward allocates through libtorch's caching allocator (PointRenderer.cu:276-528). Same arguments, results and
 * errors as trips_splat_forward, except that the workspace is a static array inside the library:
 * TRIPS_STATIC_WORKSPACE_BYTES per GPU, present from library load until the process ends. A scene whose
 * trips_splat_workspace_size exceeds that is rejected with TRIPS_ERR_WORKSPACE_SMALL (nothing is launched);
 * desc->max_list_entries lowers the need. The call allocates nothing on the host or the device and creates no
 * events (the per-kernel timer of trips_profile_enable does not cover it). All calls on one GPU share the one array:
 * calls that overlap on the same GPU (two streams, two threads, two contexts) race; calls on one stream are ordered
 * and each call clears the counters it relies on. trips_splat_check_static(ctx, stream) reports on the last such call.
 * The caller still passes the images and, with desc->train, the saved state. */
#define TRIPS_STATIC_WORKSPACE_BYTES (64u << 20)
int trips_splat_forward_static(TripsCtx* ctx, const TripsSplatDesc* desc, const TripsSplatIn* in, const TripsSplatOut* out,
                               void* stream);

/* Synchronises `stream` and reports what the last forward that used `workspace` found on the device: a list
 * overflow (TRIPS_ERR_LIST_OVERFLOW, only possible when desc->max_list_entries was set below the worst case) or
 * values of `index` outside [0, num_texels) (TRIPS_ERR_INVALID_ARG; such points are left out of the image, the
 * reference reads past its tables). */
int trips_splat_check(TripsCtx* ctx, const void* workspace, void* stream);

/* The same for the last trips_splat_forward_static on this context's GPU (its workspace is inside the library). */
int trips_splat_check_static(TripsCtx* ctx, void* stream);

/* Counters of the last forward of view `view` kept in the saved state: [0]=valid points, [1]=E list entries,
 * [2]=R retained entries, [3]=P pyramid pixels. Synchronises `stream`. */
int trips_splat_counters(TripsCtx* ctx, const TripsSplatDesc* desc, const void* saved, int view, int64_t counters[4],
                         void* stream);

/* Debug / parity export: writes for view `view` the sorted, depth-limited per-pixel point-id lists as a dense
 * [P,K] int32 array (-1 padded; all min(len,K) sorted entries), the per-pixel number of retained entries [P]
 * (those the blend kept, transmittance >= 0.001) and the per-pixel list length [P] (before the top-K cut; a length
 * above 4 194 303 is reported as that number).
 * Pixels are numbered layer by layer, row-major inside a layer. Any of the three may be NULL. */
int trips_splat_export_lists(TripsCtx* ctx, const TripsSplatDesc* desc, const void* saved, int view,
                             int32_t* device_lists, int32_t* device_retained, int32_t* device_lengths, void* stream);

/* Per-point projection records of view `view` from the saved state, as the reference keeps them in
 * temp_full_buffer / temp_depth_buffer / temp_max_layer_buffer (RenderForward.cu:1077-1083):
 * ip [N,2], depth [N] (-1 = culled), size_px [N], max_layer [N]. Any may be NULL. */
int trips_splat_export_points(TripsCtx* ctx, const TripsSplatDesc* desc, const void* saved, int view, float* device_ip,
                              float* device_depth, float* device_size_px, int32_t* device_max_layer, void* stream);

/* ---- fused Adam over several parameter tensors (MyAdam.cu:41-88) ---- */
enum { TRIPS_DTYPE_F32 = 0, TRIPS_DTYPE_F64 = 1 };
enum { TRIPS_STEPS_I64 = 0, TRIPS_STEPS_I32 = 1 };

typedef struct TripsAdamTensor {
    void* weights;        /* [n] f32 or f64 (master weights, updated in place) */
    const void* grads;    /* [n] same dtype as weights */
    float* first_moment;  /* [n] f32 */
    float* second_moment; /* [n] f32 */
    void* steps;          /* [n] per-element step counter: int64 (the reference's state tensor, MyAdam.cu:188-205) or int32 */
    int64_t n;
    int32_t dtype; /* TRIPS_DTYPE_* */
    float lr;
    float beta1, beta2, eps;
    float relative_weight_decay, absolute_weight_decay;
    float weight_clipping_magnitude; /* 0 = off */
    float lower_lr_bound, upper_lr_bound; /* 0 and FLT_MAX unless adabound (MyAdam.cu:213-221) */
    float loss_scale;                     /* 1 (MyAdam.cu:231) */
    int32_t steps_dtype;                  /* TRIPS_STEPS_*: int32 counters save 8 of the 44 bytes an updated element moves */
} TripsAdamTensor;

/* `tensors` is a HOST array of n_tensors descriptors; one launch covers all of them. */
int trips_adam_step_fused(TripsCtx* ctx, const TripsAdamTensor* tensors, int n_tensors, void* stream);

/* The same step (MyAdam.cu:41-88,164-345) for the four parameter tensors of a point cloud at once, optimiser state
 * packed per point: tensors[0] = t_position [N,4], tensors[1] = t_point_size [N] (NeuralPointCloudCuda.cpp:103-108),
 * tensors[2] = texture [C,N], tensors[3] = confidence [N] (NeuralTexture.cpp:53-55), all float32; their first_moment /
 * second_moment / steps fields are ignored. `state`: N rows of `row_bytes` bytes (a multiple of 128), zero-filled by
 * the caller before the first step; a row holds {first moment f32, second moment f32, step counter i32} for the
 * point's 6 + C elements in the order position xyzw, size, descriptors 0..C-1, confidence. An element is updated
 * exactly as by trips_adam_step_fused (bit-identical weights and moments); a point whose gradients are all zero is
 * skipped without its row being read, which per-tensor state arrays cannot offer: there the state of such a point
 * shares every line with its neighbours'. Point removal / addition (MyAdam.cu:346-415) = row selection / appended
 * zero rows. */
int trips_adam_points_state_size(int num_points, int num_channels, size_t* bytes, int* row_bytes);
int trips_adam_step_points(TripsCtx* ctx, const TripsAdamTensor tensors[4], int num_points, int num_channels, void* state,
                           void* stream);

/* pose <- se3_exp(t with rotation part * 0.1) * pose; t <- 0   (PointRenderer.cu:1428-1447)
 * tangent [F,6] f64 device, poses_se3 [F,8] f64 device. */
int trips_apply_tangent(TripsCtx* ctx, double* tangent, double* poses_se3, int n, void* stream);

/* ---- per-kernel timing (stands in for the reference's CudaTimerSystem scopes "Count Render", "Splat",
 * "FastSortAndBlendMore", "BlendBackwardsBilinearFast"; RenderForward.cu:1090,1238,1271, PointRenderer.cu:1338) ----
 * While enabled, every kernel the library launches through `ctx` is bracketed by HIP events on its stream.
 * trips_profile_read waits for those events, returns per kernel name the summed milliseconds and the number of
 * launches since the last read, and resets the accumulation. names[i] point to static strings. */
#define TRIPS_PROFILE_MAX_KERNELS 32
int trips_profile_enable(TripsCtx* ctx, int enabled);
int trips_profile_read(TripsCtx* ctx, int* n, const char* names[TRIPS_PROFILE_MAX_KERNELS],
                       float ms[TRIPS_PROFILE_MAX_KERNELS], int launches[TRIPS_PROFILE_MAX_KERNELS]);

/* ---- a knob for tests (no counterpart in the reference) ----
 * The backward keeps the (point, layer) rows between its two passes in one of two forms and chooses per view on the
 * device: rows of all pairs cleared beforehand, or a flag byte per row for views in which few pairs are retained by a
 * pixel. Both give the same gradients bit for bit. mode: 0 = choose per view (default), 1 = always the first form,
 * 2 = always the second. Applies to the backward calls made through `ctx` from then on. */
int trips_splat_pair_rows_mode(TripsCtx* ctx, int mode);

#ifdef __cplusplus
}
#endif
#endif /* TRIPS_SPLAT_H */
