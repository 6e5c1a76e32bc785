// Host side of the C ABI declared in include/trips_splat.h: argument checks, buffer carving, launches.
// Nothing here allocates device memory or synchronises, except the calls documented as synchronising
// (trips_splat_check, trips_splat_counters).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "splat_internal.h"

namespace trips
{
hipError_t launch_forward_view(const ForwardParams& p, int channels, bool train, bool first_view, hipStream_t stream,
                               Profiler* prof);
hipError_t launch_backward_view(const BackwardParams& p, int channels, hipStream_t stream, Profiler* prof);
hipError_t launch_adam(const TripsAdamTensor* tensors, int n_tensors, hipStream_t stream, Profiler* prof);
int adam_points_row_chunks(int channels);
hipError_t launch_adam_points(const TripsAdamTensor tensors[4], int num_points, int channels, void* state, hipStream_t stream,
                              Profiler* prof);
hipError_t launch_apply_tangent(double* tangent, double* poses, int n, hipStream_t stream);
hipError_t launch_export_points(const float* rec, int rec_floats, const float* prec, const int32_t* cid_of, int n, float* ip,
                                float* depth, float* size_px, int32_t* max_layer, hipStream_t stream);
hipError_t launch_sum_i32(const int32_t* v, long long n, unsigned mask, unsigned long long* out, hipStream_t stream);
hipError_t launch_export_lists(const PyramidGeom& g, int K, const int32_t* lists, const int32_t* retained,
                               const int32_t* pid_of, int32_t* out_lists, int32_t* out_retained,
                               int32_t* out_lengths, hipStream_t stream);
}  // namespace trips

using namespace trips;

namespace
{
thread_local char g_error[512] = "";

// Workspace of trips_splat_forward_static, the entry point for callers that cannot allocate: one array per GPU the
// library runs on, held until the process ends. Host code must not use this name as an address (it is a host-side
// stand-in); every use goes through the pointer hipGetSymbolAddress returns for the current device, kept in the
// context.
static __device__ __align__(256) unsigned char scratch[TRIPS_STATIC_WORKSPACE_BYTES];
}

namespace trips
{
int set_error(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}
}  // namespace trips

namespace
{
template <typename... A>
int fail(int code, const char* fmt, A... a)
{
    return trips::set_error(code, fmt, a...);
}

int hip_fail(hipError_t e, const char* what)
{
    return fail(TRIPS_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

bool channels_ok(int c) { return c == 3 || c == 4 || c == 6 || c == 8 || c == 16; }

int check_desc(const TripsSplatDesc* d)
{
    if (!d) return fail(TRIPS_ERR_INVALID_ARG, "desc is NULL");
    if (d->abi_version != TRIPS_ABI_VERSION)
        return fail(TRIPS_ERR_INVALID_ARG, "abi_version %d, library has %d", d->abi_version, TRIPS_ABI_VERSION);
    if (d->num_points < 0) return fail(TRIPS_ERR_INVALID_ARG, "num_points < 0");
    if (d->num_texels < 0) return fail(TRIPS_ERR_INVALID_ARG, "num_texels < 0");
    if (!channels_ok(d->num_channels))
        return fail(TRIPS_ERR_UNSUPPORTED, "num_channels %d not in {3,4,6,8,16}", d->num_channels);
    if (d->num_layers < 1 || d->num_layers > TRIPS_MAX_LAYERS)
        return fail(TRIPS_ERR_INVALID_ARG, "num_layers %d not in 1..%d", d->num_layers, TRIPS_MAX_LAYERS);
    if (d->list_depth != 8 && d->list_depth != 16)
        return fail(TRIPS_ERR_UNSUPPORTED, "list_depth %d not in {8,16}", d->list_depth);
    if (d->num_views < 1 || d->num_views > TRIPS_MAX_VIEWS)
        return fail(TRIPS_ERR_INVALID_ARG, "num_views %d not in 1..%d", d->num_views, TRIPS_MAX_VIEWS);
    if (d->num_images < 1 || d->num_cameras < 1) return fail(TRIPS_ERR_INVALID_ARG, "num_images / num_cameras < 1");
    if (d->layout != TRIPS_LAYOUT_CHW && d->layout != TRIPS_LAYOUT_HWC) return fail(TRIPS_ERR_INVALID_ARG, "layout");
    if (d->background_mode != TRIPS_BG_REFERENCE && d->background_mode != TRIPS_BG_CONSISTENT)
        return fail(TRIPS_ERR_INVALID_ARG, "background_mode");
    if (d->max_list_entries < 0) return fail(TRIPS_ERR_INVALID_ARG, "max_list_entries < 0");
    const int w = d->views[0].w, h = d->views[0].h;
    if (w < 1 || h < 1 || w > 32768 || h > 32768) return fail(TRIPS_ERR_INVALID_ARG, "view size %dx%d", w, h);
    for (int b = 0; b < d->num_views; ++b)
    {
        const TripsView& v = d->views[b];
        if (v.w != w || v.h != h) return fail(TRIPS_ERR_INVALID_ARG, "views must share one size");
        if (v.camera_model_type != 0)
            return fail(TRIPS_ERR_UNSUPPORTED, "camera_model_type %d: only pinhole+distortion (0)", v.camera_model_type);
        if (v.image_index < 0 || v.image_index >= d->num_images)
            return fail(TRIPS_ERR_INVALID_ARG, "view %d: image_index %d out of range", b, v.image_index);
        if (v.camera_index < 0 || v.camera_index >= d->num_cameras)
            return fail(TRIPS_ERR_INVALID_ARG, "view %d: camera_index %d out of range", b, v.camera_index);
    }
    // A (point, layer) pair is filed once (one bin entry, one key, one row of the backward), and the prefix sums over
    // the pairs are 32-bit: no scan may exceed the worst case of N L pairs, whatever the capacity the caller grants (a
    // smaller max_list_entries only drops entries, it does not shorten the scans). The list entries that the counters
    // report, four per pair, are counted in 64 bits.
    if ((long long)d->num_points * d->num_layers > 0x7fffffffll)
        return fail(TRIPS_ERR_UNSUPPORTED, "N*L = %lld (point, layer) pairs exceed 2^31-1", (long long)d->num_points * d->num_layers);
    if (d->max_list_entries > 4ll * 0x7fffffffll) return fail(TRIPS_ERR_UNSUPPORTED, "max_list_entries exceeds 4 (2^31-1)");
    {
        // one LDS counter per 32 x 32 tile of the pyramid in the binning kernels
        long long bins = 0;
        int cw = w, ch = h;
        for (int l = 0; l < d->num_layers; ++l)
        {
            bins += (long long)((cw + kTile - 1) / kTile) * ((ch + kTile - 1) / kTile);
            if (!d->floor_layer_sizes)
            {
                ch = (int)std::ceil(float(ch) / 2.f);
                cw = (int)std::ceil(float(cw) / 2.f);
            }
            else
            {
                ch = ch / 2;
                cw = cw / 2;
            }
        }
        if (bins > kMaxBins)
            return fail(TRIPS_ERR_UNSUPPORTED, "%lld tiles of 32x32 pixels, at most %d (about 4096 x 2700 pixels)", bins, kMaxBins);
    }
    return TRIPS_OK;
}

void make_geom(const TripsSplatDesc& d, PyramidGeom& g)
{
    int cw = d.views[0].w, ch = d.views[0].h;
    g.num_layers = d.num_layers;
    g.off[0]     = 0;
    g.bin_off[0] = 0;
    for (int l = 0; l < TRIPS_MAX_LAYERS; ++l)
    {
        if (l < d.num_layers)
        {
            g.w[l]           = cw;
            g.h[l]           = ch;
            g.off[l + 1]     = g.off[l] + cw * ch;
            g.tiles_x[l]     = (cw + kTile - 1) / kTile;
            g.tiles_y[l]     = (ch + kTile - 1) / kTile;
            g.bin_off[l + 1] = g.bin_off[l] + g.tiles_x[l] * g.tiles_y[l];
            g.tiles_x_magic[l] = g.tiles_x[l] > 0 ? ((1u << 30) + (uint32_t)g.tiles_x[l] - 1u) / (uint32_t)g.tiles_x[l] : 0u;
            if (!d.floor_layer_sizes)
            {
                // PointRenderer.cu:385-389
                ch = (int)std::ceil(float(ch) / 2.f);
                cw = (int)std::ceil(float(cw) / 2.f);
            }
            else
            {
                ch = ch / 2;
                cw = cw / 2;
            }
        }
        else
        {
            g.w[l]           = 0;
            g.h[l]           = 0;
            g.off[l + 1]     = g.off[l];
            g.tiles_x[l]     = 0;
            g.tiles_y[l]     = 0;
            g.bin_off[l + 1] = g.bin_off[l];
            g.tiles_x_magic[l] = 0;
        }
    }
}

// number of internally numbered pixels (tiles padded to 32 x 32), as a 64-bit value for the range check
long long pyramid_pixels_checked(const TripsSplatDesc& d)
{
    long long P = 0;
    int cw = d.views[0].w, ch = d.views[0].h;
    for (int l = 0; l < d.num_layers; ++l)
    {
        P += (long long)((cw + kTile - 1) / kTile) * ((ch + kTile - 1) / kTile) * kTilePixels;
        if (!d.floor_layer_sizes)
        {
            ch = (int)std::ceil(float(ch) / 2.f);
            cw = (int)std::ceil(float(cw) / 2.f);
        }
        else
        {
            ch = ch / 2;
            cw = cw / 2;
        }
    }
    return P;
}

SavedLayout saved_layout(const TripsSplatDesc& d, const PyramidGeom& g)
{
    SavedLayout s;
    const size_t N = (size_t)d.num_points, P = (size_t)g.bin_off[d.num_layers] * kTilePixels, K = (size_t)d.list_depth;
    const size_t rf = (size_t)record_floats(d.num_channels);
    size_t o        = 0;
    s.header        = o;
    o += align256(sizeof(ViewHeader));
    s.rec = o;
    o += align256(N * rf * sizeof(float));
    s.prec = o;
    o += align256(N * kPointRecordFloats * sizeof(float));
    s.lists = o;
    o += align256(P * K * sizeof(int32_t));
    s.retained = o;
    o += align256(P * sizeof(int32_t));
    s.tags = o;
    o += align256(P * 16);
    s.cid_of = o;
    o += align256(N * sizeof(int32_t));
    s.pid_of = o;
    o += align256(N * sizeof(int32_t));
    s.over_first = o;
    o += align256(N * sizeof(int32_t));
    s.chunk_valid = o;
    o += align256((size_t)(kBinGroups + kRetainedParts) * sizeof(int32_t));
    s.bytes_per_view = o;
    return s;
}

WorkspaceLayout workspace_layout(const TripsSplatDesc& d, const PyramidGeom& g)
{
    WorkspaceLayout w;
    const size_t N = (size_t)d.num_points, NB = (size_t)g.bin_off[d.num_layers], P = NB * kTilePixels;
    // a (point, layer) pair is filed once and appears in the lists of the four pixels of its footprint
    w.capacity     = d.max_list_entries > 0 ? ((size_t)d.max_list_entries + 3) / 4 : N * (size_t)d.num_layers;
    size_t o       = 0;
    // status header (overflow flag of the whole call), then for eval mode, which has no saved state to live
    // in, the per-view counters and the per-point records
    o += align256(sizeof(ViewHeader));
    o += align256(sizeof(ViewHeader));
    o += align256(N * (size_t)record_floats(d.num_channels) * sizeof(float));
    w.chunk_valid = o;
    o += align256((size_t)kBinGroups * (kBinThreads / 64) * sizeof(int32_t));
    w.prec = o;
    o += align256(N * kPointRecordFloats * sizeof(float));
    w.counts = o;
    o += align256(P * sizeof(int32_t));
    w.run = o;  // directly behind counts: one fill clears both
    o += align256(P * sizeof(int32_t));
    w.cursor = o;
    o += align256(P * sizeof(int32_t));
    w.slice_start = o;
    o += align256((NB + 1) * sizeof(int32_t));
    // every long list has at least kLongList / kLongSegment full segments, so the partial ones add at most half
    w.max_long_items = std::min<size_t>(w.capacity / kLongSegment * 3 / 2 + 16, (size_t)1 << 27);
    w.long_count     = o;
    o += align256(sizeof(int32_t));
    w.long_items = o;
    o += align256(w.max_long_items * sizeof(int2));
    w.cand = o;
    o += align256(w.max_long_items * 16 * sizeof(unsigned long long));
    w.bin_count = o;
    o += align256(NB * sizeof(int32_t));
    w.bin_start = o;
    o += align256((NB + 1) * sizeof(int32_t));
    w.bin_hist = o;
    o += align256((size_t)kBinGroups * NB * sizeof(int32_t));
    w.bin_entries = o;
    o += align256(w.capacity * (N <= ((size_t)1 << kPackedIdBits) ? sizeof(unsigned long long) : sizeof(uint4)));
    w.keys = o;
    o += align256(w.capacity * sizeof(unsigned long long));
    w.bytes = o;
    return w;
}
}  // namespace

namespace
{
BackwardWorkspaceLayout backward_workspace_layout(const TripsSplatDesc& d, const PyramidGeom& g)
{
    BackwardWorkspaceLayout w;
    // a row per (point, layer) pair: two per point by its compact number, the rest as many as the forward can file
    const size_t extra_layers = d.num_layers > kInlineLayers ? (size_t)(d.num_layers - kInlineLayers) : 0;
    const size_t row          = (size_t)pair_row_floats((d.num_channels + 3) & ~3) * sizeof(float);
    w.over_capacity = (size_t)d.num_points * extra_layers;
    if (d.max_list_entries > 0) w.over_capacity = std::min(w.over_capacity, ((size_t)d.max_list_entries + 3) / 4);
    size_t o      = align256(sizeof(ViewHeader));  // keeps the status block of the forward intact
    w.rows_inline = o;
    o += align256((size_t)d.num_points * kInlineLayers * row);
    w.rows_over = o;
    o += align256(w.over_capacity * row);
    w.flags = o;
    o += align256((size_t)d.num_points * TRIPS_MAX_LAYERS);
    w.mode = o;
    o += 256;
    w.bytes = o;
    return w;
}
}  // namespace

extern "C" {

const char* trips_version(void) { return "trips_splat 0.1 (gfx950)"; }
const char* trips_last_error_string(void) { return g_error; }

int trips_ctx_create(TripsCtx** out_ctx, int device)
{
    if (!out_ctx) return fail(TRIPS_ERR_INVALID_ARG, "out_ctx is NULL");
    int count    = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess) return hip_fail(e, "hipGetDeviceCount");
    if (device < 0 || device >= count) return fail(TRIPS_ERR_INVALID_ARG, "device %d of %d", device, count);
    // address of this device's copy of the static scratch array, with that device current
    int previous = 0;
    e            = hipGetDevice(&previous);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    e = hipSetDevice(device);
    if (e != hipSuccess) return hip_fail(e, "hipSetDevice");
    void* ptr = nullptr;
    e         = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    (void)hipSetDevice(previous);
    if (e != hipSuccess || !ptr) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    TripsCtx* c       = new TripsCtx;
    c->device         = device;
    c->static_scratch = ptr;
    *out_ctx          = c;
    return TRIPS_OK;
}

int trips_ctx_destroy(TripsCtx* ctx)
{
    delete ctx;
    return TRIPS_OK;
}

int trips_splat_layer_sizes(const TripsSplatDesc* desc, int32_t* w, int32_t* h)
{
    if (int e = check_desc(desc)) return e;
    if (!w || !h) return fail(TRIPS_ERR_INVALID_ARG, "w / h is NULL");
    PyramidGeom g;
    make_geom(*desc, g);
    for (int l = 0; l < desc->num_layers; ++l)
    {
        w[l] = g.w[l];
        h[l] = g.h[l];
    }
    return TRIPS_OK;
}

int trips_splat_workspace_size(const TripsSplatDesc* desc, size_t* bytes)
{
    if (int e = check_desc(desc)) return e;
    if (!bytes) return fail(TRIPS_ERR_INVALID_ARG, "bytes is NULL");
    if (pyramid_pixels_checked(*desc) > 0x7fffffffll) return fail(TRIPS_ERR_UNSUPPORTED, "pyramid has more than 2^31-1 pixels");
    PyramidGeom g;
    make_geom(*desc, g);
    const size_t fwd = workspace_layout(*desc, g).bytes;
    const size_t bwd = desc->train ? backward_workspace_layout(*desc, g).bytes : 0;
    *bytes           = fwd > bwd ? fwd : bwd;
    return TRIPS_OK;
}

int trips_splat_saved_size(const TripsSplatDesc* desc, size_t* bytes)
{
    if (int e = check_desc(desc)) return e;
    if (!bytes) return fail(TRIPS_ERR_INVALID_ARG, "bytes is NULL");
    if (pyramid_pixels_checked(*desc) > 0x7fffffffll) return fail(TRIPS_ERR_UNSUPPORTED, "pyramid has more than 2^31-1 pixels");
    PyramidGeom g;
    make_geom(*desc, g);
    *bytes = saved_layout(*desc, g).bytes_per_view * (size_t)desc->num_views;
    return TRIPS_OK;
}

}  // extern "C"

namespace
{
int forward_impl(TripsCtx* ctx, const TripsSplatDesc* desc, const TripsSplatIn* in, const TripsSplatOut* out,
                 void* workspace, size_t workspace_bytes, void* stream_, bool use_profiler)
{
    if (!ctx) return fail(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    if (int e = check_desc(desc)) return e;
    if (!in || !out) return fail(TRIPS_ERR_INVALID_ARG, "in / out is NULL");
    if (pyramid_pixels_checked(*desc) > 0x7fffffffll) return fail(TRIPS_ERR_UNSUPPORTED, "pyramid has more than 2^31-1 pixels");
    const TripsSplatDesc& d = *desc;
    if (d.num_points > 0 && (!in->position || !in->point_size || !in->index))
        return fail(TRIPS_ERR_INVALID_ARG, "position / point_size / index is NULL");
    if (!in->texture || !in->confidence || !in->background || !in->poses_se3 || !in->intrinsics)
        if (d.num_points > 0 || !in->background || !in->poses_se3 || !in->intrinsics)
            return fail(TRIPS_ERR_INVALID_ARG, "texture / confidence / background / poses_se3 / intrinsics is NULL");
    for (int l = 0; l < d.num_layers; ++l)
        if (!out->image[l]) return fail(TRIPS_ERR_INVALID_ARG, "image[%d] is NULL", l);
    const bool train = d.train != 0;
    if (train && !out->saved) return fail(TRIPS_ERR_INVALID_ARG, "saved is NULL in train mode");
    if (!workspace) return fail(TRIPS_ERR_INVALID_ARG, "workspace is NULL");
    if ((reinterpret_cast<uintptr_t>(workspace) & 255) || (train && (reinterpret_cast<uintptr_t>(out->saved) & 255)))
        return fail(TRIPS_ERR_INVALID_ARG, "workspace / saved must be 256-byte aligned");

    PyramidGeom g;
    make_geom(d, g);
    const WorkspaceLayout wl = workspace_layout(d, g);
    if (workspace_bytes < wl.bytes)
        return fail(TRIPS_ERR_WORKSPACE_SMALL, "workspace has %zu bytes, %zu needed", workspace_bytes, wl.bytes);
    const SavedLayout sl = saved_layout(d, g);
    hipStream_t stream   = reinterpret_cast<hipStream_t>(stream_);
    char* ws             = reinterpret_cast<char*>(workspace);

    for (int b = 0; b < d.num_views; ++b)
    {
        ForwardParams p;
        std::memset(&p, 0, sizeof(p));
        p.position   = reinterpret_cast<const float4*>(in->position);
        p.point_size = in->point_size;
        p.index      = in->index;
        p.texture    = in->texture;
        p.confidence = in->confidence;
        p.background = in->background;
        p.pose       = in->poses_se3 + 8 * (size_t)d.views[b].image_index;
        p.intrinsics = in->intrinsics + 13 * (size_t)d.views[b].camera_index;
        p.dropout    = (train && in->dropout) ? in->dropout + (size_t)b * d.num_points : nullptr;
        p.displacement = in->displacement ? in->displacement + (size_t)b * d.num_points * 3 : nullptr;
        p.geom       = g;
        p.view       = d.views[b];
        p.num_points = d.num_points;
        p.num_texels = d.num_texels;
        p.num_layers = d.num_layers;
        p.list_depth = d.list_depth;
        p.view_index = b;
        p.num_views  = d.num_views;
        p.layout     = d.layout;
        p.background_mode           = d.background_mode;
        p.drop_out_points_by_radius = d.drop_out_points_by_radius;
        p.viewer_only               = d.viewer_only;
        p.drop_out_radius_threshold = d.drop_out_radius_threshold;
        p.dist_cutoff               = d.dist_cutoff;
        p.stability_cutoff_value    = d.stability_cutoff_value;
        p.chunk_valid = reinterpret_cast<int32_t*>(ws + wl.chunk_valid);
        p.counts     = reinterpret_cast<int32_t*>(ws + wl.counts);
        p.cursor     = reinterpret_cast<int32_t*>(ws + wl.cursor);
        p.bin_count  = reinterpret_cast<int32_t*>(ws + wl.bin_count);
        p.bin_start  = reinterpret_cast<int32_t*>(ws + wl.bin_start);
        p.bin_hist   = reinterpret_cast<int32_t*>(ws + wl.bin_hist);
        p.bin_groups = kBinGroups;
        p.points_per_block = (d.num_points + kBinGroups - 1) / kBinGroups;
        p.run         = reinterpret_cast<int32_t*>(ws + wl.run);
        p.slice_start = reinterpret_cast<int32_t*>(ws + wl.slice_start);
        p.long_count  = reinterpret_cast<int32_t*>(ws + wl.long_count);
        p.long_items  = reinterpret_cast<int2*>(ws + wl.long_items);
        p.cand        = reinterpret_cast<unsigned long long*>(ws + wl.cand);
        p.max_long_items = (int32_t)wl.max_long_items;
        p.bin_entries   = ws + wl.bin_entries;
        p.keys       = reinterpret_cast<unsigned long long*>(ws + wl.keys);
        p.capacity   = (long long)wl.capacity;
        if (train)
        {
            char* sv     = reinterpret_cast<char*>(out->saved) + sl.bytes_per_view * (size_t)b;
            p.header     = reinterpret_cast<ViewHeader*>(sv + sl.header);
            p.rec        = reinterpret_cast<float*>(sv + sl.rec);
            p.prec       = reinterpret_cast<float*>(sv + sl.prec);
            p.rec_floats = record_floats(d.num_channels);
            p.lists      = reinterpret_cast<int32_t*>(sv + sl.lists);
            p.retained   = reinterpret_cast<int32_t*>(sv + sl.retained);
            p.tags       = reinterpret_cast<unsigned char*>(sv + sl.tags);
            p.over_first = reinterpret_cast<int32_t*>(sv + sl.over_first);
            p.saved_chunk_valid = reinterpret_cast<int32_t*>(sv + sl.chunk_valid);
            p.cid_of     = reinterpret_cast<int32_t*>(sv + sl.cid_of);
            p.pid_of     = reinterpret_cast<int32_t*>(sv + sl.pid_of);
        }
        else
        {
            p.header     = reinterpret_cast<ViewHeader*>(ws + align256(sizeof(ViewHeader)));
            p.rec        = reinterpret_cast<float*>(ws + 2 * align256(sizeof(ViewHeader)));
            p.prec       = reinterpret_cast<float*>(ws + wl.prec);
            p.rec_floats = record_floats(d.num_channels);
        }
        p.status = reinterpret_cast<ViewHeader*>(ws);
        for (int l = 0; l < d.num_layers; ++l) p.image[l] = out->image[l];
        hipError_t e = launch_forward_view(p, d.num_channels, train, b == 0, stream,
                                           (use_profiler && ctx->prof.enabled) ? &ctx->prof : nullptr);
        if (e != hipSuccess) return hip_fail(e, "forward launch");
    }
    return TRIPS_OK;
}
}  // namespace

extern "C" {

int trips_splat_forward(TripsCtx* ctx, const TripsSplatDesc* desc, const TripsSplatIn* in, const TripsSplatOut* out,
                        void* workspace, size_t workspace_bytes, void* stream)
{
    return forward_impl(ctx, desc, in, out, workspace, workspace_bytes, stream, true);
}

int trips_splat_forward_static(TripsCtx* ctx, const TripsSplatDesc* desc, const TripsSplatIn* in, const TripsSplatOut* out,
                               void* stream)
{
    if (!ctx) return fail(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    // what the forward itself carves out of a workspace (the backward's tables are not part of it: the backward takes a
    // caller-owned workspace)
    if (int e = check_desc(desc)) return e;
    if (pyramid_pixels_checked(*desc) > 0x7fffffffll) return fail(TRIPS_ERR_UNSUPPORTED, "pyramid has more than 2^31-1 pixels");
    PyramidGeom g;
    make_geom(*desc, g);
    const size_t need = workspace_layout(*desc, g).bytes;
    if (need > (size_t)TRIPS_STATIC_WORKSPACE_BYTES)
        return fail(TRIPS_ERR_WORKSPACE_SMALL,
                    "the forward of this scene needs %zu bytes of workspace, the static one holds %zu: use trips_splat_forward "
                    "with a caller-owned workspace, or lower max_list_entries",
                    need, (size_t)TRIPS_STATIC_WORKSPACE_BYTES);
    // no event creation either: the per-kernel timer is left out of this entry point
    return forward_impl(ctx, desc, in, out, ctx->static_scratch, (size_t)TRIPS_STATIC_WORKSPACE_BYTES, stream, false);
}

int trips_splat_backward(TripsCtx* ctx, const TripsSplatDesc* desc, const TripsSplatIn* in, const void* saved,
                         const float* const grad_image[TRIPS_MAX_LAYERS], const TripsSplatGrads* grads,
                         void* workspace, size_t workspace_bytes, void* stream_)
{
    if (!ctx) return fail(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    if (int e = check_desc(desc)) return e;
    const TripsSplatDesc& d = *desc;
    if (!d.train) return fail(TRIPS_ERR_INVALID_ARG, "backward needs a forward run with train = 1");
    if (!in || !saved || !grad_image || !grads) return fail(TRIPS_ERR_INVALID_ARG, "in / saved / grad_image / grads is NULL");
    if (!in->background || !in->poses_se3 || !in->intrinsics)
        return fail(TRIPS_ERR_INVALID_ARG, "background / poses_se3 / intrinsics is NULL");
    if (d.num_points > 0 && (!in->position || !in->index))
        return fail(TRIPS_ERR_INVALID_ARG, "position / index is NULL (the backward reads them again, unchanged since the forward)");
    if (!grads->d_texture || !grads->d_confidence || !grads->d_background)
        return fail(TRIPS_ERR_INVALID_ARG, "d_texture / d_confidence / d_background is required");
    for (int l = 0; l < d.num_layers; ++l)
        if (!grad_image[l]) return fail(TRIPS_ERR_INVALID_ARG, "grad_image[%d] is NULL", l);
    if (reinterpret_cast<uintptr_t>(saved) & 255) return fail(TRIPS_ERR_INVALID_ARG, "saved must be 256-byte aligned");

    PyramidGeom g;
    make_geom(d, g);
    const SavedLayout sl = saved_layout(d, g);
    const BackwardWorkspaceLayout bl = backward_workspace_layout(d, g);
    if (!workspace) return fail(TRIPS_ERR_INVALID_ARG, "workspace is NULL");
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return fail(TRIPS_ERR_INVALID_ARG, "workspace must be 256-byte aligned");
    if (workspace_bytes < bl.bytes)
        return fail(TRIPS_ERR_WORKSPACE_SMALL, "workspace has %zu bytes, %zu needed", workspace_bytes, bl.bytes);
    char* ws             = reinterpret_cast<char*>(workspace);
    hipStream_t stream   = reinterpret_cast<hipStream_t>(stream_);
    for (int b = 0; b < d.num_views; ++b)
    {
        BackwardParams p;
        std::memset(&p, 0, sizeof(p));
        const char* sv = reinterpret_cast<const char*>(saved) + sl.bytes_per_view * (size_t)b;
        p.background   = in->background;
        p.pose         = in->poses_se3 + 8 * (size_t)d.views[b].image_index;
        p.intrinsics   = in->intrinsics + 13 * (size_t)d.views[b].camera_index;
        p.point_size   = in->point_size;
        p.position     = reinterpret_cast<const float4*>(in->position);
        p.displacement = in->displacement ? in->displacement + (size_t)b * d.num_points * 3 : nullptr;
        p.index        = in->index;
        p.geom         = g;
        p.view         = d.views[b];
        p.num_points   = d.num_points;
        p.num_texels   = d.num_texels;
        p.num_layers   = d.num_layers;
        p.list_depth   = d.list_depth;
        p.view_index   = b;
        p.num_views    = d.num_views;
        p.layout       = d.layout;
        p.dist_cutoff  = d.dist_cutoff;
        p.rec          = reinterpret_cast<const float*>(sv + sl.rec);
        p.prec         = reinterpret_cast<const float*>(sv + sl.prec);
        p.rec_floats   = record_floats(d.num_channels);
        p.lists        = reinterpret_cast<const int32_t*>(sv + sl.lists);
        p.retained     = reinterpret_cast<const int32_t*>(sv + sl.retained);
        p.cid_of       = reinterpret_cast<const int32_t*>(sv + sl.cid_of);
        p.header       = reinterpret_cast<const ViewHeader*>(sv + sl.header);
        p.tags         = reinterpret_cast<const unsigned char*>(sv + sl.tags);
        p.over_first   = reinterpret_cast<const int32_t*>(sv + sl.over_first);
        p.chunk_valid  = reinterpret_cast<const int32_t*>(sv + sl.chunk_valid);
        p.bin_groups   = kBinGroups;
        p.points_per_block = (d.num_points + kBinGroups - 1) / kBinGroups;
        p.rows_inline  = reinterpret_cast<float*>(ws + bl.rows_inline);
        p.rows_over    = reinterpret_cast<float*>(ws + bl.rows_over);
        p.flags        = reinterpret_cast<unsigned char*>(ws + bl.flags);
        p.mode         = reinterpret_cast<int32_t*>(ws + bl.mode);
        p.force_mode   = ctx->pair_rows_mode;
        p.over_capacity = (long long)bl.over_capacity;
        p.blocks_off[0] = 0;
        for (int l = 0; l < TRIPS_MAX_LAYERS; ++l)
        {
            // blocks of 16 x 16 pixels, 15 apart, so that every pixel is the first-15 part of exactly one block
            const int nx = l < d.num_layers ? (g.w[l] + 14) / 15 : 0, ny = l < d.num_layers ? (g.h[l] + 14) / 15 : 0;
            p.blocks_x[l]       = nx;
            p.blocks_off[l + 1] = p.blocks_off[l] + nx * ny;
        }
        for (int l = 0; l < d.num_layers; ++l) p.grad_image[l] = grad_image[l];
        p.d_texture    = grads->d_texture;
        p.d_confidence = grads->d_confidence;
        p.d_background = grads->d_background;
        p.d_position   = grads->d_position;
        p.d_point_size = grads->d_point_size;
        p.d_pose       = grads->d_pose ? grads->d_pose + 6 * (size_t)d.views[b].image_index : nullptr;
        p.d_intrinsics = grads->d_intrinsics ? grads->d_intrinsics + 13 * (size_t)d.views[b].camera_index : nullptr;
        p.overwrite    = (grads->overwrite_point_grads != 0 && b == 0) ? 1 : 0;  // later views add to the first one's
        p.clear_block_sums = (grads->clear_block_sums != 0 && b == 0) ? 1 : 0;
        p.d_pose_all       = grads->d_pose;
        p.d_intrinsics_all = grads->d_intrinsics;
        p.num_images       = d.num_images;
        p.num_cameras      = d.num_cameras;
        hipError_t e   = launch_backward_view(p, d.num_channels, stream, ctx->prof.enabled ? &ctx->prof : nullptr);
        if (e != hipSuccess) return hip_fail(e, "backward launch");
    }
    return TRIPS_OK;
}

}  // extern "C"

namespace
{
int check_status_block(const void* header_owner, void* stream_)
{
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    ViewHeader h;
    hipError_t e = hipMemcpyAsync(&h, header_owner, sizeof(h), hipMemcpyDeviceToHost, stream);
    if (e != hipSuccess) return hip_fail(e, "hipMemcpyAsync");
    e = hipStreamSynchronize(stream);
    if (e != hipSuccess) return hip_fail(e, "hipStreamSynchronize");
    if (h.bad_index) return fail(TRIPS_ERR_INVALID_ARG, "index holds values outside [0, num_texels): those points were left out");
    if (h.overflow) return fail(TRIPS_ERR_LIST_OVERFLOW, "%llu list entries dropped: max_list_entries too small", 4 * h.overflow);
    return TRIPS_OK;
}
}  // namespace

extern "C" {

int trips_splat_check(TripsCtx* ctx, const void* workspace, void* stream_)
{
    if (!ctx) return fail(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    if (!workspace) return fail(TRIPS_ERR_INVALID_ARG, "workspace is NULL (trips_splat_check_static reports on the static one)");
    return check_status_block(workspace, stream_);
}

int trips_splat_check_static(TripsCtx* ctx, void* stream_)
{
    if (!ctx) return fail(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    if (!ctx->static_scratch) return fail(TRIPS_ERR_INVALID_ARG, "this context has no static workspace");
    return check_status_block(ctx->static_scratch, stream_);
}

int trips_splat_counters(TripsCtx* ctx, const TripsSplatDesc* desc, const void* saved, int view, int64_t counters[4],
                         void* stream_)
{
    if (!ctx) return fail(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    if (int e = check_desc(desc)) return e;
    if (!saved || !counters) return fail(TRIPS_ERR_INVALID_ARG, "saved / counters is NULL");
    if (view < 0 || view >= desc->num_views) return fail(TRIPS_ERR_INVALID_ARG, "view out of range");
    PyramidGeom g;
    make_geom(*desc, g);
    const SavedLayout sl = saved_layout(*desc, g);
    hipStream_t stream   = reinterpret_cast<hipStream_t>(stream_);
    char* sv             = const_cast<char*>(reinterpret_cast<const char*>(saved)) + sl.bytes_per_view * (size_t)view;
    ViewHeader* hd       = reinterpret_cast<ViewHeader*>(sv + sl.header);
    const long long P    = g.off[desc->num_layers];
    const long long Pi   = (long long)g.bin_off[desc->num_layers] * kTilePixels;  // padding rows hold 0
    // (the low bits of a pixel's word: its retained entries)
    hipError_t e = launch_sum_i32(reinterpret_cast<const int32_t*>(sv + sl.retained), Pi, (unsigned)kRetainedMask, &hd->retained, stream);
    if (e != hipSuccess) return hip_fail(e, "retained sum");
    ViewHeader h;
    e = hipMemcpyAsync(&h, hd, sizeof(h), hipMemcpyDeviceToHost, stream);
    if (e != hipSuccess) return hip_fail(e, "hipMemcpyAsync");
    e = hipStreamSynchronize(stream);
    if (e != hipSuccess) return hip_fail(e, "hipStreamSynchronize");
    counters[0] = (int64_t)h.n_valid;
    counters[1] = (int64_t)(4 * h.n_entries);  // the header counts (point, layer) pairs, each in four pixel lists
    counters[2] = (int64_t)h.retained;
    counters[3] = (int64_t)P;
    return TRIPS_OK;
}

int trips_splat_export_lists(TripsCtx* ctx, const TripsSplatDesc* desc, const void* saved, int view,
                             int32_t* device_lists, int32_t* device_retained, int32_t* device_lengths, void* stream_)
{
    if (!ctx) return fail(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    if (int e = check_desc(desc)) return e;
    if (!saved) return fail(TRIPS_ERR_INVALID_ARG, "saved is NULL");
    if (view < 0 || view >= desc->num_views) return fail(TRIPS_ERR_INVALID_ARG, "view out of range");
    PyramidGeom g;
    make_geom(*desc, g);
    const SavedLayout sl = saved_layout(*desc, g);
    hipStream_t stream   = reinterpret_cast<hipStream_t>(stream_);
    const char* sv       = reinterpret_cast<const char*>(saved) + sl.bytes_per_view * (size_t)view;
    hipError_t e = launch_export_lists(g, desc->list_depth, reinterpret_cast<const int32_t*>(sv + sl.lists),
                                       reinterpret_cast<const int32_t*>(sv + sl.retained),
                                       reinterpret_cast<const int32_t*>(sv + sl.pid_of), device_lists, device_retained,
                                       device_lengths, stream);
    if (e != hipSuccess) return hip_fail(e, "export copy");
    return TRIPS_OK;
}

int trips_splat_export_points(TripsCtx* ctx, const TripsSplatDesc* desc, const void* saved, int view, float* device_ip,
                              float* device_depth, float* device_size_px, int32_t* device_max_layer, void* stream_)
{
    if (!ctx) return fail(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    if (int e = check_desc(desc)) return e;
    if (!saved) return fail(TRIPS_ERR_INVALID_ARG, "saved is NULL");
    if (view < 0 || view >= desc->num_views) return fail(TRIPS_ERR_INVALID_ARG, "view out of range");
    PyramidGeom g;
    make_geom(*desc, g);
    const SavedLayout sl = saved_layout(*desc, g);
    const char* sv       = reinterpret_cast<const char*>(saved) + sl.bytes_per_view * (size_t)view;
    hipError_t e = launch_export_points(reinterpret_cast<const float*>(sv + sl.rec), record_floats(desc->num_channels),
                                        reinterpret_cast<const float*>(sv + sl.prec),
                                        reinterpret_cast<const int32_t*>(sv + sl.cid_of), desc->num_points, device_ip, device_depth, device_size_px, device_max_layer,
                                        reinterpret_cast<hipStream_t>(stream_));
    if (e != hipSuccess) return hip_fail(e, "export points");
    return TRIPS_OK;
}

int trips_adam_step_fused(TripsCtx* ctx, const TripsAdamTensor* tensors, int n_tensors, void* stream_)
{
    if (!ctx) return fail(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    if (n_tensors < 0 || (n_tensors > 0 && !tensors)) return fail(TRIPS_ERR_INVALID_ARG, "tensors");
    for (int i = 0; i < n_tensors; ++i)
    {
        const TripsAdamTensor& t = tensors[i];
        if (t.n < 0) return fail(TRIPS_ERR_INVALID_ARG, "tensor %d: n < 0", i);
        if (t.n == 0) continue;
        if (!t.weights || !t.grads || !t.first_moment || !t.second_moment || !t.steps)
            return fail(TRIPS_ERR_INVALID_ARG, "tensor %d: NULL pointer", i);
        if (t.dtype != TRIPS_DTYPE_F32 && t.dtype != TRIPS_DTYPE_F64)
            return fail(TRIPS_ERR_UNSUPPORTED, "tensor %d: dtype %d", i, t.dtype);
        if (!(t.loss_scale != 0.f)) return fail(TRIPS_ERR_INVALID_ARG, "tensor %d: loss_scale is 0", i);
        if (t.steps_dtype != TRIPS_STEPS_I64 && t.steps_dtype != TRIPS_STEPS_I32)
            return fail(TRIPS_ERR_UNSUPPORTED, "tensor %d: steps_dtype %d", i, t.steps_dtype);
    }
    hipError_t e = launch_adam(tensors, n_tensors, reinterpret_cast<hipStream_t>(stream_), ctx->prof.enabled ? &ctx->prof : nullptr);
    if (e != hipSuccess) return hip_fail(e, "adam launch");
    return TRIPS_OK;
}

int trips_adam_points_state_size(int num_points, int num_channels, size_t* bytes, int* row_bytes)
{
    if (!bytes) return fail(TRIPS_ERR_INVALID_ARG, "bytes is NULL");
    if (num_points < 0) return fail(TRIPS_ERR_INVALID_ARG, "num_points < 0");
    if (!channels_ok(num_channels)) return fail(TRIPS_ERR_UNSUPPORTED, "num_channels %d not in {3,4,6,8,16}", num_channels);
    const int row = adam_points_row_chunks(num_channels) * 16;
    if (row_bytes) *row_bytes = row;
    *bytes = (size_t)num_points * (size_t)row;
    return TRIPS_OK;
}

int trips_adam_step_points(TripsCtx* ctx, const TripsAdamTensor tensors[4], int num_points, int num_channels, void* state,
                           void* stream_)
{
    if (!ctx) return fail(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    if (!tensors) return fail(TRIPS_ERR_INVALID_ARG, "tensors is NULL");
    if (num_points < 0) return fail(TRIPS_ERR_INVALID_ARG, "num_points < 0");
    if (!channels_ok(num_channels)) return fail(TRIPS_ERR_UNSUPPORTED, "num_channels %d not in {3,4,6,8,16}", num_channels);
    if (num_points == 0) return TRIPS_OK;
    if (!state || (reinterpret_cast<uintptr_t>(state) & 127)) return fail(TRIPS_ERR_INVALID_ARG, "state must be a 128-byte aligned device pointer");
    const long long want[4] = {4ll * num_points, num_points, (long long)num_channels * num_points, num_points};
    for (int i = 0; i < 4; ++i)
    {
        const TripsAdamTensor& t = tensors[i];
        if (t.n != want[i]) return fail(TRIPS_ERR_INVALID_ARG, "tensor %d: %lld elements, %lld expected", i, (long long)t.n, want[i]);
        if (!t.weights || !t.grads) return fail(TRIPS_ERR_INVALID_ARG, "tensor %d: NULL pointer", i);
        if (t.dtype != TRIPS_DTYPE_F32) return fail(TRIPS_ERR_UNSUPPORTED, "tensor %d: dtype %d (the point parameters are float32)", i, t.dtype);
        if (!(t.loss_scale != 0.f)) return fail(TRIPS_ERR_INVALID_ARG, "tensor %d: loss_scale is 0", i);
    }
    if ((reinterpret_cast<uintptr_t>(tensors[0].weights) & 15) || (reinterpret_cast<uintptr_t>(tensors[0].grads) & 15))
        return fail(TRIPS_ERR_INVALID_ARG, "position and its gradient must be 16-byte aligned");
    hipError_t e = launch_adam_points(tensors, num_points, num_channels, state, reinterpret_cast<hipStream_t>(stream_),
                                      ctx->prof.enabled ? &ctx->prof : nullptr);
    if (e != hipSuccess) return hip_fail(e, "adam launch");
    return TRIPS_OK;
}

int trips_apply_tangent(TripsCtx* ctx, double* tangent, double* poses_se3, int n, void* stream_)
{
    if (!ctx) return fail(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    if (n < 0 || (n > 0 && (!tangent || !poses_se3))) return fail(TRIPS_ERR_INVALID_ARG, "tangent / poses_se3");
    hipError_t e = launch_apply_tangent(tangent, poses_se3, n, reinterpret_cast<hipStream_t>(stream_));
    if (e != hipSuccess) return hip_fail(e, "apply_tangent launch");
    return TRIPS_OK;
}

int trips_splat_pair_rows_mode(TripsCtx* ctx, int mode)
{
    if (!ctx) return fail(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    if (mode < 0 || mode > 2) return fail(TRIPS_ERR_INVALID_ARG, "mode must be 0, 1 or 2");
    ctx->pair_rows_mode = mode;
    return TRIPS_OK;
}

int trips_profile_enable(TripsCtx* ctx, int enabled)
{
    if (!ctx) return fail(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    ctx->prof.enabled = enabled != 0;
    return TRIPS_OK;
}

int trips_profile_read(TripsCtx* ctx, int* n, const char* names[TRIPS_PROFILE_MAX_KERNELS],
                       float ms[TRIPS_PROFILE_MAX_KERNELS], int launches[TRIPS_PROFILE_MAX_KERNELS])
{
    if (!ctx || !n || !names || !ms || !launches) return fail(TRIPS_ERR_INVALID_ARG, "NULL argument");
    int count = 0;
    for (auto& sp : ctx->prof.spans)
    {
        hipError_t e = hipEventSynchronize(sp.b);
        if (e != hipSuccess) return hip_fail(e, "hipEventSynchronize");
        float t = 0.f;
        e       = hipEventElapsedTime(&t, sp.a, sp.b);
        if (e != hipSuccess) return hip_fail(e, "hipEventElapsedTime");
        int k = 0;
        while (k < count && std::strcmp(names[k], sp.name) != 0) ++k;
        if (k == count)
        {
            if (count == TRIPS_PROFILE_MAX_KERNELS) continue;
            names[k]    = sp.name;
            ms[k]       = 0.f;
            launches[k] = 0;
            ++count;
        }
        ms[k] += t;
        launches[k] += 1;
        ctx->prof.pool.push_back(sp.a);
        ctx->prof.pool.push_back(sp.b);
    }
    ctx->prof.spans.clear();
    *n = count;
    return TRIPS_OK;
}

}  // extern "C"
