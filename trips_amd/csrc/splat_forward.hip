// Forward kernels of the splat path for gfx950 (wave64).
//
//   project_bin_kernel   <- CountAndCollectTiled (projection, validity, layer selection)
//                           src/lib/rendering/RenderForward.cu:168-366
//   bin_scan / bin_scatter / tile_count / tile_scatter
//                        <- per-pixel counting (:355-361), cub ExclusiveSum section (:1155-1232) and
//                           SplattingPass (:368-436)
//   cell_sort_kernel / blend_kernel
//                        <- FastSortFusedNew    src/lib/rendering/RenderForward.cu:474-1059
//
// Differences in shape, not in result. The reference increments one global counter per (point, layer, corner),
// scans layer by layer with two blocking read-backs each, and takes one more global atomic per entry to place
// its key. Scattered global atomics run at about 2.7e10 per second on this GPU, so here a (point, layer) pair is
// first binned, once, into the 32 x 32 pixel tile of its footprint's first pixel (workgroup-private LDS histograms
// and a column scan: no global atomics); a workgroup per tile then counts, scans and places the keys of its 1024
// cells with LDS atomics, one key per pair, and the blend gathers a pixel's list from the four cells whose
// footprints cover it. The sort is done per cell (each serves four pixels); a pixel is one lane of a wavefront that
// owns 8 x 8 of them, merges its four cell lists and blends front to back, instead of two lists per 32-lane warp; the
// per-point record gathered by the blend carries position, size, confidence and descriptor together; what is kept
// for the backward is the sorted id list per pixel (64 B) and a byte per list position that says which cell the
// entry came from and where it stood in that cell's list, instead of 16 x 7 floats.
#include "row16.h"
#include "splat_internal.h"
#include "trips_math.h"

#include <type_traits>

#pragma clang fp contract(off)

namespace trips
{
typedef unsigned vu4 __attribute__((ext_vector_type(4)));
typedef float vf4 __attribute__((ext_vector_type(4)));
typedef int vi4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ Camera load_camera(const double* pose, const float* intr, const TripsView& v,
                                              float dist_cutoff)
{
    Camera c;
    c.V  = load_pose(pose);
    c.fx = intr[0];
    c.fy = intr[1];
    c.cx = intr[2];
    c.cy = intr[3];
    c.s  = intr[4];
    c.no_distortion = true;
    for (int i = 0; i < 8; ++i)
    {
        c.dist[i] = intr[5 + i];
        c.no_distortion = c.no_distortion && c.dist[i] == 0.f;
    }
    c.cfx         = v.crop_transform[0];
    c.cfy         = v.crop_transform[1];
    c.ccx         = v.crop_transform[2];
    c.ccy         = v.crop_transform[3];
    c.cs          = v.crop_transform[4];
    c.r00         = v.crop_rotation[0];
    c.r01         = v.crop_rotation[1];
    c.r10         = v.crop_rotation[2];
    c.r11         = v.crop_rotation[3];
    c.centre_x    = float(v.w / 2);
    c.centre_y    = float(v.h / 2);
    c.dist_cutoff = dist_cutoff;
    return c;
}

// ---------------------------------------------------------------------------------------------------------
// Projection, validity and layer selection of one point (CountAndCollectTiled, RenderForward.cu:168-366; its per-pixel
// counter updates become per-tile ones).
struct PointProjection
{
    bool valid;
    int tex;        // descriptor column
    int layers;     // layers the point is written to (0 if culled)
    float ipx, ipy, z, size_px;
    float d_softplus;  // softplus'(raw size), training mode
};

// What the projection reads of a point in point order (fetched one step ahead of its use).
struct PointInputs
{
    int tex;  // descriptor column
    float4 pos;
    float raw_size;
};

__device__ __forceinline__ PointInputs load_point(const ForwardParams& p, int pid)
{
    PointInputs in;
    in.tex      = p.index[pid];
    in.pos      = p.position[pid];
    in.raw_size = p.point_size[pid];
    return in;
}

// `s_hist`: LDS counters, one per tile; every layer the point is written to adds one to the tile of the footprint's
// first pixel (px, py). (The footprint (px..px+1, py..py+1) lies inside the image because px < w-1 and py < h-1.)
template <bool TRAIN>
__device__ __forceinline__ PointProjection project_point(const ForwardParams& p, const Camera& cam, int pid, const PointInputs& in,
                                                         int* s_hist, bool& not_identity, bool& bad_index)
{
    PointProjection o;
    o.valid  = false;
    o.layers = 0;
    o.ipx = o.ipy = 0.f;
    o.z       = -1.f;
    o.size_px = 0.f;
    o.d_softplus = 0.f;
    const int L = p.num_layers;
    bool skip   = false;
    o.tex       = in.tex;
    not_identity |= (o.tex != pid);
    if ((unsigned)o.tex >= (unsigned)p.num_texels)
    {
        // a column outside the descriptor table: leave the point out (reported by the status query) rather
        // than read past the tables
        bad_index    = true;
        not_identity = true;  // the backward then never uses the point's own number as a column
        skip         = true;
    }
    if (p.viewer_only && !skip)
    {
        if (p.confidence[o.tex] < p.stability_cutoff_value) skip = true;
    }
    if (TRAIN && p.dropout)
    {
        if (p.dropout[pid] == 1.f) skip = true;
    }
    if (skip) return o;
    float4 pos = in.pos;
    if (p.displacement)
    {
        const float* dsp = p.displacement + (size_t)pid * 3;
        pos.x += dsp[0];
        pos.y += dsp[1];
        pos.z += dsp[2];
    }
    float d_softplus    = 0.f;
    const float size    = TRAIN ? softplus_and_derivative(in.raw_size, &d_softplus) : softplus(in.raw_size);
    const Projected pr  = project(cam, pos.x, pos.y, pos.z);
    const float z       = pr.z;
    float radius_px     = pr.scale * pos.w / z;
    const float size_px = pr.scale * size / z;

    auto valid = [&](float x, float y, int layer, float radius) -> bool
    {
        if (z <= 0.f) return false;
        if (!(x >= 0.f) || x >= float(p.geom.w[layer] - 1) || !(y >= 0.f) || y >= float(p.geom.h[layer] - 1)) return false;
        if (p.drop_out_points_by_radius && float(trunc_sat(radius)) < p.drop_out_radius_threshold) return false;
        return true;
    };
    if (!valid(pr.ipx, pr.ipy, 0, radius_px)) return o;
    int layer_higher = 0;
    if (size_px > 1.f)
    {
        int lo, hi;
        log2_floor_ceil(size_px, lo, hi);
        layer_higher = min(hi, L - 1);
    }
    int layer = 0;
    float lx = pr.ipx, ly = pr.ipy;
    for (; layer < layer_higher + 1; ++layer, lx *= 0.5f, ly *= 0.5f, radius_px *= 0.5f)
    {
        const int px = (int)floorf(lx), py = (int)floorf(ly);
        if (!valid(float(px), float(py), layer, radius_px)) break;
        atomicAdd(s_hist + p.geom.bin_off[layer] + (py >> kTileShift) * p.geom.tiles_x[layer] + (px >> kTileShift), 1);
    }
    o.valid   = true;
    o.layers  = layer;
    o.ipx     = pr.ipx;
    o.ipy     = pr.ipy;
    o.z       = z;
    o.size_px = size_px;
    o.d_softplus = d_softplus;
    return o;
}

// Calls f(px, py, counter of the tile of (px, py)) for the layers a point is written to.
template <typename F>
__device__ __forceinline__ void for_point_tiles(const PyramidGeom& g, const PointProjection& o, int* tile_table, F&& f)
{
    float lx = o.ipx, ly = o.ipy;
    for (int layer = 0; layer < o.layers; ++layer, lx *= 0.5f, ly *= 0.5f)
    {
        const int px = (int)floorf(lx), py = (int)floorf(ly);
        f(px, py, tile_table + g.bin_off[layer] + (py >> kTileShift) * g.tiles_x[layer] + (px >> kTileShift));
    }
}

// A workgroup of the two binning kernels owns one contiguous chunk of points and walks it one point per thread at a
// time. The valid points of the chunk are numbered in point order from the chunk's first point number on ("compact numbers":
// cid = chunk begin + rank among the chunk's valid points; per step a ballot per wavefront and one exchange of the
// wavefront counts through LDS). The numbers grow with the point id, so a sort key built from them orders like one
// built from point ids; the records written at them are dense from the start of every chunk (whole lines, nothing
// for culled points).
__device__ __forceinline__ void chunk_point_range(const ForwardParams& p, int& begin, int& end)
{
    begin = min(p.num_points, (int)blockIdx.x * p.points_per_block);
    end   = min(p.num_points, begin + p.points_per_block);
}

// Projection, validity, layer selection; the records of the valid points at their compact numbers; LDS histogram of
// the tiles that this workgroup's points fall into.
template <int C, bool TRAIN>
__global__ __launch_bounds__(kBinThreads) void project_bin_kernel(const ForwardParams p)
{
    constexpr int CPAD  = (C + 3) & ~3;
    constexpr int NREC  = 1 + CPAD / 4;  // float4 per blend record
    constexpr int WAVES = kBinThreads / 64;
    extern __shared__ int s_hist[];  // bin entries of this workgroup's points, one counter per tile
    __shared__ int s_valid[2][WAVES];  // valid points of every wavefront in this step (two steps in flight)
    __shared__ int s_flags;            // bit 0: not_identity, bit 1: bad_index, of any point of the chunk
    const Camera cam  = load_camera(p.pose, p.intrinsics, p.view, p.dist_cutoff);
    const int L       = p.num_layers;
    const int NB      = p.geom.bin_off[L];
    bool not_identity = false;  // some point's descriptor column differs from its own index
    bool bad_index    = false;
    for (int i = threadIdx.x; i < NB; i += kBinThreads) s_hist[i] = 0;
    if (threadIdx.x == 0) s_flags = 0;
    __syncthreads();

    int begin, end;
    chunk_point_range(p, begin, end);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int next       = begin;  // workgroup-uniform: compact number of the chunk's next valid point
    int next_pair  = 0;      // workgroup-uniform: overflow rows of the chunk's points so far
    int step       = 0;
    // the loads of the next step's points are in flight while this step's are projected
    PointInputs nxt;
    nxt.tex = 0, nxt.pos = make_float4(0.f, 0.f, 0.f, 0.f), nxt.raw_size = 0.f;
    if (begin + (int)threadIdx.x < end) nxt = load_point(p, begin + (int)threadIdx.x);
    for (int base = begin; base < end; base += kBinThreads, step ^= 1)
    {
        const int pid        = base + threadIdx.x;
        const PointInputs in = nxt;
        if (pid + kBinThreads < end) nxt = load_point(p, pid + kBinThreads);
        // the descriptor of the point is requested before it is known whether the point is visible: the loads then run
        // beside the projection instead of after it
        float conf = 0.f;
        float d[CPAD];
#pragma unroll
        for (int c = 0; c < CPAD; ++c) d[c] = 0.f;
        if (pid < end && (unsigned)in.tex < (unsigned)p.num_texels)
        {
            conf = p.confidence[in.tex];
#pragma unroll
            for (int c = 0; c < C; ++c) d[c] = p.texture[(size_t)c * p.num_texels + in.tex];
        }
        PointProjection o;
        o.valid  = false;
        o.layers = 0;
        if (pid < end) o = project_point<TRAIN>(p, cam, pid, in, s_hist, not_identity, bad_index);
        const unsigned long long vm = __ballot(o.valid);
        const unsigned long long below = (1ull << lane) - 1ull;
        // rows of the backward's overflow table (one per layer past the second) of the wavefront's points before this
        // one, and of the wavefront: 0..6 per point, one ballot per bit
        int pairs_before = 0, pairs_wave = 0;
        if (TRAIN)
        {
            const int extra = max(o.layers - kInlineLayers, 0);
#pragma unroll
            for (int b = 0; b < 3; ++b)
            {
                const unsigned long long m = __ballot((extra >> b) & 1);
                pairs_before += (int)__popcll(m & below) << b;
                pairs_wave += (int)__popcll(m) << b;
            }
        }
        // both counts of a wavefront in one word (at most 64 valid points and 384 rows per wavefront, 1024 and 6144 per
        // step: 16 bits each); every wavefront then takes the prefix over the 16 words in its first 16 lanes
        if (lane == 0) s_valid[step][wave] = (int)__popcll(vm) | (pairs_wave << 16);
        __syncthreads();
        static_assert(WAVES == 16, "the prefix below runs over one 16-lane row");
        const int word = lane < WAVES ? s_valid[step][lane] : 0;  // the counts of wavefront w in lane w
        int inc        = word;
#pragma unroll
        for (int o = 1; o < WAVES; o <<= 1)
        {
            const int t = __shfl_up(inc, o);
            if (lane >= o) inc += t;
        }
        const int upto = __shfl(inc, WAVES - 1);     // the step's totals
        const int excl = __shfl(inc - word, wave);   // the wavefronts before this one
        const int before = excl & 0xFFFF, pbefore = excl >> 16, total = upto & 0xFFFF, ptotal = upto >> 16;
        const int cid        = next + before + (int)__popcll(vm & below);
        const int first_pair = next_pair + pbefore + pairs_before;  // within the chunk; the scatter pass adds the chunk's first
        next += total;
        next_pair += ptotal;
        if (pid >= end) continue;
        if (TRAIN) p.cid_of[pid] = o.valid ? cid : -1;
        if (!o.valid) continue;

        // record for the blend (and the pixel pass of the backward)
        float4 recv[NREC];
        recv[0] = make_float4(o.ipx, o.ipy, encode_size_field(o.size_px, L), conf);
#pragma unroll
        for (int q = 0; q < CPAD / 4; ++q) recv[1 + q] = make_float4(d[4 * q], d[4 * q + 1], d[4 * q + 2], d[4 * q + 3]);
        float4* rec = reinterpret_cast<float4*>(p.rec + (size_t)cid * p.rec_floats);
#pragma unroll
        for (int q = 0; q < NREC; ++q) __builtin_nontemporal_store(vf4{recv[q].x, recv[q].y, recv[q].z, recv[q].w}, reinterpret_cast<vf4*>(rec) + q);
        // point record: depth and layers for the scatter pass; softplus' and the size for the backward
        __builtin_nontemporal_store(vf4{TRAIN ? o.d_softplus : 0.f, o.z, __int_as_float(o.layers), o.size_px},
                                    reinterpret_cast<vf4*>(p.prec) + cid);
        if (TRAIN)
        {
            __builtin_nontemporal_store(pid, p.pid_of + cid);
            __builtin_nontemporal_store(first_pair, p.over_first + cid);
        }
    }
    {
        const int flags = (__ballot(not_identity) != 0 ? 1 : 0) | (__ballot(bad_index) != 0 ? 2 : 0);
        if (flags && lane == 0) atomicOr(&s_flags, flags);
    }

    // this workgroup's row of the histogram matrix [workgroup][bin]; its valid points and flags for the scan kernel,
    // which adds the chunks up (no counter of the view is touched here: nothing has to be cleared before this kernel)
    __syncthreads();
    int32_t* row = p.bin_hist + (size_t)blockIdx.x * NB;
    for (int i = threadIdx.x; i < NB; i += kBinThreads) row[i] = s_hist[i];
    if (threadIdx.x == 0)
    {
        p.chunk_valid[blockIdx.x]                = next - begin;
        p.chunk_valid[p.bin_groups + blockIdx.x] = s_flags;
        p.chunk_valid[2 * p.bin_groups + blockIdx.x] = 0;
        p.chunk_valid[3 * p.bin_groups + blockIdx.x] = next_pair;
    }
}

// ---------------------------------------------------------------------------------------------------------
// Everything between the projection and the scatter that ONE workgroup can do, in one launch:
//   * the view's counters, written (not added to, so that nothing has to clear them first): valid points and flags
//     summed over the chunks of the projection, entries from the scan; on the first view of a call the status block
//     of the whole call as well;
//   * exclusive scan of the tile totals: bin_start[i] = sum_{k<i} bin_count[k], bin_start[NB] = total;
//   * slices of split tiles: a tile with more than kSliceEntries bin entries (hundreds of points per pixel, e.g.
//     tight clusters) would keep a single workgroup busy for milliseconds; it is cut into slices of kSliceEntries
//     entries, each a workgroup of its own. slice_start[t] = number of slices of split tiles before tile t.
// The workgroups after the first clear `clear_n` 16-byte words at `clear` (the per-cell counters of the list
// kernels), which saves a launch of its own.
__global__ __launch_bounds__(1024) void scan_plan_kernel(const int32_t* __restrict__ bin_count, int32_t* __restrict__ bin_start,
                                                         int32_t* __restrict__ slice_start, int NB, long long capacity,
                                                         int32_t* __restrict__ chunk_valid, int G, ViewHeader* header,
                                                         ViewHeader* status, int first_view, int32_t* __restrict__ long_count,
                                                         uint4* __restrict__ clear, long long clear_n, int32_t* __restrict__ saved_chunk_valid)
{
    if (blockIdx.x > 0)
    {
        for (long long i = (long long)(blockIdx.x - 1) * 1024 + threadIdx.x; i < clear_n; i += (long long)(gridDim.x - 1) * 1024)
            clear[i] = make_uint4(0u, 0u, 0u, 0u);
        return;
    }
    __shared__ int s_wave[2][16];
    __shared__ int s_carry[2];
    __shared__ unsigned long long s_valid_total, s_same_total;
    __shared__ int s_flags;
    __shared__ int s_over_total;
    if (threadIdx.x == 0)
    {
        s_over_total = 0;
        s_carry[0] = s_carry[1] = 0;
        s_valid_total = s_same_total = 0;
        s_flags                 = 0;
        *long_count             = 0;
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    {
        // sums over the chunks: per wavefront first, then one LDS atomic per wavefront and sum
        unsigned long long v = 0, st = 0;
        int f = 0;
        for (int g = threadIdx.x; g < G; g += 1024)
        {
            v += (unsigned long long)(unsigned)chunk_valid[g];
            f |= chunk_valid[G + g];
            st += (unsigned long long)(unsigned)chunk_valid[2 * G + g];
        }
        // number of every chunk's first overflow row: exclusive prefix of the chunks' row counts (G <= 1024)
        {
            const int mine = (int)threadIdx.x < G ? chunk_valid[3 * G + threadIdx.x] : 0;
            int inc        = mine;
            for (int o = 1; o < 64; o <<= 1)
            {
                const int t = __shfl_up(inc, o);
                if (lane >= o) inc += t;
            }
            if (lane == 63) s_wave[0][wave] = inc;
            __syncthreads();
            int prefix = inc - mine;
            for (int w = 0; w < wave; ++w) prefix += s_wave[0][w];
            if ((int)threadIdx.x < G) chunk_valid[4 * G + threadIdx.x] = prefix;
            if ((int)threadIdx.x == G - 1) s_over_total = prefix + mine;
            if (saved_chunk_valid && (int)threadIdx.x < G) saved_chunk_valid[threadIdx.x] = chunk_valid[threadIdx.x];
            if (saved_chunk_valid && (int)threadIdx.x < kRetainedParts) saved_chunk_valid[G + threadIdx.x] = 0;  // (the blend adds)
            __syncthreads();
        }
        for (int o = 32; o > 0; o >>= 1)
        {
            v += __shfl_xor(v, o);
            st += __shfl_xor(st, o);
            f |= __shfl_xor(f, o);
        }
        if (lane == 0)
        {
            if (v) atomicAdd(&s_valid_total, v);
            if (st) atomicAdd(&s_same_total, st);
            if (f) atomicOr(&s_flags, f);
        }
    }
    for (int base = 0; base < NB; base += 1024)
    {
        const int idx = base + threadIdx.x;
        const int v   = idx < NB ? bin_count[idx] : 0;
        int inc       = v;
        for (int o = 1; o < 64; o <<= 1)
        {
            int t = __shfl_up(inc, o);
            if (lane >= o) inc += t;
        }
        if (lane == 63) s_wave[0][wave] = inc;
        __syncthreads();
        int wave_prefix = 0;
        for (int w = 0; w < wave; ++w) wave_prefix += s_wave[0][w];
        const int carry = s_carry[0];
        const int ex    = carry + wave_prefix + inc - v;  // first slot of the tile
        if (idx < NB) bin_start[idx] = ex;
        // slices of the tile's entries that fit the capacity
        int sl = 0;
        if (idx < NB)
        {
            const long long first = ex;
            long long last        = (long long)ex + v;
            if (last > capacity) last = capacity;
            const long long n = last > first ? last - first : 0;
            sl                = n > kSliceEntries ? (int)((n + kSliceEntries - 1) / kSliceEntries) : 0;
        }
        int inc2 = sl;
        for (int o = 1; o < 64; o <<= 1)
        {
            int t = __shfl_up(inc2, o);
            if (lane >= o) inc2 += t;
        }
        if (lane == 63) s_wave[1][wave] = inc2;
        __syncthreads();
        int wave_prefix2 = 0;
        for (int w = 0; w < wave; ++w) wave_prefix2 += s_wave[1][w];
        const int carry2 = s_carry[1];
        if (idx < NB) slice_start[idx] = carry2 + wave_prefix2 + inc2 - sl;
        __syncthreads();
        if (threadIdx.x == 1023)
        {
            s_carry[0] = carry + wave_prefix + inc;
            s_carry[1] = carry2 + wave_prefix2 + inc2;
        }
        __syncthreads();
    }
    if (threadIdx.x == 0)
    {
        bin_start[NB]   = s_carry[0];
        slice_start[NB] = s_carry[1];
        const unsigned long long bad = (unsigned long long)((s_flags >> 1) & 1);
        header->n_valid      = s_valid_total;
        header->n_entries    = (unsigned long long)(unsigned)s_carry[0];
        header->overflow     = 0;
        header->retained     = 0;
        header->not_identity = (unsigned long long)(s_flags & 1);
        header->bad_index    = 0;
        header->same_tile_as_previous = s_same_total;
        header->overflow_rows         = (unsigned long long)(unsigned)s_over_total;
        if (first_view)
        {
            status->n_valid = status->n_entries = status->overflow = status->retained = status->not_identity = 0;
            status->bad_index                                                       = bad;
            status->same_tile_as_previous = status->overflow_rows = 0;
        }
        else if (bad)
            status->bad_index = 1;  // (the views of a call run one after the other on the stream)
    }
}

// ---------------------------------------------------------------------------------------------------------
// Column-wise exclusive prefix of the histogram matrix [workgroup][bin]: afterwards hist[g][bin] = entries of
// `bin` that come from workgroups before g, and bin_count[bin] = the column total. No atomics anywhere in the
// binning, since atomics on a few thousand hot counters serialise. A workgroup owns 16 columns; its 16 row
// segments are summed side by side, prefixed through LDS, then each segment writes its rows' prefixes (one thread
// walking a whole column is a chain of G dependent-latency steps).
constexpr int kScanCols = 16, kScanSegs = 16;
__global__ __launch_bounds__(256) void bin_column_scan_kernel(int32_t* __restrict__ hist, int32_t* __restrict__ bin_count,
                                                              int NB, int G)
{
    __shared__ int s_seg[kScanSegs][kScanCols];
    const int c = threadIdx.x % kScanCols, seg = threadIdx.x / kScanCols;
    const int bin = blockIdx.x * kScanCols + c;
    const int rows = (G + kScanSegs - 1) / kScanSegs;
    const int g0 = seg * rows, g1 = min(G, g0 + rows);
    const bool live = bin < NB;
    int32_t* col    = hist + bin;
    int sum         = 0;
    if (live)
        for (int g = g0; g < g1; g += 8)
        {
            int v[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = (g + k < g1) ? col[(size_t)(g + k) * NB] : 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) sum += v[k];
        }
    s_seg[seg][c] = sum;
    __syncthreads();
    int run = 0;
    for (int k = 0; k < seg; ++k) run += s_seg[k][c];
    if (!live) return;
    for (int g = g0; g < g1; g += 8)
    {
        int v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = (g + k < g1) ? col[(size_t)(g + k) * NB] : 0;
#pragma unroll
        for (int k = 0; k < 8; ++k)
        {
            if (g + k < g1) col[(size_t)(g + k) * NB] = run;
            run += v[k];
        }
    }
    if (seg == kScanSegs - 1) bin_count[bin] = run;
}

// ---------------------------------------------------------------------------------------------------------
// A bin entry holds what the list kernels need of a (point, layer) pair: the depth bits, the compact point number and
// the cell of its tile that the footprint starts at. Depths of valid points are positive (31 bits), a cell takes 10
// bits, so clouds of up to 2^23 points have entries of 8 bytes; larger ones use 16.
template <bool PACKED>
struct BinEntry;
template <>
struct BinEntry<true>
{
    using T = u64;
    static __device__ __forceinline__ T make(unsigned zbits, unsigned cid, int px, int py)
    {
        const unsigned cell = (unsigned)((py & (kTile - 1)) << kTileShift) | (unsigned)(px & (kTile - 1));
        return ((u64)zbits << (kPackedIdBits + 2 * kTileShift)) | ((u64)cid << (2 * kTileShift)) | cell;
    }
    static __device__ __forceinline__ int cell(const T& e) { return (int)((unsigned)e & (kTilePixels - 1)); }
    static __device__ __forceinline__ u64 key(const T& e)
    {
        return ((e >> (kPackedIdBits + 2 * kTileShift)) << 32) | ((e >> (2 * kTileShift)) & ((1u << kPackedIdBits) - 1));
    }
};
template <>
struct BinEntry<false>
{
    using T = uint4;
    static __device__ __forceinline__ T make(unsigned zbits, unsigned cid, int px, int py)
    {
        const unsigned cell = (unsigned)((py & (kTile - 1)) << kTileShift) | (unsigned)(px & (kTile - 1));
        return make_uint4(zbits, cid, cell, 0u);
    }
    static __device__ __forceinline__ int cell(const T& e) { return (int)e.z; }
    static __device__ __forceinline__ u64 key(const T& e) { return ((u64)e.x << 32) | (u64)e.y; }
};
static_assert(kTilePixels == 1 << (2 * kTileShift), "a cell number takes 2 kTileShift bits");

// One bin entry per (point, layer), in the tile of the footprint's first pixel. A workgroup walks
// the records that its chunk of the points left at the compact numbers; its slots inside every bin are contiguous
// and start at bin_start[bin] + hist[workgroup][bin].
template <bool PACKED>
__global__ __launch_bounds__(kBinThreads) void bin_scatter_kernel(const ForwardParams p)
{
    using E = BinEntry<PACKED>;
    typename E::T* __restrict__ entries = reinterpret_cast<typename E::T*>(p.bin_entries);
    extern __shared__ int s_cur[];
    const int NB       = p.geom.bin_off[p.num_layers];
    const int32_t* row = p.bin_hist + (size_t)blockIdx.x * NB;
    for (int i = threadIdx.x; i < NB; i += kBinThreads) s_cur[i] = p.bin_start[i] + row[i];
    __syncthreads();
    int begin, end;
    chunk_point_range(p, begin, end);
    const int n      = p.chunk_valid[blockIdx.x];
    const int pair_base = p.chunk_valid[4 * p.bin_groups + blockIdx.x];
    unsigned dropped = 0;
    constexpr int U  = 2;  // records of a thread in flight together
    for (int cid0 = begin + (int)threadIdx.x; cid0 < begin + n; cid0 += U * kBinThreads)
    {
        float4 tail[U];  // {softplus', depth, layers, size_px}
        float2 ip[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
        {
            const int cid = cid0 + u * kBinThreads;
            if (cid < begin + n)
            {
                const vf4 t = __builtin_nontemporal_load(reinterpret_cast<const vf4*>(p.prec) + cid);
                tail[u]     = make_float4(t.x, t.y, t.z, t.w);
                ip[u]   = *reinterpret_cast<const float2*>(p.rec + (size_t)cid * p.rec_floats);
                // the point's first overflow row: the projection numbered it within the chunk, the scan found the chunk's first
                if (p.over_first) p.over_first[cid] += pair_base;
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
        {
            const int cid = cid0 + u * kBinThreads;
            if (cid >= begin + n) break;
            PointProjection o;
            o.ipx    = ip[u].x;
            o.ipy    = ip[u].y;
            o.layers = __float_as_int(tail[u].z);
            const unsigned zbits = __float_as_uint(tail[u].y);
            for_point_tiles(p.geom, o, s_cur,
                            [&](int px, int py, int* bc)
                            {
                                const int slot = atomicAdd(bc, 1);
                                if ((unsigned long long)(unsigned)slot < (unsigned long long)p.capacity)
                                    entries[slot] = E::make(zbits, (unsigned)cid, px, py);
                                else
                                    dropped += 1;
                            });
        }
    }
    if (dropped) atomicAdd(&p.status->overflow, (u64)dropped);
}

// ---------------------------------------------------------------------------------------------------------
// Walks entries [0, n) with the workgroup, U loads of a thread in flight together.
template <int THREADS, int U, typename T, typename F>
__device__ __forceinline__ void for_entries(const T* __restrict__ entries, int n, F&& f)
{
    for (int i0 = threadIdx.x; i0 < n; i0 += U * THREADS)
    {
        T e[U];
#pragma unroll
        for (int j = 0; j < U; ++j)
            if (i0 + THREADS * j < n) e[j] = entries[i0 + THREADS * j];
#pragma unroll
        for (int j = 0; j < U; ++j)
            if (i0 + THREADS * j < n) f(e[j]);
    }
}

// The keys of a tile are filed by cell: the cell (px, py) holds the points whose 2 x 2 footprint starts at that pixel,
// so that a (point, layer) pair is written once and the four pixels it covers gather it from the cell. There is one key
// per bin entry: the keys of a tile start where its bin entries do.
// One workgroup per tile (blocks [0, NB)) plus one per slice of a split tile (blocks from NB on; those past the
// number of slices the plan found return at once). Pass `SCATTER == false`: count the entries of the tile's 1024
// cells in LDS and write the counts (split tiles only). Pass `SCATTER == true`: the counts of a tile that is not
// split, then the exclusive scan of the 1024 counts, per-cell list starts, and the 64-bit keys (depth bits << 32 | compact point number) into their lists. A slice adds its counts to the
// tile's with atomics; when it places its keys it first counts its own entries per cell again and claims that many
// slots of each cell's list with one atomic.
// (THREADS: 256 for the counting pass, whose idle workgroups for unused slices are cheaper that way; 1024 for the
// placement pass, where two workgroups per CU with their 64 KB of LDS then make 32 wavefronts instead of 8)
constexpr int kScatterThreads = 1024;
template <bool SCATTER, int THREADS, bool PACKED>
__global__ __launch_bounds__(THREADS) void tile_lists_kernel(const ForwardParams p)
{
    using E  = BinEntry<PACKED>;
    using ET = typename E::T;
    __shared__ int s_cnt[kTilePixels];
    // per-cell entries of a slice (placement pass only; one word in the counting pass, whose code below never runs)
    __shared__ int s_mine[SCATTER ? kTilePixels : 1];
    auto mine = [&](int i) -> int& { return s_mine[SCATTER ? i : 0]; };
    __shared__ int s_wave[THREADS / 64];
    const int NB = p.geom.bin_off[p.num_layers];
    int bin      = blockIdx.x;
    int slice    = -1;  // -1: the tile's own workgroup
    if (bin >= NB)
    {
        const int e = bin - NB;
        if (e >= p.slice_start[NB]) return;
        // the tile with slice_start[t] <= e < slice_start[t + 1]: a split one, tiles without slices have empty ranges
        int lo = 0, hi = NB;
        while (hi - lo > 1)
        {
            const int mid = (lo + hi) >> 1;
            if (p.slice_start[mid] <= e)
                lo = mid;
            else
                hi = mid;
        }
        bin   = lo;
        slice = e - p.slice_start[bin];
    }
    long long first = p.bin_start[bin];
    long long last  = p.bin_start[bin + 1];
    if (last > p.capacity) last = p.capacity;  // entries beyond the capacity were dropped by the scatter
    const bool split = last - first > kSliceEntries;
    if (slice >= 0)
    {
        first += (long long)slice * kSliceEntries;
        last = min(last, first + kSliceEntries);
    }
    const int n          = first < last ? (int)(last - first) : 0;
    const ET* entries    = reinterpret_cast<const ET*>(p.bin_entries) + first;
    int32_t* counts      = p.counts + (size_t)bin * kTilePixels;

    if (!SCATTER)
    {
        if (slice < 0) return;  // the slices count for a split tile; any other tile is counted where its keys are placed
        for (int i = threadIdx.x; i < kTilePixels; i += THREADS) s_cnt[i] = 0;
        __syncthreads();
        // (sixteen loads of a thread in flight: the slices of a view are few, and the kernel lasts as long as one slice's
        // round trips to memory, one after the other)
        for_entries<THREADS, 16>(entries, n, [&](const ET& e) { atomicAdd(&s_cnt[E::cell(e)], 1); });
        __syncthreads();
        for (int i = threadIdx.x; i < kTilePixels; i += THREADS)
        {
            const int c = s_cnt[i];
            if (c) atomicAdd(&counts[i], c);  // cleared before this kernel
        }
        return;
    }

    // This workgroup files at most kSliceEntries entries: a thread reads its share once, all loads in flight together,
    // and keeps it in registers from the count to the placement.
    constexpr int MAXE = (kSliceEntries + THREADS - 1) / THREADS;
    ET mine_e[MAXE];
    const int n_filed = split && slice < 0 ? 0 : n;  // (the workgroup of a split tile files nothing itself)
#pragma unroll
    for (int j = 0; j < MAXE; ++j)
        if ((int)threadIdx.x + j * THREADS < n_filed) mine_e[j] = entries[(int)threadIdx.x + j * THREADS];
    auto for_mine = [&](auto&& f)
    {
#pragma unroll
        for (int j = 0; j < MAXE; ++j)
            if ((int)threadIdx.x + j * THREADS < n_filed) f(mine_e[j]);
    };
    // exclusive scan of the tile's 1024 lengths: PER consecutive pixels per thread
    constexpr int PER = kTilePixels / THREADS;
    const int base4   = threadIdx.x * PER;
    int v[PER], sum = 0;
    if (!split)
    {
        for (int i = threadIdx.x; i < kTilePixels; i += THREADS) s_cnt[i] = 0;
        __syncthreads();
        for_mine([&](const ET& e) { atomicAdd(&s_cnt[E::cell(e)], 1); });
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < PER; ++i)
    {
        if (split)
            v[i] = counts[base4 + i];
        else
            counts[base4 + i] = v[i] = s_cnt[base4 + i];  // (the slots that this thread overwrites with the list starts below)
        sum += v[i];
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int inc = sum;
    for (int o = 1; o < 64; o <<= 1)
    {
        int t = __shfl_up(inc, o);
        if (lane >= o) inc += t;
    }
    if (lane == 63) s_wave[wave] = inc;
    if (slice >= 0)
        for (int i = threadIdx.x; i < kTilePixels; i += THREADS) mine(i) = 0;
    __syncthreads();
    int prefix = inc - sum;
    for (int w = 0; w < wave; ++w) prefix += s_wave[w];
    const int key_start = p.bin_start[bin];  // one key per bin entry: the tile's keys start where its entries do
    int32_t* cursor     = p.cursor + (size_t)bin * kTilePixels;
#pragma unroll
    for (int i = 0; i < PER; ++i)
    {
        s_cnt[base4 + i] = key_start + prefix;  // running slot of the cell
        if (slice < 0)
        {
            int where = key_start + prefix;
            if (v[i] > kLongList && (long long)key_start + prefix + v[i] <= p.capacity)
            {
                // a long list: hand its segments to the reduction pass and point the cell at their results
                const int nseg = (v[i] + kLongSegment - 1) / kLongSegment;
                const int base = atomicAdd(p.long_count, nseg);
                if (base + nseg <= p.max_long_items)
                {
                    for (int sg = 0; sg < nseg; ++sg)
                        p.long_items[base + sg] = make_int2(key_start + prefix + sg * kLongSegment, min(kLongSegment, v[i] - sg * kLongSegment));
                    where = -1 - base;
                }
            }
            cursor[base4 + i] = where;
        }
        prefix += v[i];
    }
    if (split && slice < 0) return;  // the slices place the keys
    __syncthreads();
    unsigned dropped = 0;
    if (slice >= 0)
    {
        // this slice's share of every cell's list: count, then claim the slots with one atomic per cell
        int32_t* run = p.run + (size_t)bin * kTilePixels;
        for_mine([&](const ET& e) { atomicAdd(&mine(E::cell(e)), 1); });
        __syncthreads();
        for (int i = threadIdx.x; i < kTilePixels; i += THREADS)
        {
            const int c = mine(i);
            if (c) s_cnt[i] += atomicAdd(&run[i], c);  // cleared before the counting kernel
        }
        __syncthreads();
        for_mine(
                    [&](const ET& e)
                    {
                        const u64 key  = E::key(e);
                        const int slot = atomicAdd(&s_cnt[E::cell(e)], 1);
                        if ((unsigned long long)(unsigned)slot < (unsigned long long)p.capacity)
                            p.keys[slot] = key;
                        else
                            dropped += 1;
                    });
        if (dropped) atomicAdd(&p.status->overflow, (u64)dropped);
        return;
    }
    // Keys of a tile whose lists fit into LDS are staged there and copied out with full-line stores; the keys of
    // bigger tiles go to their lists directly (8-byte stores scattered over the tile's region).
    extern __shared__ u64 s_keys[];
    const int tile_total = p.bin_start[bin + 1] - key_start;
    const bool staged    = tile_total <= kStageKeys && (long long)key_start + tile_total <= p.capacity;
    for_mine(
                [&](const ET& e)
                {
                    const u64 key  = E::key(e);
                    const int slot = atomicAdd(&s_cnt[E::cell(e)], 1);
                    if (staged)
                        s_keys[slot - key_start] = key;
                    else if ((unsigned long long)(unsigned)slot < (unsigned long long)p.capacity)
                        p.keys[slot] = key;
                    else
                        dropped += 1;
                });
    if (staged)
    {
        __syncthreads();
        u64* dst = p.keys + key_start;
        for (int i = threadIdx.x; i < tile_total; i += THREADS) __builtin_nontemporal_store(s_keys[i], dst + i);
    }
    if (dropped) atomicAdd(&p.status->overflow, (u64)dropped);
}

// ---------------------------------------------------------------------------------------------------------
// A pixel's list is the union of the lists of the four cells whose 2 x 2 footprints cover it: (x-1, y-1), (x, y-1),
// (x-1, y), (x, y) (CountAndCollectTiled adds every point to the four pixels of its footprint,
// RenderForward.cu:300-366; here a point is filed once, under its footprint's first pixel, and the pixels gather).
// The K nearest entries of a pixel are among the K nearest of each of its cells, and a cell serves four pixels, so the
// sort (FastSortFusedNew, RenderForward.cu:474-1059) is split:
//   cell_sort_kernel   every cell's list sorted in place, ascending, and cut to its 16 smallest keys: a list of up to
//                      8 keys by one lane (a sorting network over registers), a longer one by a 16-lane DPP row that
//                      streams it in chunks of 16.
//   blend_kernel       a wavefront owns an 8 x 8 block of pixels, one pixel per lane: a pixel with up to 8 entries
//                      sorts them with a network, any other merges the (sorted, cut) lists of its four cells; then the
//                      alpha blend front to back (RenderForward.cu:820-1048).
// A pixel's colour is summed in the order of a balanced binary tree over the list positions.
constexpr int kLaneSortMax = 8;   // longest list that a lane sorts with a network
constexpr int kStagedKeys  = 8;   // keys per cell that blend_kernel stages in LDS for the merging lanes

// {first key (negative: a long list, whose candidates are in `cand`), readable keys, entries} of a cell
__device__ __forceinline__ int4 cell_info(const ForwardParams& p, int cell)
{
    const int len   = p.counts[cell];
    const int start = p.cursor[cell];  // negative: a long list, reduced to candidates by long_list_reduce_kernel
    // keys actually there: the key storage may have ended inside the list
    const int rd = start < 0 ? ((len + kLongSegment - 1) / kLongSegment) * 16 : (int)max(0ll, min((long long)len, p.capacity - start));
    return make_int4(start, rd, len, 0);
}

// the keys of a cell: in the key array, or the candidate rows that the reduction pass left for a long list
__device__ __forceinline__ u64* cell_keys(const ForwardParams& p, int start)
{
    return start >= 0 ? p.keys + (unsigned)start : p.cand + (size_t)(unsigned)(-1 - start) * 16;
}

// the same for the cell (cx, cy) of the layer of `tc`, its readable keys cut to the kCellKeep that cell_sort_kernel
// left in order (empty outside the layer and in its last row and column, where no footprint starts)
__device__ __forceinline__ int4 load_cell(const ForwardParams& p, const TileCtx& tc, int cx, int cy)
{
    int4 r = make_int4(0, 0, 0, 0);
    if (cx >= 0 && cy >= 0 && cx < tc.w - 1 && cy < tc.h - 1)
    {
        const int bin = tc.bin + ((cx - tc.x0) >> kTileShift) + ((cy - tc.y0) >> kTileShift) * tc.tiles_x;  // shifts round down
        r   = cell_info(p, (bin << (2 * kTileShift)) | ((cy & (kTile - 1)) << kTileShift) | (cx & (kTile - 1)));
        r.y = min(r.y, kCellKeep);
    }
    return r;
}

template <int C>
__device__ __forceinline__ void store_pixel(const ForwardParams& p, float* img, int lw, int lh, int gx, int gy, const float (&col)[C])
{
    // offsets inside one view's image stay far below 2^32 (the pyramid has at most kMaxBins tiles)
    if (p.layout == TRIPS_LAYOUT_CHW)
    {
        const size_t plane = (size_t)lw * lh;
        float* o           = img + ((size_t)p.view_index * C) * plane;
        const unsigned at  = __umul24((unsigned)gy, (unsigned)lw) + (unsigned)gx;
#pragma unroll
        for (int c = 0; c < C; ++c) __builtin_nontemporal_store(col[c], (o + c * plane) + at);
    }
    else
    {
        float* o          = img + ((size_t)p.view_index * lh * lw) * C;
        const unsigned at = (__umul24((unsigned)gy, (unsigned)lw) + (unsigned)gx) * C;
#pragma unroll
        for (int c = 0; c < C; ++c) __builtin_nontemporal_store(col[c], o + at + c);
    }
}

// ---- one list per lane: sorting networks over registers (Batcher's odd-even merge sort; keys are distinct or the
// all-ones filler) ----
__device__ __forceinline__ void sort_pair(u64& a, u64& b)
{
    const bool sw = b < a;
    const u64 lo = sw ? b : a, hi = sw ? a : b;
    a = lo;
    b = hi;
}
// a key with a tag that travels with it
struct TaggedKey
{
    u64 key;
    int tag;
};
__device__ __forceinline__ void sort_pair(TaggedKey& a, TaggedKey& b)
{
    const bool sw = b.key < a.key;
    const TaggedKey lo{sw ? b.key : a.key, sw ? b.tag : a.tag}, hi{sw ? a.key : b.key, sw ? a.tag : b.tag};
    a = lo;
    b = hi;
}
template <typename T>
__device__ __forceinline__ void lane_sort4(T (&k)[kLaneSortMax])
{
    sort_pair(k[0], k[1]), sort_pair(k[2], k[3]);
    sort_pair(k[0], k[2]), sort_pair(k[1], k[3]);
    sort_pair(k[1], k[2]);
}
template <typename T>
__device__ __forceinline__ void lane_sort8(T (&k)[kLaneSortMax])
{
    sort_pair(k[0], k[1]), sort_pair(k[2], k[3]), sort_pair(k[4], k[5]), sort_pair(k[6], k[7]);
    sort_pair(k[0], k[2]), sort_pair(k[1], k[3]), sort_pair(k[4], k[6]), sort_pair(k[5], k[7]);
    sort_pair(k[1], k[2]), sort_pair(k[5], k[6]);
    sort_pair(k[0], k[4]), sort_pair(k[1], k[5]), sort_pair(k[2], k[6]), sort_pair(k[3], k[7]);
    sort_pair(k[2], k[4]), sort_pair(k[3], k[5]);
    sort_pair(k[1], k[2]), sort_pair(k[3], k[4]), sort_pair(k[5], k[6]);
}
// ascending sort of the first nmax (wave-uniform) of the lane's keys
template <typename T>
__device__ __forceinline__ void lane_sort(T (&k)[kLaneSortMax], int nmax)
{
    if (nmax > 4)
        lane_sort8(k);
    else if (nmax > 2)
        lane_sort4(k);
    else if (nmax > 1)
        sort_pair(k[0], k[1]);
}
// largest value of v (0 .. LIMIT) over the wavefront's lanes, as a scalar
template <int LIMIT>
__device__ __forceinline__ int wave_max_small(int v)
{
    int m = 0;
#pragma unroll
    for (int t = 1; t <= LIMIT; ++t)
        if (__ballot(v >= t)) m = t;
    return m;
}

// Sum of a sequence in the order of a balanced binary tree over the positions, (0 + 1) + (2 + 3), ...: push<J>(v) for
// J = 0, 1, ..., then total(). A skipped tail counts as zeros.
template <int C, int LEVELS>
struct TreeSum
{
    float acc[LEVELS][C];
    __device__ __forceinline__ TreeSum()
    {
#pragma unroll
        for (int l = 0; l < LEVELS; ++l)
#pragma unroll
            for (int c = 0; c < C; ++c) acc[l][c] = 0.f;
    }
    template <int J>
    __device__ __forceinline__ void push(const float (&v)[C])
    {
        float t[C];
#pragma unroll
        for (int c = 0; c < C; ++c) t[c] = v[c];
#pragma unroll
        for (int l = 0; l < LEVELS; ++l)
        {
            if ((J >> l) & 1)
            {
#pragma unroll
                for (int c = 0; c < C; ++c) t[c] = acc[l][c] + t[c], acc[l][c] = 0.f;
            }
            else
            {
#pragma unroll
                for (int c = 0; c < C; ++c) acc[l][c] = t[c];
                break;
            }
        }
    }
    __device__ __forceinline__ void total(float (&out)[C])
    {
#pragma unroll
        for (int c = 0; c < C; ++c) out[c] = acc[0][c];
#pragma unroll
        for (int l = 1; l < LEVELS; ++l)
#pragma unroll
            for (int c = 0; c < C; ++c) out[c] = acc[l][c] + out[c];
    }
};

// ---------------------------------------------------------------------------------------------------------
__device__ __forceinline__ u64 shfl16(u64 v, int src)
{
    unsigned lo = (unsigned)v, hi = (unsigned)(v >> 32);
    lo = __shfl(lo, src, 16);
    hi = __shfl(hi, src, 16);
    return ((u64)hi << 32) | lo;
}

// The 16 smallest of key_at(0 .. readable - 1) for each of the wavefront's four 16-lane rows, ascending over the row's
// lanes (all-ones where the row has fewer keys). A chunk of 16 further keys is sorted and merged only if one of them
// beats the current 16th; most chunks of a long list are passed over, so the loop runs at the latency of its loads:
// four chunks are requested together and the next four are in flight while these are looked at. The first 16 + 64
// keys can be requested ahead of the call (row_top16_first), e.g. while the rows still work on other lists.
struct RowKeys
{
    u64 k0;              // keys 0..15
    u64 f0, f1, f2, f3;  // keys 16..79
};
template <typename KeyAt>
__device__ __forceinline__ void row_load4(KeyAt&& key_at, int readable, int base, u64& f0, u64& f1, u64& f2, u64& f3)
{
    const int i = base + (int)(threadIdx.x & 15);
    const u64 kInf = ~0ull;
    f0 = i < readable ? key_at(i) : kInf;
    f1 = i + 16 < readable ? key_at(i + 16) : kInf;
    f2 = i + 32 < readable ? key_at(i + 32) : kInf;
    f3 = i + 48 < readable ? key_at(i + 48) : kInf;
}
template <typename KeyAt>
__device__ __forceinline__ RowKeys row_top16_first(KeyAt&& key_at, int readable)
{
    RowKeys r;
    const int sub = threadIdx.x & 15;
    r.k0 = sub < readable ? key_at(sub) : ~0ull;
    row_load4(key_at, readable, 16, r.f0, r.f1, r.f2, r.f3);
    return r;
}
template <typename KeyAt>
__device__ __forceinline__ u64 row_top16(KeyAt&& key_at, int readable, const RowKeys& first)
{
    const int lane = threadIdx.x & 63;
    const int grp  = lane >> 4;
    int maxlen = readable;
    maxlen     = max(maxlen, __shfl_xor(maxlen, 16));
    maxlen     = max(maxlen, __shfl_xor(maxlen, 32));
    const u64 grp_mask = 0xFFFFull << (grp * 16);
    maxlen             = __builtin_amdgcn_readfirstlane(maxlen);
    u64 best = row_sort16(first.k0);
    auto consider = [&](u64 k)
    {
        const u64 worst = shfl16(best, 15);
        const bool need = k < worst;
        if (__ballot(need) & grp_mask)
        {
            k           = row_sort16(k);
            const u64 r = row_xor_u64<15>(k);  // reversed: lane i sees the (15-i)-th smallest new key
            best        = best < r ? best : r;
            best        = row_merge16(best);
        }
    };
    if (maxlen > 16)
    {
        u64 c0 = first.f0, c1 = first.f1, c2 = first.f2, c3 = first.f3;
        u64 n0 = c0, n1 = c1, n2 = c2, n3 = c3;
        for (int base = 16; base < maxlen; base += 64)
        {
            if (base + 64 < maxlen) row_load4(key_at, readable, base + 64, n0, n1, n2, n3);
            consider(c0);
            if (base + 16 < maxlen) consider(c1);
            if (base + 32 < maxlen) consider(c2);
            if (base + 48 < maxlen) consider(c3);
            c0 = n0, c1 = n1, c2 = n2, c3 = n3;
        }
    }
    return best;
}
template <typename KeyAt>
__device__ __forceinline__ u64 row_top16(KeyAt&& key_at, int readable)
{
    return row_top16(key_at, readable, row_top16_first(key_at, readable));
}

// Reduction pass over the segments of long lists (tile_lists_kernel hands them out): a 16-lane row keeps the 16
// smallest keys of a segment. Persistent workgroups, the four rows of a wavefront take consecutive segments.
__global__ __launch_bounds__(256) void long_list_reduce_kernel(const ForwardParams p)
{
    const int n    = min(*p.long_count, p.max_long_items);
    const int lane = threadIdx.x & 63;
    const int rows = gridDim.x * 16;
    for (int first = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 4; first < n; first += rows)
    {
        const int item = first + (lane >> 4);
        int2 seg       = make_int2(0, 0);
        if (item < n) seg = p.long_items[item];
        if (seg.x < 0 || seg.y < 0 || seg.y > kLongSegment || (long long)seg.x + seg.y > p.capacity) seg = make_int2(0, 0);
        const u64* src = p.keys + seg.x;
        const u64 best = row_top16([&](int i) { return src[i]; }, seg.y);
        if (item < n) p.cand[(size_t)item * 16 + (lane & 15)] = best;
    }
}

// Every cell's list in ascending order, in place; of a list longer than kCellKeep its kCellKeep smallest keys, at its
// start. A workgroup takes 64 consecutive cells (their lists follow each other in the key array); the sixteen
// workgroups of a tile run on the XCD that blends the tile. The first wavefront sorts the lists of up to kLaneSortMax
// keys, one cell per lane, with a network; the longer lists are taken, one after the other, by whichever of the
// sixteen 16-lane rows of the workgroup's four wavefronts is free, and streamed (a wavefront that kept all 64 cells to
// itself walked up to 64 long lists one after the other, four at a time: in a crowded tile that chain of memory round
// trips was the kernel's duration). The other three wavefronts start on the long lists while the first sorts the
// short ones.
__global__ __launch_bounds__(256) void cell_sort_kernel(const ForwardParams p)
{
    __shared__ int s_start[64], s_rd[64];
    __shared__ unsigned char s_long[64];  // lanes of the cells with a longer list
    __shared__ int s_num_long, s_next;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int NB   = p.geom.bin_off[p.num_layers];
    const long long lblock = xcd_tile_block(blockIdx.x, 16);
    if (lblock >= (long long)NB * 16) return;
    int4 info = make_int4(0, 0, 0, 0);
    if (wave == 0)
    {
        const int cell = (int)lblock * 64 + lane;
        info           = cell_info(p, cell);
        const int rd   = info.y;
        const u64 longer = __ballot(rd > kLaneSortMax);
        s_start[lane] = info.x, s_rd[lane] = rd;
        if (rd > kLaneSortMax) s_long[__popcll(longer & ((1ull << lane) - 1ull))] = (unsigned char)lane;
        if (lane == 0) s_num_long = (int)__popcll(longer), s_next = 0;
    }
    __syncthreads();
    // ---- up to kLaneSortMax keys: one cell per lane of the first wavefront, while the other wavefronts start on the
    // longer lists ----
    if (wave == 0)
    {
        const int rd    = info.y;
        u64* const base = cell_keys(p, info.x);
        const int mine = rd <= kLaneSortMax ? rd : 0;
        const int nmax = wave_max_small<kLaneSortMax>(mine);
        if (nmax > 1)
        {
            u64 k[kLaneSortMax];
#pragma unroll
            for (int i = 0; i < kLaneSortMax; ++i)
            {
                k[i] = ~0ull;
                if (i < nmax && i < mine) k[i] = base[i];
            }
            lane_sort(k, nmax);
            if (mine > 1)
            {
#pragma unroll
                for (int i = 0; i < kLaneSortMax; ++i)
                    if (i < nmax && i < mine) base[i] = k[i];
            }
        }
    }
    // ---- longer lists: one cell per 16-lane row; a row takes the next list that nobody has taken yet (the first
    // wavefront's rows join when its short lists are done), and the first keys of a row's next list are requested
    // before it works on this one ----
    const int num_long = s_num_long;
    if (num_long == 0) return;
    const int sub = lane & 15;
    struct Pass
    {
        u64* base;
        int readable;
        RowKeys first;
    };
    auto take = [&]()
    {
        int index = 0;
        if (sub == 0) index = atomicAdd(&s_next, 1);
        return __shfl(index, lane & ~15);
    };
    auto pass_of = [&](int index)
    {
        Pass ps;
        const bool has = index < num_long;
        const int src  = has ? (int)s_long[index] : 0;
        ps.base        = cell_keys(p, s_start[src]);
        ps.readable    = has ? s_rd[src] : 0;
        u64* const rb  = ps.base;
        ps.first       = row_top16_first([&](int i) { return rb[i]; }, ps.readable);
        return ps;
    };
    int index = take();
    Pass cur  = pass_of(index);
    // (the rows of a wavefront walk in step: until none of them has a list)
    while (__ballot(index < num_long) != 0ull)
    {
        const int next_index = take();
        Pass nxt             = pass_of(next_index);
        u64* const rb  = cur.base;
        const u64 best = row_top16([&](int i) { return rb[i]; }, cur.readable, cur.first);
        if (sub < min(cur.readable, kCellKeep)) rb[sub] = best;
        cur   = nxt;
        index = next_index;
    }
}

// One pixel per lane, 8 x 8 pixels per wavefront, a quarter of a tile per workgroup (the four of a tile on one XCD).
template <int C, bool TRAIN>
__global__ __launch_bounds__(256) void blend_kernel(const ForwardParams p)
{
    constexpr int CPAD = (C + 3) & ~3;
    constexpr int RF   = 4 + CPAD;  // floats per blend record
    constexpr int NQ   = CPAD / 4;
    constexpr int BATCH = CPAD <= 8 ? 8 : 4;  // list positions whose records are requested together
    __shared__ int4 s_cells[4][81];
    __shared__ u64 s_keys[4][81 * kStagedKeys];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int NB   = p.geom.bin_off[p.num_layers];
    const long long lblock = xcd_tile_block(blockIdx.x, 4);
    if (lblock >= (long long)NB * 4) return;
    const int bin = (int)(lblock >> 2), quarter = (int)(lblock & 3);
    const TileCtx tc = tile_ctx(p.geom, bin);
    const int bx = ((quarter & 1) << 4) + ((wave & 1) << 3), by = ((quarter >> 1) << 4) + ((wave >> 1) << 3);
    const int lx = lane & 7, ly = lane >> 3;
    const int pix = (bin << (2 * kTileShift)) | ((by + ly) << kTileShift) | (bx + lx);
    const int gx = tc.x0 + bx + lx, gy = tc.y0 + by + ly;
    const bool live = gx < tc.w && gy < tc.h;  // false for the padding of partial tiles
    if (tc.x0 + bx >= tc.w || tc.y0 + by >= tc.h)
    {
        // a block of padding: its rows of the saved tables are defined as empty
        if (TRAIN) __builtin_nontemporal_store(0, p.retained + pix);
        return;
    }

    // The block gathers from the 9 x 9 cells (gx0 - 1 .. gx0 + 7) x (gy0 - 1 .. gy0 + 7): one cell per lane, then
    // the 17 that are left; a pixel takes its four from LDS.
    {
        const int i1 = lane, i2 = 64 + lane;
        s_cells[wave][i1] = load_cell(p, tc, tc.x0 + bx - 1 + i1 % 9, tc.y0 + by - 1 + i1 / 9);
        if (i2 < 81) s_cells[wave][i2] = load_cell(p, tc, tc.x0 + bx - 1 + i2 % 9, tc.y0 + by - 1 + i2 / 9);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int ci0 = ly * 9 + lx;  // the pixel's cells: ci0, ci0 + 1, ci0 + 9, ci0 + 10
    const int4 c0 = s_cells[wave][ci0], c1 = s_cells[wave][ci0 + 1], c2 = s_cells[wave][ci0 + 9], c3 = s_cells[wave][ci0 + 10];
    const int total  = live ? c0.y + c1.y + c2.y + c3.y : 0;  // keys to choose from (each cell's cut to kCellKeep)
    const int length = c0.z + c1.z + c2.z + c3.z;             // entries (0 for padding: its cells are empty)
    const int n      = min(total, p.list_depth);              // list positions that hold an entry
    const bool merges = total > kLaneSortMax;

    unsigned id[16];  // compact numbers of the pixel's entries, nearest first
    // where each entry came from, for the backward: which of the pixel's four cells (bits 4..5) and its place in that
    // cell's sorted list (bits 0..3); one byte per list position, four positions per word
    unsigned tagw[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < 16; ++j) id[j] = ~0u;

    // ---- up to kLaneSortMax keys: load them all, sort with a network ----
    {
        const int mine = merges ? 0 : total;
        const int nmax = wave_max_small<kLaneSortMax>(mine);
        if (nmax > 0)
        {
            // position i of the concatenation of the four cell lists lies in cell (i >= o1) + (i >= o2) + (i >= o3)
            // (sums of steps rather than a chain of selects: the compiler turns the chain into a table in memory);
            // none of these cells has a long list
            TaggedKey k[kLaneSortMax];
            const int o1 = c0.y, o2 = o1 + c1.y, o3 = o2 + c2.y;
            const int b0 = c0.x, b1 = c1.x - o1, b2 = c2.x - o2, b3 = c3.x - o3;
#pragma unroll
            for (int i = 0; i < kLaneSortMax; ++i)
            {
                k[i].key = ~0ull;
                k[i].tag = 0;
                if (i < nmax)
                {
                    const int base = b0 + (i >= o1 ? b1 - b0 : 0) + (i >= o2 ? b2 - b1 : 0) + (i >= o3 ? b3 - b2 : 0);
                    if (i < mine) k[i].key = p.keys[(unsigned)(base + i)];
                    // cell w, place i - (first position of cell w)
                    if (TRAIN)
                        k[i].tag = (((i >= o1) + (i >= o2) + (i >= o3)) << 4) |
                                   (i - ((i >= o1 ? o1 : 0) + (i >= o2 ? o2 - o1 : 0) + (i >= o3 ? o3 - o2 : 0)));
                }
            }
            lane_sort(k, nmax);
#pragma unroll
            for (int i = 0; i < kLaneSortMax; ++i)
                if (i < mine)
                {
                    id[i] = (unsigned)k[i].key;
                    tagw[i / 4] |= (unsigned)k[i].tag << (8 * (i & 3));
                }
        }
    }
    // ---- more: merge the four sorted cell lists. The first kStagedKeys keys of the block's cells wait in LDS; a
    // lane that needs more of one cell reads them from memory. ----
    const u64 merging = __ballot(merges);
    if (merging)
    {
        // slot s = cell (s / kStagedKeys), key (s % kStagedKeys): kStagedKeys lanes read consecutive keys of a cell
        static_assert(kStagedKeys == 8, "the slot arithmetic below");
#pragma unroll 1
        for (int s0 = 0; s0 < 81 * kStagedKeys; s0 += 64)
        {
            const int s = s0 + lane;
            if (s < 81 * kStagedKeys)
            {
                const int4 c = s_cells[wave][s >> 3];
                if ((s & 7) < c.y) s_keys[wave][s] = cell_keys(p, c.x)[s & 7];
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (merges)
        {
            const u64 kInf = ~0ull;
            // key q of one of the pixel's cells (all-ones past its end)
            auto key_of = [&](int ci, const int4& c, int q) -> u64
            {
                u64 v = kInf;
                if (q < c.y) v = q < kStagedKeys ? s_keys[wave][ci * kStagedKeys + q] : cell_keys(p, c.x)[q];
                return v;
            };
            u64 h0 = key_of(ci0, c0, 0), h1 = key_of(ci0 + 1, c1, 0), h2 = key_of(ci0 + 9, c2, 0), h3 = key_of(ci0 + 10, c3, 0);
            int q0 = 0, q1 = 0, q2 = 0, q3 = 0;  // heads of the four lists
#pragma unroll
            for (int j = 0; j < 16; ++j)
            {
                if (j < n)
                {
                    const bool b01 = h1 < h0, b23 = h3 < h2;
                    const u64 m01 = b01 ? h1 : h0, m23 = b23 ? h3 : h2;
                    const bool hi = m23 < m01;
                    id[j]         = (unsigned)(hi ? m23 : m01);
                    const int w   = hi ? (b23 ? 3 : 2) : (b01 ? 1 : 0);  // the list that gave the key
                    if (TRAIN) tagw[j / 4] |= (unsigned)((w << 4) | (w == 0 ? q0 : w == 1 ? q1 : w == 2 ? q2 : q3)) << (8 * (j & 3));
                    q0 += w == 0, q1 += w == 1, q2 += w == 2, q3 += w == 3;
                    if (j + 1 < n)
                    {
                        const int ci   = ci0 + (w & 1) + 9 * (w >> 1);
                        const int4 c   = w == 0 ? c0 : w == 1 ? c1 : w == 2 ? c2 : c3;
                        const int q    = w == 0 ? q0 : w == 1 ? q1 : w == 2 ? q2 : q3;
                        const u64 next = key_of(ci, c, q);
                        h0 = w == 0 ? next : h0, h1 = w == 1 ? next : h1, h2 = w == 2 ? next : h2, h3 = w == 3 ? next : h3;
                    }
                }
            }
        }
    }

    // ---- blend (RenderForward.cu:820-1048), front to back ----
    const int nmax = wave_max_small<16>(n);  // longest list of the block
    TreeSum<C, 5> sum;  // (five levels: up to 16 positions)
    float T       = 1.f;
    float bgw     = 1.f;  // empty list -> 1
    int ret       = 0;    // length of the leading run of kept entries
    bool run_open = true;
    float4 r0[BATCH], rd[BATCH][NQ];
    // one list position, its number a compile-time constant (the arrays indexed by it stay in registers)
    auto position = [&](auto jc)
    {
        constexpr int j = decltype(jc)::value;
        constexpr int b = j % BATCH;
        const bool has  = j < n;
        float a         = 0.f;
        if (has) a = entry_alpha(r0[b], tc.layer, p.num_layers, gx, gy);
        const float Tc  = (T >= kAlphaDestCutoff) ? T : 0.f;
        const bool kept = has && Tc >= kAlphaDestCutoff;
        run_open        = run_open && kept;
        if (run_open) ret = j + 1;
        const float wgt = has ? Tc * a : 0.f;
        float pr[C];
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            const float4 t = rd[b][c / 4];
            const float d  = (c & 3) == 0 ? t.x : (c & 3) == 1 ? t.y : (c & 3) == 2 ? t.z : t.w;
            pr[c]          = has ? wgt * d : 0.f;
        }
        sum.template push<j>(pr);
        // background weight (RenderForward.cu:1002-1022): taken at the last list position
        if (j == n - 1) bgw = (p.background_mode == TRIPS_BG_REFERENCE) ? Tc : T * (1.f - a);
        T = T * (1.f - a);
    };
    // the records of BATCH positions are requested together, then the positions are walked
    auto batch = [&](auto first)
    {
        constexpr int j0 = decltype(first)::value;
#pragma unroll
        for (int b = 0; b < BATCH; ++b)
        {
            r0[b] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int q = 0; q < NQ; ++q) rd[b][q] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (j0 + b < nmax && j0 + b < n)
            {
                const float4* rec = reinterpret_cast<const float4*>(p.rec + (size_t)id[j0 + b] * RF);
                r0[b]             = rec[0];
#pragma unroll
                for (int q = 0; q < NQ; ++q) rd[b][q] = rec[1 + q];
            }
        }
        if (j0 + 0 < nmax) position(std::integral_constant<int, j0 + 0>{});
        if (j0 + 1 < nmax) position(std::integral_constant<int, j0 + 1>{});
        if (j0 + 2 < nmax) position(std::integral_constant<int, j0 + 2>{});
        if (j0 + 3 < nmax) position(std::integral_constant<int, j0 + 3>{});
        if constexpr (BATCH > 4)
        {
            if (j0 + 4 < nmax) position(std::integral_constant<int, j0 + 4>{});
            if (j0 + 5 < nmax) position(std::integral_constant<int, j0 + 5>{});
            if (j0 + 6 < nmax) position(std::integral_constant<int, j0 + 6>{});
            if (j0 + 7 < nmax) position(std::integral_constant<int, j0 + 7>{});
        }
    };
    if (nmax > 0) batch(std::integral_constant<int, 0>{});
    if constexpr (BATCH == 4)
    {
        if (nmax > 4) batch(std::integral_constant<int, 4>{});
        if (nmax > 8) batch(std::integral_constant<int, 8>{});
        if (nmax > 12) batch(std::integral_constant<int, 12>{});
    }
    else if (nmax > 8)
        batch(std::integral_constant<int, 8>{});

    float col[C];
    sum.total(col);
    if (live)
    {
        if (bgw >= kAlphaDestCutoff)
        {
#pragma unroll
            for (int c = 0; c < C; ++c) col[c] += p.background[c] * (bgw * 1.f);
        }
        store_pixel<C>(p, p.image[tc.layer], tc.w, tc.h, gx, gy, col);
    }
    // saved state, also for padding pixels (empty) so that every row of the tables is defined
    if (TRAIN)
    {
        // (bits 0..4: retained entries; bits 5..9: list positions that hold an id. Only those are stored below: the
        // backward reads the retained ones, the export fills the rest of a row with -1 itself. Bits 10..31: length of
        // the pixel's list before the cut to K, for the export; saturates.)
        __builtin_nontemporal_store(live ? (int)((unsigned)ret | ((unsigned)n << kRetainedBits) |
                                                 ((unsigned)min(length, kMaxExportedLength) << (2 * kRetainedBits)))
                                         : 0,
                                    p.retained + pix);
        // four positions at a time, the block's 64 pixels side by side (list_word)
        vi4* const mine = reinterpret_cast<vi4*>(p.lists + list_word((unsigned)pix, 0, p.list_depth));
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (4 * q < nmax && 4 * q < n)
                __builtin_nontemporal_store(vi4{(int)id[4 * q], (int)id[4 * q + 1], (int)id[4 * q + 2], (int)id[4 * q + 3]}, mine + (q << 6));
        if (n > 0) __builtin_nontemporal_store(vu4{tagw[0], tagw[1], tagw[2], tagw[3]}, reinterpret_cast<vu4*>(p.tags) + (unsigned)pix);
        // the view's retained entries, for the backward's choice of how it keeps its pair rows: estimated from every
        // kRetainedSample-th workgroup, one atomic per wavefront (the sum of 64 values of at most 16, a ballot per bit),
        // spread over kRetainedParts counters
        unsigned wave_ret = 0;
        if (blockIdx.x % (unsigned)kRetainedSample == 0)
        {
#pragma unroll
            for (int b = 0; b < 5; ++b) wave_ret += (unsigned)__popcll(__ballot(live && ((ret >> b) & 1))) << b;
        }
        if (lane == 0 && wave_ret)
            atomicAdd(p.saved_chunk_valid + p.bin_groups + (int)((blockIdx.x / (unsigned)kRetainedSample * 4u + (unsigned)wave) % (unsigned)kRetainedParts), (int)wave_ret);
    }
}

// ---------------------------------------------------------------------------------------------------------
// host-side launchers
#define TRIPS_DISPATCH_C(C_, ...)             \
    switch (C_)                               \
    {                                         \
        case 3: { constexpr int CC = 3; __VA_ARGS__; break; }   \
        case 4: { constexpr int CC = 4; __VA_ARGS__; break; }   \
        case 6: { constexpr int CC = 6; __VA_ARGS__; break; }   \
        case 8: { constexpr int CC = 8; __VA_ARGS__; break; }   \
        case 16: { constexpr int CC = 16; __VA_ARGS__; break; } \
        default: return hipErrorInvalidValue; \
    }

hipError_t launch_forward_view(const ForwardParams& p, int channels, bool train, bool first_view, hipStream_t stream,
                               Profiler* prof)
{
    const int NB = p.geom.bin_off[p.num_layers];

    const int G           = p.bin_groups;
    const size_t lds_hist = (size_t)NB * sizeof(int);
    // compact point numbers are below num_points: entries of 8 bytes when they fit kPackedIdBits bits
    const bool packed = p.num_points <= (1 << kPackedIdBits);
    {
        ProfScope ps(prof, "project_bin", stream);
        if (train)
        {
            TRIPS_DISPATCH_C(channels, hipLaunchKernelGGL((project_bin_kernel<CC, true>), dim3(G), dim3(kBinThreads), lds_hist, stream, p));
        }
        else
        {
            TRIPS_DISPATCH_C(channels, hipLaunchKernelGGL((project_bin_kernel<CC, false>), dim3(G), dim3(kBinThreads), lds_hist, stream, p));
        }
    }
    {
        ProfScope ps(prof, "bin_scan", stream);
        hipLaunchKernelGGL(bin_column_scan_kernel, dim3((NB + kScanCols - 1) / kScanCols), dim3(256), 0, stream, p.bin_hist, p.bin_count, NB, G);
        // counts and run are neighbours in the workspace: cleared together, by the workgroups behind the scanning one
        const long long quads = 2ll * NB * kTilePixels / 4;
        hipLaunchKernelGGL(scan_plan_kernel, dim3(1 + (unsigned)std::min<long long>((quads + 1023) / 1024, 1024)), dim3(1024), 0, stream,
                           p.bin_count, p.bin_start, p.slice_start, NB, p.capacity, p.chunk_valid, G, p.header, p.status, first_view ? 1 : 0,
                           p.long_count, reinterpret_cast<uint4*>(p.counts), quads, p.saved_chunk_valid);
    }
    {
        ProfScope ps(prof, "bin_scatter", stream);
        if (packed)
            hipLaunchKernelGGL(bin_scatter_kernel<true>, dim3(G), dim3(kBinThreads), lds_hist, stream, p);
        else
            hipLaunchKernelGGL(bin_scatter_kernel<false>, dim3(G), dim3(kBinThreads), lds_hist, stream, p);
    }
    // workgroups for the slices of split tiles: at most capacity / kSliceEntries full slices plus one partial slice
    // per split tile
    const int max_slices = (int)std::min<long long>(2 * (p.capacity / kSliceEntries) + 1, 1 << 20);
    {
        ProfScope ps(prof, "tile_count", stream);
        if (packed)
            hipLaunchKernelGGL((tile_lists_kernel<false, 256, true>), dim3(NB + max_slices), dim3(256), 0, stream, p);
        else
            hipLaunchKernelGGL((tile_lists_kernel<false, 256, false>), dim3(NB + max_slices), dim3(256), 0, stream, p);
    }
    {
        ProfScope ps(prof, "tile_scatter", stream);
        // (64 KB of LDS with the static tables: above the default limit of a launch)
        const void* fn = packed ? reinterpret_cast<const void*>(&tile_lists_kernel<true, kScatterThreads, true>)
                                : reinterpret_cast<const void*>(&tile_lists_kernel<true, kScatterThreads, false>);
        const hipError_t lds = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(kStageKeys * sizeof(u64)));
        if (lds != hipSuccess) return lds;
        if (packed)
            hipLaunchKernelGGL((tile_lists_kernel<true, kScatterThreads, true>), dim3(NB + max_slices), dim3(kScatterThreads),
                               kStageKeys * sizeof(u64), stream, p);
        else
            hipLaunchKernelGGL((tile_lists_kernel<true, kScatterThreads, false>), dim3(NB + max_slices), dim3(kScatterThreads),
                               kStageKeys * sizeof(u64), stream, p);
    }
    {
        ProfScope ps(prof, "long_lists", stream);
        const int blocks = std::min((p.max_long_items + 15) / 16, 2048);
        hipLaunchKernelGGL(long_list_reduce_kernel, dim3(blocks), dim3(256), 0, stream, p);
    }
    const long long tiles8 = (((long long)NB + kNumXcd - 1) / kNumXcd) * kNumXcd;  // tiles rounded up to 8
    const int quarter_tiles = (int)(tiles8 * 4);                                   // a quarter tile per workgroup
    {
        ProfScope ps(prof, "cell_sort", stream);
        hipLaunchKernelGGL(cell_sort_kernel, dim3((unsigned)(tiles8 * 16)), dim3(256), 0, stream, p);  // 64 cells per workgroup
    }
    {
        ProfScope ps(prof, "blend", stream);
        if (train)
        {
            TRIPS_DISPATCH_C(channels, hipLaunchKernelGGL((blend_kernel<CC, true>), dim3(quarter_tiles), dim3(256), 0, stream, p));
        }
        else
        {
            TRIPS_DISPATCH_C(channels, hipLaunchKernelGGL((blend_kernel<CC, false>), dim3(quarter_tiles), dim3(256), 0, stream, p));
        }
    }
    return hipGetLastError();
}

}  // namespace trips
