// Internal structures shared by the host-side C ABI and the HIP kernels of the splat path.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/trips_splat.h"

#include <vector>

namespace trips
{
// Optional HIP-event bracket around every kernel launch (host side only).
struct Profiler
{
    struct Span
    {
        const char* name;
        hipEvent_t a, b;
    };
    bool enabled = false;
    std::vector<Span> spans;
    std::vector<hipEvent_t> pool;

    hipEvent_t get_event()
    {
        if (!pool.empty())
        {
            hipEvent_t e = pool.back();
            pool.pop_back();
            return e;
        }
        hipEvent_t e = nullptr;
        if (hipEventCreate(&e) != hipSuccess) return nullptr;
        return e;
    }
    void begin(const char* name, hipStream_t s)
    {
        if (!enabled) return;
        Span sp{name, get_event(), get_event()};
        if (!sp.a || !sp.b) return;
        (void)hipEventRecord(sp.a, s);
        spans.push_back(sp);
    }
    void end(hipStream_t s)
    {
        if (!enabled || spans.empty()) return;
        (void)hipEventRecord(spans.back().b, s);
    }
    ~Profiler()
    {
        for (auto& sp : spans)
        {
            (void)hipEventDestroy(sp.a);
            (void)hipEventDestroy(sp.b);
        }
        for (auto e : pool) (void)hipEventDestroy(e);
    }
};

struct ProfScope
{
    Profiler* p;
    hipStream_t s;
    ProfScope(Profiler* p_, const char* name, hipStream_t s_) : p(p_), s(s_)
    {
        if (p) p->begin(name, s);
    }
    ~ProfScope()
    {
        if (p) p->end(s);
    }
};

// records the message trips_last_error_string() returns on this thread; returns `code`
int set_error(int code, const char* fmt, ...);

}  // namespace trips

// The opaque context of the C ABI.
struct TripsCtx
{
    int device;
    trips::Profiler prof;
    // this device's copy of the library's static scratch array (trips_splat_forward_static), resolved when the
    // context is created
    void* static_scratch = nullptr;
    int pair_rows_mode = 0;  // trips_splat_pair_rows_mode: 0 = the backward chooses per view
};

namespace trips
{
// Per-point records written by the projection kernel, for the VALID points of a view only, at the point's compact
// number cid (see chunk_point_range: dense runs in point order; cid_of / pid_of translate). The 64-bit sort key of a
// list entry is depth bits << 32 | cid: cid grows with the point id, so the order is that of depth bits << 32 |
// point id.
//   rec[cid]   4 + Cpad floats {ip.x, ip.y, size field (see encode_size_field), confidence, descriptor[0..C)}:
//              everything the blend and the pixel pass of the backward need in one aligned gather of 32 bytes at
//              C = 4 (the reference reads a 5-float record, the confidence and C descriptor planes,
//              src/lib/rendering/RenderForward.cu:875-899,952). Kept apart from the rest because a scattered gather
//              costs the bytes of the whole aligned block it touches.
//   prec[cid]  4 floats {softplus'(raw size), depth, layers written, size_px}: read by the kernel that makes the bin
//              entries and, in point order, by the point pass of the backward, which transforms the point into view
//              space again rather than have the projection kernel write those 12 bytes per point as well.
__host__ __device__ inline int record_floats(int channels) { return 4 + ((channels + 3) & ~3); }
constexpr int kPointRecordFloats = 4;

// Pixels are binned into 32 x 32 tiles per layer. Internally a pixel is numbered tile-major:
// (bin << 10) | (y & 31) << 5 | (x & 31), bin = bin_off[layer] + tile_y * tiles_x[layer] + tile_x, so that a
// tile's 1024 counters, list offsets and saved lists are contiguous (partial tiles are padded with empty pixels).
// The exports of the C ABI translate back to the row-major numbering (off[]).
constexpr int kTileShift  = 5;
constexpr int kTile       = 1 << kTileShift;
constexpr int kTilePixels = kTile * kTile;
// (One workgroup of 1024 threads per CU: three of 512, with the projection kernel held to 80 registers, measured 1 %
// slower over the step: the histogram matrix grows with the number of workgroups.)
constexpr int kPackedIdBits = 23;  // clouds of up to 2^23 points have bin entries of 8 bytes (31 depth bits, id, 10 cell bits)
// a pixel's word of the saved state: retained entries | list positions that hold an id << 5 | list length << 10
constexpr int kRetainedBits = 5, kRetainedMask = (1 << kRetainedBits) - 1;
constexpr int kMaxExportedLength = (1 << (32 - 2 * kRetainedBits)) - 1;  // longer lists are exported as this length
constexpr int kBinThreads = 1024;   // workgroup size of the two binning kernels
constexpr int kBinGroups  = 256;    // workgroups (= contiguous chunks of points) of the two binning kernels
constexpr int kMaxBins    = 15360;  // one LDS counter per tile in the binning kernels (60 KB)
// bin entries of a tile above which the tile is split into slices of that many entries, one workgroup each
constexpr int kSliceEntries = 8192;
// A pixel list longer than kLongList keys is cut into segments of kLongSegment keys; a pass of its own keeps the 16
// smallest keys of every segment (a 16-lane row each), and the blend kernel then sorts those instead of the list.
constexpr int kLongList    = 512;
constexpr int kLongSegment = 256;
constexpr int kStageKeys  = 7168;   // keys of one tile staged in LDS before they are written (56 KB)
// keys of a cell that can reach a pixel's list (the larger list depth): the forward sorts every cell's list and keeps
// this many
constexpr int kCellKeep = 16;

struct PyramidGeom
{
    int32_t num_layers;
    int32_t w[TRIPS_MAX_LAYERS];
    int32_t h[TRIPS_MAX_LAYERS];
    int32_t off[TRIPS_MAX_LAYERS + 1];  // row-major numbering: first pixel of each layer; off[L] = P
    int32_t tiles_x[TRIPS_MAX_LAYERS];
    int32_t tiles_y[TRIPS_MAX_LAYERS];
    int32_t bin_off[TRIPS_MAX_LAYERS + 1];  // first bin of each layer; bin_off[L] = number of bins
    // ceil(2^30 / tiles_x): (4 t * magic) >> 32 == t / tiles_x for t and tiles_x below 2^14 (kMaxBins is)
    uint32_t tiles_x_magic[TRIPS_MAX_LAYERS];
};

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2. Kernels that walk pixels remap their
// workgroup number so that all workgroups of one 32 x 32 tile run on the same XCD (the records a tile's pixels
// share are then fetched once per tile instead of once per workgroup), while consecutive tiles go to different
// XCDs (layers differ a lot in list length, so a contiguous range per XCD would be unbalanced).
// `per_tile` = workgroups per tile; the result may be >= the number of real workgroups (no work then).
constexpr int kNumXcd = 8;
__device__ inline long long xcd_tile_block(long long block, int per_tile)
{
    const long long xcd = block % kNumXcd, k = block / kNumXcd;
    const long long tile = (k / per_tile) * kNumXcd + xcd;
    return tile * per_tile + k % per_tile;
}

__host__ __device__ inline int pix_index(const PyramidGeom& g, int layer, int x, int y)
{
    const int bin = g.bin_off[layer] + (y >> kTileShift) * g.tiles_x[layer] + (x >> kTileShift);
    return (bin << (2 * kTileShift)) | ((y & (kTile - 1)) << kTileShift) | (x & (kTile - 1));
}

// The same on the device: tile counts and pixel coordinates are far below 2^24, so the full-rate 24-bit multiply is
// exact.
__device__ inline int pix_index_mul24(const PyramidGeom& g, int layer, int x, int y)
{
    const int bin = g.bin_off[layer] + (int)__umul24((unsigned)(y >> kTileShift), (unsigned)g.tiles_x[layer]) + (x >> kTileShift);
    return (bin << (2 * kTileShift)) | ((y & (kTile - 1)) << kTileShift) | (x & (kTile - 1));
}

// The saved lists are stored by 8 x 8 blocks of pixels, four list positions at a time: the 64 pixels of a block (one
// wavefront of the blend) keep positions 4q .. 4q + 3 of their lists in 64 consecutive 16-byte words, so that the
// wavefront writes them as one kilobyte and the eight pixels of a row of the block share a line. Word of (pixel pix,
// position j) of lists of depth K:
__host__ __device__ inline size_t list_word(unsigned pix, int j, int K)
{
    const unsigned x = pix & (kTile - 1), y = (pix >> kTileShift) & (kTile - 1), bin = pix >> (2 * kTileShift);
    const unsigned block = (bin << 4) | ((y >> 3) << 2) | (x >> 3), lane = ((y & 7) << 3) | (x & 7);
    return ((((size_t)block * (unsigned)(K >> 2) + (unsigned)(j >> 2)) << 6) + lane) * 4 + (unsigned)(j & 3);
}

// What the pixels of one 32 x 32 tile share: its layer, that layer's size and the tile's first pixel.
struct TileCtx
{
    int layer, w, h, x0, y0;
    int bin, tiles_x;  // the tile's number and the tile columns of its layer
};

// `bin` must be the same for the whole wavefront and come out of a scalar register (readfirstlane): the layer search
// and the division by the layer's tile columns (a multiply by tiles_x_magic) then run on the scalar unit, once per
// wavefront, instead of per lane with an integer division.
__device__ __forceinline__ TileCtx tile_ctx(const PyramidGeom& g, int bin)
{
    int layer = 0, first = 0, tsx = g.tiles_x[0], w = g.w[0], h = g.h[0];
    unsigned magic = g.tiles_x_magic[0];
#pragma unroll
    for (int l = 1; l < TRIPS_MAX_LAYERS; ++l)
    {
        if (l < g.num_layers && bin >= g.bin_off[l])
        {
            layer = l;
            first = g.bin_off[l];
            tsx   = g.tiles_x[l];
            magic = g.tiles_x_magic[l];
            w     = g.w[l];
            h     = g.h[l];
        }
    }
    const unsigned t  = (unsigned)(bin - first);
    const unsigned ty = __umulhi(4u * t, magic);
    const unsigned tx = t - ty * (unsigned)tsx;
    TileCtx c;
    c.layer = layer;
    c.w     = w;
    c.h     = h;
    c.x0    = (int)(tx << kTileShift);
    c.y0    = (int)(ty << kTileShift);
    c.bin     = bin;
    c.tiles_x = tsx;
    return c;
}

// Header at the start of each view's saved state (and of the workspace status block).
struct ViewHeader
{
    unsigned long long n_valid;     // points that passed the validity test
    unsigned long long n_entries;   // (point, layer) pairs filed (from the scan); each is in four pixel lists: E = 4 x
    unsigned long long overflow;    // entries dropped because the list storage was too small
    unsigned long long retained;    // R: sum of the retained entries (filled by the counters query)
    unsigned long long not_identity;  // some point's descriptor column differs from its own index
    unsigned long long bad_index;   // some point's descriptor column lies outside [0, num_texels): the point was skipped
    // valid points whose finest-layer tile is also that of the point before them in memory: near n_valid for a cloud
    // stored along a space-filling curve, near zero for one in random order (the backward chooses its exchange layout
    // by it)
    unsigned long long same_tile_as_previous;
    // rows of the backward's overflow table that the view's points own: sum over the valid points of max(layers - 2, 0)
    unsigned long long overflow_rows;
};

// Most (point, layer) pairs of a usual view are retained by some pixel, and the backward then clears and reads the rows
// of all pairs. In a view whose lists are mostly hidden behind their first entries only a few pairs are: the backward
// then keeps a flag byte per row instead, clears only those, and its point pass reads only the rows whose flag the tile
// pass has set. The blend kernel adds the view's retained entries up in kRetainedParts counters (one atomic per
// wavefront; on a single counter they would queue up for longer than the kernel runs), the backward's first kernel
// sums them and leaves the choice in the workspace for the two passes.
constexpr int kRetainedParts = 256;
// (An estimate is enough for that choice, both ways of keeping the rows give the same gradients: every
// kRetainedSample-th workgroup of the blend kernel contributes.)
constexpr int kRetainedSample = 16;
__host__ __device__ inline bool sparse_pair_rows(unsigned long long retained, unsigned long long pairs) { return 4ull * retained < pairs; }

// Layout of one view's saved state (all offsets in bytes, 256-aligned)
struct SavedLayout
{
    size_t header;    // ViewHeader
    size_t rec;       // float [N * record_floats]
    size_t prec;      // float [N * kPointRecordFloats]
    size_t lists;     // int32 [Pi / 64, K / 4, 64, 4] (see list_word)  Pi = number of bins * 1024 (tile-major, padded); a pixel's positions past its ids are undefined
    size_t retained;  // int32 [Pi]: retained entries in bits 0..4, list positions that hold an id (min(length, K)) in bits 5..9, list length from bit 10
    size_t tags;      // uint8 [Pi, 16]  where a list position came from: which of the pixel's four cells (bits 4..5) and its
                      // place in that cell's sorted list (bits 0..3); a row's positions past its ids are undefined
    size_t cid_of;    // int32 [N] compact number of every point (-1 = culled)
    size_t pid_of;    // int32 [N] point of every compact number (the first n_valid are defined)
    size_t over_first;  // int32 [N] by compact number: for a point written to more than two layers, the number of its
                        // first row in the backward's overflow table (rows numbered densely in point order)
    size_t chunk_valid;  // int32 [kBinGroups] valid points of every chunk of the binning kernels (their compact numbers
                         // start at the chunk's first point number), then [kRetainedParts] partial sums of the view's
                         // retained entries
    size_t bytes_per_view;
};

// The backward sums, per (point, layer) pair, what the four pixels of the footprint contribute before the projection
// chain: the descriptor gradient sum_corners T alpha dL/dimage (Cpad floats) and dL/dalpha of each corner (4 floats).
// The rows of a point's first two layers sit at its compact number (most points are written to one or two layers: the
// tile pass then needs no look-up to place a row), those of further layers in an overflow table.
__host__ __device__ constexpr int pair_row_floats(int cpad) { return cpad + 4; }
constexpr int kInlineLayers = 2;

struct BackwardWorkspaceLayout
{
    size_t rows_inline;  // float [N, kInlineLayers, pair_row_floats] by compact number
    size_t rows_over;    // float [over_capacity, pair_row_floats]
    size_t flags;         // uint8 [N, TRIPS_MAX_LAYERS] by compact number: 1 where the tile pass wrote the pair's row
                          // (only for views in which few pairs are retained)
    size_t mode;          // int32: 1 = only flagged rows exist (written by the prologue kernel)
    size_t over_capacity;
    size_t bytes;
};

struct WorkspaceLayout
{
    size_t chunk_valid;   // int32 [5 G]  per chunk of the binning kernels: valid points, flags, (unused), overflow rows of the
                          //              backward, and (from the scan) the number of the chunk's first overflow row
    size_t prec;         // float4 [N]         point records, when there is no saved state to hold them
    size_t counts;       // int32 [Pi]   list length per cell (the points whose 2 x 2 footprint starts at that pixel)
    size_t cursor;       // int32 [Pi]   first key of each cell's list (-1 - first candidate row for a long list)
    size_t run;          // int32 [Pi]   keys of a cell already claimed by slices of a split tile (zeroed per view)
    size_t slice_start;  // int32 [NB+1] exclusive scan of the slices of split tiles (0 for a tile that is not split)
    size_t long_count;   // int32 [1]    segments of long lists handed out so far
    size_t long_items;   // int2  [max_long_items] {first key, number of keys} of each segment of a long list
    size_t cand;         // uint64 [max_long_items * 16] the 16 smallest keys of each segment
    size_t max_long_items;
    size_t bin_count;    // int32 [NB]   bin entries per tile
    size_t bin_start;    // int32 [NB+1] exclusive scan of bin_count
    size_t bin_hist;     // int32 [G, NB] bin entries per (workgroup, tile), then its column-wise exclusive prefix
    size_t bin_entries;  // [capacity] {depth bits, compact point number, cell}, one per (point, layer), by tile: 8 bytes each for up to 2^23 points, else 16
    size_t keys;         // uint64 [capacity] depth bits << 32 | compact point number, by cell
    size_t capacity;     // (point, layer) pairs
    size_t bytes;
};

inline size_t align256(size_t x) { return (x + 255) & ~size_t(255); }

struct ForwardParams
{
    // scene
    const float4* position;
    const float* point_size;
    const int32_t* index;
    const float* texture;
    const float* confidence;
    const float* background;
    const double* pose;      // 8 doubles of this view's image
    const float* intrinsics; // 13 floats of this view's camera
    const float* dropout;    // this view's row or nullptr
    const float* displacement;  // this view's [N,3] or nullptr
    // geometry
    PyramidGeom geom;
    TripsView view;
    int32_t num_points, num_texels, num_layers, list_depth;
    int32_t view_index, num_views;
    int32_t layout, background_mode;
    int32_t drop_out_points_by_radius, viewer_only;
    float drop_out_radius_threshold, dist_cutoff, stability_cutoff_value;
    // buffers
    int32_t* chunk_valid;
    int32_t* cid_of;  // training only: compact number of every point, -1 = culled
    int32_t* pid_of;  // training only: point of every compact number
    int32_t* counts;
    int32_t* cursor;
    int32_t* bin_count;
    int32_t* bin_start;
    int32_t* bin_hist;
    int32_t bin_groups, points_per_block;
    int32_t* run;
    int32_t* slice_start;
    int32_t* long_count;
    int2* long_items;
    unsigned long long* cand;
    int32_t max_long_items;
    void* bin_entries;
    unsigned long long* keys;
    long long capacity;
    float* rec;
    float* prec;
    int32_t rec_floats;
    int32_t* lists;
    int32_t* retained;
    unsigned char* tags;  // training only
    int32_t* over_first;  // training only
    int32_t* saved_chunk_valid;  // training only: [kBinGroups + kRetainedParts]
    ViewHeader* header;  // counters of this view
    ViewHeader* status;  // overflow flag of the whole forward call (start of the workspace)
    float* image[TRIPS_MAX_LAYERS];
};

struct BackwardParams
{
    const float* background;
    const double* pose;
    const float* intrinsics;
    const float* point_size;
    const float4* position;     // as the forward saw them
    const float* displacement;  // this view's [N,3] or nullptr
    const int32_t* index;
    PyramidGeom geom;
    TripsView view;
    int32_t num_points, num_texels, num_layers, list_depth;
    int32_t view_index, num_views, layout;
    float dist_cutoff;
    const float* rec;
    const float* prec;
    int32_t rec_floats;
    const int32_t* lists;
    const int32_t* retained;
    const int32_t* cid_of;
    const ViewHeader* header;
    const float* grad_image[TRIPS_MAX_LAYERS];
    const unsigned char* tags;  // [Pi, 16] (saved state) cell and place in the cell's list of every list position
    const int32_t* over_first;   // [N] (saved state) by compact number
    const int32_t* chunk_valid;  // [kBinGroups + kRetainedParts] (saved state)
    int32_t* mode;               // (workspace) 1 = only flagged rows exist
    int32_t force_mode;          // 0 = chosen per view from the retained entries, 1 = rows of all pairs, 2 = flagged rows
    int32_t bin_groups, points_per_block;
    float* rows_inline;  // [N, kInlineLayers, pair_row_floats] (workspace)
    float* rows_over;    // [over_capacity, pair_row_floats] (workspace)
    unsigned char* flags;  // [N, TRIPS_MAX_LAYERS] (workspace) by compact number
    // blocks of the tile pass (16 x 16 pixels, 15 apart): first block of each layer, blocks per block row of each layer
    int32_t blocks_off[TRIPS_MAX_LAYERS + 1];
    int32_t blocks_x[TRIPS_MAX_LAYERS];
    long long over_capacity;
    float* d_texture;
    float* d_confidence;
    float* d_background;
    float* d_position;
    float* d_point_size;
    double* d_pose;       // row of this view's image or nullptr
    float* d_intrinsics;  // row of this view's camera or nullptr
    int32_t overwrite;    // the per-point outputs are written, not added to (first view of a call in that mode)
    // first view of a call that clears the block sums itself: all of d_background, d_pose and d_intrinsics
    int32_t clear_block_sums;
    double* d_pose_all;       // [num_images][6] or nullptr
    float* d_intrinsics_all;  // [num_cameras][13] or nullptr
    int32_t num_images, num_cameras;
};

}  // namespace trips
