// Backward kernels of the splat path for gfx950 (wave64).
//
//   backward_tiles_kernel + backward_points_kernel <- BlendBackwardsBilinearTiled
//                                                     src/lib/rendering/RenderBackward.cu:90-618
//
// The reference walks one pixel list per thread and scatters every entry's gradient with float atomics
// (3 position + 1 size + 1 confidence + C descriptor atomics per retained entry). Scattered atomics run at about
// 2e10 per second on this GPU, and what bounds the kernels of this path is the number of scattered memory requests,
// whatever their size. So the four pixels of a point's footprint meet in LDS, not in memory:
//   1. tiles: a workgroup walks a block of 16 x 16 pixels, one pixel per lane, and owns the 15 x 15 cells whose four
//      pixels lie inside it (a cell = the footprints that start at that pixel); blocks overlap by one row and one
//      column, which the neighbours walk again. A lane recomputes alpha and transmittance of its pixel's retained
//      entries from the per-point record exactly as the forward computed them, forms dL/dalpha (the "all later
//      entries" sum of RenderBackward.cu:284-301 is a running sum from the back of the list) and leaves
//      {dL/dalpha, T alpha} of every entry in LDS, together with the entry's list position under the (cell, place in
//      the cell's list, corner) that the forward noted for it. After a barrier every (point, layer) pair is formed
//      once, by the wavefront of the first of its corner pixels that retained it: the pairs are queued and dealt to
//      the lanes, a lane collects the four corner pixels' entries and writes ONE row per pair: sum over the corners of
//      T alpha dL/dimage and the four dL/dalpha. The rows of a point's first two layers sit at its compact number,
//      further layers in an overflow table.
//   2. points: the (point, layer) pairs of 64 consecutive points are dealt out to the lanes; a lane reads its pair's
//      row, evaluates the bilinear weights' Jacobian and the layer factor per corner (PointBlending.h:216-264,
//      RenderBackward.cu:366-438); the point's own lane sums the image-space gradient of all its entries and runs the
//      projection chain ONCE (the chain is linear in the image-space gradient, RenderBackward.cu:385-417), then stores
//      or adds its gradients. Pose / intrinsics partials stay in registers over a grid-stride loop before one
//      block-level reduction and one atomic per value and block (the reference keeps them in shared double arrays,
//      :160-187,546-617).
// A prologue kernel clears the rows (or, for a view in which few pairs are retained, one flag byte per row) beforehand.
// The per-point gradients are summed in a fixed order and are bit-reproducible from run to run; the few block sums
// (background, pose, intrinsics) are added with one atomic per workgroup, in an order that varies.
#include "row16.h"
#include "splat_internal.h"
#include "trips_math.h"

#include <type_traits>

#pragma clang fp contract(off)

namespace trips
{
__device__ __forceinline__ Camera load_camera_bw(const double* pose, const float* intr, const TripsView& v,
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

typedef float vf4 __attribute__((ext_vector_type(4)));
typedef int vi4 __attribute__((ext_vector_type(4)));
typedef unsigned vu4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ double wave_sum(double v)
{
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
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

// ---------------------------------------------------------------------------------------------------------
// Pass 1: per block of 16 x 16 cells.
constexpr int kBlockSide   = 16;                       // pixels per side of a workgroup's block: one pixel per lane
constexpr int kBlockCells  = kBlockSide - 1;           // cells per side whose footprints lie inside those pixels
constexpr int kBlockPixels = kBlockSide * kBlockSide;  // 256
constexpr int kListMax     = 16;                       // entries of a pixel's list (the larger list depth)

// LDS of a block: {dL/dalpha, T alpha} per (list position, pixel); dL/dimage per (channel, pixel); per (place in the
// cell's sorted list, cell) the list positions of that point's entry in its four corner pixels (0xFF: none). The pixel or the cell is the fastest index everywhere: neighbouring lanes, neighbouring banks.
__host__ __device__ constexpr size_t tiles_lds_bytes(int cpad)
{
    return (size_t)kBlockPixels * kListMax * 8 + (size_t)kBlockPixels * cpad * 4 + (size_t)kBlockCells * kBlockCells * kCellKeep * 4;
}

template <int C>
__global__ __launch_bounds__(256) void backward_tiles_kernel(const BackwardParams p)
{
    constexpr int CPAD  = (C + 3) & ~3;
    constexpr int RF    = 4 + CPAD;  // floats per blend record
    constexpr int NQ    = CPAD / 4;
    constexpr int PRF   = pair_row_floats(CPAD);
    // list positions whose records are requested together (the LDS of a block bounds the wavefronts per SIMD before the
    // registers do)
    constexpr int BATCH = CPAD <= 4 ? 8 : 4;
    extern __shared__ __align__(16) unsigned char s_mem[];
    float2* const s_ex     = reinterpret_cast<float2*>(s_mem);
    float* const s_g       = reinterpret_cast<float*>(s_mem + (size_t)kBlockPixels * kListMax * 8);
    unsigned* const s_rank = reinterpret_cast<unsigned*>(s_mem + (size_t)kBlockPixels * kListMax * 8 + (size_t)kBlockPixels * CPAD * 4);
    __shared__ double s_acc[4][C];
    // (point, layer) pairs that wait for a lane of their wavefront: slot = place * 225 + cell, and the point's compact
    // number. The queue is emptied down to fewer than kQueueSlack pairs before a list position adds up to 64.
    constexpr int kQueueSlack = 32, kQueue = kQueueSlack + 64;
    __shared__ unsigned short s_qslot[4][kQueue];
    __shared__ int s_qcid[4][kQueue];

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // Blocks of 16 x 16 pixels that overlap by one row and one column (so that every cell's four pixels lie in one
    // block): block (i, j) of a layer starts at pixel (15 i, 15 j). Runs of eight blocks of a block row share an XCD.
    const long long lblock = xcd_tile_block(blockIdx.x, 8);
    if (lblock >= p.blocks_off[p.num_layers]) return;
    int layer = 0;
#pragma unroll
    for (int l = 1; l < TRIPS_MAX_LAYERS; ++l)
        if (l < p.num_layers && lblock >= p.blocks_off[l]) layer = l;
    const int in_layer = (int)lblock - p.blocks_off[layer];
    const int byi = in_layer / p.blocks_x[layer], bxi = in_layer - byi * p.blocks_x[layer];
    const int lw = p.geom.w[layer], lh = p.geom.h[layer];
    const int x0 = bxi * kBlockCells, y0 = byi * kBlockCells;  // the block's first pixel
    const float* const gi = p.grad_image[layer];

    float acc_bg[C];  // a lane sees a few pixels: its own sums stay in single precision, everything across lanes is double
#pragma unroll
    for (int c = 0; c < C; ++c) acc_bg[c] = 0.f;

    // ---- the block's pixels, one per lane, a wavefront taking 8 x 8 of them (the four pixels of a footprint then
    // mostly sit in one wavefront and share their gathers) ----
    {
        const int px = ((wave & 1) << 3) + (lane & 7), py = ((wave >> 1) << 3) + (lane >> 3);
        const int t  = py * kBlockSide + px;
        const int gx = x0 + px, gy = y0 + py;
        const bool inside = gx < lw && gy < lh;
        // (the last row and column are the first of the neighbours' blocks)
        const bool owned   = inside && px < kBlockCells && py < kBlockCells;
        const unsigned pix = inside ? (unsigned)pix_index_mul24(p.geom, layer, gx, gy) : 0u;
        // the pixel's retained count, its list (compact numbers and where each entry came from) and dL/dimage are all
        // requested before the first is looked at; list positions past the retained ones hold anything and are not used
        int word = 0;
        int id[kListMax];
        const vi4* mine = nullptr;  // the pixel's list: positions 4q .. 4q + 3 at mine[64 q]
        unsigned tagw[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < kListMax; ++j) id[j] = 0;
        if (inside)
        {
            word = p.retained[pix];
            mine = reinterpret_cast<const vi4*>(p.lists + list_word(pix, 0, p.list_depth));
            {
                const vi4 v = __builtin_nontemporal_load(mine);
                id[0] = v.x, id[1] = v.y, id[2] = v.z, id[3] = v.w;
            }
            const vu4 v = __builtin_nontemporal_load(reinterpret_cast<const vu4*>(p.tags) + pix);
            tagw[0] = v.x, tagw[1] = v.y, tagw[2] = v.z, tagw[3] = v.w;
        }

        float g[C];
#pragma unroll
        for (int c = 0; c < C; ++c) g[c] = 0.f;
        if (inside)
        {
            // offsets inside one view's image stay far below 2^32 (the pyramid has at most kMaxBins tiles)
            if (p.layout == TRIPS_LAYOUT_CHW)
            {
                const size_t plane = (size_t)lw * lh;
                const float* o     = gi + ((size_t)p.view_index * C) * plane;
                const unsigned at  = __umul24((unsigned)gy, (unsigned)lw) + (unsigned)gx;
#pragma unroll
                for (int c = 0; c < C; ++c) g[c] = (o + c * plane)[at];
            }
            else
            {
                const float* o    = gi + ((size_t)p.view_index * lh * lw) * C;
                const unsigned at = (__umul24((unsigned)gy, (unsigned)lw) + (unsigned)gx) * C;
#pragma unroll
                for (int c = 0; c < C; ++c) g[c] = o[at + c];
            }
        }
        // no entry yet under any (cell, place): cleared while the loads above travel
        for (int i = threadIdx.x; i < kBlockCells * kBlockCells * kCellKeep / 4; i += 256)
            reinterpret_cast<uint4*>(s_rank)[i] = make_uint4(~0u, ~0u, ~0u, ~0u);
        __syncthreads();
        const int m    = word & kRetainedMask;
        const int mmax = wave_max_small<kListMax>(m);
        // (two thirds of the pixels of a typical view retain at most four entries: the rest of a list only where needed)
#pragma unroll
        for (int q = 1; q < 4; ++q)
        {
            if (4 * q < mmax && 4 * q < m)
            {
                const vi4 v = __builtin_nontemporal_load(mine + (q << 6));
                id[4 * q] = v.x, id[4 * q + 1] = v.y, id[4 * q + 2] = v.z, id[4 * q + 3] = v.w;
            }
        }
#pragma unroll
        for (int c = 0; c < CPAD; ++c) s_g[c * kBlockPixels + t] = c < C ? g[c] : 0.f;
        float sbg = 0.f;
#pragma unroll
        for (int c = 0; c < C; ++c) sbg += p.background[c] * g[c];

        // front to back: alpha, transmittance (the forward's chain), descriptor . dL/dimage
        float A[kListMax], Tr[kListMax], S[kListMax];
#pragma unroll
        for (int j = 0; j < kListMax; ++j) A[j] = 0.f, Tr[j] = 0.f, S[j] = 0.f;
        float T = 1.f;
        float4 r0[BATCH], rd[BATCH][NQ];
        auto position = [&](auto jc)
        {
            constexpr int j = decltype(jc)::value;
            constexpr int b = j % BATCH;
            const bool has  = j < m;
            float a         = 0.f;
            if (has) a = entry_alpha(r0[b], layer, p.num_layers, gx, gy);
            float s = 0.f;
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                const float4 t4 = rd[b][c / 4];
                const float d   = (c & 3) == 0 ? t4.x : (c & 3) == 1 ? t4.y : (c & 3) == 2 ? t4.z : t4.w;
                s += d * g[c];
            }
            A[j]  = a;
            Tr[j] = T;
            S[j]  = has ? s : 0.f;
            T     = T * (1.f - a);
        };
        auto batch = [&](auto first)
        {
            constexpr int j0 = decltype(first)::value;
#pragma unroll
            for (int b = 0; b < BATCH; ++b)
            {
                r0[b] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int q = 0; q < NQ; ++q) rd[b][q] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (j0 + b < mmax && j0 + b < m)
                {
                    const float4* rec = reinterpret_cast<const float4*>(p.rec + (size_t)(unsigned)id[j0 + b] * RF);
                    r0[b]             = rec[0];
#pragma unroll
                    for (int q = 0; q < NQ; ++q) rd[b][q] = rec[1 + q];
                }
            }
            if (j0 + 0 < mmax) position(std::integral_constant<int, j0 + 0>{});
            if (j0 + 1 < mmax) position(std::integral_constant<int, j0 + 1>{});
            if (j0 + 2 < mmax) position(std::integral_constant<int, j0 + 2>{});
            if (j0 + 3 < mmax) position(std::integral_constant<int, j0 + 3>{});
            if constexpr (BATCH > 4)
            {
                if (j0 + 4 < mmax) position(std::integral_constant<int, j0 + 4>{});
                if (j0 + 5 < mmax) position(std::integral_constant<int, j0 + 5>{});
                if (j0 + 6 < mmax) position(std::integral_constant<int, j0 + 6>{});
                if (j0 + 7 < mmax) position(std::integral_constant<int, j0 + 7>{});
            }
        };
        if (mmax > 0) batch(std::integral_constant<int, 0>{});
        if constexpr (BATCH == 4)
        {
            if (mmax > 4) batch(std::integral_constant<int, 4>{});
            if (mmax > 8) batch(std::integral_constant<int, 8>{});
            if (mmax > 12) batch(std::integral_constant<int, 12>{});
        }
        else if (mmax > 8)
            batch(std::integral_constant<int, 8>{});

        // transmittance after the m retained entries decides whether the background is reached
        // (RenderBackward.cu:205-210,302-308); T is that product (1 for an empty list)
        const float T_after   = T;
        const bool bg_reached = inside && (T_after >= 0.001f);
        if (bg_reached && owned)
        {
#pragma unroll
            for (int c = 0; c < C; ++c) acc_bg[c] += T_after * g[c];
        }
        const float bg_term = bg_reached ? T_after * sbg : 0.f;

        // back to front: dL/dalpha_j = T_j s_j - (sum_{i>j} T_i alpha_i s_i + background term) / (1 - alpha_j + 1e-9)
        // (RenderBackward.cu:262-302); the entry goes to LDS under its pixel and under its (cell, place)
        float later = 0.f;  // sum over the entries behind this one
#pragma unroll
        for (int j = kListMax - 1; j >= 0; --j)
        {
            if (j < mmax)
            {
                const float ta = Tr[j] * A[j];
                if (j < m)
                {
                    const float dem        = 1.f / (1.f - A[j] + 1e-9f);
                    const float grad_alpha = Tr[j] * S[j] - (later + bg_term) * dem;
                    s_ex[j * kBlockPixels + t] = make_float2(grad_alpha, ta);
                    const unsigned tag     = (tagw[j / 4] >> (8 * (j & 3))) & 0xFFu;
                    const int w = (int)(tag >> 4) & 3, place = (int)(tag & 15u);
                    // the cell the entry came from: (x-1, y-1), (x, y-1), (x-1, y), (x, y) for w = 0..3; this pixel is corner
                    // 3 - w of that footprint
                    const int cxl = px - 1 + (w & 1), cyl = py - 1 + (w >> 1);
                    if ((unsigned)cxl < (unsigned)kBlockCells && (unsigned)cyl < (unsigned)kBlockCells)
                    {
                        const int slot = place * (kBlockCells * kBlockCells) + cyl * kBlockCells + cxl;
                        reinterpret_cast<unsigned char*>(s_rank)[slot * 4 + (3 - w)] = (unsigned char)j;
                    }
                }
                later += ta * S[j];
            }
        }
        __syncthreads();

        // ---- a row per (point, layer) pair that some pixel retained. Each pair is formed once: by the wavefront of
        // the first of its four corner pixels that retained it, whose lane still holds the point's compact number.
        // The pairs are unevenly spread over the pixels, so a wavefront queues {slot, compact number} of the pairs its
        // pixels are first for, position by position, and whenever enough wait, each lane forms one row. ----
        constexpr int kCells           = kBlockCells * kBlockCells;
        unsigned short* const qslot    = s_qslot[wave];
        int* const qcid                = s_qcid[wave];
        const bool inline_row          = layer < kInlineLayers;  // (the same for the whole block)
        const bool sparse              = *p.mode != 0;  // (the same for the whole view)
        const unsigned long long below = (1ull << lane) - 1ull;
        int waiting = 0;  // pairs in the queue (the same in every lane)
        // forms the rows of the first `n` pairs of the queue (n <= 64)
        auto form_rows = [&](int n)
        {
            if (lane < n)
            {
                const int slot  = qslot[lane];
                const int cid   = qcid[lane];
                int row_of      = cid;
                const int place = slot / kCells, c2 = slot - place * kCells;
                const int cyl = c2 / kBlockCells, cxl = c2 - cyl * kBlockCells;
                const unsigned w4 = s_rank[slot];
                // past the second layer: the number of the point's first row in the overflow table
                if (!inline_row) row_of = p.over_first[row_of];
                float tex[CPAD], ga[4];
#pragma unroll
                for (int c = 0; c < CPAD; ++c) tex[c] = 0.f;
#pragma unroll
                for (int corner = 0; corner < 4; ++corner)
                {
                    const unsigned r = (w4 >> (8 * corner)) & 0xFFu;
                    ga[corner]       = 0.f;
                    if (r == 0xFFu) continue;
                    const int tp   = (cyl + (corner >> 1)) * kBlockSide + cxl + (corner & 1);
                    const float2 e = s_ex[(int)r * kBlockPixels + tp];
                    ga[corner]     = e.x;
#pragma unroll
                    for (int c = 0; c < C; ++c) tex[c] += e.y * s_g[c * kBlockPixels + tp];
                }
                const long long over = (long long)row_of + (layer - kInlineLayers);
                if (inline_row || over < p.over_capacity)
                {
                    vf4* row = reinterpret_cast<vf4*>(inline_row ? p.rows_inline + ((size_t)(unsigned)row_of * kInlineLayers + layer) * PRF
                                                                 : p.rows_over + (size_t)over * PRF);
#pragma unroll
                    for (int q = 0; q < NQ; ++q) row[q] = vf4{tex[4 * q], tex[4 * q + 1], tex[4 * q + 2], tex[4 * q + 3]};
                    row[NQ] = vf4{ga[0], ga[1], ga[2], ga[3]};
                    if (sparse) p.flags[(size_t)(unsigned)cid * TRIPS_MAX_LAYERS + layer] = 1;
                }
            }
        };
        // the first 64 pairs leave the queue, the others move up
        auto pop64 = [&]()
        {
            form_rows(min(waiting, 64));
            unsigned short mslot = 0;
            int mcid             = 0;
            if (64 + lane < waiting) mslot = qslot[64 + lane], mcid = qcid[64 + lane];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            if (64 + lane < waiting) qslot[lane] = mslot, qcid[lane] = mcid;
            waiting = max(waiting - 64, 0);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        };
        // four list positions at a time (a loop over all sixteen, unrolled, would repeat the row code sixteen times;
        // one that is not unrolled would index the registers that hold the list)
#pragma unroll 1
        for (int q4 = 0; q4 < kListMax / 4; ++q4)
        {
            if (4 * q4 >= mmax) break;
            const unsigned tw = q4 == 0 ? tagw[0] : q4 == 1 ? tagw[1] : q4 == 2 ? tagw[2] : tagw[3];
            int idq[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) idq[i] = q4 == 0 ? id[i] : q4 == 1 ? id[4 + i] : q4 == 2 ? id[8 + i] : id[12 + i];
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                const int j = 4 * q4 + i;
                if (j >= mmax) break;
                bool own = false;
                int slot = 0;
                if (j < m)
                {
                    const unsigned tag = (tw >> (8 * i)) & 0xFFu;
                    const int w = (int)(tag >> 4) & 3, place = (int)(tag & 15u);
                    const int cxl = px - 1 + (w & 1), cyl = py - 1 + (w >> 1);
                    if ((unsigned)cxl < (unsigned)kBlockCells && (unsigned)cyl < (unsigned)kBlockCells)
                    {
                        slot              = place * kCells + cyl * kBlockCells + cxl;
                        const unsigned w4 = s_rank[slot];
                        // this pixel is corner 3 - w of the footprint: it forms the row if no corner before it retained the point
                        const int first = (w4 & 0xFFu) != 0xFFu ? 0 : ((w4 >> 8) & 0xFFu) != 0xFFu ? 1 : ((w4 >> 16) & 0xFFu) != 0xFFu ? 2 : 3;
                        own             = first == 3 - w;
                    }
                }
                const unsigned long long mask = __ballot(own);
                if (!mask) continue;
                if (own)
                {
                    const int at = waiting + (int)__popcll(mask & below);
                    qslot[at]    = (unsigned short)slot;
                    qcid[at]     = idq[i];
                }
                waiting += (int)__popcll(mask);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                if (waiting >= kQueueSlack) pop64();
            }
        }
        while (waiting > 0) pop64();
    }

#pragma unroll
    for (int i = 0; i < C; ++i)
    {
        double v = wave_sum((double)acc_bg[i]);
        if (lane == 0) s_acc[threadIdx.x >> 6][i] = v;
    }
    __syncthreads();
    if (threadIdx.x < C)
    {
        const int i = threadIdx.x;
        double v    = s_acc[0][i] + s_acc[1][i] + s_acc[2][i] + s_acc[3][i];
        if (v != 0.0) unsafeAtomicAdd(p.d_background + i, (float)v);
    }
}

// ---------------------------------------------------------------------------------------------------------
// Pass 2: per point. A wavefront takes 64 consecutive points. The work of a point is one item per layer it was written
// to; points differ in the layers they reach, so the items of the 64 points are dealt out to the lanes through LDS,
// one item per lane and round (usually one or two rounds): the items of a round are consecutive (point, layer) pairs,
// whose rows are consecutive in memory, and every lane works instead of all lanes walking the layers of the deepest
// point. An item's sums return through LDS and each point adds its items up in layer order. What does not change from
// point to point (camera, rotation matrix) waits in LDS rather than in registers.
constexpr int kItemFloats(int cpad) { return 4 + cpad; }  // {confidence, ip.x, ip.y, size} sums, then the descriptor's

struct PointPassCamera
{
    Camera cam;
    float R[9];
};

template <int C>
__global__ __launch_bounds__(256) void backward_points_kernel(const BackwardParams p)
{
    constexpr int CPAD = (C + 3) & ~3;
    constexpr int RF   = 4 + CPAD;  // floats per blend record
    constexpr int NQ   = CPAD / 4;
    constexpr int PRF  = pair_row_floats(CPAD);
    constexpr int NACC = 6 + 5 + 8;  // pose, K, distortion
    constexpr int NIT  = kItemFloats(CPAD);
    const int lane     = threadIdx.x & 63;
    const int wave     = threadIdx.x >> 6;
    const bool want_pose = p.d_pose != nullptr;
    const bool want_intr = p.d_intrinsics != nullptr;
    const bool want_size = p.d_point_size != nullptr;
    const bool identity  = p.header->not_identity == 0;  // index[pid] == pid for every point
    const bool overwrite = p.overwrite != 0;             // outputs are written, not added to
    const bool sparse    = *p.mode != 0;  // only the flagged rows exist
    // In that mode every point stores all its outputs (zeros where it has no gradient), all lanes at one place, so that
    // whole lines are written. (Descriptor columns other than the points' own, and all of them when the index is not
    // the identity, were cleared by the prologue kernel.)

    __shared__ PointPassCamera s_cam;
    // what an item needs of its point {ip.x, ip.y, size field, confidence, size_px, softplus' * d size_px / d size,
    // number of its first overflow row, compact number}, then the point in view space, kept here for the point's own lane
    __shared__ float s_point[4][64][11];
    __shared__ unsigned short s_item[4][64 * TRIPS_MAX_LAYERS];  // lane of the point | layer << 8
    __shared__ __align__(16) float s_sums[4][64][NIT];           // sums of the items of one round
    if (threadIdx.x == 0)
    {
        s_cam.cam = load_camera_bw(p.pose, p.intrinsics, p.view, p.dist_cutoff);
        rotation_matrix(s_cam.cam.V, s_cam.R);
    }
    __syncthreads();

    // a thread sees a handful of points: its own sums stay in single precision, everything across threads is double
    float acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = 0.f;

    const int stride = (int)gridDim.x * 256;
    // The compact number of a point is requested two steps ahead and its point record one step ahead, so that a step
    // starts with both in hand (a step otherwise begins with two dependent round trips to memory).
    const float4 kNoRecord = make_float4(0.f, -1.f, 0.f, 0.f);
    int cid_cur = -1, cid_next = -1;
    float4 tail_cur = kNoRecord;
    {
        const long long pid0 = (long long)blockIdx.x * 256 + (int)threadIdx.x;
        if (pid0 < p.num_points) cid_cur = p.cid_of[pid0];
        if (pid0 + stride < p.num_points) cid_next = p.cid_of[pid0 + stride];
        if (cid_cur >= 0) tail_cur = reinterpret_cast<const float4*>(p.prec)[cid_cur];
    }
    for (int base = blockIdx.x * 256; base < p.num_points; base += stride)
    {
        asm volatile("" ::: "memory");  // what waits in LDS is read where it is used, in every step
        const int pid = base + (int)threadIdx.x;
        // the records of a valid point sit at its compact number (valid points numbered in point order: lanes that are
        // neighbours here are neighbours there)
        const int cid   = cid_cur;
        const bool live = cid >= 0;
        // {softplus'(raw size), depth, layers written, size_px}
        const float4 tail = tail_cur;
        {
            // in flight during this step: the next step's point record, the compact number of the step after it
            cid_cur              = cid_next;
            tail_cur             = cid_cur >= 0 ? reinterpret_cast<const float4*>(p.prec)[cid_cur] : kNoRecord;
            const long long pid3 = (long long)pid + 2ll * stride;
            cid_next             = pid3 < p.num_points ? p.cid_of[pid3] : -1;
        }
        // {ip.x, ip.y, size field, confidence} of the blend record and the position: requested here, beside the point
        // record, unless the flags decide first whether the point has any row at all
        float4 r0 = make_float4(0.f, 0.f, 0.f, 0.f), pos = make_float4(0.f, 0.f, 0.f, 0.f);
        auto load_point_inputs = [&]()
        {
            r0  = *reinterpret_cast<const float4*>(p.rec + (size_t)(unsigned)cid * RF);
            pos = p.position[pid];
            if (p.displacement)
            {
                const float* dsp = p.displacement + (size_t)pid * 3;
                pos.x += dsp[0];
                pos.y += dsp[1];
                pos.z += dsp[2];
            }
        };
        if (live && !sparse) load_point_inputs();
        int max_layer = live ? __float_as_int(tail.z) : 0;
        // (a point of one or two layers has no overflow rows, and its number there is not looked at)
        const int first = max_layer > kInlineLayers ? p.over_first[cid] : 0;
        // (rows past the capacity of the overflow table do not exist: the forward reported the overflow)
        if (max_layer > kInlineLayers && (long long)first + (max_layer - kInlineLayers) > p.over_capacity)
            max_layer = kInlineLayers + (int)max(0ll, p.over_capacity - first);
        // the layers whose rows the point's items read: all it was written to, or those whose flag the tile pass set
        unsigned layer_mask = (1u << max_layer) - 1u;
        if (sparse && live)
        {
            // (one byte per layer at the point's compact number)
            const unsigned long long eight = *reinterpret_cast<const unsigned long long*>(p.flags + (size_t)(unsigned)cid * TRIPS_MAX_LAYERS);
            unsigned flagged = 0;
#pragma unroll
            for (int l = 0; l < TRIPS_MAX_LAYERS; ++l)
                if ((eight >> (8 * l)) & 0xFFull) flagged |= 1u << l;
            layer_mask &= flagged;
            if (layer_mask) load_point_inputs();
        }
        if (live && layer_mask)
        {
            // the point in view space, exactly as the projection kernel computed it
            float view[3];
            transform_point(s_cam.cam.V, pos.x, pos.y, pos.z, view);
            const float J_softmax_proj = s_cam.cam.fx * s_cam.cam.cfx / fmaxf(view[2], 0.f);
            float* sp = s_point[wave][lane];
            sp[0] = r0.x, sp[1] = r0.y, sp[2] = r0.z, sp[3] = r0.w, sp[4] = tail.w, sp[5] = tail.x * J_softmax_proj;
            sp[6] = __int_as_float(first);
            sp[7] = view[0], sp[8] = view[1], sp[9] = view[2];
            sp[10] = __int_as_float(cid);
        }

        // ---- the point's items: the layers it was written to ----
        const int my_items = (int)__popc(layer_mask);
        int first_item     = my_items;  // inclusive prefix over the wavefront, then made exclusive
        for (int o = 1; o < 64; o <<= 1)
        {
            const int t = __shfl_up(first_item, o);
            if (lane >= o) first_item += t;
        }
        const int num_items = __builtin_amdgcn_readlane(first_item, 63);  // <= 64 * 8
        first_item -= my_items;
        {
            int at = first_item;
            for (int l = 0; l < max_layer; ++l)
                if ((layer_mask >> l) & 1u) s_item[wave][at++] = (unsigned short)(lane | (l << 8));
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        float conf_grad = 0.f, size_grad = 0.f, d0 = 0.f, d1 = 0.f;
        float tex_grad[C];
#pragma unroll
        for (int c = 0; c < C; ++c) tex_grad[c] = 0.f;
        bool any = false;  // some pixel retained the point

        for (int round = 0; round < num_items; round += 64)
        {
            float i_conf = 0.f, i_d0 = 0.f, i_d1 = 0.f, i_size = 0.f;
            float i_tex[CPAD];
#pragma unroll
            for (int c = 0; c < CPAD; ++c) i_tex[c] = 0.f;
            if (round + lane < num_items)
            {
                // one layer of one point: its row holds the descriptor sums, then dL/dalpha of the four corners (zeros
                // where no pixel retained the point)
                const unsigned item = s_item[wave][round + lane];
                const int layer     = (int)(item >> 8);
                const float* sp     = s_point[wave][item & 63u];
                const float ipx = sp[0], ipy = sp[1], size_field = sp[2], conf = sp[3], size_px = sp[4], size_chain = sp[5];
                const vf4* row = reinterpret_cast<const vf4*>(
                    layer < kInlineLayers ? p.rows_inline + ((size_t)(unsigned)__float_as_int(sp[10]) * kInlineLayers + layer) * PRF
                                          : p.rows_over + ((size_t)__float_as_int(sp[6]) + (layer - kInlineLayers)) * PRF);
                vf4 tq[NQ];
#pragma unroll
                for (int q = 0; q < NQ; ++q) tq[q] = __builtin_nontemporal_load(row + q);
                const vf4 gav     = __builtin_nontemporal_load(row + NQ);
                const float ga[4] = {gav.x, gav.y, gav.z, gav.w};
                const float mfac = 1.f / float(1 << layer);
                const float ux = ipx * mfac, uy = ipy * mfac;
                const float fx = floorf(ux), fy = floorf(uy);
                const int px = (int)fx, py = (int)fy;
                const float sx = ux - fx, sy = uy - fy;
                float lfac = 1.f, J_lf = 0.f;
                if (want_size) lfac = layer_factor_encoded_grad(size_field, size_px, layer, p.num_layers, &J_lf);
#pragma unroll
                for (int corner = 0; corner < 4; ++corner)
                {
                    const int gx = px + (corner & 1), gy = py + (corner >> 1);
                    const float grad_alpha = ga[corner];
                    // blend_fac_index / compute_blending_fac (PointBlending.h:216-264)
                    // the four cases of the reference's switch on y_i + x_i as selects (same products, exact negations)
                    const bool x_hi = !(float(gx) < ux), y_hi = !(float(gy) < uy);
                    const float wx = x_hi ? sx : 1.f - sx, wy = y_hi ? sy : 1.f - sy;
                    float blend    = wx * wy;
                    const float J0 = x_hi ? wy : -wy;
                    const float J1 = y_hi ? wx : -wx;
                    if (fabsf(ux - float(gx)) > 1.f || fabsf(uy - float(gy)) > 1.f) blend *= 0.f;
                    i_conf += blend * lfac * grad_alpha;
                    const float gbs = conf * lfac * grad_alpha;
                    i_d0 += J0 * gbs;
                    i_d1 += J1 * gbs;
                    if (want_size)
                    {
                        const float grad_layer_ps = size_chain * J_lf * grad_alpha;
                        i_size += blend * conf * grad_layer_ps;
                    }
                }
#pragma unroll
                for (int c = 0; c < CPAD; ++c)
                {
                    const vf4 t4 = tq[c / 4];
                    i_tex[c]     = (c & 3) == 0 ? t4.x : (c & 3) == 1 ? t4.y : (c & 3) == 2 ? t4.z : t4.w;
                }
                float4* out = reinterpret_cast<float4*>(s_sums[wave][lane]);
                out[0]      = make_float4(i_conf, i_d0, i_d1, i_size);
#pragma unroll
                for (int q = 0; q < NQ; ++q) out[1 + q] = make_float4(i_tex[4 * q], i_tex[4 * q + 1], i_tex[4 * q + 2], i_tex[4 * q + 3]);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            // the point's items of this round, in layer order
            const int j_end = min(first_item + my_items, round + 64);
            for (int j = max(first_item, round); j < j_end; ++j)
            {
                const float4* in = reinterpret_cast<const float4*>(s_sums[wave][j - round]);
                const float4 a   = in[0];
                bool nz          = a.x != 0.f || a.y != 0.f || a.z != 0.f || a.w != 0.f;
                conf_grad += a.x;
                d0 += a.y;
                d1 += a.z;
                size_grad += a.w;
#pragma unroll
                for (int q = 0; q < NQ; ++q)
                {
                    const float4 t = in[1 + q];
                    nz             = nz || t.x != 0.f || t.y != 0.f || t.z != 0.f || t.w != 0.f;
                    if (4 * q < C) tex_grad[4 * q] += t.x;
                    if (4 * q + 1 < C) tex_grad[4 * q + 1] += t.y;
                    if (4 * q + 2 < C) tex_grad[4 * q + 2] += t.z;
                    if (4 * q + 3 < C) tex_grad[4 * q + 3] += t.w;
                }
                any = any || nz;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        if (pid >= p.num_points || (!live && !overwrite)) continue;
        const int tex = identity ? pid : p.index[pid];  // (a column outside the table: the point was culled)
        if (!any && !overwrite) continue;

        float g_point[3] = {0.f, 0.f, 0.f}, g_pose[6], g_k[5], g_dis[8];
        if (any)
        {
            const float* sp = s_point[wave][lane];
            project_backward(s_cam.cam, s_cam.R, sp[7], sp[8], sp[9], d0, d1, g_point, g_pose, g_k, g_dis, want_intr);
            if (want_pose)
            {
#pragma unroll
                for (int k = 0; k < 6; ++k) acc[k] += g_pose[k];
            }
            if (want_intr)
            {
#pragma unroll
                for (int k = 0; k < 5; ++k) acc[6 + k] += g_k[k];
#pragma unroll
                for (int k = 0; k < 8; ++k) acc[11 + k] += g_dis[k];
            }
        }

        if (identity && overwrite)
        {
#pragma unroll
            for (int c = 0; c < C; ++c) p.d_texture[(size_t)c * p.num_texels + tex] = tex_grad[c];
            p.d_confidence[tex] = conf_grad;
        }
        else if (identity)
        {
#pragma unroll
            for (int c = 0; c < C; ++c) p.d_texture[(size_t)c * p.num_texels + tex] += tex_grad[c];
            p.d_confidence[tex] += conf_grad;
        }
        else if (any)
        {
#pragma unroll
            for (int c = 0; c < C; ++c) unsafeAtomicAdd(p.d_texture + (size_t)c * p.num_texels + tex, tex_grad[c]);
            unsafeAtomicAdd(p.d_confidence + tex, conf_grad);
        }
        if (want_size)
        {
            if (overwrite)
                p.d_point_size[pid] = size_grad;
            else
                p.d_point_size[pid] += size_grad;
        }
        if (p.d_position)
        {
            float4* dp = reinterpret_cast<float4*>(p.d_position) + pid;
            float4 v   = overwrite ? make_float4(0.f, 0.f, 0.f, 0.f) : *dp;
            v.x += g_point[0];
            v.y += g_point[1];
            v.z += g_point[2];
            *dp = v;
        }
    }

    if (!want_pose && !want_intr) return;
    __shared__ double s_acc[4][NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i)
    {
        const bool used = (i < 6) ? want_pose : want_intr;
        if (!used) continue;
        double v = wave_sum((double)acc[i]);
        if (lane == 0) s_acc[threadIdx.x >> 6][i] = v;
    }
    __syncthreads();
    if (threadIdx.x < NACC)
    {
        const int i     = threadIdx.x;
        const bool used = (i < 6) ? want_pose : want_intr;
        if (used)
        {
            double v = s_acc[0][i] + s_acc[1][i] + s_acc[2][i] + s_acc[3][i];
            if (v != 0.0)
            {
                if (i < 6)
                    unsafeAtomicAdd(p.d_pose + i, v);
                else
                    unsafeAtomicAdd(p.d_intrinsics + (i - 6), (float)v);
            }
        }
    }
}

// Before the two passes of a view: the rows of the view's pairs start as zeros (the tile pass writes the rows of the
// pairs that some pixel retained, the point pass reads all rows of a point): the two inline rows of every valid point
// (compact numbers are dense within each chunk of the binning kernels) and the overflow rows that the forward counted.
// For a view in which few pairs are retained (sparse_pair_rows) the flag bytes of the rows are cleared instead; the choice
// is left in the workspace for the two passes.
// On the first view of a call also, in
// overwrite mode (`texels`): the descriptor and confidence gradients of the columns that the point pass does not write
// itself. With the identity index (the forward noted it in the header) those are the columns past the last point;
// otherwise all of them, the point pass then adds with atomics. `clear_sums`: the block sums that both passes add to
// (background, every pose row, every intrinsics row).
__global__ __launch_bounds__(256) void backward_prologue_kernel(const ViewHeader* __restrict__ header, const int32_t* __restrict__ chunk_valid,
                                                                int bin_groups, int points_per_block, float* __restrict__ rows_inline,
                                                                float* __restrict__ rows_over, unsigned char* __restrict__ flags, int32_t* __restrict__ mode, int force_mode, int pair_row, long long over_capacity,
                                                                float* __restrict__ d_texture,
                                                                float* __restrict__ d_confidence, int channels, int num_texels,
                                                                int num_points, int texels, int clear_sums,
                                                                float* __restrict__ d_background, double* __restrict__ d_pose,
                                                                int num_images, float* __restrict__ d_intrinsics, int num_cameras)
{
    long long over_rows = (long long)header->overflow_rows;
    if (over_rows > over_capacity) over_rows = over_capacity;
    // the view's retained entries: every workgroup adds the blend kernel's partial sums up for itself
    __shared__ unsigned long long s_retained[4];
    {
        unsigned long long r = (unsigned long long)(unsigned)chunk_valid[bin_groups + threadIdx.x];  // (kRetainedParts = 256 threads)
        for (int o = 32; o > 0; o >>= 1) r += __shfl_xor(r, o);
        if ((threadIdx.x & 63) == 0) s_retained[threadIdx.x >> 6] = r;
        __syncthreads();
    }
    const bool sparse = force_mode == 0 ? sparse_pair_rows((s_retained[0] + s_retained[1] + s_retained[2] + s_retained[3]) * kRetainedSample, header->n_entries)
                                        : force_mode == 2;
    if (blockIdx.x == 0 && threadIdx.x == 0) *mode = sparse ? 1 : 0;
    if (sparse)
    {
        // (the table ends on a multiple of 256 bytes: whole 16-byte words are cleared)
        const long long words = ((long long)num_points * TRIPS_MAX_LAYERS + 15) / 16;
        for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < words; i += (long long)gridDim.x * 256)
            reinterpret_cast<vu4*>(flags)[i] = vu4{0u, 0u, 0u, 0u};
    }
    else
    {
        // (rows are a multiple of four floats)
        const int row_quads = kInlineLayers * pair_row / 4;
        for (int chunk = blockIdx.x; chunk < bin_groups; chunk += gridDim.x)
        {
            const int begin = min(num_points, chunk * points_per_block);
            const int quads = chunk_valid[chunk] * row_quads;
            vf4* dst        = reinterpret_cast<vf4*>(rows_inline) + (size_t)begin * row_quads;
            for (int i = threadIdx.x; i < quads; i += 256) __builtin_nontemporal_store(vf4{0.f, 0.f, 0.f, 0.f}, dst + i);
        }
        const long long quads = over_rows * pair_row / 4;
        vf4* dst              = reinterpret_cast<vf4*>(rows_over);
        for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < quads; i += (long long)gridDim.x * 256)
            __builtin_nontemporal_store(vf4{0.f, 0.f, 0.f, 0.f}, dst + i);
    }
    if (clear_sums && blockIdx.x == 0)
    {
        if (d_background)
            for (int i = threadIdx.x; i < channels; i += 256) d_background[i] = 0.f;
        if (d_pose)
            for (int i = threadIdx.x; i < num_images * 6; i += 256) d_pose[i] = 0.0;
        if (d_intrinsics)
            for (int i = threadIdx.x; i < num_cameras * 13; i += 256) d_intrinsics[i] = 0.f;
    }
    if (!texels) return;
    const int first = header->not_identity == 0 ? min(num_points, num_texels) : 0;
    const int n     = num_texels - first;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < (long long)n * (channels + 1); i += (long long)gridDim.x * 256)
    {
        const int c = (int)(i / n), t = first + (int)(i - (long long)c * n);
        if (c < channels)
            d_texture[(size_t)c * num_texels + t] = 0.f;
        else
            d_confidence[t] = 0.f;
    }
}

template <int C>
hipError_t launch_tiles(const BackwardParams& p, int blocks, hipStream_t stream)
{
    const size_t lds = tiles_lds_bytes((C + 3) & ~3);
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&backward_tiles_kernel<C>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((backward_tiles_kernel<C>), dim3(blocks), dim3(256), lds, stream, p);
    return hipSuccess;
}

#define TRIPS_BW_DISPATCH(KERNEL, BLOCKS)                                                                      \
    switch (channels)                                                                                          \
    {                                                                                                          \
        case 3: hipLaunchKernelGGL((KERNEL<3>), dim3(BLOCKS), dim3(256), 0, stream, p); break;                 \
        case 4: hipLaunchKernelGGL((KERNEL<4>), dim3(BLOCKS), dim3(256), 0, stream, p); break;                 \
        case 6: hipLaunchKernelGGL((KERNEL<6>), dim3(BLOCKS), dim3(256), 0, stream, p); break;                 \
        case 8: hipLaunchKernelGGL((KERNEL<8>), dim3(BLOCKS), dim3(256), 0, stream, p); break;                 \
        case 16: hipLaunchKernelGGL((KERNEL<16>), dim3(BLOCKS), dim3(256), 0, stream, p); break;               \
        default: return hipErrorInvalidValue;                                                                  \
    }

hipError_t launch_backward_view(const BackwardParams& p, int channels, hipStream_t stream, Profiler* prof)
{
    const int N = p.num_points;
    {
        ProfScope ps(prof, "backward_prologue", stream);
        hipLaunchKernelGGL(backward_prologue_kernel, dim3(2048), dim3(256), 0, stream, p.header, p.chunk_valid, p.bin_groups,
                           p.points_per_block, p.rows_inline, p.rows_over, p.flags, p.mode, p.force_mode, pair_row_floats((channels + 3) & ~3),
                           p.over_capacity, p.d_texture, p.d_confidence, channels, p.num_texels,
                           N, p.overwrite, p.clear_block_sums, p.d_background, p.d_pose_all, p.num_images, p.d_intrinsics_all,
                           p.num_cameras);
    }
    {
        // (no points: only the background receives gradient)
        ProfScope ps(prof, "backward_tiles", stream);
        const long long blocks8 = (((long long)p.blocks_off[p.num_layers] + 8 * kNumXcd - 1) / (8 * kNumXcd)) * (8 * kNumXcd);  // whole runs of 8 blocks x 8 XCDs
        const int blocks        = (int)blocks8;
        hipError_t e            = hipErrorInvalidValue;
        switch (channels)
        {
            case 3: e = launch_tiles<3>(p, blocks, stream); break;
            case 4: e = launch_tiles<4>(p, blocks, stream); break;
            case 6: e = launch_tiles<6>(p, blocks, stream); break;
            case 8: e = launch_tiles<8>(p, blocks, stream); break;
            case 16: e = launch_tiles<16>(p, blocks, stream); break;
            default: break;
        }
        if (e != hipSuccess) return e;
    }
    if (N > 0)
    {
        ProfScope ps(prof, "backward_points", stream);
        // (four workgroups per CU, each walking its share of the points: every further workgroup adds its atomics on the
        // pose and intrinsics sums)
        const int blocks = min((N + 255) / 256, 1024);
        TRIPS_BW_DISPATCH(backward_points_kernel, blocks);
    }
    return hipGetLastError();
}

}  // namespace trips
