// Backward kernels of the splat path for gfx950 (wave64).
//
//   backward_pixels_kernel + backward_points_kernel <- BlendBackwardsBilinearTiled
//                                                      src/lib/rendering/RenderBackward.cu:90-618
//
// The reference walks one pixel list per thread and scatters every entry's gradient with float atomics
// (3 position + 1 size + 1 confidence + C descriptor atomics per retained entry). Scattered atomics run at
// about 2e10 per second on this GPU while scattered loads run at 5e10 and cost the same for 4 or 64 bytes,
// so the work is split in two passes without atomics on the per-point arrays:
//   1. pixels: a 16-lane row (an 8-lane half row for short lists) owns a pixel, each lane one retained entry. Alpha and transmittance are recomputed
//      from the per-point record exactly as the forward computed them; the "all later entries" sum of
//      RenderBackward.cu:284-301 is a suffix sum across the row. Per entry it writes {dL/dalpha, T*alpha*dL/dimage}
//      into the pixel's row of a [P,K] table. The forward's blend kernel has left one byte per retained entry, its
//      rank in the pixel's list, in the point's 32-slot table (slot = layer * 4 + footprint corner; two planes of 16
//      slots per point, layers 0..3 and 4..7).
//   2. points: one thread per point walks its slots, gathers those records (one aligned load each), sums the image-space gradient of all its entries and runs the projection chain ONCE
//      (the chain is linear in the image-space gradient, RenderBackward.cu:385-417), then adds its gradients
//      with plain read-modify-writes. Pose / intrinsics partials stay in double registers over a grid-stride
//      loop before one block-level reduction and one atomic per value and block (the reference keeps them in
//      shared double arrays, :160-187,546-617).
// Gradients are therefore summed in a fixed order and are bit-reproducible from run to run.
#include "row16.h"
#include "splat_internal.h"
#include "trips_math.h"

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

typedef float vf2 __attribute__((ext_vector_type(2)));
typedef float vf4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ double wave_sum(double v)
{
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}


// ---------------------------------------------------------------------------------------------------------
// Pass 1: per pixel row. Writes the pixel's exchange row {g[0..Cpad), {dL/dalpha_j, T_j alpha_j} for j < entry_row_entries}.
// 64 / ROW consecutive pixels starting at pix_first: ROW = 16 lanes per pixel, or 8 when none of them retained more
// than 8 entries. m_in = retained entries of this lane's pixel (the caller has them already).
template <int C, int ROW, bool SECOND>
__device__ __forceinline__ void backward_pixel_rows(const BackwardParams& p, const TileCtx& tc, const float* gi, int pix_first,
                                                    int m_in, float (&acc_bg)[C])
{
    constexpr int CPAD = (C + 3) & ~3;
    constexpr int RF   = 4 + CPAD;          // floats per blend record
    const int lane     = threadIdx.x & 63;
    const int sub      = lane & (ROW - 1);
    const int grp      = lane / ROW;
    const int kshift   = p.list_depth == 16 ? 4 : 3;
    // the group's pixels lie side by side in one row of the tile
    const int pix   = pix_first + grp;
    const int layer = tc.layer, lw = tc.w, lh = tc.h;
    const int gx = tc.x0 + (pix & (kTile - 1)), gy = tc.y0 + ((pix >> kTileShift) & (kTile - 1));
    const bool live = gx < lw && gy < lh;  // false for the padding of partial tiles

    const int m    = live ? m_in : 0;
    const bool has = sub < m;
    int mmax       = m;
    if (ROW == 8) mmax = max(mmax, __shfl_xor(mmax, 8));
    mmax           = max(mmax, __shfl_xor(mmax, 16));
    mmax           = max(mmax, __shfl_xor(mmax, 32));
    mmax           = __builtin_amdgcn_readfirstlane(mmax);

    float g[C];
    {
        // offsets inside one view's image stay far below 2^32 (the pyramid has at most kMaxBins tiles)
        if (p.layout == TRIPS_LAYOUT_CHW)
        {
            const size_t plane = (size_t)lw * lh;
            const float* o     = gi + ((size_t)p.view_index * C) * plane;
            const unsigned at  = __umul24((unsigned)gy, (unsigned)lw) + (unsigned)gx;
#pragma unroll
            for (int c = 0; c < C; ++c) g[c] = live ? (o + c * plane)[at] : 0.f;
        }
        else
        {
            const float* o    = gi + ((size_t)p.view_index * lh * lw) * C;
            const unsigned at = (__umul24((unsigned)gy, (unsigned)lw) + (unsigned)gx) * C;
#pragma unroll
            for (int c = 0; c < C; ++c) g[c] = live ? o[at + c] : 0.f;
        }
    }

    int cid = 0;  // compact number of the entry's point
    float desc[CPAD];
#pragma unroll
    for (int c = 0; c < CPAD; ++c) desc[c] = 0.f;
    float a = 0.f;
    if (has)
    {
        cid               = __builtin_nontemporal_load(p.lists + (((size_t)(unsigned)pix << kshift) + sub));
        const float4* rec = reinterpret_cast<const float4*>(p.rec + (size_t)(unsigned)cid * RF);
        const float4 r0   = rec[0];
#pragma unroll
        for (int q = 0; q < CPAD / 4; ++q)
        {
            const float4 t  = rec[1 + q];
            desc[4 * q]     = t.x;
            desc[4 * q + 1] = t.y;
            desc[4 * q + 2] = t.z;
            desc[4 * q + 3] = t.w;
        }
        const float mfac = __uint_as_float((uint32_t)(127 - layer) << 23);  // 2^-layer
        const float ux = r0.x * mfac, uy = r0.y * mfac;
        float w = (1.f - fabsf(ux - float(gx))) * (1.f - fabsf(uy - float(gy)));
        if (fabsf(ux - float(gx)) > 1.f || fabsf(uy - float(gy)) > 1.f) w = 0.f;
        a = w * r0.w;
        a *= layer_factor_encoded(r0.z, layer, p.num_layers);
    }

    // exclusive transmittance, same chain as the forward
    const float T = ROW == 8 ? half_exclusive_product(1.f - a, mmax) : row_exclusive_product(1.f - a, mmax);
    // transmittance after the m retained entries decides whether the background is reached
    // (RenderBackward.cu:205-210,302-308)
    float T_after = T * (1.f - a);
    T_after       = __shfl(T_after, max(m - 1, 0), ROW);
    if (m == 0) T_after = 1.f;
    const bool bg_reached = live && (T_after >= 0.001f);

    float s = 0.f, sbg = 0.f;
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        s += desc[c] * g[c];
        sbg += p.background[c] * g[c];
    }
    const float ta = T * a;
    const float q  = has ? ta * s : 0.f;
    float later    = ROW == 8 ? half_exclusive_suffix_sum(q) : row_exclusive_suffix_sum(q);  // entries i > j
    if (bg_reached) later += T_after * sbg;
    const float dem        = 1.f / (1.f - a + 1e-9f);
    const float grad_alpha = T * s - later * dem;

    if (bg_reached && sub == 0)
    {
#pragma unroll
        for (int c = 0; c < C; ++c) acc_bg[c] += T_after * g[c];
    }
    // For pass 2, one row of 64 bytes (128 above 8 channels) per pixel: the pixel's image gradient (a point finds all
    // channels and its entry in one line) followed by {dL/dalpha, T alpha} of the first entry_row_entries retained
    // entries; the entries beyond that go to a table of their own.
    // Rows of 64 bytes are written a second time, one row further on (see BackwardParams).
    constexpr int KIN       = entry_row_entries(CPAD);
    constexpr bool kShifted = entry_row_floats(CPAD) == 16;
    float* row              = p.entry_grad + (size_t)(unsigned)pix * entry_row_floats(CPAD);
    constexpr bool second   = kShifted && SECOND;
    float* row2             = kShifted ? p.entry_grad_shifted + (size_t)(unsigned)pix * 16 : nullptr;
    if (has && sub >= KIN)
        __builtin_nontemporal_store(vf2{grad_alpha, ta}, reinterpret_cast<vf2*>(p.entry_over) + ((size_t)(unsigned)pix * (16 - KIN) + (sub - KIN)));
    if (CPAD == 4)
    {
        // the whole row with one store instruction, 8 bytes per lane: lanes 0 and 1 the image gradient, lanes 2..7 the
        // entries of lanes 0..5 (64 contiguous bytes per pixel instead of a 16-byte and six 8-byte pieces)
        const float ga_before = row_shr<2>(grad_alpha, 0.f), ta_before = row_shr<2>(ta, 0.f);
        const float g2 = C > 2 ? g[C > 2 ? 2 : 0] : 0.f, g3 = C > 3 ? g[C > 3 ? 3 : 0] : 0.f;
        const vf2 v      = sub == 0 ? vf2{g[0], g[1]} : sub == 1 ? vf2{g2, g3} : vf2{ga_before, ta_before};
        const bool store = sub < 2 ? m > 0 : (sub < 8 && sub - 2 < m);
        if (store)
        {
            __builtin_nontemporal_store(v, reinterpret_cast<vf2*>(row) + sub);
            if (second) __builtin_nontemporal_store(v, reinterpret_cast<vf2*>(row2) + sub);
        }
    }
    else
    {
        if (has && sub < KIN)
        {
            __builtin_nontemporal_store(vf2{grad_alpha, ta}, reinterpret_cast<vf2*>(row + CPAD) + sub);
            if (second) __builtin_nontemporal_store(vf2{grad_alpha, ta}, reinterpret_cast<vf2*>(row2 + CPAD) + sub);
        }
        if (sub == 0 && m > 0)
        {
            float gp[CPAD];
#pragma unroll
            for (int c = 0; c < CPAD; ++c) gp[c] = c < C ? g[c] : 0.f;
#pragma unroll
            for (int q = 0; q < CPAD / 4; ++q)
            {
                __builtin_nontemporal_store(vf4{gp[4 * q], gp[4 * q + 1], gp[4 * q + 2], gp[4 * q + 3]}, reinterpret_cast<vf4*>(row) + q);
                if (second)
                    __builtin_nontemporal_store(vf4{gp[4 * q], gp[4 * q + 1], gp[4 * q + 2], gp[4 * q + 3]}, reinterpret_cast<vf4*>(row2) + q);
            }
        }
    }
}

// SECOND: the exchange rows are written twice (see BackwardParams::entry_grad_shifted).
template <int C, bool SECOND>
__device__ __forceinline__ void backward_pixels_body(const BackwardParams& p)
{
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // a lane sees a few dozen pixels: its own sums stay in single precision, everything across lanes is double
    float acc_bg[C];
#pragma unroll
    for (int i = 0; i < C; ++i) acc_bg[i] = 0.f;

    // A workgroup walks quarters of tiles (256 pixels = 32 groups of eight), 4 workgroups per tile, all on one XCD.
    // A wavefront takes every fourth group; it reads the retained counts of all its 64 pixels with one load, so the
    // choice of the row width and the rows' own lengths cost no further memory round trip.
    constexpr int kPerTile      = 4;
    constexpr int kQuarter      = kTilePixels / kPerTile;
    const long long num_tiles   = p.geom.bin_off[p.num_layers];
    const long long tile_stride = (long long)(gridDim.x / (kPerTile * kNumXcd)) * kNumXcd;

    for (long long lbl = xcd_tile_block(blockIdx.x, kPerTile); lbl < num_tiles * kPerTile; lbl += tile_stride * kPerTile)
    {
        const int lb = (int)lbl;  // quarter tile number; all its pixels exist (tiles are padded to 1024 pixels)
        // the quarter's pixels share a tile: its layer and position are found once, on the scalar unit
        const TileCtx tc      = tile_ctx(p.geom, lb / kPerTile);
        const float* const gi = p.grad_image[tc.layer];
        // lane -> pixel (lane % 8) of this wavefront's group number lane / 8
        const int my_pix = lb * kQuarter + ((lane >> 3) * 4 + wave) * 8 + (lane & 7);
        int m_all        = p.retained[my_pix] & kRetainedMask;  // (low bits of the word) 0 for the padding of partial tiles
        int m_grp        = m_all;
        m_grp            = max(m_grp, __shfl_xor(m_grp, 1));
        m_grp            = max(m_grp, __shfl_xor(m_grp, 2));
        m_grp            = max(m_grp, __shfl_xor(m_grp, 4));
#pragma unroll 1
        for (int it = 0; it < 8; ++it)
        {
            const int pix_first = lb * kQuarter + (it * 4 + wave) * 8;
            const int m8        = __builtin_amdgcn_readfirstlane(__shfl(m_grp, it * 8));
            if (m8 <= 8)
                backward_pixel_rows<C, 8, SECOND>(p, tc, gi, pix_first, __shfl(m_all, it * 8 + (lane >> 3)), acc_bg);
            else
            {
                backward_pixel_rows<C, 16, SECOND>(p, tc, gi, pix_first, __shfl(m_all, it * 8 + (lane >> 4)), acc_bg);
                backward_pixel_rows<C, 16, SECOND>(p, tc, gi, pix_first + 4, __shfl(m_all, it * 8 + 4 + (lane >> 4)), acc_bg);
            }
        }
    }

    __shared__ double s_acc[4][C];
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

// (up to 4 channels the kernel needs 77 registers: seven wavefronts per SIMD; held to the 64 of eight it spills)
// The two forms of the body are separate code: a flag tested at every store costs registers that the kernel lacks.
template <int C>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(C <= 4 ? 7 : 1))) void backward_pixels_kernel(const BackwardParams p)
{
    if (entry_row_floats((C + 3) & ~3) == 16 && use_shifted_rows(*p.header))
        backward_pixels_body<C, true>(p);
    else
        backward_pixels_body<C, false>(p);
}

// ---------------------------------------------------------------------------------------------------------
// Pass 2: per point. A wavefront takes 64 consecutive points. The work of a point is one item per layer in which some
// pixel retained it (the rank bytes say which); points differ in the layers they reach, so the items of the 64 points
// are dealt out to the lanes through LDS, one item per lane and round (usually one round): every lane then issues the
// gathers of its item at once, instead of all lanes walking the layers of the deepest point one memory round trip
// after the other. An item's sums return through LDS and each point adds its items up in layer order.
// The kernel is a chain of dependent memory round trips per step; it is kept short: the compact number of a step's
// point is requested one step ahead, and what does not change from step to step (camera, rotation matrix) waits in LDS
// rather than in registers, which the items need.
constexpr int kItemFloats(int cpad) { return 4 + cpad; }  // {confidence, ip.x, ip.y, size} sums, then the descriptor's

struct PointPassCamera
{
    Camera cam;
    float R[9];
};

template <int C>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(C <= 4 ? 4 : 1))) void backward_points_kernel(const BackwardParams p)
{
    constexpr int CPAD = (C + 3) & ~3;
    constexpr int KIN  = entry_row_entries(CPAD);
    constexpr int RF   = 4 + CPAD;  // floats per blend record
    constexpr int NACC = 6 + 5 + 8;  // pose, K, distortion
    constexpr int NIT  = kItemFloats(CPAD);
    const int lane     = threadIdx.x & 63;
    const int wave     = threadIdx.x >> 6;
    const bool want_pose = p.d_pose != nullptr;
    const bool want_intr = p.d_intrinsics != nullptr;
    const bool want_size = p.d_point_size != nullptr;
    const bool identity  = p.header->not_identity == 0;  // index[pid] == pid for every point
    const bool overwrite = p.overwrite != 0;             // outputs are written, not added to
    const bool shifted_rows = entry_row_floats(CPAD) == 16 && use_shifted_rows(*p.header);
    // In that mode every point stores all its outputs (zeros where it has no gradient), all lanes at one place, so that
    // whole lines are written. (Descriptor columns other than the points' own, and all of them when the index is not
    // the identity, were cleared by zero_texel_grads_kernel.)

    __shared__ PointPassCamera s_cam;
    // what an item needs of its point {ip.x, ip.y, size field, confidence, size_px, softplus' * d size_px / d size},
    // then the point in view space, kept here for the point's own lane
    __shared__ float s_point[4][64][9];
    __shared__ uint2 s_item[4][64 * 8];                 // {lane of the point | layer << 8, the layer's four rank bytes}
    __shared__ __align__(16) float s_sums[4][64][NIT];  // sums of the items of one round
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
    int cid_next     = -1;
    {
        const int pid0 = (int)blockIdx.x * 256 + (int)threadIdx.x;
        if (pid0 < p.num_points) cid_next = p.cid_of[pid0];
    }
    for (int base = blockIdx.x * 256; base < p.num_points; base += stride)
    {
        asm volatile("" ::: "memory");  // what waits in LDS is read where it is used, in every step
        const int pid = base + (int)threadIdx.x;
        // the records of a valid point sit at its compact number (valid points numbered in point order: lanes that are
        // neighbours here are neighbours there)
        const int cid   = cid_next;
        const bool live = cid >= 0;
        {
            const long long pid2 = (long long)pid + stride;
            cid_next             = pid2 < p.num_points ? p.cid_of[pid2] : -1;  // in flight during this step
        }
        // {softplus'(raw size), depth, layers written, size_px}
        const float4 tail = live ? reinterpret_cast<const float4*>(p.prec)[cid] : make_float4(0.f, -1.f, 0.f, 0.f);
        const int max_layer = live ? __float_as_int(tail.z) : 0;
        uint4 rk0 = make_uint4(~0u, ~0u, ~0u, ~0u), rk1 = rk0;
        if (live)
        {
            const float4 r0 = *reinterpret_cast<const float4*>(p.rec + (size_t)(unsigned)cid * RF);  // ip.x ip.y size field conf
            // the point in view space, exactly as the projection kernel computed it
            float4 pos = p.position[pid];
            if (p.displacement)
            {
                const float* dsp = p.displacement + (size_t)pid * 3;
                pos.x += dsp[0];
                pos.y += dsp[1];
                pos.z += dsp[2];
            }
            rk0 = *reinterpret_cast<const uint4*>(p.rank + (size_t)cid * 16);
            // layers 4..7: a row of the second plane, defined only for the points that were written to those layers
            if (max_layer > 4) rk1 = *reinterpret_cast<const uint4*>(p.rank + (size_t)p.num_points * 16 + (size_t)cid * 16);
            float view[3];
            transform_point(s_cam.cam.V, pos.x, pos.y, pos.z, view);
            const float J_softmax_proj = s_cam.cam.fx * s_cam.cam.cfx / fmaxf(view[2], 0.f);
            float* sp = s_point[wave][lane];
            sp[0] = r0.x, sp[1] = r0.y, sp[2] = r0.z, sp[3] = r0.w, sp[4] = tail.w, sp[5] = tail.x * J_softmax_proj;
            sp[6] = view[0], sp[7] = view[1], sp[8] = view[2];
        }

        // ---- the point's items: the layers it was written to in which some corner pixel retained it ----
        const unsigned words[8] = {rk0.x, rk0.y, rk0.z, rk0.w, rk1.x, rk1.y, rk1.z, rk1.w};
        unsigned layer_mask = 0;
#pragma unroll
        for (int l = 0; l < 8; ++l)
            if (l < max_layer && words[l] != 0xFFFFFFFFu) layer_mask |= 1u << l;
        const int my_items = __popc(layer_mask);
        int first_item     = my_items;  // inclusive prefix over the wavefront, then made exclusive
        for (int o = 1; o < 64; o <<= 1)
        {
            const int t = __shfl_up(first_item, o);
            if (lane >= o) first_item += t;
        }
        const int num_items = __builtin_amdgcn_readlane(first_item, 63);  // <= 64 * 8
        first_item -= my_items;
        {
            int k = first_item;
#pragma unroll
            for (int l = 0; l < 8; ++l)
                if (layer_mask & (1u << l)) s_item[wave][k++] = make_uint2((unsigned)lane | ((unsigned)l << 8), words[l]);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        float conf_grad = 0.f, size_grad = 0.f, d0 = 0.f, d1 = 0.f;
        float tex_grad[C];
#pragma unroll
        for (int c = 0; c < C; ++c) tex_grad[c] = 0.f;
        const bool any = my_items > 0;

        for (int round = 0; round < num_items; round += 64)
        {
            if (round + lane < num_items)
            {
                // one layer of one point: the four gathers are issued together, then consumed in corner order
                const uint2 item    = s_item[wave][round + lane];
                const int layer     = (int)(item.x >> 8);
                const unsigned word = item.y;
                const float* sp     = s_point[wave][item.x & 63u];
                const float ipx = sp[0], ipy = sp[1], size_field = sp[2], conf = sp[3], size_px = sp[4], size_chain = sp[5];
                const float mfac = 1.f / float(1 << layer);
                const float ux = ipx * mfac, uy = ipy * mfac;
                const float fx = floorf(ux), fy = floorf(uy);
                const int px = (int)fx, py = (int)fy;
                const float sx = ux - fx, sy = uy - fy;
                float lfac = 1.f, J_lf = 0.f;
                if (want_size) lfac = layer_factor_encoded_grad(size_field, size_px, layer, p.num_layers, &J_lf);
                float2 e[4];
                float4 gq[4][CPAD / 4];
                // 64-byte rows: a footprint that starts at an odd pixel reads the copy in which its two pixels of a
                // row share a line (not across the border of a tile, where they are not neighbours in memory)
                const float* rows = (shifted_rows && (px & 1) && (px & (kTile - 1)) != kTile - 1)
                                        ? p.entry_grad_shifted
                                        : p.entry_grad;
#pragma unroll
                for (int corner = 0; corner < 4; ++corner)
                {
                    const unsigned j = (word >> (8 * corner)) & 0xFFu;
                    const int gx = px + (corner & 1), gy = py + (corner >> 1);
                    const unsigned pix = (unsigned)pix_index_mul24(p.geom, layer, gx, gy);
                    const bool on      = j != 0xFFu;
                    const float* row   = rows + (size_t)pix * entry_row_floats(CPAD);  // the pixel's row
                    const unsigned jj  = j & 15u;
                    const float2* src2 = jj < (unsigned)KIN ? reinterpret_cast<const float2*>(row + CPAD) + jj
                                                            : reinterpret_cast<const float2*>(p.entry_over) + ((size_t)pix * (16 - KIN) + (jj - KIN));
                    e[corner]          = on ? *src2 : make_float2(0.f, 0.f);
                    const float4* src  = reinterpret_cast<const float4*>(row);
#pragma unroll
                    for (int q = 0; q < CPAD / 4; ++q) gq[corner][q] = on ? src[q] : make_float4(0.f, 0.f, 0.f, 0.f);
                }
                float i_conf = 0.f, i_d0 = 0.f, i_d1 = 0.f, i_size = 0.f;
                float i_tex[CPAD];
#pragma unroll
                for (int c = 0; c < CPAD; ++c) i_tex[c] = 0.f;
#pragma unroll
                for (int corner = 0; corner < 4; ++corner)
                {
                    const unsigned j = (word >> (8 * corner)) & 0xFFu;
                    if (j == 0xFFu) continue;
                    const int gx = px + (corner & 1), gy = py + (corner >> 1);
                    float gv[CPAD];
#pragma unroll
                    for (int q = 0; q < CPAD / 4; ++q)
                    {
                        gv[4 * q]     = gq[corner][q].x;
                        gv[4 * q + 1] = gq[corner][q].y;
                        gv[4 * q + 2] = gq[corner][q].z;
                        gv[4 * q + 3] = gq[corner][q].w;
                    }
                    const float grad_alpha = e[corner].x;
                    const float ta         = e[corner].y;
#pragma unroll
                    for (int c = 0; c < C; ++c) i_tex[c] += ta * gv[c];
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
                float4* out = reinterpret_cast<float4*>(s_sums[wave][lane]);
                out[0]      = make_float4(i_conf, i_d0, i_d1, i_size);
#pragma unroll
                for (int q = 0; q < CPAD / 4; ++q) out[1 + q] = make_float4(i_tex[4 * q], i_tex[4 * q + 1], i_tex[4 * q + 2], i_tex[4 * q + 3]);
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
                conf_grad += a.x;
                d0 += a.y;
                d1 += a.z;
                size_grad += a.w;
#pragma unroll
                for (int q = 0; q < CPAD / 4; ++q)
                {
                    const float4 t = in[1 + q];
                    if (4 * q < C) tex_grad[4 * q] += t.x;
                    if (4 * q + 1 < C) tex_grad[4 * q + 1] += t.y;
                    if (4 * q + 2 < C) tex_grad[4 * q + 2] += t.z;
                    if (4 * q + 3 < C) tex_grad[4 * q + 3] += t.w;
                }
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
            project_backward(s_cam.cam, s_cam.R, sp[6], sp[7], sp[8], d0, d1, g_point, g_pose, g_k, g_dis, want_intr);
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

// Before the two passes of the first view. Overwrite mode (`texels`): the descriptor and confidence gradients of the
// columns that the point pass does not write itself. With the identity index (the forward noted it in the header)
// those are the columns past the last point; otherwise all of them, the point pass then adds with atomics.
// `clear_sums`: the block sums that both passes add to (background, every pose row, every intrinsics row).
__global__ __launch_bounds__(256) void zero_texel_grads_kernel(const ViewHeader* __restrict__ header, float* __restrict__ d_texture,
                                                               float* __restrict__ d_confidence, int channels, int num_texels,
                                                               int num_points, int texels, int clear_sums,
                                                               float* __restrict__ d_background, double* __restrict__ d_pose,
                                                               int num_images, float* __restrict__ d_intrinsics, int num_cameras)
{
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
    const int P           = p.geom.bin_off[p.num_layers] * kTilePixels;
    const int N           = p.num_points;
    // (no points: only the background receives gradient)
    if (p.overwrite || p.clear_block_sums)
        hipLaunchKernelGGL(zero_texel_grads_kernel, dim3(p.overwrite ? 1024 : 1), dim3(256), 0, stream, p.header, p.d_texture,
                           p.d_confidence, channels, p.num_texels, N, p.overwrite, p.clear_block_sums, p.d_background, p.d_pose_all,
                           p.num_images, p.d_intrinsics_all, p.num_cameras);
    {
        ProfScope ps(prof, "backward_pixels", stream);
        const long long waves = ((long long)P + 3) / 4;
        long long blocks_ll   = (waves + 3) / 4;
        int blocks            = (int)(blocks_ll < 8192 ? (blocks_ll < 1 ? 1 : blocks_ll) : 8192);
        blocks                = ((blocks + 4 * kNumXcd - 1) / (4 * kNumXcd)) * (4 * kNumXcd);  // whole groups of 8 tiles x 4
        TRIPS_BW_DISPATCH(backward_pixels_kernel, blocks);
    }
    if (N > 0)
    {
        ProfScope ps(prof, "backward_points", stream);
        const int blocks = min((N + 255) / 256, 4096);
        TRIPS_BW_DISPATCH(backward_points_kernel, blocks);
    }
    return hipGetLastError();
}

}  // namespace trips
