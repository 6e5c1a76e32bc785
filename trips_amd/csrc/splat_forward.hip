// Forward kernels of the splat path for gfx950 (wave64).
//
//   project_count_kernel   <- CountAndCollectTiled     src/lib/rendering/RenderForward.cu:168-366
//   scan_*_kernel          <- cub ExclusiveSum section src/lib/rendering/RenderForward.cu:1155-1232
//   scatter_keys_kernel    <- SplattingPass            src/lib/rendering/RenderForward.cu:368-436
//   sort_blend_kernel      <- FastSortFusedNew         src/lib/rendering/RenderForward.cu:474-1059
//
// Differences in shape, not in result: all pyramid layers share ONE counter array and ONE scan (the reference
// scans layer by layer with two blocking read-backs each); a wavefront holds four pixel lists of 16 lanes
// (one DPP row each) instead of two per 32-lane warp; the per-point record gathered by the blend carries
// position, size, confidence and descriptor together; what is kept for the backward is the sorted id list
// per pixel (64 B) instead of 16 x 7 floats.
#include "splat_internal.h"
#include "trips_math.h"

#pragma clang fp contract(off)

namespace trips
{
using u64 = unsigned long long;

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
    for (int i = 0; i < 8; ++i) c.dist[i] = intr[5 + i];
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

__global__ __launch_bounds__(256) void fill_i32_kernel(int32_t* __restrict__ p, int32_t v, long long n)
{
    long long i      = (long long)blockIdx.x * 256 + threadIdx.x;
    long long stride = (long long)gridDim.x * 256;
    for (; i < n; i += stride) p[i] = v;
}

__global__ void clear_header_kernel(ViewHeader* h)
{
    if (threadIdx.x == 0)
    {
        h->n_valid   = 0;
        h->n_entries = 0;
        h->overflow  = 0;
        for (int i = 0; i < 5; ++i) h->reserved[i] = 0;
    }
}

// ---------------------------------------------------------------------------------------------------------
// Projection, validity, layer selection, per-pixel counting. One point per thread, grid-stride.
template <int C, bool TRAIN>
__global__ __launch_bounds__(256) void project_count_kernel(const ForwardParams p)
{
    constexpr int CPAD = (C + 3) & ~3;
    const Camera cam   = load_camera(p.pose, p.intrinsics, p.view, p.dist_cutoff);
    const int L        = p.num_layers;
    unsigned my_valid  = 0;
    bool not_identity  = false;  // some point's descriptor column differs from its own index

    for (int pid = blockIdx.x * 256 + threadIdx.x; pid < p.num_points; pid += gridDim.x * 256)
    {
        float4 ptk  = make_float4(0.f, 0.f, -1.f, 0.f);
        bool skip   = false;
        const int tex = p.index[pid];
        not_identity |= (tex != pid);
        if (p.viewer_only)
        {
            if (p.confidence[tex] < p.stability_cutoff_value) skip = true;
        }
        if (TRAIN && p.dropout)
        {
            if (p.dropout[pid] == 1.f) skip = true;
        }
        if (!skip)
        {
            const float4 pos = p.position[pid];
            const float size = softplus(p.point_size[pid]);
            const Projected pr = project(cam, pos.x, pos.y, pos.z);
            const float z      = pr.z;
            float radius_px    = pr.scale * pos.w / z;
            const float size_px = pr.scale * size / z;
            float ipx = pr.ipx, ipy = pr.ipy;

            auto valid = [&](float x, float y, int layer, float radius) -> bool
            {
                if (z <= 0.f) return false;
                if (!(x >= 0.f) || x >= float(p.geom.w[layer] - 1) || !(y >= 0.f) || y >= float(p.geom.h[layer] - 1))
                    return false;
                if (p.drop_out_points_by_radius && float(trunc_sat(radius)) < p.drop_out_radius_threshold)
                    return false;
                return true;
            };

            if (valid(ipx, ipy, 0, radius_px))
            {
                my_valid += 1;
                int layer_higher = 0;
                if (size_px > 1.f)
                {
                    int lo, hi;
                    log2_floor_ceil(size_px, lo, hi);
                    layer_higher = min(hi, L - 1);
                }
                int layer = 0;
                float lx = ipx, ly = ipy;
                for (; layer < layer_higher + 1; ++layer, lx *= 0.5f, ly *= 0.5f, radius_px *= 0.5f)
                {
                    const int px = (int)floorf(lx), py = (int)floorf(ly);
                    if (!valid(float(px), float(py), layer, radius_px)) break;
                    int32_t* base = p.counts + p.geom.off[layer] + py * p.geom.w[layer] + px;
                    atomicAdd(base, 1);
                    atomicAdd(base + 1, 1);
                    atomicAdd(base + p.geom.w[layer], 1);
                    atomicAdd(base + p.geom.w[layer] + 1, 1);
                }
                ptk = make_float4(ipx, ipy, z, __int_as_float(layer));

                // record for blend (+ backward)
                float4* rec = reinterpret_cast<float4*>(p.rec + (size_t)pid * p.rec_floats);
                rec[0]      = make_float4(ipx, ipy, size_px, p.confidence[tex]);
                float d[CPAD];
#pragma unroll
                for (int c = 0; c < CPAD; ++c) d[c] = c < C ? p.texture[(size_t)c * p.num_texels + tex] : 0.f;
#pragma unroll
                for (int q = 0; q < CPAD / 4; ++q) rec[1 + q] = make_float4(d[4 * q], d[4 * q + 1], d[4 * q + 2], d[4 * q + 3]);
                if (TRAIN)
                {
                    rec[1 + CPAD / 4] = make_float4(pr.vx, pr.vy, pr.vz, softplus_backward(p.point_size[pid]));
                    rec[2 + CPAD / 4] = make_float4(__int_as_float(tex), z, __int_as_float(layer), 0.f);
                }
            }
        }
        if (TRAIN && !(ptk.z > 0.f))
        {
            // culled: only the tail {texture index, depth = -1, layers = 0} is defined
            float4* rec       = reinterpret_cast<float4*>(p.rec + (size_t)pid * p.rec_floats);
            rec[2 + CPAD / 4] = make_float4(__int_as_float(tex), -1.f, __int_as_float(0), 0.f);
        }
        p.ptk[pid] = ptk;
    }

    // one counter update per block
    __shared__ unsigned s_valid[4];
    unsigned v = my_valid;
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    if ((threadIdx.x & 63) == 0) s_valid[threadIdx.x >> 6] = v;
    __syncthreads();
    if (threadIdx.x == 0)
    {
        unsigned t = s_valid[0] + s_valid[1] + s_valid[2] + s_valid[3];
        if (t) atomicAdd(&p.header->n_valid, (u64)t);
    }
    if (__ballot(not_identity) != 0 && (threadIdx.x & 63) == 0) atomicOr(&p.header->reserved[1], 1ull);
}

// ---------------------------------------------------------------------------------------------------------
// Exclusive scan of the P per-pixel counts (all layers concatenated): reduce, spine, apply.
__device__ __forceinline__ int block_reduce_sum(int v, int* smem)
{
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = v;
    __syncthreads();
    int t = 0;
    for (unsigned i = 0; i < blockDim.x / 64; ++i) t += smem[i];
    __syncthreads();
    return t;
}

__global__ __launch_bounds__(256) void scan_reduce_kernel(const int32_t* __restrict__ counts, int32_t* __restrict__ block_sums,
                                                          int n)
{
    __shared__ int smem[4];
    const int base = blockIdx.x * kScanTile;
    int s          = 0;
    for (int i = threadIdx.x; i < kScanTile; i += 256)
    {
        int idx = base + i;
        if (idx < n) s += counts[idx];
    }
    s = block_reduce_sum(s, smem);
    if (threadIdx.x == 0) block_sums[blockIdx.x] = s;
}

// single block: exclusive scan of the block sums in place, total to the header
__global__ __launch_bounds__(1024) void scan_spine_kernel(int32_t* __restrict__ block_sums, int nb, ViewHeader* header)
{
    __shared__ int s_wave[16];
    __shared__ int s_carry;
    if (threadIdx.x == 0) s_carry = 0;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int base = 0; base < nb; base += 1024)
    {
        int idx = base + threadIdx.x;
        int v   = idx < nb ? block_sums[idx] : 0;
        int inc = v;
        for (int o = 1; o < 64; o <<= 1)
        {
            int t = __shfl_up(inc, o);
            if (lane >= o) inc += t;
        }
        if (lane == 63) s_wave[wave] = inc;
        __syncthreads();
        int wave_prefix = 0;
        for (int w = 0; w < wave; ++w) wave_prefix += s_wave[w];
        int carry = s_carry;
        if (idx < nb) block_sums[idx] = carry + wave_prefix + inc - v;
        __syncthreads();
        if (threadIdx.x == 1023) s_carry = carry + wave_prefix + inc;
        __syncthreads();
    }
    if (threadIdx.x == 0) header->n_entries = (u64)(unsigned)s_carry;
}

__global__ __launch_bounds__(256) void scan_apply_kernel(const int32_t* __restrict__ counts,
                                                         const int32_t* __restrict__ block_sums,
                                                         int32_t* __restrict__ cursor, int n)
{
    __shared__ int s_wave[4];
    constexpr int PER = kScanTile / 256;  // 16 consecutive elements per thread
    const int base    = blockIdx.x * kScanTile + threadIdx.x * PER;
    int v[PER];
    int sum = 0;
#pragma unroll
    for (int i = 0; i < PER; ++i)
    {
        int idx = base + i;
        v[i]    = idx < n ? counts[idx] : 0;
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
    __syncthreads();
    int prefix = block_sums[blockIdx.x] + inc - sum;
    for (int w = 0; w < wave; ++w) prefix += s_wave[w];
#pragma unroll
    for (int i = 0; i < PER; ++i)
    {
        int idx = base + i;
        if (idx < n) cursor[idx] = prefix;
        prefix += v[i];
    }
}

// ---------------------------------------------------------------------------------------------------------
// 64-bit keys (depth bits << 32 | point id) into the pixel lists. Thread = (point, corner).
__global__ __launch_bounds__(256) void scatter_keys_kernel(const ForwardParams p)
{
    const long long tid = (long long)blockIdx.x * 256 + threadIdx.x;
    const int pid       = int(tid >> 2);
    const int sub       = int(tid & 3);
    if (pid >= p.num_points) return;
    const float4 k = p.ptk[pid];
    const float z  = k.z;
    if (!(z > 0.f)) return;
    const int max_layer = __float_as_int(k.w);
    const u64 key       = ((u64)__float_as_uint(z) << 32) | (u64)(unsigned)pid;
    float lx = k.x, ly = k.y;
    unsigned dropped = 0;
    for (int layer = 0; layer < max_layer; ++layer)
    {
        const int px = (int)floorf(lx) + (sub & 1), py = (int)floorf(ly) + (sub >> 1);
        const int pix  = p.geom.off[layer] + py * p.geom.w[layer] + px;
        const int slot = atomicAdd(p.cursor + pix, 1);
        if ((long long)slot < p.capacity)
            p.keys[slot] = key;
        else
            dropped += 1;
        lx *= 0.5f;
        ly *= 0.5f;
    }
    if (dropped) atomicAdd(&p.status->overflow, (u64)dropped);
}

// ---------------------------------------------------------------------------------------------------------
// 16-lane (one DPP row) primitives. Every group of 16 lanes is either fully active or fully inactive
// wherever these are called.
__device__ __forceinline__ u64 shfl_xor16(u64 v, int m)
{
    unsigned lo = (unsigned)v, hi = (unsigned)(v >> 32);
    lo = __shfl_xor(lo, m, 16);
    hi = __shfl_xor(hi, m, 16);
    return ((u64)hi << 32) | lo;
}

__device__ __forceinline__ u64 shfl16(u64 v, int src)
{
    unsigned lo = (unsigned)v, hi = (unsigned)(v >> 32);
    lo = __shfl(lo, src, 16);
    hi = __shfl(hi, src, 16);
    return ((u64)hi << 32) | lo;
}

// ascending bitonic sort of 16 keys, one per lane of the row
__device__ __forceinline__ u64 sort16(u64 v, int sub)
{
#pragma unroll
    for (int k = 2; k <= 16; k <<= 1)
    {
#pragma unroll
        for (int j = k >> 1; j > 0; j >>= 1)
        {
            const u64 o      = shfl_xor16(v, j);
            const bool up    = (sub & k) == 0 || k == 16;
            const bool lower = (sub & j) == 0;
            const u64 mn = v < o ? v : o, mx = v < o ? o : v;
            v = (lower == up) ? mn : mx;
        }
    }
    return v;
}

// v is bitonic over the row: ascending merge
__device__ __forceinline__ u64 merge16(u64 v, int sub)
{
#pragma unroll
    for (int j = 8; j > 0; j >>= 1)
    {
        const u64 o      = shfl_xor16(v, j);
        const bool lower = (sub & j) == 0;
        const u64 mn = v < o ? v : o, mx = v < o ? o : v;
        v = lower ? mn : mx;
    }
    return v;
}

// Top-16 of each pixel list by key, then the alpha blend. One wavefront = four pixels, 16 lanes each.
template <int C, bool TRAIN>
__global__ __launch_bounds__(256) void sort_blend_kernel(const ForwardParams p)
{
    constexpr int CPAD = (C + 3) & ~3;
    const int lane     = threadIdx.x & 63;
    const int sub      = lane & 15;
    const int grp      = lane >> 4;
    const int P        = p.geom.off[p.num_layers];
    const int K        = p.list_depth;
    const long long wave_global = ((long long)blockIdx.x * 256 + threadIdx.x) >> 6;
    const long long pix_ll      = wave_global * 4 + grp;
    const bool live             = pix_ll < P;
    const int pix               = live ? (int)pix_ll : 0;

    int len = 0, end = 0;
    if (live)
    {
        len = p.counts[pix];
        end = p.cursor[pix];
    }
    const long long start = (long long)end - len;
    // entries beyond the capacity were never written
    int readable = len;
    if (start + len > p.capacity) readable = (int)max(0ll, p.capacity - start);

    int maxlen = readable;
    maxlen     = max(maxlen, __shfl_xor(maxlen, 16));
    maxlen     = max(maxlen, __shfl_xor(maxlen, 32));

    const u64 kInf      = ~0ull;
    const u64 grp_mask  = 0xFFFFull << (grp * 16);
    u64 best            = kInf;
    for (int base = 0; base < maxlen; base += 16)
    {
        u64 k = kInf;
        if (base + sub < readable) k = p.keys[start + base + sub];
        if (base == 0)
        {
            best = sort16(k, sub);
        }
        else
        {
            const u64 worst = shfl16(best, 15);
            const bool need = k < worst;
            if (__ballot(need) & grp_mask)
            {
                k           = sort16(k, sub);
                const u64 r = shfl_xor16(k, 15);  // reversed: lane i sees the (15-i)-th smallest new key
                best        = best < r ? best : r;
                best        = merge16(best, sub);
            }
        }
    }

    // ---- blend (RenderForward.cu:820-1048) ----
    int layer = 0;
    while (layer + 1 < p.num_layers && pix >= p.geom.off[layer + 1]) ++layer;
    const int local = pix - p.geom.off[layer];
    const int lw = p.geom.w[layer], lh = p.geom.h[layer];
    const int gx = local % lw, gy = local / lw;

    const int n    = min(min(len, readable), K);
    const bool has = live && sub < n;
    const int pid  = (int)(unsigned)(best & 0xffffffffull);

    float a = 0.f;
    float desc[CPAD];
#pragma unroll
    for (int c = 0; c < CPAD; ++c) desc[c] = 0.f;
    if (has)
    {
        const float4* rec = reinterpret_cast<const float4*>(p.rec + (size_t)pid * p.rec_floats);
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
        const float m  = 1.f / float(1 << layer);
        const float ux = r0.x * m, uy = r0.y * m;
        float w        = (1.f - fabsf(ux - float(gx))) * (1.f - fabsf(uy - float(gy)));
        if (fabsf(ux - float(gx)) > 1.f || fabsf(uy - float(gy)) > 1.f) w = 0.f;
        a = w * r0.w;
        a *= layer_factor(r0.z, layer, p.num_layers, nullptr);
    }

    // exclusive transmittance: lane j latches prod_{k<j} (1 - a_k), built left to right
    float pre = 1.f, T = 1.f;
#pragma unroll
    for (int s = 1; s < 16; ++s)
    {
        pre = __shfl_up(pre * (1.f - a), 1, 16);
        if (sub == s) T = pre;
    }
    const float Tc    = (T >= kAlphaDestCutoff) ? T : 0.f;
    const bool kept   = has && Tc >= kAlphaDestCutoff;
    const unsigned kb = (unsigned)((__ballot(kept) >> (grp * 16)) & 0xFFFFull);
    const int ret     = __ffs(~kb) - 1;  // length of the leading run of kept entries (kb has at most 16 bits)

    float col[C];
    const float wgt = has ? Tc * a : 0.f;
#pragma unroll
    for (int c = 0; c < C; ++c) col[c] = wgt * desc[c];
#pragma unroll
    for (int o = 1; o < 16; o <<= 1)
    {
#pragma unroll
        for (int c = 0; c < C; ++c) col[c] = col[c] + __shfl_xor(col[c], o, 16);
    }

    // background weight (RenderForward.cu:1002-1022); empty list -> 1
    float bgw_lane = (p.background_mode == TRIPS_BG_REFERENCE) ? Tc : T * (1.f - a);
    float bgw      = __shfl(bgw_lane, max(n - 1, 0), 16);
    if (n == 0) bgw = 1.f;

    if (live && sub == 0)
    {
        if (bgw >= kAlphaDestCutoff)
        {
#pragma unroll
            for (int c = 0; c < C; ++c) col[c] += p.background[c] * (bgw * 1.f);
        }
        float* img = p.image[layer];
        if (p.layout == TRIPS_LAYOUT_CHW)
        {
            const size_t plane = (size_t)lw * lh;
            float* o           = img + ((size_t)p.view_index * C) * plane + (size_t)gy * lw + gx;
#pragma unroll
            for (int c = 0; c < C; ++c) o[c * plane] = col[c];
        }
        else
        {
            float* o = img + (((size_t)p.view_index * lh + gy) * lw + gx) * C;
#pragma unroll
            for (int c = 0; c < C; ++c) o[c] = col[c];
        }
        if (TRAIN)
        {
            p.retained[pix] = ret;
            p.lengths[pix]  = len;
        }
    }
    if (TRAIN && live && sub < K) p.lists[(size_t)pix * K + sub] = has ? pid : -1;
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
    const int P  = p.geom.off[p.num_layers];
    const int N  = p.num_points;
    const int nb = (P + kScanTile - 1) / kScanTile;

    if (first_view) hipLaunchKernelGGL(clear_header_kernel, dim3(1), dim3(64), 0, stream, p.status);
    hipLaunchKernelGGL(clear_header_kernel, dim3(1), dim3(64), 0, stream, p.header);
    {
        ProfScope ps(prof, "fill_counts", stream);
        int blocks = (int)min((long long)(P + 255) / 256, 4096ll);
        hipLaunchKernelGGL(fill_i32_kernel, dim3(max(blocks, 1)), dim3(256), 0, stream, p.counts, 0, (long long)P);
    }
    if (N > 0)
    {
        ProfScope ps(prof, "project_count", stream);
        int blocks = min((N + 255) / 256, 2048);
        if (train)
        {
            TRIPS_DISPATCH_C(channels, hipLaunchKernelGGL((project_count_kernel<CC, true>), dim3(blocks), dim3(256), 0, stream, p));
        }
        else
        {
            TRIPS_DISPATCH_C(channels, hipLaunchKernelGGL((project_count_kernel<CC, false>), dim3(blocks), dim3(256), 0, stream, p));
        }
    }
    {
        ProfScope ps(prof, "scan", stream);
        hipLaunchKernelGGL(scan_reduce_kernel, dim3(nb), dim3(256), 0, stream, p.counts, p.block_sums, P);
        hipLaunchKernelGGL(scan_spine_kernel, dim3(1), dim3(1024), 0, stream, p.block_sums, nb, p.header);
        hipLaunchKernelGGL(scan_apply_kernel, dim3(nb), dim3(256), 0, stream, p.counts, p.block_sums, p.cursor, P);
    }
    if (N > 0)
    {
        ProfScope ps(prof, "scatter_keys", stream);
        long long threads = 4ll * N;
        int blocks        = (int)((threads + 255) / 256);
        hipLaunchKernelGGL(scatter_keys_kernel, dim3(blocks), dim3(256), 0, stream, p);
    }
    {
        ProfScope ps(prof, "sort_blend", stream);
        long long waves = ((long long)P + 3) / 4;
        int blocks      = (int)((waves + 3) / 4);
        if (train)
        {
            TRIPS_DISPATCH_C(channels, hipLaunchKernelGGL((sort_blend_kernel<CC, true>), dim3(blocks), dim3(256), 0, stream, p));
        }
        else
        {
            TRIPS_DISPATCH_C(channels, hipLaunchKernelGGL((sort_blend_kernel<CC, false>), dim3(blocks), dim3(256), 0, stream, p));
        }
    }
    return hipGetLastError();
}

}  // namespace trips
