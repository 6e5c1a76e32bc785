// Backward kernel of the splat path for gfx950 (wave64).
//
//   blend_backward_kernel <- BlendBackwardsBilinearTiled  src/lib/rendering/RenderBackward.cu:90-618
//
// The reference walks one pixel list per thread, sequentially, re-reading 7 saved floats per entry. Here a
// 16-lane row owns a pixel and each lane owns one retained entry: alpha and transmittance are recomputed from
// the per-point record exactly as the forward computed them, the "all later entries" sum of
// RenderBackward.cu:284-301 becomes a suffix sum across the row, and pose / intrinsics / background partials
// stay in registers (double) over a grid-stride loop before one block-level reduction and one atomic per value
// and block (the reference keeps them in shared double arrays, :160-187,546-617).
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

__device__ __forceinline__ double wave_sum(double v)
{
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

template <int C>
__global__ __launch_bounds__(256) void blend_backward_kernel(const BackwardParams p)
{
    constexpr int CPAD = (C + 3) & ~3;
    constexpr int NACC = 6 + 5 + 8 + C;  // pose, K, distortion, background
    const int lane     = threadIdx.x & 63;
    const int sub      = lane & 15;
    const int grp      = lane >> 4;
    const int P        = p.geom.off[p.num_layers];
    const int K        = p.list_depth;
    const Camera cam   = load_camera_bw(p.pose, p.intrinsics, p.view, p.dist_cutoff);
    float R[9];
    rotation_matrix(cam.V, R);
    const bool want_pose = p.d_pose != nullptr;
    const bool want_intr = p.d_intrinsics != nullptr;
    const bool want_size = p.d_point_size != nullptr;

    double acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = 0.0;

    const long long total_waves  = ((long long)P + 3) / 4;
    const long long wave0        = ((long long)blockIdx.x * 256 + threadIdx.x) >> 6;
    const long long wave_stride  = (long long)gridDim.x * 4;

    for (long long wv = wave0; wv < total_waves; wv += wave_stride)
    {
        const long long pix_ll = wv * 4 + grp;
        const bool live        = pix_ll < P;
        const int pix          = live ? (int)pix_ll : 0;
        int layer              = 0;
        while (layer + 1 < p.num_layers && pix >= p.geom.off[layer + 1]) ++layer;
        const int local = pix - p.geom.off[layer];
        const int lw = p.geom.w[layer], lh = p.geom.h[layer];
        const int gx = local % lw, gy = local / lw;

        const int m    = live ? p.retained[pix] : 0;
        const bool has = sub < m;

        float g[C];
        {
            const float* gi = p.grad_image[layer];
            if (p.layout == TRIPS_LAYOUT_CHW)
            {
                const size_t plane = (size_t)lw * lh;
                const float* o     = gi + ((size_t)p.view_index * C) * plane + (size_t)gy * lw + gx;
#pragma unroll
                for (int c = 0; c < C; ++c) g[c] = live ? o[c * plane] : 0.f;
            }
            else
            {
                const float* o = gi + (((size_t)p.view_index * lh + gy) * lw + gx) * C;
#pragma unroll
                for (int c = 0; c < C; ++c) g[c] = live ? o[c] : 0.f;
            }
        }

        int pid = 0;
        float4 r0 = make_float4(0.f, 0.f, 0.f, 0.f), rv = make_float4(0.f, 0.f, 1.f, 0.f);
        int tex = 0;
        float desc[CPAD];
#pragma unroll
        for (int c = 0; c < CPAD; ++c) desc[c] = 0.f;
        float a = 0.f, ux = 0.f, uy = 0.f;
        if (has)
        {
            pid               = p.lists[(size_t)pix * K + sub];
            const float4* rec = reinterpret_cast<const float4*>(p.rec + (size_t)pid * p.rec_floats);
            r0                = rec[0];
#pragma unroll
            for (int q = 0; q < CPAD / 4; ++q)
            {
                const float4 t  = rec[1 + q];
                desc[4 * q]     = t.x;
                desc[4 * q + 1] = t.y;
                desc[4 * q + 2] = t.z;
                desc[4 * q + 3] = t.w;
            }
            rv                = rec[1 + CPAD / 4];
            tex               = __float_as_int(rec[2 + CPAD / 4].x);
            const float mfac  = 1.f / float(1 << layer);
            ux                = r0.x * mfac;
            uy                = r0.y * mfac;
            float w           = (1.f - fabsf(ux - float(gx))) * (1.f - fabsf(uy - float(gy)));
            if (fabsf(ux - float(gx)) > 1.f || fabsf(uy - float(gy)) > 1.f) w = 0.f;
            a = w * r0.w;
            a *= layer_factor(r0.z, layer, p.num_layers, nullptr);
        }

        // exclusive transmittance, same chain as the forward
        float pre = 1.f, T = 1.f;
#pragma unroll
        for (int s = 1; s < 16; ++s)
        {
            pre = __shfl_up(pre * (1.f - a), 1, 16);
            if (sub == s) T = pre;
        }
        // transmittance after the m retained entries: decides whether the background is reached
        // (RenderBackward.cu:205-210,302-308)
        float T_after = T * (1.f - a);
        T_after       = __shfl(T_after, max(m - 1, 0), 16);
        if (m == 0) T_after = 1.f;
        const bool bg_reached = live && (T_after >= 0.001f);

        // s_j = sum_c colour_c * grad_c ; q_j = T_j a_j s_j
        float s = 0.f, sbg = 0.f;
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            s += desc[c] * g[c];
            sbg += p.background[c] * g[c];
        }
        const float q = has ? (T * a) * s : 0.f;
        // suffix sum over later entries of the row
        float later = __shfl_down(q, 1, 16);  // entries i > j
        if (sub == 15) later = 0.f;
#pragma unroll
        for (int o = 1; o < 16; o <<= 1)
        {
            float t = __shfl_down(later, o, 16);
            if (sub + o < 16) later += t;
        }
        if (bg_reached) later += T_after * sbg;
        const float dem        = 1.f / (1.f - a + 1e-9f);
        const float grad_alpha = T * s - later * dem;

        if (bg_reached && sub == 0)
        {
#pragma unroll
            for (int c = 0; c < C; ++c) acc[19 + c] += (double)(T_after * g[c]);
        }

        if (has)
        {
            // colour gradient (RenderBackward.cu:262-267)
            const float ta = T * a;
#pragma unroll
            for (int c = 0; c < C; ++c) unsafeAtomicAdd(p.d_texture + (size_t)c * p.num_texels + tex, ta * g[c]);

            // geometric part (RenderBackward.cu:334-465)
            const float sx = ux - floorf(ux), sy = uy - floorf(uy);
            const int x_i  = float(gx) < ux ? 0 : 1;
            const int y_i  = float(gy) < uy ? 0 : 2;
            const int bi   = y_i + x_i;
            float blend, J0, J1;
            switch (bi)
            {
                case 0: blend = (1.f - sx) * (1.f - sy); J0 = sy - 1.f; J1 = sx - 1.f; break;
                case 1: blend = sx * (1.f - sy); J0 = 1.f - sy; J1 = -sx; break;
                case 2: blend = (1.f - sx) * sy; J0 = -sy; J1 = 1.f - sx; break;
                default: blend = sx * sy; J0 = sy; J1 = sx; break;
            }
            if (fabsf(ux - float(gx)) > 1.f || fabsf(uy - float(gy)) > 1.f) blend *= 0.f;
            const float conf = r0.w;
            float lfac = 1.f, J_lf = 0.f;
            if (want_size) lfac = layer_factor(r0.z, layer, p.num_layers, &J_lf);
            unsafeAtomicAdd(p.d_confidence + tex, blend * lfac * grad_alpha);

            const float gbs = conf * lfac * grad_alpha;
            float g_point[3], g_pose[6], g_k[5], g_dis[8];
            project_backward(cam, R, rv.x, rv.y, rv.z, J0 * gbs, J1 * gbs, g_point, g_pose, g_k, g_dis, want_intr);
            if (want_size)
            {
                const float J_softmax_proj = cam.fx * cam.cfx / fmaxf(rv.z, 0.f);
                const float grad_layer_ps  = rv.w * J_softmax_proj * J_lf * grad_alpha;
                unsafeAtomicAdd(p.d_point_size + pid, blend * conf * grad_layer_ps);
            }
            if (p.d_position)
            {
                float* dp = p.d_position + 4 * (size_t)pid;
                unsafeAtomicAdd(dp + 0, g_point[0]);
                unsafeAtomicAdd(dp + 1, g_point[1]);
                unsafeAtomicAdd(dp + 2, g_point[2]);
            }
            if (want_pose)
            {
#pragma unroll
                for (int k = 0; k < 6; ++k) acc[k] += (double)g_pose[k];
            }
            if (want_intr)
            {
#pragma unroll
                for (int k = 0; k < 5; ++k) acc[6 + k] += (double)g_k[k];
#pragma unroll
                for (int k = 0; k < 8; ++k) acc[11 + k] += (double)g_dis[k];
            }
        }
    }

    // block reduction, one atomic per value and block
    __shared__ double s_acc[4][NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i)
    {
        const bool used = (i < 6) ? want_pose : (i < 19 ? want_intr : true);
        if (!used) continue;
        double v = wave_sum(acc[i]);
        if (lane == 0) s_acc[threadIdx.x >> 6][i] = v;
    }
    __syncthreads();
    if (threadIdx.x < NACC)
    {
        const int i     = threadIdx.x;
        const bool used = (i < 6) ? want_pose : (i < 19 ? want_intr : true);
        if (used)
        {
            double v = s_acc[0][i] + s_acc[1][i] + s_acc[2][i] + s_acc[3][i];
            if (v != 0.0)
            {
                if (i < 6)
                    unsafeAtomicAdd(p.d_pose + i, v);
                else if (i < 19)
                    unsafeAtomicAdd(p.d_intrinsics + (i - 6), (float)v);
                else
                    unsafeAtomicAdd(p.d_background + (i - 19), (float)v);
            }
        }
    }
}

hipError_t launch_backward_view(const BackwardParams& p, int channels, hipStream_t stream, Profiler* prof)
{
    ProfScope ps(prof, "blend_backward", stream);
    const int P            = p.geom.off[p.num_layers];
    const long long waves  = ((long long)P + 3) / 4;
    long long blocks_ll    = (waves + 3) / 4;
    const int blocks       = (int)(blocks_ll < 2048 ? (blocks_ll < 1 ? 1 : blocks_ll) : 2048);
    switch (channels)
    {
        case 3: hipLaunchKernelGGL((blend_backward_kernel<3>), dim3(blocks), dim3(256), 0, stream, p); break;
        case 4: hipLaunchKernelGGL((blend_backward_kernel<4>), dim3(blocks), dim3(256), 0, stream, p); break;
        case 6: hipLaunchKernelGGL((blend_backward_kernel<6>), dim3(blocks), dim3(256), 0, stream, p); break;
        case 8: hipLaunchKernelGGL((blend_backward_kernel<8>), dim3(blocks), dim3(256), 0, stream, p); break;
        case 16: hipLaunchKernelGGL((blend_backward_kernel<16>), dim3(blocks), dim3(256), 0, stream, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace trips
