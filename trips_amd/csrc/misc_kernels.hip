// Fused multi-tensor Adam, pose update, and the small export / reduction kernels of the C ABI (gfx950).
//
//   adam_fused_kernel    <- adam_step      src/lib/models/MyAdam.cu:41-88 (one launch for all tensors instead of
//                                          one 128-thread launch per tensor, :226-288)
//   adam_points_kernel   <- the same step for the four tensors of a point cloud, optimiser state packed per point
//   apply_tangent_kernel <- ApplyTangent   src/lib/rendering/PointRenderer.cu:1428-1447
#include <float.h>

#include "splat_internal.h"
#include "trips_math.h"

#pragma clang fp contract(off)

namespace trips
{
constexpr int kAdamMaxTensors = 16;
constexpr int kAdamPerBlock   = 1024;  // 256 threads x 4 consecutive elements

struct AdamTable
{
    TripsAdamTensor t[kAdamMaxTensors];
    long long block_start[kAdamMaxTensors + 1];
    int32_t vec_ok[kAdamMaxTensors];
    int32_t n;
};

struct AdamScalars
{
    float lr, beta1, beta2, eps, rel_wd, abs_wd, clip, lo, hi, loss_scale;
};

// beta^t for a step count t: by squaring in double precision, rounded to float once. (The library powf is some 400
// instructions, and two of them per point were half of the packed kernel's work. The squarings' error doubles per
// squaring from 2^-53: below a float's for any t < 2^28, and beta^t of a beta < 1 is zero long before that.)
__device__ __forceinline__ float pow_step(float beta, uint32_t t)
{
    double r = 1.0, b = (double)beta;
    while (t)
    {
        if (t & 1u) r *= b;
        b *= b;
        t >>= 1;
    }
    return (float)r;
}

// learning rate with the bias correction of step `current_step` (MyAdam.cu:66-68)
__device__ __forceinline__ float adam_corrected_lr(const AdamScalars& h, uint32_t current_step)
{
    float learning_rate = h.lr;
    learning_rate *= sqrtf(1 - pow_step(h.beta2, current_step)) / (1 - pow_step(h.beta1, current_step));
    return learning_rate;
}

// `lr_of_step`: the corrected learning rate of step `lr_step`, if the caller has it already (two powf, a square root
// and a division that elements with equal counters share); lr_step = 0 for none.
__device__ __forceinline__ bool adam_element(const AdamScalars& h, float gradient_raw, float weight_fp, float& m,
                                             float& v, long long& step, float& new_weight, uint32_t lr_step = 0,
                                             float lr_of_step = 0.f)
{
    float gradient = gradient_raw;
    if (h.loss_scale != 1.f) gradient = gradient_raw / h.loss_scale;  // (a division by 1 changes nothing: skipped)
    if (gradient == 0.f) return false;  // parameter not seen in this step (MyAdam.cu:57-61)
    const float gradient_sq   = gradient * gradient;
    const float first_moment  = h.beta1 * m + (1 - h.beta1) * gradient;
    const float second_moment = h.beta2 * v + (1 - h.beta2) * gradient_sq;
    m                         = first_moment;
    v                         = second_moment;
    step                      = step + 1;
    const uint32_t current_step = (uint32_t)step;
    float learning_rate         = lr_of_step;
    if (current_step != lr_step) learning_rate = adam_corrected_lr(h, current_step);
    const float effective_learning_rate =
        fminf(fmaxf(learning_rate / (sqrtf(second_moment) + h.eps), h.lo), h.hi);
    const float rel            = h.rel_wd * learning_rate;
    const float ab             = h.abs_wd * learning_rate;
    const float decayed_weight = (1 - rel) * weight_fp - copysignf(ab, weight_fp);
    float w                    = decayed_weight - effective_learning_rate * first_moment;
    if (h.clip != 0.0f)
    {
        const float lo = -h.clip, hi = h.clip;
        w = w < lo ? lo : (hi < w ? hi : w);
    }
    new_weight = w;
    return true;
}

// STEP = long long (the reference's state tensor) or int
template <typename STEP>
__device__ __forceinline__ void adam_block(const AdamTable& tab, int ti)
{
    const TripsAdamTensor& T = tab.t[ti];
    const AdamScalars h      = {T.lr, T.beta1, T.beta2, T.eps, T.relative_weight_decay, T.absolute_weight_decay,
                                T.weight_clipping_magnitude, T.lower_lr_bound, T.upper_lr_bound, T.loss_scale};
    const long long i0 = ((long long)blockIdx.x - tab.block_start[ti]) * kAdamPerBlock + (long long)threadIdx.x * 4;
    if (i0 >= T.n) return;
    float* mo = T.first_moment;
    float* vo = T.second_moment;
    STEP* st  = reinterpret_cast<STEP*>(T.steps);

    if (T.dtype == TRIPS_DTYPE_F32 && tab.vec_ok[ti] && i0 + 4 <= T.n)
    {
        float* w       = reinterpret_cast<float*>(T.weights);
        const float* g = reinterpret_cast<const float*>(T.grads);
        const float4 g4 = *reinterpret_cast<const float4*>(g + i0);
        if (g4.x == 0.f && g4.y == 0.f && g4.z == 0.f && g4.w == 0.f) return;
        float4 w4 = *reinterpret_cast<const float4*>(w + i0);
        float4 m4 = *reinterpret_cast<const float4*>(mo + i0);
        float4 v4 = *reinterpret_cast<const float4*>(vo + i0);
        STEP s[4];
        if (sizeof(STEP) == 8)
        {
            *reinterpret_cast<longlong2*>(&s[0]) = *reinterpret_cast<const longlong2*>(st + i0);
            *reinterpret_cast<longlong2*>(&s[2]) = *reinterpret_cast<const longlong2*>(st + i0 + 2);
        }
        else
            *reinterpret_cast<int4*>(&s[0]) = *reinterpret_cast<const int4*>(st + i0);
        long long s0 = s[0], s1 = s[1], s2 = s[2], s3 = s[3];
        // The four elements are mostly updated together, so their counters agree: the bias correction (two powf, a square
        // root, a division) of the run's largest counter is computed once and taken by every element whose new counter
        // equals it.
        const uint32_t top = (uint32_t)max(max(s0, s1), max(s2, s3)) + 1u;
        const float top_lr = adam_corrected_lr(h, top);
        float nw;
        if (adam_element(h, g4.x, w4.x, m4.x, v4.x, s0, nw, top, top_lr)) w4.x = nw;
        if (adam_element(h, g4.y, w4.y, m4.y, v4.y, s1, nw, top, top_lr)) w4.y = nw;
        if (adam_element(h, g4.z, w4.z, m4.z, v4.z, s2, nw, top, top_lr)) w4.z = nw;
        if (adam_element(h, g4.w, w4.w, m4.w, v4.w, s3, nw, top, top_lr)) w4.w = nw;
        s[0] = (STEP)s0, s[1] = (STEP)s1, s[2] = (STEP)s2, s[3] = (STEP)s3;
        *reinterpret_cast<float4*>(w + i0)  = w4;
        *reinterpret_cast<float4*>(mo + i0) = m4;
        *reinterpret_cast<float4*>(vo + i0) = v4;
        if (sizeof(STEP) == 8)
        {
            *reinterpret_cast<longlong2*>(st + i0)     = *reinterpret_cast<longlong2*>(&s[0]);
            *reinterpret_cast<longlong2*>(st + i0 + 2) = *reinterpret_cast<longlong2*>(&s[2]);
        }
        else
            *reinterpret_cast<int4*>(st + i0) = *reinterpret_cast<int4*>(&s[0]);
        return;
    }
    for (int k = 0; k < 4; ++k)
    {
        const long long i = i0 + k;
        if (i >= T.n) break;
        float gr, wf;
        if (T.dtype == TRIPS_DTYPE_F64)
        {
            gr = (float)reinterpret_cast<const double*>(T.grads)[i];
            wf = (float)reinterpret_cast<double*>(T.weights)[i];
        }
        else
        {
            gr = reinterpret_cast<const float*>(T.grads)[i];
            wf = reinterpret_cast<float*>(T.weights)[i];
        }
        float m = mo[i], v = vo[i], nw;
        long long s = st[i];
        if (adam_element(h, gr, wf, m, v, s, nw))
        {
            mo[i] = m;
            vo[i] = v;
            st[i] = (STEP)s;
            if (T.dtype == TRIPS_DTYPE_F64)
                reinterpret_cast<double*>(T.weights)[i] = nw;
            else
                reinterpret_cast<float*>(T.weights)[i] = nw;
        }
    }
}

__global__ __launch_bounds__(256) void adam_fused_kernel(const AdamTable tab)
{
    int ti = 0;
    while (ti + 1 < tab.n && (long long)blockIdx.x >= tab.block_start[ti + 1]) ++ti;
    if (tab.t[ti].steps_dtype == TRIPS_STEPS_I32)
        adam_block<int>(tab, ti);
    else
        adam_block<long long>(tab, ti);
}

hipError_t launch_adam(const TripsAdamTensor* tensors, int n_tensors, hipStream_t stream, Profiler* prof)
{
    ProfScope ps(prof, "adam_fused", stream);
    int done = 0;
    while (done < n_tensors)
    {
        AdamTable tab;
        tab.n           = 0;
        long long block = 0;
        while (done < n_tensors && tab.n < kAdamMaxTensors)
        {
            const TripsAdamTensor& T = tensors[done++];
            if (T.n <= 0) continue;
            tab.t[tab.n]           = T;
            tab.block_start[tab.n] = block;
            auto al16              = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
            tab.vec_ok[tab.n] = al16(T.weights) && al16(T.grads) && al16(T.first_moment) && al16(T.second_moment) &&
                                al16(T.steps);
            block += (T.n + kAdamPerBlock - 1) / kAdamPerBlock;
            tab.n += 1;
        }
        tab.block_start[tab.n] = block;
        if (tab.n == 0 || block == 0) continue;
        if (block > 0x7fffffffll) return hipErrorInvalidValue;
        hipLaunchKernelGGL(adam_fused_kernel, dim3((unsigned)block), dim3(256), 0, stream, tab);
    }
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------------
// The four parameter tensors of a point cloud (position [N,4], size [N], descriptors [C,N], confidence [N]) stepped
// together, with the optimiser state packed per point: one row of CHUNKS x 16 bytes holding {first moment, second
// moment, step counter} of the point's 6 + C elements (position xyzw, size, descriptors, confidence). A point that
// was not seen has zero gradients everywhere and is skipped as a whole (MyAdam.cu:57-61 per element): with per-tensor
// state arrays its state shares every line with its neighbours' and travels anyway; packed, the row of a point that
// is skipped is never touched. Same arithmetic per element as adam_fused_kernel.
// One thread per point. The rows of a wavefront's live points pass through LDS so that the accesses to memory stay
// whole lines: 64 / CHUNKS rows per load instruction, lane = (row, 16-byte chunk).
struct AdamPointsParams
{
    float *w_pos, *w_size, *w_tex, *w_conf;
    const float *g_pos, *g_size, *g_tex, *g_conf;
    uint4* state;  // [N][CHUNKS]
    long long tex_stride;  // elements between two descriptor rows
    int num_points;
    AdamScalars h[4];  // position, size, descriptors, confidence
};

template <int C, int CHUNKS>
__global__ __launch_bounds__(256) void adam_points_kernel(const AdamPointsParams p)
{
    constexpr int E   = 6 + C;
    constexpr int LS  = CHUNKS + 1;  // LDS row stride in 16-byte words: an odd multiple spreads the rows over the banks
    constexpr int RPP = 64 / CHUNKS;  // rows per load instruction
    static_assert(3 * E <= 4 * CHUNKS, "row too short");
    __shared__ uint4 s_rows[4][64 * LS];
    __shared__ unsigned char s_list[4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long long first = (long long)blockIdx.x * 256 + wave * 64;  // first point of this wavefront
    const long long point = first + lane;
    const bool in         = point < p.num_points;
    float g[E];
    {
        const float4 gp = in ? reinterpret_cast<const float4*>(p.g_pos)[point] : make_float4(0.f, 0.f, 0.f, 0.f);
        g[0] = gp.x, g[1] = gp.y, g[2] = gp.z, g[3] = gp.w;
        g[4] = in ? p.g_size[point] : 0.f;
#pragma unroll
        for (int c = 0; c < C; ++c) g[5 + c] = in ? p.g_tex[c * p.tex_stride + point] : 0.f;
        g[5 + C] = in ? p.g_conf[point] : 0.f;
    }
    bool live = false;
#pragma unroll
    for (int e = 0; e < E; ++e) live = live || g[e] != 0.f;
    const unsigned long long mask = __ballot(live);
    if (mask == 0) return;  // (no barrier below: a wavefront is on its own)
    const int nlive = (int)__popcll(mask);
    if (live) s_list[wave][__popcll(mask & ((1ull << lane) - 1ull))] = (unsigned char)lane;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // the weights of the live points: in flight beside the rows
    float w[E];
#pragma unroll
    for (int e = 0; e < E; ++e) w[e] = 0.f;
    if (live)
    {
        const float4 wp = reinterpret_cast<const float4*>(p.w_pos)[point];
        w[0] = wp.x, w[1] = wp.y, w[2] = wp.z, w[3] = wp.w;
        w[4] = p.w_size[point];
#pragma unroll
        for (int c = 0; c < C; ++c) w[5 + c] = p.w_tex[c * p.tex_stride + point];
        w[5 + C] = p.w_conf[point];
    }
    const int my_r = lane / CHUNKS, my_c = lane - my_r * CHUNKS;
    {
        // every load of the wavefront's rows is issued before the first one is waited for (as a loop that loads and
        // stores pass by pass the round trips to memory ran one after the other)
        constexpr int PASSES = (64 + RPP - 1) / RPP;
        uint4 v[PASSES];
        int src[PASSES];
#pragma unroll
        for (int it = 0; it < PASSES; ++it)
        {
            const int r = it * RPP + my_r;
            src[it]     = -1;
            v[it]       = make_uint4(0u, 0u, 0u, 0u);
            if (my_r < RPP && r < nlive)
            {
                src[it] = s_list[wave][r];
                v[it]   = p.state[(first + src[it]) * CHUNKS + my_c];
            }
        }
#pragma unroll
        for (int it = 0; it < PASSES; ++it)
            if (src[it] >= 0) s_rows[wave][src[it] * LS + my_c] = v[it];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (live)
    {
        uint32_t row[4 * CHUNKS];
#pragma unroll
        for (int j = 0; j < CHUNKS; ++j)
        {
            const uint4 t = s_rows[wave][lane * LS + j];
            row[4 * j] = t.x, row[4 * j + 1] = t.y, row[4 * j + 2] = t.z, row[4 * j + 3] = t.w;
        }
        // The elements of a tensor are mostly updated together, so their counters agree: the bias correction of the
        // tensor's largest counter is computed once and taken by every element whose new counter equals it.
        int top[4] = {0, 0, 0, 0};
#pragma unroll
        for (int e = 0; e < E; ++e)
        {
            const int t = e < 4 ? 0 : e == 4 ? 1 : e < 5 + C ? 2 : 3;
            top[t]      = max(top[t], (int)row[3 * e + 2]);
        }
        // (and tensors with the same learning rate and betas whose largest counters agree share it: usually all four)
        float top_lr[4];
        top_lr[0] = adam_corrected_lr(p.h[0], (uint32_t)(top[0] + 1));
#pragma unroll
        for (int t = 1; t < 4; ++t)
        {
            const bool same_scalars = p.h[t].lr == p.h[0].lr && p.h[t].beta1 == p.h[0].beta1 && p.h[t].beta2 == p.h[0].beta2;
            const bool shares       = same_scalars && top[t] == top[0];
            top_lr[t]               = top_lr[0];
            if (__ballot(!shares))  // (skipped by the whole wavefront in the usual case)
            {
                if (!shares) top_lr[t] = adam_corrected_lr(p.h[t], (uint32_t)(top[t] + 1));
            }
        }
#pragma unroll
        for (int e = 0; e < E; ++e)
        {
            const int t = e < 4 ? 0 : e == 4 ? 1 : e < 5 + C ? 2 : 3;
            float m = __uint_as_float(row[3 * e]), v = __uint_as_float(row[3 * e + 1]), nw;
            long long s = (long long)(int)row[3 * e + 2];
            if (adam_element(p.h[t], g[e], w[e], m, v, s, nw, (uint32_t)(top[t] + 1), top_lr[t]))
            {
                w[e]           = nw;
                row[3 * e]     = __float_as_uint(m);
                row[3 * e + 1] = __float_as_uint(v);
                row[3 * e + 2] = (uint32_t)(int)s;
            }
        }
        reinterpret_cast<float4*>(p.w_pos)[point] = make_float4(w[0], w[1], w[2], w[3]);
        p.w_size[point]                          = w[4];
#pragma unroll
        for (int c = 0; c < C; ++c) p.w_tex[c * p.tex_stride + point] = w[5 + c];
        p.w_conf[point] = w[5 + C];
#pragma unroll
        for (int j = 0; j < CHUNKS; ++j)
            s_rows[wave][lane * LS + j] = make_uint4(row[4 * j], row[4 * j + 1], row[4 * j + 2], row[4 * j + 3]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int base = 0; base < nlive; base += RPP)
    {
        const int r = base + my_r;
        if (my_r < RPP && r < nlive)
        {
            const int src                          = s_list[wave][r];
            p.state[(first + src) * CHUNKS + my_c] = s_rows[wave][src * LS + my_c];
        }
    }
}

// 16-byte chunks of a packed state row: 12 bytes per element, rounded up to whole 128-byte lines
int adam_points_row_chunks(int channels) { return ((6 + channels) * 12 + 127) / 128 * 8; }

hipError_t launch_adam_points(const TripsAdamTensor tensors[4], int num_points, int channels, void* state, hipStream_t stream,
                              Profiler* prof)
{
    ProfScope ps(prof, "adam_fused", stream);
    if (num_points <= 0) return hipSuccess;
    AdamPointsParams p;
    p.w_pos = (float*)tensors[0].weights, p.w_size = (float*)tensors[1].weights, p.w_tex = (float*)tensors[2].weights,
    p.w_conf = (float*)tensors[3].weights;
    p.g_pos = (const float*)tensors[0].grads, p.g_size = (const float*)tensors[1].grads, p.g_tex = (const float*)tensors[2].grads,
    p.g_conf = (const float*)tensors[3].grads;
    p.state      = reinterpret_cast<uint4*>(state);
    p.tex_stride = num_points;
    p.num_points = num_points;
    for (int i = 0; i < 4; ++i)
    {
        const TripsAdamTensor& T = tensors[i];
        p.h[i] = AdamScalars{T.lr, T.beta1, T.beta2, T.eps, T.relative_weight_decay, T.absolute_weight_decay,
                             T.weight_clipping_magnitude, T.lower_lr_bound, T.upper_lr_bound, T.loss_scale};
    }
    const unsigned blocks = (unsigned)((num_points + 255) / 256);
    switch (channels)
    {
        case 3: hipLaunchKernelGGL((adam_points_kernel<3, 8>), dim3(blocks), dim3(256), 0, stream, p); break;
        case 4: hipLaunchKernelGGL((adam_points_kernel<4, 8>), dim3(blocks), dim3(256), 0, stream, p); break;
        case 6: hipLaunchKernelGGL((adam_points_kernel<6, 16>), dim3(blocks), dim3(256), 0, stream, p); break;
        case 8: hipLaunchKernelGGL((adam_points_kernel<8, 16>), dim3(blocks), dim3(256), 0, stream, p); break;
        case 16: hipLaunchKernelGGL((adam_points_kernel<16, 24>), dim3(blocks), dim3(256), 0, stream, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// pose <- se3_exp(t with rotation * 0.1) * pose; t <- 0. Sophus' exp restated (quaternion half-angle form,
// V = I + (1-cos)/th^2 W + (th-sin)/th^3 W^2, first-order renormalisation of the product quaternion).
__global__ __launch_bounds__(128) void apply_tangent_kernel(double* tangent, double* poses, int n)
{
    const int i = blockIdx.x * 128 + threadIdx.x;
    if (i >= n) return;
    double* t = tangent + 6 * (size_t)i;
    double* p = poses + 8 * (size_t)i;
    const double u[3] = {t[0], t[1], t[2]};
    const double w[3] = {t[3] * 0.1, t[4] * 0.1, t[5] * 0.1};
    const double th2  = w[0] * w[0] + w[1] * w[1] + w[2] * w[2];
    const double th   = sqrt(th2);
    double imag, real;
    if (th < 1e-10)
    {
        const double th4 = th2 * th2;
        imag             = 0.5 - th2 / 48.0 + th4 / 3840.0;
        real             = 1.0 - th2 / 8.0 + th4 / 384.0;
    }
    else
    {
        imag = sin(0.5 * th) / th;
        real = cos(0.5 * th);
    }
    const double x1 = imag * w[0], y1 = imag * w[1], z1 = imag * w[2], w1 = real;
    const double W[9] = {0, -w[2], w[1], w[2], 0, -w[0], -w[1], w[0], 0};
    double W2[9];
    for (int r = 0; r < 3; ++r)
        for (int c = 0; c < 3; ++c)
        {
            double s = 0;
            for (int k = 0; k < 3; ++k) s += W[3 * r + k] * W[3 * k + c];
            W2[3 * r + c] = s;
        }
    const double R1[9] = {1 - 2 * (y1 * y1 + z1 * z1), 2 * (x1 * y1 - z1 * w1),     2 * (x1 * z1 + y1 * w1),
                          2 * (x1 * y1 + z1 * w1),     1 - 2 * (x1 * x1 + z1 * z1), 2 * (y1 * z1 - x1 * w1),
                          2 * (x1 * z1 - y1 * w1),     2 * (y1 * z1 + x1 * w1),     1 - 2 * (x1 * x1 + y1 * y1)};
    double Vm[9];
    if (th < 1e-10)
    {
        for (int k = 0; k < 9; ++k) Vm[k] = R1[k];
    }
    else
    {
        const double a = (1 - cos(th)) / th2, b = (th - sin(th)) / (th2 * th);
        for (int k = 0; k < 9; ++k) Vm[k] = (k % 4 == 0 ? 1.0 : 0.0) + a * W[k] + b * W2[k];
    }
    double t1[3];
    for (int r = 0; r < 3; ++r) t1[r] = Vm[3 * r] * u[0] + Vm[3 * r + 1] * u[1] + Vm[3 * r + 2] * u[2];
    const double x2 = p[0], y2 = p[1], z2 = p[2], w2 = p[3];
    double q[4] = {w1 * x2 + x1 * w2 + y1 * z2 - z1 * y2, w1 * y2 - x1 * z2 + y1 * w2 + z1 * x2,
                   w1 * z2 + x1 * y2 - y1 * x2 + z1 * w2, w1 * w2 - x1 * x2 - y1 * y2 - z1 * z2};
    const double sn = q[0] * q[0] + q[1] * q[1] + q[2] * q[2] + q[3] * q[3];
    if (sn != 1.0)
    {
        const double sc = 2.0 / (1.0 + sn);
        for (int k = 0; k < 4; ++k) q[k] *= sc;
    }
    double tn[3];
    for (int r = 0; r < 3; ++r) tn[r] = t1[r] + R1[3 * r] * p[4] + R1[3 * r + 1] * p[5] + R1[3 * r + 2] * p[6];
    for (int k = 0; k < 4; ++k) p[k] = q[k];
    for (int k = 0; k < 3; ++k) p[4 + k] = tn[k];
    for (int k = 0; k < 6; ++k) t[k] = 0.0;
}

hipError_t launch_apply_tangent(double* tangent, double* poses, int n, hipStream_t stream)
{
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(apply_tangent_kernel, dim3((n + 127) / 128), dim3(128), 0, stream, tangent, poses, n);
    return hipGetLastError();
}

// ---- exports from the saved state ----
// (the records are kept per valid point, at its compact number)
__global__ __launch_bounds__(256) void export_points_kernel(const float* __restrict__ rec, int rec_floats,
                                                            const float* __restrict__ prec, const int32_t* __restrict__ cid_of,
                                                            int n, float* ip, float* depth, float* size_px, int32_t* max_layer)
{
    const int pid = blockIdx.x * 256 + threadIdx.x;
    if (pid >= n) return;
    const int cid   = cid_of[pid];
    const bool ok   = cid >= 0;
    const float* r  = rec + (size_t)(ok ? cid : 0) * rec_floats;
    // {softplus'(raw size), depth, max_layer, size_px}
    const float4 tl = ok ? reinterpret_cast<const float4*>(prec)[cid] : make_float4(0.f, -1.f, 0.f, 0.f);
    if (ip)
    {
        ip[2 * (size_t)pid]     = ok ? r[0] : 0.f;
        ip[2 * (size_t)pid + 1] = ok ? r[1] : 0.f;
    }
    if (depth) depth[pid] = tl.y;
    if (size_px) size_px[pid] = ok ? tl.w : 0.f;
    if (max_layer) max_layer[pid] = ok ? __float_as_int(tl.z) : 0;
}

hipError_t launch_export_points(const float* rec, int rec_floats, const float* prec, const int32_t* cid_of, int n, float* ip,
                                float* depth, float* size_px, int32_t* max_layer, hipStream_t stream)
{
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(export_points_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, rec, rec_floats, prec, cid_of, n, ip,
                       depth, size_px, max_layer);
    return hipGetLastError();
}

// saved tables are tile-major (padded); the exports are row-major, layer by layer
__global__ __launch_bounds__(256) void export_lists_kernel(const PyramidGeom g, int K, const int32_t* __restrict__ lists,
                                                           const int32_t* __restrict__ retained,
                                                           const int32_t* __restrict__ pid_of, int32_t* out_lists,
                                                           int32_t* out_retained, int32_t* out_lengths)
{
    const int P = g.off[g.num_layers];
    const int r = blockIdx.x * 256 + threadIdx.x;
    if (r >= P) return;
    int layer = 0;
    while (layer + 1 < g.num_layers && r >= g.off[layer + 1]) ++layer;
    const int local = r - g.off[layer];
    const int x = local % g.w[layer], y = local / g.w[layer];
    const int ip = pix_index(g, layer, x, y);
    const unsigned word = (unsigned)retained[ip];  // retained entries | filled list positions << 5 | list length << 10
    const int filled    = (int)((word >> kRetainedBits) & kRetainedMask);
    if (out_retained) out_retained[r] = (int)(word & kRetainedMask);
    if (out_lengths) out_lengths[r] = (int)(word >> (2 * kRetainedBits));
    if (out_lists)
        for (int k = 0; k < K; ++k)
        {
            const int cid                = k < filled ? lists[list_word((unsigned)ip, k, K)] : -1;  // compact number of the point
            out_lists[(size_t)r * K + k] = cid >= 0 ? pid_of[cid] : -1;
        }
}

hipError_t launch_export_lists(const PyramidGeom& g, int K, const int32_t* lists, const int32_t* retained,
                               const int32_t* pid_of, int32_t* out_lists, int32_t* out_retained,
                               int32_t* out_lengths, hipStream_t stream)
{
    const int P = g.off[g.num_layers];
    if (P <= 0) return hipSuccess;
    hipLaunchKernelGGL(export_lists_kernel, dim3((P + 255) / 256), dim3(256), 0, stream, g, K, lists, retained, pid_of,
                       out_lists, out_retained, out_lengths);
    return hipGetLastError();
}

__global__ __launch_bounds__(256) void sum_i32_kernel(const int32_t* __restrict__ v, long long n, unsigned mask,
                                                      unsigned long long* out)
{
    __shared__ unsigned long long s[4];
    unsigned long long acc = 0;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256)
        acc += (unsigned long long)((unsigned)v[i] & mask);
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
    if ((threadIdx.x & 63) == 0) s[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) atomicAdd(out, s[0] + s[1] + s[2] + s[3]);
}

// *out = sum of (v[i] & mask)
hipError_t launch_sum_i32(const int32_t* v, long long n, unsigned mask, unsigned long long* out, hipStream_t stream)
{
    hipError_t e = hipMemsetAsync(out, 0, sizeof(unsigned long long), stream);
    if (e != hipSuccess) return e;
    if (n <= 0) return hipSuccess;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL(sum_i32_kernel, dim3(blocks), dim3(256), 0, stream, v, n, mask, out);
    return hipGetLastError();
}

}  // namespace trips
