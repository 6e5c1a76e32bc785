// Backward of the decoder-only gated-convolution U-Net on the gfx950 matrix cores: what libtorch's autograd does
// for MultiScaleUnet2dDecOnlySmallFixedImpl::forward in the reference (src/lib/models/Networks.h:1139-1191, blocks
// at :751-787 and :999-1098), as hand-written kernels over the state the training forward saved.
//
//   final_backward_kernel     1x1 output convolution: gradient of x_0, split into dL/d in[0] and, through the gate,
//                             the gradient of the finest block's pre-activations; its weight and bias gradients
//   conv_bwd_data_kernel      gradient of a block's input: the forward's implicit GEMM with flipped, transposed
//                             weights (M = 256 pixels, N = input channels, K = 9 taps x pre-activations)
//   up2_adjoint_gate_kernel   adjoint of the bilinear 2x upsampling (a gather over <= 4 x 4 finer pixels), then
//                             dL/d in[i+1] and the gate of the coarser block
//   conv_bwd_weight_kernel    weight gradients: GEMM with the pixels as the reduction dimension. Both operands are
//                             needed pixel-contiguous; the tiles stay pixel-major in LDS, as they are assembled, and
//                             the operands are fetched with the transposing LDS read (ds_read_b64_tr_b16);
//                             persistent workgroups keep their partial sums in registers over many tiles; the
//                             bias gradients (sums of the pre-activation gradients) are one more MFMA per tile row
//                             against a matrix of ones
//   bias_grad_kernel          bias gradients alone, when no weight gradient is asked for
//   reduce_weight_grad_kernel
//
// Intermediate gradients are fp16 and carried multiplied by grad_scale; every fp32 result is divided by it again.
#include <algorithm>
#include <cmath>
#include <cstring>

#include "unet_common.h"

namespace trips
{

// d(elu(f) * sigmoid(m)) for an incoming gradient da
// (`act`: the gated value itself, elu(f) * sigmoid(m), with the forward's formula)
__device__ __forceinline__ void gate_backward(float da, float f, float m, float& df, float& dm, float& act)
{
    const float s  = __builtin_amdgcn_rcpf(1.f + __expf(-m));  // 1 ulp; the gradients are rounded to fp16 next
    const float ex = __expf(f);
    const float e  = f > 0.f ? f : ex - 1.f;
    const float de = f > 0.f ? 1.f : ex;
    df             = da * s * de;
    dm             = da * e * s * (1.f - s);
    act            = e * s;
}
__device__ __forceinline__ void gate_backward(float da, float f, float m, float& df, float& dm)
{
    float act;
    gate_backward(da, f, m, df, dm, act);
}

// wt[tap'][c][n] = W[n][c][8 - tap']: the data gradient is a correlation of the pre-activation gradient with the
// spatially flipped kernel, input and output channels exchanged
// (all levels in one launch, the level is blockIdx.y: a launch per level costs more than the work itself)
struct PackTLevel
{
    const float *wf, *wm;
    int cout, cin_real, cin_pad, npad;
    _Float16* wt;
};
struct PackTTable
{
    PackTLevel lv[TRIPS_UNET_MAX_LEVELS];
};
__global__ __launch_bounds__(256) void pack_conv_weights_T_kernel(const PackTTable t)
{
    const PackTLevel& l = t.lv[blockIdx.y];
    const float* __restrict__ wf = l.wf;
    const float* __restrict__ wm = l.wm;
    const int cout = l.cout, cin_real = l.cin_real, cin_pad = l.cin_pad, npad = l.npad;
    _Float16* __restrict__ wt = l.wt;
    const int total = 9 * cin_pad * npad;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256)
    {
        const int n = i % npad, c = (i / npad) % cin_pad, tap = i / (npad * cin_pad);
        const int half = npad / 2;
        const int o    = n < half ? n : n - half;
        float v        = 0.f;
        if (o < cout && c < cin_real) v = (n < half ? wf : wm)[((size_t)o * cin_real + c) * 9 + (8 - tap)];
        wt[i] = _Float16(v);
    }
}

__global__ __launch_bounds__(256) void fill_f32_kernel(float* __restrict__ p, float v, int n)
{
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) p[i] = v;
}

struct FinalBwdParams
{
    int H, W, c_feat, cact, cact_store, cout, npad;
    float scale;
    const float* feat;        // [C][H][W]
    const _Float16* pre;      // [H][W][npad]
    const float* weight;      // [cout][c_feat + cact]
    const float* d_out;       // [cout][H][W]
    float* d_feat;            // [C][H][W], written
    _Float16* dpre;           // [H][W][npad], written
    float* part;              // [gridDim.x][4 * (4 + CS) + 4] sums of this launch's workgroups (WGRAD)
    int chunks;               // ceil(pixels / kFinalPixelsPerBlock)
};

// One pass over the pixels of the finest level: dL/d in[0], the gated block's pre-activation gradients and, when
// WGRAD, the weight and bias gradients of the 1x1 convolution. Every thread keeps the cout x cin products of its
// pixels in registers, a workgroup folds them through LDS and writes its sums once (final_reduce_kernel adds the
// workgroups up: atomics of a thousand workgroups on these few addresses would serialise in one L2 channel).
// (The library is compiled without contraction of products and sums; this kernel is bound by its arithmetic
// instructions, and its sums are written as fused multiply-adds.)
// CS = halves per pixel of the block output.
// CI = image channels the kernel has room for (4, 8 or 16).
template <int CS, bool WGRAD, int CI>
__global__ __launch_bounds__(256) void final_backward_kernel(const FinalBwdParams p)
{
    constexpr int MAXC = CI + CS;
    // LPP lanes share a pixel, one per 16 bytes of its pre-activation row (feature groups first, then mask groups),
    // so that a wavefront reads and writes whole lines of the channels-innermost arrays. The feature and the mask
    // lane of a channel group exchange their values with one cross-lane read.
    constexpr int LPP = CS <= 16 ? 4 : CS <= 32 ? 8 : 16;
    constexpr int PPW = 64 / LPP;  // pixels per wavefront and iteration
    __shared__ float s_w[4 * MAXC];
    __shared__ float s_sum[4 * MAXC + 4];
    const int cin = p.c_feat + p.cact;
    // weights as the forward used them (fp16), laid out [k][CI image channels | CS block outputs], zero where unused
    for (int i = threadIdx.x; i < 4 * MAXC; i += 256)
    {
        const int k = i / MAXC, r = i - k * MAXC;
        const int c = r < CI ? (r < p.c_feat ? r : -1) : (r - CI < p.cact ? p.c_feat + r - CI : -1);
        s_w[i]      = (k < p.cout && c >= 0) ? float(_Float16(p.weight[k * cin + c])) : 0.f;
    }
    for (int i = threadIdx.x; i < 4 * MAXC + 4; i += 256) s_sum[i] = 0.f;
    __syncthreads();
    const size_t plane = (size_t)p.H * p.W;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane % LPP, sub = lane / LPP;
    const int hg       = p.npad / 16;                    // 16-byte groups in each half of a pre-activation row
    const bool is_f    = g < hg;
    const bool in_row  = g < 2 * hg;                     // lanes past the row idle (rows of 96 halves on 16 lanes)
    const int ch0      = 8 * (is_f ? g : g - hg);        // first of this lane's 8 channels
    const int partner  = is_f ? lane + hg : lane - hg;   // the lane with the other half of the same channels
    // ... and the image channels g, g + LPP, ... (one each for up to LPP image channels)
    constexpr int NI = (CI + LPP - 1) / LPP;
    bool has_img[NI];
#pragma unroll
    for (int j = 0; j < NI; ++j) has_img[j] = g + LPP * j < p.c_feat;
    // The feature lane and the mask lane of a group hold the same eight channels once they have exchanged their values:
    // the feature lane works out the first four (gradients of both pre-activations, the block's output), the mask lane
    // the other four, and they exchange what the other one stores.
    const int c0 = ch0 + (is_f ? 0 : 4);  // first of the four channels this lane works out
    float wj[4][4], wimg[4][NI];
#pragma unroll
    for (int k = 0; k < 4; ++k)
    {
#pragma unroll
        for (int j = 0; j < NI; ++j) wimg[k][j] = has_img[j] ? s_w[k * MAXC + g + LPP * j] : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) wj[k][i] = (in_row && c0 + i < CS) ? s_w[k * MAXC + CI + c0 + i] : 0.f;
    }
    float acc[4][4];
    float acc_img[4][NI], accb[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int j = 0; j < NI; ++j) acc_img[k][j] = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[k][i] = 0.f;

    struct Loaded
    {
        float g[4], x[NI];
        half8 mine;
    };
    auto load = [&](size_t pix, bool valid)
    {
        Loaded l;
#pragma unroll
        for (int k = 0; k < 4; ++k) l.g[k] = (valid && k < p.cout) ? p.d_out[k * plane + pix] : 0.f;
#pragma unroll
        for (int j = 0; j < NI; ++j) l.x[j] = (WGRAD && valid && has_img[j]) ? p.feat[(size_t)(g + LPP * j) * plane + pix] : 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) l.mine[i] = _Float16(0.f);
        if (valid && in_row) l.mine = *reinterpret_cast<const half8*>(p.pre + pix * p.npad + 8 * g);
        return l;
    };
    constexpr int STEP = 4 * PPW;  // pixels per iteration of the workgroup
    for (int chunk = blockIdx.x; chunk < p.chunks; chunk += gridDim.x)
    {
        const size_t p1 = std::min(plane, (size_t)(chunk + 1) * kFinalPixelsPerBlock);
        size_t base     = (size_t)chunk * kFinalPixelsPerBlock + wave * PPW;
        Loaded next     = load(base + sub, base + sub < p1);
        for (; base < p1; base += STEP)
        {
            const size_t pix = base + sub;
            const bool valid = pix < p1;
            const Loaded cur = next;
            if (base + STEP < p1) next = load(pix + STEP, pix + STEP < p1);  // in flight while this pixel is worked on
            // the other half (mask values for a feature lane and the reverse) of the same 8 channels
            typedef int intx4 __attribute__((ext_vector_type(4)));
            intx4 raw = __builtin_bit_cast(intx4, cur.mine), oth;
#pragma unroll
            for (int q = 0; q < 4; ++q) oth[q] = __shfl(raw[q], partner);
            const half8 other = __builtin_bit_cast(half8, oth);
            const half8 f8 = is_f ? cur.mine : other, m8 = is_f ? other : cur.mine;
            half4 keep, give;  // what this lane stores of its four channels, and what its partner stores of them
            float v[4];        // the block's output as the forward's 1x1 convolution read it (fp16)
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                float da = 0.f;
#pragma unroll
                for (int k = 0; k < 4; ++k) da = __builtin_fmaf(wj[k][i], cur.g[k], da);
                float df, dm, a;
                gate_backward(da * p.scale, float(is_f ? f8[i] : f8[4 + i]), float(is_f ? m8[i] : m8[4 + i]), df, dm, a);
                keep[i] = _Float16(is_f ? df : dm);
                give[i] = _Float16(is_f ? dm : df);
                v[i]    = (valid && in_row && c0 + i < p.cact) ? float(_Float16(a)) : 0.f;
            }
            typedef int intx2 __attribute__((ext_vector_type(2)));
            const intx2 give_raw = __builtin_bit_cast(intx2, give);
            intx2 got_raw;
            got_raw[0] = __shfl(give_raw[0], partner);
            got_raw[1] = __shfl(give_raw[1], partner);
            const half4 got = __builtin_bit_cast(half4, got_raw);
            // a feature lane stores the feature gradients of the eight channels: its own four, then the partner's
            const half8 out = is_f ? half8{keep[0], keep[1], keep[2], keep[3], got[0], got[1], got[2], got[3]}
                                   : half8{got[0], got[1], got[2], got[3], keep[0], keep[1], keep[2], keep[3]};
            if (valid && in_row) *reinterpret_cast<half8*>(p.dpre + pix * p.npad + 8 * g) = out;
#pragma unroll
            for (int j = 0; j < NI; ++j)
            {
                if (valid && has_img[j])
                {
                    float d = 0.f;
#pragma unroll
                    for (int k = 0; k < 4; ++k) d = __builtin_fmaf(wimg[k][j], cur.g[k], d);
                    p.d_feat[(size_t)(g + LPP * j) * plane + pix] = d;
                }
            }
            if (WGRAD)
            {
                float xr[NI];
#pragma unroll
                for (int j = 0; j < NI; ++j) xr[j] = float(_Float16(cur.x[j]));
#pragma unroll
                for (int k = 0; k < 4; ++k)
                {
                    accb[k] += cur.g[k];
#pragma unroll
                    for (int j = 0; j < NI; ++j) acc_img[k][j] = __builtin_fmaf(cur.g[k], xr[j], acc_img[k][j]);
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[k][i] = __builtin_fmaf(cur.g[k], v[i], acc[k][i]);
                }
            }
        }
    }
    if (!WGRAD) return;
    // fold the lanes that hold the same channels with a butterfly first: many lanes adding to one LDS address would
    // be serialised
    auto fold = [](float v)
    {
#pragma unroll
        for (int o = 32; o >= LPP; o >>= 1) v += __shfl_xor(v, o);
        return v;
    };
#pragma unroll
    for (int k = 0; k < 4; ++k)
    {
        const float b = fold(accb[k]);
        if (lane == 0) atomicAdd(&s_sum[4 * MAXC + k], b);
#pragma unroll
        for (int j = 0; j < NI; ++j)
        {
            const float im = fold(acc_img[k][j]);
            if (lane < LPP && has_img[j]) atomicAdd(&s_sum[k * MAXC + g + LPP * j], im);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            const float v = fold(acc[k][i]);
            if (lane < LPP && in_row && c0 + i < CS) atomicAdd(&s_sum[k * MAXC + CI + c0 + i], v);
        }
    }
    __syncthreads();
    float* part = p.part + (size_t)blockIdx.x * (4 * MAXC + 4);
    for (int t = threadIdx.x; t < 4 * MAXC + 4; t += 256) part[t] = s_sum[t];
}

// Adds up `rows` partial-sum rows of `cols` floats: workgroup c sums column c, thread 0 holds the result.
__device__ __forceinline__ float block_column_sum(const float* __restrict__ part, int rows, int cols, int c)
{
    __shared__ float s_red[4];
    float s = 0.f;
    for (int r = threadIdx.x; r < rows; r += 256) s += part[(size_t)r * cols + c];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
    if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = s;
    __syncthreads();
    return (s_red[0] + s_red[1]) + (s_red[2] + s_red[3]);
}

// d_weight [cout][c_feat + cact] and d_bias [cout] of the 1x1 convolution from final_backward_kernel's partial sums
// (row layout [k][ci image channels | CS block outputs], then 4 biases; maxc = ci + CS); one workgroup per result
__global__ __launch_bounds__(256) void final_reduce_kernel(const float* __restrict__ part, int rows, int maxc, int ci, int c_feat, int cact,
                                                           int cout, float* __restrict__ d_weight, float* __restrict__ d_bias)
{
    const int cin = c_feat + cact;
    const int t   = blockIdx.x;  // < cout * cin + cout
    int col;
    float* dst;
    if (t < cout * cin)
    {
        const int k = t / cin, c = t - k * cin;
        col = k * maxc + (c < c_feat ? c : ci + (c - c_feat));
        dst = d_weight + t;
    }
    else
    {
        col = 4 * maxc + (t - cout * cin);
        dst = d_bias + (t - cout * cin);
    }
    if (!(t < cout * cin ? d_weight : d_bias)) return;  // the caller asked for one of the two only
    const float s = block_column_sum(part, rows, 4 * maxc + 4, col);
    if (threadIdx.x == 0) *dst = s;
}

// ---------------------------------------------------------------------------------------------------------
struct BwdDataParams
{
    int H, W, c_feat;
    float scale_inv;
    const _Float16* dpre;  // [H][W][KC]
    const _Float16* wt;    // [9][NN][KC]
    float* d_feat;         // [C][H][W], accumulated
    _Float16* d_in;        // [H][W][NN] or nullptr (start block: nothing below)
};

// CI = image channels the kernel has room for (4, 8 or 16): positions [0, C) of the block input are the level's image.
template <int KC, int NN, int THREADS, int CI>
__global__ __launch_bounds__(THREADS) void conv_bwd_data_kernel(const BwdDataParams p)
{
    constexpr int MB = 16 / (THREADS / 64);  // 16-pixel row blocks of a wavefront: two rows of the tile, or one
    constexpr int ROW    = KC + kLdsChanPad;
    constexpr int GROUPS = KC / 8;
    constexpr int NB     = NN / 16;
    extern __shared__ _Float16 smem[];
    _Float16* s_patch = smem;
    const int x0 = blockIdx.x * kConvTileW, y0 = blockIdx.y * kConvTileH;
    ConvTapStage<KC, NN, THREADS> taps;
    conv_tap_fetch(taps, p.wt, 0);  // in flight while the patch is loaded
    _Float16* s_taps = s_patch + kConvPatchH * kConvPatchW * ROW;  // the staged taps of the weights
    // the patch of pre-activation gradients, four 16-byte loads of a thread in flight together
    constexpr int kItems = kConvPatchH * kConvPatchW * GROUPS;
    for (int item0 = threadIdx.x; item0 < kItems; item0 += 4 * THREADS)
    {
        // (every load unconditional, at a position clamped into the image, and all four requested before the first is
        // used: a load under a condition is waited for where the condition ends)
        uint4 raw[4];
        bool in[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            const int item = min(item0 + THREADS * j, kItems - 1);
            const int g = item % GROUPS, pp = item / GROUPS;
            const int py = pp / kConvPatchW, px = pp - py * kConvPatchW;
            const int y = y0 + py - 1, x = x0 + px - 1;
            in[j]  = y >= 0 && y < p.H && x >= 0 && x < p.W;
            raw[j] = *reinterpret_cast<const uint4*>(p.dpre + ((size_t)min(max(y, 0), p.H - 1) * p.W + min(max(x, 0), p.W - 1)) * KC + 8 * g);
        }
        half8 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            asm volatile("" : "+v"(raw[j].x), "+v"(raw[j].y), "+v"(raw[j].z), "+v"(raw[j].w));
            if (!in[j]) raw[j] = make_uint4(0u, 0u, 0u, 0u);
            v[j] = __builtin_bit_cast(half8, raw[j]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            const int item = item0 + THREADS * j;
            if (item < kItems) *reinterpret_cast<half8*>(s_patch + (size_t)(item / GROUPS) * ROW + 8 * (item % GROUPS)) = v[j];
        }
    }
    conv_tap_stage(taps, s_taps);
    __syncthreads();
    floatx4 acc[MB][NB];
    conv_taps_mfma<KC, NN, true, THREADS>(s_patch, s_taps, p.wt, taps, acc);  // a lane: four channels of one pixel
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lrow = lane & 15;
    // ---- epilogue: the tile staged in LDS (the patch is no longer needed) and written channels innermost with
    // 16-byte stores, whole lines at a time; the image channels' share kept in fp32 beside it ----
    constexpr int OS   = NN + kLdsChanPad;
    _Float16* s_out    = smem;                                                                   // [256][OS]
    float* s_img       = reinterpret_cast<float*>(smem + kConvTileH * kConvTileW * OS);          // [CI][256]
    __syncthreads();  // every wavefront is done reading the patch
#pragma unroll
    for (int m = 0; m < MB; ++m)
    {
        const int tp = (MB == 4 ? 2 * wave + (m >> 1) : wave) * kConvTileW + (m & 1) * 16 + lrow;  // this lane's pixel of the block
#pragma unroll
        for (int n = 0; n < NB; ++n)
        {
            const int c0 = 16 * n + (lane >> 4) * 4;  // this lane's four channels
            *reinterpret_cast<half4*>(s_out + tp * OS + c0) =
                half4{_Float16(acc[m][n][0]), _Float16(acc[m][n][1]), _Float16(acc[m][n][2]), _Float16(acc[m][n][3])};
            if (n == 0 && c0 < CI)
            {
#pragma unroll
                for (int i = 0; i < 4; ++i) s_img[(c0 + i) * (kConvTileH * kConvTileW) + tp] = acc[m][0][i];
            }
        }
    }
    __syncthreads();
    if (p.d_in) store_tile_nhwc<THREADS>(s_out, OS, NN / 8, p.d_in, NN, x0, y0, p.W, p.H);
    {
        const size_t plane = (size_t)p.H * p.W;
        const int y = y0 + threadIdx.x / kConvTileW, x = x0 + threadIdx.x % kConvTileW;
        if ((int)threadIdx.x < kConvTileH * kConvTileW && y < p.H && x < p.W)
        {
            float old[CI];
#pragma unroll
            for (int c = 0; c < CI; ++c) old[c] = c < p.c_feat ? p.d_feat[c * plane + (size_t)y * p.W + x] : 0.f;
#pragma unroll
            for (int c = 0; c < CI; ++c)
                if (c < p.c_feat) p.d_feat[c * plane + (size_t)y * p.W + x] = old[c] + s_img[c * (kConvTileH * kConvTileW) + threadIdx.x] * p.scale_inv;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
struct UpAdjointParams
{
    int H, W;      // finer level, whose block input gradient is given
    int Hb, Wb;    // this (coarser) level
    int cin_fine;  // halves per pixel of d_in
    int c_feat, cout, npad;
    float scale_inv;
    const _Float16* d_in;  // [H][W][cin_fine]: position k = channel k of cat(in, up2(x))
    const _Float16* pre;   // [Hb][Wb][npad]
    float* d_feat;         // [C][Hb][Wb], written
    _Float16* dpre;        // [Hb][Wb][npad], written
};

// weight with which finer row / column `dst` reads coarser row / column `src`
__device__ __forceinline__ float up2_weight(int dst, int fine_size, int src, int coarse_size)
{
    if (dst < 0 || dst >= fine_size) return 0.f;
    int i0, i1;
    float l;
    up2_source(dst, coarse_size, i0, i1, l);
    return (i0 == src ? 1.f - l : 0.f) + (i1 == src ? l : 0.f);
}

// SHIFT = (2 C) % 8: the block outputs of the coarser level start at position 2 C of the finer block's input, which is
// a multiple of 8 halves only for C = 4; otherwise a group of eight outputs straddles two aligned groups of positions.
template <int SHIFT>
__global__ __launch_bounds__(256) void up2_adjoint_gate_kernel(const UpAdjointParams p)
{
    const int half   = p.npad / 2;
    const int C      = p.c_feat;
    // the coarser level's image sits at positions [C, 2C) of the finer block's input: the aligned groups of eight
    // positions g0 .. g0 + ig - 1 (one group up to C = 4 and for C = 8, two for 6 and 16)
    const int g0 = C / 8, ig = (2 * C - 1) / 8 - g0 + 1;
    const int groups = ig + half / 8;  // groups 0 .. ig - 1: the image below; then 8 block outputs each
    const size_t pb  = (size_t)p.Hb * p.Wb;
    const int base8  = (2 * C) & ~7;  // aligned position at or before the first block output
    for (size_t item = (size_t)blockIdx.x * 256 + threadIdx.x; item < pb * groups; item += (size_t)gridDim.x * 256)
    {
        const int q     = (int)(item % groups);
        const size_t bp = item / groups;
        const int Y = (int)(bp / p.Wb), X = (int)(bp - (size_t)Y * p.Wb);
        // the pre-activations first: in flight during the gather
        const int ch0 = 8 * (q - ig);
        half8 f8, m8;
#pragma unroll
        for (int i = 0; i < 8; ++i) f8[i] = m8[i] = _Float16(0.f);
        if (q >= ig)
        {
            f8 = *reinterpret_cast<const half8*>(p.pre + bp * p.npad + ch0);
            m8 = *reinterpret_cast<const half8*>(p.pre + bp * p.npad + half + ch0);
        }
        float wy[4], wx[4];
#pragma unroll
        for (int k = 0; k < 4; ++k)
        {
            wy[k] = up2_weight(2 * Y - 1 + k, p.H, Y, p.Hb);
            wx[k] = up2_weight(2 * X - 1 + k, p.W, X, p.Wb);
        }
        // the adjoint of the upsampling for the eight positions from `pos` on (a multiple of 8)
        auto gather = [&](int pos, float (&a)[8])
        {
#pragma unroll
            for (int i = 0; i < 8; ++i) a[i] = 0.f;
            if (pos >= p.cin_fine) return;
            // all 16 gathers are issued before the first one is used (a load inside a branch on its weight would be
            // waited for there: 16 memory round trips in a row); pixels outside the image have weight 0 and are read
            // at a clamped position instead
            half8 v[4][4];
            int xoff[4];  // (a row of the finer level stays below 2^31 halves)
#pragma unroll
            for (int kx = 0; kx < 4; ++kx) xoff[kx] = min(max(2 * X - 1 + kx, 0), p.W - 1) * p.cin_fine + pos;
#pragma unroll
            for (int ky = 0; ky < 4; ++ky)
            {
                const int y         = min(max(2 * Y - 1 + ky, 0), p.H - 1);
                const _Float16* row = p.d_in + (size_t)y * p.W * p.cin_fine;
#pragma unroll
                for (int kx = 0; kx < 4; ++kx) v[ky][kx] = *reinterpret_cast<const half8*>(row + xoff[kx]);
            }
#pragma unroll
            for (int ky = 0; ky < 4; ++ky)
            {
#pragma unroll
                for (int kx = 0; kx < 4; ++kx)
                {
                    const float w = wy[ky] * wx[kx];
                    if (w != 0.f)
                    {
                        // (one fused multiply-add that reads the fp16 value, instead of a conversion, a product and a sum)
#pragma unroll
                        for (int i = 0; i < 8; ++i) a[i] = __builtin_fmaf(w, float(v[ky][kx][i]), a[i]);
                    }
                }
            }
        };
        // (one gather for all lanes of a wavefront, whatever their group: lanes of both kinds sit side by side)
        float a[8];
        const int first = q < ig ? 8 * (g0 + q) : base8 + ch0;  // first of the eight positions this item gathers
        gather(first, a);
        if (q < ig)
        {
            // positions [0, C) are the finer level's own image, [C, 2C) this level's
#pragma unroll
            for (int i = 0; i < 8; ++i)
            {
                const int c = first + i - C;  // (a[] only with compile-time indices: else the array goes to scratch memory)
                if (c >= 0 && c < C) p.d_feat[(size_t)c * pb + bp] = a[i] * p.scale_inv;
            }
        }
        else
        {
            // output ch0 + i of this level sits at position 2 C + ch0 + i = base8 + ch0 + SHIFT + i
            if (SHIFT != 0)
            {
                float hi[8];
                gather(base8 + ch0 + 8, hi);
#pragma unroll
                for (int i = 0; i < 8; ++i) a[i] = SHIFT + i < 8 ? a[(SHIFT + i) & 7] : hi[(SHIFT + i) & 7];
            }
            _Float16* dp = p.dpre + bp * p.npad;
            half8 of, om;
#pragma unroll
            for (int i = 0; i < 8; ++i)
            {
                float df, dm;
                gate_backward(ch0 + i < p.cout ? a[i] : 0.f, float(f8[i]), float(m8[i]), df, dm);
                of[i] = _Float16(df);
                om[i] = _Float16(dm);
            }
            *reinterpret_cast<half8*>(dp + ch0)        = of;
            *reinterpret_cast<half8*>(dp + half + ch0) = om;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
struct BiasGradParams
{
    size_t pixels;
    int npad, cout;
    float scale_inv;
    const _Float16* dpre;  // [pixels][npad]
    float* d_bias_f;       // [cout], accumulated (zeroed by the caller)
    float* d_bias_m;
};

constexpr int kBiasChunk = 1024;
__global__ __launch_bounds__(256) void bias_grad_kernel(const BiasGradParams p)
{
    __shared__ float s_sum[128];
    if (threadIdx.x < 128) s_sum[threadIdx.x] = 0.f;
    __syncthreads();
    const int groups = p.npad / 8;
    const int lanes  = 256 / groups;  // pixels in flight per block
    const int g = threadIdx.x % groups, sub = threadIdx.x / groups;
    if (sub < lanes)
    {
        float a[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) a[i] = 0.f;
        const size_t p0 = (size_t)blockIdx.x * kBiasChunk, p1 = std::min(p.pixels, p0 + kBiasChunk);
        for (size_t pix = p0 + sub; pix < p1; pix += lanes)
        {
            const half8 v = *reinterpret_cast<const half8*>(p.dpre + pix * p.npad + 8 * g);
#pragma unroll
            for (int i = 0; i < 8; ++i) a[i] += float(v[i]);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) atomicAdd(&s_sum[8 * g + i], a[i]);
    }
    __syncthreads();
    if ((int)threadIdx.x < p.npad)
    {
        const int n = threadIdx.x, half = p.npad / 2;
        const int o = n < half ? n : n - half;
        if (o < p.cout)
        {
            float* dst = n < half ? p.d_bias_f : p.d_bias_m;
            if (dst) atomicAdd(dst + o, s_sum[n] * p.scale_inv);
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
struct BwdWeightParams
{
    int H, W, Hb, Wb;
    int c_feat, cb_store;
    int tiles_x, tiles;
    const float* feat;
    const float* feat_below;
    const _Float16* act_below;
    const _Float16* dpre;  // [H][W][NPAD]
    float* part;           // [gridDim.x][9][NPAD][CIN]
    // bias gradients = sums of dpre over the pixels, taken from the transposed tile while it is in LDS
    float* bias_part;      // [gridDim.x][NPAD] or nullptr
};

// Pixel-major tiles and the transposing LDS read. Both operands of the weight-gradient GEMM are needed with eight
// consecutive pixels per lane, while the tiles are assembled (and arrive from memory) with the channels of a pixel side
// by side. ds_read_b64_tr_b16 closes the gap: the 16 lanes of a group read a 4 x 16 block of halves row by row (lane
// i: row i / 4, columns 4 (i % 4) .. + 3) and each receives one column (lane n: rows 0 .. 3 of column n). Two such
// reads give a lane the eight pixels of its channel; the tiles stay as the forward kernel builds them, written with
// 16-byte stores (written transposed, 2 bytes at a time, the staging took most of the kernel's time).
typedef short short4v __attribute__((ext_vector_type(4)));
// rows `pix` .. `pix + 7` of column `col0 + lane % 16` of a tile [pixel][stride halves]; `col0` a multiple of 16
__device__ __forceinline__ half8 lds_read_pixels_of_channel(const _Float16* tile, int stride, int pix, int col0)
{
    const int i = threadIdx.x & 15;
    const _Float16* src = tile + (size_t)(pix + (i >> 2)) * stride + col0 + (i & 3) * 4;
    using lds_ptr = __attribute__((address_space(3))) short4v*;
    const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)src);
    const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(src + 4 * stride));
    union
    {
        short s[8];
        half8 h;
    } u;
#pragma unroll
    for (int k = 0; k < 4; ++k)
    {
        u.s[k]     = lo[k];
        u.s[4 + k] = hi[k];
    }
    return u.h;
}

// The same for the three horizontal taps at once: pixels `pix + dx` .. `pix + dx + 7`, dx = 0, 1, 2, of column
// `col0 + lane % 16`, from three reads of four pixels (ten of the twelve are used; the last two may lie past the
// tile, inside the workgroup's LDS) instead of six: the window of dx = 2 is a whole register further, the window of
// dx = 1 is stitched together with four funnel shifts.
__device__ __forceinline__ void lds_read_pixel_windows(const _Float16* tile, int stride, int pix, int col0, half8 (&w)[3])
{
    const int i = threadIdx.x & 15;
    const _Float16* src = tile + (size_t)(pix + (i >> 2)) * stride + col0 + (i & 3) * 4;
    using lds_ptr = __attribute__((address_space(3))) short4v*;
    union
    {
        short4v v[3];
        unsigned d[6];
    } in;
    in.v[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)src);
    in.v[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(src + 4 * stride));
    in.v[2] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(src + 8 * stride));
    union
    {
        unsigned d[4];
        half8 h;
    } out;
#pragma unroll
    for (int k = 0; k < 4; ++k) out.d[k] = in.d[k];
    w[0] = out.h;
#pragma unroll
    for (int k = 0; k < 4; ++k) out.d[k] = __builtin_amdgcn_alignbit(in.d[k + 1], in.d[k], 16);
    w[1] = out.h;
#pragma unroll
    for (int k = 0; k < 4; ++k) out.d[k] = in.d[k + 1];
    w[2] = out.h;
}

// THREADS: 256, or 512 for the largest shape, whose 9 x NPAD x CIN sums are 288 registers per lane of four wavefronts.
// CI: image channels the kernel has room for (4, 8 or 16; C <= CI)
template <int CIN, int NPAD, bool BIAS, int THREADS, int CI>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(CIN == 32 && NPAD == 32 ? 4 : 1))) void conv_bwd_weight_kernel(const BwdWeightParams p)
{
    constexpr int IQ = CI / 4;  // 16-byte items that carry the image of a pixel of the level below
    constexpr int ROW    = CIN + kLdsChanPad;   // halves per pixel of the input patch
    constexpr int DS     = NPAD + kLdsChanPad;  // halves per pixel of the gradient tile
    constexpr int GROUPS = CIN / 8;
    constexpr int NB     = NPAD / 16;
    constexpr int CB     = CIN / 16;
    // The wavefronts split the NPAD x CIN result: CBW ways over the 16-channel input blocks, NBW ways over the
    // 16-channel pre-activation blocks; each keeps all 9 taps of its blocks. Per tile row a wavefront reads its A
    // fragments (pre-activation gradients, the same for every tap) once and one B fragment per tap and input block.
    constexpr int CBW    = CB < 4 ? CB : 4;
    // (More wavefronts than 16 x 16 blocks to deal out: the wavefronts also split the rows of a tile, RW ways; the
    // shares are added up through LDS at the end.)
    constexpr int WAVES  = THREADS / 64;
    constexpr int NBW    = wgrad_nbw(CIN, NPAD);
    constexpr int RW     = wgrad_row_split(CIN, NPAD);
    static_assert(THREADS == wgrad_threads(CIN, NPAD) && CBW == wgrad_cbw(CIN), "work split");
    constexpr int MYCB   = CB / CBW;
    constexpr int MYNB   = NB / NBW;
    constexpr int MYROWS = kConvTileH / RW;
    static_assert(CB % CBW == 0 && NB % NBW == 0 && CBW * NBW * RW == WAVES && kConvTileH % RW == 0, "block split");
    extern __shared__ _Float16 smem[];
    _Float16* s_patch = smem;                                           // [kConvPatchH * kConvPatchW][ROW]
    _Float16* s_below = s_patch + kConvPatchH * kConvPatchW * ROW;      // [kBelowH * kBelowW][ROW]
    _Float16* s_d     = s_below + kBelowH * kBelowW * ROW;              // [kConvTileH * kConvTileW][DS]
    const bool has_below = p.Hb > 0;
    const int C          = p.c_feat;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lk = (lane >> 4) * 8;

    const int cb0 = (wave % CBW) * MYCB, nb0 = (RW == 1 ? wave / CBW : (wave / CBW) % NBW) * MYNB;
    const int share = RW == 1 ? 0 : wave / (CBW * NBW);
    const int row0  = share * MYROWS;           // this wavefront's rows of a tile
    const int set   = blockIdx.x;               // the workgroup's set of partial sums
    floatx4 acc[9][MYNB][MYCB];
#pragma unroll
    for (int t = 0; t < 9; ++t)
#pragma unroll
        for (int n = 0; n < MYNB; ++n)
#pragma unroll
            for (int c = 0; c < MYCB; ++c) acc[t][n][c] = floatx4{0.f, 0.f, 0.f, 0.f};
    // Bias gradients = sums of the pre-activation gradients over the pixels: one more MFMA per tile row and block with
    // a matrix of ones as the other operand (every column of the result is the row sum), by the wavefronts that own
    // the first input blocks.
    floatx4 bias_acc[MYNB];
#pragma unroll
    for (int n = 0; n < MYNB; ++n) bias_acc[n] = floatx4{0.f, 0.f, 0.f, 0.f};
    half8 ones;
#pragma unroll
    for (int i = 0; i < 8; ++i) ones[i] = _Float16(1.f);

    // ---- stage 1 in two halves: every global load of a tile is issued into registers (a thread's loads are all in
    // flight together), and written to LDS one tile later, so that the loads of tile t + 1 travel while tile t is
    // upsampled and multiplied ----
    constexpr int kFeatItems  = (kConvPatchH * kConvPatchW + THREADS - 1) / THREADS;
    constexpr int kMaxPerPix  = IQ + CIN / 8;  // image below (four channels per item) + groups of 8 block outputs
    constexpr int kBelowItems = (kBelowH * kBelowW * kMaxPerPix + THREADS - 1) / THREADS;
    constexpr int kDpreGroups = NPAD / 8;  // 16-byte groups of a pixel's gradient row
    constexpr int kDpreItems  = (kConvTileH * kConvTileW * kDpreGroups + THREADS - 1) / THREADS;
    struct TileLoads
    {
        float feat[kFeatItems][CI];
        uint4 below[kBelowItems];
        half8 dpre[kDpreItems];
    };
    const int act_groups = p.cb_store / 8;
    const int per_pixel  = IQ + act_groups;
    auto issue_loads = [&](int tile, TileLoads& r)
    {
        const int ty = tile / p.tiles_x, tx = tile - ty * p.tiles_x;
        const int x0 = tx * kConvTileW, y0 = ty * kConvTileH;
        const int by0 = y0 / 2 - 1, bx0 = x0 / 2 - 1;
        const size_t plane = (size_t)p.H * p.W;
#pragma unroll
        for (int k = 0; k < kFeatItems; ++k)
        {
            const int item = threadIdx.x + THREADS * k;
            const int py = item / kConvPatchW, px = item - py * kConvPatchW;
            const int y = y0 + py - 1, x = x0 + px - 1;
            const bool in = item < kConvPatchH * kConvPatchW && y >= 0 && y < p.H && x >= 0 && x < p.W;
#pragma unroll
            for (int c = 0; c < CI; ++c) r.feat[k][c] = (in && c < C) ? p.feat[c * plane + (size_t)y * p.W + x] : 0.f;
        }
        if (has_below)
        {
            const size_t pb = (size_t)p.Hb * p.Wb;
#pragma unroll
            for (int k = 0; k < kBelowItems; ++k)
            {
                const int item = threadIdx.x + THREADS * k;
                r.below[k]     = make_uint4(0u, 0u, 0u, 0u);
                if (item < kBelowH * kBelowW * per_pixel)
                {
                    const int q = item % per_pixel, bp = item / per_pixel;
                    const int rr = bp / kBelowW, c0 = bp - rr * kBelowW;
                    const int yy = min(max(by0 + rr, 0), p.Hb - 1), xx = min(max(bx0 + c0, 0), p.Wb - 1);
                    if (q < IQ)
                    {
                        float f[4];
#pragma unroll
                        for (int c = 0; c < 4; ++c) f[c] = 4 * q + c < C ? p.feat_below[(size_t)(4 * q + c) * pb + (size_t)yy * p.Wb + xx] : 0.f;
                        r.below[k] = make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3]));
                    }
                    else
                        r.below[k] = *reinterpret_cast<const uint4*>(p.act_below + ((size_t)yy * p.Wb + xx) * p.cb_store + 8 * (q - IQ));
                }
            }
        }
#pragma unroll
        for (int k = 0; k < kDpreItems; ++k)
        {
            const int item = threadIdx.x + THREADS * k;
            const int g = item % kDpreGroups, tp = item / kDpreGroups;
            const int y = y0 + tp / kConvTileW, x = x0 + tp % kConvTileW;
#pragma unroll
            for (int i = 0; i < 8; ++i) r.dpre[k][i] = _Float16(0.f);
            if (tp < kConvTileH * kConvTileW && y < p.H && x < p.W)
                r.dpre[k] = *reinterpret_cast<const half8*>(p.dpre + ((size_t)y * p.W + x) * NPAD + 8 * g);
        }
    };
    // this level's image into channels [0, C) of a patch pixel (the channels [C, 8) follow from the upsampling, or are
    // zero for the start block, whose other channels are cleared once, below)
    auto put_image = [&](int item, const float (&v)[CI])
    {
        _Float16* row = s_patch + (size_t)item * ROW;
        if (CI == 4 && has_below && C == 4)
            *reinterpret_cast<half4*>(row) = half4{_Float16(v[0]), _Float16(v[1]), _Float16(v[2]), _Float16(v[3])};
        else if (has_below)
        {
#pragma unroll
            for (int c = 0; c < CI; ++c)  // a run-time bound would put the register array into scratch memory
                if (c < C) row[c] = _Float16(v[c]);
        }
        else
        {
            // start block: the image is the whole input; the first groups of eight written whole (v is zero past C)
#pragma unroll
            for (int g8 = 0; g8 < (CI + 7) / 8; ++g8)
            {
                half8 h;
#pragma unroll
                for (int i = 0; i < 8; ++i) h[i] = 8 * g8 + i < CI ? _Float16(v[8 * g8 + i < CI ? 8 * g8 + i : 0]) : _Float16(0.f);
                *reinterpret_cast<half8*>(row + 8 * g8) = h;
            }
        }
    };
    // four channels 4 qi .. 4 qi + 3 of the image of the level below into positions C + 4 qi .. of a below-patch pixel
    auto put_below_image = [&](int bp, int qi, const float (&v)[4])
    {
        _Float16* row = s_below + (size_t)bp * ROW;
        if (CI == 4 && C == 4)
            *reinterpret_cast<half4*>(row + 4) = half4{_Float16(v[0]), _Float16(v[1]), _Float16(v[2]), _Float16(v[3])};
        else
        {
#pragma unroll
            for (int c = 0; c < 4; ++c)
                if (4 * qi + c < C) row[C + 4 * qi + c] = _Float16(v[c]);
        }
        if (qi == 0)
            for (int c = 2 * C + p.cb_store; c < CIN; ++c) row[c] = _Float16(0.f);
    };
    // eight block outputs of the level below (item q >= IQ) into positions 2 C + 8 (q - IQ) .. of a below-patch pixel
    auto put_below_act = [&](int bp, int q, const uint4& v)
    {
        _Float16* row = s_below + (size_t)bp * ROW;
        const int pos = 2 * C + 8 * (q - IQ);
        if (C == 4)
            *reinterpret_cast<uint4*>(row + pos) = v;
        else
        {
            // (positions that are not a multiple of 8: element by element; outputs past the padded input are padding)
            const half8 a = __builtin_bit_cast(half8, v);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (pos + i < CIN) row[pos + i] = a[i];
        }
    };
    auto commit_loads = [&](const TileLoads& r)
    {
#pragma unroll
        for (int k = 0; k < kFeatItems; ++k)
        {
            const int item = threadIdx.x + THREADS * k;
            if (item < kConvPatchH * kConvPatchW) put_image(item, r.feat[k]);
        }
        if (has_below)
        {
#pragma unroll
            for (int k = 0; k < kBelowItems; ++k)
            {
                const int item = threadIdx.x + THREADS * k;
                if (item < kBelowH * kBelowW * per_pixel)
                {
                    const int q = item % per_pixel, bp = item / per_pixel;
                    if (q < IQ)
                    {
                        const float f[4] = {__uint_as_float(r.below[k].x), __uint_as_float(r.below[k].y), __uint_as_float(r.below[k].z),
                                            __uint_as_float(r.below[k].w)};
                        put_below_image(bp, q, f);
                    }
                    else
                        put_below_act(bp, q, r.below[k]);
                }
            }
        }
#pragma unroll
        for (int k = 0; k < kDpreItems; ++k)
        {
            const int item = threadIdx.x + THREADS * k;
            if (item < kConvTileH * kConvTileW * kDpreGroups)
                *reinterpret_cast<half8*>(s_d + (size_t)(item / kDpreGroups) * DS + 8 * (item % kDpreGroups)) = r.dpre[k];
        }
    };

    // the same without registers in between, for the shapes that have none to spare
    auto stream_stage1 = [&](int x0, int y0, int by0, int bx0)
    {
        {
            const size_t plane = (size_t)p.H * p.W;
            for (int item = threadIdx.x; item < kConvPatchH * kConvPatchW; item += THREADS)
            {
                const int py = item / kConvPatchW, px = item - py * kConvPatchW;
                const int y = y0 + py - 1, x = x0 + px - 1;
                const bool in = y >= 0 && y < p.H && x >= 0 && x < p.W;
                float v[CI];
#pragma unroll
                for (int c = 0; c < CI; ++c) v[c] = (in && c < C) ? p.feat[c * plane + (size_t)y * p.W + x] : 0.f;
                put_image(item, v);
            }
        }
        if (has_below)
        {
            const size_t pb = (size_t)p.Hb * p.Wb;
            for (int item = threadIdx.x; item < kBelowH * kBelowW * per_pixel; item += THREADS)
            {
                const int q = item % per_pixel, bp = item / per_pixel;
                const int r = bp / kBelowW, c0 = bp - r * kBelowW;
                const int yy = min(max(by0 + r, 0), p.Hb - 1), xx = min(max(bx0 + c0, 0), p.Wb - 1);
                if (q < IQ)
                {
                    float v[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) v[c] = 4 * q + c < C ? p.feat_below[(size_t)(4 * q + c) * pb + (size_t)yy * p.Wb + xx] : 0.f;
                    put_below_image(bp, q, v);
                }
                else
                {
                    put_below_act(bp, q, *reinterpret_cast<const uint4*>(p.act_below + ((size_t)yy * p.Wb + xx) * p.cb_store + 8 * (q - IQ)));
                }
            }
        }
        for (int item = threadIdx.x; item < kConvTileH * kConvTileW * kDpreGroups; item += THREADS)
        {
            const int g = item % kDpreGroups, tp = item / kDpreGroups;
            const int y = y0 + tp / kConvTileW, x = x0 + tp % kConvTileW;
            half8 v;
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = _Float16(0.f);
            if (y < p.H && x < p.W) v = *reinterpret_cast<const half8*>(p.dpre + ((size_t)y * p.W + x) * NPAD + 8 * g);
            *reinterpret_cast<half8*>(s_d + (size_t)tp * DS + 8 * g) = v;
        }
    };

    // start block: the channels beyond the image's groups of eight of a patch pixel are never written and stay zero
    constexpr int kImageGroups = (CI + 7) / 8;
    if (!has_below)
        for (int i = threadIdx.x; i < kConvPatchH * kConvPatchW * (GROUPS - kImageGroups); i += THREADS)
        {
            half8 z;
#pragma unroll
            for (int k = 0; k < 8; ++k) z[k] = _Float16(0.f);
            *reinterpret_cast<half8*>(s_patch + (size_t)(i / (GROUPS - kImageGroups)) * ROW + 8 * (kImageGroups + i % (GROUPS - kImageGroups))) = z;
        }

    // with 64 input channels and more than 64 pre-activations the accumulators leave no registers for a tile in flight
    constexpr bool kPrefetch = !(CIN == 64 && NPAD > 64);
    TileLoads cur;
    if (kPrefetch && (int)blockIdx.x < p.tiles) issue_loads(blockIdx.x, cur);
    for (int tile = blockIdx.x; tile < p.tiles; tile += gridDim.x)
    {
        const int ty = tile / p.tiles_x, tx = tile - ty * p.tiles_x;
        const int x0 = tx * kConvTileW, y0 = ty * kConvTileH;
        const int by0 = y0 / 2 - 1, bx0 = x0 / 2 - 1;
        __syncthreads();  // the previous tile's operands have been consumed (and the zero fill is done)
        if (!kPrefetch)
            stream_stage1(x0, y0, by0, bx0);
        else
            commit_loads(cur);
        if (kPrefetch && tile + (int)gridDim.x < p.tiles) issue_loads(tile + gridDim.x, cur);  // travels during stage 2 and the taps
        if (has_below)
        {
            __syncthreads();
            // ---- stage 2: bilinear 2x upsampling from the below patch into channels [C, CIN) of the patch, in packed
            // fp16 exactly as the forward kernel does it (the weights are products of 0, 1/4, 3/4 and 1) ----
            for (int item = threadIdx.x; item < kConvPatchH * kConvPatchW * GROUPS; item += THREADS)
            {
                const int g = item % GROUPS, pp = item / GROUPS;
                const int py = pp / kConvPatchW, px = pp - py * kConvPatchW;
                const int y = y0 + py - 1, x = x0 + px - 1;
                half8 h;
#pragma unroll
                for (int i = 0; i < 8; ++i) h[i] = _Float16(0.f);
                if (y >= 0 && y < p.H && x >= 0 && x < p.W)
                {
                    int ya, yb, xa, xb;
                    float ly, lx;
                    up2_source(y, p.Hb, ya, yb, ly);
                    up2_source(x, p.Wb, xa, xb, lx);
                    const _Float16 w00 = _Float16((1.f - ly) * (1.f - lx)), w01 = _Float16((1.f - ly) * lx);
                    const _Float16 w10 = _Float16(ly * (1.f - lx)), w11 = _Float16(ly * lx);
                    const half8 a = *reinterpret_cast<const half8*>(s_below + ((ya - by0) * kBelowW + (xa - bx0)) * ROW + 8 * g);
                    const half8 b = *reinterpret_cast<const half8*>(s_below + ((ya - by0) * kBelowW + (xb - bx0)) * ROW + 8 * g);
                    const half8 c = *reinterpret_cast<const half8*>(s_below + ((yb - by0) * kBelowW + (xa - bx0)) * ROW + 8 * g);
                    const half8 d = *reinterpret_cast<const half8*>(s_below + ((yb - by0) * kBelowW + (xb - bx0)) * ROW + 8 * g);
                    const half8 W00 = {w00, w00, w00, w00, w00, w00, w00, w00}, W01 = {w01, w01, w01, w01, w01, w01, w01, w01};
                    const half8 W10 = {w10, w10, w10, w10, w10, w10, w10, w10}, W11 = {w11, w11, w11, w11, w11, w11, w11, w11};
                    h = __builtin_elementwise_fma(d, W11, __builtin_elementwise_fma(c, W10, __builtin_elementwise_fma(b, W01, a * W00)));
                }
                _Float16* dst = s_patch + (size_t)pp * ROW + 8 * g;
                if (8 * g < C)
                {
                    // [0, C) holds this level's image
                    if (CI == 4 && C == 4)
                        *reinterpret_cast<half4*>(dst + 4) = half4{h[4], h[5], h[6], h[7]};
                    else
                    {
#pragma unroll
                        for (int i = 0; i < 8; ++i)
                            if (8 * g + i >= C) dst[i] = h[i];
                    }
                }
                else
                    *reinterpret_cast<half8*>(dst) = h;
            }
        }
        __syncthreads();
        // ---- dW[tap][n][c] += sum over the tile's pixels of dpre[pixel][n] * x[pixel + tap][c] ----
#pragma unroll
        for (int r = row0; r < row0 + MYROWS; ++r)
        {
            half8 a[MYNB];
#pragma unroll
            for (int n = 0; n < MYNB; ++n)
            {
                a[n] = lds_read_pixels_of_channel(s_d, DS, r * kConvTileW + lk, (nb0 + n) * 16);
                if (BIAS && cb0 == 0) bias_acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[n], ones, bias_acc[n], 0, 0, 0);
            }
#pragma unroll
            for (int dy = 0; dy < 3; ++dy)
            {
#pragma unroll
                for (int c = 0; c < MYCB; ++c)
                {
                    half8 b[3];
                    lds_read_pixel_windows(s_patch, ROW, (r + dy) * kConvPatchW + lk, (cb0 + c) * 16, b);
#pragma unroll
                    for (int dx = 0; dx < 3; ++dx)
#pragma unroll
                        for (int n = 0; n < MYNB; ++n)
                            acc[3 * dy + dx][n][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b[dx], a[n], acc[3 * dy + dx][n][c], 0, 0, 0);
                }
            }
        }
    }

    if (RW > 1)
    {
        // the row shares of a workgroup add their sums up through LDS (the tiles are consumed), so that the workgroup
        // writes one set: share s > 0 leaves its registers there, share 0 adds them
        static_assert(RW <= 2, "row shares");
        __syncthreads();
        floatx4* s_sum = reinterpret_cast<floatx4*>(smem);  // [wavefront of the share][tap and bias][block][lane]
        constexpr int PER_WAVE = (9 * MYNB * MYCB + MYNB) * 64;
        floatx4* mine = s_sum + (size_t)(wave % (CBW * NBW)) * PER_WAVE + lane;
        if (share > 0)
        {
#pragma unroll
            for (int t = 0; t < 9; ++t)
#pragma unroll
                for (int n = 0; n < MYNB; ++n)
#pragma unroll
                    for (int c = 0; c < MYCB; ++c) mine[((t * MYNB + n) * MYCB + c) * 64] = acc[t][n][c];
#pragma unroll
            for (int n = 0; n < MYNB; ++n) mine[(9 * MYNB * MYCB + n) * 64] = bias_acc[n];
        }
        __syncthreads();
        if (share > 0) return;
#pragma unroll
        for (int t = 0; t < 9; ++t)
#pragma unroll
            for (int n = 0; n < MYNB; ++n)
#pragma unroll
                for (int c = 0; c < MYCB; ++c) acc[t][n][c] += mine[((t * MYNB + n) * MYCB + c) * 64];
#pragma unroll
        for (int n = 0; n < MYNB; ++n) bias_acc[n] += mine[(9 * MYNB * MYCB + n) * 64];
    }
    if (BIAS && cb0 == 0 && (lane & 15) == 0)
    {
        // column 0 of the row sums: this lane holds rows (lane / 16) * 4 .. + 3 of every block
        float* dst = p.bias_part + (size_t)set * NPAD;
#pragma unroll
        for (int n = 0; n < MYNB; ++n)
#pragma unroll
            for (int i = 0; i < 4; ++i) dst[(nb0 + n) * 16 + (lane >> 4) * 4 + i] = bias_acc[n][i];
    }
    float* part = p.part + (size_t)set * 9 * NPAD * CIN;
    const int lrow = lane & 15;
    // (the input channels are the rows of the MFMA result: a lane holds four neighbouring ones of output lrow)
#pragma unroll
    for (int tap = 0; tap < 9; ++tap)
#pragma unroll
        for (int n = 0; n < MYNB; ++n)
#pragma unroll
            for (int c = 0; c < MYCB; ++c)
                *reinterpret_cast<float4*>(part + ((size_t)tap * NPAD + (nb0 + n) * 16 + lrow) * CIN + (cb0 + c) * 16 + (lane >> 4) * 4) =
                    make_float4(acc[tap][n][c][0], acc[tap][n][c][1], acc[tap][n][c][2], acc[tap][n][c][3]);
}

// Sum of the partial weight gradients of all workgroups (and images), in two steps so that many loads are in
// flight and every load is a full line: slice y of kReduceSlices sums its share of the partials element by element
// (consecutive threads = consecutive elements), then the slices are summed into the reference's [Cout][Cin][3][3].
// All levels in one launch each (the level is blockIdx.z): a launch per level and step costs more than the sums.
constexpr int kReduceSlices = 16;
struct ReduceLevel
{
    const float* part;  // [groups][total]
    float* sliced;      // [kReduceSlices][total]
    int groups, total;
    int cout, cin_real, cin_pad, npad;
    float *d_wf, *d_wm;
    const float* bias_part;  // [groups][npad] or nullptr
    float *d_bf, *d_bm;
};
struct ReduceTable
{
    ReduceLevel lv[TRIPS_UNET_MAX_LEVELS];
    float scale_inv;
};
__global__ __launch_bounds__(256) void reduce_weight_grad_slices_kernel(const ReduceTable t)
{
    const ReduceLevel& l = t.lv[blockIdx.z];
    const float* __restrict__ part = l.part;
    float* __restrict__ sliced     = l.sliced;
    const int groups = l.groups, total = l.total;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int per = (groups + kReduceSlices - 1) / kReduceSlices;
    const int g0 = blockIdx.y * per, g1 = min(groups, g0 + per);
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    int g = g0;
    for (; g + 4 <= g1; g += 4)
    {
        s0 += part[(size_t)g * total + i];
        s1 += part[(size_t)(g + 1) * total + i];
        s2 += part[(size_t)(g + 2) * total + i];
        s3 += part[(size_t)(g + 3) * total + i];
    }
    for (; g < g1; ++g) s0 += part[(size_t)g * total + i];
    sliced[(size_t)blockIdx.y * total + i] = (s0 + s1) + (s2 + s3);
}

// ... and, in the workgroups behind those of the weights, the bias gradients from the per-workgroup sums
__global__ __launch_bounds__(256) void reduce_weight_grad_kernel(const ReduceTable t)
{
    const ReduceLevel& l = t.lv[blockIdx.z];
    const float* __restrict__ sliced = l.sliced;
    const int cout = l.cout, cin_real = l.cin_real, cin_pad = l.cin_pad, npad = l.npad;
    const float scale_inv = t.scale_inv;
    float* __restrict__ d_wf = l.d_wf;
    float* __restrict__ d_wm = l.d_wm;
    const int total = 9 * npad * cin_pad;
    const int wblocks = (total + 255) / 256;
    if ((int)blockIdx.x >= wblocks)
    {
        // one workgroup per pre-activation channel
        const int n = blockIdx.x - wblocks, half = npad / 2;
        if (n >= npad || !l.bias_part) return;
        const int o = n < half ? n : n - half;
        float* dst  = n < half ? l.d_bf : l.d_bm;
        if (o >= cout || !dst) return;
        const float s = block_column_sum(l.bias_part, l.groups, npad, n);
        if (threadIdx.x == 0) dst[o] = s * scale_inv;
        return;
    }
    const int i     = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int c = i % cin_pad, n = (i / cin_pad) % npad, tap = i / (cin_pad * npad);
    const int half = npad / 2;
    const int o    = n < half ? n : n - half;
    if (o >= cout || c >= cin_real) return;
    float* dst = n < half ? d_wf : d_wm;
    if (!dst) return;
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < kReduceSlices; ++k) s += sliced[(size_t)k * total + i];
    dst[((size_t)o * cin_real + c) * 9 + tap] = s * scale_inv;
}

// ---------------------------------------------------------------------------------------------------------
namespace
{
template <int KC, int NN, int CI>
hipError_t launch_bwd_data(const BwdDataParams& p, hipStream_t stream)
{
    // the patch and the staged taps of the weights
    const size_t lds_in  = ((size_t)kConvPatchH * kConvPatchW * (KC + kLdsChanPad) + ConvTapStage<KC, NN, 512>::LDS_HALVES) * sizeof(_Float16);
    const size_t lds_out = (size_t)kConvTileH * kConvTileW * ((NN + kLdsChanPad) * sizeof(_Float16) + CI * sizeof(float));
    const size_t lds     = std::max(lds_in, lds_out);
    constexpr int THREADS = 512;  // eight wavefronts per tile, as in the forward convolution
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_bwd_data_kernel<KC, NN, THREADS, CI>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    dim3 grid((p.W + kConvTileW - 1) / kConvTileW, (p.H + kConvTileH - 1) / kConvTileH);
    hipLaunchKernelGGL((conv_bwd_data_kernel<KC, NN, THREADS, CI>), grid, dim3(THREADS), lds, stream, p);
    return hipGetLastError();
}

hipError_t dispatch_bwd_data(const BwdDataParams& p, int npad, int cin_pad, hipStream_t stream)
{
#define TRIPS_BD(KC_, NN_)                                                                   \
    if (npad == KC_ && cin_pad == NN_)                                                       \
        return p.c_feat <= 4 ? launch_bwd_data<KC_, NN_, 4>(p, stream)                       \
                             : p.c_feat <= 8 ? launch_bwd_data<KC_, NN_, 8>(p, stream) : launch_bwd_data<KC_, NN_, 16>(p, stream);
    TRIPS_BD(32, 32) TRIPS_BD(64, 32) TRIPS_BD(96, 32) TRIPS_BD(128, 32)
    TRIPS_BD(32, 64) TRIPS_BD(64, 64) TRIPS_BD(96, 64) TRIPS_BD(128, 64)
#undef TRIPS_BD
    return hipErrorInvalidValue;
}

template <int CIN, int NPAD, bool BIAS, int CI>
hipError_t launch_bwd_weight(const BwdWeightParams& p, int groups, hipStream_t stream)
{
    constexpr int THREADS = wgrad_threads(CIN, NPAD);
    const size_t lds = ((size_t)(kConvPatchH * kConvPatchW + kBelowH * kBelowW) * (CIN + kLdsChanPad) +
                        (size_t)kConvTileH * kConvTileW * (NPAD + kLdsChanPad)) *
                       sizeof(_Float16);  // up to 133 KB
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_bwd_weight_kernel<CIN, NPAD, BIAS, THREADS, CI>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((conv_bwd_weight_kernel<CIN, NPAD, BIAS, THREADS, CI>), dim3(groups), dim3(THREADS), lds, stream, p);
    return hipGetLastError();
}

template <int CI>
hipError_t dispatch_bwd_weight_ci(const BwdWeightParams& p, int cin_pad, int npad, int groups, hipStream_t stream)
{
#define TRIPS_BW(CIN_, NPAD_)                                                                  \
    if (cin_pad == CIN_ && npad == NPAD_)                                                      \
        return p.bias_part ? launch_bwd_weight<CIN_, NPAD_, true, CI>(p, groups, stream) \
                                          : launch_bwd_weight<CIN_, NPAD_, false, CI>(p, groups, stream);
    TRIPS_BW(32, 32) TRIPS_BW(32, 64) TRIPS_BW(32, 96) TRIPS_BW(32, 128)
    TRIPS_BW(64, 32) TRIPS_BW(64, 64) TRIPS_BW(64, 96) TRIPS_BW(64, 128)
#undef TRIPS_BW
    return hipErrorInvalidValue;
}

hipError_t dispatch_bwd_weight(const BwdWeightParams& p, int cin_pad, int npad, int groups, hipStream_t stream)
{
    if (p.c_feat <= 4) return dispatch_bwd_weight_ci<4>(p, cin_pad, npad, groups, stream);
    if (p.c_feat <= 8) return dispatch_bwd_weight_ci<8>(p, cin_pad, npad, groups, stream);
    return dispatch_bwd_weight_ci<16>(p, cin_pad, npad, groups, stream);
}
}  // namespace
}  // namespace trips

using namespace trips;

extern "C" {

int trips_unet_backward_workspace_size(const TripsUnetDesc* desc, size_t* bytes)
{
    if (int e = check_unet_desc(desc)) return e;
    if (!bytes) return set_error(TRIPS_ERR_INVALID_ARG, "bytes is NULL");
    *bytes = make_plan(*desc).backward_bytes;
    return TRIPS_OK;
}

int trips_unet_backward(TripsCtx* ctx, const TripsUnetDesc* desc, const TripsUnetWeights* weights,
                        const float* const inputs[TRIPS_UNET_MAX_LEVELS], const void* saved, const float* d_output,
                        float grad_scale, const TripsUnetGrads* grads, void* workspace, size_t workspace_bytes,
                        void* stream_)
{
    if (!ctx) return set_error(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    if (int e = check_unet_desc(desc)) return e;
    if (!weights || !inputs || !saved || !d_output || !grads || !workspace) return set_error(TRIPS_ERR_INVALID_ARG, "NULL argument");
    const TripsUnetDesc& d = *desc;
    const int C = d.num_input_channels, L = d.num_levels;
    if (!(grad_scale > 0.f) || !std::isfinite(grad_scale)) return set_error(TRIPS_ERR_INVALID_ARG, "grad_scale must be positive");
    for (int i = 0; i < L; ++i)
    {
        if (!inputs[i]) return set_error(TRIPS_ERR_INVALID_ARG, "inputs[%d] is NULL", i);
        if (!grads->inputs[i]) return set_error(TRIPS_ERR_INVALID_ARG, "grads->inputs[%d] is NULL", i);
        if (!weights->feature_weight[i] || !weights->mask_weight[i])
            return set_error(TRIPS_ERR_INVALID_ARG, "weights of block %d are NULL", i);
    }
    if (!weights->final_weight) return set_error(TRIPS_ERR_INVALID_ARG, "final weights are NULL");
    if ((reinterpret_cast<uintptr_t>(workspace) & 255) || (reinterpret_cast<uintptr_t>(saved) & 255))
        return set_error(TRIPS_ERR_INVALID_ARG, "workspace / saved must be 256-byte aligned");
    const NetPlan np = make_plan(d);
    if (workspace_bytes < np.backward_bytes)
        return set_error(TRIPS_ERR_WORKSPACE_SMALL, "workspace has %zu bytes, %zu needed", workspace_bytes, np.backward_bytes);
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    char* ws           = reinterpret_cast<char*>(workspace);
    const char* sv     = reinterpret_cast<const char*>(saved);
    Profiler* prof     = ctx->prof.enabled ? &ctx->prof : nullptr;
    const float scale_inv = 1.f / grad_scale;
    const int K           = d.num_output_channels;
    const int ci          = C <= 4 ? 4 : C <= 8 ? 8 : 16;  // image channels the kernels are built with room for

    auto act_ptr = [&](int level, int b)
    {
        const LevelPlan& l = np.lv[level];
        return reinterpret_cast<const _Float16*>(sv + l.saved_act_off) + (size_t)b * l.H * l.W * l.cout_store;
    };
    auto pre_ptr = [&](int level, int b)
    {
        const LevelPlan& l = np.lv[level];
        return reinterpret_cast<const _Float16*>(sv + l.saved_pre_off) + (size_t)b * l.H * l.W * l.npad;
    };
    auto dpre_ptr = [&](int level, int b)
    {
        const LevelPlan& l = np.lv[level];
        return reinterpret_cast<_Float16*>(ws + l.dpre_off) + (size_t)b * l.H * l.W * l.npad;
    };
    auto din_ptr = [&](int level, int b)
    {
        const LevelPlan& l = np.lv[level];
        return reinterpret_cast<_Float16*>(ws + l.din_off) + (size_t)b * l.H * l.W * l.cin_pad;
    };
    auto fill = [&](float* p, int n)
    {
        if (p && n > 0) hipLaunchKernelGGL(fill_f32_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, p, 0.f, n);
    };

    {
        ProfScope ps(prof, "unet_bwd_prepare", stream);
        PackTTable pt;
        int most = 0;
        for (int i = 0; i < L; ++i)
        {
            const LevelPlan& lv = np.lv[i];
            pt.lv[i] = PackTLevel{weights->feature_weight[i], weights->mask_weight[i], lv.cout, lv.cin_real, lv.cin_pad, lv.npad,
                                  reinterpret_cast<_Float16*>(ws + lv.wt_off)};
            most     = std::max(most, 9 * lv.npad * lv.cin_pad);
        }
        hipLaunchKernelGGL(pack_conv_weights_T_kernel, dim3((most + 255) / 256, L), dim3(256), 0, stream, pt);
        for (int i = 0; i < L; ++i)
        {
            const LevelPlan& lv = np.lv[i];
            if (!grads->feature_weight[i] && !grads->mask_weight[i])  // bias_grad_kernel accumulates; otherwise they are written
            {
                fill(grads->feature_bias[i], lv.cout);
                fill(grads->mask_bias[i], lv.cout);
            }
        }
    }
    {
        ProfScope ps(prof, "unet_bwd_final", stream);
        const LevelPlan& lv = np.lv[0];
        const size_t plane  = (size_t)lv.H * lv.W;
        for (int b = 0; b < d.batch; ++b)
        {
            FinalBwdParams p;
            std::memset(&p, 0, sizeof(p));
            p.H = lv.H, p.W = lv.W, p.c_feat = C, p.cact = lv.cout, p.cact_store = lv.cout_store, p.cout = K, p.npad = lv.npad;
            p.scale    = grad_scale;
            p.feat     = inputs[0] + (size_t)b * C * plane;
            p.pre      = pre_ptr(0, b);
            p.weight   = weights->final_weight;
            p.d_out    = d_output + (size_t)b * K * plane;
            p.d_feat   = grads->inputs[0] + (size_t)b * C * plane;
            p.dpre     = dpre_ptr(0, b);
            p.chunks   = (int)((plane + kFinalPixelsPerBlock - 1) / kFinalPixelsPerBlock);
            p.part     = reinterpret_cast<float*>(ws + np.final_part_off) + (size_t)b * np.final_groups * (4 * (ci + lv.cout_store) + 4);
            const bool wgrad = grads->final_weight || grads->final_bias;
            const int chunks = wgrad ? np.final_groups : p.chunks;
            switch (lv.cout_store)
            {
#define TRIPS_FW_CI(CS_, CI_)                                                                                     \
    if (wgrad)                                                                                                    \
        hipLaunchKernelGGL((final_backward_kernel<CS_, true, CI_>), dim3(chunks), dim3(256), 0, stream, p);       \
    else                                                                                                          \
        hipLaunchKernelGGL((final_backward_kernel<CS_, false, CI_>), dim3(chunks), dim3(256), 0, stream, p);
#define TRIPS_FW(CS_)                \
    case CS_:                        \
        if (ci == 4)                 \
        {                            \
            TRIPS_FW_CI(CS_, 4)      \
        }                            \
        else if (ci == 8)            \
        {                            \
            TRIPS_FW_CI(CS_, 8)      \
        }                            \
        else                         \
        {                            \
            TRIPS_FW_CI(CS_, 16)     \
        }                            \
        break;
                TRIPS_FW(8) TRIPS_FW(16) TRIPS_FW(24) TRIPS_FW(32) TRIPS_FW(40) TRIPS_FW(48) TRIPS_FW(56) TRIPS_FW(64)
#undef TRIPS_FW
#undef TRIPS_FW_CI
                default: return set_error(TRIPS_ERR_UNSUPPORTED, "block output stride %d", lv.cout_store);
            }
        }
        if (grads->final_weight || grads->final_bias)
        {
            hipLaunchKernelGGL(final_reduce_kernel, dim3(K * (C + lv.cout) + K), dim3(256), 0, stream,
                               reinterpret_cast<const float*>(ws + np.final_part_off), d.batch * np.final_groups, ci + lv.cout_store, ci, C,
                               lv.cout, K, grads->final_weight, grads->final_bias);
        }
    }
    static const char* const kDataNames[TRIPS_UNET_MAX_LEVELS]   = {"unet_bwd_data_l0", "unet_bwd_data_l1", "unet_bwd_data_l2", "unet_bwd_data_l3",
                                                                    "unet_bwd_data_l4", "unet_bwd_data_l5", "unet_bwd_data_l6", "unet_bwd_data_l7"};
    static const char* const kWeightNames[TRIPS_UNET_MAX_LEVELS] = {"unet_bwd_weight_l0", "unet_bwd_weight_l1", "unet_bwd_weight_l2", "unet_bwd_weight_l3",
                                                                    "unet_bwd_weight_l4", "unet_bwd_weight_l5", "unet_bwd_weight_l6", "unet_bwd_weight_l7"};
    for (int i = 0; i < L; ++i)
    {
        const LevelPlan& lv = np.lv[i];
        const size_t plane  = (size_t)lv.H * lv.W;
        const bool below    = i < L - 1;
        {
            ProfScope ps(prof, kWeightNames[i], stream);
            for (int b = 0; b < d.batch; ++b)
            {
                BiasGradParams bp;
                bp.pixels    = plane;
                bp.npad      = lv.npad;
                bp.cout      = lv.cout;
                bp.scale_inv = scale_inv;
                bp.dpre      = dpre_ptr(i, b);
                bp.d_bias_f  = grads->feature_bias[i];
                bp.d_bias_m  = grads->mask_bias[i];
                const bool want_w = grads->feature_weight[i] || grads->mask_weight[i];
                if ((bp.d_bias_f || bp.d_bias_m) && !want_w)  // otherwise the weight-gradient kernel sums them on its way
                    hipLaunchKernelGGL(bias_grad_kernel, dim3((unsigned)((plane + kBiasChunk - 1) / kBiasChunk)), dim3(256), 0, stream, bp);

                BwdWeightParams wp;
                std::memset(&wp, 0, sizeof(wp));
                wp.H = lv.H, wp.W = lv.W, wp.c_feat = C;
                wp.tiles_x = (lv.W + kConvTileW - 1) / kConvTileW;
                wp.tiles   = wp.tiles_x * ((lv.H + kConvTileH - 1) / kConvTileH);
                wp.feat    = inputs[i] + (size_t)b * C * plane;
                wp.dpre    = dpre_ptr(i, b);
                wp.part    = reinterpret_cast<float*>(ws + lv.part_off) + (size_t)b * lv.groups * 9 * lv.npad * lv.cin_pad;
                if (bp.d_bias_f || bp.d_bias_m)
                    wp.bias_part = reinterpret_cast<float*>(ws + lv.bias_part_off) + (size_t)b * lv.groups * lv.npad;
                if (below)
                {
                    const LevelPlan& lb = np.lv[i + 1];
                    wp.Hb = lb.H, wp.Wb = lb.W, wp.cb_store = lb.cout_store;
                    wp.feat_below = inputs[i + 1] + (size_t)b * C * lb.H * lb.W;
                    wp.act_below  = act_ptr(i + 1, b);
                }
                if (grads->feature_weight[i] || grads->mask_weight[i])
                {
                    hipError_t e = dispatch_bwd_weight(wp, lv.cin_pad, lv.npad, lv.groups, stream);
                    if (e != hipSuccess) return set_error(TRIPS_ERR_HIP, "weight gradient launch (level %d): %s", i, hipGetErrorString(e));
                }
            }
        }
        {
            ProfScope ps(prof, kDataNames[i], stream);
            for (int b = 0; b < d.batch; ++b)
            {
                BwdDataParams dp;
                dp.H = lv.H, dp.W = lv.W, dp.c_feat = C;
                dp.scale_inv = scale_inv;
                dp.dpre      = dpre_ptr(i, b);
                dp.wt        = reinterpret_cast<const _Float16*>(ws + lv.wt_off);
                dp.d_feat    = grads->inputs[i] + (size_t)b * C * plane;
                dp.d_in      = below ? din_ptr(i, b) : nullptr;
                hipError_t e = dispatch_bwd_data(dp, lv.npad, lv.cin_pad, stream);
                if (e != hipSuccess) return set_error(TRIPS_ERR_HIP, "data gradient launch (level %d): %s", i, hipGetErrorString(e));
                if (below)
                {
                    const LevelPlan& lb = np.lv[i + 1];
                    UpAdjointParams up;
                    up.H = lv.H, up.W = lv.W, up.Hb = lb.H, up.Wb = lb.W;
                    up.cin_fine  = lv.cin_pad;
                    up.c_feat    = C;
                    up.cout      = lb.cout;
                    up.npad      = lb.npad;
                    up.scale_inv = scale_inv;
                    up.d_in      = din_ptr(i, b);
                    up.pre       = pre_ptr(i + 1, b);
                    up.d_feat    = grads->inputs[i + 1] + (size_t)b * C * lb.H * lb.W;
                    up.dpre      = dpre_ptr(i + 1, b);
                    const size_t items = (size_t)lb.H * lb.W * ((2 * C - 1) / 8 - C / 8 + 1 + lb.npad / 16);
                    const int blocks   = (int)std::min<size_t>((items + 255) / 256, 1u << 20);
                    switch ((2 * C) & 7)
                    {
                        case 0: hipLaunchKernelGGL(up2_adjoint_gate_kernel<0>, dim3(blocks), dim3(256), 0, stream, up); break;
                        case 2: hipLaunchKernelGGL(up2_adjoint_gate_kernel<2>, dim3(blocks), dim3(256), 0, stream, up); break;
                        case 4: hipLaunchKernelGGL(up2_adjoint_gate_kernel<4>, dim3(blocks), dim3(256), 0, stream, up); break;
                        default: hipLaunchKernelGGL(up2_adjoint_gate_kernel<6>, dim3(blocks), dim3(256), 0, stream, up); break;
                    }
                }
            }
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return set_error(TRIPS_ERR_HIP, "backward launch (level %d): %s", i, hipGetErrorString(e));
    }
    // the partial weight and bias gradients of all levels are summed at the end, one launch per step of the sum
    {
        ProfScope ps(prof, "unet_bwd_reduce", stream);
        ReduceTable rt;
        rt.scale_inv = scale_inv;
        int n = 0, most = 0, most_npad = 0;
        for (int i = 0; i < L; ++i)
        {
            const LevelPlan& lv = np.lv[i];
            if (!grads->feature_weight[i] && !grads->mask_weight[i]) continue;
            ReduceLevel& r = rt.lv[n++];
            r.part      = reinterpret_cast<const float*>(ws + lv.part_off);
            r.sliced    = reinterpret_cast<float*>(ws + lv.sliced_off);
            r.groups    = d.batch * lv.groups;
            r.total     = 9 * lv.npad * lv.cin_pad;
            r.cout = lv.cout, r.cin_real = lv.cin_real, r.cin_pad = lv.cin_pad, r.npad = lv.npad;
            r.d_wf = grads->feature_weight[i], r.d_wm = grads->mask_weight[i];
            const bool bias = grads->feature_bias[i] || grads->mask_bias[i];
            r.bias_part = bias ? reinterpret_cast<const float*>(ws + lv.bias_part_off) : nullptr;
            r.d_bf = grads->feature_bias[i], r.d_bm = grads->mask_bias[i];
            most      = std::max(most, r.total);
            most_npad = std::max(most_npad, lv.npad);
        }
        if (n > 0)
        {
            hipLaunchKernelGGL(reduce_weight_grad_slices_kernel, dim3((most + 255) / 256, kReduceSlices, n), dim3(256), 0, stream, rt);
            hipLaunchKernelGGL(reduce_weight_grad_kernel, dim3((most + 255) / 256 + most_npad, 1, n), dim3(256), 0, stream, rt);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return set_error(TRIPS_ERR_HIP, "gradient sums launch: %s", hipGetErrorString(e));
        }
    }
    return TRIPS_OK;
}

}  // extern "C"
