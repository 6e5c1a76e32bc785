// Forward of the decoder-only gated-convolution U-Net on the gfx950 matrix cores.
//
//   gated_conv3x3_kernel <- SmallDecStartBlockImpl::forward / UpsampleDecOnlySmallBlockFixedImpl::forward
//                           src/lib/models/Networks.h:751-787, 999-1098
//                           and, in the finest block's epilogue, the `final` 1x1 Sequential of
//                           MultiScaleUnet2dDecOnlySmallFixedImpl, Networks.h:1129-1131
//
// The reference runs, per level, upsample -> cat -> two 3x3 convolutions -> elu / sigmoid -> multiply -> cat as
// separate libtorch ops on NCHW tensors, materialising every intermediate. Here one kernel per level does all of
// it as an implicit GEMM: M = 256 output pixels of an 8 x 32 patch, N = feature and mask outputs side by side,
// K = 9 taps x input channels. The input patch (with its one-pixel halo) is assembled in LDS, channels innermost:
// channels [0, C) come straight from this level's splat image, the others are the bilinear 2x upsampling of the
// level below (its splat image, then its convolution outputs), computed while loading, so neither the upsampled
// tensor nor the concatenations ever exist in memory. Activations between levels are fp16, channels innermost.
// MFMA: v_mfma_f32_16x16x32_f16; lane l holds, of A, row l % 16 and the 8 consecutive K values (l / 16) * 8 ..,
// of B the same for column l % 16, and of the 16 x 16 result rows (l / 16) * 4 .. + 3 of column l % 16.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstring>

#include "unet_common.h"

namespace trips
{
struct ConvParams
{
    int H, W;            // this level
    int Hb, Wb;          // level below (0 x 0 for the start block)
    int c_feat;          // channels of the splat images (C)
    int cb_store;        // halves per pixel of act_below (multiple of 8; channels past the real ones hold zero)
    int cout;            // real outputs of each of the two convolutions
    int cout_store;      // halves per pixel of `out` (multiple of 8)
    const float* feat;        // [C][H][W]
    const float* feat_below;  // [C][Hb][Wb]
    const _Float16* act_below;  // [Hb][Wb][cb_store]
    const _Float16* wpack;    // [9][NPAD][CIN]
    const float* bias;        // [NPAD]: feature biases, then mask biases, each padded to NPAD / 2
    _Float16* out;            // [H][W][cout_store], or nullptr when only the fused 1x1 consumes the block's output
    _Float16* pre;            // [H][W][NPAD] pre-activations (feature | mask) for the backward, or nullptr
    // the finest block also applies the net's 1x1 output convolution to x_0 = cat(image, block output)
    const float* final_w;     // [final_cout][C + cout] or nullptr
    const float* final_b;     // [final_cout]
    float* final_out;         // [final_cout][H][W]
    int final_cout;
};

// A loaded value that is only needed under a condition is otherwise loaded under that condition by the compiler, in a
// branch that waits for it before it ends. Values passed through here exist where this is called, whatever they are
// used for later: called for all loads of a stage after the last of them, it keeps them in flight together.
__device__ __forceinline__ void loaded(float& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void loaded(uint4& v) { asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w)); }

// CI: image channels the kernel has room for (4, 8 or 16; C <= CI)
template <int CIN, int NPAD, int THREADS, int CI>
__global__ __launch_bounds__(THREADS) void gated_conv3x3_kernel(const ConvParams p)
{
    constexpr int IQ = CI / 4;  // 16-byte items that carry the image of a pixel of the level below
    constexpr int MB = 16 / (THREADS / 64);  // 16-pixel row blocks of a wavefront: two rows of the tile, or one
    constexpr int ROW  = CIN + kLdsChanPad;  // halves per patch pixel in LDS
    constexpr int NB   = NPAD / 16;          // 16-column blocks; the first half are feature outputs
    constexpr int HB   = NB / 2;
    extern __shared__ _Float16 smem[];
    _Float16* s_patch = smem;  // [kConvPatchH * kConvPatchW][ROW]

    const int x0 = blockIdx.x * kConvTileW, y0 = blockIdx.y * kConvTileH;
    const bool has_below = p.Hb > 0;
    ConvTapStage<CIN, NPAD, THREADS> taps;
    conv_tap_fetch(taps, p.wpack, 0);  // in flight while the patch is assembled
    // weights and biases of the 1x1 output convolution, rounded to fp16 like every other operand
    constexpr int kFwBias = 4 * (CI + 64);  // [final_cout <= 4][C + cout <= CI + 64] weights, then the biases
    __shared__ float s_fw[kFwBias + 4];

    // ---- stage 1: everything the patch needs from memory, all loads of a thread in flight together ----
    // (a) this level's image -> channels [0, C) of the patch; (b) the level below, x_{i+1} = cat(image, activations),
    // as a (TILE/2 + 2)^2 patch in the same row format, channel k of the concatenated input at row position k.
    // Every load below is unconditional, at an address clamped into its array, and what a thread does not need is
    // replaced by zero afterwards: a load inside a branch is waited for before the branch is left, and the eight or
    // nine round trips to memory of a thread then ran one after the other (72 % of a tile's life at the finest level).
    constexpr int GROUPS = CIN / 8;
    _Float16* s_below    = s_patch + kConvPatchH * kConvPatchW * ROW;  // [kBelowH * kBelowW][ROW]
    const int by0 = y0 / 2 - 1, bx0 = x0 / 2 - 1;
    const int C   = p.c_feat;
    constexpr int kFeatItems  = (kConvPatchH * kConvPatchW + THREADS - 1) / THREADS;
    constexpr int kMaxPerPix  = IQ + CIN / 8;  // image below (four channels per item) + groups of 8 block outputs
    constexpr int kBelowItems = (kBelowH * kBelowW * kMaxPerPix + THREADS - 1) / THREADS;
    float feat_v[kFeatItems][CI];
    bool feat_in[kFeatItems];
    uint4 below_v[kBelowItems];
    float below_f[kBelowItems][4];
    bool below_have[kBelowItems], below_img[kBelowItems];
    const int act_groups = has_below ? p.cb_store / 8 : 0;
    const int per_pixel  = IQ + act_groups;  // items 0 .. IQ - 1 of a pixel: the image below; others: 8 activations each
    // item / per_pixel without an integer division: items stay below 2^11 and per_pixel below 2^5, so the quotient of
    // item + 1/2 is at least 1/64 away from every integer, far more than the rounding of the product
    const float inv_per_pixel = 1.f / float(per_pixel);
    auto pixel_of_item        = [&](int item) { return (int)((float(item) + 0.5f) * inv_per_pixel); };
    // the 1x1's weights and biases: requested here, stored to LDS with the patch
    constexpr int kFwItems = (kFwBias + THREADS - 1) / THREADS;
    float fw_v[kFwItems], fb_v = 0.f;
    const int fw_n = p.final_out ? p.final_cout * (p.c_feat + p.cout) : 0;
    if (p.final_out)
    {
#pragma unroll
        for (int k = 0; k < kFwItems; ++k) fw_v[k] = p.final_w[min((int)threadIdx.x + THREADS * k, fw_n - 1)];
        fb_v = p.final_b[min((int)threadIdx.x, p.final_cout - 1)];
    }
    {
        const size_t plane = (size_t)p.H * p.W;
#pragma unroll
        for (int k = 0; k < kFeatItems; ++k)
        {
            const int item = (int)threadIdx.x + THREADS * k;
            const int py = item / kConvPatchW, px = item - py * kConvPatchW;
            const int y = y0 + py - 1, x = x0 + px - 1;
            const bool in = item < kConvPatchH * kConvPatchW && y >= 0 && y < p.H && x >= 0 && x < p.W;
            const float* src = p.feat + (size_t)min(max(y, 0), p.H - 1) * p.W + min(max(x, 0), p.W - 1);
            feat_in[k] = in;
#pragma unroll
            for (int c = 0; c < CI; ++c) feat_v[k][c] = src[(c < C ? c : 0) * plane];
        }
    }
    if (has_below)
    {
        const size_t pb = (size_t)p.Hb * p.Wb;
#pragma unroll
        for (int k = 0; k < kBelowItems; ++k)
        {
            const int item = (int)threadIdx.x + THREADS * k;
            // (kBelowItems is sized for the widest level below; a round in which no thread has an item is skipped as a
            // whole: the finest level of the usual plan has 432 items for its 512 threads)
            if (THREADS * k >= kBelowH * kBelowW * per_pixel) break;
            const bool have = item < kBelowH * kBelowW * per_pixel;
            const int it    = have ? item : 0;
            const int bp = pixel_of_item(it), q = it - bp * per_pixel;
            const int r = bp / kBelowW, c0 = bp - r * kBelowW;
            const int yy = min(max(by0 + r, 0), p.Hb - 1), xx = min(max(bx0 + c0, 0), p.Wb - 1);
            const bool img = q < IQ;
            // an image item: four planes of the image below; any other item reads plane 0 four times and drops it
            const float* src = p.feat_below + (size_t)yy * p.Wb + xx;
#pragma unroll
            for (int c = 0; c < 4; ++c) below_f[k][c] = src[(size_t)(img && 4 * q + c < C ? 4 * q + c : 0) * pb];
            // an item of block outputs: eight of them; an image item reads the pixel's first eight and drops them
            below_v[k]    = *reinterpret_cast<const uint4*>(p.act_below + ((size_t)yy * p.Wb + xx) * p.cb_store + 8 * (img ? 0 : q - IQ));
            below_have[k] = have;
            below_img[k]  = img;
        }
    }
    // ---- all loads are on their way: from here on their values are used ----
    if (p.final_out)
    {
#pragma unroll
        for (int k = 0; k < kFwItems; ++k) loaded(fw_v[k]);
        loaded(fb_v);
    }
#pragma unroll
    for (int k = 0; k < kFeatItems; ++k)
#pragma unroll
        for (int c = 0; c < CI; ++c)
        {
            loaded(feat_v[k][c]);
            if (!(feat_in[k] && c < C)) feat_v[k][c] = 0.f;
        }
    if (has_below)
    {
#pragma unroll
        for (int k = 0; k < kBelowItems; ++k)
        {
            if (THREADS * k >= kBelowH * kBelowW * per_pixel) break;
            const int item = (int)threadIdx.x + THREADS * k;
            const int it   = below_have[k] ? item : 0;
            const int q    = it - pixel_of_item(it) * per_pixel;
#pragma unroll
            for (int c = 0; c < 4; ++c)
            {
                loaded(below_f[k][c]);
                if (!(below_img[k] && 4 * q + c < C)) below_f[k][c] = 0.f;
            }
            loaded(below_v[k]);
            if (below_img[k])
                below_v[k] = make_uint4(__float_as_uint(below_f[k][0]), __float_as_uint(below_f[k][1]), __float_as_uint(below_f[k][2]),
                                        __float_as_uint(below_f[k][3]));
            if (!below_have[k]) below_v[k] = make_uint4(0u, 0u, 0u, 0u);
        }
    }
    if (p.final_out)
    {
#pragma unroll
        for (int k = 0; k < kFwItems; ++k)
            if ((int)threadIdx.x + THREADS * k < fw_n) s_fw[(int)threadIdx.x + THREADS * k] = float(_Float16(fw_v[k]));
        if ((int)threadIdx.x < p.final_cout) s_fw[kFwBias + (int)threadIdx.x] = fb_v;
    }
#pragma unroll
    for (int k = 0; k < kFeatItems; ++k)
    {
        const int item = (int)threadIdx.x + THREADS * k;
        if (item < kConvPatchH * kConvPatchW)
        {
            _Float16* row = s_patch + (size_t)item * ROW;
            if (CI == 4 && C == 4)  // one 8-byte LDS store instead of four 2-byte ones
                *reinterpret_cast<half4*>(row) =
                    half4{_Float16(feat_v[k][0]), _Float16(feat_v[k][1]), _Float16(feat_v[k][2]), _Float16(feat_v[k][3])};
            else
            {
#pragma unroll
                for (int c = 0; c < CI; ++c)  // (a run-time bound would put the register array into scratch memory)
                    if (c < C) row[c] = _Float16(feat_v[k][c]);
            }
            if (!has_below)
            {
                // start block: the image is the whole input
                for (int c = C; c < CIN; ++c) row[c] = _Float16(0.f);
            }
        }
    }
    if (has_below)
    {
#pragma unroll
        for (int k = 0; k < kBelowItems; ++k)
        {
            const int item = (int)threadIdx.x + THREADS * k;
            if (THREADS * k >= kBelowH * kBelowW * per_pixel) break;
            if (item < kBelowH * kBelowW * per_pixel)
            {
                const int bp = pixel_of_item(item), q = item - bp * per_pixel;
                _Float16* row = s_below + (size_t)bp * ROW;
                if (q < IQ)
                {
                    const float f[4] = {__uint_as_float(below_v[k].x), __uint_as_float(below_v[k].y), __uint_as_float(below_v[k].z),
                                        __uint_as_float(below_v[k].w)};
                    if (CI == 4 && C == 4)
                        *reinterpret_cast<half4*>(row + 4) = half4{_Float16(f[0]), _Float16(f[1]), _Float16(f[2]), _Float16(f[3])};
                    else
                    {
#pragma unroll
                        for (int c = 0; c < 4; ++c)
                            if (4 * q + c < C) row[C + 4 * q + c] = _Float16(f[c]);
                    }
                    if (q == 0)
                        for (int c = 2 * C + p.cb_store; c < CIN; ++c) row[c] = _Float16(0.f);  // padding channels
                }
                else
                {
                    const int pos = 2 * C + 8 * (q - IQ);
                    if (C == 4)
                        *reinterpret_cast<uint4*>(row + pos) = below_v[k];
                    else
                    {
                        const half8 a = __builtin_bit_cast(half8, below_v[k]);
                        for (int i = 0; i < 8; ++i)
                            if (pos + i < CIN) row[pos + i] = a[i];
                    }
                }
            }
        }
        __syncthreads();
        // ---- stage 2: bilinear 2x upsampling from the below patch into channels [C, CIN) of the patch ----
        // A thread takes a pixel of the patch and walks its groups of 8 channels: the pixel's position, sources and
        // weights are worked out once (with an item per (pixel, group) that arithmetic was most of the stage).
        for (int pp = (int)threadIdx.x; pp < kConvPatchH * kConvPatchW; pp += THREADS)
        {
            const int py = pp / kConvPatchW, px = pp - py * kConvPatchW;
            const int y = y0 + py - 1, x = x0 + px - 1;
            const bool inside = y >= 0 && y < p.H && x >= 0 && x < p.W;
            // The interpolation runs in packed fp16: the weights are products of 0, 1/4, 3/4 and 1 (exact in fp16), the
            // operands are fp16 already and the result is stored as fp16; three fused multiply-adds per pair of channels
            // instead of eight conversions and four fp32 operations per channel.
            int ya = by0, yb = by0, xa = bx0, xb = bx0;
            float ly = 0.f, lx = 0.f;
            if (inside)
            {
                up2_source(y, p.Hb, ya, yb, ly);
                up2_source(x, p.Wb, xa, xb, lx);
            }
            const _Float16 w00 = _Float16((1.f - ly) * (1.f - lx)), w01 = _Float16((1.f - ly) * lx);
            const _Float16 w10 = _Float16(ly * (1.f - lx)), w11 = _Float16(ly * lx);
            const half8 W00 = {w00, w00, w00, w00, w00, w00, w00, w00}, W01 = {w01, w01, w01, w01, w01, w01, w01, w01};
            const half8 W10 = {w10, w10, w10, w10, w10, w10, w10, w10}, W11 = {w11, w11, w11, w11, w11, w11, w11, w11};
            const _Float16* sa = s_below + ((ya - by0) * kBelowW + (xa - bx0)) * ROW;
            const _Float16* sb = s_below + ((ya - by0) * kBelowW + (xb - bx0)) * ROW;
            const _Float16* sc = s_below + ((yb - by0) * kBelowW + (xa - bx0)) * ROW;
            const _Float16* sd = s_below + ((yb - by0) * kBelowW + (xb - bx0)) * ROW;
            _Float16* drow     = s_patch + (size_t)pp * ROW;
#pragma unroll
            for (int g = 0; g < GROUPS; ++g)
            {
                half8 h;
#pragma unroll
                for (int i = 0; i < 8; ++i) h[i] = _Float16(0.f);
                if (inside)
                {
                    const half8 a = *reinterpret_cast<const half8*>(sa + 8 * g);
                    const half8 b = *reinterpret_cast<const half8*>(sb + 8 * g);
                    const half8 c = *reinterpret_cast<const half8*>(sc + 8 * g);
                    const half8 d = *reinterpret_cast<const half8*>(sd + 8 * g);
                    h = __builtin_elementwise_fma(d, W11, __builtin_elementwise_fma(c, W10, __builtin_elementwise_fma(b, W01, a * W00)));
                }
                _Float16* dst = drow + 8 * g;
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
    }

    __syncthreads();  // patch complete; the patch of the level below is no longer needed
    // the staged taps of the weights, in place of the patch of the level below
    _Float16* s_taps = s_patch + kConvPatchH * kConvPatchW * ROW;
    conv_tap_stage(taps, s_taps);
    __syncthreads();
    floatx4 acc[MB][NB];
    conv_taps_mfma<CIN, NPAD, true, THREADS>(s_patch, s_taps, p.wpack, taps, acc);  // a lane: four channels of one pixel
    const int lane = (int)threadIdx.x & 63, wave = (int)threadIdx.x >> 6;
    const int lrow = lane & 15, lk = (lane >> 4) * 8;

    // ---- epilogue: elu(feature) * sigmoid(mask) in fp16, staged in LDS (the patch is no longer needed) and
    // written channels innermost with full-line stores; the pre-activations too when the backward needs them ----
    constexpr int IPAD = CI > kLdsChanPad ? CI : kLdsChanPad;  // padding columns of a staged row: room for the image
    constexpr int AS = NPAD / 2 + IPAD, PS = NPAD + kLdsChanPad;
    _Float16* s_act = smem;                                      // [256][AS]
    _Float16* s_pre = smem + kConvTileH * kConvTileW * AS;       // [256][PS]
    float my_feat[CI];  // this thread's pixel of the image, as the convolution saw it (fp16)
#pragma unroll
    for (int c = 0; c < CI; ++c) my_feat[c] = 0.f;
    const bool owns_pixel = THREADS == kConvTileH * kConvTileW || (int)threadIdx.x < kConvTileH * kConvTileW;  // one thread per pixel
    if (p.final_out && owns_pixel)
    {
        const _Float16* row = s_patch + (size_t)(((int)threadIdx.x / kConvTileW + 1) * kConvPatchW + (int)threadIdx.x % kConvTileW + 1) * ROW;
#pragma unroll
        for (int c = 0; c < CI; ++c)
            if (c < C) my_feat[c] = float(row[c]);
    }
    __syncthreads();  // every wavefront is done reading the patch
#pragma unroll
    for (int m = 0; m < MB; ++m)
    {
        const int tp = (MB == 4 ? 2 * wave + (m >> 1) : wave) * kConvTileW + (m & 1) * 16 + lrow;  // this lane's pixel of the block
#pragma unroll
        for (int j = 0; j < HB; ++j)
        {
            const int ch0   = 16 * j + (lane >> 4) * 4;  // this lane's four channels
            const float4 bf = *reinterpret_cast<const float4*>(p.bias + ch0), bm = *reinterpret_cast<const float4*>(p.bias + NPAD / 2 + ch0);
            const float f[4] = {acc[m][j][0] + bf.x, acc[m][j][1] + bf.y, acc[m][j][2] + bf.z, acc[m][j][3] + bf.w};
            // (both 0 for padding channels)
            const float g[4] = {acc[m][HB + j][0] + bm.x, acc[m][HB + j][1] + bm.y, acc[m][HB + j][2] + bm.z, acc[m][HB + j][3] + bm.w};
            if (p.pre)
            {
                *reinterpret_cast<half4*>(s_pre + tp * PS + ch0)            = half4{_Float16(f[0]), _Float16(f[1]), _Float16(f[2]), _Float16(f[3])};
                *reinterpret_cast<half4*>(s_pre + tp * PS + NPAD / 2 + ch0) = half4{_Float16(g[0]), _Float16(g[1]), _Float16(g[2]), _Float16(g[3])};
            }
            half4 out;
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                const float e = f[i] > 0.f ? f[i] : (__expf(f[i]) - 1.f);
                // v_rcp_f32 is good to 1 ulp of fp32 and the product is rounded to fp16 next: no IEEE division needed
                const float sg = __builtin_amdgcn_rcpf(1.f + __expf(-g[i]));
                out[i]         = ch0 + i < p.cout ? _Float16(e * sg) : _Float16(0.f);
            }
            *reinterpret_cast<half4*>(s_act + tp * AS + ch0) = out;
        }
    }
    __syncthreads();
    if (p.out) store_tile_nhwc<THREADS>(s_act, AS, p.cout_store / 8, p.out, p.cout_store, x0, y0, p.W, p.H);
    if (p.pre) store_tile_nhwc<THREADS, true>(s_pre, PS, NPAD / 8, p.pre, NPAD, x0, y0, p.W, p.H);
    if (p.final_out)
    {
        // `final` of the net (Networks.h:1129-1131) on the matrix cores: per 16 pixels one MFMA per 32 input channels,
        // A = the staged tile rows (block outputs, then the image in the row's padding columns), B = the 1x1 weights,
        // rounded to fp16 like every other operand, outputs in the first columns.
        constexpr int KF  = NPAD / 2 + IPAD;  // block outputs (padded) | image | zeros
        constexpr int KFB = (KF + 31) / 32;
        const int cin     = C + p.cout;
        // the image joins the staged rows (columns NPAD/2 .. NPAD/2 + IPAD - 1; nobody has read them yet)
        if (owns_pixel)
        {
            _Float16* row = s_act + (size_t)(int)threadIdx.x * AS + NPAD / 2;
#pragma unroll
            for (int c = 0; c < IPAD; ++c) row[c] = (c < CI && c < C) ? _Float16(my_feat[c < CI ? c : 0]) : _Float16(0.f);
        }
        half8 bfin[KFB];
#pragma unroll
        for (int kb = 0; kb < KFB; ++kb)
#pragma unroll
            for (int i = 0; i < 8; ++i)
            {
                const int k = kb * 32 + lk + i;  // position in a staged row
                float w     = 0.f;
                if (lrow < p.final_cout)
                {
                    if (k < p.cout)
                        w = s_fw[lrow * cin + C + k];
                    else if (k >= NPAD / 2 && k < NPAD / 2 + C)
                        w = s_fw[lrow * cin + (k - NPAD / 2)];
                }
                bfin[kb][i] = _Float16(w);  // exact: the table holds fp16 values
            }
        __syncthreads();  // image columns in place
        const size_t plane = (size_t)p.H * p.W;
        const float fb     = lrow < p.final_cout ? s_fw[kFwBias + lrow] : 0.f;
#pragma unroll
        for (int m = 0; m < MB; ++m)
        {
            const int tp0 = (MB == 4 ? 2 * wave + (m >> 1) : wave) * kConvTileW + (m & 1) * 16;  // first pixel of this 16-pixel block
            floatx4 o     = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kb = 0; kb < KFB; ++kb)
            {
                half8 a;
#pragma unroll
                for (int i = 0; i < 8; ++i) a[i] = _Float16(0.f);
                if (kb * 32 + lk < KF) a = *reinterpret_cast<const half8*>(s_act + (size_t)(tp0 + lrow) * AS + kb * 32 + lk);
                o = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bfin[kb], o, 0, 0, 0);
            }
            // lane: output channel lrow, pixels tp0 + (lane / 16) * 4 .. + 3
            if (lrow < p.final_cout)
            {
                const int tp = tp0 + (lane >> 4) * 4;
                const int y = y0 + tp / kConvTileW, x = x0 + tp % kConvTileW;
                float* dst = p.final_out + lrow * plane + (size_t)y * p.W + x;
                if (y < p.H)
                {
                    if (x + 3 < p.W && (reinterpret_cast<uintptr_t>(dst) & 15) == 0)
                        *reinterpret_cast<float4*>(dst) = make_float4(o[0] + fb, o[1] + fb, o[2] + fb, o[3] + fb);
                    else
                    {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            if (x + i < p.W) dst[i] = o[i] + fb;
                    }
                }
            }
        }
    }
}

// wpack[tap][n][c]: n < NPAD/2 feature output n, else mask output n - NPAD/2; zero outside the real ranges.
// All levels in one launch, the level is blockIdx.y (a launch per level costs more than the work itself).
struct PackLevel
{
    const float *wf, *bf, *wm, *bm;
    int cout, cin_real, cin_pad, npad;
    _Float16* wpack;
    float* bias;
};
struct PackTable
{
    PackLevel lv[TRIPS_UNET_MAX_LEVELS];
};
__global__ __launch_bounds__(256) void pack_conv_weights_kernel(const PackTable t)
{
    const PackLevel& l = t.lv[blockIdx.y];
    const float* __restrict__ wf = l.wf;
    const float* __restrict__ bf = l.bf;
    const float* __restrict__ wm = l.wm;
    const float* __restrict__ bm = l.bm;
    const int cout = l.cout, cin_real = l.cin_real, cin_pad = l.cin_pad, npad = l.npad;
    _Float16* __restrict__ wpack = l.wpack;
    float* __restrict__ bias     = l.bias;
    const int total = 9 * npad * cin_pad;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256)
    {
        const int c = i % cin_pad, n = (i / cin_pad) % npad, tap = i / (cin_pad * npad);
        const int half = npad / 2;
        const int o    = n < half ? n : n - half;
        float v        = 0.f;
        if (o < cout && c < cin_real) v = (n < half ? wf : wm)[((size_t)o * cin_real + c) * 9 + tap];
        wpack[i] = _Float16(v);
    }
    for (int n = blockIdx.x * 256 + threadIdx.x; n < npad; n += gridDim.x * 256)
    {
        const int half = npad / 2;
        const int o    = n < half ? n : n - half;
        bias[n]        = o < cout ? (n < half ? bf : bm)[o] : 0.f;
    }
}

// ---------------------------------------------------------------------------------------------------------
namespace
{
template <int CIN, int NPAD, int CI>
hipError_t launch_conv(const ConvParams& p, hipStream_t stream)
{
    constexpr int ROW  = CIN + kLdsChanPad;
    constexpr int IPAD = CI > kLdsChanPad ? CI : kLdsChanPad;
    // the patch, then the patch of the level below or (later) the staged taps of the weights, whichever is larger
    const size_t lds_in  = (size_t)(kConvPatchH * kConvPatchW * ROW + std::max(kBelowH * kBelowW * ROW, ConvTapStage<CIN, NPAD, 512>::LDS_HALVES)) * sizeof(_Float16);
    const size_t lds_out = (size_t)kConvTileH * kConvTileW * ((NPAD / 2 + IPAD) + (p.pre ? NPAD + kLdsChanPad : 0)) * sizeof(_Float16);
    const size_t lds     = std::max(lds_in, lds_out);  // up to 104 KB when the largest block saves its pre-activations
    // eight wavefronts per tile (one row each): the phases around the tap loop run at the latency of their loads and LDS
    // round trips, and twice the wavefronts per tile hide twice as much of it
    constexpr int THREADS = 512;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gated_conv3x3_kernel<CIN, NPAD, THREADS, CI>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    dim3 grid((p.W + kConvTileW - 1) / kConvTileW, (p.H + kConvTileH - 1) / kConvTileH);
    hipLaunchKernelGGL((gated_conv3x3_kernel<CIN, NPAD, THREADS, CI>), grid, dim3(THREADS), lds, stream, p);
    return hipGetLastError();
}

template <int CI>
hipError_t dispatch_conv_ci(const ConvParams& p, int cin_pad, int npad, hipStream_t stream)
{
    if (cin_pad == 32)
    {
        if (npad == 32) return launch_conv<32, 32, CI>(p, stream);
        if (npad == 64) return launch_conv<32, 64, CI>(p, stream);
        if (npad == 96) return launch_conv<32, 96, CI>(p, stream);
        if (npad == 128) return launch_conv<32, 128, CI>(p, stream);
    }
    else
    {
        if (npad == 32) return launch_conv<64, 32, CI>(p, stream);
        if (npad == 64) return launch_conv<64, 64, CI>(p, stream);
        if (npad == 96) return launch_conv<64, 96, CI>(p, stream);
        if (npad == 128) return launch_conv<64, 128, CI>(p, stream);
    }
    return hipErrorInvalidValue;
}

// (the kernel is built for 4, 8 and 16 image channels; fewer use the next size up)
hipError_t dispatch_conv(const ConvParams& p, int cin_pad, int npad, hipStream_t stream)
{
    if (p.c_feat <= 4) return dispatch_conv_ci<4>(p, cin_pad, npad, stream);
    if (p.c_feat <= 8) return dispatch_conv_ci<8>(p, cin_pad, npad, stream);
    return dispatch_conv_ci<16>(p, cin_pad, npad, stream);
}
}  // namespace
}  // namespace trips

using namespace trips;

extern "C" {

int trips_unet_workspace_size(const TripsUnetDesc* desc, size_t* bytes)
{
    if (int e = check_unet_desc(desc)) return e;
    if (!bytes) return set_error(TRIPS_ERR_INVALID_ARG, "bytes is NULL");
    *bytes = make_plan(*desc).bytes;
    return TRIPS_OK;
}

int trips_unet_saved_size(const TripsUnetDesc* desc, size_t* bytes)
{
    if (int e = check_unet_desc(desc)) return e;
    if (!bytes) return set_error(TRIPS_ERR_INVALID_ARG, "bytes is NULL");
    *bytes = make_plan(*desc).saved_bytes;
    return TRIPS_OK;
}

int trips_unet_flops(const TripsUnetDesc* desc, double* flops)
{
    if (int e = check_unet_desc(desc)) return e;
    if (!flops) return set_error(TRIPS_ERR_INVALID_ARG, "flops is NULL");
    const NetPlan np = make_plan(*desc);
    double f         = 0.0;
    for (int i = 0; i < desc->num_levels; ++i)
        f += 2.0 * 2.0 * 9.0 * np.lv[i].cin_real * np.lv[i].cout * (double)np.lv[i].H * np.lv[i].W;
    f += 2.0 * desc->filters[0] * desc->num_output_channels * (double)desc->level_h[0] * desc->level_w[0];
    *flops = f * desc->batch;
    return TRIPS_OK;
}

int trips_unet_forward(TripsCtx* ctx, const TripsUnetDesc* desc, const TripsUnetWeights* weights,
                       const float* const inputs[TRIPS_UNET_MAX_LEVELS], float* output, void* saved, void* workspace,
                       size_t workspace_bytes, void* stream_)
{
    if (!ctx) return set_error(TRIPS_ERR_INVALID_ARG, "ctx is NULL");
    if (int e = check_unet_desc(desc)) return e;
    if (!weights || !inputs || !output || !workspace) return set_error(TRIPS_ERR_INVALID_ARG, "NULL argument");
    const TripsUnetDesc& d = *desc;
    const int C = d.num_input_channels, L = d.num_levels;
    for (int i = 0; i < L; ++i)
    {
        if (!inputs[i]) return set_error(TRIPS_ERR_INVALID_ARG, "inputs[%d] is NULL", i);
        if (!weights->feature_weight[i] || !weights->feature_bias[i] || !weights->mask_weight[i] || !weights->mask_bias[i])
            return set_error(TRIPS_ERR_INVALID_ARG, "weights of block %d are NULL", i);
    }
    if (!weights->final_weight || !weights->final_bias) return set_error(TRIPS_ERR_INVALID_ARG, "final weights are NULL");
    if ((reinterpret_cast<uintptr_t>(workspace) & 255) || (reinterpret_cast<uintptr_t>(saved) & 255))
        return set_error(TRIPS_ERR_INVALID_ARG, "workspace / saved must be 256-byte aligned");
    const NetPlan np = make_plan(d);
    if (workspace_bytes < np.bytes)
        return set_error(TRIPS_ERR_WORKSPACE_SMALL, "workspace has %zu bytes, %zu needed", workspace_bytes, np.bytes);
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    char* ws           = reinterpret_cast<char*>(workspace);
    char* sv           = reinterpret_cast<char*>(saved);
    Profiler* prof     = ctx->prof.enabled ? &ctx->prof : nullptr;
    // block outputs live in the saved state when there is one (the backward reads them), else in the workspace
    auto act_ptr = [&](int level, int b)
    {
        const LevelPlan& l = np.lv[level];
        char* base         = sv ? sv + l.saved_act_off : ws + l.act_off;
        return reinterpret_cast<_Float16*>(base) + (size_t)b * l.H * l.W * l.cout_store;
    };

    if (!d.weights_packed)
    {
        ProfScope ps(prof, "unet_pack_weights", stream);
        PackTable pt;
        int most = 0;
        for (int i = 0; i < L; ++i)
        {
            const LevelPlan& lv = np.lv[i];
            pt.lv[i] = PackLevel{weights->feature_weight[i], weights->feature_bias[i], weights->mask_weight[i], weights->mask_bias[i],
                                 lv.cout, lv.cin_real, lv.cin_pad, lv.npad, reinterpret_cast<_Float16*>(ws + lv.wpack_off),
                                 reinterpret_cast<float*>(ws + lv.bias_off)};
            most     = std::max(most, 9 * lv.npad * lv.cin_pad);
        }
        hipLaunchKernelGGL(pack_conv_weights_kernel, dim3((most + 255) / 256, L), dim3(256), 0, stream, pt);
    }
    static const char* const kLevelNames[TRIPS_UNET_MAX_LEVELS] = {"unet_conv_l0", "unet_conv_l1", "unet_conv_l2", "unet_conv_l3",
                                                                   "unet_conv_l4", "unet_conv_l5", "unet_conv_l6", "unet_conv_l7"};
    for (int i = L - 1; i >= 0; --i)
    {
        const LevelPlan& lv = np.lv[i];
        ProfScope ps(prof, kLevelNames[i], stream);
        for (int b = 0; b < d.batch; ++b)
        {
            ConvParams p;
            std::memset(&p, 0, sizeof(p));
            p.H          = lv.H;
            p.W          = lv.W;
            p.c_feat     = C;
            p.cout       = lv.cout;
            p.cout_store = lv.cout_store;
            p.feat       = inputs[i] + (size_t)b * C * lv.H * lv.W;
            p.wpack      = reinterpret_cast<const _Float16*>(ws + lv.wpack_off);
            p.bias       = reinterpret_cast<const float*>(ws + lv.bias_off);
            // (nobody reads the finest block's output again: its 1x1 runs in the same kernel, and the backward takes
            // it from the pre-activations)
            p.out        = i == 0 ? nullptr : act_ptr(i, b);
            p.pre        = sv ? reinterpret_cast<_Float16*>(sv + lv.saved_pre_off) + (size_t)b * lv.H * lv.W * lv.npad : nullptr;
            if (i < L - 1)
            {
                const LevelPlan& lb = np.lv[i + 1];
                p.Hb         = lb.H;
                p.Wb         = lb.W;
                p.cb_store   = lb.cout_store;
                p.feat_below = inputs[i + 1] + (size_t)b * C * lb.H * lb.W;
                p.act_below  = act_ptr(i + 1, b);
            }
            if (i == 0)
            {
                p.final_w    = weights->final_weight;
                p.final_b    = weights->final_bias;
                p.final_out  = output + (size_t)b * d.num_output_channels * lv.H * lv.W;
                p.final_cout = d.num_output_channels;
            }
            hipError_t e = dispatch_conv(p, lv.cin_pad, lv.npad, stream);
            if (e != hipSuccess) return set_error(TRIPS_ERR_HIP, "gated conv launch (level %d): %s", i, hipGetErrorString(e));
        }
    }
    return TRIPS_OK;
}

}  // extern "C"
