// Pieces shared by the forward and backward kernels of the reconstruction net (gfx950).
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "../../include/trips_unet.h"
#include "splat_internal.h"

namespace trips
{
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kConvTileH   = 8;
constexpr int kConvTileW   = 32;
constexpr int kConvPatchH  = kConvTileH + 2;
constexpr int kConvPatchW  = kConvTileW + 2;
constexpr int kBelowH      = kConvTileH / 2 + 2;  // rows / columns of the level below that an upsampled patch touches
constexpr int kBelowW      = kConvTileW / 2 + 2;
constexpr int kFinalPixelsPerBlock = 512;   // pixels a workgroup of the 1x1 convolution's backward takes at a time
constexpr int kUnetMaxImageChannels = 16;  // channels of the splat images (the descriptor widths of the splat: 3, 4, 6, 8, 16)
constexpr int kFinalPartFloats     = 4 * (kUnetMaxImageChannels + 64) + 4;  // its partial sums: [4 outputs][<= 16 image + <= 64 block channels], 4 biases
constexpr int kLdsChanPad  = 8;  // halves added to every LDS row so that 16 lanes reading 16 bytes hit 64 distinct banks

// source row / column and weight of torch's bilinear upsampling with scale_factor 2, align_corners = false
// (area_pixel_compute_source_index: src = max(0, (dst + 0.5) * 0.5 - 0.5))
__device__ __forceinline__ void up2_source(int dst, int in_size, int& i0, int& i1, float& lambda)
{
    float src = (float(dst) + 0.5f) * 0.5f - 0.5f;
    src       = src < 0.f ? 0.f : src;
    i0        = (int)src;
    i0        = i0 < in_size - 1 ? i0 : in_size - 1;
    i1        = i0 + 1 < in_size ? i0 + 1 : in_size - 1;
    lambda    = src - float(i0);
}


// The 9-tap implicit-GEMM core shared by the forward convolution and the data gradient. A operands are 16-byte LDS
// reads from a (8+2) x (32+2) pixel patch with KIN channels innermost (row stride KIN + 8 halves). B operands (packed
// weights [tap][NOUT][KIN]) reach the matrix cores through LDS as well: with every wavefront loading its own
// fragments from memory, each of a tile's four wavefronts pulled the level's whole weight set (18 - 147 KB) out of
// the L2 again, 0.6 GB per launch at the two finest levels, and that traffic, not the MFMAs, set the length of the
// tap loop. Now the workgroup copies the weights into LDS and every wavefront reads its fragments from there: a
// quarter of the L2 traffic, the same bank-conflict-free row layout as the patch. A tap's MFMAs take far less time
// than a round trip to the L2, so as many taps as the LDS has room for are staged together: all nine (requested when
// the kernel starts; the tap loop then has neither loads nor barriers), or three (the next three travel in
// registers while these are multiplied; two barriers per three taps), or one (two buffers, one barrier per tap).
// A wavefront owns two rows of the 8 x 32 output tile = four 16-pixel row blocks; acc[m][n] is the 16 x 16 block of
// pixels m, outputs 16n .. 16n+15.
// THREADS = threads of the workgroup: 256 (a wavefront owns two rows of the tile = four 16-pixel row blocks) or 512 (one
// row = two row blocks).
constexpr int kTapLdsBytes = 28 * 1024;  // LDS that the staged taps of a workgroup may take
template <int KIN, int NOUT, int THREADS = 256>
struct ConvTapStage
{
    static constexpr int NB    = NOUT / 16;
    static constexpr int KB    = KIN / 32;
    static constexpr int ROW   = KIN + kLdsChanPad;   // halves per output row of a tap in LDS
    static constexpr int ITEMS = NOUT * KIN / 8;      // 16-byte words per tap
    static constexpr int MB    = 16 / (THREADS / 64);  // 16-pixel row blocks of a wavefront
    static constexpr int BUF   = NOUT * ROW;           // halves per tap in LDS
    // taps staged together
    static constexpr int T = 9 * BUF * 2 <= kTapLdsBytes ? 9 : 3 * BUF * 2 <= kTapLdsBytes ? 3 : 1;
    static constexpr int STAGE_ITEMS = T * ITEMS;      // 16-byte words per stage
    static constexpr int PER   = (STAGE_ITEMS + THREADS - 1) / THREADS;  // per thread
    static constexpr int LDS_HALVES = (T == 1 ? 2 : T) * BUF;  // what the kernel provides at s_taps
    half8 r[PER];
};

// this thread's share of taps `tap` .. `tap` + T - 1 from memory into registers (the packed weights are dense:
// [tap][NOUT][KIN])
template <int KIN, int NOUT, int THREADS>
__device__ __forceinline__ void conv_tap_fetch(ConvTapStage<KIN, NOUT, THREADS>& st, const _Float16* __restrict__ wpack, int tap)
{
    using S = ConvTapStage<KIN, NOUT, THREADS>;
    const half8* src = reinterpret_cast<const half8*>(wpack + (size_t)tap * NOUT * KIN);
#pragma unroll
    for (int j = 0; j < S::PER; ++j)
    {
        const int item = threadIdx.x + THREADS * j;
        if (S::STAGE_ITEMS % THREADS == 0 || item < S::STAGE_ITEMS) st.r[j] = src[item];
    }
}

// ... and from the registers into the tap buffers at s_tap (T of them, one after the other)
template <int KIN, int NOUT, int THREADS>
__device__ __forceinline__ void conv_tap_stage(const ConvTapStage<KIN, NOUT, THREADS>& st, _Float16* s_tap)
{
    using S = ConvTapStage<KIN, NOUT, THREADS>;
#pragma unroll
    for (int j = 0; j < S::PER; ++j)
    {
        const int item = threadIdx.x + THREADS * j;
        if (S::STAGE_ITEMS % THREADS == 0 || item < S::STAGE_ITEMS)
        {
            const int t = item / S::ITEMS, w = item - t * S::ITEMS;
            *reinterpret_cast<half8*>(s_tap + t * S::BUF + (w / (KIN / 8)) * S::ROW + (w % (KIN / 8)) * 8) = st.r[j];
        }
    }
}

// Precondition: the first T taps sit at s_taps (conv_tap_fetch(.., 0) + conv_tap_stage) and a barrier has passed since.
// Every thread of the workgroup must call this (it contains barriers unless all nine taps are staged).
// Result layout: lane l holds, of the 16 x 16 block acc[m][n], pixels (l / 16) * 4 .. + 3 of output 16n + l % 16; with
// OUTPUTS_IN_ROWS (the operands of the MFMA exchanged) outputs 16n + (l / 16) * 4 .. + 3 of pixel l % 16, four
// neighbouring channels of one pixel, which an epilogue can store as one 8-byte word.
template <int KIN, int NOUT, bool OUTPUTS_IN_ROWS = false, int THREADS = 256>
__device__ __forceinline__ void conv_taps_mfma(const _Float16* s_patch, _Float16* s_taps, const _Float16* __restrict__ wpack,
                                               ConvTapStage<KIN, NOUT, THREADS>& st,
                                               floatx4 (&acc)[ConvTapStage<KIN, NOUT, THREADS>::MB][NOUT / 16])
{
    using S = ConvTapStage<KIN, NOUT, THREADS>;
    constexpr int MB = S::MB;
    constexpr int ROW = KIN + kLdsChanPad;
    constexpr int NB  = S::NB;
    constexpr int KB  = S::KB;
    constexpr int T   = S::T;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lrow = lane & 15, lk = (lane >> 4) * 8;
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int n = 0; n < NB; ++n) acc[m][n] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int tap = 0; tap < 9; ++tap)
    {
        const int dy = tap / 3, dx = tap - dy * 3;  // patch coordinates already include the halo
        // the next stage's weights: requested before this stage's first tap is multiplied
        if (T < 9 && tap % T == 0 && tap + T < 9) conv_tap_fetch(st, wpack, tap + T);
        const _Float16* sb = s_taps + (T == 1 ? tap & 1 : tap % T) * S::BUF;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
        {
            half8 bfrag[NB];
#pragma unroll
            for (int n = 0; n < NB; ++n) bfrag[n] = *reinterpret_cast<const half8*>(sb + (n * 16 + lrow) * S::ROW + kb * 32 + lk);
#pragma unroll
            for (int m = 0; m < MB; ++m)
            {
                const int r = MB == 4 ? 2 * wave + (m >> 1) : wave, cb = (m & 1) * 16;
                const half8 a = *reinterpret_cast<const half8*>(s_patch + ((r + dy) * kConvPatchW + cb + lrow + dx) * ROW + kb * 32 + lk);
#pragma unroll
                for (int n = 0; n < NB; ++n)
                    acc[m][n] = OUTPUTS_IN_ROWS ? __builtin_amdgcn_mfma_f32_16x16x32_f16(bfrag[n], a, acc[m][n], 0, 0, 0)
                                                : __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bfrag[n], acc[m][n], 0, 0, 0);
            }
        }
        if (T == 1)
        {
            if (tap + 1 < 9) conv_tap_stage(st, s_taps + ((tap + 1) & 1) * S::BUF);
            __syncthreads();  // the next tap is in place; nobody reads this tap's buffer any more
        }
        else if (T < 9 && tap % T == T - 1 && tap + 1 < 9)
        {
            __syncthreads();  // nobody reads this stage's taps any more
            conv_tap_stage(st, s_taps);
            __syncthreads();  // the next stage is in place
        }
    }
    if (T != 1) __syncthreads();  // (as after the last tap of the one-tap form: patch and taps may be overwritten now)
}

// Copies `groups` x 8 halves per pixel of an 8 x 32 tile staged in LDS ([256][lds_stride]) to a channels-innermost
// image ([H][W][dst_stride]) with 16-byte stores: consecutive lanes write consecutive 16 bytes, so a tile row leaves
// as whole lines (2-byte stores straight from the MFMA result layout cost twice the memory requests). STREAM: with
// the non-temporal hint, for data that nothing reads again soon.
template <int THREADS = 256, bool STREAM = false>
__device__ __forceinline__ void store_tile_nhwc(const _Float16* s_tile, int lds_stride, int groups, _Float16* dst,
                                                int dst_stride, int x0, int y0, int W, int H)
{
    for (int item = threadIdx.x; item < kConvTileH * kConvTileW * groups; item += THREADS)
    {
        const int g = item % groups, tp = item / groups;
        const int y = y0 + tp / kConvTileW, x = x0 + tp % kConvTileW;
        if (y < H && x < W)
        {
            const half8 v = *reinterpret_cast<const half8*>(s_tile + (size_t)tp * lds_stride + 8 * g);
            half8* to     = reinterpret_cast<half8*>(dst + ((size_t)y * W + x) * dst_stride + 8 * g);
            if (STREAM)
                __builtin_nontemporal_store(v, to);
            else
                *to = v;
        }
    }
}

// Work split of the weight-gradient kernel for a (padded input channels, padded pre-activations) shape: threads per
// workgroup; how many ways the wavefronts split the 16-channel input blocks, the 16-channel pre-activation blocks and,
// where there are more wavefronts than blocks, the rows of a tile.
constexpr int wgrad_threads(int cin, int npad) { return (cin == 32 && npad == 96) ? 256 : 512; }
constexpr int wgrad_cbw(int cin) { return cin / 16 < 4 ? cin / 16 : 4; }
constexpr int wgrad_nbw(int cin, int npad)
{
    return (wgrad_threads(cin, npad) / 64) / wgrad_cbw(cin) < npad / 16 ? (wgrad_threads(cin, npad) / 64) / wgrad_cbw(cin) : npad / 16;
}
constexpr int wgrad_row_split(int cin, int npad) { return (wgrad_threads(cin, npad) / 64) / (wgrad_cbw(cin) * wgrad_nbw(cin, npad)); }

// ---- host-side plan of a network: per level the padded GEMM sizes and where its buffers live ----
inline int round_up(int v, int m) { return (v + m - 1) / m * m; }

struct LevelPlan
{
    int H, W, cin_real, cin_pad, cout, npad, cout_store;
    size_t wpack_off, bias_off, act_off;  // bytes into the forward workspace
    size_t saved_act_off, saved_pre_off;  // bytes into the saved state (training)
    // bytes into the backward workspace
    size_t wt_off;      // packed transposed weights [9][cin_pad][npad] fp16
    size_t dpre_off;    // gradient of the pre-activations [B][H][W][npad] fp16
    size_t din_off;     // gradient of the block input [B][H][W][cin_pad] fp16
    size_t part_off;    // partial weight gradients [groups][9][npad][cin_pad] fp32
    size_t sliced_off;  // partial sums of the partials [16][9][npad][cin_pad] fp32
    size_t bias_part_off;  // per-workgroup sums of the pre-activation gradients [batch * groups][npad] fp32
    int groups;         // persistent workgroups of the weight-gradient kernel (per image)
};

struct NetPlan
{
    LevelPlan lv[TRIPS_UNET_MAX_LEVELS];
    size_t bytes;           // forward workspace
    size_t saved_bytes;     // saved state
    size_t backward_bytes;  // backward workspace
    size_t final_part_off;  // backward workspace: per-workgroup sums of the 1x1 convolution's weight and bias gradients
    int final_groups;       // persistent workgroups of the finest level's first backward kernel (per image)
};

inline int check_unet_desc(const TripsUnetDesc* d)
{
    if (!d) return set_error(TRIPS_ERR_INVALID_ARG, "desc is NULL");
    if (d->abi_version != TRIPS_ABI_VERSION)
        return set_error(TRIPS_ERR_INVALID_ARG, "abi_version %d, library has %d", d->abi_version, TRIPS_ABI_VERSION);
    if (d->num_levels < 1 || d->num_levels > TRIPS_UNET_MAX_LEVELS)
        return set_error(TRIPS_ERR_INVALID_ARG, "num_levels %d not in 1..%d", d->num_levels, TRIPS_UNET_MAX_LEVELS);
    if (d->num_input_channels < 1 || d->num_input_channels > kUnetMaxImageChannels)
        return set_error(TRIPS_ERR_UNSUPPORTED, "num_input_channels %d not in 1..%d", d->num_input_channels, kUnetMaxImageChannels);
    if (d->num_output_channels < 1 || d->num_output_channels > 4)
        return set_error(TRIPS_ERR_UNSUPPORTED, "num_output_channels %d not in 1..4", d->num_output_channels);
    if (d->batch < 1) return set_error(TRIPS_ERR_INVALID_ARG, "batch < 1");
    const int C = d->num_input_channels, L = d->num_levels;
    for (int i = 0; i < L; ++i)
    {
        if (d->level_w[i] < 1 || d->level_h[i] < 1 || d->level_w[i] > 32768 || d->level_h[i] > 32768)
            return set_error(TRIPS_ERR_INVALID_ARG, "level %d size %dx%d", i, d->level_w[i], d->level_h[i]);
        if (i > 0)
        {
            const int w = d->level_w[i - 1], h = d->level_h[i - 1];
            const bool okw = d->level_w[i] == w / 2 || d->level_w[i] == (w + 1) / 2;
            const bool okh = d->level_h[i] == h / 2 || d->level_h[i] == (h + 1) / 2;
            if (!okw || !okh || 2 * d->level_w[i] < w || 2 * d->level_h[i] < h)
                return set_error(TRIPS_ERR_UNSUPPORTED, "level %d (%dx%d) must be half of level %d (%dx%d), rounded up", i,
                                 d->level_w[i], d->level_h[i], i - 1, w, h);
        }
        const int cout = d->filters[i] - ((i == 0 && L > 1) ? C : 2 * C);
        if (cout < 1 || cout > 64)
            return set_error(TRIPS_ERR_UNSUPPORTED, "filters[%d] = %d gives %d convolution outputs (1..64 supported)", i,
                             d->filters[i], cout);
        if (i + 1 < L && d->filters[i + 1] > 64)
            return set_error(TRIPS_ERR_UNSUPPORTED, "filters[%d] = %d input channels (at most 64 supported)", i + 1,
                             d->filters[i + 1]);
    }
    return TRIPS_OK;
}

// Block i convolves cat(in[i], up2(x_{i+1})) (F[i+1] channels; C for the start block) to F[i] - 2C outputs
// (F[0] - C for the last block when it is not also the start block), Networks.h:1034-1037,1104-1118.
inline NetPlan make_plan(const TripsUnetDesc& d)
{
    NetPlan np;
    const int C = d.num_input_channels, L = d.num_levels;
    size_t o = 0;
    for (int i = 0; i < L; ++i)
    {
        LevelPlan& lv = np.lv[i];
        lv.H          = d.level_h[i];
        lv.W          = d.level_w[i];
        lv.cin_real   = (i == L - 1) ? C : d.filters[i + 1];
        lv.cin_pad    = lv.cin_real <= 32 ? 32 : 64;
        lv.cout       = d.filters[i] - ((i == 0 && L > 1) ? C : 2 * C);
        lv.npad       = 2 * round_up(lv.cout, 16);
        lv.cout_store = round_up(lv.cout, 8);
        lv.wpack_off  = o;
        o += align256((size_t)9 * lv.npad * lv.cin_pad * sizeof(_Float16));
        lv.bias_off = o;
        o += align256((size_t)lv.npad * sizeof(float));
    }
    for (int i = 0; i < L; ++i)
    {
        // (the finest block's output never leaves its kernel: the 1x1 convolution that reads it runs there, and the
        // backward recomputes it from the saved pre-activations)
        np.lv[i].act_off = o;
        if (i > 0) o += align256((size_t)d.batch * np.lv[i].H * np.lv[i].W * np.lv[i].cout_store * sizeof(_Float16));
    }
    np.bytes = o;
    size_t sv = 0, bw = 0;
    for (int i = 0; i < L; ++i)
    {
        LevelPlan& lv       = np.lv[i];
        const size_t pixels = (size_t)d.batch * lv.H * lv.W;
        lv.saved_act_off    = sv;
        if (i > 0) sv += align256(pixels * lv.cout_store * sizeof(_Float16));
        lv.saved_pre_off = sv;
        sv += align256(pixels * lv.npad * sizeof(_Float16));
        lv.wt_off = bw;
        bw += align256((size_t)9 * lv.cin_pad * lv.npad * sizeof(_Float16));
        lv.dpre_off = bw;
        bw += align256(pixels * lv.npad * sizeof(_Float16));
        lv.din_off = bw;
        bw += align256(pixels * lv.cin_pad * sizeof(_Float16));
        const int tiles = ((lv.W + kConvTileW - 1) / kConvTileW) * ((lv.H + kConvTileH - 1) / kConvTileH);
        // persistent workgroups of the weight-gradient kernel: as many as are resident at once (two per CU for the
        // smallest shape, else one); every further one would only add a set of partial sums to write and reduce
        const int resident = (lv.cin_pad * lv.npad <= 1024 ? 2 : 1) * 256;
        lv.groups          = tiles < resident ? tiles : resident;
        lv.part_off     = bw;
        bw += align256((size_t)d.batch * lv.groups * 9 * lv.npad * lv.cin_pad * sizeof(float));
        lv.sliced_off = bw;
        bw += align256((size_t)16 * 9 * lv.npad * lv.cin_pad * sizeof(float));
        lv.bias_part_off = bw;
        bw += align256((size_t)d.batch * lv.groups * lv.npad * sizeof(float));
    }
    {
        const size_t chunks = ((size_t)np.lv[0].H * np.lv[0].W + kFinalPixelsPerBlock - 1) / kFinalPixelsPerBlock;
        // as many workgroups as are resident at once (three per CU at the kernel's 160 registers) walk the chunks: a
        // second, partly filled round of one-chunk workgroups cost a third of the kernel's time
        np.final_groups     = chunks < 768 ? (int)chunks : 768;
        np.final_part_off   = bw;
        bw += align256((size_t)d.batch * np.final_groups * kFinalPartFloats * sizeof(float));
    }
    np.saved_bytes    = sv;
    np.backward_bytes = bw;
    return np;
}


}  // namespace trips
