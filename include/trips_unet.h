/* C ABI of the reconstruction net that consumes the splat's image pyramid: TRIPS' decoder-only multi-scale
 * gated-convolution U-Net on the MI355X matrix cores (fp16 operands, fp32 accumulation). Same library and context
 * as trips_splat.h.
 *
 * Replaces, for inference, MultiScaleUnet2dDecOnlySmallFixedImpl::forward
 * (src/lib/models/Networks.h:1080-1208 of the reference) with its blocks
 *   SmallDecStartBlockImpl                 (Networks.h:751-787)
 *   UpsampleDecOnlySmallBlockFixedImpl     (Networks.h:999-1098)
 * for upsample_mode = bilinear, conv_block_up = gated, norm_layer_up = id, activation = elu, last_act = id
 * (configs/train_normalnet.ini:200-219).
 *
 * Network (L = num_levels, C = num_input_channels, F = filters):
 *   x_{L-1}  = cat(in[L-1], gated3x3(in[L-1]; C -> F[L-1] - 2C))
 *   x_i      = cat(in[i], gated3x3(cat(in[i], up2(x_{i+1})); F[i+1] -> F[i] - 2C))   for i = L-2 .. 1
 *   x_0      = cat(in[0], gated3x3(cat(in[0], up2(x_1)); F[1] -> F[0] - C))
 *   out      = conv1x1(x_0; F[0] -> num_output_channels)
 * gated3x3(x) = elu(conv_f(x)) * sigmoid(conv_m(x)), 3x3, stride 1, zero padding 1; up2 = bilinear, scale 2,
 * align_corners = false, centre-cropped to the size of in[i] when 2*size(x_{i+1}) is larger.
 * The gated block itself lives in a dependency the reference does not vendor (Saiga, PartialConvUnet2d.h); its
 * form here is the published one of gated convolutions.
 */
#ifndef TRIPS_UNET_H
#define TRIPS_UNET_H

#include <stddef.h>
#include <stdint.h>

#include "trips_splat.h"

#ifdef __cplusplus
extern "C" {
#endif

#define TRIPS_UNET_MAX_LEVELS 8

typedef struct TripsUnetDesc {
    int32_t abi_version;          /* TRIPS_ABI_VERSION */
    int32_t num_levels;           /* L, 1..8: in[0..L-1] are consumed (MultiScaleUnet2dParams::num_layers) */
    int32_t num_input_channels;   /* C, 1..16 (4 in every shipped config; the kernels are built with room for 4, 8, 16) */
    int32_t num_output_channels;  /* 1..4 (3) */
    int32_t batch;                /* images per call */
    int32_t filters[TRIPS_UNET_MAX_LEVELS];  /* F[0..L-1] (filters_network); conv outputs must be >= 1 and <= 64 */
    int32_t level_w[TRIPS_UNET_MAX_LEVELS];  /* size of in[i]; level i+1 must be ceil or floor of half of level i */
    int32_t level_h[TRIPS_UNET_MAX_LEVELS];
    int32_t weights_packed;       /* trips_unet_forward only. Nonzero: `workspace` still holds the fp16 weights that an
                                     earlier forward with the same desc and the same weight values packed there, and
                                     nothing has written to it since except such forwards (a viewer's frames: the weights
                                     change when a checkpoint is loaded, not per frame); the call skips the packing.
                                     0: the weights are packed by this call (training: they change every step). */
} TripsUnetDesc;

/* Weights in the reference's tensor layouts (torch::nn::Conv2d): weight [Cout, Cin, 3, 3] and bias [Cout], fp32,
 * device pointers. Block i < L-1 is up[i], block L-1 is the start block. */
typedef struct TripsUnetWeights {
    const float* feature_weight[TRIPS_UNET_MAX_LEVELS];
    const float* feature_bias[TRIPS_UNET_MAX_LEVELS];
    const float* mask_weight[TRIPS_UNET_MAX_LEVELS];
    const float* mask_bias[TRIPS_UNET_MAX_LEVELS];
    const float* final_weight; /* [num_output_channels, F[0], 1, 1] */
    const float* final_bias;   /* [num_output_channels] */
} TripsUnetWeights;

/* Gradients of one backward call, fp32, the reference's layouts, device pointers. Everything is written, not
 * accumulated; NULL members are skipped. */
typedef struct TripsUnetGrads {
    float* feature_weight[TRIPS_UNET_MAX_LEVELS];
    float* feature_bias[TRIPS_UNET_MAX_LEVELS];
    float* mask_weight[TRIPS_UNET_MAX_LEVELS];
    float* mask_bias[TRIPS_UNET_MAX_LEVELS];
    float* final_weight;
    float* final_bias;
    float* inputs[TRIPS_UNET_MAX_LEVELS]; /* dL/d in[i]: the splat's grad_image of level i; required for i < L */
} TripsUnetGrads;

/* Bytes of scratch trips_unet_forward needs (packed fp16 weights and, without a saved state, the fp16 block
 * outputs of every level). */
int trips_unet_workspace_size(const TripsUnetDesc* desc, size_t* bytes);
/* Bytes of the state a training forward keeps for the backward (fp16 block outputs and pre-activations). */
int trips_unet_saved_size(const TripsUnetDesc* desc, size_t* bytes);
/* Bytes of scratch trips_unet_backward needs. */
int trips_unet_backward_workspace_size(const TripsUnetDesc* desc, size_t* bytes);

/* inputs[i]: [batch, C, level_h[i], level_w[i]] fp32 (the splat's output layout TRIPS_LAYOUT_CHW);
 * output: [batch, num_output_channels, level_h[0], level_w[0]] fp32; saved: NULL for inference, else
 * trips_unet_saved_size bytes, 256-byte aligned. Stream-ordered, allocates nothing. */
int trips_unet_forward(TripsCtx* ctx, const TripsUnetDesc* desc, const TripsUnetWeights* weights,
                       const float* const inputs[TRIPS_UNET_MAX_LEVELS], float* output, void* saved, void* workspace,
                       size_t workspace_bytes, void* stream);

/* Backward of the forward that wrote `saved` (same desc, weights and inputs). d_output: [batch, out, H, W] fp32.
 * Intermediate gradients are fp16: they are carried multiplied by grad_scale (a power of two such as 65536 keeps
 * dL/doutput ~ 1e-7 of a mean loss over millions of pixels in range) and every fp32 result is divided by it again.
 * Replaces what autograd does for MultiScaleUnet2dDecOnlySmallFixedImpl::forward in the reference
 * (src/lib/models/Networks.h:1139-1191). Stream-ordered, allocates nothing. */
int trips_unet_backward(TripsCtx* ctx, const TripsUnetDesc* desc, const TripsUnetWeights* weights,
                        const float* const inputs[TRIPS_UNET_MAX_LEVELS], const void* saved, const float* d_output,
                        float grad_scale, const TripsUnetGrads* grads, void* workspace, size_t workspace_bytes,
                        void* stream);

/* Multiply-accumulate operations (2 flops each) of one forward call, for utilisation figures. */
int trips_unet_flops(const TripsUnetDesc* desc, double* flops);

#ifdef __cplusplus
}
#endif
#endif
