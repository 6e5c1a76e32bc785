// C++ / libtorch host side of the reconstruction net over the C ABI of include/trips_unet.h: the classes a TRIPS
// build instantiates from src/lib/models/Networks.h, with the same registered module names, so that
// torch::save / torch::load archives of the network keep their layout:
//   MultiScaleUnet2dParams                  (ini section [MultiScaleUnet2dParams], configs/train_normalnet.ini:200-219)
//   SmallDecStartBlock                      Networks.h:751-787   registers "conv"
//   UpsampleDecOnlySmallBlockFixed          Networks.h:999-1098  registers "up", "convolution"
//   MultiScaleUnet2dDecOnlySmallFixed       Networks.h:1080-1208 registers "start", "up1".., "final"
// GatedBlock is Saiga's (un-vendored): Sequentials "feature_transform" (conv, elu) and "mask_transform"
// (conv, sigmoid). The modules hold parameters only; forward() runs the HIP kernels (fp16 operands on the matrix
// cores), recording one autograd node whose backward is trips_unet_backward.
#pragma once
#include <torch/torch.h>

#include <string>
#include <vector>

#include "../../../include/trips_unet.h"

struct MultiScaleUnet2dParams
{
    int num_input_layers         = 5;
    int num_input_channels       = 4;
    int num_output_channels      = 3;
    int num_layers               = 5;
    bool half_float              = false;  // the device path always runs fp16 operands with fp32 accumulation
    std::string upsample_mode    = "bilinear";
    std::string norm_layer_up    = "id";
    std::string last_act         = "id";
    std::string conv_block_up    = "gated";
    std::string activation       = "elu";
    std::string network_version  = "MultiScaleUnet2dDecOnlySmallFixed";
    std::vector<int> filters_network = {32, 32, 32, 32, 32, 32, 32, 32};
};

class GatedBlockImpl : public torch::nn::Module
{
   public:
    GatedBlockImpl(int in_channels, int out_channels);
    torch::nn::Conv2d feature_conv = nullptr, mask_conv = nullptr;
    torch::nn::Sequential feature_transform, mask_transform;
};
TORCH_MODULE(GatedBlock);

class SmallDecStartBlockImpl : public torch::nn::Module
{
   public:
    SmallDecStartBlockImpl(int in_channels, int out_channels);
    GatedBlock conv = nullptr;
};
TORCH_MODULE(SmallDecStartBlock);

class UpsampleDecOnlySmallBlockFixedImpl : public torch::nn::Module
{
   public:
    UpsampleDecOnlySmallBlockFixedImpl(int in_channels, int conv_out_channels);
    torch::nn::Sequential up;
    GatedBlock convolution = nullptr;
};
TORCH_MODULE(UpsampleDecOnlySmallBlockFixed);

class MultiScaleUnet2dDecOnlySmallFixedImpl : public torch::nn::Module
{
   public:
    explicit MultiScaleUnet2dDecOnlySmallFixedImpl(MultiScaleUnet2dParams params);

    // inputs: the splat's image pyramid, [B, C, H_l, W_l] fp32 per level, finest first; returns [B, out, H, W]
    at::Tensor forward(std::vector<torch::Tensor> inputs);

    // gated block of pyramid level i (the start block's for the coarsest level)
    GatedBlock block(int i);
    // parameters in the order of the C structs: per level feature weight, bias, mask weight, bias; then final
    std::vector<torch::Tensor> ordered_parameters();
    TripsUnetDesc desc(const std::vector<torch::Tensor>& inputs) const;

    MultiScaleUnet2dParams params;
    float grad_scale = 65536.f;  // factor the fp16 gradients inside the backward are carried with
    torch::nn::Sequential final;
    torch::nn::Conv2d final_conv = nullptr;
    SmallDecStartBlock start = nullptr;
    UpsampleDecOnlySmallBlockFixed up[TRIPS_UNET_MAX_LEVELS - 1] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    torch::Tensor forward_workspace, backward_workspace;

    // A viewer sets this: the weights then count as unchanged from one forward without gradients to the next (they
    // are packed to fp16 once, not per frame). Whoever changes them in place afterwards (load, an optimiser step)
    // calls invalidate_packed_weights().
    bool reuse_packed_weights = false;
    void invalidate_packed_weights() { packed_key.clear(); }

   private:
    at::Tensor forward_without_grad(std::vector<torch::Tensor> ins, std::vector<torch::Tensor> prm);
    std::vector<uint64_t> packed_key;  // workspace, level sizes and weight pointers of the last packing
};
TORCH_MODULE(MultiScaleUnet2dDecOnlySmallFixed);
