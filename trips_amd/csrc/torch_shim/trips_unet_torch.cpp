// Implementation of trips_unet_torch.h: marshals libtorch tensors into the C ABI of the net. No kernels here.
#include "trips_unet_torch.h"

#include <c10/hip/HIPStream.h>

#include "trips_torch.h"

namespace
{
TripsCtx* unet_context(const torch::Tensor& t)
{
    TORCH_CHECK(t.is_cuda(), "trips: the net needs GPU tensors (there is no CPU implementation)");
    return trips_shim_context(t.get_device());
}

void* stream_of(const torch::Tensor& t) { return (void*)c10::hip::getCurrentHIPStream(t.get_device()).stream(); }

void check(int rc, const char* what) { TORCH_CHECK(rc == TRIPS_OK, what, ": ", trips_last_error_string()); }

torch::Tensor bytes_on(const torch::Tensor& like, size_t n)
{
    return torch::empty({(int64_t)std::max<size_t>(n, 256)}, torch::TensorOptions().dtype(torch::kUInt8).device(like.device()));
}

TripsUnetWeights weights_struct(int L, const std::vector<torch::Tensor>& p)
{
    TripsUnetWeights w{};
    for (int i = 0; i < L; ++i)
    {
        w.feature_weight[i] = p[4 * i].data_ptr<float>();
        w.feature_bias[i]   = p[4 * i + 1].data_ptr<float>();
        w.mask_weight[i]    = p[4 * i + 2].data_ptr<float>();
        w.mask_bias[i]      = p[4 * i + 3].data_ptr<float>();
    }
    w.final_weight = p[4 * L].data_ptr<float>();
    w.final_bias   = p[4 * L + 1].data_ptr<float>();
    return w;
}

struct UnetFunction : public torch::autograd::Function<UnetFunction>
{
    // tensors = L inputs, then the ordered parameters
    static torch::autograd::variable_list forward(torch::autograd::AutogradContext* ctx, int64_t net_ptr,
                                                  at::TensorList tensors)
    {
        auto* net   = reinterpret_cast<MultiScaleUnet2dDecOnlySmallFixedImpl*>(net_ptr);
        const int L = net->params.num_layers;
        std::vector<torch::Tensor> ins(tensors.begin(), tensors.begin() + L), prm(tensors.begin() + L, tensors.end());
        for (auto& t : ins) t = t.detach().contiguous();
        for (auto& t : prm) t = t.detach().to(ins[0].device(), torch::kFloat32).contiguous();
        const TripsUnetDesc d    = net->desc(ins);
        const TripsUnetWeights w = weights_struct(L, prm);
        size_t ws = 0, sv = 0;
        check(trips_unet_workspace_size(&d, &ws), "trips_unet_workspace_size");
        check(trips_unet_saved_size(&d, &sv), "trips_unet_saved_size");
        if (!net->forward_workspace.defined() || (size_t)net->forward_workspace.numel() < ws || net->forward_workspace.device() != ins[0].device())
            net->forward_workspace = bytes_on(ins[0], ws);
        torch::Tensor saved = bytes_on(ins[0], sv);
        torch::Tensor out   = torch::empty({d.batch, d.num_output_channels, d.level_h[0], d.level_w[0]}, ins[0].options());
        const float* in_ptrs[TRIPS_UNET_MAX_LEVELS] = {};
        for (int i = 0; i < L; ++i) in_ptrs[i] = ins[i].data_ptr<float>();
        check(trips_unet_forward(unet_context(ins[0]), &d, &w, in_ptrs, out.data_ptr<float>(), saved.data_ptr(),
                                 net->forward_workspace.data_ptr(), (size_t)net->forward_workspace.numel(), stream_of(ins[0])),
              "trips_unet_forward");
        ctx->saved_data["net"] = net_ptr;
        std::vector<torch::Tensor> keep = ins;
        keep.insert(keep.end(), prm.begin(), prm.end());
        keep.push_back(saved);
        ctx->saved_data["tensors"] = keep;
        return {out};
    }

    static torch::autograd::variable_list backward(torch::autograd::AutogradContext* ctx, torch::autograd::variable_list grad_output)
    {
        auto* net   = reinterpret_cast<MultiScaleUnet2dDecOnlySmallFixedImpl*>(ctx->saved_data["net"].toInt());
        const int L = net->params.num_layers;
        std::vector<torch::Tensor> keep = ctx->saved_data["tensors"].toTensorVector();
        std::vector<torch::Tensor> ins(keep.begin(), keep.begin() + L), prm(keep.begin() + L, keep.end() - 1);
        torch::Tensor saved      = keep.back();
        const TripsUnetDesc d    = net->desc(ins);
        const TripsUnetWeights w = weights_struct(L, prm);
        size_t ws = 0;
        check(trips_unet_backward_workspace_size(&d, &ws), "trips_unet_backward_workspace_size");
        if (!net->backward_workspace.defined() || (size_t)net->backward_workspace.numel() < ws || net->backward_workspace.device() != ins[0].device())
            net->backward_workspace = bytes_on(ins[0], ws);
        torch::Tensor d_out = grad_output[0].contiguous().to(torch::kFloat32);
        TripsUnetGrads g{};
        std::vector<torch::Tensor> d_ins, d_prm;
        for (auto& t : ins) d_ins.push_back(torch::empty_like(t));
        for (auto& t : prm) d_prm.push_back(torch::empty_like(t));
        for (int i = 0; i < L; ++i)
        {
            g.feature_weight[i] = d_prm[4 * i].data_ptr<float>();
            g.feature_bias[i]   = d_prm[4 * i + 1].data_ptr<float>();
            g.mask_weight[i]    = d_prm[4 * i + 2].data_ptr<float>();
            g.mask_bias[i]      = d_prm[4 * i + 3].data_ptr<float>();
            g.inputs[i]         = d_ins[i].data_ptr<float>();
        }
        g.final_weight = d_prm[4 * L].data_ptr<float>();
        g.final_bias   = d_prm[4 * L + 1].data_ptr<float>();
        const float* in_ptrs[TRIPS_UNET_MAX_LEVELS] = {};
        for (int i = 0; i < L; ++i) in_ptrs[i] = ins[i].data_ptr<float>();
        check(trips_unet_backward(unet_context(ins[0]), &d, &w, in_ptrs, saved.data_ptr(), d_out.data_ptr<float>(), net->grad_scale, &g,
                                  net->backward_workspace.data_ptr(), (size_t)net->backward_workspace.numel(), stream_of(ins[0])),
              "trips_unet_backward");
        torch::autograd::variable_list result = {torch::Tensor()};  // net_ptr
        result.insert(result.end(), d_ins.begin(), d_ins.end());
        result.insert(result.end(), d_prm.begin(), d_prm.end());
        return result;
    }
};
}  // namespace

GatedBlockImpl::GatedBlockImpl(int in_channels, int out_channels)
{
    feature_conv = torch::nn::Conv2d(torch::nn::Conv2dOptions(in_channels, out_channels, 3).padding(1));
    mask_conv    = torch::nn::Conv2d(torch::nn::Conv2dOptions(in_channels, out_channels, 3).padding(1));
    feature_transform->push_back(feature_conv);
    feature_transform->push_back(torch::nn::ELU());
    mask_transform->push_back(mask_conv);
    mask_transform->push_back(torch::nn::Sigmoid());
    register_module("feature_transform", feature_transform);
    register_module("mask_transform", mask_transform);
}

SmallDecStartBlockImpl::SmallDecStartBlockImpl(int in_channels, int out_channels)
{
    conv = GatedBlock(in_channels, out_channels);
    register_module("conv", conv);
}

UpsampleDecOnlySmallBlockFixedImpl::UpsampleDecOnlySmallBlockFixedImpl(int in_channels, int conv_out_channels)
{
    up->push_back(torch::nn::Upsample(
        torch::nn::UpsampleOptions().scale_factor(std::vector<double>{2.0, 2.0}).mode(torch::kBilinear).align_corners(false)));
    convolution = GatedBlock(in_channels, conv_out_channels);
    register_module("up", up);
    register_module("convolution", convolution);
}

MultiScaleUnet2dDecOnlySmallFixedImpl::MultiScaleUnet2dDecOnlySmallFixedImpl(MultiScaleUnet2dParams p) : params(p)
{
    TORCH_CHECK(p.upsample_mode == "bilinear" && p.norm_layer_up == "id" && p.last_act == "id" && p.conv_block_up == "gated" &&
                    p.activation == "elu",
                "trips: only upsample_mode=bilinear, norm_layer_up=id, last_act=id, conv_block_up=gated, activation=elu are built");
    TORCH_CHECK(p.num_layers >= 1 && p.num_layers <= TRIPS_UNET_MAX_LEVELS && p.num_input_layers >= p.num_layers &&
                    (int)p.filters_network.size() >= p.num_layers,
                "trips: num_layers / num_input_layers / filters_network do not fit");
    const int L = p.num_layers, C = p.num_input_channels;
    const auto& F = p.filters_network;
    // Networks.h:1104-1118: the start block outputs F[L-1] - 2C, block i outputs F[i] - 2C (F[0] - C for the last)
    start = SmallDecStartBlock(C, F[L - 1] - 2 * C);
    register_module("start", start);
    for (int i = L - 2; i >= 0; --i)
    {
        up[i] = UpsampleDecOnlySmallBlockFixed(F[i + 1], F[i] - (i == 0 ? C : 2 * C));
        register_module("up" + std::to_string(i + 1), up[i]);
    }
    final_conv = torch::nn::Conv2d(torch::nn::Conv2dOptions(F[0], p.num_output_channels, 1));
    final->push_back(final_conv);
    final->push_back(torch::nn::Identity());
    register_module("final", final);
}

GatedBlock MultiScaleUnet2dDecOnlySmallFixedImpl::block(int i)
{
    return i == params.num_layers - 1 ? start->conv : up[i]->convolution;
}

std::vector<torch::Tensor> MultiScaleUnet2dDecOnlySmallFixedImpl::ordered_parameters()
{
    std::vector<torch::Tensor> out;
    for (int i = 0; i < params.num_layers; ++i)
    {
        GatedBlock b = block(i);
        out.push_back(b->feature_conv->weight);
        out.push_back(b->feature_conv->bias);
        out.push_back(b->mask_conv->weight);
        out.push_back(b->mask_conv->bias);
    }
    out.push_back(final_conv->weight);
    out.push_back(final_conv->bias);
    return out;
}

TripsUnetDesc MultiScaleUnet2dDecOnlySmallFixedImpl::desc(const std::vector<torch::Tensor>& inputs) const
{
    TripsUnetDesc d{};
    d.abi_version         = TRIPS_ABI_VERSION;
    d.num_levels          = params.num_layers;
    d.num_input_channels  = params.num_input_channels;
    d.num_output_channels = params.num_output_channels;
    d.batch               = (int)inputs[0].size(0);
    for (int i = 0; i < params.num_layers; ++i)
    {
        d.filters[i] = params.filters_network[i];
        d.level_w[i] = (int)inputs[i].size(3);
        d.level_h[i] = (int)inputs[i].size(2);
    }
    return d;
}

at::Tensor MultiScaleUnet2dDecOnlySmallFixedImpl::forward(std::vector<torch::Tensor> inputs)
{
    TORCH_CHECK((int)inputs.size() == params.num_input_layers, "trips: ", inputs.size(), " input layers, params.num_input_layers = ",
                params.num_input_layers);
    const int L = params.num_layers;
    torch::autograd::variable_list tensors;
    for (int i = 0; i < L; ++i)
    {
        TORCH_CHECK(inputs[i].defined() && inputs[i].dim() == 4 && inputs[i].size(1) == params.num_input_channels &&
                        inputs[i].scalar_type() == torch::kFloat32,
                    "trips: inputs[", i, "] must be float32 [B, ", params.num_input_channels, ", H, W]");
        tensors.push_back(inputs[i]);
    }
    bool needs_grad = false;
    for (auto& p : ordered_parameters())
    {
        tensors.push_back(p);
        needs_grad |= p.requires_grad();
    }
    for (int i = 0; i < L; ++i) needs_grad |= inputs[i].requires_grad();
    if (!torch::GradMode::is_enabled() || !needs_grad)
        return forward_without_grad(std::vector<torch::Tensor>(tensors.begin(), tensors.begin() + L),
                                    std::vector<torch::Tensor>(tensors.begin() + L, tensors.end()));
    packed_key.clear();  // (the training forward packs into the same workspace, and the weights are about to change)
    return UnetFunction::apply(reinterpret_cast<int64_t>(this), at::TensorList(tensors))[0];
}

// Nothing is kept for a backward: the block outputs live in the workspace.
at::Tensor MultiScaleUnet2dDecOnlySmallFixedImpl::forward_without_grad(std::vector<torch::Tensor> ins, std::vector<torch::Tensor> prm)
{
    const int L = params.num_layers;
    for (auto& t : ins) t = t.detach().contiguous();
    for (auto& t : prm) t = t.detach().to(ins[0].device(), torch::kFloat32).contiguous();
    TripsUnetDesc d          = desc(ins);
    const TripsUnetWeights w = weights_struct(L, prm);
    size_t ws = 0;
    check(trips_unet_workspace_size(&d, &ws), "trips_unet_workspace_size");
    if (!forward_workspace.defined() || (size_t)forward_workspace.numel() < ws || forward_workspace.device() != ins[0].device())
        forward_workspace = bytes_on(ins[0], ws);
    std::vector<uint64_t> key{(uint64_t)reinterpret_cast<uintptr_t>(forward_workspace.data_ptr()), (uint64_t)d.batch};
    for (int i = 0; i < L; ++i) key.push_back(((uint64_t)d.level_w[i] << 32) | (uint64_t)d.level_h[i]);
    for (auto& t : prm) key.push_back((uint64_t)reinterpret_cast<uintptr_t>(t.data_ptr()));
    if (reuse_packed_weights && key == packed_key) d.weights_packed = 1;
    packed_key = key;
    torch::Tensor out = torch::empty({d.batch, d.num_output_channels, d.level_h[0], d.level_w[0]}, ins[0].options());
    const float* in_ptrs[TRIPS_UNET_MAX_LEVELS] = {};
    for (int i = 0; i < L; ++i) in_ptrs[i] = ins[i].data_ptr<float>();
    check(trips_unet_forward(unet_context(ins[0]), &d, &w, in_ptrs, out.data_ptr<float>(), /*saved*/ nullptr,
                             forward_workspace.data_ptr(), (size_t)forward_workspace.numel(), stream_of(ins[0])),
          "trips_unet_forward");
    return out;
}
