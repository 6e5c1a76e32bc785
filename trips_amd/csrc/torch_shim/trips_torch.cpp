// Implementation of trips_torch.h: marshals libtorch tensors into the C ABI. No kernels here.
#include "trips_torch.h"

#include <c10/hip/HIPStream.h>
#include <torch/custom_class.h>
#include <torch/library.h>

#include <cfloat>
#include <map>
#include <mutex>
#include <stdexcept>
#include <string>

namespace
{
// one context per device for the whole process
struct ContextTable
{
    std::mutex lock;
    std::map<int, TripsCtx*> by_device;
    ~ContextTable()
    {
        for (auto& kv : by_device) trips_ctx_destroy(kv.second);
    }
};
ContextTable g_contexts;
}  // namespace

TripsCtx* trips_shim_context(int device)
{
    std::lock_guard<std::mutex> guard(g_contexts.lock);
    auto it = g_contexts.by_device.find(device);
    if (it != g_contexts.by_device.end()) return it->second;
    TripsCtx* c = nullptr;
    int rc      = trips_ctx_create(&c, device);
    TORCH_CHECK(rc == TRIPS_OK, "trips_ctx_create: ", trips_last_error_string());
    g_contexts.by_device[device] = c;
    return c;
}

namespace
{
TripsCtx* context_for(const torch::Tensor& t)
{
    TORCH_CHECK(t.is_cuda(), "trips: tensors must live on the GPU (there is no CPU implementation of the splat path)");
    return trips_shim_context(t.get_device());
}

void* current_stream(const torch::Tensor& t) { return (void*)c10::hip::getCurrentHIPStream(t.get_device()).stream(); }

void check(int rc, const char* what)
{
    TORCH_CHECK(rc == TRIPS_OK, what, ": ", trips_last_error_string());
}

TripsSplatDesc make_desc(const NeuralRenderInfo& info, const torch::Tensor& texture)
{
    const RenderParams& p = info.params;
    TORCH_CHECK(p.render_mode == 4 && p.use_layer_point_size && p.render_points_in_all_lower_resolutions &&
                    !p.combine_lists,
                "trips: only render_mode 4 (TILED_BILINEAR_BLEND) with use_layer_point_size, "
                "render_points_in_all_lower_resolutions and !combine_lists is implemented");
    TORCH_CHECK(info.scene, "NeuralRenderInfo::scene is null");
    TORCH_CHECK(!info.images.empty() && info.images.size() <= TRIPS_MAX_VIEWS, "1..", TRIPS_MAX_VIEWS, " images per call");
    TripsSplatDesc d{};
    d.abi_version               = TRIPS_ABI_VERSION;
    d.num_points                = info.scene->point_cloud_cuda->Size();
    d.num_texels                = (int)texture.size(1);
    d.num_channels              = (int)texture.size(0);
    d.num_layers                = info.num_layers;
    d.list_depth                = p.max_pixels_per_list;
    d.num_views                 = (int)info.images.size();
    d.num_images                = (int)info.scene->poses->poses_se3.size(0);
    d.num_cameras               = (int)info.scene->intrinsics->intrinsics.size(0);
    d.train                     = info.train ? 1 : 0;
    d.layout                    = info.train ? TRIPS_LAYOUT_CHW : TRIPS_LAYOUT_HWC;
    d.floor_layer_sizes         = p.floor_layer_sizes ? 1 : 0;
    d.background_mode           = p.background_mode;
    d.drop_out_points_by_radius = p.drop_out_points_by_radius ? 1 : 0;
    d.drop_out_radius_threshold = p.drop_out_radius_threshold;
    d.dist_cutoff               = p.dist_cutoff;
    d.viewer_only               = p.viewer_only ? 1 : 0;
    d.stability_cutoff_value    = p.stability_cutoff_value;
    d.max_list_entries          = 0;
    for (size_t i = 0; i < info.images.size(); ++i)
    {
        const ReducedImageInfo& im = info.images[i];
        TripsView& v               = d.views[i];
        v.w                        = im.w;
        v.h                        = im.h;
        v.image_index              = im.image_index;
        v.camera_index             = im.camera_index;
        v.camera_model_type        = im.camera_model_type;
        for (int k = 0; k < 5; ++k) v.crop_transform[k] = im.crop_transform[k];
        for (int k = 0; k < 4; ++k) v.crop_rotation[k] = im.crop_rotation[k];
    }
    return d;
}

torch::Tensor alloc_bytes(size_t n, const torch::Device& dev)
{
    return torch::empty({(int64_t)std::max<size_t>(n, 256)}, torch::TensorOptions().dtype(torch::kUInt8).device(dev));
}

struct SavedForBackward : public torch::CustomClassHolder
{
    TripsSplatDesc desc;
    torch::Tensor saved_state;
    torch::Tensor position, point_size, index, texture, confidence, background, poses_se3, intrinsics, dropout;
    torch::Tensor displacement;  // [B,N,3] when the scene optimises per-view displacements
    // The backward reads position, point_size, index, poses, intrinsics and displacement again through these
    // tensors (the saved state holds per-point records, not copies of the inputs). Their version counters at the
    // time of the forward: an in-place change in between (an optimiser step or ApplyTangent under gradient
    // accumulation) would silently give gradients of another scene, so the backward refuses it.
    std::vector<std::pair<const char*, uint32_t>> versions;
    std::vector<torch::Tensor> versioned;
    void remember(const char* name, const torch::Tensor& t)
    {
        if (!t.defined()) return;
        versions.emplace_back(name, t._version());
        versioned.push_back(t);
    }
    void check_unchanged() const
    {
        for (size_t i = 0; i < versioned.size(); ++i)
            TORCH_CHECK(versioned[i]._version() == versions[i].second, "PointRender::backward: ", versions[i].first,
                        " was modified in place after the forward that this backward belongs to");
    }
};

TripsSplatIn make_in(const SavedForBackward& s)
{
    TripsSplatIn in{};
    in.position   = s.position.data_ptr<float>();
    in.point_size = s.point_size.data_ptr<float>();
    in.index      = s.index.data_ptr<int32_t>();
    in.texture    = s.texture.data_ptr<float>();
    in.confidence = s.confidence.data_ptr<float>();
    in.background = s.background.data_ptr<float>();
    in.poses_se3  = s.poses_se3.data_ptr<double>();
    in.intrinsics = s.intrinsics.data_ptr<float>();
    in.dropout    = s.dropout.defined() ? s.dropout.data_ptr<float>() : nullptr;
    in.displacement = s.displacement.defined() ? s.displacement.data_ptr<float>() : nullptr;
    return in;
}
}  // namespace

// custom classes travel through IValue / saved_data, as in the reference (RenderInfo.cpp:14-18)
TORCH_LIBRARY(trips_amd, m)
{
    m.class_<NeuralRenderInfo>("NeuralRenderInfo").def(torch::init());
    m.class_<SavedForBackward>("SavedForBackward").def(torch::init());
}

void PointRendererCache::Build(NeuralRenderInfo* info, const TripsSplatDesc& d, size_t workspace_bytes)
{
    std::vector<int64_t> key = {d.num_channels, d.num_points, d.num_layers, d.num_views,
                                d.views[0].h,   d.views[0].w, d.list_depth, d.train};
    const auto dev           = info->scene->texture->texture.device();
    if (key != cache_size || !workspace.defined() || (size_t)workspace.numel() < workspace_bytes)
    {
        workspace      = alloc_bytes(workspace_bytes, dev);
        cache_size     = key;
        dropout_points = torch::Tensor();
    }
    if (info->train && info->params.dropout > 0)
    {
        if (!dropout_points.defined())
            dropout_points = torch::empty({d.num_views, d.num_points}, torch::TensorOptions().dtype(torch::kFloat32).device(dev));
        dropout_points.bernoulli_(info->params.dropout);
    }
    else
    {
        dropout_points = torch::Tensor();
    }
}

namespace torch::autograd
{
variable_list PointRender::forward(AutogradContext* ctx, Variable texture, Variable background_color, Variable points,
                                   Variable pose_tangents, Variable intrinsics, Variable confidence,
                                   Variable dynamic_refinement, Variable layer_of_point, IValue info_v)
{
    ctx->saved_data["render_info"] = info_v;
    NeuralRenderInfo* info         = info_v.toCustomClass<NeuralRenderInfo>().get();
    TORCH_CHECK(info->cache, "NeuralRenderInfo::cache is null");
    TripsCtx* tc = context_for(texture);

    auto s          = c10::make_intrusive<SavedForBackward>();
    s->desc         = make_desc(*info, texture);
    s->position     = points.contiguous();
    s->point_size   = layer_of_point.contiguous();
    s->index        = info->scene->point_cloud_cuda->t_index.contiguous();
    s->texture      = texture.contiguous();
    s->confidence   = confidence.contiguous();
    s->background   = background_color.contiguous();
    s->poses_se3    = info->scene->poses->poses_se3.contiguous();
    s->intrinsics   = intrinsics.contiguous();
    TORCH_CHECK(s->index.scalar_type() == torch::kInt32 && s->poses_se3.scalar_type() == torch::kFloat64 &&
                    pose_tangents.scalar_type() == torch::kFloat64,
                "t_index must be int32, poses_se3 / tangent_poses float64");
    const TripsSplatDesc& d = s->desc;
    if (dynamic_refinement.defined() && dynamic_refinement.dim() > 1)  // a [1] dummy otherwise, PointRenderer.cu:705-706
    {
        TORCH_CHECK(dynamic_refinement.dim() == 3 && dynamic_refinement.size(0) == d.num_views &&
                        dynamic_refinement.size(1) == d.num_points && dynamic_refinement.size(2) == 3,
                    "dynamic_refinement must be [views, points, 3]");
        s->displacement = dynamic_refinement.detach().to(torch::kFloat32).contiguous();
    }

    size_t ws_bytes = 0, saved_bytes = 0;
    check(trips_splat_workspace_size(&d, &ws_bytes), "trips_splat_workspace_size");
    check(trips_splat_saved_size(&d, &saved_bytes), "trips_splat_saved_size");
    info->cache->Build(info, d, ws_bytes);
    s->dropout = info->cache->dropout_points;
    if (info->train) s->saved_state = alloc_bytes(saved_bytes, texture.device());

    int32_t lw[TRIPS_MAX_LAYERS], lh[TRIPS_MAX_LAYERS];
    check(trips_splat_layer_sizes(&d, lw, lh), "trips_splat_layer_sizes");
    variable_list images;
    TripsSplatOut out{};
    for (int l = 0; l < d.num_layers; ++l)
    {
        auto opt = torch::TensorOptions().dtype(torch::kFloat32).device(texture.device());
        images.push_back(info->train ? torch::empty({d.num_views, d.num_channels, lh[l], lw[l]}, opt)
                                     : torch::empty({d.num_views, lh[l], lw[l], d.num_channels}, opt));
        out.image[l] = images.back().data_ptr<float>();
    }
    out.saved       = info->train ? s->saved_state.data_ptr() : nullptr;
    TripsSplatIn in = make_in(*s);
    check(trips_splat_forward(tc, &d, &in, &out, info->cache->workspace.data_ptr(), (size_t)info->cache->workspace.numel(),
                              current_stream(texture)),
          "trips_splat_forward");
    s->remember("t_position", s->position);
    s->remember("t_point_size", s->point_size);
    s->remember("t_index", s->index);
    s->remember("poses_se3", s->poses_se3);
    s->remember("intrinsics", s->intrinsics);
    s->remember("dynamic_refinement_t", s->displacement);
    ctx->saved_data["trips_saved"] = IValue(s);
    if (!info->train)
        for (auto& im : images) im = im.permute({0, 3, 1, 2});  // PointRenderer.cu:747-749
    // depth buffers, then background masks: allocated and zero in the reference's path too
    auto zeros_like_layers = [&]()
    {
        for (int l = 0; l < d.num_layers; ++l)
            images.push_back(torch::zeros({d.num_views, 1, lh[l], lw[l]}, torch::TensorOptions().dtype(torch::kFloat32).device(texture.device())));
    };
    if (info->params.add_depth_to_network) zeros_like_layers();
    if (info->params.output_background_mask) zeros_like_layers();
    return images;
}

variable_list PointRender::backward(AutogradContext* ctx, variable_list grad_output)
{
    IValue info_v          = ctx->saved_data["render_info"];
    NeuralRenderInfo* info = info_v.toCustomClass<NeuralRenderInfo>().get();
    auto s                 = ctx->saved_data["trips_saved"].toCustomClass<SavedForBackward>();
    TORCH_CHECK(s->saved_state.defined(), "PointRender::backward needs a forward with info->train == true");
    s->check_unchanged();
    const TripsSplatDesc& d = s->desc;
    TripsCtx* tc            = context_for(s->texture);
    const auto dev          = s->texture.device();

    // The outputs PointRendererCache::Build(info, false) creates zero-initialised (PointRenderer.cu:226-272). The four
    // per-point ones are written by the kernels, every element (overwrite_point_grads), so they start uninitialised;
    // the small ones are added to and start at zero.
    torch::Tensor g_texture    = torch::empty_like(s->texture);
    torch::Tensor g_confidence = torch::empty_like(s->confidence);
    torch::Tensor g_background = torch::empty_like(s->background);  // the block sums are cleared by the backward itself
    torch::Tensor g_points, g_layer, g_pose, g_intrinsics;
    if (ctx->needs_input_grad(2)) g_points = torch::empty_like(s->position);
    if (ctx->needs_input_grad(7)) g_layer = torch::empty_like(s->point_size);
    if (ctx->needs_input_grad(3))
        g_pose = torch::empty({d.num_images, 6}, torch::TensorOptions().dtype(torch::kFloat64).device(dev));
    if (ctx->needs_input_grad(4)) g_intrinsics = torch::empty_like(s->intrinsics);

    std::vector<torch::Tensor> gi;
    const float* gptr[TRIPS_MAX_LAYERS] = {};
    for (int l = 0; l < d.num_layers; ++l)
    {
        if (grad_output[l].defined())
        {
            TORCH_CHECK(grad_output[l].scalar_type() == torch::kFloat32, "image gradient ", l, " must be float32");
            gi.push_back(grad_output[l].contiguous());
        }
        else
        {
            // a layer nobody consumed (a net with fewer levels than the pyramid) arrives without a gradient
            int32_t lw[TRIPS_MAX_LAYERS], lh[TRIPS_MAX_LAYERS];
            check(trips_splat_layer_sizes(&d, lw, lh), "trips_splat_layer_sizes");
            gi.push_back(torch::zeros({d.num_views, d.num_channels, lh[l], lw[l]}, torch::TensorOptions().dtype(torch::kFloat32).device(dev)));
        }
        gptr[l] = gi.back().data_ptr<float>();
    }
    TripsSplatGrads g{};
    g.d_texture     = g_texture.data_ptr<float>();
    g.d_confidence  = g_confidence.data_ptr<float>();
    g.d_background  = g_background.data_ptr<float>();
    g.d_position    = g_points.defined() ? g_points.data_ptr<float>() : nullptr;
    g.d_point_size  = g_layer.defined() ? g_layer.data_ptr<float>() : nullptr;
    g.d_pose        = g_pose.defined() ? g_pose.data_ptr<double>() : nullptr;
    g.d_intrinsics  = g_intrinsics.defined() ? g_intrinsics.data_ptr<float>() : nullptr;
    g.overwrite_point_grads = 1;
    g.clear_block_sums      = 1;
    TripsSplatIn in = make_in(*s);
    check(trips_splat_backward(tc, &d, &in, s->saved_state.data_ptr(), gptr, &g, info->cache->workspace.data_ptr(),
                               (size_t)info->cache->workspace.numel(), current_stream(s->texture)),
          "trips_splat_backward");
    // order of PointRenderer.cu:1423-1426 (dynamic-refinement gradient undefined), then one for `info`
    return {g_texture, g_background, g_points, g_pose, g_intrinsics, g_confidence, Variable(), g_layer, Variable()};
}
}  // namespace torch::autograd

std::vector<torch::Tensor> BlendPointCloud(NeuralRenderInfo* info)
{
    torch::intrusive_ptr<NeuralRenderInfo> render_data = torch::make_intrusive<NeuralRenderInfo>(*info);
    TORCH_CHECK(render_data->scene && render_data->scene->texture, "scene / texture missing");
    if (!render_data->scene->dynamic_refinement_t.defined())
        render_data->scene->dynamic_refinement_t = torch::zeros({1}, render_data->scene->texture->texture.options());
    return torch::autograd::PointRender::apply(
        render_data->scene->texture->texture, render_data->scene->texture->background_color,
        render_data->scene->point_cloud_cuda->t_position, render_data->scene->poses->tangent_poses,
        render_data->scene->intrinsics->intrinsics, render_data->scene->texture->confidence_value_of_point,
        render_data->scene->dynamic_refinement_t, render_data->scene->point_cloud_cuda->t_point_size,
        torch::IValue(render_data));
}

void ApplyTangentToPose(torch::Tensor tangent, torch::Tensor pose)
{
    TORCH_CHECK(tangent.is_contiguous() && pose.is_contiguous(), "tangent / pose must be contiguous");
    TORCH_CHECK(tangent.scalar_type() == torch::kFloat64 && pose.scalar_type() == torch::kFloat64, "float64 expected");
    check(trips_apply_tangent(context_for(pose), tangent.data_ptr<double>(), pose.data_ptr<double>(), (int)tangent.size(0),
                              current_stream(pose)),
          "trips_apply_tangent");
}

void PoseModule_::ApplyTangent() { ApplyTangentToPose(tangent_poses, poses_se3); }

namespace torch::optim
{
MyAdam::MyAdam(std::vector<OptimizerParamGroup> param_groups, MyAdamOptions defaults)
    : Optimizer(std::move(param_groups), std::make_unique<MyAdamOptions>(defaults))
{
    TORCH_CHECK(defaults.lr() >= 0, "Invalid learning rate: ", defaults.lr());
    TORCH_CHECK(defaults.eps() >= 0, "Invalid epsilon value: ", defaults.eps());
    auto betas = defaults.betas();
    TORCH_CHECK(0 <= std::get<0>(betas) && std::get<0>(betas) < 1.0, "Invalid beta parameter at index 0: ", std::get<0>(betas));
    TORCH_CHECK(0 <= std::get<1>(betas) && std::get<1>(betas) < 1.0, "Invalid beta parameter at index 1: ", std::get<1>(betas));
    TORCH_CHECK(defaults.relative_weight_decay() >= 0, "Invalid relative_weight_decay value: ", defaults.relative_weight_decay());
    TORCH_CHECK(defaults.absolute_weight_decay() >= 0, "Invalid absolute_weight_decay value: ", defaults.absolute_weight_decay());
}

bool MyAdam::describe(Tensor& p, OptimizerParamGroup& group, bool packed, TripsAdamTensor& t, std::vector<Tensor>& keep)
{
    auto grad = p.grad();
    TORCH_CHECK(!grad.is_sparse(), "Adam does not support sparse gradients");
    TORCH_CHECK(p.is_contiguous(), "MyAdam needs contiguous parameters");
    TORCH_CHECK(p.scalar_type() == torch::kFloat || p.scalar_type() == torch::kDouble, "float32 / float64 only");
    auto& options = static_cast<MyAdamOptions&>(group.options());
    int64_t current_step = 0;
    t                    = TripsAdamTensor{};
    if (!packed)
    {
        auto it = state_.find(p.unsafeGetTensorImpl());
        if (it == state_.end())
        {
            auto st = std::make_unique<MyAdamParamState>();
            st->param_steps(torch::zeros_like(p, MemoryFormat::Preserve).to(torch::kInt32));
            st->first_moments(torch::zeros_like(p, MemoryFormat::Preserve).to(torch::kFloat32));
            st->second_moments(torch::zeros_like(p, MemoryFormat::Preserve).to(torch::kFloat32));
            st->current_step(0);
            state_[p.unsafeGetTensorImpl()] = std::move(st);
        }
        auto& st = static_cast<MyAdamParamState&>(*state_[p.unsafeGetTensorImpl()]);
        st.current_step(st.current_step() + 1);
        current_step    = st.current_step();
        t.first_moment  = st.first_moments().data_ptr<float>();
        t.second_moment = st.second_moments().data_ptr<float>();
        t.steps         = st.param_steps().data_ptr();
        t.steps_dtype   = st.param_steps().scalar_type() == torch::kInt32 ? TRIPS_STEPS_I32 : TRIPS_STEPS_I64;
    }
    const double beta1 = std::get<0>(options.betas()), beta2 = std::get<1>(options.betas());
    Tensor g = grad.contiguous();
    keep.push_back(g);
    t.weights                   = p.data_ptr();
    t.grads                     = g.data_ptr();
    t.n                         = p.numel();
    t.dtype                     = p.scalar_type() == torch::kDouble ? TRIPS_DTYPE_F64 : TRIPS_DTYPE_F32;
    t.lr                        = (float)options.lr();
    t.beta1                     = (float)beta1;
    t.beta2                     = (float)beta2;
    t.eps                       = (float)options.eps();
    t.relative_weight_decay     = (float)options.relative_weight_decay();
    t.absolute_weight_decay     = (float)options.absolute_weight_decay();
    t.weight_clipping_magnitude = (float)options.weight_clipping_magnitude();
    t.lower_lr_bound            = 0;
    t.upper_lr_bound            = FLT_MAX;
    t.loss_scale                = 1.f;
    if (options.adabound() && !packed)
    {
        // AdaBound bounds, MyAdam.cu:213-221
        t.lower_lr_bound = 0.1f - 0.1f / ((1 - (float)beta2) * (float)current_step + 1);
        t.upper_lr_bound = 0.1f + 0.1f / ((1 - (float)beta2) * (float)current_step);
    }
    return true;
}

void MyAdam::save(serialize::OutputArchive& archive) const
{
    int64_t index = 0;
    for (const auto& group : param_groups_)
        for (const auto& p : group.params())
        {
            const std::string key = std::to_string(index++);
            auto it               = state_.find(p.unsafeGetTensorImpl());
            if (it == state_.end()) continue;
            const auto& st = static_cast<const MyAdamParamState&>(*it->second);
            archive.write(key + "/first_moments", st.first_moments());
            archive.write(key + "/second_moments", st.second_moments());
            archive.write(key + "/param_steps", st.param_steps());
            archive.write(key + "/current_step", torch::tensor(st.current_step(), torch::kInt64));
        }
}

void MyAdam::load(serialize::InputArchive& archive)
{
    int64_t index = 0;
    for (auto& group : param_groups_)
        for (auto& p : group.params())
        {
            const std::string key = std::to_string(index++);
            Tensor m, v, steps, current;
            if (!archive.try_read(key + "/first_moments", m)) continue;
            archive.read(key + "/second_moments", v);
            archive.read(key + "/param_steps", steps);
            archive.read(key + "/current_step", current);
            TORCH_CHECK(m.sizes() == p.sizes(), "MyAdam::load: state of parameter ", key, " does not fit its shape");
            auto st = std::make_unique<MyAdamParamState>();
            st->first_moments(m.to(p.device()).contiguous());
            st->second_moments(v.to(p.device()).contiguous());
            st->param_steps(steps.to(p.device()).contiguous());
            st->current_step(current.item<int64_t>());
            state_[p.unsafeGetTensorImpl()] = std::move(st);
        }
}

torch::Tensor MyAdam::step(LossClosure closure)
{
    NoGradGuard no_grad;
    Tensor loss = {};
    if (closure != nullptr)
    {
        at::AutoGradMode enable_grad(true);
        loss = closure();
    }
    std::vector<TripsAdamTensor> descs;
    std::vector<Tensor> keep;
    Tensor any;
    for (auto& group : param_groups_)
    {
        for (auto& p : group.params())
        {
            if (!p.grad().defined()) continue;
            TripsAdamTensor t;
            describe(p, group, false, t, keep);
            descs.push_back(t);
            any = p;
        }
    }
    if (!descs.empty())
        check(trips_adam_step_fused(context_for(any), descs.data(), (int)descs.size(), current_stream(any)),
              "trips_adam_step_fused");
    return loss;
}

MyAdamPoints::MyAdamPoints(std::vector<OptimizerParamGroup> param_groups, Tensor position, Tensor point_size, Tensor texture,
                           Tensor confidence, MyAdamOptions defaults)
    : MyAdam(std::move(param_groups), defaults)
{
    packed_[0] = position, packed_[1] = point_size, packed_[2] = texture, packed_[3] = confidence;
    for (auto& q : packed_)
    {
        TORCH_CHECK(q.defined() && q.scalar_type() == torch::kFloat && q.is_contiguous(),
                    "MyAdamPoints: the point parameters must be contiguous float32 tensors");
        bool found = false;
        for (auto& group : param_groups_)
            for (auto& p : group.params()) found = found || p.unsafeGetTensorImpl() == q.unsafeGetTensorImpl();
        TORCH_CHECK(found, "MyAdamPoints: position, point_size, texture and confidence must be among the optimised parameters");
    }
}

int MyAdamPoints::slot_of(const Tensor& p) const
{
    for (int i = 0; i < 4; ++i)
        if (packed_[i].unsafeGetTensorImpl() == p.unsafeGetTensorImpl()) return i;
    return -1;
}

torch::Tensor MyAdamPoints::step(LossClosure closure)
{
    NoGradGuard no_grad;
    Tensor loss = {};
    if (closure != nullptr)
    {
        at::AutoGradMode enable_grad(true);
        loss = closure();
    }
    bool any_packed_grad = false;
    for (auto& q : packed_) any_packed_grad = any_packed_grad || q.grad().defined();
    std::vector<TripsAdamTensor> descs;
    TripsAdamTensor packed_descs[4];
    std::vector<Tensor> keep;
    Tensor any;
    for (auto& group : param_groups_)
    {
        for (auto& p : group.params())
        {
            const int slot = slot_of(p);
            if (slot < 0)
            {
                if (!p.grad().defined()) continue;
                TripsAdamTensor t;
                describe(p, group, false, t, keep);
                descs.push_back(t);
                any = p;
                continue;
            }
            if (!any_packed_grad) continue;
            const bool has_grad = p.grad().defined();
            if (!has_grad)
            {
                // a point parameter without a gradient in this step: zeros leave it and its state as they are
                if (!zero_grads_[slot].defined() || zero_grads_[slot].sizes() != p.sizes()) zero_grads_[slot] = torch::zeros_like(p);
                p.mutable_grad() = zero_grads_[slot];
            }
            describe(p, group, true, packed_descs[slot], keep);
            if (!has_grad) p.mutable_grad() = Tensor();
            if (has_grad) packed_steps_[slot] += 1;
            auto& options = static_cast<MyAdamOptions&>(group.options());
            if (options.adabound() && packed_steps_[slot] > 0)
            {
                const float beta2                 = (float)std::get<1>(options.betas());
                packed_descs[slot].lower_lr_bound = 0.1f - 0.1f / ((1 - beta2) * (float)packed_steps_[slot] + 1);
                packed_descs[slot].upper_lr_bound = 0.1f + 0.1f / ((1 - beta2) * (float)packed_steps_[slot]);
            }
        }
    }
    if (any_packed_grad)
    {
        const int64_t n = packed_[0].size(0), c = packed_[2].size(0);
        TORCH_CHECK(packed_[0].dim() == 2 && packed_[0].size(1) == 4 && packed_[2].dim() == 2 && packed_[2].size(1) == n &&
                        packed_[1].numel() == n && packed_[3].numel() == n,
                    "MyAdamPoints: position [N,4], point_size [N], texture [C,N], confidence [N] expected");
        size_t bytes = 0;
        int row      = 0;
        check(trips_adam_points_state_size((int)n, (int)c, &bytes, &row), "trips_adam_points_state_size");
        if (!packed_state.defined())
            packed_state = torch::zeros({n, row / 4}, torch::TensorOptions().dtype(torch::kInt32).device(packed_[0].device()));
        TORCH_CHECK(packed_state.size(0) == n && packed_state.size(1) == row / 4,
                    "MyAdamPoints: the number of points changed without shrinkInternalState / appendToInternalState");
        check(trips_adam_step_points(context_for(packed_[0]), packed_descs, (int)n, (int)c, packed_state.data_ptr(),
                                     current_stream(packed_[0])),
              "trips_adam_step_points");
    }
    if (!descs.empty())
        check(trips_adam_step_fused(context_for(any), descs.data(), (int)descs.size(), current_stream(any)),
              "trips_adam_step_fused");
    return loss;
}

void MyAdamPoints::save(serialize::OutputArchive& archive) const
{
    MyAdam::save(archive);  // (the four packed parameters have no per-tensor state and are passed over)
    if (packed_state.defined()) archive.write("points/packed_state", packed_state);
    archive.write("points/steps", torch::tensor(std::vector<int64_t>(packed_steps_, packed_steps_ + 4), torch::kInt64));
}

void MyAdamPoints::load(serialize::InputArchive& archive)
{
    MyAdam::load(archive);
    Tensor rows, steps;
    if (archive.try_read("points/packed_state", rows)) packed_state = rows.to(packed_[0].device()).contiguous();
    archive.read("points/steps", steps);
    for (int i = 0; i < 4; ++i) packed_steps_[i] = steps[i].item<int64_t>();
}

void MyAdamPoints::shrinkInternalState(int param_group_index, torch::Tensor indices_to_keep)
{
    TORCH_CHECK(param_group_index < (int)param_groups_.size());
    for (auto& p : param_groups_[param_group_index].params())
        if (slot_of(p) == 2 && packed_state.defined())
            packed_state = packed_state.index_select(0, indices_to_keep.squeeze().to(packed_state.device())).contiguous();
    MyAdam::shrinkInternalState(param_group_index, indices_to_keep);  // (the packed four have no per-tensor state)
}

void MyAdamPoints::appendToInternalState(int param_group_index, int new_size)
{
    TORCH_CHECK(param_group_index < (int)param_groups_.size());
    for (auto& p : param_groups_[param_group_index].params())
        if (slot_of(p) == 2 && packed_state.defined())
            packed_state = torch::cat({packed_state, torch::zeros({new_size - packed_state.size(0), packed_state.size(1)},
                                                                  packed_state.options())})
                               .contiguous();
    MyAdam::appendToInternalState(param_group_index, new_size);
}

// state follows the last dimension of the parameter (MyAdam.cu:346-415)
void MyAdam::shrinkInternalState(int param_group_index, torch::Tensor indices_to_keep)
{
    TORCH_CHECK(param_group_index < (int)param_groups_.size());
    for (auto& p : param_groups_[param_group_index].params())
    {
        auto it = state_.find(p.unsafeGetTensorImpl());
        if (it == state_.end()) continue;
        auto& st   = static_cast<MyAdamParamState&>(*it->second);
        auto keepf = [&](torch::Tensor t)
        { return t.index_select(t.dim() - 1, indices_to_keep.squeeze().to(t.device())).contiguous(); };
        st.first_moments(keepf(st.first_moments()));
        st.second_moments(keepf(st.second_moments()));
        st.param_steps(keepf(st.param_steps()));
    }
}

void MyAdam::appendToInternalState(int param_group_index, int new_size)
{
    TORCH_CHECK(param_group_index < (int)param_groups_.size());
    for (auto& p : param_groups_[param_group_index].params())
    {
        auto it = state_.find(p.unsafeGetTensorImpl());
        if (it == state_.end()) continue;
        auto& st  = static_cast<MyAdamParamState&>(*it->second);
        auto grow = [&](torch::Tensor t)
        {
            std::vector<int64_t> sizes(t.sizes().begin(), t.sizes().end());
            sizes.back() = new_size - t.size(-1);
            return torch::cat({t, torch::zeros(sizes, t.options())}, -1).contiguous();
        };
        st.first_moments(grow(st.first_moments()));
        st.second_moments(grow(st.second_moments()));
        st.param_steps(grow(st.param_steps()));
    }
}
}  // namespace torch::optim
