// libtorch host side of the splat path: the reference's operator surface over the C ABI (include/trips_splat.h).
//
// Same names, argument order and return arity as the reference so that its callers compile unchanged against
// this header for the render path (paths relative to the reference checkout):
//   ReducedImageInfo             src/lib/data/SceneData.h:40-61
//   RenderParams (subset)        src/lib/data/Settings.h:19-83
//   NeuralRenderInfo             src/lib/rendering/PointRenderer.h:23-34
//   PointRendererCache           src/lib/rendering/PointRenderer.h:120-232
//   torch::autograd::PointRender src/lib/rendering/PointRenderer.h:39-47, RenderInfo.cpp:44-80
//   BlendPointCloud              src/lib/rendering/PointRenderer.h:53, RenderInfo.cpp:27-40
//   ApplyTangentToPose           src/lib/rendering/PointRenderer.h:64, PointRenderer.cu:1449-1456
//   torch::optim::MyAdam         src/lib/models/MyAdam.h:28-85
// Saiga / Sophus types of the reference (IntrinsicsPinholef, Matrix<float,2,2>, CudaTimerSystem) are replaced by
// plain arrays and an opaque pointer; NeuralScene is reduced to the tensors the operator reads.
#pragma once
#include <torch/torch.h>

#include <array>
#include <memory>
#include <vector>

#include "../../../include/trips_splat.h"

struct ReducedImageInfo
{
    int w = 0, h = 0;
    int image_index          = -1;
    int camera_index         = -1;
    int camera_model_type    = 0;                        // CameraModel::PINHOLE_DISTORTION
    std::array<float, 5> crop_transform = {1, 1, 0, 0, 0};  // fx fy cx cy s
    std::array<float, 4> crop_rotation  = {1, 0, 0, 1};     // row-major 2x2
};

struct RenderParams
{
    float dropout                               = 0.25f;
    float drop_out_radius_threshold             = 0.6f;
    bool drop_out_points_by_radius              = true;
    int num_texture_channels                    = -1;
    float dist_cutoff                           = 20.f;
    float stability_cutoff_value                = 10000.f;
    bool viewer_only                            = false;
    int render_mode                             = 4;  // TILED_BILINEAR_BLEND, the only mode implemented
    bool use_layer_point_size                   = true;
    bool combine_lists                          = false;
    bool render_points_in_all_lower_resolutions = true;
    bool normalize_grads                        = false;
    // The path implemented here never writes these two outputs in the reference either (RenderForward.cu:43 keeps
    // blend_out commented out, no kernel of the new path takes the depth buffers): they come back as zeros, after
    // the L images, so that the output arity matches (PointRenderer.cu:482-505,1183-1190)
    bool add_depth_to_network   = false;
    bool output_background_mask = false;
    // not in the reference
    int background_mode     = TRIPS_BG_REFERENCE;
    int max_pixels_per_list = 16;  // PointRenderer.h:178
    bool floor_layer_sizes  = false;  // network_version == "MultiScaleUnet2d", PointRenderer.cu:385-394
};

// The tensors of the reference's NeuralScene that the operator reads, under the same member paths.
struct NeuralTexture_
{
    torch::Tensor texture;                    // [C,N]
    torch::Tensor background_color;           // [C]
    torch::Tensor confidence_value_of_point;  // [1,N]
};
struct NeuralPointCloudCuda_
{
    torch::Tensor t_position;    // [N,4]
    torch::Tensor t_point_size;  // [N,1]
    torch::Tensor t_index;       // [N,1] int32
    int Size() const { return (int)t_position.size(0); }
};
struct PoseModule_
{
    torch::Tensor poses_se3;      // [F,8] f64
    torch::Tensor tangent_poses;  // [F,6] f64
    void ApplyTangent();
};
struct IntrinsicsModule_
{
    torch::Tensor intrinsics;  // [Cam,13]
};
struct NeuralScene
{
    std::shared_ptr<NeuralTexture_> texture                 = std::make_shared<NeuralTexture_>();
    std::shared_ptr<NeuralPointCloudCuda_> point_cloud_cuda = std::make_shared<NeuralPointCloudCuda_>();
    std::shared_ptr<PoseModule_> poses                      = std::make_shared<PoseModule_>();
    std::shared_ptr<IntrinsicsModule_> intrinsics           = std::make_shared<IntrinsicsModule_>();
    torch::Tensor dynamic_refinement_t;  // dummy [1] tensor when no displacement is optimised
};

class PointRendererCache;

class NeuralRenderInfo : public torch::CustomClassHolder
{
   public:
    NeuralScene* scene = nullptr;
    std::vector<ReducedImageInfo> images;
    RenderParams params;
    int num_layers            = 1;
    bool train                = true;
    int current_epoch         = 0;
    void* timer_system        = nullptr;  // accepted for interface parity (CUDA::CudaTimerSystem* in the reference)
    PointRendererCache* cache = nullptr;
};

class PointRendererCache
{
   public:
    // (Re)allocates the workspace when the size key changes and draws the drop-out mask (PointRenderer.cu:285-309,516-521)
    void Build(NeuralRenderInfo* info, const TripsSplatDesc& desc, size_t workspace_bytes);

    torch::Tensor workspace;       // uint8
    torch::Tensor dropout_points;  // [batch, num_points] or undefined
    std::vector<int64_t> cache_size;
};

namespace torch::autograd
{
struct PointRender : public Function<PointRender>
{
    // returns a tensor for every layer
    static variable_list forward(AutogradContext* ctx, Variable texture, Variable background_color, Variable points,
                                 Variable pose_tangents, Variable intrinsics, Variable confidence,
                                 Variable dynamic_refinement, Variable layer_value_of_point, IValue info);
    static variable_list backward(AutogradContext* ctx, variable_list grad_output);
};
}  // namespace torch::autograd

// Render the scene into a batch of images; every image is a pyramid of layers in different resolutions
std::vector<torch::Tensor> BlendPointCloud(NeuralRenderInfo* info);

void ApplyTangentToPose(torch::Tensor tangent, torch::Tensor pose);

namespace torch::optim
{
struct MyAdamOptions : public OptimizerCloneableOptions<MyAdamOptions>
{
    MyAdamOptions(double lr = 1e-3) { set_lr(lr); }
    TORCH_ARG(double, lr) = 1e-3;
    typedef std::tuple<double, double> betas_t;
    TORCH_ARG(betas_t, betas)                    = std::make_tuple(0.9, 0.999);
    TORCH_ARG(double, eps)                       = 1e-8;
    TORCH_ARG(double, relative_weight_decay)     = 0;
    TORCH_ARG(double, absolute_weight_decay)     = 0;
    TORCH_ARG(double, weight_clipping_magnitude) = 0;
    TORCH_ARG(bool, adabound)                    = false;

   public:
    ~MyAdamOptions() override = default;
    double get_lr() const override { return lr(); }
    void set_lr(const double lr) override { this->lr(lr); }
};

struct MyAdamParamState : public OptimizerCloneableParamState<MyAdamParamState>
{
    TORCH_ARG(torch::Tensor, param_steps);
    TORCH_ARG(torch::Tensor, first_moments);
    TORCH_ARG(torch::Tensor, second_moments);
    TORCH_ARG(int64_t, current_step) = 0;

   public:
    ~MyAdamParamState() override = default;
};

class MyAdam : public Optimizer
{
   public:
    explicit MyAdam(std::vector<OptimizerParamGroup> param_groups, MyAdamOptions defaults = {});
    explicit MyAdam(std::vector<Tensor> params, MyAdamOptions defaults = {})
        : MyAdam({OptimizerParamGroup(std::move(params))}, defaults)
    {
    }
    torch::Tensor step(LossClosure closure = nullptr) override;
    virtual void shrinkInternalState(int param_group_index, torch::Tensor indices_to_keep);
    virtual void appendToInternalState(int param_group_index, int new_size);
    // The state of every parameter (moments, per-element step counters, step count) under "<index in group order>/...";
    // the reference leaves both unimplemented (MyAdam.cu:417-425). A checkpoint resumes bit for bit.
    void save(serialize::OutputArchive& archive) const override;
    void load(serialize::InputArchive& archive) override;

   protected:
    // one parameter's step description for the library (creates its state on first use unless `packed`)
    bool describe(Tensor& p, OptimizerParamGroup& group, bool packed, TripsAdamTensor& t, std::vector<Tensor>& keep);
};

// MyAdam whose state for the four parameter tensors of a point cloud (t_position [N,4], t_point_size [N,1],
// texture [C,N], confidence_value_of_point [1,N]; NeuralPointCloudCuda.cpp:103-108, NeuralTexture.cpp:53-55) is one
// row per point of {first moment, second moment, step counter} of the point's elements. The four must be among the
// parameters of the groups (each group's options apply as usual); every other parameter is stepped as MyAdam steps
// it. Same arithmetic per element, bit-identical results; a point whose gradients are all zero is skipped without its
// state being read. Point removal / addition: the rows follow the group that holds `texture`.
class MyAdamPoints : public MyAdam
{
   public:
    MyAdamPoints(std::vector<OptimizerParamGroup> param_groups, Tensor position, Tensor point_size, Tensor texture,
                 Tensor confidence, MyAdamOptions defaults = {});
    torch::Tensor step(LossClosure closure = nullptr) override;
    void shrinkInternalState(int param_group_index, torch::Tensor indices_to_keep) override;
    void appendToInternalState(int param_group_index, int new_size) override;
    // the per-tensor state of the other parameters as MyAdam saves it, plus the rows and the step counts of the four
    void save(serialize::OutputArchive& archive) const override;
    void load(serialize::InputArchive& archive) override;
    torch::Tensor packed_state;  // [N, row bytes / 4] int32, defined after the first step

   private:
    int slot_of(const Tensor& p) const;
    Tensor packed_[4];
    Tensor zero_grads_[4];
    int64_t packed_steps_[4] = {0, 0, 0, 0};
};
}  // namespace torch::optim

// The library context of a device, shared by every thread of the process (forward runs on the caller's thread, backward
// on the autograd engine's): created on first use, destroyed when the shim is unloaded. trips_profile_enable on it
// therefore covers forward and backward kernels alike.
TripsCtx* trips_shim_context(int device);
