// pybind11 entry points that drive the C++ operator surface from Python tests.
#include <torch/extension.h>

#include "trips_torch.h"

namespace
{
struct Session
{
    NeuralScene scene;
    PointRendererCache cache;
    std::unique_ptr<torch::optim::MyAdam> optimizer;
};

std::vector<torch::Tensor> blend_point_cloud(Session& s, std::vector<std::vector<double>> views, int num_layers, bool train,
                                             double dropout, int background_mode, int list_depth)
{
    NeuralRenderInfo info;
    info.scene      = &s.scene;
    info.num_layers = num_layers;
    info.train      = train;
    info.cache      = &s.cache;
    info.params.dropout                   = (float)dropout;
    info.params.drop_out_points_by_radius = false;
    info.params.background_mode           = background_mode;
    info.params.max_pixels_per_list       = list_depth;
    info.params.num_texture_channels      = (int)s.scene.texture->texture.size(0);
    for (auto& v : views)
    {
        // w h image_index camera_index [crop fx fy cx cy s] [rot r00 r01 r10 r11]
        ReducedImageInfo im;
        im.w            = (int)v.at(0);
        im.h            = (int)v.at(1);
        im.image_index  = (int)v.at(2);
        im.camera_index = (int)v.at(3);
        if (v.size() >= 9)
            for (int k = 0; k < 5; ++k) im.crop_transform[k] = (float)v[4 + k];
        if (v.size() >= 13)
            for (int k = 0; k < 4; ++k) im.crop_rotation[k] = (float)v[9 + k];
        info.images.push_back(im);
    }
    return BlendPointCloud(&info);
}
}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    py::class_<Session>(m, "Session")
        .def(py::init<>())
        .def("set_scene",
             [](Session& s, torch::Tensor texture, torch::Tensor background, torch::Tensor confidence, torch::Tensor position,
                torch::Tensor point_size, torch::Tensor index, torch::Tensor poses_se3, torch::Tensor tangent_poses,
                torch::Tensor intrinsics)
             {
                 s.scene.texture->texture                   = texture;
                 s.scene.texture->background_color          = background;
                 s.scene.texture->confidence_value_of_point = confidence;
                 s.scene.point_cloud_cuda->t_position       = position;
                 s.scene.point_cloud_cuda->t_point_size     = point_size;
                 s.scene.point_cloud_cuda->t_index          = index;
                 s.scene.poses->poses_se3                   = poses_se3;
                 s.scene.poses->tangent_poses               = tangent_poses;
                 s.scene.intrinsics->intrinsics             = intrinsics;
             })
        .def("blend_point_cloud", &blend_point_cloud, py::arg("views"), py::arg("num_layers"), py::arg("train") = true,
             py::arg("dropout") = 0.0, py::arg("background_mode") = 0, py::arg("list_depth") = 16)
        .def("apply_tangent", [](Session& s) { s.scene.poses->ApplyTangent(); })
        .def("make_adam",
             [](Session& s, std::vector<torch::Tensor> params, double lr)
             { s.optimizer = std::make_unique<torch::optim::MyAdam>(params, torch::optim::MyAdamOptions(lr)); })
        .def("adam_step", [](Session& s) { s.optimizer->step(); });
}
