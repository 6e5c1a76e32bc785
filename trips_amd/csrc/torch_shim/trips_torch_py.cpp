// pybind11 entry points that drive the C++ operator surface from Python tests.
#include <torch/extension.h>

#include "trips_scene_io.h"
#include "trips_torch.h"
#include "trips_unet_torch.h"

namespace
{
struct Session
{
    NeuralScene scene;
    PointRendererCache cache;
    std::unique_ptr<torch::optim::MyAdam> optimizer;
};

std::vector<torch::Tensor> blend_point_cloud(Session& s, std::vector<std::vector<double>> views, int num_layers, bool train,
                                             double dropout, int background_mode, int list_depth, bool add_depth,
                                             bool background_mask)
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
    info.params.add_depth_to_network      = add_depth;
    info.params.output_background_mask    = background_mask;
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

namespace
{
struct UnetSession
{
    MultiScaleUnet2dDecOnlySmallFixed net = nullptr;
    UnetSession(std::vector<int> filters, int num_layers, int num_input_layers, int num_input_channels)
    {
        MultiScaleUnet2dParams p;
        p.filters_network    = filters;
        p.num_layers         = num_layers;
        p.num_input_layers   = num_input_layers;
        p.num_input_channels = num_input_channels;
        net                  = MultiScaleUnet2dDecOnlySmallFixed(p);
    }
    std::vector<std::pair<std::string, torch::Tensor>> named_parameters()
    {
        std::vector<std::pair<std::string, torch::Tensor>> out;
        for (auto& kv : net->named_parameters()) out.emplace_back(kv.key(), kv.value());
        return out;
    }
};

SceneModules make_modules(torch::Tensor position, torch::Tensor point_size, torch::Tensor index, torch::Tensor color,
                          torch::Tensor texture, torch::Tensor background, torch::Tensor confidence, torch::Tensor poses_se3,
                          torch::Tensor intrinsics)
{
    SceneModules s;
    s.point_cloud_cuda = NeuralPointCloudCudaModule(position, point_size, index, color);
    s.texture          = NeuralTextureModule(texture, background, confidence);
    s.poses            = PoseModule(poses_se3);
    s.intrinsics       = IntrinsicsModule(intrinsics);
    return s;
}

py::dict modules_to_dict(const SceneModules& s)
{
    py::dict d;
    auto put = [&](const char* prefix, const torch::nn::Module& m)
    {
        for (auto& kv : m.named_parameters()) d[py::str(std::string(prefix) + "." + kv.key())] = kv.value();
        for (auto& kv : m.named_buffers()) d[py::str(std::string(prefix) + "." + kv.key())] = kv.value();
    };
    put("points", *s.point_cloud_cuda);
    put("texture", *s.texture);
    put("poses", *s.poses);
    put("intrinsics", *s.intrinsics);
    d["texture.prepared_confidence"] = s.texture->confidence_value_of_point;
    return d;
}
}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    py::class_<UnetSession>(m, "UnetSession")
        .def(py::init<std::vector<int>, int, int, int>(), py::arg("filters"), py::arg("num_layers"), py::arg("num_input_layers"),
             py::arg("num_input_channels") = 4)
        .def("named_parameters", &UnetSession::named_parameters)
        .def("cuda", [](UnetSession& s) { s.net->to(torch::kCUDA); })
        .def("forward", [](UnetSession& s, std::vector<torch::Tensor> inputs) { return s.net->forward(inputs); })
        .def("forward_no_grad",
             [](UnetSession& s, std::vector<torch::Tensor> inputs)
             {
                 torch::NoGradGuard guard;
                 return s.net->forward(inputs);
             })
        .def("set_reuse_packed_weights", [](UnetSession& s, bool on) { s.net->reuse_packed_weights = on; })
        .def("invalidate_packed_weights", [](UnetSession& s) { s.net->invalidate_packed_weights(); })
        .def("save", [](UnetSession& s, const std::string& file) { torch::save(s.net, file); })
        .def("load", [](UnetSession& s, const std::string& file) { torch::load(s.net, file); });

    m.def("save_checkpoint",
          [](const std::string& dir, const std::string& name, torch::Tensor position, torch::Tensor point_size, torch::Tensor index,
             torch::Tensor color, torch::Tensor texture, torch::Tensor background, torch::Tensor confidence, torch::Tensor poses_se3,
             torch::Tensor intrinsics, bool reduced)
          { SaveCheckpoint(make_modules(position, point_size, index, color, texture, background, confidence, poses_se3, intrinsics), dir, name, reduced); });
    m.def("load_checkpoint",
          [](const std::string& dir, const std::string& name, int64_t num_points, int64_t channels, int64_t frames, int64_t cameras)
          {
              // modules of the right shapes, as a TRIPS build has after constructing the scene; the archives overwrite them
              auto f32 = torch::kFloat32;
              SceneModules s = make_modules(torch::zeros({num_points, 4}, f32), torch::zeros({num_points, 1}, f32),
                                            torch::zeros({num_points, 1}, torch::kInt32), torch::zeros({num_points, 4}, f32),
                                            torch::zeros({channels, num_points}, f32), torch::zeros({channels}, f32),
                                            torch::zeros({1, num_points}, f32), torch::zeros({frames, 8}, torch::kFloat64),
                                            torch::zeros({cameras, 13}, f32));
              const int n = LoadCheckpoint(s, dir, name);
              py::dict d  = modules_to_dict(s);
              d["archives_loaded"] = n;
              return d;
          });
    m.def("load_scene",
          [](const std::string& dir)
          {
              SceneData s = LoadScene(dir);
              py::dict d;
              d["scene_name"]     = s.scene_name;
              d["image_names"]    = s.image_names;
              d["camera_indices"] = s.camera_indices;
              d["poses_se3"]      = PosesToSe3(s.poses);
              d["intrinsics"]     = CamerasToIntrinsics(s.scene_cameras);
              std::vector<std::pair<int, int>> sizes;
              for (auto& c : s.scene_cameras) sizes.emplace_back(c.w, c.h);
              d["camera_sizes"] = sizes;
              if (s.point_position.defined()) d["point_position"] = s.point_position;
              if (s.point_normal.defined()) d["point_normal"] = s.point_normal;
              if (s.point_color.defined()) d["point_color"] = s.point_color;
              return d;
          });
    m.def("save_camera",
          [](const std::string& file, int w, int h, std::vector<float> K, std::vector<float> distortion)
          {
              SceneCameraParams c;
              c.w = w, c.h = h;
              for (size_t i = 0; i < 5; ++i) c.K[i] = K.at(i);
              for (size_t i = 0; i < 8; ++i) c.distortion[i] = distortion.at(i);
              SaveSceneCameraParams(c, file);
          });
    m.def("save_poses",
          [](const std::string& file, std::vector<std::array<double, 7>> poses) { SavePoses(poses, file); });
    m.def("load_poses", [](const std::string& file) { return LoadPoses(file); });

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
        .def("set_dynamic_refinement", [](Session& s, torch::Tensor t) { s.scene.dynamic_refinement_t = t; })
        .def("blend_point_cloud", &blend_point_cloud, py::arg("views"), py::arg("num_layers"), py::arg("train") = true,
             py::arg("dropout") = 0.0, py::arg("background_mode") = 0, py::arg("list_depth") = 16,
             py::arg("add_depth_to_network") = false, py::arg("output_background_mask") = false)
        .def("apply_tangent", [](Session& s) { s.scene.poses->ApplyTangent(); })
        .def("make_adam",
             [](Session& s, std::vector<torch::Tensor> params, double lr)
             { s.optimizer = std::make_unique<torch::optim::MyAdam>(params, torch::optim::MyAdamOptions(lr)); })
        .def("make_adam_points",
             [](Session& s, std::vector<torch::Tensor> others, double lr)
             {
                 // one group per point tensor (descriptors with twice the learning rate), one for the rest
                 auto& pc = *s.scene.point_cloud_cuda;
                 auto& tx = *s.scene.texture;
                 std::vector<torch::optim::OptimizerParamGroup> groups;
                 groups.emplace_back(std::vector<torch::Tensor>{pc.t_position});
                 groups.emplace_back(std::vector<torch::Tensor>{pc.t_point_size});
                 groups.emplace_back(std::vector<torch::Tensor>{tx.texture}, std::make_unique<torch::optim::MyAdamOptions>(2 * lr));
                 groups.emplace_back(std::vector<torch::Tensor>{tx.confidence_value_of_point});
                 if (!others.empty()) groups.emplace_back(others);
                 s.optimizer = std::make_unique<torch::optim::MyAdamPoints>(groups, pc.t_position, pc.t_point_size, tx.texture,
                                                                            tx.confidence_value_of_point,
                                                                            torch::optim::MyAdamOptions(lr));
             })
        .def("adam_step", [](Session& s) { s.optimizer->step(); })
        .def("adam_save",
             [](Session& s, const std::string& path)
             {
                 torch::serialize::OutputArchive archive;
                 s.optimizer->save(archive);
                 archive.save_to(path);
             })
        .def("adam_load",
             [](Session& s, const std::string& path)
             {
                 torch::serialize::InputArchive archive;
                 archive.load_from(path);
                 s.optimizer->load(archive);
             });
}
