// On-disk formats of a TRIPS scene, so that real scenes and checkpoints can be loaded into the operator:
//   * checkpoint archives  scene_<name>_{points,texture,poses,intrinsics}.pth written by NeuralScene::SaveCheckpoint
//     (src/lib/data/NeuralScene.cpp:602-628 of the reference) = torch::save of modules whose registered names are
//       NeuralPointCloudCuda  t_position (param), t_index, t_original_color (buffers), t_point_size (param)
//                             (src/lib/rendering/NeuralPointCloudCuda.cpp:103-108)
//       NeuralTexture         texture, background_color, confidence_value_of_point (params, the raw values)
//                             (src/lib/models/NeuralTexture.cpp:53-55)
//       PoseModule            tangent_poses (param), poses_se3 (buffer)   (src/lib/data/NeuralStructure.cpp:34-35)
//       IntrinsicsModule      intrinsics (param)                            (NeuralStructure.cpp:142)
//     and poses.txt beside them (SceneData::SavePoses, src/lib/data/SceneData.cpp:458-469)
//   * the ADOP scene directory (scenes/README.md:65-101): dataset.ini, camera ini files, poses.txt, images.txt,
//     camera_indices.txt, point_cloud.ply
// Host code only (libtorch + the C++ standard library).
#pragma once
#include <torch/torch.h>

#include <array>
#include <string>
#include <vector>

class NeuralPointCloudCudaModuleImpl : public torch::nn::Module
{
   public:
    // position [N,4] f32 (xyz + drop-out radius), point_size [N,1] f32 (raw), index [N,1] i32, original_color [N,4] f32
    NeuralPointCloudCudaModuleImpl(torch::Tensor position, torch::Tensor point_size, torch::Tensor index,
                                   torch::Tensor original_color, bool use_pointsize = true);
    int Size() const { return (int)t_position.size(0); }
    torch::Tensor t_position, t_point_size, t_index, t_original_color;
};
TORCH_MODULE(NeuralPointCloudCudaModule);

class NeuralTextureModuleImpl : public torch::nn::Module
{
   public:
    NeuralTextureModuleImpl(torch::Tensor texture_raw, torch::Tensor background_color_raw, torch::Tensor confidence_raw);
    // src/lib/models/NeuralTexture.h:40-57
    void PrepareConfidence(float narrowing_param_times_epoch);
    void PrepareTexture(bool abs);
    torch::Tensor texture_raw, background_color_raw, confidence_raw;  // what the archive holds
    torch::Tensor texture, background_color, confidence_value_of_point;  // what the operator reads
};
TORCH_MODULE(NeuralTextureModule);

class PoseModuleImpl : public torch::nn::Module
{
   public:
    // poses_se3 [F,8] f64: world -> camera, quaternion xyzw, translation, padding
    explicit PoseModuleImpl(torch::Tensor poses_se3);
    torch::Tensor poses_se3, tangent_poses;
};
TORCH_MODULE(PoseModule);

class IntrinsicsModuleImpl : public torch::nn::Module
{
   public:
    explicit IntrinsicsModuleImpl(torch::Tensor intrinsics);  // [Cam,13] f32: fx fy cx cy s + 8 distortion
    torch::Tensor intrinsics;
};
TORCH_MODULE(IntrinsicsModule);

struct SceneModules
{
    NeuralPointCloudCudaModule point_cloud_cuda = nullptr;
    NeuralTextureModule texture                 = nullptr;
    PoseModule poses                            = nullptr;
    IntrinsicsModule intrinsics                 = nullptr;
};

// checkpoint_dir/scene_<scene_name>_{texture,points,poses,intrinsics}.pth and ..._poses.txt; `reduced` skips the two
// large archives, as in the reference
void SaveCheckpoint(const SceneModules& scene, const std::string& checkpoint_dir, const std::string& scene_name, bool reduced = false);
// loads whichever of the four archives exist into the (already constructed, same-shaped) modules; returns their count
int LoadCheckpoint(SceneModules& scene, const std::string& checkpoint_dir, const std::string& scene_name);

// ---- ADOP scene directory ----
struct SceneCameraParams  // camera ini file, section [SceneCameraParams] (src/lib/data/SceneData.cpp:1298-1340)
{
    int w = 0, h = 0;
    std::array<float, 5> K{};           // fx fy cx cy s
    std::array<float, 8> distortion{};  // 8-parameter model
};

struct SceneData
{
    std::string scene_path, scene_name;
    std::vector<SceneCameraParams> scene_cameras;
    std::vector<std::array<double, 7>> poses;  // camera -> world: qx qy qz qw tx ty tz (poses.txt)
    std::vector<std::string> image_names;      // images.txt
    std::vector<int> camera_indices;           // camera_indices.txt
    torch::Tensor point_position;              // [N,3] f32 (point_cloud.ply)
    torch::Tensor point_normal;                // [N,3] f32 or undefined
    torch::Tensor point_color;                 // [N,4] f32 in 0..1, white when the file has none
};

SceneCameraParams LoadSceneCameraParams(const std::string& ini_file);
void SaveSceneCameraParams(const SceneCameraParams& cam, const std::string& ini_file);
std::vector<std::array<double, 7>> LoadPoses(const std::string& file);
void SavePoses(const std::vector<std::array<double, 7>>& poses, const std::string& file);
// ascii and binary_little_endian PLY with float/double x y z, optional nx ny nz, optional uchar/float red green blue [alpha]
void LoadPly(const std::string& file, torch::Tensor& position, torch::Tensor& normal, torch::Tensor& color);
SceneData LoadScene(const std::string& scene_dir);

// world -> camera rows of PoseModule from the camera -> world poses of poses.txt (NeuralStructure.cpp:20-35)
torch::Tensor PosesToSe3(const std::vector<std::array<double, 7>>& camera_to_world);
// [Cam,13] intrinsics tensor (NeuralStructure.cpp:104-142)
torch::Tensor CamerasToIntrinsics(const std::vector<SceneCameraParams>& cams);
