// Implementation of trips_scene_io.h. Host code only.
#include "trips_scene_io.h"

#include <cstdint>
#include <cstring>
#include <filesystem>
#include <fstream>
#include <iomanip>
#include <map>
#include <sstream>

namespace fs = std::filesystem;

NeuralPointCloudCudaModuleImpl::NeuralPointCloudCudaModuleImpl(torch::Tensor position, torch::Tensor point_size, torch::Tensor index,
                                                               torch::Tensor original_color, bool use_pointsize)
{
    TORCH_CHECK(position.dim() == 2 && position.size(1) == 4, "t_position must be [N,4]");
    t_position       = register_parameter("t_position", position.contiguous());
    t_index          = register_buffer("t_index", index.contiguous());
    t_original_color = register_buffer("t_original_color", original_color.contiguous());
    if (use_pointsize)
        t_point_size = register_parameter("t_point_size", point_size.contiguous());
    else
        t_point_size = point_size.contiguous();
}

NeuralTextureModuleImpl::NeuralTextureModuleImpl(torch::Tensor tex, torch::Tensor bg, torch::Tensor conf)
{
    texture_raw          = register_parameter("texture", tex.contiguous());
    background_color_raw = register_parameter("background_color", bg.contiguous());
    confidence_raw       = register_parameter("confidence_value_of_point", conf.contiguous());
    PrepareConfidence(0.f);
    PrepareTexture(false);
}

void NeuralTextureModuleImpl::PrepareConfidence(float narrowing_param_times_epoch)
{
    confidence_value_of_point = torch::sigmoid((10.f + narrowing_param_times_epoch) * confidence_raw);
}

void NeuralTextureModuleImpl::PrepareTexture(bool abs)
{
    texture          = abs ? torch::abs(texture_raw) : texture_raw;
    background_color = abs ? torch::abs(background_color_raw) : background_color_raw;
}

PoseModuleImpl::PoseModuleImpl(torch::Tensor se3)
{
    TORCH_CHECK(se3.dim() == 2 && se3.size(1) == 8 && se3.scalar_type() == torch::kFloat64, "poses_se3 must be [F,8] float64");
    tangent_poses = register_parameter("tangent_poses", torch::zeros({se3.size(0), 6}, se3.options()));
    poses_se3     = register_buffer("poses_se3", se3.contiguous());
}

IntrinsicsModuleImpl::IntrinsicsModuleImpl(torch::Tensor k)
{
    TORCH_CHECK(k.dim() == 2 && k.size(1) == 13, "intrinsics must be [Cam,13]");
    intrinsics = register_parameter("intrinsics", k.contiguous());
}

static std::vector<std::array<double, 7>> download_camera_to_world(const torch::Tensor& poses_se3)
{
    // inverse of a unit-quaternion pose: q^-1 = conj(q), t^-1 = -(q^-1 t)
    torch::Tensor p = poses_se3.detach().to(torch::kCPU).contiguous();
    auto a          = p.accessor<double, 2>();
    std::vector<std::array<double, 7>> out((size_t)p.size(0));
    for (int64_t i = 0; i < p.size(0); ++i)
    {
        const double x = -a[i][0], y = -a[i][1], z = -a[i][2], w = a[i][3];
        const double tx = a[i][4], ty = a[i][5], tz = a[i][6];
        // rotate t by the conjugate quaternion: v + 2 w (u x v) + 2 u x (u x v), u = (x, y, z)
        const double cx = y * tz - z * ty, cy = z * tx - x * tz, cz = x * ty - y * tx;
        const double rx = tx + 2 * (w * cx + (y * cz - z * cy));
        const double ry = ty + 2 * (w * cy + (z * cx - x * cz));
        const double rz = tz + 2 * (w * cz + (x * cy - y * cx));
        out[(size_t)i] = {x, y, z, w, -rx, -ry, -rz};
    }
    return out;
}

void SaveCheckpoint(const SceneModules& scene, const std::string& dir, const std::string& scene_name, bool reduced)
{
    const std::string prefix = dir + "/scene_" + scene_name + "_";
    if (!reduced)
    {
        if (scene.texture) torch::save(scene.texture, prefix + "texture.pth");
        if (scene.point_cloud_cuda) torch::save(scene.point_cloud_cuda, prefix + "points.pth");
    }
    if (scene.poses)
    {
        torch::save(scene.poses, prefix + "poses.pth");
        SavePoses(download_camera_to_world(scene.poses->poses_se3), prefix + "poses.txt");
    }
    if (scene.intrinsics) torch::save(scene.intrinsics, prefix + "intrinsics.pth");
}

int LoadCheckpoint(SceneModules& scene, const std::string& dir, const std::string& scene_name)
{
    const std::string prefix = dir + "/scene_" + scene_name + "_";
    int n = 0;
    if (scene.point_cloud_cuda && fs::exists(prefix + "points.pth")) torch::load(scene.point_cloud_cuda, prefix + "points.pth"), ++n;
    if (scene.texture && fs::exists(prefix + "texture.pth"))
    {
        torch::load(scene.texture, prefix + "texture.pth");
        scene.texture->PrepareConfidence(0.f);
        scene.texture->PrepareTexture(false);
        ++n;
    }
    if (scene.poses && fs::exists(prefix + "poses.pth")) torch::load(scene.poses, prefix + "poses.pth"), ++n;
    if (scene.intrinsics && fs::exists(prefix + "intrinsics.pth")) torch::load(scene.intrinsics, prefix + "intrinsics.pth"), ++n;
    return n;
}

// ---- ini (section headers, key = value, '#' comments) ----
static std::map<std::string, std::string> read_ini(const std::string& file)
{
    std::ifstream in(file);
    TORCH_CHECK(in.good(), "cannot open ", file);
    std::map<std::string, std::string> kv;
    std::string line;
    while (std::getline(in, line))
    {
        const size_t hash = line.find('#');
        if (hash != std::string::npos) line = line.substr(0, hash);
        const size_t eq = line.find('=');
        if (eq == std::string::npos) continue;
        auto trim = [](std::string s)
        {
            const char* ws = " \t\r\n";
            const size_t a = s.find_first_not_of(ws);
            if (a == std::string::npos) return std::string();
            return s.substr(a, s.find_last_not_of(ws) - a + 1);
        };
        kv[trim(line.substr(0, eq))] = trim(line.substr(eq + 1));
    }
    return kv;
}

template <size_t N>
static std::array<float, N> parse_floats(const std::string& s, const char* what)
{
    std::array<float, N> out{};
    std::stringstream ss(s);
    for (size_t i = 0; i < N; ++i)
    {
        double d;
        TORCH_CHECK(bool(ss >> d), what, ": expected ", N, " numbers, got '", s, "'");
        out[i] = (float)d;
    }
    return out;
}

SceneCameraParams LoadSceneCameraParams(const std::string& ini_file)
{
    auto kv = read_ini(ini_file);
    SceneCameraParams c;
    TORCH_CHECK(kv.count("w") && kv.count("h") && kv.count("K"), ini_file, ": w, h and K are required");
    c.w = std::stoi(kv["w"]);
    c.h = std::stoi(kv["h"]);
    c.K = parse_floats<5>(kv["K"], "K");
    if (kv.count("distortion")) c.distortion = parse_floats<8>(kv["distortion"], "distortion");
    return c;
}

void SaveSceneCameraParams(const SceneCameraParams& c, const std::string& ini_file)
{
    std::ofstream out(ini_file);
    TORCH_CHECK(out.good(), "cannot write ", ini_file);
    out << "[SceneCameraParams]\n" << "w = " << c.w << "\n" << "h = " << c.h << "\n";
    out << std::setprecision(15) << std::scientific;
    out << "# fx fy cx cy s\nK = ";
    for (size_t i = 0; i < 5; ++i) out << double(c.K[i]) << (i < 4 ? " " : "\n");
    out << "# 8 paramter distortion model. see distortion.h\ndistortion = ";
    for (size_t i = 0; i < 8; ++i) out << double(c.distortion[i]) << (i < 7 ? " " : "\n");
}

std::vector<std::array<double, 7>> LoadPoses(const std::string& file)
{
    std::ifstream in(file);
    TORCH_CHECK(in.good(), "cannot open ", file);
    std::vector<std::array<double, 7>> poses;
    std::string line;
    while (std::getline(in, line))
    {
        std::stringstream ss(line);
        std::array<double, 7> p{};
        int k = 0;
        while (k < 7 && (ss >> p[(size_t)k])) ++k;
        if (k == 0) continue;
        TORCH_CHECK(k == 7, file, ": a pose line needs qx qy qz qw tx ty tz");
        poses.push_back(p);
    }
    return poses;
}

void SavePoses(const std::vector<std::array<double, 7>>& poses, const std::string& file)
{
    std::ofstream out(file);
    TORCH_CHECK(out.good(), "cannot write ", file);
    out << std::scientific << std::setprecision(15);
    for (auto& p : poses) out << p[0] << " " << p[1] << " " << p[2] << " " << p[3] << " " << p[4] << " " << p[5] << " " << p[6] << "\n";
}

static std::vector<std::string> read_lines(const std::string& file)
{
    std::vector<std::string> out;
    std::ifstream in(file);
    std::string line;
    while (std::getline(in, line))
    {
        while (!line.empty() && (line.back() == '\r' || line.back() == ' ')) line.pop_back();
        if (!line.empty()) out.push_back(line);
    }
    return out;
}

void LoadPly(const std::string& file, torch::Tensor& position, torch::Tensor& normal, torch::Tensor& color)
{
    std::ifstream in(file, std::ios::binary);
    TORCH_CHECK(in.good(), "cannot open ", file);
    std::string line;
    std::getline(in, line);
    TORCH_CHECK(line.rfind("ply", 0) == 0, file, ": not a PLY file");
    struct Prop
    {
        std::string type, name;
    };
    std::vector<Prop> props;
    bool binary = false, in_vertex = false;
    int64_t n = -1;
    while (std::getline(in, line))
    {
        while (!line.empty() && line.back() == '\r') line.pop_back();
        std::stringstream ss(line);
        std::string tok;
        ss >> tok;
        if (tok == "format")
        {
            std::string f;
            ss >> f;
            TORCH_CHECK(f == "ascii" || f == "binary_little_endian", file, ": PLY format ", f, " is not supported");
            binary = f == "binary_little_endian";
        }
        else if (tok == "element")
        {
            std::string name;
            int64_t count;
            ss >> name >> count;
            in_vertex = name == "vertex";
            if (in_vertex) n = count;
        }
        else if (tok == "property" && in_vertex)
        {
            Prop p;
            ss >> p.type >> p.name;
            TORCH_CHECK(p.type != "list", file, ": list properties on vertices are not supported");
            props.push_back(p);
        }
        else if (tok == "end_header")
            break;
    }
    TORCH_CHECK(n >= 0, file, ": no vertex element");
    auto size_of = [&](const std::string& t) -> int
    {
        if (t == "float" || t == "float32" || t == "int" || t == "int32" || t == "uint" || t == "uint32") return 4;
        if (t == "double" || t == "float64") return 8;
        if (t == "uchar" || t == "uint8" || t == "char" || t == "int8") return 1;
        if (t == "short" || t == "int16" || t == "ushort" || t == "uint16") return 2;
        TORCH_CHECK(false, file, ": PLY type ", t);
        return 0;
    };
    auto find = [&](const std::string& name)
    {
        for (size_t i = 0; i < props.size(); ++i)
            if (props[i].name == name) return (int)i;
        return -1;
    };
    const int ix = find("x"), iy = find("y"), iz = find("z");
    TORCH_CHECK(ix >= 0 && iy >= 0 && iz >= 0, file, ": x y z are required");
    const int inx = find("nx"), iny = find("ny"), inz = find("nz");
    const int ir = find("red"), ig = find("green"), ib = find("blue"), ia = find("alpha");
    const bool has_n = inx >= 0 && iny >= 0 && inz >= 0, has_c = ir >= 0 && ig >= 0 && ib >= 0;
    position = torch::empty({n, 3}, torch::kFloat32);
    if (has_n) normal = torch::empty({n, 3}, torch::kFloat32);
    color    = torch::ones({n, 4}, torch::kFloat32);
    float* P = position.data_ptr<float>();
    float* Nn = has_n ? normal.data_ptr<float>() : nullptr;
    float* Cc = color.data_ptr<float>();
    std::vector<double> v(props.size());
    std::vector<char> row;
    int stride = 0;
    for (auto& p : props) stride += size_of(p.type);
    row.resize((size_t)stride);
    for (int64_t i = 0; i < n; ++i)
    {
        if (binary)
        {
            in.read(row.data(), stride);
            TORCH_CHECK(in.gcount() == stride, file, ": truncated vertex data");
            int off = 0;
            for (size_t k = 0; k < props.size(); ++k)
            {
                const std::string& t = props[k].type;
                const char* src      = row.data() + off;
                if (t == "float" || t == "float32") { float f; std::memcpy(&f, src, 4); v[k] = f; }
                else if (t == "double" || t == "float64") { double d; std::memcpy(&d, src, 8); v[k] = d; }
                else if (t == "uchar" || t == "uint8") v[k] = (unsigned char)src[0];
                else if (t == "char" || t == "int8") v[k] = (signed char)src[0];
                else if (t == "short" || t == "int16") { int16_t s; std::memcpy(&s, src, 2); v[k] = s; }
                else if (t == "ushort" || t == "uint16") { uint16_t s; std::memcpy(&s, src, 2); v[k] = s; }
                else if (t == "int" || t == "int32") { int32_t s; std::memcpy(&s, src, 4); v[k] = s; }
                else { uint32_t s; std::memcpy(&s, src, 4); v[k] = s; }
                off += size_of(t);
            }
        }
        else
        {
            for (size_t k = 0; k < props.size(); ++k) TORCH_CHECK(bool(in >> v[k]), file, ": truncated vertex data");
        }
        P[3 * i] = (float)v[(size_t)ix], P[3 * i + 1] = (float)v[(size_t)iy], P[3 * i + 2] = (float)v[(size_t)iz];
        if (has_n) Nn[3 * i] = (float)v[(size_t)inx], Nn[3 * i + 1] = (float)v[(size_t)iny], Nn[3 * i + 2] = (float)v[(size_t)inz];
        if (has_c)
        {
            const bool bytes = size_of(props[(size_t)ir].type) == 1;
            const double s   = bytes ? 1.0 / 255.0 : 1.0;
            Cc[4 * i] = (float)(v[(size_t)ir] * s), Cc[4 * i + 1] = (float)(v[(size_t)ig] * s), Cc[4 * i + 2] = (float)(v[(size_t)ib] * s);
            if (ia >= 0) Cc[4 * i + 3] = (float)(v[(size_t)ia] * s);
        }
    }
}

SceneData LoadScene(const std::string& scene_dir)
{
    SceneData s;
    s.scene_path = fs::canonical(scene_dir).string();
    s.scene_name = fs::path(s.scene_path).filename().string();
    TORCH_CHECK(!s.scene_name.empty(), "empty scene name");
    std::vector<std::string> camera_files = {"camera.ini"};
    std::string file_point_cloud          = "point_cloud.ply";
    const std::string dataset_ini         = s.scene_path + "/dataset.ini";
    TORCH_CHECK(fs::exists(dataset_ini), dataset_ini, " is required");
    {
        auto kv = read_ini(dataset_ini);
        if (kv.count("camera_files"))
        {
            camera_files.clear();
            std::stringstream ss(kv["camera_files"]);
            std::string f;
            while (ss >> f) camera_files.push_back(f);
        }
        if (kv.count("file_point_cloud")) file_point_cloud = kv["file_point_cloud"];
    }
    for (auto& f : camera_files) s.scene_cameras.push_back(LoadSceneCameraParams(s.scene_path + "/" + f));
    TORCH_CHECK(!s.scene_cameras.empty(), "no camera files");
    s.poses          = LoadPoses(s.scene_path + "/poses.txt");
    s.image_names    = read_lines(s.scene_path + "/images.txt");
    for (auto& l : read_lines(s.scene_path + "/camera_indices.txt")) s.camera_indices.push_back(std::stoi(l));
    TORCH_CHECK(s.poses.size() == s.image_names.size() && s.poses.size() == s.camera_indices.size(),
                "poses.txt, images.txt and camera_indices.txt must have one line per image");
    for (int c : s.camera_indices) TORCH_CHECK(c >= 0 && c < (int)s.scene_cameras.size(), "camera index ", c, " out of range");
    if (fs::exists(s.scene_path + "/" + file_point_cloud))
        LoadPly(s.scene_path + "/" + file_point_cloud, s.point_position, s.point_normal, s.point_color);
    return s;
}

torch::Tensor PosesToSe3(const std::vector<std::array<double, 7>>& c2w)
{
    torch::Tensor t = torch::zeros({(int64_t)c2w.size(), 8}, torch::kFloat64);
    auto a          = t.accessor<double, 2>();
    for (size_t i = 0; i < c2w.size(); ++i)
    {
        double x = c2w[i][0], y = c2w[i][1], z = c2w[i][2], w = c2w[i][3];
        const double nrm = std::sqrt(x * x + y * y + z * z + w * w);
        x /= nrm, y /= nrm, z /= nrm, w /= nrm;
        const double ux = -x, uy = -y, uz = -z;  // conjugate
        const double tx = c2w[i][4], ty = c2w[i][5], tz = c2w[i][6];
        const double cx = uy * tz - uz * ty, cy = uz * tx - ux * tz, cz = ux * ty - uy * tx;
        const double rx = tx + 2 * (w * cx + (uy * cz - uz * cy));
        const double ry = ty + 2 * (w * cy + (uz * cx - ux * cz));
        const double rz = tz + 2 * (w * cz + (ux * cy - uy * cx));
        a[(int64_t)i][0] = ux, a[(int64_t)i][1] = uy, a[(int64_t)i][2] = uz, a[(int64_t)i][3] = w;
        a[(int64_t)i][4] = -rx, a[(int64_t)i][5] = -ry, a[(int64_t)i][6] = -rz;
    }
    return t;
}

torch::Tensor CamerasToIntrinsics(const std::vector<SceneCameraParams>& cams)
{
    torch::Tensor t = torch::zeros({(int64_t)cams.size(), 13}, torch::kFloat32);
    auto a          = t.accessor<float, 2>();
    for (size_t i = 0; i < cams.size(); ++i)
    {
        for (int k = 0; k < 5; ++k) a[(int64_t)i][k] = cams[i].K[(size_t)k];
        for (int k = 0; k < 8; ++k) a[(int64_t)i][5 + k] = cams[i].distortion[(size_t)k];
    }
    return t;
}
