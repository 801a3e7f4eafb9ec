// bindings.cpp — pybind11 front end of the libTorch wrapper, used by the tests to drive PointRender /
// PointRenderModuleForward exactly as the C++ pipeline would (same objects, same autograd function).
#include <torch/extension.h>

#include "PointRendererHip.h"
#include "SceneDataHip.h"

namespace py = pybind11;

struct PyScene
{
    NeuralScene scene;
    PointRendererCache cache;
    StageTimerSystem timer;  // what a caller hangs on NeuralRenderInfo::timer_system (render(..., timed = true))

    PyScene(torch::Tensor position, c10::optional<torch::Tensor> normal, torch::Tensor index, torch::Tensor texture,
            torch::Tensor background, torch::Tensor poses_se3, torch::Tensor tangent_poses, torch::Tensor intrinsics,
            c10::optional<torch::Tensor> env)
    {
        scene.point_cloud_cuda = NeuralPointCloudCuda(position, normal.has_value() ? *normal : torch::Tensor(), index);
        // the leaf tensors stay the caller's objects so that autograd delivers the gradients to them
        scene.point_cloud_cuda->t_position = position;
        scene.texture                      = std::make_shared<NeuralTextureHolder>();
        scene.texture->texture             = texture;
        scene.texture->background_color    = background;
        scene.poses                        = std::make_shared<PoseModuleHolder>();
        scene.poses->poses_se3             = poses_se3;
        scene.poses->tangent_poses         = tangent_poses;
        scene.intrinsics                   = std::make_shared<IntrinsicsModuleHolder>();
        scene.intrinsics->intrinsics       = intrinsics;
        if (env.has_value())
        {
            scene.environment_map          = std::make_shared<EnvironmentMapHolder>();
            scene.environment_map->texture = *env;
        }
    }
};

static RenderParams ParamsFromDict(const py::dict& d)
{
    RenderParams p;
    p.drop_out_points_by_radius = false;
    p.dropout                   = 0;
    p.dist_cutoff               = 1e4f;
#define GET(name, type) \
    if (d.contains(#name)) p.name = d[#name].cast<type>()
    GET(test_backward_mode, int);
    GET(check_normal, bool);
    GET(render_points, bool);
    GET(super_sampling, bool);
    GET(dropout, float);
    GET(depth_accept, float);
    GET(ghost_gradients, bool);
    GET(drop_out_radius_threshold, float);
    GET(drop_out_points_by_radius, bool);
    GET(distortion_gradient_factor, float);
    GET(K_gradient_factor, float);
    GET(dist_cutoff, float);
    GET(output_background_mask, bool);
    GET(output_background_mask_value, float);
    GET(normalize_mode, int);
    GET(debug_print_num_rendered_points, bool);
#undef GET
    return p;
}

// views: (w, h, image_index, camera_index, camera_model, crop_fx, crop_fy, crop_cx, crop_cy, crop_s)
using ViewTuple = std::tuple<int, int, int, int, int, float, float, float, float, float>;

static std::vector<torch::Tensor> Render(PyScene& s, const std::vector<ViewTuple>& views, const py::dict& params,
                                         int num_layers, bool training, bool through_module, bool timed,
                                         bool cat_env_to_color)
{
    NeuralRenderInfo nri;
    nri.scene        = &s.scene;
    nri.num_layers   = num_layers;
    nri.params       = ParamsFromDict(params);
    nri.cache        = &s.cache;
    nri.timer_system = timed ? &s.timer : nullptr;
    for (auto& v : views)
    {
        ReducedImageInfo i;
        i.w                 = std::get<0>(v);
        i.h                 = std::get<1>(v);
        i.image_index       = std::get<2>(v);
        i.camera_index      = std::get<3>(v);
        i.camera_model_type = (CameraModel)std::get<4>(v);
        i.crop_transform    = {std::get<5>(v), std::get<6>(v), std::get<7>(v), std::get<8>(v), std::get<9>(v)};
        nri.images.push_back(i);
    }
    if (!through_module) return BlendPointCloud(&nri);
    PointRenderModuleOptions opt;
    opt.cat_env_to_color = cat_env_to_color;
    auto [images, masks] = PointRenderModuleForward(&nri, &s.cache, opt, training);
    images.insert(images.end(), masks.begin(), masks.end());
    return images;
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    py::class_<PyScene>(m, "Scene")
        .def(py::init<torch::Tensor, c10::optional<torch::Tensor>, torch::Tensor, torch::Tensor, torch::Tensor,
                      torch::Tensor, torch::Tensor, torch::Tensor, c10::optional<torch::Tensor>>(),
             py::arg("position"), py::arg("normal"), py::arg("index"), py::arg("texture"), py::arg("background"),
             py::arg("poses_se3"), py::arg("tangent_poses"), py::arg("intrinsics"), py::arg("env") = py::none())
        .def("apply_tangent", [](PyScene& s) { s.scene.poses->ApplyTangent(); })
        // the scene's StageTimerSystem, used as the reference's viewer uses its timer system: begin_frame(), render
        // calls with timed = true (and their backward passes), end_frame(), stage_times()
        .def("begin_frame", [](PyScene& s) { s.timer.BeginFrame(); })
        .def("end_frame", [](PyScene& s) { s.timer.EndFrame(); })
        .def("stage_times", [](PyScene& s) {
            py::dict d;
            for (auto& [name, e] : s.timer.Stages())
                d[py::str(name)] = py::make_tuple(e.last_ms, e.total_ms, e.calls, e.frames);
            return d;
        });
    m.def("render", &Render, py::arg("scene"), py::arg("views"), py::arg("params"), py::arg("num_layers"),
          py::arg("training") = true, py::arg("through_module") = false, py::arg("timed") = false,
          py::arg("cat_env_to_color") = false);
    m.def("apply_tangent_to_pose", &ApplyTangentToPose);
    // point-cloud processing of a new scene (SceneDataHip.cpp)
    m.def("knn_distance", &KNearestNeighbourDistance, py::arg("position"), py::arg("n") = 4);
    m.def("morton_codes", &MortonCodes);
    m.def("reorder_morton64", &ReorderMorton64);
    m.def("point_distance_to_camera",
          [](torch::Tensor position, torch::Tensor poses, torch::Tensor intrinsics, const std::vector<ViewTuple>& frames) {
              std::vector<ReducedImageInfo> f;
              for (auto& v : frames)
              {
                  ReducedImageInfo i;
                  i.w                 = std::get<0>(v);
                  i.h                 = std::get<1>(v);
                  i.image_index       = std::get<2>(v);
                  i.camera_index      = std::get<3>(v);
                  i.camera_model_type = (CameraModel)std::get<4>(v);
                  i.crop_transform    = {std::get<5>(v), std::get<6>(v), std::get<7>(v), std::get<8>(v), std::get<9>(v)};
                  f.push_back(i);
              }
              return PointDistanceToCamera(position, poses, intrinsics, f);
          });
    m.def("remove_lonely_points", &RemoveLonelyPoints, py::arg("position"), py::arg("camera_distance"), py::arg("n") = 5,
          py::arg("dis_th") = 0.02f);
    m.def("remove_close_points", &RemoveClosePoints, py::arg("position"), py::arg("camera_distance"),
          py::arg("dis_th") = 0.00005f);
    m.def("sort_blocks_by_radius", &SortBlocksByRadius, py::arg("radius"), py::arg("block_size") = 256);
    m.def("preprocess_point_cloud",
          [](torch::Tensor position, c10::optional<torch::Tensor> normal, int n, int block_size, int64_t seed) {
              auto r = PreprocessPointCloud(position, normal.has_value() ? *normal : torch::Tensor(), n, block_size, seed);
              return std::make_tuple(r.position, r.normal.defined() ? c10::optional<torch::Tensor>(r.normal) : c10::nullopt,
                                     r.data, r.order);
          },
          py::arg("position"), py::arg("normal") = py::none(), py::arg("n") = 4, py::arg("block_size") = 256,
          py::arg("seed") = 0);
    m.def("filter_point_cloud",
          [](torch::Tensor position, torch::Tensor poses, torch::Tensor intrinsics, const std::vector<ViewTuple>& frames) {
              std::vector<ReducedImageInfo> f;
              for (auto& v : frames)
              {
                  ReducedImageInfo i;
                  i.w                 = std::get<0>(v);
                  i.h                 = std::get<1>(v);
                  i.image_index       = std::get<2>(v);
                  i.camera_index      = std::get<3>(v);
                  i.camera_model_type = (CameraModel)std::get<4>(v);
                  f.push_back(i);
              }
              return FilterPointCloud(position, poses, intrinsics, f);
          });
}
