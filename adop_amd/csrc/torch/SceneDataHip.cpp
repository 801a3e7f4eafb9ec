// SceneDataHip.cpp — see SceneDataHip.h.
#include "SceneDataHip.h"

#include <c10/hip/HIPStream.h>

#include "../../../include/adop_raster.h"

namespace
{
void* Stream()
{
    return (void*)c10::hip::getCurrentHIPStream().stream();
}

void Check(adop_status st)
{
    TORCH_CHECK(st == ADOP_OK, "adop_raster: ", adop_last_error_string());
}

torch::Tensor CheckedPosition(torch::Tensor position)
{
    TORCH_CHECK(position.is_cuda() && position.scalar_type() == torch::kFloat32 && position.dim() == 2 &&
                    position.size(1) == 4,
                "position must be a [N,4] float tensor on the device");
    return position.contiguous();
}

// bounding box of the cloud as host floats (one reduction over the contiguous array)
void BoundingBox(const torch::Tensor& position, float* mn, float* mx)
{
    auto [lo, hi] = torch::aminmax(position, 0);
    auto both     = torch::stack({lo, hi}).cpu();
    auto a        = both.accessor<float, 2>();
    for (int k = 0; k < 3; ++k)
    {
        mn[k] = a[0][k];
        mx[k] = a[1][k];
    }
}

torch::Tensor Workspace(size_t bytes, const torch::Tensor& like)
{
    return torch::empty({(int64_t)(bytes > 0 ? bytes : 1)}, like.options().dtype(torch::kUInt8));
}
}  // namespace

torch::Tensor KNearestNeighbourDistance(torch::Tensor position, int n)
{
    position = CheckedPosition(position);
    const int N = (int)position.size(0);
    auto out    = torch::empty({N}, position.options());
    auto ws     = Workspace(adop_knn_workspace_size(N), position);
    float mn[3], mx[3];
    BoundingBox(position, mn, mx);
    Check(adop_knn_distance(position.data_ptr<float>(), N, n, mn, mx, out.data_ptr<float>(), ws.data_ptr(),
                            (size_t)ws.numel(), Stream()));
    return out;
}

torch::Tensor MortonCodes(torch::Tensor position)
{
    position = CheckedPosition(position);
    const int N = (int)position.size(0);
    auto codes  = torch::empty({N}, position.options().dtype(torch::kInt64));
    float mn[3], mx[3];
    BoundingBox(position, mn, mx);
    Check(adop_morton_codes(position.data_ptr<float>(), N, mn, mx, (uint64_t*)codes.data_ptr<int64_t>(), Stream()));
    return codes;
}

torch::Tensor ReorderMorton64(torch::Tensor position)
{
    return std::get<1>(torch::sort(MortonCodes(position), /*stable=*/true, 0, false));
}

torch::Tensor PointDistanceToCamera(torch::Tensor position, torch::Tensor poses_se3, torch::Tensor intrinsics,
                                    const std::vector<ReducedImageInfo>& frames)
{
    position   = CheckedPosition(position);
    poses_se3  = poses_se3.contiguous();
    intrinsics = intrinsics.contiguous();
    TORCH_CHECK(poses_se3.is_cuda() && poses_se3.scalar_type() == torch::kFloat64 && poses_se3.size(1) == 8);
    TORCH_CHECK(intrinsics.is_cuda() && intrinsics.scalar_type() == torch::kFloat32 && intrinsics.size(1) == 13);
    adop_scene s{};
    s.position        = position.data_ptr<float>();
    s.num_points      = (int32_t)position.size(0);
    s.poses_se3       = poses_se3.data_ptr<double>();
    s.num_poses       = (int32_t)poses_se3.size(0);
    s.intrinsics      = intrinsics.data_ptr<float>();
    s.num_cameras     = (int32_t)intrinsics.size(0);
    s.intrinsics_cols = 13;
    std::vector<adop_view> views;
    for (const auto& i : frames)
        views.push_back(adop_view{i.w, i.h, i.image_index, i.camera_index, (int32_t)i.camera_model_type,
                                  i.crop_transform.fx, i.crop_transform.fy, i.crop_transform.cx, i.crop_transform.cy,
                                  i.crop_transform.s});
    auto out = torch::empty({position.size(0)}, position.options());
    auto ws  = Workspace(adop_frames_workspace_size((int32_t)views.size()), position);
    Check(adop_point_distance_to_camera(&s, views.data(), (int32_t)views.size(), out.data_ptr<float>(), ws.data_ptr(),
                                        (size_t)ws.numel(), Stream()));
    return out;
}

torch::Tensor RemoveLonelyPoints(torch::Tensor position, torch::Tensor camera_distance, int n, float dis_th)
{
    // d / cam_dis > dis_th erases the point (SceneData.cpp:585-590)
    return torch::logical_not(KNearestNeighbourDistance(position, n) / camera_distance > dis_th);
}

torch::Tensor RemoveClosePoints(torch::Tensor position, torch::Tensor camera_distance, float dis_th)
{
    position = CheckedPosition(position);
    const int N = (int)position.size(0);
    auto radius = (dis_th / camera_distance).to(torch::kFloat32).contiguous();  // :619
    auto state  = torch::empty({N}, position.options().dtype(torch::kInt32));
    const int rounds = 8;
    auto undecided   = torch::empty({rounds}, position.options().dtype(torch::kInt32));
    auto ws          = Workspace(adop_knn_workspace_size(N), position);
    float mn[3], mx[3];
    BoundingBox(position, mn, mx);
    for (int resume = 0;; resume = 1)
    {
        Check(adop_close_points(position.data_ptr<float>(), N, radius.data_ptr<float>(), mn, mx,
                                state.data_ptr<int32_t>(), (uint32_t*)undecided.data_ptr<int32_t>(), rounds, resume,
                                ws.data_ptr(), (size_t)ws.numel(), Stream()));
        if (undecided[rounds - 1].item<int32_t>() == 0) break;  // every point waits for its earlier neighbours only
    }
    return state == 1;
}

torch::Tensor SortBlocksByRadius(torch::Tensor radius, int block_size)
{
    const int64_t n = radius.size(0), nb = n / block_size;
    auto head   = radius.slice(0, 0, nb * block_size).reshape({nb, block_size});
    auto order  = std::get<1>(torch::sort(head, /*stable=*/true, 1, false)) +
                 (torch::arange(nb, radius.options().dtype(torch::kInt64)) * block_size).unsqueeze(1);
    auto tail = torch::arange(nb * block_size, n, radius.options().dtype(torch::kInt64));
    return torch::cat({order.reshape({-1}), tail});
}

torch::Tensor RandomBlockShuffle(int64_t num_points, int block_size, at::Generator generator, torch::Device device)
{
    const int64_t nb = num_points / block_size;
    auto i64         = torch::TensorOptions().dtype(torch::kInt64);
    auto perm        = torch::randperm(nb, generator, i64.device(torch::kCPU)).to(device);
    auto idx  = (perm.unsqueeze(1) * block_size + torch::arange(block_size, i64.device(device)).unsqueeze(0)).reshape({-1});
    auto tail = torch::arange(nb * block_size, num_points, i64.device(device));
    return torch::cat({idx, tail});
}

torch::Tensor ComputeRadius(torch::Tensor position, int n, at::Generator generator)
{
    position        = CheckedPosition(position);
    const int64_t N = position.size(0);
    auto data       = torch::zeros({N, 4}, position.options());
    data.select(1, 0).copy_(KNearestNeighbourDistance(position, n));
    auto u = torch::rand({N}, generator, position.options().dtype(torch::kFloat64));  // Random::sampleDouble(0, 1), :479
    data.select(1, 2).copy_(torch::sqrt(1.0 / u.clamp_min_(1e-300)).to(torch::kFloat32));
    data.select(1, 3).copy_(data.select(1, 0) * data.select(1, 2));
    return data;
}

torch::Tensor FilterPointCloud(torch::Tensor position, torch::Tensor poses_se3, torch::Tensor intrinsics,
                               const std::vector<ReducedImageInfo>& frames, int lonely_n, float lonely_th, float close_th)
{
    position = CheckedPosition(position);
    auto ids = torch::arange(position.size(0), position.options().dtype(torch::kInt64));
    // (per point: erasing other points does not change it)
    auto cam  = PointDistanceToCamera(position, poses_se3, intrinsics, frames);
    auto keep = RemoveLonelyPoints(position, cam, lonely_n, lonely_th);
    position  = position.index({keep}).contiguous();
    cam       = cam.index({keep});
    ids       = ids.index({keep});
    keep      = RemoveClosePoints(position, cam, close_th);
    return ids.index({keep});
}

PreprocessedCloud PreprocessPointCloud(torch::Tensor position, torch::Tensor normal, int n, int block_size, int64_t seed)
{
    position      = CheckedPosition(position);
    auto host_gen = at::detail::createCPUGenerator((uint64_t)seed);
    auto dev_gen  = at::globalContext().defaultGenerator(position.device()).clone();
    dev_gen.set_current_seed((uint64_t)seed);
    auto order = ReorderMorton64(position);
    order      = order.index({RandomBlockShuffle(position.size(0), block_size, host_gen, position.device())});
    position   = position.index({order}).contiguous();
    auto data  = ComputeRadius(position, n, dev_gen);
    auto by_radius = SortBlocksByRadius(data.select(1, 3), block_size);
    PreprocessedCloud out;
    out.order    = order.index({by_radius});
    out.position = position.index({by_radius}).clone();
    out.data     = data.index({by_radius}).contiguous();
    out.position.select(1, 3).copy_(out.data.select(1, 3));
    if (normal.defined()) out.normal = normal.index({out.order}).contiguous();
    return out;
}
