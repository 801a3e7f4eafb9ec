// SceneDataHip.h — the point-cloud processing of a new scene (data/SceneData.cpp:96-104, 441-684) on device tensors:
// what SceneData does with its host vectors and kd-trees, done over the C-ABI of libadop_raster.so.  All tensors live
// on the GPU; position is [N,4] f32 (x, y, z, w unused on input).
#pragma once
#include <torch/torch.h>

#include <vector>

#include "PointRendererHip.h"

// data[i](0) of ComputeRadius (SceneData.cpp:441-463): distance to the n-th nearest other point, [N] f32.
torch::Tensor KNearestNeighbourDistance(torch::Tensor position, int n = 4);
// key of PointCloud::ReorderMorton64 (SceneData.cpp:101): [N] int64, and the permutation that sorts by it.
torch::Tensor MortonCodes(torch::Tensor position);
torch::Tensor ReorderMorton64(torch::Tensor position);
// SceneData::PointDistanceToCamera (:645-669): [N] f32.  poses_se3 [F,8] f64 (view transforms), intrinsics [K,13].
torch::Tensor PointDistanceToCamera(torch::Tensor position, torch::Tensor poses_se3, torch::Tensor intrinsics,
                                    const std::vector<ReducedImageInfo>& frames);
// keep masks ([N] bool) of SceneData::RemoveLonelyPoints (:550-595) and RemoveClosePoints (:598-642)
torch::Tensor RemoveLonelyPoints(torch::Tensor position, torch::Tensor camera_distance, int n = 5, float dis_th = 0.02f);
torch::Tensor RemoveClosePoints(torch::Tensor position, torch::Tensor camera_distance, float dis_th = 0.00005f);
// permutation of SceneData::SortBlocksByRadius (:671-684)
torch::Tensor SortBlocksByRadius(torch::Tensor radius, int block_size = 256);
// permutation of PointCloud::RandomBlockShuffle (SceneData.cpp:102): whole blocks of block_size consecutive points in
// random order (a last, shorter block stays last); the order of the blocks is drawn on the host from `generator`.
torch::Tensor RandomBlockShuffle(int64_t num_points, int block_size, at::Generator generator, torch::Device device);
// SceneData::ComputeRadius (:441-484): data [N,4] with data[:,0] = distance to the n-th neighbour, data[:,2] =
// sqrt(1 / u), u ~ U(0,1) drawn on the device from `generator`, data[:,3] = data[:,0] * data[:,2] (the drop-out radius
// the rasterizer reads as position.w).
torch::Tensor ComputeRadius(torch::Tensor position, int n, at::Generator generator);
// The two filters of a new scene in the reference's order (SceneData.cpp:98-99): ids of the surviving points, ascending.
torch::Tensor FilterPointCloud(torch::Tensor position, torch::Tensor poses_se3, torch::Tensor intrinsics,
                               const std::vector<ReducedImageInfo>& frames, int lonely_n = 5, float lonely_th = 0.02f,
                               float close_th = 0.00005f);
// The initial processing of a new scene (SceneData.cpp:101-104): ReorderMorton64, RandomBlockShuffle(256), ComputeRadius,
// SortBlocksByRadius(256).  position comes back reordered with the drop-out radius in w; order maps new to original ids.
struct PreprocessedCloud
{
    torch::Tensor position;  // [N,4]
    torch::Tensor normal;    // reordered like position, or undefined
    torch::Tensor data;      // [N,4]
    torch::Tensor order;     // [N] int64
};
PreprocessedCloud PreprocessPointCloud(torch::Tensor position, torch::Tensor normal, int n = 4, int block_size = 256,
                                       int64_t seed = 0);
