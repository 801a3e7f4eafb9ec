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
