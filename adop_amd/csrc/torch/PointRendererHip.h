// PointRendererHip.h — libTorch (ROCm) side of the rasterizer: the declarations of ADOP's
// src/lib/rendering/PointRenderer.h, NeuralPointCloudCuda.h and RenderInfo.h, implemented on top of the C-ABI
// (include/adop_raster.h) instead of the CUDA kernels.
//
// Inside the ADOP tree this file is not needed: keep ADOP's own headers and compile PointRendererHip.cpp in place
// of PointRenderer.cu.  The small structs below (ReducedImageInfo, RenderParams, NeuralScene with its holders)
// carry exactly the members the render stage reads, so that the wrapper also builds and is tested stand-alone.
#pragma once
#include <torch/torch.h>

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "../../../include/adop_raster.h"

// ---- data/SceneData.h:28-47 -----------------------------------------------------------------------
enum class CameraModel
{
    PINHOLE_DISTORTION = 0,
    OCAM               = 1,
};

struct IntrinsicsPinholef  // saiga IntrinsicsPinhole<float>: fx, fy, cx, cy, s
{
    float fx = 1, fy = 1, cx = 0, cy = 0, s = 0;
    IntrinsicsPinholef scale(float f) const { return {fx * f, fy * f, cx * f, cy * f, s * f}; }
};

struct ReducedImageInfo
{
    int w = 0, h = 0;
    int image_index               = -1;
    int camera_index              = -1;
    CameraModel camera_model_type = CameraModel::PINHOLE_DISTORTION;
    IntrinsicsPinholef crop_transform;
};

// ---- data/Settings.h:16-69 ------------------------------------------------------------------------
struct RenderParams
{
    int test_backward_mode               = 0;
    bool render_points                   = true;
    bool check_normal                    = true;
    bool super_sampling                  = false;
    float dropout                        = 0.25;
    float depth_accept                   = 0.01;
    bool ghost_gradients                 = false;
    float drop_out_radius_threshold      = 0.6;
    bool drop_out_points_by_radius       = true;
    float distortion_gradient_factor     = 0.005;
    float K_gradient_factor              = 0.5;
    int num_texture_channels             = -1;
    float dist_cutoff                    = 2;
    bool output_background_mask          = false;
    float output_background_mask_value   = 0;
    bool debug_print_num_rendered_points = false;  // prints the sum of the weights after a forward (:1502-1512)
    // not in the reference: 0 = NormalizeGradient exactly as the reference launches it, 1 = row-wise
    int normalize_mode = 0;
};

// ---- rendering/NeuralPointCloudCuda.h:19-45 ---------------------------------------------------------
class NeuralPointCloudCudaImpl : public torch::nn::Module
{
   public:
    // position [n,4] f32 (xyz, drop-out radius), normal [n,1] i32 (10-bit packed) or undefined, index [n,1] i32
    NeuralPointCloudCudaImpl(torch::Tensor position, torch::Tensor normal, torch::Tensor index);
    int Size() { return (int)t_position.size(0); }
    bool IndexIsIdentity();  // t_index[i] == i (NeuralPointCloud.h:31); evaluated once

    torch::Tensor t_position;
    torch::Tensor t_normal;
    torch::Tensor t_index;

   private:
    int index_is_identity = -1;
};
TORCH_MODULE(NeuralPointCloudCuda);

// ---- the tensors of models/NeuralTexture.h, data/NeuralStructure.h the render stage reads -----------
struct NeuralTextureHolder
{
    torch::Tensor texture;           // [C,N] f32 | f16
    torch::Tensor background_color;  // [C]
};
struct PoseModuleHolder
{
    torch::Tensor poses_se3;      // [F,8] f64, world -> camera (NeuralStructure.cpp:13-27)
    torch::Tensor tangent_poses;  // [F,6] f64
    void ApplyTangent();          // NeuralStructure.cpp:41-44
};
struct IntrinsicsModuleHolder
{
    torch::Tensor intrinsics;  // [K,13] | [K,5+P]
};
struct EnvironmentMapHolder
{
    torch::Tensor texture;  // [1,C,H,W] | [C,H,W]
};
struct NeuralScene
{
    std::shared_ptr<NeuralTextureHolder> texture;
    NeuralPointCloudCuda point_cloud_cuda = nullptr;
    std::shared_ptr<PoseModuleHolder> poses;
    std::shared_ptr<IntrinsicsModuleHolder> intrinsics;
    std::shared_ptr<EnvironmentMapHolder> environment_map;
};

// ---- rendering/PointRenderer.h ------------------------------------------------------------------------
using Packtype           = unsigned long long;
constexpr int max_layers = ADOP_MAX_LAYERS;

class PointRendererCache;

// Stands where saiga's CUDA::CudaTimerSystem stands in the reference (NeuralRenderInfo::timer_system,
// PointRenderer.h:32; the SAIGA_OPTIONAL_TIME_MEASURE scopes of PointRenderer.cu:906-1610): while a render call runs with
// a timer system attached, the library records HIP events around its stages on the call's stream
// (adop_profile_enable); EndFrame() waits for them (adop_profile_read) and adds the stage times of the frame to the
// table, under the reference's stage names.  Used as the reference's viewer uses its timer system
// (RealTimeRenderer.cpp:80,196): BeginFrame(), render calls, EndFrame(), then read.
class StageTimerSystem
{
   public:
    struct Entry
    {
        float last_ms  = 0;  // the stage's time in the last finished frame (all its launches)
        double total_ms = 0;
        long calls      = 0;  // launches of the stage over all frames
        long frames     = 0;
    };
    void BeginFrame();
    void EndFrame();
    const std::map<std::string, Entry>& Stages() const { return stages; }
    void Reset() { stages.clear(); }

   private:
    std::map<std::string, Entry> stages;
};

class NeuralRenderInfo : public torch::CustomClassHolder
{
   public:
    NeuralScene* scene = nullptr;
    std::vector<ReducedImageInfo> images;
    RenderParams params;
    int num_layers                 = 0;
    StageTimerSystem* timer_system = nullptr;  // PointRenderer.h:32
    PointRendererCache* cache      = nullptr;
};

namespace torch::autograd
{
struct PointRender : public Function<PointRender>
{
    // returns a tensor for every layer (then a mask for every layer if params.output_background_mask)
    static variable_list forward(AutogradContext* ctx, Variable texture, Variable background_color, Variable points,
                                 Variable pose_tangents, Variable intrinsics, IValue info);
    static variable_list backward(AutogradContext* ctx, variable_list grad_output);
};
// Environment map on the empty pixels (EnvironmentMapImpl::Sample, EnvironmentMap.cu:107-157, and the composition of
// RenderModule.cpp:106-127) as one autograd function over the library's fused kernels: the forward pass samples only
// where the composition looks (mask != 1) and writes the composed images, the backward pass sums the texture gradient
// per tile in LDS from the texture coordinates the forward pass kept.  Same numbers as torch's grid_sample (bilinear,
// border, align_corners) on the reference's uv followed by images + (1 - mask) * env.
struct EnvironmentMapCompose : public Function<EnvironmentMapCompose>
{
    // texture [C,H,W] | [1,C,H,W]; images: L tensors [B,C,h_l,w_l]; masks: L tensors [B,1,h_l,w_l] (not differentiated);
    // cat_env_to_color: the sampled map of every pixel is returned by itself (for torch::cat) instead of composed.
    // Returns L tensors.  The views are info's images (pinhole, or OCam as an extension).
    static variable_list forward(AutogradContext* ctx, Variable texture, at::TensorList images, at::TensorList masks,
                                 IValue info, bool cat_env_to_color);
    static variable_list backward(AutogradContext* ctx, variable_list grad_output);
};
}  // namespace torch::autograd

std::vector<torch::Tensor> BlendPointCloud(NeuralRenderInfo* info);

std::pair<std::vector<torch::Tensor>, std::vector<torch::Tensor>> BlendPointCloudForward(
    torch::autograd::AutogradContext* ctx, NeuralRenderInfo* info);
torch::autograd::variable_list BlendPointCloudBackward(torch::autograd::AutogradContext* ctx, NeuralRenderInfo* info,
                                                       torch::autograd::variable_list image_gradients);

void ApplyTangentToPose(torch::Tensor tangent, torch::Tensor pose);

struct LayerCuda
{
    int w = 0, h = 0;
    float scale = 1;
    torch::Tensor depth;
    torch::Tensor weight;
    torch::Tensor depth_index_tensor;  // int64 storage of (depth bits << 32 | point id)
};

class PointRendererCache
{
   public:
    void Build(NeuralRenderInfo* info, bool forward);
    void Allocate(NeuralRenderInfo* info, bool forward);
    void InitializeData(bool forward);

    std::vector<LayerCuda> layers_cuda;
    NeuralRenderInfo* info = nullptr;
    int num_batches        = 0;

    torch::Tensor dropout_points;  // [batch, num_points]
    std::vector<torch::Tensor> output_forward;
    std::vector<torch::Tensor> output_forward_background_mask;

    torch::Tensor output_gradient_texture;
    torch::Tensor output_gradient_background;
    torch::Tensor output_gradient_points;
    torch::Tensor output_gradient_pose_tangent;
    torch::Tensor output_gradient_pose_tangent_count;
    torch::Tensor output_gradient_point_count;
    torch::Tensor output_gradient_intrinsics;
    torch::Tensor output_gradient_intrinsics_count;
    std::vector<torch::Tensor> image_gradients;

    torch::Tensor workspace;  // uint8, adop_workspace_size bytes

    // realloc key {C, N, L, B, h, w} (PointRenderer.cu:961-969)
    std::vector<int> cache_size = {0, 0, 0, 0, 0, 0};
};

// ---- rendering/RenderModule.h ----------------------------------------------------------------------------
// forward(NeuralRenderInfo*) of PointRenderModuleImpl (RenderModule.cpp:38-144): super-sampling, BlendPointCloud,
// environment map composition.  Returns {images, masks}.
struct PointRenderModuleOptions
{
    bool cat_env_to_color   = false;
    bool cat_masks_to_color = false;
};
std::pair<std::vector<torch::Tensor>, std::vector<torch::Tensor>> PointRenderModuleForward(
    NeuralRenderInfo* nri, PointRendererCache* cache, const PointRenderModuleOptions& opt, bool training);
