// PointRendererHip.cpp — implements rendering/PointRenderer.h + RenderInfo.cpp + RenderModule.cpp:38-144 of ADOP on
// top of libadop_raster.so.  Replaces src/lib/rendering/PointRenderer.cu in an ADOP build for ROCm.
#include "PointRendererHip.h"

#include <iostream>

#include <c10/hip/HIPStream.h>

namespace
{
void* CurrentStream()
{
    return (void*)c10::hip::getCurrentHIPStream().stream();
}

adop_scene MakeScene(NeuralScene& s)
{
    adop_scene o{};
    auto& pc           = *s.point_cloud_cuda;
    o.position         = pc.t_position.data_ptr<float>();
    o.normal           = pc.t_normal.defined() ? pc.t_normal.data_ptr<int>() : nullptr;
    o.index            = (const int32_t*)pc.t_index.data_ptr();
    o.num_points       = pc.Size();
    o.texture          = s.texture->texture.data_ptr();
    o.texture_dtype    = s.texture->texture.dtype() == torch::kFloat16 ? ADOP_TEXTURE_F16 : ADOP_TEXTURE_F32;
    o.num_channels     = (int)s.texture->texture.size(0);
    o.num_texels       = (int)s.texture->texture.size(1);
    o.background_color = s.texture->background_color.data_ptr<float>();
    o.poses_se3        = s.poses->poses_se3.data_ptr<double>();
    o.num_poses        = (int)s.poses->poses_se3.size(0);
    o.intrinsics       = s.intrinsics->intrinsics.data_ptr<float>();
    o.num_cameras      = (int)s.intrinsics->intrinsics.size(0);
    o.intrinsics_cols  = (int)s.intrinsics->intrinsics.size(1);
    o.index_is_identity = (pc.IndexIsIdentity() && o.num_texels == o.num_points) ? 1 : 0;
    return o;
}

adop_view MakeView(const ReducedImageInfo& i)
{
    adop_view v{};
    v.w                 = i.w;
    v.h                 = i.h;
    v.image_index       = i.image_index;
    v.camera_index      = i.camera_index;
    v.camera_model_type = (int32_t)i.camera_model_type;
    v.crop_fx           = i.crop_transform.fx;
    v.crop_fy           = i.crop_transform.fy;
    v.crop_cx           = i.crop_transform.cx;
    v.crop_cy           = i.crop_transform.cy;
    v.crop_s            = i.crop_transform.s;
    return v;
}

adop_render_params MakeParams(const RenderParams& p)
{
    adop_render_params o{};
    o.test_backward_mode           = p.test_backward_mode;
    o.check_normal                 = p.check_normal;
    o.ghost_gradients              = p.ghost_gradients;
    o.drop_out_points_by_radius    = p.drop_out_points_by_radius;
    o.depth_accept                 = p.depth_accept;
    o.drop_out_radius_threshold    = p.drop_out_radius_threshold;
    o.dist_cutoff                  = p.dist_cutoff;
    o.distortion_gradient_factor   = p.distortion_gradient_factor;
    o.K_gradient_factor            = p.K_gradient_factor;
    o.output_background_mask       = p.output_background_mask;
    o.output_background_mask_value = p.output_background_mask_value;
    o.normalize_mode               = p.normalize_mode;
    o.skip_points                  = p.render_points ? 0 : 1;  // PointRenderer.cu:1417,1433
    return o;
}

std::vector<adop_view> MakeViews(NeuralRenderInfo* info)
{
    std::vector<adop_view> v;
    for (auto& i : info->images) v.push_back(MakeView(i));
    return v;
}

void Check(adop_status st)
{
    TORCH_CHECK(st == ADOP_OK, "adop_raster: ", adop_last_error_string());
}

// While one of these lives and a timer system is attached, the library records its stage events on this thread.
struct StageRecording
{
    bool on;
    explicit StageRecording(StageTimerSystem* t) : on(t != nullptr)
    {
        if (on) adop_profile_enable(1);
    }
    ~StageRecording()
    {
        if (on) adop_profile_enable(0);
    }
};
}  // namespace

// ---- StageTimerSystem (the role of CUDA::CudaTimerSystem behind NeuralRenderInfo::timer_system) -------------
void StageTimerSystem::BeginFrame()
{
    // events of calls that ran outside a frame are dropped
    adop_stage_time scratch[32];
    adop_profile_read(scratch, 32);
}

void StageTimerSystem::EndFrame()
{
    adop_stage_time t[32];
    const int n = adop_profile_read(t, 32);  // waits for the events of the frame's calls
    for (int i = 0; i < n; ++i)
    {
        Entry& e  = stages[t[i].name];
        e.last_ms = t[i].total_ms;
        e.total_ms += t[i].total_ms;
        e.calls += t[i].calls;
        e.frames += 1;
    }
}

// ---- NeuralPointCloudCuda ----------------------------------------------------------------------------------
NeuralPointCloudCudaImpl::NeuralPointCloudCudaImpl(torch::Tensor position, torch::Tensor normal, torch::Tensor index)
{
    TORCH_CHECK(position.dim() == 2 && position.size(1) == 4 && position.dtype() == torch::kFloat32);
    TORCH_CHECK(index.size(0) == position.size(0) && index.dtype() == torch::kInt32);
    t_position = position.contiguous().cuda();
    t_index    = index.contiguous().cuda();
    register_parameter("t_position", t_position);
    register_buffer("t_index", t_index);
    if (normal.defined())
    {
        TORCH_CHECK(normal.size(0) == position.size(0) && normal.dtype() == torch::kInt32);
        t_normal = normal.contiguous().cuda();
        register_buffer("t_normal", t_normal);
    }
}

bool NeuralPointCloudCudaImpl::IndexIsIdentity()
{
    if (index_is_identity < 0)
    {
        auto ar = torch::arange(Size(), torch::TensorOptions().dtype(torch::kInt32).device(t_index.device()));
        index_is_identity = (t_index.view({-1}) == ar).all().item<bool>() ? 1 : 0;
    }
    return index_is_identity == 1;
}

void PoseModuleHolder::ApplyTangent()
{
    ApplyTangentToPose(tangent_poses, poses_se3);
}

// ---- PointRendererCache (PointRenderer.cu:902-1090) ---------------------------------------------------------
void PointRendererCache::Build(NeuralRenderInfo* info, bool forward)
{
    this->info        = info;
    this->num_batches = (int)info->images.size();
    TORCH_CHECK(num_batches > 0);
    Allocate(info, forward);
    if (forward) InitializeData(forward);
}

void PointRendererCache::Allocate(NeuralRenderInfo* info, bool forward)
{
    auto& fd = info->images.front();
    int h = fd.h, w = fd.w;
    TORCH_CHECK(info->scene->point_cloud_cuda && info->scene->texture);
    std::vector<int> new_cache_size = {(int)info->scene->texture->texture.size(0), info->scene->point_cloud_cuda->Size(),
                                       info->num_layers, num_batches, h, w};
    if (new_cache_size == cache_size) return;
    TORCH_CHECK(info->num_layers >= 1 && info->num_layers <= max_layers, "invalid number of layers");
    auto f32 = torch::TensorOptions().device(torch::kCUDA).dtype(torch::kFloat32);
    layers_cuda.assign(info->num_layers, LayerCuda());
    float scale = 1;
    for (int i = 0; i < info->num_layers; ++i)
    {
        TORCH_CHECK(w > 0 && h > 0);
        auto& l              = layers_cuda[i];
        l.depth              = torch::empty({num_batches, 1, h, w}, f32);
        l.weight             = torch::empty({num_batches, 1, h, w}, f32);
        l.depth_index_tensor = torch::empty({num_batches, 1, h, w}, f32.dtype(torch::kInt64));
        l.w                  = w;
        l.h                  = h;
        l.scale              = scale;
        h /= 2;
        w /= 2;
        scale *= 0.5f;
    }
    adop_scene s  = MakeScene(*info->scene);
    size_t nbytes = adop_workspace_size(&s, num_batches, info->num_layers, fd.w, fd.h);
    TORCH_CHECK(nbytes > 0, "adop_workspace_size failed");
    workspace  = torch::empty({(long)nbytes}, f32.dtype(torch::kUInt8));
    cache_size = new_cache_size;
}

void PointRendererCache::InitializeData(bool forward)
{
    if (!forward) return;
    auto f32 = torch::TensorOptions().device(torch::kCUDA).dtype(torch::kFloat32);
    int C    = (int)info->scene->texture->texture.size(0);
    // created every frame because they are moved to the caller (PointRenderer.cu:1050-1071); the library clears
    // what it accumulates into, so empty() is enough
    output_forward.resize(info->num_layers);
    for (int i = 0; i < info->num_layers; ++i)
        output_forward[i] = torch::empty({num_batches, C, layers_cuda[i].h, layers_cuda[i].w}, f32);
    output_forward_background_mask.clear();
    if (info->params.output_background_mask)
        for (int i = 0; i < info->num_layers; ++i)
            output_forward_background_mask.push_back(
                torch::empty({num_batches, 1, layers_cuda[i].h, layers_cuda[i].w}, f32));
    long N = info->scene->point_cloud_cuda->Size();
    if (info->params.dropout > 0)
    {
        if (!dropout_points.defined() || dropout_points.size(0) != num_batches || dropout_points.size(1) != N)
            dropout_points = torch::empty({num_batches, N}, f32);
        dropout_points.bernoulli_(info->params.dropout);  // PointRenderer.cu:1081-1084
    }
    else
        dropout_points = torch::Tensor();  // zero_() in the reference: nothing is dropped
}

// ---- BlendPointCloudForward (PointRenderer.cu:1389-1531) ----------------------------------------------------
static adop_forward_buffers MakeForwardBuffers(NeuralRenderInfo* info, const std::vector<torch::Tensor>& depth_index,
                                               const std::vector<torch::Tensor>& depth,
                                               const std::vector<torch::Tensor>& weight,
                                               const std::vector<torch::Tensor>& out,
                                               const std::vector<torch::Tensor>& mask, const torch::Tensor& dropout)
{
    adop_forward_buffers fb{};
    fb.num_layers = info->num_layers;
    for (int l = 0; l < info->num_layers; ++l)
    {
        fb.layers[l].w           = (int)depth[l].size(3);
        fb.layers[l].h           = (int)depth[l].size(2);
        fb.layers[l].depth_index = (uint64_t*)depth_index[l].data_ptr<int64_t>();
        fb.layers[l].depth       = depth[l].data_ptr<float>();
        fb.layers[l].weight      = weight[l].data_ptr<float>();
        fb.layers[l].out         = out[l].data_ptr<float>();
        fb.layers[l].mask        = mask.empty() ? nullptr : mask[l].data_ptr<float>();
    }
    fb.dropout_points = dropout.defined() ? dropout.data_ptr<float>() : nullptr;
    return fb;
}

std::pair<std::vector<torch::Tensor>, std::vector<torch::Tensor>> BlendPointCloudForward(
    torch::autograd::AutogradContext* ctx, NeuralRenderInfo* info)
{
    TORCH_CHECK(info->cache);
    PointRendererCache& cache = *info->cache;
    cache.Build(info, true);

    std::vector<torch::Tensor> di, d, w;
    for (auto& l : cache.layers_cuda)
    {
        di.push_back(l.depth_index_tensor);
        d.push_back(l.depth);
        w.push_back(l.weight);
    }
    adop_scene scene      = MakeScene(*info->scene);
    auto views            = MakeViews(info);
    adop_render_params rp = MakeParams(info->params);
    adop_forward_buffers fb =
        MakeForwardBuffers(info, di, d, w, cache.output_forward, cache.output_forward_background_mask, cache.dropout_points);
    // projected points: a saved tensor of the backward pass (no counterpart in the reference, which projects again)
    // ... and the resolved images pixel by pixel, which the spatial gradients read at four neighbours of a pixel
    torch::Tensor point_cache, pixel_cache;
    if (ctx)
    {
        point_cache    = torch::empty({(long)views.size(), (long)scene.num_points, 4}, d[0].options());
        fb.point_cache = point_cache.data_ptr<float>();
        long pixels    = 0;
        for (auto& l : cache.layers_cuda) pixels += (long)views.size() * l.w * l.h;
        pixel_cache    = torch::empty({pixels, (long)scene.num_channels}, d[0].options());
        fb.pixel_cache = pixel_cache.data_ptr<float>();
    }
    {
        StageRecording rec(info->timer_system);
        Check(adop_forward(&scene, views.data(), (int)views.size(), &rp, &fb, cache.workspace.data_ptr(),
                           (size_t)cache.workspace.numel(), nullptr, CurrentStream()));
    }

    if (info->params.debug_print_num_rendered_points)  // PointRenderer.cu:1502-1512
    {
        double weight_sum = 0;
        for (auto& l : cache.layers_cuda) weight_sum += l.weight.sum().item().toFloat();
        std::cout << "# Rasterized Points = " << (int)weight_sum << std::endl;
    }

    if (ctx)
    {
        // saved variables in the reference's order {depth_l, weight_l}_l, out_l, dropout (:1517-1525), then the packed
        // depth|index and the masks (extra)
        std::vector<torch::Tensor> save;
        for (auto& l : cache.layers_cuda)
        {
            save.push_back(l.depth);
            save.push_back(l.weight);
        }
        save.insert(save.end(), cache.output_forward.begin(), cache.output_forward.end());
        save.push_back(cache.dropout_points.defined() ? cache.dropout_points : torch::empty({0}, d[0].options()));
        for (auto& l : cache.layers_cuda) save.push_back(l.depth_index_tensor);
        save.push_back(point_cache);
        save.push_back(pixel_cache);
        ctx->save_for_backward(save);
        ctx->saved_data["num_masks"] = (int64_t)cache.output_forward_background_mask.size();
        // the cache buffers are handed to the graph: allocate fresh ones on the next forward
        cache.cache_size = {0, 0, 0, 0, 0, 0};
    }
    return {std::move(cache.output_forward), std::move(cache.output_forward_background_mask)};
}

// ---- BlendPointCloudBackward (PointRenderer.cu:1549-1644) ---------------------------------------------------
torch::autograd::variable_list BlendPointCloudBackward(torch::autograd::AutogradContext* ctx, NeuralRenderInfo* info,
                                                       torch::autograd::variable_list _image_gradients)
{
    TORCH_CHECK(info->cache);
    PointRendererCache& cache = *info->cache;
    NeuralScene& scene        = *info->scene;
    const int L               = info->num_layers;
    cache.info                = info;
    cache.num_batches         = (int)info->images.size();

    // the first L gradients belong to the images, the rest to the masks and are ignored (:1568-1571)
    cache.image_gradients.clear();
    for (int i = 0; i < L; ++i)
    {
        TORCH_CHECK(_image_gradients[i].defined() && _image_gradients[i].dtype() == torch::kFloat32);
        cache.image_gradients.push_back(_image_gradients[i].contiguous());
    }
    auto saved = ctx->get_saved_variables();
    TORCH_CHECK((int)saved.size() == L * 4 + 3);
    std::vector<torch::Tensor> di, d, w, out;
    for (int i = 0; i < L; ++i)
    {
        d.push_back(saved[i * 2 + 0]);
        w.push_back(saved[i * 2 + 1]);
        out.push_back(saved[L * 2 + i]);
        di.push_back(saved[L * 3 + 1 + i]);
    }
    torch::Tensor dropout = saved[L * 3];
    if (dropout.numel() == 0) dropout = torch::Tensor();

    // Build(info,false): the gradient tensors (:922-949); the library clears them
    auto f32 = torch::TensorOptions().device(torch::kCUDA).dtype(torch::kFloat32);
    cache.output_gradient_texture    = torch::empty(scene.texture->texture.sizes(), f32);
    cache.output_gradient_background = torch::empty_like(scene.texture->background_color);
    cache.output_gradient_points = cache.output_gradient_point_count = torch::Tensor();
    cache.output_gradient_pose_tangent = cache.output_gradient_pose_tangent_count = torch::Tensor();
    cache.output_gradient_intrinsics = cache.output_gradient_intrinsics_count = torch::Tensor();
    if (scene.point_cloud_cuda->t_position.requires_grad())
    {
        cache.output_gradient_points      = torch::empty_like(scene.point_cloud_cuda->t_position);
        cache.output_gradient_point_count = torch::empty({cache.output_gradient_points.size(0)}, f32);
    }
    if (scene.poses->tangent_poses.requires_grad())
    {
        cache.output_gradient_pose_tangent       = torch::empty_like(scene.poses->tangent_poses);
        cache.output_gradient_pose_tangent_count = torch::empty({scene.poses->tangent_poses.size(0)}, f32);
    }
    if (scene.intrinsics->intrinsics.requires_grad())
    {
        cache.output_gradient_intrinsics       = torch::empty_like(scene.intrinsics->intrinsics);
        cache.output_gradient_intrinsics_count = torch::empty({scene.intrinsics->intrinsics.size(0)}, f32);
    }

    adop_backward_buffers gb{};
    for (int i = 0; i < L; ++i) gb.grad_out[i] = cache.image_gradients[i].data_ptr<float>();
    gb.grad_texture    = cache.output_gradient_texture.data_ptr<float>();
    gb.grad_background = cache.output_gradient_background.data_ptr<float>();
    if (cache.output_gradient_points.defined())
    {
        TORCH_CHECK(cache.output_gradient_points.size(1) == 4);
        gb.grad_points       = cache.output_gradient_points.data_ptr<float>();
        gb.grad_points_count = cache.output_gradient_point_count.data_ptr<float>();
    }
    if (cache.output_gradient_pose_tangent.defined())
    {
        TORCH_CHECK(cache.output_gradient_pose_tangent.size(1) == 6);
        gb.grad_pose       = cache.output_gradient_pose_tangent.data_ptr<double>();
        gb.grad_pose_count = cache.output_gradient_pose_tangent_count.data_ptr<float>();
    }
    if (cache.output_gradient_intrinsics.defined())
    {
        gb.grad_intrinsics       = cache.output_gradient_intrinsics.data_ptr<float>();
        gb.grad_intrinsics_count = cache.output_gradient_intrinsics_count.data_ptr<float>();
    }

    adop_scene s          = MakeScene(scene);
    auto views            = MakeViews(info);
    adop_render_params rp = MakeParams(info->params);
    std::vector<torch::Tensor> no_mask;
    adop_forward_buffers fb = MakeForwardBuffers(info, di, d, w, out, no_mask, dropout);
    fb.point_cache          = saved[L * 4 + 1].data_ptr<float>();
    fb.pixel_cache          = saved[L * 4 + 2].data_ptr<float>();
    if (!cache.workspace.defined() ||
        (size_t)cache.workspace.numel() < adop_workspace_size(&s, (int)views.size(), L, views[0].w, views[0].h))
        cache.workspace = torch::empty({(long)adop_workspace_size(&s, (int)views.size(), L, views[0].w, views[0].h)},
                                       f32.dtype(torch::kUInt8));
    {
        StageRecording rec(info->timer_system);
        Check(adop_backward(&s, views.data(), (int)views.size(), &rp, &fb, &gb, cache.workspace.data_ptr(),
                            (size_t)cache.workspace.numel(), nullptr, CurrentStream()));
    }

    torch::Tensor g_tex = cache.output_gradient_texture;
    if (scene.texture->texture.dtype() != torch::kFloat32) g_tex = g_tex.to(scene.texture->texture.dtype());
    return {std::move(g_tex), std::move(cache.output_gradient_background), std::move(cache.output_gradient_points),
            std::move(cache.output_gradient_pose_tangent), std::move(cache.output_gradient_intrinsics)};
}

// ---- RenderInfo.cpp:11-59 -----------------------------------------------------------------------------------
// NeuralRenderInfo travels through autograd as an IValue custom class (RenderInfo.cpp:11-15)
TORCH_LIBRARY(adop_raster_hip, m)
{
    m.class_<NeuralRenderInfo>("NeuralRenderInfo").def(torch::init());
}

std::vector<torch::Tensor> BlendPointCloud(NeuralRenderInfo* info)
{
    torch::intrusive_ptr<NeuralRenderInfo> render_data = torch::make_intrusive<NeuralRenderInfo>(*info);
    TORCH_CHECK(render_data->scene && render_data->scene->texture);
    return torch::autograd::PointRender::apply(
        render_data->scene->texture->texture, render_data->scene->texture->background_color,
        render_data->scene->point_cloud_cuda->t_position, render_data->scene->poses->tangent_poses,
        render_data->scene->intrinsics->intrinsics, torch::IValue(render_data));
}

namespace torch::autograd
{
variable_list PointRender::forward(AutogradContext* ctx, Variable texture, Variable background_color, Variable points,
                                   Variable pose_tangents, Variable intrinsics, IValue info)
{
    ctx->saved_data["render_info"] = info;
    auto [color, mask]             = BlendPointCloudForward(ctx, info.toCustomClass<NeuralRenderInfo>().get());
    color.insert(color.end(), mask.begin(), mask.end());
    return color;
}

variable_list PointRender::backward(AutogradContext* ctx, variable_list grad_output)
{
    IValue info  = ctx->saved_data["render_info"];
    auto in      = info.toCustomClass<NeuralRenderInfo>().get();
    auto derives = BlendPointCloudBackward(ctx, in, grad_output);
    // the last empty grad is for the 'IValue info' of the forward function
    derives.push_back(Variable());
    return derives;
}
}  // namespace torch::autograd

// ---- EnvironmentMapImpl::Sample + composition as an autograd function -------------------------------------------
namespace
{
// The forward buffers of an environment-map call: level sizes from the tensors, `out` / `mask` as given.
adop_forward_buffers EnvBuffers(int L, const std::vector<torch::Tensor>& images, const std::vector<torch::Tensor>& masks)
{
    adop_forward_buffers fb{};
    fb.num_layers = L;
    for (int l = 0; l < L; ++l)
    {
        fb.layers[l].w    = (int)images[l].size(3);
        fb.layers[l].h    = (int)images[l].size(2);
        fb.layers[l].out  = images[l].data_ptr<float>();
        fb.layers[l].mask = masks.empty() ? nullptr : masks[l].data_ptr<float>();
    }
    return fb;
}
}  // namespace

namespace torch::autograd
{
variable_list EnvironmentMapCompose::forward(AutogradContext* ctx, Variable texture, at::TensorList images_in,
                                             at::TensorList masks_in, IValue info, bool cat_env_to_color)
{
    NeuralRenderInfo* nri = info.toCustomClass<NeuralRenderInfo>().get();
    const int L           = nri->num_layers;
    TORCH_CHECK((int)images_in.size() == L && (int)masks_in.size() == L, "one image and one mask per layer");
    torch::Tensor tex = texture.dim() == 4 ? texture.squeeze(0) : texture;
    TORCH_CHECK(tex.dim() == 3 && tex.dtype() == torch::kFloat32 && tex.is_cuda(), "environment map: [C,H,W] f32 on the device");
    tex = tex.contiguous();
    std::vector<torch::Tensor> images, masks, uv(L), outs(L);
    for (int l = 0; l < L; ++l)
    {
        images.push_back(images_in[l].contiguous());
        masks.push_back(masks_in[l].contiguous());
        TORCH_CHECK(images[l].size(1) == tex.size(0), "environment map and images differ in channels");
        uv[l]   = torch::empty({images[l].size(0), images[l].size(2), images[l].size(3), 2}, images[l].options());
        outs[l] = torch::empty_like(images[l]);
    }
    adop_scene s = MakeScene(*nri->scene);
    auto views   = MakeViews(nri);
    // composed: out of place (mode 2), sampling only where mask != 1; cat: the samples of every pixel (mode 0, no mask)
    adop_forward_buffers fb = EnvBuffers(L, images, cat_env_to_color ? std::vector<torch::Tensor>() : masks);
    std::vector<float*> uv_ptr(L), out_ptr(L);
    for (int l = 0; l < L; ++l)
    {
        uv_ptr[l]  = uv[l].data_ptr<float>();
        out_ptr[l] = outs[l].data_ptr<float>();
    }
    Check(adop_env_sample(&s, views.data(), (int)views.size(), tex.data_ptr<float>(), (int)tex.size(1), (int)tex.size(2),
                          &fb, uv_ptr.data(), out_ptr.data(), cat_env_to_color ? 0 : 2, CurrentStream()));
    variable_list save = uv;
    if (!cat_env_to_color) save.insert(save.end(), masks.begin(), masks.end());
    ctx->save_for_backward(save);
    ctx->saved_data["render_info"] = info;
    ctx->saved_data["cat"]         = cat_env_to_color;
    ctx->saved_data["tex_dim"]     = (int64_t)texture.dim();
    ctx->saved_data["env_h"]       = (int64_t)tex.size(1);
    ctx->saved_data["env_w"]       = (int64_t)tex.size(2);
    return outs;
}

variable_list EnvironmentMapCompose::backward(AutogradContext* ctx, variable_list grad_output)
{
    IValue info           = ctx->saved_data["render_info"];
    NeuralRenderInfo* nri = info.toCustomClass<NeuralRenderInfo>().get();
    const int L           = nri->num_layers;
    const bool cat        = ctx->saved_data["cat"].toBool();
    const int eh = (int)ctx->saved_data["env_h"].toInt(), ew = (int)ctx->saved_data["env_w"].toInt();
    auto saved = ctx->get_saved_variables();
    std::vector<torch::Tensor> uv(saved.begin(), saved.begin() + L), masks;
    if (!cat) masks.assign(saved.begin() + L, saved.begin() + 2 * L);
    std::vector<torch::Tensor> gout(L);
    for (int l = 0; l < L; ++l)
    {
        // (a level that does not reach the loss has no gradient)
        gout[l] = grad_output[l].defined() ? grad_output[l].contiguous()
                                           : torch::zeros({uv[l].size(0), nri->scene->texture->texture.size(0), uv[l].size(1), uv[l].size(2)},
                                                          uv[l].options());
    }
    adop_scene s            = MakeScene(*nri->scene);
    auto views              = MakeViews(nri);
    adop_forward_buffers fb = EnvBuffers(L, gout, masks);  // (only sizes and masks are read)
    std::vector<const float*> g_ptr(L), uv_ptr(L);
    for (int l = 0; l < L; ++l)
    {
        g_ptr[l]  = gout[l].data_ptr<float>();
        uv_ptr[l] = uv[l].data_ptr<float>();
    }
    torch::Tensor g_tex = torch::empty({(long)s.num_channels, (long)eh, (long)ew}, gout[0].options());
    Check(adop_env_sample_backward(&s, views.data(), (int)views.size(), eh, ew, &fb, g_ptr.data(), uv_ptr.data(),
                                   g_tex.data_ptr<float>(), CurrentStream()));
    if (ctx->saved_data["tex_dim"].toInt() == 4) g_tex = g_tex.unsqueeze(0);
    // inputs: texture, L images, L masks, info, cat.  d composed / d image = 1 (composition) or nothing (cat).
    variable_list grads;
    grads.push_back(g_tex);
    for (int l = 0; l < L; ++l) grads.push_back(cat ? Variable() : grad_output[l]);
    for (int l = 0; l < L; ++l) grads.push_back(Variable());
    grads.push_back(Variable());
    grads.push_back(Variable());
    return grads;
}
}  // namespace torch::autograd

void ApplyTangentToPose(torch::Tensor tangent, torch::Tensor pose)
{
    TORCH_CHECK(tangent.is_contiguous() && pose.is_contiguous());
    Check(adop_apply_tangent(tangent.data_ptr<double>(), pose.data_ptr<double>(), (int)tangent.size(0), CurrentStream()));
}

// ---- PointRenderModuleImpl::forward(NeuralRenderInfo*) (RenderModule.cpp:38-144) --------------------------------
std::pair<std::vector<torch::Tensor>, std::vector<torch::Tensor>> PointRenderModuleForward(
    NeuralRenderInfo* nri, PointRendererCache* cache, const PointRenderModuleOptions& opt, bool training)
{
    nri->cache = cache;
    if (!training) nri->params.dropout = 0;  // RenderModule.cpp:25-28
    if (nri->params.super_sampling)
        for (auto& i : nri->images)
        {
            i.w *= 2;
            i.h *= 2;
            i.crop_transform = i.crop_transform.scale(2);
        }
    auto combined = BlendPointCloud(nri);
    std::vector<torch::Tensor> images(combined.begin(), combined.begin() + nri->num_layers);
    std::vector<torch::Tensor> point_masks;
    if (nri->params.output_background_mask)
    {
        TORCH_CHECK((int)combined.size() == nri->num_layers * 2);
        point_masks = std::vector<torch::Tensor>(combined.begin() + nri->num_layers, combined.end());
        for (auto& m : point_masks) m.detach_();
    }
    if (nri->params.super_sampling)
    {
        for (auto& img : images) img = torch::avg_pool2d(img, {2, 2});
        for (auto& img : point_masks) img = torch::avg_pool2d(img, {2, 2});
        for (auto& i : nri->images)
        {
            i.w /= 2;
            i.h /= 2;
            i.crop_transform = i.crop_transform.scale(0.5);
        }
    }
    if (nri->scene->environment_map)
    {
        // EnvironmentMapImpl::Sample + the composition (EnvironmentMap.cu:107-157, RenderModule.cpp:106-127) through
        // the library's fused kernels, with the texture gradient from adop_env_sample_backward
        TORCH_CHECK(nri->params.output_background_mask);
        torch::intrusive_ptr<NeuralRenderInfo> render_data = torch::make_intrusive<NeuralRenderInfo>(*nri);
        // (the lists go in as at::TensorList: that is the type whose elements autograd takes as inputs of the node)
        auto env = torch::autograd::EnvironmentMapCompose::apply(nri->scene->environment_map->texture,
                                                                 at::TensorList(images), at::TensorList(point_masks),
                                                                 torch::IValue(render_data), opt.cat_env_to_color);
        for (int i = 0; i < nri->num_layers; ++i)
            images[i] = opt.cat_env_to_color ? torch::cat({images[i], env[i]}, 1) : env[i];
    }
    if (opt.cat_masks_to_color)
        for (int i = 0; i < nri->num_layers; ++i) images[i] = torch::cat({images[i], point_masks[i]}, 1);
    return {images, point_masks};
}
