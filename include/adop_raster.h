/*
 * adop_raster.h — C-ABI of the MI355X (gfx950) one-pixel point rasterizer.
 *
 * Torch-free boundary: plain device pointers, explicit shapes, POD structs. Every entry point enqueues
 * work on the caller's HIP stream and returns without a device-wide synchronisation; nothing here
 * allocates device memory (the caller passes outputs plus a workspace sized by adop_workspace_size()).
 *
 * Each declaration cites the piece of darglein/ADOP it replaces (paths relative to the ADOP source tree).
 *
 * Tensor layouts are the reference's:
 *   t_position [N,4] f32 (x,y,z,drop_out_radius)    src/lib/rendering/NeuralPointCloudCuda.h:35,82-103
 *   t_normal   [N,1] i32 (3x10-bit packed normal)   NeuralPointCloudCuda.h:37,94-97
 *   t_index    [N,1] i32 (texel of the point)       NeuralPointCloudCuda.h:41,105
 *   texture    [C,N_tex] f32 (channel-major)        src/lib/models/NeuralTexture.h:62-65
 *   background [C] f32
 *   poses_se3  [F,8] f64  (qx,qy,qz,qw,tx,ty,tz,pad) world->camera  src/lib/data/NeuralStructure.cpp:13-27
 *   intrinsics [K,13] f32 (fx,fy,cx,cy,s,k1..k6,p1,p2) or [K,5+P] (c,d,e,cx,cy,world2cam poly)
 *                                                   NeuralStructure.cpp:64-133, PointRenderer.cu:78-96
 *   per level l: depth_l/weight_l/mask_l [B,1,h_l,w_l] f32, out_l [B,C,h_l,w_l] f32,
 *                h_l = h>>l, w_l = w>>l             PointRenderer.cu:996-1018,1045-1071
 */
#ifndef ADOP_RASTER_H
#define ADOP_RASTER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ADOP_MAX_LAYERS 5 /* constexpr int max_layers = 5, PointRenderer.h:20 */

/* Error convention: the reference aborts (SAIGA_ASSERT / device asserts, PointRenderer.cu:1199,362,481).
 * The C-ABI returns a status and keeps a per-thread message instead. */
typedef enum adop_status
{
    ADOP_OK                 = 0,
    ADOP_INVALID_ARG        = 1,
    ADOP_UNSUPPORTED_LAYERS = 2, /* "invalid number of layers", PointRenderer.cu:1199 */
    ADOP_HIP_ERROR          = 3,
    ADOP_WORKSPACE_TOO_SMALL = 4
} adop_status;

/* enum class CameraModel, src/lib/data/SceneData.h:28-32 */
typedef enum adop_camera_model
{
    ADOP_CAMERA_PINHOLE_DISTORTION = 0,
    ADOP_CAMERA_OCAM               = 1
} adop_camera_model;

typedef enum adop_texture_dtype
{
    ADOP_TEXTURE_F32 = 0, /* the reference's only storage type */
    ADOP_TEXTURE_F16 = 1  /* half storage, fp32 accumulation (extension for the 100M-point viewer case) */
} adop_texture_dtype;

/* struct ReducedImageInfo, SceneData.h:37-47 (passed by value to every reference kernel). */
typedef struct adop_view
{
    int32_t w, h;
    int32_t image_index;       /* row of poses_se3 */
    int32_t camera_index;      /* row of intrinsics */
    int32_t camera_model_type; /* adop_camera_model */
    float crop_fx, crop_fy, crop_cx, crop_cy, crop_s; /* IntrinsicsPinholef crop_transform */
} adop_view;

/* struct RenderParams (Settings.h:22-52) as consumed by DeviceRenderParams (PointRenderer.cu:47-117). */
typedef struct adop_render_params
{
    int32_t test_backward_mode;        /* only the value 4 changes behaviour, PointRenderer.cu:543-566 */
    int32_t check_normal;              /* back-face cull, PointRendererHelper.h:59-68 */
    int32_t ghost_gradients;           /* PointRenderer.cu:487-488 */
    int32_t drop_out_points_by_radius; /* PointRenderer.cu:261-264 */
    float depth_accept;                /* fuzzy depth threshold (relative), PointRenderer.cu:380 */
    float drop_out_radius_threshold;
    float dist_cutoff;                 /* pinhole: distortion radius cutoff; OCam: theta cutoff */
    float distortion_gradient_factor;  /* PointRenderer.cu:661 */
    float K_gradient_factor;           /* PointRenderer.cu:647 */
    int32_t output_background_mask;    /* CreateMask is run, PointRenderer.cu:1454-1460 */
    float output_background_mask_value;
    /* 0: NormalizeGradient exactly as the reference launches it (points normalised through a vec3 view of
     *    the [N,4] buffer, intrinsics always as 13 floats per row; PointRenderer.cu:1611-1636).
     * 1: row-wise normalisation (points row i by count i, intrinsics over the real row width). */
    int32_t normalize_mode;
    /* How adop_forward renders (same results either way; no counterpart in the reference):
     * 0: the library chooses; 1: direct (depth prepass and blend with global atomics, PointRenderer.cu:203-393
     * as written); 2: through screen-space tile bins (the fine levels are rendered in LDS).  0 decides by the number
     * of points per pixel of the whole image; when the cloud covers only a small part of the image, 1 is the faster. */
    int32_t forward_path;
    /* 1: adop_forward leaves the point cloud out (RenderParams::render_points == false, Settings.h:25;
     * PointRenderer.cu:1417,1433 skip DepthPrepassMulti and RenderForwardMulti): every pixel is empty and holds the
     * background colour.  adop_backward still runs over the cloud, as the reference's does (:1598-1604), against those
     * empty buffers (and ignores point_cache, which such a forward does not write).  0 (the reference's default,
     * render_points = true): rendered.  A cloud may also be empty (num_points == 0, its pointers may be NULL). */
    int32_t skip_points;
    /* The flags the caller sized the workspace with (adop_workspace_size_for; 0 = adop_workspace_size): how
     * adop_forward and adop_backward lay it out.  No counterpart in the reference. */
    uint32_t workspace_flags;
} adop_render_params;

/* Inputs owned by NeuralScene: NeuralPointCloudCuda + NeuralTexture + PoseModule + IntrinsicsModule. */
typedef struct adop_scene
{
    const float* position;   /* [N,4] */
    const int32_t* normal;   /* [N] or NULL (then check_normal must be 0; NeuralScene.cpp:28) */
    const int32_t* index;    /* [N] */
    int32_t num_points;
    const void* texture;     /* [C,N_tex] f32 or f16 */
    int32_t texture_dtype;   /* adop_texture_dtype */
    int32_t num_channels;    /* C <= 16 */
    int32_t num_texels;      /* N_tex */
    const float* background_color; /* [C] */
    const double* poses_se3; /* [F,8] */
    int32_t num_poses;
    const float* intrinsics; /* [K,intrinsics_cols] */
    int32_t num_cameras;
    int32_t intrinsics_cols;
    /* Caller's promise that index[i] == i for every point and num_texels == num_points (how the reference
     * builds t_index, NeuralPointCloud.h:31).  Lets the backward write grad_texture with plain coalesced stores
     * instead of atomics.  0 = make no assumption. */
    int32_t index_is_identity;
} adop_scene;

/* struct LayerCuda (PointRenderer.h:65-94) plus the per-level output tensors of PointRendererCache
 * (output_forward, output_forward_background_mask; PointRenderer.h:131-132). */
typedef struct adop_layer
{
    int32_t w, h;
    uint64_t* depth_index; /* [B,1,h,w] u64 = (float bits of depth << 32) | point id; PackIndex,
                              PointRendererHelper.h:30-34. Empty pixel: (bits(100000.f) << 32) | 0xFFFFFFFF */
    float* depth;          /* [B,1,h,w] high word of depth_index as f32 (saved for backward) */
    float* weight;         /* [B,1,h,w] */
    float* out;            /* [B,C,h,w] */
    float* mask;           /* [B,1,h,w] or NULL */
} adop_layer;

typedef struct adop_forward_buffers
{
    int32_t num_layers;
    adop_layer layers[ADOP_MAX_LAYERS];
    /* [B,N] f32 in {0,1}; 1 = point is dropped for that image. NULL = nothing dropped. The reference
     * draws it with bernoulli_ inside InitializeData (PointRenderer.cu:1081-1088); here it is an input so
     * that both sides of a parity test see the same mask. */
    const float* dropout_points;
    /* Optional [B,N,4] f32 (no counterpart in the reference, which projects every point again in each of its
     * three kernels): per view and point the level-0 image point (x,y), the depth (0 = culled; sign bit set = the
     * point is dropped for that image, dropout_points) and the LOD radius in pixels (0 when
     * drop_out_points_by_radius is off: nothing reads it then).  adop_forward writes it; adop_backward reads it
     * instead of projecting when the same buffer is passed back in `fwd`, with the same render parameters.  NULL: adop_forward keeps the records in the workspace, adop_backward
     * projects again.  When none of the points i..i+63 (i a multiple of 64) lands in the image of a view at any
     * level, record i of that view holds the bits 0x7FC0C011 in x (and depth 0): adop_backward then skips the run.
     * In a call with several views the other 63 records of such a run are not written (for the first 64 views, and
     * unless counters are collected): they keep whatever the buffer held.  A point outside the image at every level
     * carries a positive depth whatever its dropout flag. */
    float* point_cache;
    /* Optional [B * (w_0 h_0 + ... + w_{L-1} h_{L-1}), C] f32 (no counterpart in the reference): the resolved images
     * once more, pixel by pixel (C consecutive floats; the pixels of level 0 of all B images first, then level 1, ...;
     * inside an image row by row).  The spatial gradients read the image at the four neighbours of a pixel in all
     * channels (PointRenderer.cu:576-611), which the planar [B,C,h,w] layout serves badly.  adop_forward writes it;
     * adop_backward reads it when the same buffer is passed back in `fwd` (its image I is then what that forward pass
     * rendered, whatever happened to `out` since).  NULL: adop_backward builds the records from `out` itself. */
    float* pixel_cache;
} adop_forward_buffers;

/* DeviceBackwardParams (PointRenderer.cu:124-137) + the tensors PointRendererCache::Build(.., false)
 * creates (PointRenderer.cu:922-949). Every non-NULL gradient buffer is cleared by adop_backward. */
typedef struct adop_backward_buffers
{
    const float* grad_out[ADOP_MAX_LAYERS]; /* upstream [B,C,h_l,w_l] */
    float* grad_texture;          /* [C,N_tex] */
    float* grad_background;       /* [C] */
    float* grad_points;           /* [N,4] or NULL */
    float* grad_points_count;     /* [N]   (required iff grad_points) */
    double* grad_pose;            /* [F,6] f64 or NULL */
    float* grad_pose_count;       /* [F] */
    float* grad_intrinsics;       /* [K,intrinsics_cols] or NULL */
    float* grad_intrinsics_count; /* [K] */
} adop_backward_buffers;

/* Counters filled by the kernels (uint64 each), used for the algorithmic byte model. */
typedef struct adop_stats
{
    uint64_t visible[ADOP_MAX_LAYERS];  /* V_l: point-levels that land inside the image */
    uint64_t accepted[ADOP_MAX_LAYERS]; /* A_l: ... that also pass the fuzzy depth test and are blended */
    uint64_t spatial[ADOP_MAX_LAYERS];  /* G_l: ... that receive a ghost / spatial gradient */
    uint64_t bad_index;                 /* texture index out of range (reference: device assert :362) */
} adop_stats;

/* Size in bytes of the workspace adop_forward / adop_backward need for B views (every path, with or without a
 * point_cache: the size adop_workspace_size_for() returns for flags = 0).  It depends on the arguments only, never on
 * the tuning switches below or on the environment. */
size_t adop_workspace_size(const adop_scene* scene, int32_t num_views, int32_t num_layers, int32_t w, int32_t h);

/* A smaller workspace for callers that can promise something (no counterpart in the reference, whose buffers are all
 * torch tensors of its cache).  Per point and view the full workspace holds 8 bytes of backward work queue, 20 bytes
 * that only a forward pass WITHOUT a caller's point_cache uses (the projected points and the candidate lists of the
 * direct path) and 36 bytes that only the tile-bin forward path uses (a tile word and two bin entries):
 *   ADOP_WORKSPACE_POINT_CACHE_KEPT  every adop_forward call passes buffers->point_cache (training): the 20 bytes go;
 *   ADOP_WORKSPACE_NO_TILE_PATH      the forward pass may always take the direct path: the 36 bytes go;
 *   ADOP_WORKSPACE_SMALL_BINS        tile bins for one entry per four points and view instead of two per point and view
 *                                    (8 of the 36 bytes stay): what views take that see a part of the cloud each (the
 *                                    crops of a training batch: 0.07 entries per point and view).  Whether a call's
 *                                    entries fit is known on the device only, after the first binning pass: when they
 *                                    do not, the tile kernels return at once and the direct path's kernels, which are
 *                                    queued behind them in such a workspace (four launches that otherwise return at
 *                                    once), render the call: same results, the time of both first passes.
 * The same flags go into adop_render_params.workspace_flags of every call that uses the workspace: that is how
 * adop_forward and adop_backward lay it out.  Without tile bins the forward pass renders through the direct path (same
 * results; forward_path = 2 is then refused with ADOP_WORKSPACE_TOO_SMALL); with ADOP_WORKSPACE_POINT_CACHE_KEPT a
 * forward call that passes no point_cache is refused (ADOP_INVALID_ARG).
 * 16 crops of a 100 M-point cloud: 102 GB in full, 70 GB with the point cache kept, 25 GB with the cache kept and
 * small bins, 13 GB without bins (plus the 25.6 GB of the point cache itself). */
#define ADOP_WORKSPACE_POINT_CACHE_KEPT 1u
#define ADOP_WORKSPACE_NO_TILE_PATH 2u
#define ADOP_WORKSPACE_SMALL_BINS 4u
size_t adop_workspace_size_for(const adop_scene* scene, int32_t num_views, int32_t num_layers, int32_t w, int32_t h,
                               uint32_t flags);

/* Tuning switches (no counterpart in the reference).  The results never depend on them, only the time a call takes;
 * the defaults are what the measurements on MI355X chose.  One set per process: adop_set_tuning() replaces it (a call
 * that is being issued by another thread at that moment takes every switch either from the old or from the new set),
 * adop_get_tuning() reads it, adop_tuning_defaults() fills in the defaults.  The library reads no environment
 * variable.  Fields set to -1 mean "the library decides". */
typedef struct adop_tuning
{
    int32_t forward_path;       /* used when adop_render_params.forward_path is 0: 0 = by size (default), 1 = direct, 2 = tile bins */
    int32_t tile_slice_entries; /* entries per slice of a split bin; a bin is split from four slices' worth on (8192) */
    int32_t ghost_concurrent;   /* several views (at most 24): 1 = the spatial gradients of all views in one launch, 0 = one
                                   launch per view, -1 (default) = one launch for crop windows and clouds up to 4 M points */
    int32_t bin_shard_shift;    /* log2 of the counters per tile in the binning passes, 0..3; -1 (default) = by the tile
                                   count (up to 8 while the call has at most 4096 tiles and 16384 counters).  A value
                                   that would need more than 65536 counters is lowered until it does not. */
    int32_t direct_lists;       /* direct path without a caller's point cache: 1 = candidate lists (default), 0 = none, the blend projects again */
    int32_t prepass_ppt;        /* points per thread of the direct path's depth prepass: 1, 2, 4; 0 (default) = by the cloud size */
    int32_t prepass_group_from; /* first level at which the depth prepass merges the lanes of a wavefront by pixel (1) */
    int32_t blend_group_from;   /* the same for the direct path's blend (0) */
    int32_t list_block;         /* workgroup size of the direct path's blend in list mode: 64, 128 (default), 256 */
    int32_t count_ppt;          /* points per thread of the first binning pass: 1, 2, 4; 0 (default) = 1 up to 2^22 points, 2 above */
    int32_t scatter_ppt;        /* points per thread of the second binning pass: 1, 2 (default), 4 */
    int32_t tile_k;             /* entries per thread and batch of the tile blend: 1 (default), 2, 4 */
    int32_t normalize_fused;    /* one view: 1 (default) = the spatial-gradient kernel writes the point gradients
                                   normalised, 0 = a pass of the finalize kernel does */
    int32_t normalize_by_queue; /* one view, normalize_fused = 0: 1 (default) = that pass walks the work queue, 0 = all points */
} adop_tuning;
void adop_tuning_defaults(adop_tuning* out);
adop_status adop_set_tuning(const adop_tuning* tuning); /* ADOP_INVALID_ARG (and no change) when a field is out of range */
void adop_get_tuning(adop_tuning* out);

/* Replaces BlendPointCloudForward (PointRenderer.cu:1389-1531): InitializeData (:1039-1090),
 * DepthPrepassMulti (:203-301,1166-1203), RenderForwardMulti (:303-393,1294-1335),
 * CombineAndFill (:726-754,1268-1291), CreateMask (:828-847,1371-1387).
 * `stats` may be NULL; if not, it is a device pointer that receives adop_stats (forward fields). */
adop_status adop_forward(const adop_scene* scene, const adop_view* views, int32_t num_views,
                         const adop_render_params* params, const adop_forward_buffers* buffers, void* workspace,
                         size_t workspace_bytes, adop_stats* stats, void* hip_stream);

/* Replaces BlendPointCloudBackward (PointRenderer.cu:1549-1644): CombineAndFillBackward (:851-900),
 * RenderBackward (:396-724), NormalizeGradient (:1534-1547,1611-1636). `fwd` holds depth/weight/out as
 * left by adop_forward (the reference's saved variables, :1517-1525). */
adop_status adop_backward(const adop_scene* scene, const adop_view* views, int32_t num_views,
                          const adop_render_params* params, const adop_forward_buffers* fwd,
                          const adop_backward_buffers* grads, void* workspace, size_t workspace_bytes,
                          adop_stats* stats, void* hip_stream);

/* Replaces EnvironmentMapImpl::Sample (EnvironmentMap.cu:107-157: BuildSphericalUV + grid_sample bilinear /
 * border / align_corners) fused with the composition images += (1-mask)*env (RenderModule.cpp:121-125).
 * env_texture [C,eh,ew] f32. For level l: uv_l [B,h_l,w_l,2] (may be NULL), env_l [B,C,h_l,w_l] (may be NULL).
 * add_to_out = 0: env_l receives the samples, uv_l the coordinates of every pixel.  With 1 or 2 only the pixels the
 * composition samples (mask_l != 1) are computed: uv_l is written there only (the rest keeps what the buffer held;
 * adop_env_sample_backward reads no other), env_l is 0 elsewhere.
 * 1: out_l += (1 - mask_l) * env in place (env_l, if given, the samples).
 * 2: env_l receives the composed image out_l + (1 - mask_l) * env and out_l is left alone, as the reference composes
 * (RenderModule.cpp:121-125): adop_backward reads out_l as the image its spatial gradients see, so a training step
 * that composes in place before its backward pass shows them the environment at the empty pixels as well.
 * Pinhole views: the pixel's ray as in BuildSphericalUV (EnvironmentMap.cu:82-90: unproject2 through crop and K,
 * undistortNormalizedPointSimple).  OCam views (the reference asserts pinhole, EnvironmentMap.cu:129; this is an
 * extension): the ray comes from inverting the world2cam polynomial of the intrinsics row itself (no cam2world
 * polynomial is passed): the affine map (c,d,e,cx,cy) is undone, poly(theta) = rho is solved by 5 Newton steps from
 * the optical axis (theta = -pi/2) with theta kept in [-pi/2, pi/2], and the camera-space ray is
 * (cos(theta) * (uu,vv)/rho, -sin(theta)), i.e. the inverse of ProjectOCam (PointRendererHelper.h:85-106) wherever the
 * polynomial is monotonic; pixels the polynomial does not reach take the ray of the nearest end of that range.
 * Everything after the ray (rotation to world space, SphericalCoordinates, sampling) is EnvironmentMap.cu:41-105. */
adop_status adop_env_sample(const adop_scene* scene, const adop_view* views, int32_t num_views,
                            const float* env_texture, int32_t env_h, int32_t env_w, const adop_forward_buffers* buffers,
                            float* const* uv_levels, float* const* env_levels, int32_t add_to_out, void* hip_stream);

/* Gradient of adop_env_sample w.r.t. env_texture: grad_env [C,eh,ew] = sum over pixels of
 * (1-mask) * grad_out * bilinear weights (torch autograd of grid_sample in the reference; grad_env is cleared first).
 * uv_levels: NULL, or per level the uv_l [B,h_l,w_l,2] that adop_env_sample wrote for these views (the reference's
 * autograd keeps the sampling grid the same way): the kernel then reads the texture coordinates instead of computing
 * each pixel's ray again. */
adop_status adop_env_sample_backward(const adop_scene* scene, const adop_view* views, int32_t num_views,
                                     int32_t env_h, int32_t env_w, const adop_forward_buffers* buffers,
                                     const float* const* grad_out_levels, const float* const* uv_levels,
                                     float* grad_env, void* hip_stream);

/* Replaces ApplyTangentToPose / ApplyTangent (PointRenderer.cu:1646-1665): pose = se3_exp(tangent) * pose,
 * tangent = 0; f64. tangent [F,6], poses_se3 [F,8]. */
adop_status adop_apply_tangent(double* tangent, double* poses_se3, int32_t num_poses, void* hip_stream);

/* Point-cloud preprocessing (the rasterizer's speed depends on it: the LOD radius of every point and the order of
 * the cloud).  Replaces the host-side kd-tree search of SceneData::ComputeRadius (SceneData.cpp:441-484):
 * out_distance[i] = distance from point i to its `rank`-th nearest other point (the reference asks its tree for the
 * rank + 1 nearest, which include the point itself, and takes the last; rank = 4 there, 1..8 here), computed as
 * sqrt((dx*dx + dy*dy) + dz*dz) in fp32.  position [N,4] f32 (xyz used), N > rank; bbox_min / bbox_max: host
 * float[3], a box that contains the cloud (the search lays its grids over the bulk of the cloud inside it; points
 * far from the rest cost a scan of all points each). */
size_t adop_knn_workspace_size(int32_t num_points);
adop_status adop_knn_distance(const float* position, int32_t num_points, int32_t rank, const float* bbox_min,
                              const float* bbox_max, float* out_distance, void* workspace, size_t workspace_bytes,
                              void* hip_stream);

/* Replaces SceneData::PointDistanceToCamera (SceneData.cpp:645-669): out_distance[i] = distance from point i to
 * the nearest camera that sees it (z > 0 and the projection through the frame's pinhole + distortion model,
 * FrameData::Project3 :26-34, inside [0,w) x [0,h)); sqrt(105235545) where no frame does.  `frames`: one adop_view
 * per frame (w, h, image_index, camera_index; the crop transform is not used); scene: position, poses_se3,
 * intrinsics [K,13].  Workspace: adop_frames_workspace_size(num_frames) bytes. */
size_t adop_frames_workspace_size(int32_t num_frames);
adop_status adop_point_distance_to_camera(const adop_scene* scene, const adop_view* frames, int32_t num_frames,
                                          float* out_distance, void* workspace, size_t workspace_bytes,
                                          void* hip_stream);

/* adop_point_distance_to_camera without a workspace, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The
 * per-frame constants live in an array inside the library (132 bytes per frame, adop_static_max_frames() = 1024
 * frames = 132 KiB per GPU, held until the process ends); more frames are rejected with ADOP_INVALID_ARG.  The call
 * allocates and frees nothing; the first call on a device looks the array's address up (make that call outside a
 * stream capture).  All calls on one GPU share the array: calls that overlap on one GPU (different streams or
 * threads) race; calls on one stream are ordered and safe.  Results equal adop_point_distance_to_camera's. */
int32_t adop_static_max_frames(void);
adop_status adop_point_distance_to_camera_static(const adop_scene* scene, const adop_view* frames, int32_t num_frames,
                                                 float* out_distance, void* hip_stream);

/* Replaces the sequential sweep of SceneData::RemoveClosePoints (SceneData.cpp:598-642): state[i] = 2 (erased) when a
 * point j < i with state[j] = 1 (kept) lies closer than radius[i] (d2 < radius^2 in fp32), else 1; the result equals
 * the sweep in index order.  The points are decided in rounds (a point waits for its earlier neighbours):
 * round_undecided [num_rounds] (device) receives the number of points still 0 (undecided) after every round; when
 * the last entry is not 0 call again with resume = 1 and the workspace untouched.  state [N] int32 (device),
 * radius [N] f32, workspace: adop_knn_workspace_size(num_points) bytes. */
adop_status adop_close_points(const float* position, int32_t num_points, const float* radius, const float* bbox_min,
                              const float* bbox_max, int32_t* state, uint32_t* round_undecided, int32_t num_rounds,
                              int32_t resume, void* workspace, size_t workspace_bytes, void* hip_stream);

/* The sort key of PointCloud::ReorderMorton64 (SceneData.cpp:101): out_codes[i] = 63-bit Morton code of point i, 21
 * bits per axis of its position inside the bounding box (x in the lowest bit).  position [N,4] f32, out_codes [N] u64. */
adop_status adop_morton_codes(const float* position, int32_t num_points, const float* bbox_min, const float* bbox_max,
                              uint64_t* out_codes, void* hip_stream);

/* Stage timers.  The reference wraps each stage in SAIGA_OPTIONAL_TIME_MEASURE(name, info->timer_system)
 * (PointRenderer.cu:906,913,919,1095,1414,1430,1447,1565,1594,1602,1610); here HIP events are recorded on the
 * caller's stream around each stage while profiling is enabled on the calling thread.  Stage names are the
 * reference's: "Initialize", "DepthPrepass", "RenderForward", "CombineAndFill", "Prepare Backward",
 * "CombineAndFillBackward", "RenderBackward/descriptor" and "RenderBackward/spatial" (the two kernels RenderBackward is
 * split into), "Post Process Gradient".  When the forward runs through the tile bins (forward_path 2), "DepthPrepass"
 * and "RenderForward" are replaced by "BinCount", "BinScatter", "TileDepth" and "TileBlend". */
typedef struct adop_stage_time
{
    char name[32];
    float total_ms; /* summed over calls since the last read */
    int32_t calls;
} adop_stage_time;

adop_status adop_profile_enable(int32_t enable);
/* Waits for the recorded events, aggregates them by stage name into out[0..max_entries) and clears the
 * recording.  Returns the number of entries written.  Which calls are recorded is a switch of the thread that issues
 * them (adop_profile_enable); what they record goes to one list of the process, which this call takes whole, whatever
 * thread it is called from (a framework may run the backward pass on a thread of its own). */
int32_t adop_profile_read(adop_stage_time* out, int32_t max_entries);

/* Message for the last non-OK status returned on the calling thread. */
const char* adop_last_error_string(void);

/* Library version / build identification. */
const char* adop_version(void);

#ifdef __cplusplus
}
#endif
#endif /* ADOP_RASTER_H */
