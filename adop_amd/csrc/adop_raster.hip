// adop_raster.hip — C-ABI of the one-pixel point rasterizer and the launch sequences (gfx950 / CDNA4).
//
// One forward call (reference: BlendPointCloudForward, PointRenderer.cu:1389-1531) runs one of two paths
// (adop_render_params.forward_path; 0 lets the library choose).
// Tile path (binned_kernels.hip, tile_kernels.hip):
//   clear           depth_index / blend accumulators of the coarse levels, tile counters; one workgroup also turns
//                   poses_se3 (f64) / intrinsics rows into the per-view constants          (InitializeData :1039-1090)
//   bin_count       per point: projection (kept as the point cache), entries per 16x16-pixel screen tile
//   tile_scan       prefix sum of the tile counts
//   bin_scatter     per point: 16-byte entry into the bin of its tile (and of the tile of its level-1 pixel)
//   tile_depth      per tile: 64-bit min of (depth bits | point id) in LDS, levels 0-1 owned, coarser ones merged
//                   with global atomics                                                     (DepthPrepassMulti :203-301)
//   tile_blend      per tile: fuzzy depth test, per-pixel lists in LDS, gather; levels 0-1 resolved to the outputs,
//                   coarser levels added to the accumulators                                (RenderForwardMulti :303-393)
//   resolve         coarse levels: out = sum/weight or background, weight, mask, f32 depth (:726-754,:828-847)
// Direct path (forward_kernels.hip): clear, prepass (per point/view/level: pre-reduced 64-bit atomicMin), blend (per
// point: fuzzy depth test, pre-reduced descriptor sums, one cache-line atomic per pixel), resolve.
// One backward call (BlendPointCloudBackward, :1549-1644; backward_kernels.hip):
//   interleave      per pixel: background-gradient partial sums (CombineAndFillBackward :851-900), the pixel-major
//                   [image | upstream gradient] array and (depth, weight) pairs the next kernels gather from; one
//                   workgroup computes the per-view constants
//   backward_tex    per point, all views in one pass: depth tests, descriptor gradient (written once), which levels get
//                   a ghost / spatial gradient (RenderBackward :396-489); appends those points to a work queue per
//                   view, or, for small clouds, per group of twelve views
//   backward_ghost  per queue item (one launch per view or per group): four-neighbour gather, image-space gradient,
//                   ProjectPoint*Backward (:491-724); pose / intrinsics sums per thread in fp32, per workgroup in f64,
//                   one partial row per workgroup and view
//   finalize        partial rows -> grad_background / grad_pose / grad_intrinsics, NormalizeGradient (:1534-1547) of
//                   all outputs (one view: the point gradients by walking the work queue)
//
// No MFMA anywhere: the path is scan + scatter/gather + atomics, bounded by HBM and atomic transaction rate.
#include <hip/hip_runtime.h>

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/adop_raster.h"
#include "common.h"
#include "launch.h"

#pragma clang fp contract(off)

namespace adop
{
thread_local std::string g_last_error;

adop_status fail(adop_status s, const std::string& msg)
{
    g_last_error = msg;
    return s;
}

#define ADOP_HIP_CHECK(expr)                                                                             \
    do                                                                                                   \
    {                                                                                                    \
        hipError_t e_ = (expr);                                                                          \
        if (e_ != hipSuccess)                                                                            \
            return fail(ADOP_HIP_ERROR, std::string(#expr) + ": " + hipGetErrorString(e_));              \
    } while (0)

// Stage timers: HIP events recorded on the caller's stream around each kernel launch when profiling is enabled
// on the calling thread (the reference's SAIGA_OPTIONAL_TIME_MEASURE scopes, PointRenderer.cu:906-1610).
struct StageEvent
{
    const char* name;
    hipEvent_t start, stop;
};
// Which calls are recorded is a switch of the calling thread; the recorded events go to one list of the process, so
// that a thread can read what another thread's calls recorded (a framework may run the backward pass on a thread of
// its own: torch's autograd engine does).
thread_local bool g_profile = false;
std::mutex g_stage_mutex;
std::vector<StageEvent> g_stage_events;
std::vector<hipEvent_t> g_event_pool;

hipEvent_t take_event()  // (g_stage_mutex held)
{
    if (!g_event_pool.empty())
    {
        hipEvent_t e = g_event_pool.back();
        g_event_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
}

struct StageScope
{
    hipStream_t st;
    hipEvent_t stop = nullptr;
    StageScope(const char* name, hipStream_t s) : st(s)
    {
        if (!g_profile) return;
        std::lock_guard<std::mutex> lock(g_stage_mutex);
        hipEvent_t a = take_event(), b = take_event();
        if (!a || !b) return;
        (void)hipEventRecord(a, st);
        g_stage_events.push_back({name, a, b});
        stop = b;
    }
    ~StageScope()
    {
        if (stop) (void)hipEventRecord(stop, st);
    }
};

// The process's tuning switches: one atomic word per field, so that a call being issued while another thread replaces
// the set reads every switch whole (from the old or from the new set).
constexpr int kTuningFields = sizeof(adop_tuning) / sizeof(int32_t);
static_assert(sizeof(adop_tuning) == kTuningFields * sizeof(int32_t), "adop_tuning holds int32 fields only");
constexpr adop_tuning kTuningDefaults = {/*forward_path*/ 0,    /*tile_slice_entries*/ kSliceEntries,
                                         /*ghost_concurrent*/ -1, /*bin_shard_shift*/ -1,
                                         /*direct_lists*/ 1,    /*prepass_ppt*/ 0,
                                         /*prepass_group_from*/ 1, /*blend_group_from*/ 0,
                                         /*list_block*/ 128,    /*count_ppt*/ 0,
                                         /*scatter_ppt*/ 2,     /*tile_k*/ 1,
                                         /*normalize_fused*/ 1, /*normalize_by_queue*/ 1};
struct TuningStore
{
    std::atomic<int32_t> f[kTuningFields];
    TuningStore()
    {
        const int32_t* d = (const int32_t*)&kTuningDefaults;
        for (int k = 0; k < kTuningFields; ++k) f[k].store(d[k], std::memory_order_relaxed);
    }
};
TuningStore g_tuning;

adop_tuning tuning_now()
{
    adop_tuning t;
    int32_t* d = (int32_t*)&t;
    for (int k = 0; k < kTuningFields; ++k) d[k] = g_tuning.f[k].load(std::memory_order_relaxed);
    return t;
}

struct WorkspaceLayout
{
    size_t views;       // ViewConst[B]
    size_t bg_partial;  // double[kBgBlocks * kMaxChannels]
    size_t pt_partial;  // double[B * kPartialBlocks * kPartialStride]
    size_t scratch;     // double[num_poses*7 + num_cameras*(cols+1)]
    size_t fin_mini;    // double[kFinalizeParts * (kMaxChannels + B * kPartialStride)]: first-stage rows of finalize
    size_t pixels;      // float[B * P * max(S, 2C)]: blend accumulators (forward) / [I|G] array (backward)
    size_t dw;          // float2[B * P]: (depth, weight) per pixel for the backward descriptor pass
    size_t q_counts;    // uint32[B][kNumQueues]: one set of sub-queue counters per view; + the finalize ticket
    size_t q_items;     // uint64[B][kNumQueues * q_cap]
    uint32_t q_cap;
    size_t proj;        // float4[B * list_stride]: projected points of the forward pass when the caller keeps no point_cache
    size_t list_stride; // N rounded up to whole prepass workgroups
    size_t list_ids;    // uint32[B * list_stride]: candidate lists of the direct forward path (records in proj)
    size_t list_count;  // uint32[B * 4 * ceil(N / 256)]
    size_t bin_count;   // uint32[max tiles]           tile bins of the forward pass
    size_t bin_offset;  // uint32[max tiles + 1]
    size_t bin_order;   // uint4[max tiles + slice_rows()]
    size_t bin_rows;    // float[slice_rows()][slice_row_floats()]: partial results of the slices of split bins
    size_t bin_info;    // uint32[B * N]
    size_t bin_entries; // float4[kTileLevels * B * N]
    size_t bin_cap;     // entries
    size_t bin_overflow;  // uint32: set by the prefix sum when the call has more entries than bin_cap
    size_t common;      // end of what every call uses (all that adop_backward needs)
    bool has_lists, has_bins;
    size_t total;
};

constexpr int kTileLevels = 2;  // levels the tile path renders in LDS (a point has at most one bin entry per such level)
constexpr int kTilePathMinPoints = 1 << 16;
constexpr int kTilePathMaxPointsPerPixel = 16;
constexpr int kWindowCloudShare = 16;  // a crop window is taken to see 1/16 of the cloud
// A tile is one workgroup from its first entry to its last: a call with few tiles leaves most of the GPU idle in the
// tile kernels, whose time per point then grows like 1 / tiles (measured on Morton-ordered clouds, forward:
// 18 us per million points from ~4 000 tiles up, 75 us at 1 024 tiles, 180 us at 256; the direct path: 26 us whatever
// the image), while the direct path pays ~15 us more per call for its accumulators of all levels.
constexpr int kTilePathMinTiles = 512;       // below: the direct path (256 tiles: 1.2 to 3 x faster from 100 k points up)
constexpr int kTilePathEnoughTiles = 2800;   // from here on the tile path is the faster one per point
constexpr double kTilePathUsPerMTiles = 73728.0;  // us per million points x tiles of the call
constexpr double kDirectPathUsPerM = 26.0, kDirectPathFixedUs = 15.0;
constexpr int kConcurrentMaxPoints = 4000000;  // backward: full views of a larger cloud get a spatial-gradient launch each

size_t max_tiles(int B, int w0, int h0)
{
    size_t tx = (((size_t)(w0 > 0 ? w0 : 1) - 1) >> kTileShiftX) + 1;
    size_t ty = (((size_t)(h0 > 0 ? h0 : 1) - 1) >> kTileShiftY) + 1;
    return tx * ty * (size_t)B;
}

// floats per pixel of the blend accumulators: C sums + the weight, padded to a power of two so that the group
// of lanes flushing one pixel never straddles a cache line
int accum_stride(int C)
{
    int s = 1;
    while (s < C + 1) s *= 2;
    return s;
}

size_t pyramid_pixels(int L, int w, int h)
{
    size_t p = 0;
    for (int l = 0; l < L; ++l)
    {
        p += (size_t)(w > 0 ? w : 0) * (size_t)(h > 0 ? h : 0);
        w /= 2;
        h /= 2;
    }
    return p;
}

size_t align_up(size_t v, size_t a)
{
    return (v + a - 1) / a * a;
}

constexpr uint32_t kWorkspaceFlags =
    ADOP_WORKSPACE_POINT_CACHE_KEPT | ADOP_WORKSPACE_NO_TILE_PATH | ADOP_WORKSPACE_SMALL_BINS;

// Can the tile path take a cloud of n points in B views of w0 x h0?  (Point ids need 28 bits of the bin entry, the bin
// offsets are 32-bit with at most kTileLevels entries per point and view, the tile word holds 24 bits of tile.)
bool can_bin(long long n, int B, int w0, int h0)
{
    return n > 0 && n < (1ll << 28) && (size_t)kTileLevels * (size_t)B * (size_t)n < ((size_t)1 << 32) &&
           max_tiles(B, w0, h0) < ((size_t)1 << 24);
}

// flags: ADOP_WORKSPACE_*.  What every call uses comes first (the backward pass uses nothing else), then what a forward
// pass without a caller's point cache uses, then the tile bins; the last two may be left out, and the bins are when
// the tile path cannot take the cloud anyway (can_bin).
WorkspaceLayout layout(const adop_scene* s, int B, int L, int w0, int h0, uint32_t flags = 0)
{
    WorkspaceLayout w;
    memset(&w, 0, sizeof(w));
    const size_t n = (size_t)(s->num_points > 0 ? s->num_points : 0);
    size_t o     = 0;
    w.views      = o;
    o            = align_up(o + sizeof(ViewConst) * (size_t)B, 256);
    w.bg_partial = o;
    o            = align_up(o + sizeof(double) * kBgBlocks * kMaxChannels, 256);
    w.pt_partial = o;
    o            = align_up(o + sizeof(double) * (size_t)B * kPartialBlocks * kPartialStride, 256);
    w.scratch    = o;
    o = align_up(o + sizeof(double) * ((size_t)s->num_poses * 7 + (size_t)s->num_cameras * (s->intrinsics_cols + 1)),
                 256);
    w.fin_mini = o;
    o = align_up(o + sizeof(double) * kFinalizeParts * (kMaxChannels + (size_t)B * kPartialStride), 256);
    w.pixels = o;
    int per  = accum_stride(s->num_channels) > 2 * s->num_channels ? accum_stride(s->num_channels) : 2 * s->num_channels;
    o        = align_up(o + sizeof(float) * (size_t)B * pyramid_pixels(L, w0, h0) * (size_t)per, 256);
    w.dw = o;
    o    = align_up(o + sizeof(float2) * (size_t)B * pyramid_pixels(L, w0, h0), 256);
    // backward work queue: workgroup k of backward_tex_kernel appends to sub-queue k % kNumQueues
    size_t blocks = (n + kBlock - 1) / kBlock;
    w.q_cap       = (uint32_t)(((blocks + kNumQueues - 1) / kNumQueues) * kBlock);
    if (w.q_cap == 0) w.q_cap = kBlock;
    w.q_counts = o;
    o          = align_up(o + sizeof(uint32_t) * ((size_t)B * kNumQueues + 1), 256);
    w.q_items  = o;
    o          = align_up(o + sizeof(unsigned long long) * (size_t)B * kNumQueues * w.q_cap, 256);
    w.common   = o;
    // (a view's slots are rounded up to whole prepass workgroups of at most 4 * kBlock points: list mode)
    const size_t n_pad = ((n + 4 * kBlock - 1) / (4 * kBlock)) * (4 * kBlock);
    w.list_stride = n_pad;
    w.has_lists   = (flags & ADOP_WORKSPACE_POINT_CACHE_KEPT) == 0;
    if (w.has_lists)
    {
        w.proj       = o;
        o            = align_up(o + sizeof(float4) * (size_t)B * n_pad, 256);
        w.list_ids   = o;
        o            = align_up(o + sizeof(uint32_t) * (size_t)B * n_pad, 256);
        w.list_count = o;
        o            = align_up(o + 4 * sizeof(uint32_t) * (size_t)B * ((n + kBlock - 1) / kBlock), 256);
    }
    w.has_bins = (flags & ADOP_WORKSPACE_NO_TILE_PATH) == 0 && can_bin((long long)n, B, w0, h0);
    if (w.has_bins)
    {
        size_t T     = max_tiles(B, w0, h0);
        w.bin_count  = o;  // followed by the row counter and the tickets of the split bins: one range to clear
        const size_t max_rows = (size_t)slice_rows((long long)n, B);
        const size_t counters = bin_counter_capacity(T);
        o            = align_up(o + sizeof(uint32_t) * (counters + 1 + 2 * max_rows), 256);
        w.bin_offset = o;
        o            = align_up(o + sizeof(uint32_t) * (counters + 1), 256);
        w.bin_order  = o;
        o            = align_up(o + sizeof(uint4) * (T + max_rows), 256);
        w.bin_rows   = o;
        o            = align_up(o + sizeof(float) * max_rows * (size_t)slice_row_floats(s->num_channels > 0 ? s->num_channels : 1), 256);
        // every entry the call can have, or (ADOP_WORKSPACE_SMALL_BINS) one per four points and view: what views take
        // that see a part of the cloud each; a call with more falls back to the direct path on the device
        w.bin_cap = (size_t)kTileLevels * (size_t)B * n;
        if (flags & ADOP_WORKSPACE_SMALL_BINS) w.bin_cap = ((size_t)B * n + 3) / 4 + 1024;
        w.bin_overflow = o;
        o              = align_up(o + sizeof(uint32_t), 256);
        w.bin_info   = o;
        o            = align_up(o + sizeof(uint32_t) * (size_t)B * n, 256);
        w.bin_entries = o;
        o            = align_up(o + sizeof(float4) * w.bin_cap, 256);
    }
    w.total      = o;
    return w;
}

adop_status validate(const adop_scene* s, const adop_view* views, int B, const adop_render_params* rp,
                     const adop_forward_buffers* fb)
{
    if (!s || !views || !rp || !fb) return fail(ADOP_INVALID_ARG, "null argument");
    if (B < 1) return fail(ADOP_INVALID_ARG, "num_views must be >= 1");  // SAIGA_ASSERT(num_batches > 0), :909
    if (fb->num_layers < 1 || fb->num_layers > ADOP_MAX_LAYERS)
        return fail(ADOP_UNSUPPORTED_LAYERS, "invalid number of layers");  // :1199
    if (s->num_points < 0 || (s->num_points > 0 && (!s->position || !s->index)))
        return fail(ADOP_INVALID_ARG, "point cloud missing");
    if (s->num_points > (1 << 30)) return fail(ADOP_INVALID_ARG, "at most 2^30 points per call");
    if (rp->check_normal && !s->normal && s->num_points > 0)
        return fail(ADOP_INVALID_ARG, "check_normal requires normals");  // NeuralScene.cpp:28
    if (s->num_channels < 1 || s->num_channels > kMaxChannels)
        return fail(ADOP_INVALID_ARG, "num_channels must be in [1,16]");
    if (!s->texture || s->num_texels < 1 || !s->background_color) return fail(ADOP_INVALID_ARG, "texture missing");
    if (s->texture_dtype != ADOP_TEXTURE_F32 && s->texture_dtype != ADOP_TEXTURE_F16)
        return fail(ADOP_INVALID_ARG, "unknown texture dtype");
    if (!s->poses_se3 || !s->intrinsics || s->num_poses < 1 || s->num_cameras < 1)
        return fail(ADOP_INVALID_ARG, "poses / intrinsics missing");
    if (s->intrinsics_cols < 5 || s->intrinsics_cols > kMaxIntrinsicsCols)
        return fail(ADOP_INVALID_ARG, "intrinsics_cols out of range");
    if (s->index_is_identity && s->num_texels != s->num_points)
        return fail(ADOP_INVALID_ARG, "index_is_identity needs num_texels == num_points");
    int w = views[0].w, h = views[0].h;
    for (int b = 0; b < B; ++b)
    {
        const adop_view& v = views[b];
        if (v.w != w || v.h != h) return fail(ADOP_INVALID_ARG, "all views of a batch must have the same size");
        if (v.image_index < 0 || v.image_index >= s->num_poses)
            return fail(ADOP_INVALID_ARG, "image_index out of range");  // :232,1172
        if (v.camera_index < 0 || v.camera_index >= s->num_cameras)
            return fail(ADOP_INVALID_ARG, "camera_index out of range");
        if (v.camera_model_type == ADOP_CAMERA_PINHOLE_DISTORTION)
        {
            if (s->intrinsics_cols != 13) return fail(ADOP_INVALID_ARG, "pinhole intrinsics need 13 columns");
        }
        else if (v.camera_model_type == ADOP_CAMERA_OCAM)
        {
            if (s->intrinsics_cols < 6) return fail(ADOP_INVALID_ARG, "OCam intrinsics need >= 6 columns");
        }
        else
            return fail(ADOP_INVALID_ARG, "unknown camera model");
    }
    for (int l = 0; l < fb->num_layers; ++l)
    {
        const adop_layer& L = fb->layers[l];
        if (L.w != w || L.h != h || w <= 0 || h <= 0)
            return fail(ADOP_INVALID_ARG, "layer sizes must be w>>l, h>>l and positive");  // :996-1018
        if (!L.depth_index || !L.depth || !L.weight || !L.out) return fail(ADOP_INVALID_ARG, "layer buffer missing");
        w /= 2;
        h /= 2;
    }
    size_t per_image = 0;
    for (int l = 0; l < fb->num_layers; ++l) per_image += (size_t)fb->layers[l].w * fb->layers[l].h;
    if (per_image * (size_t)B >= (size_t)1 << 31) return fail(ADOP_INVALID_ARG, "too many pixels");
    if ((size_t)views[0].w * views[0].h >= (size_t)1 << 28) return fail(ADOP_INVALID_ARG, "image too large");
    return ADOP_OK;
}

Levels make_levels(const adop_scene* s, int B, const adop_forward_buffers* fb, const adop_backward_buffers* gb)
{
    Levels lv;
    memset(&lv, 0, sizeof(lv));
    lv.num = fb->num_layers;
    lv.B   = B;
    lv.C   = s->num_channels;
    int acc = 0;
    for (int l = 0; l < fb->num_layers; ++l)
    {
        const adop_layer& L = fb->layers[l];
        lv.pix_prefix[l]    = acc;
        acc += L.w * L.h;
        lv.l[l].w           = L.w;
        lv.l[l].h           = L.h;
        lv.l[l].depth_index = L.depth_index;
        lv.l[l].depth       = L.depth;
        lv.l[l].weight      = L.weight;
        lv.l[l].out         = L.out;
        lv.l[l].mask        = L.mask;
        lv.l[l].gin         = gb ? gb->grad_out[l] : nullptr;
    }
    for (int l = fb->num_layers; l <= ADOP_MAX_LAYERS; ++l) lv.pix_prefix[l] = acc;
    lv.irec       = fb->pixel_cache;  // (adop_backward: the workspace when the caller kept none)
    lv.irec_ready = fb->pixel_cache != nullptr;
    return lv;
}

CloudArg make_cloud(const adop_scene* s, const adop_forward_buffers* fb)
{
    CloudArg c;
    c.position   = (const float4*)s->position;
    c.normal     = s->normal;
    c.index      = s->index;
    c.n          = s->num_points;
    c.texture    = s->texture;
    c.num_texels = s->num_texels;
    c.intrinsics = s->intrinsics;
    c.dropout    = fb->dropout_points;
    c.cache      = (float4*)fb->point_cache;
    c.list_ids   = nullptr;
    c.list_count = nullptr;
    c.list_span  = 0;
    c.list_stride = 0;
    return c;
}

ParamArg make_params(const adop_render_params* rp)
{
    ParamArg p;
    p.test_backward_mode         = rp->test_backward_mode;
    p.check_normal               = rp->check_normal;
    p.ghost_gradients            = rp->ghost_gradients;
    p.drop_by_radius             = rp->drop_out_points_by_radius;
    p.depth_accept               = rp->depth_accept;
    p.drop_threshold             = rp->drop_out_radius_threshold;
    p.dist_cutoff                = rp->dist_cutoff;
    p.distortion_gradient_factor = rp->distortion_gradient_factor;
    p.K_gradient_factor          = rp->K_gradient_factor;
    return p;
}

// The per-view constants: up to 32 views go into *fused, for the first kernel of the call to compute; more views
// (or no fused kernel) take prepare_views launches.
adop_status upload_views(const adop_scene* s, const adop_view* views, int B, ViewConst* dst, hipStream_t st,
                         ViewPrep* fused = nullptr)
{
    if (fused)
    {
        memset(fused, 0, sizeof(*fused));
        if (B <= 32)
        {
            for (int k = 0; k < B; ++k) fused->chunk.v[k] = views[k];
            fused->count      = B;
            fused->cols       = s->intrinsics_cols;
            fused->poses      = s->poses_se3;
            fused->intrinsics = s->intrinsics;
            fused->out        = dst;
            return ADOP_OK;
        }
    }
    for (int first = 0; first < B; first += 32)
    {
        ViewChunk ch;
        memset(&ch, 0, sizeof(ch));
        int count = B - first < 32 ? B - first : 32;
        for (int k = 0; k < count; ++k) ch.v[k] = views[first + k];
        launch_prepare_views(ch, first, count, s->poses_se3, s->intrinsics, s->intrinsics_cols, dst, st);
    }
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

adop_status fill_async(void* p, size_t bytes, uint32_t v, hipStream_t st)
{
    if (!p || bytes == 0) return ADOP_OK;
    launch_fill_u32((uint32_t*)p, bytes / 4, v, st);
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

int pixel_grid(const Levels& lv, int first_level = 0)
{
    size_t total = (size_t)(lv.pix_prefix[lv.num] - lv.pix_prefix[first_level]) * lv.B;
    size_t want  = (total + kBlock - 1) / kBlock;
    return (int)(want < 16384 ? (want ? want : 1) : 16384);
}

}  // namespace adop

// Scratch memory of the one entry point that takes no workspace (adop_point_distance_to_camera_static): the per-frame
// constants of up to kStaticMaxFrames frames.  Every GPU the library runs on holds its own copy of the array until the
// process ends.  In host code the name `scratch` is only a handle for hipGetSymbolAddress: the address the kernels get
// is the one that call returns for the current device, kept per device below.
constexpr int kStaticMaxFrames = 1024;
static __device__ __align__(256) unsigned char scratch[sizeof(adop::ViewConst) * kStaticMaxFrames];

namespace adop
{
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (looked up once per device).
adop_status scratch_of_current_device(void** out)
{
    int dev = -1;
    ADOP_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(ADOP_HIP_ERROR, "device ordinal out of range");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev])
    {
        void* p = nullptr;
        ADOP_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(ADOP_HIP_ERROR, "hipGetSymbolAddress returned no address for the scratch array");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return ADOP_OK;
}
}  // namespace adop

using namespace adop;

extern "C"
{
size_t adop_workspace_size(const adop_scene* scene, int32_t num_views, int32_t num_layers, int32_t w, int32_t h)
{
    if (!scene || num_views < 1 || num_layers < 1 || num_layers > ADOP_MAX_LAYERS || w < 1 || h < 1) return 0;
    if (scene->num_channels < 1 || scene->num_channels > kMaxChannels) return 0;
    return layout(scene, num_views, num_layers, w, h).total;
}

size_t adop_workspace_size_for(const adop_scene* scene, int32_t num_views, int32_t num_layers, int32_t w, int32_t h,
                               uint32_t flags)
{
    if (!scene || num_views < 1 || num_layers < 1 || num_layers > ADOP_MAX_LAYERS || w < 1 || h < 1) return 0;
    if (scene->num_channels < 1 || scene->num_channels > kMaxChannels) return 0;
    if (flags & ~kWorkspaceFlags) return 0;
    return layout(scene, num_views, num_layers, w, h, flags).total;
}

void adop_tuning_defaults(adop_tuning* out)
{
    if (out) *out = kTuningDefaults;
}

adop_status adop_set_tuning(const adop_tuning* t)
{
    if (!t) return fail(ADOP_INVALID_ARG, "null argument");
    auto one_of = [](int v, std::initializer_list<int> ok) {
        for (int k : ok)
            if (v == k) return true;
        return false;
    };
    if (t->forward_path < 0 || t->forward_path > 2) return fail(ADOP_INVALID_ARG, "tuning: forward_path must be 0, 1 or 2");
    if (t->tile_slice_entries < 1) return fail(ADOP_INVALID_ARG, "tuning: tile_slice_entries must be positive");
    if (t->ghost_concurrent < -1 || t->ghost_concurrent > 1) return fail(ADOP_INVALID_ARG, "tuning: ghost_concurrent must be -1, 0 or 1");
    if (t->bin_shard_shift < -1 || t->bin_shard_shift > 3) return fail(ADOP_INVALID_ARG, "tuning: bin_shard_shift must be -1 .. 3");
    if (!one_of(t->direct_lists, {0, 1}) || !one_of(t->normalize_fused, {0, 1}) || !one_of(t->normalize_by_queue, {0, 1}))
        return fail(ADOP_INVALID_ARG, "tuning: direct_lists, normalize_fused and normalize_by_queue are 0 or 1");
    if (!one_of(t->prepass_ppt, {0, 1, 2, 4}) || !one_of(t->count_ppt, {0, 1, 2, 4}) || !one_of(t->scatter_ppt, {1, 2, 4}) ||
        !one_of(t->tile_k, {1, 2, 4}))
        return fail(ADOP_INVALID_ARG, "tuning: points / entries per thread must be 1, 2 or 4 (prepass_ppt, count_ppt: or 0)");
    if (t->prepass_group_from < 0 || t->prepass_group_from > ADOP_MAX_LAYERS || t->blend_group_from < 0 ||
        t->blend_group_from > ADOP_MAX_LAYERS)
        return fail(ADOP_INVALID_ARG, "tuning: a level is 0 .. ADOP_MAX_LAYERS");
    if (!one_of(t->list_block, {64, 128, 256})) return fail(ADOP_INVALID_ARG, "tuning: list_block must be 64, 128 or 256");
    const int32_t* d = (const int32_t*)t;
    for (int k = 0; k < kTuningFields; ++k) g_tuning.f[k].store(d[k], std::memory_order_relaxed);
    return ADOP_OK;
}

void adop_get_tuning(adop_tuning* out)
{
    if (out) *out = tuning_now();
}

// RenderParams::render_points == false (PointRenderer.cu:1417,1433): the forward pass runs on an empty cloud (its
// workspace layout lies inside the one the caller sized for the whole cloud).
static const adop_scene* leave_out_points(const adop_scene* scene, adop_scene* copy)
{
    *copy                   = *scene;
    copy->num_points        = 0;
    copy->index_is_identity = 0;
    return copy;
}

adop_status adop_forward(const adop_scene* scene, const adop_view* views, int32_t num_views,
                         const adop_render_params* params, const adop_forward_buffers* buffers, void* workspace,
                         size_t workspace_bytes, adop_stats* stats, void* hip_stream)
{
    adop_status st = validate(scene, views, num_views, params, buffers);
    if (st != ADOP_OK) return st;
    adop_scene without_points;
    if (params->skip_points) scene = leave_out_points(scene, &without_points);
    // (the layout the caller sized the workspace with: adop_render_params.workspace_flags)
    if (params->workspace_flags & ~kWorkspaceFlags) return fail(ADOP_INVALID_ARG, "unknown workspace flag");
    const WorkspaceLayout wl = layout(scene, num_views, buffers->num_layers, views[0].w, views[0].h, params->workspace_flags);
    if (!workspace || workspace_bytes < wl.total) return fail(ADOP_WORKSPACE_TOO_SMALL, "workspace too small");
    if (!wl.has_lists && !buffers->point_cache && !params->skip_points)
        return fail(ADOP_INVALID_ARG, "ADOP_WORKSPACE_POINT_CACHE_KEPT: the forward pass needs point_cache");
    const adop_tuning tn = tuning_now();
    hipStream_t stream = (hipStream_t)hip_stream;
    ViewConst* dviews  = (ViewConst*)((char*)workspace + wl.views);

    ViewPrep vp;
    st = upload_views(scene, views, num_views, dviews, stream, &vp);
    if (st != ADOP_OK) return st;
    Levels lv   = make_levels(scene, num_views, buffers, nullptr);
    CloudArg pc = make_cloud(scene, buffers);
    ParamArg rp = make_params(params);

    if (stats)
    {
        st = fill_async(stats, sizeof(adop_stats), 0, stream);
        if (st != ADOP_OK) return st;
    }
    const int C      = scene->num_channels;
    const int S      = accum_stride(C);
    float* accum     = (float*)((char*)workspace + wl.pixels);
    const bool half  = scene->texture_dtype == ADOP_TEXTURE_F16;

    // Tile path: only where the workspace holds the bins (a caller may leave them out, and layout() does when the cloud
    // is beyond what the bin entries can address); a handful of points is faster through the direct path.
    int path = params->forward_path ? params->forward_path : tn.forward_path;
    if (path < 0 || path > 2) return fail(ADOP_INVALID_ARG, "forward_path must be 0, 1 or 2");
    const bool bins_possible = can_bin(scene->num_points, num_views, views[0].w, views[0].h);
    if (path == 2 && bins_possible && !wl.has_bins)
        return fail(ADOP_WORKSPACE_TOO_SMALL, "forward_path = 2 needs a workspace with the tile bins");
    // The tile path bins every projected point; a cloud with very many points per pixel is faster through the direct
    // path, whose early depth test drops most of them before they cost anything.
    // A batch of windows into their frames (crop offsets: the crops of a training step) counts with the share of the
    // cloud that a window sees, taken as 1/16: a 512 x 512 window of a 1920 x 1080 frame holds an eighth of the
    // frame's points, and a frame about half of the cloud.
    if (path == 0)
    {
        bool windows = num_views > 1;
        for (int b = 0; b < num_views; ++b) windows = windows && (views[b].crop_cx != 0.f || views[b].crop_cy != 0.f);
        const size_t per_pixel = (size_t)kTilePathMaxPointsPerPixel * (windows ? kWindowCloudShare : 1);
        const size_t tiles     = max_tiles(num_views, views[0].w, views[0].h);
        const double seen      = (double)scene->num_points / (windows ? kWindowCloudShare : 1);  // points a view handles
        const bool filled      = tiles >= (size_t)kTilePathEnoughTiles ||
                            seen * 1e-6 * (kTilePathUsPerMTiles / (double)tiles - kDirectPathUsPerM) <= kDirectPathFixedUs;
        path = (scene->num_points >= kTilePathMinPoints &&
                (size_t)scene->num_points <= per_pixel * views[0].w * views[0].h && tiles >= (size_t)kTilePathMinTiles &&
                filled)
                   ? 2
                   : 1;
    }
    if (path == 2 && !wl.has_bins) path = 1;

    if (path == 2)
    {
        if (!pc.cache) pc.cache = (float4*)((char*)workspace + wl.proj);  // (has_lists: checked above)
        BinArg bin;
        bin.lt      = kTileLevels < lv.num ? kTileLevels : lv.num;
        bin.tiles_x = ((views[0].w - 1) >> kTileShiftX) + 1;
        bin.tiles_y = ((views[0].h - 1) >> kTileShiftY) + 1;
        bin.count   = (uint32_t*)((char*)workspace + wl.bin_count);
        bin.offset  = (uint32_t*)((char*)workspace + wl.bin_offset);
        bin.order   = (uint4*)((char*)workspace + wl.bin_order);
        bin.rows    = (float*)((char*)workspace + wl.bin_rows);
        bin.entries = (float4*)((char*)workspace + wl.bin_entries);
        bin.info    = (uint32_t*)((char*)workspace + wl.bin_info);
        const int T = bin.tiles_x * bin.tiles_y * num_views;
        bin.shard_shift   = bin_shard_shift((size_t)T, tn.bin_shard_shift);
        bin.num_tiles     = T;
        const int counters = T << bin.shard_shift;
        bin.row_count = bin.count + counters;
        bin.tickets   = bin.count + counters + 1;
        bin.max_rows   = slice_rows(scene->num_points, num_views);
        bin.row_floats = slice_row_floats(scene->num_channels);
        bin.slice_entries = (uint32_t)tn.tile_slice_entries;
        // smaller bins than the call can fill: the prefix sum tells the kernels behind it whether the entries fit
        const bool capped = wl.bin_cap < (size_t)kTileLevels * (size_t)num_views * (size_t)scene->num_points;
        bin.overflow      = capped ? (uint32_t*)((char*)workspace + wl.bin_overflow) : nullptr;
        bin.cap           = (uint32_t)(wl.bin_cap < 0xFFFFFFFFull ? wl.bin_cap : 0xFFFFFFFFull);
        {
            StageScope sc("Initialize", stream);
            // tile counters, and for the coarse levels the packed depth and the global accumulators of the direct path
            size_t first   = (size_t)lv.pix_prefix[bin.lt] * lv.B * S;
            size_t accum_n = (size_t)lv.pix_prefix[lv.num] * lv.B * S - first;
            int grid       = pixel_grid(lv, bin.lt) > 32 ? pixel_grid(lv, bin.lt) : 32;
            launch_clear(lv, bin.lt, grid, accum + first, S % 4 == 0 ? accum_n : 0, bin.count, counters + 1 + 2 * bin.max_rows, vp, stream);
            if (S % 4 != 0 && (st = fill_async(accum + first, accum_n * sizeof(float), 0, stream)) != ADOP_OK) return st;
        }
        {
            StageScope sc("BinCount", stream);
            launch_bin(0, pc, dviews, lv, rp, bin, stats, tn, stream);
        }
        {
            StageScope sc("BinScatter", stream);
            launch_tile_scan(bin, counters, stream);
            launch_bin(1, pc, dviews, lv, rp, bin, nullptr, tn, stream);
        }
        {
            StageScope sc("TileDepth", stream);
            launch_tile_depth(lv, bin, T, stream);
        }
        {
            StageScope sc("TileBlend", stream);
            ADOP_HIP_CHECK(launch_tile_blend(pc, lv, rp, bin, T, half, accum, S, scene->background_color,
                                             params->output_background_mask, params->output_background_mask_value,
                                             scene->index_is_identity, stats, tn, stream));
        }
        if (bin.lt < lv.num)
        {
            StageScope sc("CombineAndFill", stream);
            launch_resolve(lv, bin.lt, pixel_grid(lv, bin.lt), accum, S, scene->background_color,
                           params->output_background_mask, params->output_background_mask_value, stream,
                           Gate{bin.overflow, 0u});
        }
        if (capped)
        {
            // The direct path, queued behind the tile kernels: its kernels start only when the entries did not fit (the
            // tile kernels have then returned at once).  It renders the call from the beginning: all levels cleared,
            // the counters counted again; the point records the first binning pass left are written once more.
            const Gate over{bin.overflow, 1u};
            const size_t accum_n = (size_t)lv.pix_prefix[lv.num] * lv.B * S;
            ViewPrep none;
            memset(&none, 0, sizeof(none));
            {
                StageScope sc("Initialize", stream);
                launch_clear(lv, 0, pixel_grid(lv), accum, S % 4 == 0 ? accum_n : 0, nullptr, 0, none, stream, over, stats);
                // (an accumulator stride that is no multiple of four floats: cleared whether needed or not)
                if (S % 4 != 0 && (st = fill_async(accum, accum_n * sizeof(float), 0, stream)) != ADOP_OK) return st;
            }
            {
                StageScope sc("DepthPrepass", stream);
                launch_prepass(pc, dviews, lv, rp, stats, tn, stream, over);
            }
            {
                StageScope sc("RenderForward", stream);
                launch_blend(pc, dviews, lv, rp, half, accum, S, stats, tn, stream, over);
            }
            {
                StageScope sc("CombineAndFill", stream);
                launch_resolve(lv, 0, pixel_grid(lv), accum, S, scene->background_color, params->output_background_mask,
                               params->output_background_mask_value, stream, over);
            }
        }
        ADOP_HIP_CHECK(hipGetLastError());
        return ADOP_OK;
    }

    // Without a caller's point cache (no backward pass follows) the prepass hands the blend compacted lists of the
    // points that can still pass a depth test instead of a record per point.
    if (!pc.cache && tn.direct_lists && scene->num_points > 0)
    {
        pc.cache      = (float4*)((char*)workspace + wl.proj);
        pc.list_ids   = (uint32_t*)((char*)workspace + wl.list_ids);
        pc.list_count = (uint32_t*)((char*)workspace + wl.list_count);
        pc.list_span  = prepass_points_per_block(scene->num_points, tn.prepass_ppt);
        pc.list_stride = wl.list_stride;
    }
    size_t accum_n   = (size_t)lv.pix_prefix[lv.num] * lv.B * S;  // floats, multiple of 4 unless S < 4
    {
        StageScope sc("Initialize", stream);
        if (S % 4 == 0)
            launch_clear(lv, 0, pixel_grid(lv), accum, accum_n, nullptr, 0, vp, stream);
        else
        {
            launch_clear(lv, 0, pixel_grid(lv), accum, 0, nullptr, 0, vp, stream);
            if ((st = fill_async(accum, accum_n * sizeof(float), 0, stream)) != ADOP_OK) return st;
        }
    }
    {
        StageScope sc("DepthPrepass", stream);
        launch_prepass(pc, dviews, lv, rp, stats, tn, stream);
    }
    {
        StageScope sc("RenderForward", stream);
        launch_blend(pc, dviews, lv, rp, half, accum, S, stats, tn, stream);
    }
    {
        StageScope sc("CombineAndFill", stream);
        launch_resolve(lv, 0, pixel_grid(lv), accum, S, scene->background_color, params->output_background_mask,
                       params->output_background_mask_value, stream);
    }
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

adop_status adop_backward(const adop_scene* scene, const adop_view* views, int32_t num_views,
                          const adop_render_params* params, const adop_forward_buffers* fwd,
                          const adop_backward_buffers* grads, void* workspace, size_t workspace_bytes,
                          adop_stats* stats, void* hip_stream)
{
    adop_status st = validate(scene, views, num_views, params, fwd);
    if (st != ADOP_OK) return st;
    if (!grads || !grads->grad_texture || !grads->grad_background)
        return fail(ADOP_INVALID_ARG, "grad_texture / grad_background missing");
    for (int l = 0; l < fwd->num_layers; ++l)
        if (!grads->grad_out[l]) return fail(ADOP_INVALID_ARG, "upstream gradient missing");  // :1131,1589
    if (grads->grad_points && !grads->grad_points_count) return fail(ADOP_INVALID_ARG, "grad_points_count missing");
    if (grads->grad_pose && !grads->grad_pose_count) return fail(ADOP_INVALID_ARG, "grad_pose_count missing");
    if (grads->grad_intrinsics && !grads->grad_intrinsics_count)
        return fail(ADOP_INVALID_ARG, "grad_intrinsics_count missing");
    // (the backward pass uses the first part of the workspace only, which every layout has)
    if (params->workspace_flags & ~kWorkspaceFlags) return fail(ADOP_INVALID_ARG, "unknown workspace flag");
    WorkspaceLayout wl = layout(scene, num_views, fwd->num_layers, views[0].w, views[0].h, params->workspace_flags);
    if (!workspace || workspace_bytes < wl.total) return fail(ADOP_WORKSPACE_TOO_SMALL, "workspace too small");
    const adop_tuning tn = tuning_now();
    hipStream_t stream = (hipStream_t)hip_stream;
    ViewConst* dviews  = (ViewConst*)((char*)workspace + wl.views);
    double* bg_partial = (double*)((char*)workspace + wl.bg_partial);
    double* pt_partial = (double*)((char*)workspace + wl.pt_partial);
    double* scratch    = (double*)((char*)workspace + wl.scratch);

    ViewPrep vp;
    st = upload_views(scene, views, num_views, dviews, stream, &vp);
    if (st != ADOP_OK) return st;
    Levels lv   = make_levels(scene, num_views, fwd, grads);
    CloudArg pc = make_cloud(scene, fwd);
    // (a forward pass that left the points out wrote no projected points; the backward pass runs over the cloud all
    // the same, as the reference's does, PointRenderer.cu:1598-1604, against the empty depth and weight buffers)
    if (params->skip_points) pc.cache = nullptr;
    ParamArg rp = make_params(params);
    const int C = scene->num_channels;
    const int N = scene->num_points;

    // Build(info,false): zero the gradient tensors (:922-949)
    {
        StageScope sc("Prepare Backward", stream);
        // with an identity index and a vectorised channel count backward_tex_kernel writes every texel itself
        const bool tex_self_clearing = scene->index_is_identity && (C == 4 || C == 8) && N > 0;
        if (!tex_self_clearing &&
            (st = fill_async(grads->grad_texture, sizeof(float) * (size_t)C * scene->num_texels, 0, stream)) != ADOP_OK)
            return st;
        // grad_points / grad_points_count: every row is written by the kernels of the first view
        // (backward_tex_kernel clears the rows without a spatial gradient, backward_ghost_kernel writes the others)
        if (stats)
        {
            // keep the forward counters, clear only the backward ones
            if ((st = fill_async(stats->spatial, sizeof(uint64_t) * ADOP_MAX_LAYERS, 0, stream)) != ADOP_OK)
                return st;
        }
    }

    float* ig     = (float*)((char*)workspace + wl.pixels);
    float2* dw    = (float2*)((char*)workspace + wl.dw);
    if (!lv.irec) lv.irec = ig;  // interleave_kernel leaves the image records in front of the gradient records
    int bg_blocks = pixel_grid(lv) < kBgBlocks ? pixel_grid(lv) : kBgBlocks;
    {
        StageScope sc("CombineAndFillBackward", stream);
        launch_interleave(lv, bg_blocks, ig, dw, bg_partial, (uint32_t*)((char*)workspace + wl.q_counts), vp, stream);
    }
    int want_pose = grads->grad_pose != nullptr;
    int want_intr = grads->grad_intrinsics != nullptr;
    int pt_blocks = (N + kBlock - 1) / kBlock;
    if (pt_blocks > kPartialBlocks) pt_blocks = kPartialBlocks;
    if (pt_blocks < 1) pt_blocks = 1;
    bool half = scene->texture_dtype == ADOP_TEXTURE_F16;
    QueueArg q;
    q.counts = (uint32_t*)((char*)workspace + wl.q_counts);
    q.items  = (unsigned long long*)((char*)workspace + wl.q_items);
    q.cap    = wl.q_cap;
    // Several views (up to kConcurrentViews): the spatial gradients of all views run side by side in one launch; the
    // descriptor pass tells every item whether other views add to the same point's gradient row (those rows are summed
    // with float atomics, all others written by their one owner).  Otherwise: one launch per view, each adding to the
    // point gradients in the order of the views.
    // Side by side pays while a launch per view would be small or the views share few points (the crop windows of a
    // training batch; a cloud of at most kConcurrentMaxPoints points); full views of a large cloud, which share most
    // of their points, fill a launch each and need no atomics that way (8 views of 20 M points: 1.76 against 1.82 ms).
    // adop_tuning.ghost_concurrent = 1 forces the one launch, 0 the launch per view.
    bool windows         = num_views > 1;
    for (int b = 0; b < num_views; ++b) windows = windows && (views[b].crop_cx != 0.f || views[b].crop_cy != 0.f);
    const bool want_conc = tn.ghost_concurrent >= 0 ? tn.ghost_concurrent != 0 : (windows || N <= kConcurrentMaxPoints);
    q.concurrent         = num_views > 1 && num_views <= kConcurrentViews && want_conc ? 1 : 0;
    // One view: the spatial-gradient kernel normalises the point gradients itself (adop_tuning.normalize_fused = 0: a
    // pass of the finalize kernel does).
    q.normalize = (num_views == 1 && grads->grad_points && tn.normalize_fused) ? (params->normalize_mode == 0 ? 1 : 2) : 0;
    if (N < 1)
    {
        // nothing writes the partial rows: clear them for finalize
        if ((st = fill_async(pt_partial, sizeof(double) * (size_t)num_views * kPartialBlocks * kPartialStride, 0,
                             stream)) != ADOP_OK)
            return st;
    }
    {
        // one pass over the points for all views: the descriptor gradient is summed in registers and written once
        StageScope sc("RenderBackward/descriptor", stream);
        launch_backward_tex(pc, dviews, lv, rp, half, ig, dw, grads, scene->index_is_identity, q, stats, stream);
    }
    if (q.concurrent)
    {
        StageScope sc("RenderBackward/spatial", stream);
        launch_backward_ghost(pc, dviews, lv, rp, half, ig, grads, want_pose, want_intr, scene->index_is_identity, -1, q,
                              pt_blocks, pt_partial, stream);
    }
    else
        for (int b = 0; b < num_views; ++b)
        {
            StageScope sc("RenderBackward/spatial", stream);
            launch_backward_ghost(pc, dviews, lv, rp, half, ig, grads, want_pose, want_intr, scene->index_is_identity, b,
                                  q, pt_blocks, pt_partial, stream);
        }
    StageScope post("Post Process Gradient", stream);
    launch_finalize(dviews, num_views, C, bg_partial, bg_blocks, pt_partial, pt_blocks, grads, scene->num_poses,
                    scene->num_cameras, scene->intrinsics_cols, params->normalize_mode, scratch,
                    (double*)((char*)workspace + wl.fin_mini), q.counts + (size_t)num_views * kNumQueues, N, q, tn, stream);
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

static adop_status env_common(const adop_scene* scene, const adop_view* views, int32_t num_views,
                              const adop_forward_buffers* buffers, int env_h, int env_w)
{
    if (!scene || !views || !buffers || num_views < 1) return fail(ADOP_INVALID_ARG, "null argument");
    if (buffers->num_layers < 1 || buffers->num_layers > ADOP_MAX_LAYERS)
        return fail(ADOP_UNSUPPORTED_LAYERS, "invalid number of layers");
    if (env_h < 1 || env_w < 1) return fail(ADOP_INVALID_ARG, "environment map size");
    if (num_views > 32) return fail(ADOP_INVALID_ARG, "environment map: at most 32 views per call");
    for (int b = 0; b < num_views; ++b)
    {
        // The reference samples pinhole views only (SAIGA_ASSERT(cam.camera_model_type == PINHOLE_DISTORTION),
        // EnvironmentMap.cu:129); OCam views are an extension here: pixel -> ray through ocam_unproject.
        if (views[b].camera_model_type == ADOP_CAMERA_PINHOLE_DISTORTION)
        {
            if (scene->intrinsics_cols != 13) return fail(ADOP_INVALID_ARG, "pinhole intrinsics need 13 columns");
        }
        else if (views[b].camera_model_type == ADOP_CAMERA_OCAM)
        {
            if (scene->intrinsics_cols < 6 || scene->intrinsics_cols > kMaxIntrinsicsCols)
                return fail(ADOP_INVALID_ARG, "OCam intrinsics need 6 .. 24 columns");
        }
        else
            return fail(ADOP_INVALID_ARG, "unknown camera model");
        if (views[b].image_index < 0 || views[b].image_index >= scene->num_poses || views[b].camera_index < 0 ||
            views[b].camera_index >= scene->num_cameras)
            return fail(ADOP_INVALID_ARG, "view index out of range");
    }
    if (!scene->poses_se3 || !scene->intrinsics) return fail(ADOP_INVALID_ARG, "poses / intrinsics missing");
    return ADOP_OK;
}

static ViewChunk make_chunk(const adop_view* views, int n)
{
    ViewChunk ch;
    memset(&ch, 0, sizeof(ch));
    for (int k = 0; k < n; ++k) ch.v[k] = views[k];
    return ch;
}

adop_status adop_env_sample(const adop_scene* scene, const adop_view* views, int32_t num_views,
                            const float* env_texture, int32_t env_h, int32_t env_w, const adop_forward_buffers* buffers,
                            float* const* uv_levels, float* const* env_levels, int32_t add_to_out, void* hip_stream)
{
    adop_status st = env_common(scene, views, num_views, buffers, env_h, env_w);
    if (st != ADOP_OK) return st;
    if (!env_texture) return fail(ADOP_INVALID_ARG, "env_texture missing");
    if (add_to_out < 0 || add_to_out > 2) return fail(ADOP_INVALID_ARG, "add_to_out must be 0, 1 or 2");
    hipStream_t stream = (hipStream_t)hip_stream;
    ViewChunk chunk    = make_chunk(views, num_views);
    Levels lv = make_levels(scene, num_views, buffers, nullptr);
    EnvLevels ev;
    memset(&ev, 0, sizeof(ev));
    for (int l = 0; l < buffers->num_layers; ++l)
    {
        ev.uv[l]  = uv_levels ? uv_levels[l] : nullptr;
        ev.env[l] = env_levels ? env_levels[l] : nullptr;
        if (add_to_out && !buffers->layers[l].out) return fail(ADOP_INVALID_ARG, "out buffer missing");
        if (add_to_out == 2 && !ev.env[l]) return fail(ADOP_INVALID_ARG, "add_to_out = 2 writes the composed image to env_levels");
    }
    launch_env_sample(chunk, scene->poses_se3, scene->intrinsics, lv, ev, env_texture, env_h, env_w, add_to_out,
                      scene->intrinsics_cols, stream);
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

adop_status adop_env_sample_backward(const adop_scene* scene, const adop_view* views, int32_t num_views, int32_t env_h,
                                     int32_t env_w, const adop_forward_buffers* buffers,
                                     const float* const* grad_out_levels, const float* const* uv_levels,
                                     float* grad_env, void* hip_stream)
{
    adop_status st = env_common(scene, views, num_views, buffers, env_h, env_w);
    if (st != ADOP_OK) return st;
    if (!grad_out_levels || !grad_env) return fail(ADOP_INVALID_ARG, "gradient buffers missing");
    hipStream_t stream = (hipStream_t)hip_stream;
    ViewChunk chunk    = make_chunk(views, num_views);
    Levels lv = make_levels(scene, num_views, buffers, nullptr);
    EnvLevels ev;
    memset(&ev, 0, sizeof(ev));
    for (int l = 0; l < buffers->num_layers; ++l)
    {
        if (!grad_out_levels[l]) return fail(ADOP_INVALID_ARG, "upstream gradient missing");
        ev.gout[l] = grad_out_levels[l];
        // (the texture coordinates the forward call stored, if the caller kept them; every level or none)
        if (uv_levels && !uv_levels[l]) return fail(ADOP_INVALID_ARG, "uv_levels: a level is missing");
        ev.uv[l] = uv_levels ? const_cast<float*>(uv_levels[l]) : nullptr;
    }
    st = fill_async(grad_env, sizeof(float) * (size_t)scene->num_channels * env_h * env_w, 0, stream);
    if (st != ADOP_OK) return st;
    launch_env_backward(chunk, scene->poses_se3, scene->intrinsics, lv, ev, grad_env, env_h, env_w, scene->intrinsics_cols,
                        stream);
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

adop_status adop_apply_tangent(double* tangent, double* poses_se3, int32_t num_poses, void* hip_stream)
{
    if (!tangent || !poses_se3 || num_poses < 0) return fail(ADOP_INVALID_ARG, "null argument");
    if (num_poses == 0) return ADOP_OK;
    launch_apply_tangent(tangent, poses_se3, num_poses, (hipStream_t)hip_stream);
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

// Grids of the nearest-neighbour search: both are sized on the device (preprocess_kernels.hip), the second one within a
// budget of cells that grows with the cloud.
static uint32_t knn_max_cells(int32_t num_points)
{
    size_t want = (size_t)(num_points > 0 ? num_points : 0) * 16;
    if (want < ((size_t)1 << 22)) want = (size_t)1 << 22;  // > kKnnCoarseDim^3
    if (want > ((size_t)1 << 27)) want = (size_t)1 << 27;
    return (uint32_t)want;
}

constexpr uint32_t kKnnFirstCells = 160u * 160u * 160u;  // the first grid has at most 160 cells per axis

struct KnnWorkspace
{
    KnnGrid *grid, *grid0;  // second (search) grid and first grid, device
    float* sample;
    uint32_t *count, *offset, *chunk;  // second grid
    uint32_t *count0, *offset0;        // first grid
    float4 *sorted, *sorted0;
    uint32_t *list, *list2, *counts;
    size_t total;
};

static KnnWorkspace knn_layout(void* workspace, int32_t num_points)
{
    const uint32_t cells = knn_max_cells(num_points);
    const size_t n       = (size_t)(num_points > 0 ? num_points : 0);
    size_t o             = 0;
    auto take            = [&](size_t bytes) {
        const size_t at = o;
        o               = align_up(o + bytes, 256);
        return at;
    };
    const size_t o_grid = take(sizeof(KnnGrid)), o_grid0 = take(sizeof(KnnGrid));
    const size_t o_sample  = take(sizeof(float) * 2048);
    const size_t o_counts  = take(sizeof(uint32_t) * 2);
    const size_t o_count   = take(sizeof(uint32_t) * (size_t)cells);
    const size_t o_offset  = take(sizeof(uint32_t) * ((size_t)cells + 1));
    const size_t o_chunk   = take(sizeof(uint32_t) * knn_chunk_words(cells));
    const size_t o_count0  = take(sizeof(uint32_t) * (size_t)kKnnFirstCells);
    const size_t o_offset0 = take(sizeof(uint32_t) * ((size_t)kKnnFirstCells + 1));
    const size_t o_sorted  = take(sizeof(float4) * n);
    const size_t o_sorted0 = take(sizeof(float4) * n);
    const size_t o_list    = take(sizeof(uint32_t) * n);
    const size_t o_list2   = take(sizeof(uint32_t) * n);
    KnnWorkspace w;
    memset(&w, 0, sizeof(w));
    w.total = o;
    if (workspace)
    {
        char* base = (char*)workspace;
        w.grid     = (KnnGrid*)(base + o_grid);
        w.grid0    = (KnnGrid*)(base + o_grid0);
        w.sample   = (float*)(base + o_sample);
        w.counts   = (uint32_t*)(base + o_counts);
        w.count    = (uint32_t*)(base + o_count);
        w.offset   = (uint32_t*)(base + o_offset);
        w.chunk    = (uint32_t*)(base + o_chunk);
        w.count0   = (uint32_t*)(base + o_count0);
        w.offset0  = (uint32_t*)(base + o_offset0);
        w.sorted   = (float4*)(base + o_sorted);
        w.sorted0  = (float4*)(base + o_sorted0);
        w.list     = (uint32_t*)(base + o_list);
        w.list2    = (uint32_t*)(base + o_list2);
    }
    return w;
}

size_t adop_knn_workspace_size(int32_t num_points)
{
    if (num_points < 0) return 0;
    return knn_layout(nullptr, num_points).total;
}

// The points in cell order of the search grid (both in the workspace).  build = false: the workspace still holds them
// from the last call.
static adop_status knn_prepare(const float* position, int32_t num_points, const float* bbox_min, const float* bbox_max,
                               int sample_rank, void* workspace, size_t workspace_bytes, bool build, hipStream_t stream,
                               KnnWorkspace* out)
{
    if (!workspace || workspace_bytes < adop_knn_workspace_size(num_points))
        return fail(ADOP_WORKSPACE_TOO_SMALL, "workspace too small");
    *out = knn_layout(workspace, num_points);
    if (!build) return ADOP_OK;
    KnnGrid box;  // the caller's bounding box; the grids are sized on the device
    memset(&box, 0, sizeof(box));
    for (int k = 0; k < 3; ++k)
    {
        box.min[k] = bbox_min[k];
        box.ext[k] = bbox_max[k] - bbox_min[k];
        if (!(box.ext[k] >= 0) || !(box.ext[k] < 1.0e30f)) return fail(ADOP_INVALID_ARG, "bounding box is not finite");
    }
    const uint32_t max_cells = knn_max_cells(num_points);
    const float4* pos        = (const float4*)position;
    // first grid (kept: the search falls back on it for points in sparse parts of the cloud)
    launch_knn_first_grid(pos, num_points, box, out->grid0, stream);
    launch_knn_build(pos, num_points, out->grid0, kKnnFirstCells, out->count0, out->offset0, out->chunk, out->sorted0,
                     stream);
    const int samples = knn_num_samples(num_points);
    if (!launch_knn_sample(sample_rank, out->sorted0, num_points, out->grid0, out->offset0, out->sample, samples, stream))
        return fail(ADOP_INVALID_ARG, "rank must be 1..8");
    // second grid
    launch_knn_refine_grid(out->sample, samples, out->grid0, out->grid, max_cells, stream);
    launch_knn_build(pos, num_points, out->grid, max_cells, out->count, out->offset, out->chunk, out->sorted, stream);
    return ADOP_OK;
}

adop_status adop_knn_distance(const float* position, int32_t num_points, int32_t rank, const float* bbox_min,
                              const float* bbox_max, float* out_distance, void* workspace, size_t workspace_bytes,
                              void* hip_stream)
{
    if (!position || !bbox_min || !bbox_max || !out_distance) return fail(ADOP_INVALID_ARG, "null argument");
    if (rank < 1 || rank > 8) return fail(ADOP_INVALID_ARG, "rank must be 1..8");
    if (num_points <= rank) return fail(ADOP_INVALID_ARG, "the cloud needs more than `rank` points");
    hipStream_t stream = (hipStream_t)hip_stream;
    KnnWorkspace w;
    adop_status st =
        knn_prepare(position, num_points, bbox_min, bbox_max, rank, workspace, workspace_bytes, true, stream, &w);
    if (st != ADOP_OK) return st;
    if ((st = fill_async(w.counts, 2 * sizeof(uint32_t), 0, stream)) != ADOP_OK) return st;
    KnnSearchArg a{w.grid, w.grid0, w.sorted, w.sorted0, w.offset, w.offset0, w.list, w.list2, w.counts};
    if (!launch_knn_search(rank, num_points, a, out_distance, stream))
        return fail(ADOP_INVALID_ARG, "rank must be 1..8");
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

adop_status adop_close_points(const float* position, int32_t num_points, const float* radius, const float* bbox_min,
                              const float* bbox_max, int32_t* state, uint32_t* round_undecided, int32_t num_rounds,
                              int32_t resume, void* workspace, size_t workspace_bytes, void* hip_stream)
{
    if (!position || !radius || !bbox_min || !bbox_max || !state || !round_undecided)
        return fail(ADOP_INVALID_ARG, "null argument");
    if (num_points < 1) return fail(ADOP_INVALID_ARG, "empty cloud");
    if (num_rounds < 1 || num_rounds > 1024) return fail(ADOP_INVALID_ARG, "num_rounds must be 1..1024");
    hipStream_t stream = (hipStream_t)hip_stream;
    KnnWorkspace w;
    // (the grid is sized for the 4th-neighbour distance, the one the cloud's radii come from)
    adop_status st =
        knn_prepare(position, num_points, bbox_min, bbox_max, 4, workspace, workspace_bytes, !resume, stream, &w);
    if (st != ADOP_OK) return st;
    if (!resume && (st = fill_async(state, sizeof(int32_t) * (size_t)num_points, 0, stream)) != ADOP_OK) return st;
    if ((st = fill_async(round_undecided, sizeof(uint32_t) * (size_t)num_rounds, 0, stream)) != ADOP_OK) return st;
    for (int r = 0; r < num_rounds; ++r)
        launch_close_points(w.sorted, num_points, w.grid, w.offset, radius, state, round_undecided, r, stream);
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

size_t adop_frames_workspace_size(int32_t num_frames)
{
    return num_frames < 1 ? 0 : align_up(sizeof(ViewConst) * (size_t)num_frames, 256);
}

// Argument checks shared by the two camera-distance entry points.
static adop_status camera_distance_check(const adop_scene* scene, const adop_view* frames, int32_t num_frames,
                                         const float* out_distance)
{
    if (!scene || !frames || !out_distance) return fail(ADOP_INVALID_ARG, "null argument");
    if (num_frames < 1) return fail(ADOP_INVALID_ARG, "num_frames must be >= 1");
    if (scene->num_points < 0 || !scene->position) return fail(ADOP_INVALID_ARG, "point cloud missing");
    if (!scene->poses_se3 || !scene->intrinsics || scene->num_poses < 1 || scene->num_cameras < 1)
        return fail(ADOP_INVALID_ARG, "poses / intrinsics missing");
    if (scene->intrinsics_cols != 13) return fail(ADOP_INVALID_ARG, "pinhole intrinsics need 13 columns");
    for (int f = 0; f < num_frames; ++f)
    {
        const adop_view& v = frames[f];
        // FrameData::Project3 (SceneData.cpp:26-34) is the pinhole + distortion model
        if (v.camera_model_type != ADOP_CAMERA_PINHOLE_DISTORTION)
            return fail(ADOP_INVALID_ARG, "the camera distance needs the pinhole model");
        if (v.image_index < 0 || v.image_index >= scene->num_poses || v.camera_index < 0 ||
            v.camera_index >= scene->num_cameras || v.w < 1 || v.h < 1)
            return fail(ADOP_INVALID_ARG, "frame out of range");
    }
    return ADOP_OK;
}

// The per-frame constants go to `dviews` (device memory for num_frames ViewConst), then every point is tested against
// every frame.
static adop_status camera_distance_run(const adop_scene* scene, const adop_view* frames, int32_t num_frames,
                                       float* out_distance, ViewConst* dviews, hipStream_t stream)
{
    if (scene->num_points == 0) return ADOP_OK;
    adop_status st = upload_views(scene, frames, num_frames, dviews, stream);
    if (st != ADOP_OK) return st;
    launch_camera_distance((const float4*)scene->position, scene->num_points, dviews, num_frames, out_distance, stream);
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

adop_status adop_point_distance_to_camera(const adop_scene* scene, const adop_view* frames, int32_t num_frames,
                                          float* out_distance, void* workspace, size_t workspace_bytes,
                                          void* hip_stream)
{
    adop_status st = camera_distance_check(scene, frames, num_frames, out_distance);
    if (st != ADOP_OK) return st;
    if (!workspace || workspace_bytes < adop_frames_workspace_size(num_frames))
        return fail(ADOP_WORKSPACE_TOO_SMALL, "workspace too small");
    return camera_distance_run(scene, frames, num_frames, out_distance, (ViewConst*)workspace, (hipStream_t)hip_stream);
}

int32_t adop_static_max_frames(void)
{
    return kStaticMaxFrames;
}

adop_status adop_point_distance_to_camera_static(const adop_scene* scene, const adop_view* frames, int32_t num_frames,
                                                 float* out_distance, void* hip_stream)
{
    adop_status st = camera_distance_check(scene, frames, num_frames, out_distance);
    if (st != ADOP_OK) return st;
    if (num_frames > kStaticMaxFrames)
        return fail(ADOP_INVALID_ARG, "adop_point_distance_to_camera_static takes at most " +
                                          std::to_string(kStaticMaxFrames) +
                                          " frames per call (the size of the library's own scratch array); use "
                                          "adop_point_distance_to_camera with a workspace for more");
    void* dviews = nullptr;
    if ((st = scratch_of_current_device(&dviews)) != ADOP_OK) return st;
    // Nothing of the array has to start at zero: the constants of frames 0 .. num_frames-1 are written before the
    // distance kernel reads them, and it reads no others.
    return camera_distance_run(scene, frames, num_frames, out_distance, (ViewConst*)dviews, (hipStream_t)hip_stream);
}

adop_status adop_morton_codes(const float* position, int32_t num_points, const float* bbox_min, const float* bbox_max,
                              uint64_t* out_codes, void* hip_stream)
{
    if (!position || !bbox_min || !bbox_max || !out_codes || num_points < 0) return fail(ADOP_INVALID_ARG, "null argument");
    if (num_points == 0) return ADOP_OK;
    float scale[3];
    for (int k = 0; k < 3; ++k)
    {
        const float ext = bbox_max[k] - bbox_min[k];
        if (!(ext >= 0) || !(ext < 1.0e30f)) return fail(ADOP_INVALID_ARG, "bounding box is not finite");
        scale[k] = ext > 0 ? 2097151.f / ext : 0.f;
    }
    launch_morton((const float4*)position, num_points, bbox_min, scale, (unsigned long long*)out_codes,
                  (hipStream_t)hip_stream);
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

adop_status adop_profile_enable(int32_t enable)
{
    g_profile = enable != 0;
    return ADOP_OK;
}

int32_t adop_profile_read(adop_stage_time* out, int32_t max_entries)
{
    int n = 0;
    std::vector<StageEvent> events;
    {
        std::lock_guard<std::mutex> lock(g_stage_mutex);
        events.swap(g_stage_events);
    }
    for (StageEvent& e : events)
    {
        float ms = 0.f;
        if (hipEventSynchronize(e.stop) == hipSuccess && hipEventElapsedTime(&ms, e.start, e.stop) == hipSuccess)
        {
            int k = 0;
            for (; k < n; ++k)
                if (strcmp(out[k].name, e.name) == 0) break;
            if (k == n && n < max_entries)
            {
                memset(&out[n], 0, sizeof(out[n]));
                strncpy(out[n].name, e.name, sizeof(out[n].name) - 1);
                ++n;
            }
            if (k < n)
            {
                out[k].total_ms += ms;
                out[k].calls += 1;
            }
        }
    }
    std::lock_guard<std::mutex> lock(g_stage_mutex);
    for (StageEvent& e : events)
    {
        g_event_pool.push_back(e.start);
        g_event_pool.push_back(e.stop);
    }
    return n;
}

const char* adop_last_error_string(void)
{
    return g_last_error.c_str();
}

const char* adop_version(void)
{
    return "adop_raster 0.3 (gfx950)";
}
}  // extern "C"
