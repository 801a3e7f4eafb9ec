// adop_raster.hip — HIP kernels (gfx950 / CDNA4) and C-ABI of the one-pixel point rasterizer.
//
// Pipeline of one forward call (reference: BlendPointCloudForward, PointRenderer.cu:1389-1531):
//   prepare_views   poses_se3 (f64) / intrinsics rows -> per-view constants in the workspace
//   clear           depth_index = (bits(100000.f)<<32)|~0, weight = 0, out = 0         (InitializeData :1039-1090)
//   prepass         per point, per view, per level: 64-bit atomicMin of (depth bits | point id)  (:203-301)
//   blend           per point: fuzzy depth test, descriptor accumulation with fp32 atomics       (:303-393)
//   resolve         per pixel: out/=weight or background, mask, f32 depth = high word            (:726-754,:828-847)
// and of one backward call (BlendPointCloudBackward, :1549-1644):
//   background_grad per pixel partial sums (CombineAndFillBackward :851-900)
//   render_backward per point: descriptor gradient + ghost/spatial gradient (RenderBackward :396-724); the
//                   per-image pose and per-camera intrinsics sums are kept per thread in f64, reduced per block
//                   and written as per-block partials (no same-address atomics)
//   finalize        partials -> grad_background / grad_pose / grad_intrinsics, NormalizeGradient (:1534-1547)
//
// No MFMA anywhere: the path is scan + scatter/gather + atomics, bounded by HBM and L2 atomic throughput.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <string>
#include <vector>

#include "../../include/adop_raster.h"
#include "device_math.h"

#pragma clang fp contract(off)

namespace adop
{
constexpr int kBlock       = 256;
constexpr int kMaxChannels = 16;
constexpr int kPartialBlocks = 2048;       // grid of the grid-stride kernels that produce per-block partials
constexpr int kPartialStride = 24;         // doubles per (block, view), 21 used: 6 pose, pose count, intr count, 13 intr
constexpr int kAcc = 21;
constexpr int kMaxIntrinsicsCols = 24;     // 5 affine + up to 19 polynomial coefficients / 13 pinhole
constexpr uint64_t kClearPacked = (uint64_t(0x47C35000u) << 32) | 0xFFFFFFFFull;  // bits(100000.f), PointRenderer.cu:1045

struct LevelArg
{
    int32_t w, h;
    uint64_t* depth_index;
    float* depth;
    float* weight;
    float* out;
    float* mask;
    const float* gin;  // upstream gradient (backward only)
};

struct Levels
{
    int32_t num;
    int32_t B;
    int32_t C;
    int32_t pix_prefix[ADOP_MAX_LAYERS + 1];  // prefix sum of w*h over levels (one image)
    LevelArg l[ADOP_MAX_LAYERS];
};

struct CloudArg
{
    const float4* position;
    const int32_t* normal;
    const int32_t* index;
    int32_t n;
    const void* texture;
    int32_t num_texels;
    const float* intrinsics;
    const float* dropout;  // [B,N] or null
};

struct ParamArg
{
    int32_t test_backward_mode;
    int32_t check_normal;
    int32_t ghost_gradients;
    int32_t drop_by_radius;
    float depth_accept;
    float drop_threshold;
    float dist_cutoff;
    float distortion_gradient_factor;
    float K_gradient_factor;
};

struct ViewChunk
{
    adop_view v[32];
};

// ------------------------------------------------------------------------------------------------
// small kernels
// ------------------------------------------------------------------------------------------------

__global__ void fill_u32_kernel(uint32_t* __restrict__ p, size_t n, uint32_t v)
{
    size_t i      = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

// d_render_params.Pose() / PinholeIntrinsics() / OcamIntrinsics() (PointRenderer.cu:73-96) for one view.
__device__ __forceinline__ ViewConst make_view_const(const adop_view& v, const double* __restrict__ poses,
                                                     const float* __restrict__ intrinsics, int cols)
{
    ViewConst c;
    const double* p = poses + 8 * (size_t)v.image_index;
    float x = (float)p[0], y = (float)p[1], z = (float)p[2], w = (float)p[3];
    float n = sqrtf(((x * x + y * y) + z * z) + w * w);  // Sophus SO3f(quaternion) normalises
    c.qx    = x / n;
    c.qy    = y / n;
    c.qz    = z / n;
    c.qw    = w / n;
    c.tx    = (float)p[4];
    c.ty    = (float)p[5];
    c.tz    = (float)p[6];
    const float* row = intrinsics + (size_t)cols * v.camera_index;
    for (int i = 0; i < 5; ++i) c.k[i] = 0;
    for (int i = 0; i < 8; ++i) c.d[i] = 0;
    if (v.camera_model_type == ADOP_CAMERA_PINHOLE_DISTORTION)
    {
        for (int i = 0; i < 5; ++i) c.k[i] = row[i];
        for (int i = 0; i < 8; ++i) c.d[i] = row[5 + i];
    }
    c.crop[0]      = v.crop_fx;
    c.crop[1]      = v.crop_fy;
    c.crop[2]      = v.crop_cx;
    c.crop[3]      = v.crop_cy;
    c.crop[4]      = v.crop_s;
    c.w            = v.w;
    c.h            = v.h;
    c.image_index  = v.image_index;
    c.camera_index = v.camera_index;
    c.model        = v.camera_model_type;
    c.intr_offset  = cols * v.camera_index;
    c.npoly        = cols - 5;
    c.pad          = 0;
    return c;
}

// Once per call: the per-view constants every point kernel reads through uniform loads.
__global__ void prepare_views_kernel(ViewChunk chunk, int first, int count, const double* __restrict__ poses,
                                     const float* __restrict__ intrinsics, int cols, ViewConst* __restrict__ out)
{
    int t = threadIdx.x;
    if (t >= count) return;
    out[first + t] = make_view_const(chunk.v[t], poses, intrinsics, cols);
}

// InitializeData (PointRenderer.cu:1039-1090): one thread per pixel of every level and image.
__global__ __launch_bounds__(kBlock) void clear_kernel(Levels lv)
{
    int per_image = lv.pix_prefix[lv.num];
    size_t total  = (size_t)per_image * lv.B;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride)
    {
        int b = (int)(t / per_image);
        int r = (int)(t - (size_t)b * per_image);
        int l = 0;
#pragma unroll
        for (int k = 1; k < ADOP_MAX_LAYERS; ++k)
            if (k < lv.num && r >= lv.pix_prefix[k]) l = k;
        const LevelArg& L = lv.l[l];
        int p             = r - lv.pix_prefix[l];
        size_t hw         = (size_t)L.w * L.h;
        size_t o          = (size_t)b * hw + p;
        L.depth_index[o]  = kClearPacked;
        L.weight[o]       = 0.f;
        for (int c = 0; c < lv.C; ++c) L.out[((size_t)b * lv.C + c) * hw + p] = 0.f;
    }
}

template <typename T>
__device__ __forceinline__ T wave_sum(T v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    return v;
}

__device__ __forceinline__ void stat_add(uint64_t* dst, bool pred)
{
    unsigned long long m = __ballot(pred);
    if (m && (threadIdx.x & 63) == (__ffsll((long long)m) - 1))
        atomicAdd((unsigned long long*)dst, (unsigned long long)__popcll(m));
}

// ------------------------------------------------------------------------------------------------
// forward point kernels
// ------------------------------------------------------------------------------------------------

// DepthPrepassMulti (PointRenderer.cu:203-301) on the packed buffer the reference keeps as "old rendering"
// (LayerCuda::depth_index_tensor, PackIndex): min over (depth bits << 32 | point id).  The plain load before the
// atomic is the reference's early-z (:278); a stale value only costs a redundant atomic.
template <bool STATS>
__global__ __launch_bounds__(kBlock) void prepass_kernel(CloudArg pc, const ViewConst* __restrict__ views, Levels lv,
                                                         ParamArg rp, adop_stats* stats)
{
    int i      = blockIdx.x * kBlock + threadIdx.x;
    bool valid = i < pc.n;
    float4 P   = valid ? pc.position[i] : make_float4(0, 0, 0, 0);
    V3 pos     = {P.x, P.y, P.z};
    V3 nrm     = {0, 0, 0};
    if (valid && pc.normal) nrm = unpack_normal10(pc.normal[i]);

    for (int b = 0; b < lv.B; ++b)
    {
        const ViewConst& vc = views[b];
        V2 ip;
        V3 view_p;
        float z, radius_pixels;
        bool ok = valid && project_point(vc, pc.intrinsics, pos, nrm, P.w, rp.check_normal != 0, rp.dist_cutoff,
                                         lv.l[0].w, &ip, &z, &radius_pixels, &view_p);
        if (!STATS && !ok) continue;
        bool alive = ok;
#pragma unroll
        for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
        {
            if (l >= lv.num) break;
            if (rp.drop_by_radius && radius_pixels < rp.drop_threshold) alive = false;  // break, :261-264
            const LevelArg& L = lv.l[l];
            int px = f2i_rn(ip.x), py = f2i_rn(ip.y);
            bool in = alive && (unsigned)px < (unsigned)L.w && (unsigned)py < (unsigned)L.h;
            if (STATS) stat_add(&stats->visible[l], in);
            if (in)
            {
                uint64_t pk   = ((uint64_t)f2u(z) << 32) | (uint32_t)i;
                uint64_t* dst = L.depth_index + ((size_t)b * L.h + py) * L.w + px;
                uint64_t cur  = __builtin_nontemporal_load(dst);
                if (pk < cur) atomicMin((unsigned long long*)dst, (unsigned long long)pk);
            }
            radius_pixels *= 0.5f;
            ip.x *= 0.5f;
            ip.y *= 0.5f;
        }
    }
}

template <bool HALF>
__device__ __forceinline__ float tex_fetch(const void* tex, size_t o)
{
    if (HALF) return __half2float(((const __half*)tex)[o]);
    return ((const float*)tex)[o];
}

// RenderForwardMulti (PointRenderer.cu:303-393).
template <bool HALF, bool STATS>
__global__ __launch_bounds__(kBlock) void blend_kernel(CloudArg pc, const ViewConst* __restrict__ views, Levels lv,
                                                       ParamArg rp, adop_stats* stats)
{
    int i      = blockIdx.x * kBlock + threadIdx.x;
    bool valid = i < pc.n;
    float4 P   = valid ? pc.position[i] : make_float4(0, 0, 0, 0);
    V3 pos     = {P.x, P.y, P.z};
    V3 nrm     = {0, 0, 0};
    if (valid && pc.normal) nrm = unpack_normal10(pc.normal[i]);
    int tex_index = valid ? pc.index[i] : 0;
    bool tex_ok   = (unsigned)tex_index < (unsigned)pc.num_texels;  // device assert :362
    const float accept = rp.depth_accept + 1;

    for (int b = 0; b < lv.B; ++b)
    {
        bool dropped = valid && pc.dropout && pc.dropout[(size_t)b * pc.n + i] == 1.f;  // :314-315
        const ViewConst& vc = views[b];
        V2 ip;
        V3 view_p;
        float z, radius_pixels;
        bool ok = valid && !dropped &&
                  project_point(vc, pc.intrinsics, pos, nrm, P.w, rp.check_normal != 0, rp.dist_cutoff, lv.l[0].w, &ip,
                                &z, &radius_pixels, &view_p);
        if (STATS) stat_add(&stats->bad_index, ok && !tex_ok);
        ok = ok && tex_ok;
        if (!STATS && !ok) continue;
        bool alive = ok;
#pragma unroll
        for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
        {
            if (l >= lv.num) break;
            if (rp.drop_by_radius && radius_pixels < rp.drop_threshold) alive = false;
            const LevelArg& L = lv.l[l];
            int px = f2i_rn(ip.x), py = f2i_rn(ip.y);
            bool in = alive && (unsigned)px < (unsigned)L.w && (unsigned)py < (unsigned)L.h;
            bool acc = false;
            if (in)
            {
                size_t hw = (size_t)L.w * L.h;
                size_t p  = (size_t)py * L.w + px;
                // high word of the packed pixel = depth
                float image_depth = __uint_as_float((uint32_t)(L.depth_index[(size_t)b * hw + p] >> 32));
                acc               = !(z > image_depth * accept);  // :380
                if (acc)
                {
                    float* o = L.out + (size_t)b * lv.C * hw + p;
                    for (int c = 0; c < lv.C; ++c)
                    {
                        float t = tex_fetch<HALF>(pc.texture, (size_t)c * pc.num_texels + tex_index);
                        unsafeAtomicAdd(o + (size_t)c * hw, t);
                    }
                    unsafeAtomicAdd(L.weight + (size_t)b * hw + p, 1.f);
                }
            }
            if (STATS) stat_add(&stats->accepted[l], acc);
            radius_pixels *= 0.5f;
            ip.x *= 0.5f;
            ip.y *= 0.5f;
        }
    }
}

// CombineAndFill (:726-754) + CreateMask (:828-847) + the f32 depth the reference saves for backward.
__global__ __launch_bounds__(kBlock) void resolve_kernel(Levels lv, const float* __restrict__ background,
                                                         int write_mask, float mask_value)
{
    int per_image = lv.pix_prefix[lv.num];
    size_t total  = (size_t)per_image * lv.B;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride)
    {
        int b = (int)(t / per_image);
        int r = (int)(t - (size_t)b * per_image);
        int l = 0;
#pragma unroll
        for (int k = 1; k < ADOP_MAX_LAYERS; ++k)
            if (k < lv.num && r >= lv.pix_prefix[k]) l = k;
        const LevelArg& L = lv.l[l];
        int p             = r - lv.pix_prefix[l];
        size_t hw         = (size_t)L.w * L.h;
        size_t o          = (size_t)b * hw + p;
        float cou         = L.weight[o];
        L.depth[o]        = __uint_as_float((uint32_t)(L.depth_index[o] >> 32));
        float* out        = L.out + (size_t)b * lv.C * hw + p;
        if (cou == 0)
        {
            for (int c = 0; c < lv.C; ++c) out[(size_t)c * hw] = background[c];
        }
        else
        {
            for (int c = 0; c < lv.C; ++c) out[(size_t)c * hw] = out[(size_t)c * hw] / cou;
        }
        if (write_mask && L.mask) L.mask[o] = (cou == 0) ? mask_value : 1.f;
    }
}

// ------------------------------------------------------------------------------------------------
// backward kernels
// ------------------------------------------------------------------------------------------------

// CombineAndFillBackward (:851-900): sum of the upstream gradient over empty pixels, per channel.
// Per-thread partial in fp32 over a handful of pixels, wave/block reduction in f64, one f64 partial per block.
__global__ __launch_bounds__(kBlock) void background_grad_kernel(Levels lv, double* __restrict__ partial)
{
    __shared__ double red[kBlock / 64][kMaxChannels];
    float acc[kMaxChannels];
#pragma unroll
    for (int c = 0; c < kMaxChannels; ++c) acc[c] = 0;
    int per_image = lv.pix_prefix[lv.num];
    size_t total  = (size_t)per_image * lv.B;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride)
    {
        int b = (int)(t / per_image);
        int r = (int)(t - (size_t)b * per_image);
        int l = 0;
#pragma unroll
        for (int k = 1; k < ADOP_MAX_LAYERS; ++k)
            if (k < lv.num && r >= lv.pix_prefix[k]) l = k;
        const LevelArg& L = lv.l[l];
        int p             = r - lv.pix_prefix[l];
        size_t hw         = (size_t)L.w * L.h;
        if (L.weight[(size_t)b * hw + p] == 0)
        {
            const float* g = L.gin + (size_t)b * lv.C * hw + p;
#pragma unroll
            for (int c = 0; c < kMaxChannels; ++c)
                if (c < lv.C) acc[c] += g[(size_t)c * hw];
        }
    }
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int c = 0; c < kMaxChannels; ++c)
    {
        double v = wave_sum<double>((double)acc[c]);
        if (lane == 0) red[wave][c] = v;
    }
    __syncthreads();
    if (threadIdx.x < kMaxChannels)
    {
        double v = 0;
        for (int w = 0; w < kBlock / 64; ++w) v += red[w][threadIdx.x];
        partial[(size_t)blockIdx.x * kMaxChannels + threadIdx.x] = v;
    }
}

// RenderBackward (PointRenderer.cu:396-724).  Grid-stride over points so that the pose / intrinsics sums can live
// in registers (f64) for the whole kernel; they leave the block as one partial row per (block, view).
template <bool HALF, bool STATS>
__global__ __launch_bounds__(kBlock) void render_backward_kernel(CloudArg pc, const ViewConst* __restrict__ views,
                                                                  Levels lv, ParamArg rp, float* __restrict__ gtex,
                                                                  float* __restrict__ gpoints,
                                                                  float* __restrict__ gpoints_count, int want_pose,
                                                                  int want_intr, int view_b,
                                                                  double* __restrict__ partial, adop_stats* stats)
{
    __shared__ double red[kBlock / 64][kPartialStride];
    const int b         = view_b;
    const ViewConst& vc = views[b];
    const float accept  = rp.depth_accept + 1;
    const int C         = lv.C;

    double acc[kAcc];
#pragma unroll
    for (int k = 0; k < kAcc; ++k) acc[k] = 0;

    const int n_round = ((pc.n + kBlock - 1) / kBlock) * kBlock;
    for (int i = blockIdx.x * kBlock + threadIdx.x; i < n_round; i += gridDim.x * kBlock)
    {
        bool valid = i < pc.n;
        float4 P   = valid ? pc.position[i] : make_float4(0, 0, 0, 0);
        V3 pos     = {P.x, P.y, P.z};
        V3 nrm     = {0, 0, 0};
        if (valid && pc.normal) nrm = unpack_normal10(pc.normal[i]);
        bool drop_out = valid && pc.dropout && pc.dropout[(size_t)b * pc.n + i] == 1.f;
        V2 ip;
        V3 view_p;
        float z, radius_pixels;
        bool ok = valid && project_point(vc, pc.intrinsics, pos, nrm, P.w, rp.check_normal != 0, rp.dist_cutoff,
                                         lv.l[0].w, &ip, &z, &radius_pixels, &view_p);
        int tex_index = valid ? pc.index[i] : 0;
        ok            = ok && (unsigned)tex_index < (unsigned)pc.num_texels;
        if (!STATS && !ok) continue;

        float scale = 1;
        bool alive  = ok;
        // running value of grad_points[i] / count[i]; loaded at the first contribution so that the additions
        // happen in the reference's order (view after view, level after level)
        float gp[3] = {0, 0, 0};
        float gp_n  = 0;
        bool gp_live = false;
#pragma unroll
        for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
        {
            if (l >= lv.num) break;
            const LevelArg& L = lv.l[l];
            int px = f2i_rn(ip.x), py = f2i_rn(ip.y);
            bool lod_skip = rp.drop_by_radius && radius_pixels < rp.drop_threshold;  // continue, :451-454
            bool in       = alive && !lod_skip && (unsigned)px < (unsigned)L.w && (unsigned)py < (unsigned)L.h;
            bool spatial  = false;
            if (in)
            {
                size_t hw = (size_t)L.w * L.h;
                size_t p  = (size_t)py * L.w + px;
                float image_depth = L.depth[(size_t)b * hw + p];
                if (z > image_depth * accept)
                {
                    alive = false;  // break, :462
                }
                else
                {
                    float w          = L.weight[(size_t)b * hw + p];
                    const float* gin = L.gin + (size_t)b * C * hw;
                    bool go          = true;
                    if (!drop_out)
                    {
                        if (w == 0)
                            go = false;  // continue, :473
                        else
                        {
                            float iw = 1.f / w;
                            for (int c = 0; c < C; ++c)
                            {
                                float g = iw * gin[(size_t)c * hw + p];
                                unsafeAtomicAdd(gtex + (size_t)c * pc.num_texels + tex_index, g);
                            }
                        }
                    }
                    bool point_grad = (rp.ghost_gradients && drop_out) | (!rp.ghost_gradients && !drop_out);
                    int ex          = min(px, L.w - 1 - px);
                    int ey          = min(py, L.h - 1 - py);
                    if (go && point_grad && min(ex, ey) > 2)  // distanceFromEdge > 2, :489
                    {
                        spatial          = true;
                        const float* I   = L.out + (size_t)b * C * hw;
                        const size_t n0  = p - 1, n1 = p + 1, n2 = p - L.w, n3 = p + L.w;
                        const float* Wp  = L.weight + (size_t)b * hw;
                        const float* Dp  = L.depth + (size_t)b * hw;
                        float Wn[4]      = {Wp[n0], Wp[n1], Wp[n2], Wp[n3]};
                        float Dn[4]      = {Dp[n0], Dp[n1], Dp[n2], Dp[n3]};
                        const size_t nb[4] = {n0, n1, n2, n3};
                        float dR_dpx = 0, dR_dpy = 0;
                        for (int c = 0; c < C; ++c)
                        {
                            float T_p = tex_fetch<HALF>(pc.texture, (size_t)c * pc.num_texels + tex_index);
                            float v[4];
#pragma unroll
                            for (int k = 0; k < 4; ++k)
                            {
                                float I_x = I[(size_t)c * hw + nb[k]];
                                float G_x = gin[(size_t)c * hw + nb[k]];
                                float dI;
                                if (rp.test_backward_mode == 4)
                                {
                                    float W_x = Wn[k], D_x = Dn[k];
                                    if (W_x == 0 || z * accept < D_x)
                                        dI = T_p - I_x;
                                    else if (z > D_x * accept)
                                        dI = 0;
                                    else
                                        dI = (W_x / (W_x + 1) * I_x + 1 / (W_x + 1) * T_p - I_x);
                                }
                                else
                                    dI = T_p - I_x;
                                v[k] = dI * G_x;
                            }
                            float a0 = -v[0], a1 = v[1], b0 = -v[2], b1 = v[3];
                            dR_dpx += 0.5f * (a0 + a1);
                            dR_dpy += 0.5f * (b0 + b1);
                        }
                        V2 dR_dp      = {dR_dpx / (float)C, dR_dpy / (float)C};
                        float crop2[5] = {vc.crop[0] * scale, vc.crop[1] * scale, vc.crop[2] * scale,
                                          vc.crop[3] * scale, vc.crop[4] * scale};  // crop.scale(scale), :616
                        BackwardOut bo;
                        project_point_backward(vc, pc.intrinsics, view_p, dR_dp, crop2, rp.dist_cutoff, &bo);
                        if (gpoints)
                        {
                            if (!gp_live)
                            {
                                const float* g = gpoints + 4 * (size_t)i;
                                gp[0]          = g[0];
                                gp[1]          = g[1];
                                gp[2]          = g[2];
                                gp_n           = gpoints_count[i];
                                gp_live        = true;
                            }
                            gp[0] += bo.g_point[0];
                            gp[1] += bo.g_point[1];
                            gp[2] += bo.g_point[2];
                            gp_n += 1.f;
                        }
                        if (want_pose)
                        {
#pragma unroll
                            for (int k = 0; k < 6; ++k) acc[k] += (double)bo.g_pose[k];
                            acc[6] += 1.0;
                        }
                        if (want_intr)
                        {
                            if (vc.model == 0)
                            {
                                float kf = rp.K_gradient_factor;
                                bo.g_k[4] *= 0.1f;
                                bo.g_k[4] *= 0;  // :653-654
#pragma unroll
                                for (int k = 0; k < 5; ++k) acc[8 + k] += (double)(kf * bo.g_k[k]);
                                float df = rp.distortion_gradient_factor;
                                bo.g_dis[2] *= 0.25f;
                                bo.g_dis[3] *= 0.1f;
                                bo.g_dis[4] *= 0.1f;
                                bo.g_dis[5] *= 0.1f;
                                bo.g_dis[6] *= 0.1f;
                                bo.g_dis[7] *= 0.1f;
#pragma unroll
                                for (int k = 0; k < 8; ++k) acc[13 + k] += (double)(df * bo.g_dis[k]);
                                acc[7] += 1.0 / 1024.0;  // :680-681
                            }
                            else
                            {
#pragma unroll
                                for (int k = 0; k < 5; ++k) acc[8 + k] += (double)bo.g_k[k];
                                acc[7] += 1.0;  // :718
                            }
                        }
                    }
                }
            }
            if (STATS) stat_add(&stats->spatial[l], spatial);
            scale *= 0.5f;
            radius_pixels *= 0.5f;
            ip.x *= 0.5f;
            ip.y *= 0.5f;
        }
        if (gp_live)
        {
            // one thread owns point i for this view; views are launched one after another on the stream
            float* g = gpoints + 4 * (size_t)i;
            g[0]     = gp[0];
            g[1]     = gp[1];
            g[2]     = gp[2];
            gpoints_count[i] = gp_n;
        }
    }

    if (want_pose || want_intr)
    {
        int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
        for (int k = 0; k < 21; ++k)
        {
            double v = wave_sum<double>(acc[k]);
            if (lane == 0) red[wave][k] = v;
        }
        __syncthreads();
        if (threadIdx.x < 21)
        {
            double v = 0;
            for (int w = 0; w < kBlock / 64; ++w) v += red[w][threadIdx.x];
            partial[((size_t)b * gridDim.x + blockIdx.x) * kPartialStride + threadIdx.x] = v;
        }
    }
}

// Reduces the per-block partial rows and runs NormalizeGradient (:1534-1547, launches :1611-1636) for the
// background / pose / intrinsics outputs.  One block.
__global__ __launch_bounds__(kBlock) void finalize_kernel(const ViewConst* __restrict__ views, int B, int C,
                                                          const double* __restrict__ bg_partial, int bg_blocks,
                                                          const double* __restrict__ pt_partial, int pt_blocks,
                                                          float* __restrict__ gbg, double* __restrict__ gpose,
                                                          float* __restrict__ gpose_count, int num_poses,
                                                          float* __restrict__ gintr, float* __restrict__ gintr_count,
                                                          int num_cameras, int cols, int normalize_mode,
                                                          double* __restrict__ scratch)
{
    __shared__ double sh[kBlock];
    // background
    for (int c = 0; c < C; ++c)
    {
        double v = 0;
        for (int k = threadIdx.x; k < bg_blocks; k += kBlock) v += bg_partial[(size_t)k * kMaxChannels + c];
        sh[threadIdx.x] = v;
        __syncthreads();
        for (int s = kBlock / 2; s > 0; s >>= 1)
        {
            if (threadIdx.x < s) sh[threadIdx.x] += sh[threadIdx.x + s];
            __syncthreads();
        }
        if (threadIdx.x == 0) gbg[c] = (float)sh[0];
        __syncthreads();
    }
    if (!gpose && !gintr) return;

    // scratch: [num_poses*7] pose sums + count, then [num_cameras*(cols+1)] intrinsics sums + count
    double* sp = scratch;
    double* si = scratch + (size_t)num_poses * 7;
    for (int k = threadIdx.x; k < num_poses * 7 + num_cameras * (cols + 1); k += kBlock) scratch[k] = 0;
    __syncthreads();
    for (int b = 0; b < B; ++b)
    {
        for (int q = 0; q < 21; ++q)
        {
            double v = 0;
            for (int k = threadIdx.x; k < pt_blocks; k += kBlock)
                v += pt_partial[((size_t)b * pt_blocks + k) * kPartialStride + q];
            sh[threadIdx.x] = v;
            __syncthreads();
            for (int s = kBlock / 2; s > 0; s >>= 1)
            {
                if (threadIdx.x < s) sh[threadIdx.x] += sh[threadIdx.x + s];
                __syncthreads();
            }
            if (threadIdx.x == 0)
            {
                const ViewConst& vc = views[b];
                double t            = sh[0];
                if (q < 6)
                    sp[(size_t)vc.image_index * 7 + q] += t;
                else if (q == 6)
                    sp[(size_t)vc.image_index * 7 + 6] += t;
                else if (q == 7)
                    si[(size_t)vc.camera_index * (cols + 1) + cols] += t;
                else if (q - 8 < cols)
                    si[(size_t)vc.camera_index * (cols + 1) + (q - 8)] += t;
            }
            __syncthreads();
        }
    }
    if (gpose)
    {
        for (int f = threadIdx.x; f < num_poses; f += kBlock)
        {
            float c        = (float)sp[(size_t)f * 7 + 6];
            gpose_count[f] = c;
            for (int k = 0; k < 6; ++k)
            {
                double t                   = sp[(size_t)f * 7 + k];
                gpose[(size_t)f * 6 + k] = (c > 0) ? t / (double)c : t;
            }
        }
    }
    if (gintr)
    {
        for (int k = threadIdx.x; k < num_cameras * cols; k += kBlock)
            gintr[k] = (float)si[(size_t)(k / cols) * (cols + 1) + (k % cols)];
        for (int k = threadIdx.x; k < num_cameras; k += kBlock) gintr_count[k] = (float)si[(size_t)k * (cols + 1) + cols];
        __syncthreads();
        if (threadIdx.x == 0)
        {
            int total = num_cameras * cols;
            if (normalize_mode == 0)
            {
                // NormalizeGradient<float,13> whatever the row width (:1633)
                for (int t = 0; t < num_cameras; ++t)
                {
                    float c = gintr_count[t];
                    if (c > 0)
                        for (int k = 0; k < 13; ++k)
                            if (13 * t + k < total) gintr[13 * t + k] = gintr[13 * t + k] / c;
                }
            }
            else
            {
                for (int t = 0; t < num_cameras; ++t)
                {
                    float c = gintr_count[t];
                    if (c > 0)
                        for (int k = 0; k < cols; ++k) gintr[cols * t + k] = gintr[cols * t + k] / c;
                }
            }
        }
    }
}

// NormalizeGradient<float,3> on the [N,4] point-gradient buffer (:1620-1627).  mode 0 reproduces the reference's
// vec3 view (element t = floats 3t..3t+2 divided by count[t]); mode 1 normalises row t by count[t].
__global__ __launch_bounds__(kBlock) void normalize_points_kernel(float* __restrict__ g, const float* __restrict__ count,
                                                                  int n, int mode)
{
    int t = blockIdx.x * kBlock + threadIdx.x;
    if (t >= n) return;
    float c = count[t];
    if (!(c > 0)) return;
    size_t o = (mode == 0) ? 3 * (size_t)t : 4 * (size_t)t;
    g[o + 0] = g[o + 0] / c;
    g[o + 1] = g[o + 1] / c;
    g[o + 2] = g[o + 2] / c;
}

// ------------------------------------------------------------------------------------------------
// environment map (EnvironmentMap.cu:41-157) and its composition (RenderModule.cpp:106-127)
// ------------------------------------------------------------------------------------------------

__device__ __forceinline__ V2 k_unproject2(const float* K, V2 ip)
{
    float y = (ip.y - K[3]) / K[1];
    float x = ((ip.x - K[2]) - K[4] * y) / K[0];
    return {x, y};
}

// undistortNormalizedPointSimple: OpenCV fixed-point iteration, 5 rounds.
__device__ __forceinline__ V2 undistort_simple(V2 p, const float* D)
{
    float k1 = D[0], k2 = D[1], k3 = D[2], k4 = D[3], k5 = D[4], k6 = D[5], p1 = D[6], p2 = D[7];
    float x0 = p.x, y0 = p.y, x = p.x, y = p.y;
    for (int it = 0; it < 5; ++it)
    {
        float r2     = x * x + y * y;
        float icdist = (1.0f + ((k6 * r2 + k5) * r2 + k4) * r2) / (1.0f + ((k3 * r2 + k2) * r2 + k1) * r2);
        float dx     = 2.0f * p1 * x * y + p2 * (r2 + 2.0f * x * x);
        float dy     = p1 * (r2 + 2.0f * y * y) + 2.0f * p2 * x * y;
        x            = (x0 - dx) * icdist;
        y            = (y0 - dy) * icdist;
    }
    return {x, y};
}

// BuildSphericalUV + SphericalCoordinates for pixel (gx,gy) of a level whose crop is scaled by `sc`.
__device__ __forceinline__ V2 spherical_uv(const ViewConst& vc, float sc, int gx, int gy)
{
    float cr[5] = {vc.crop[0] * sc, vc.crop[1] * sc, vc.crop[2] * sc, vc.crop[3] * sc, vc.crop[4] * sc};
    V3 t    = {vc.tx, vc.ty, vc.tz};
    V3 rt   = quat_rotate(-vc.qx, -vc.qy, -vc.qz, vc.qw, t);
    V3 tinv = {-rt.x, -rt.y, -rt.z};
    V2 ip   = {(float)gx, (float)gy};
    V2 dist_p = k_unproject2(vc.k, k_unproject2(cr, ip));
    V2 np     = undistort_simple(dist_p, vc.d);
    V3 inp    = {np.x, np.y, 1};
    V3 r      = quat_rotate(-vc.qx, -vc.qy, -vc.qz, vc.qw, inp);
    V3 wp     = {r.x + tinv.x, r.y + tinv.y, r.z + tinv.z};
    V3 d      = {wp.x - tinv.x, wp.y - tinv.y, wp.z - tinv.z};
    float n   = sqrtf(dot3(d, d));
    d         = {d.x / n, d.y / n, d.z / n};
    float phi = atan2_poly(-d.z, d.x);
    float x   = phi / (2.0f * ADOP_PI);
    x         = x - floorf(x);
    float th  = acos_poly(d.y);
    float y   = 1 - th / ADOP_PI;
    return {x * 2 - 1, y * 2 - 1};
}

struct Bilinear
{
    int x0, y0;
    float w00, w01, w10, w11;
    bool x1ok, y1ok;
};

// grid_sample(bilinear, padding border, align_corners=true) addressing
__device__ __forceinline__ Bilinear bilinear_setup(V2 uv, int ew, int eh)
{
    float fx = (uv.x + 1) * 0.5f * (float)(ew - 1);
    float fy = (uv.y + 1) * 0.5f * (float)(eh - 1);
    fx       = fminf(fmaxf(fx, 0.f), (float)(ew - 1));
    fy       = fminf(fmaxf(fy, 0.f), (float)(eh - 1));
    Bilinear s;
    s.x0     = (int)floorf(fx);
    s.y0     = (int)floorf(fy);
    float ax = fx - (float)s.x0, ay = fy - (float)s.y0;
    s.w00    = (1 - ax) * (1 - ay);
    s.w01    = ax * (1 - ay);
    s.w10    = (1 - ax) * ay;
    s.w11    = ax * ay;
    s.x1ok   = s.x0 + 1 < ew;
    s.y1ok   = s.y0 + 1 < eh;
    return s;
}

struct EnvLevels
{
    float* uv[ADOP_MAX_LAYERS];
    float* env[ADOP_MAX_LAYERS];
    const float* gout[ADOP_MAX_LAYERS];
};

__global__ __launch_bounds__(kBlock) void env_sample_kernel(ViewChunk chunk, const double* __restrict__ poses,
                                                            const float* __restrict__ intrinsics, Levels lv,
                                                            EnvLevels ev, const float* __restrict__ tex, int eh, int ew,
                                                            int add_to_out)
{
    int per_image = lv.pix_prefix[lv.num];
    size_t total  = (size_t)per_image * lv.B;
    size_t t      = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total) return;
    int b = (int)(t / per_image);
    int r = (int)(t - (size_t)b * per_image);
    int l = 0;
#pragma unroll
    for (int k = 1; k < ADOP_MAX_LAYERS; ++k)
        if (k < lv.num && r >= lv.pix_prefix[k]) l = k;
    const LevelArg& L = lv.l[l];
    int p             = r - lv.pix_prefix[l];
    int gy = p / L.w, gx = p - gy * L.w;
    size_t hw   = (size_t)L.w * L.h;
    float sc    = 1;
    for (int k = 0; k < l; ++k) sc /= 2;
    float bgw = 1.f;
    if (add_to_out && L.mask) bgw = 1.f - L.mask[(size_t)b * hw + p];
    bool need = ev.uv[l] || ev.env[l] || (add_to_out && bgw != 0.f);
    if (!need) return;
    V2 uv = spherical_uv(make_view_const(chunk.v[b], poses, intrinsics, 13), sc, gx, gy);
    if (ev.uv[l])
    {
        ev.uv[l][((size_t)b * hw + p) * 2 + 0] = uv.x;
        ev.uv[l][((size_t)b * hw + p) * 2 + 1] = uv.y;
    }
    if (!ev.env[l] && !(add_to_out && bgw != 0.f)) return;
    Bilinear s = bilinear_setup(uv, ew, eh);
    for (int c = 0; c < lv.C; ++c)
    {
        const float* tc = tex + (size_t)c * eh * ew;
        float a         = 0;
        a += tc[(size_t)s.y0 * ew + s.x0] * s.w00;
        if (s.x1ok) a += tc[(size_t)s.y0 * ew + s.x0 + 1] * s.w01;
        if (s.y1ok) a += tc[(size_t)(s.y0 + 1) * ew + s.x0] * s.w10;
        if (s.x1ok && s.y1ok) a += tc[(size_t)(s.y0 + 1) * ew + s.x0 + 1] * s.w11;
        size_t o = ((size_t)b * lv.C + c) * hw + p;
        if (ev.env[l]) ev.env[l][o] = a;
        if (add_to_out) L.out[o] = L.out[o] + bgw * a;
    }
}

__global__ __launch_bounds__(kBlock) void env_backward_kernel(ViewChunk chunk, const double* __restrict__ poses,
                                                              const float* __restrict__ intrinsics, Levels lv,
                                                              EnvLevels ev, float* __restrict__ genv, int eh, int ew)
{
    int per_image = lv.pix_prefix[lv.num];
    size_t total  = (size_t)per_image * lv.B;
    size_t t      = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total) return;
    int b = (int)(t / per_image);
    int r = (int)(t - (size_t)b * per_image);
    int l = 0;
#pragma unroll
    for (int k = 1; k < ADOP_MAX_LAYERS; ++k)
        if (k < lv.num && r >= lv.pix_prefix[k]) l = k;
    const LevelArg& L = lv.l[l];
    int p             = r - lv.pix_prefix[l];
    int gy = p / L.w, gx = p - gy * L.w;
    size_t hw = (size_t)L.w * L.h;
    float sc  = 1;
    for (int k = 0; k < l; ++k) sc /= 2;
    float bgw = 1.f;
    if (L.mask) bgw = 1.f - L.mask[(size_t)b * hw + p];
    if (bgw == 0.f) return;
    V2 uv      = spherical_uv(make_view_const(chunk.v[b], poses, intrinsics, 13), sc, gx, gy);
    Bilinear s = bilinear_setup(uv, ew, eh);
    for (int c = 0; c < lv.C; ++c)
    {
        float g   = bgw * ev.gout[l][((size_t)b * lv.C + c) * hw + p];
        float* tc = genv + (size_t)c * eh * ew;
        unsafeAtomicAdd(tc + (size_t)s.y0 * ew + s.x0, g * s.w00);
        if (s.x1ok) unsafeAtomicAdd(tc + (size_t)s.y0 * ew + s.x0 + 1, g * s.w01);
        if (s.y1ok) unsafeAtomicAdd(tc + (size_t)(s.y0 + 1) * ew + s.x0, g * s.w10);
        if (s.x1ok && s.y1ok) unsafeAtomicAdd(tc + (size_t)(s.y0 + 1) * ew + s.x0 + 1, g * s.w11);
    }
}

// ApplyTangent (PointRenderer.cu:1646-1657): pose = Sophus::se3_expd(tangent) * pose; tangent = 0.  f64.
__global__ void apply_tangent_kernel(double* __restrict__ tangent, double* __restrict__ poses, int n)
{
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    double* t = tangent + 6 * (size_t)i;
    double* p = poses + 8 * (size_t)i;
    double ux = t[0], uy = t[1], uz = t[2], wx = t[3], wy = t[4], wz = t[5];
    double th2 = wx * wx + wy * wy + wz * wz;
    double th  = sqrt(th2);
    double im, re, a, bb;
    if (th < 1e-10)
    {
        double th4 = th2 * th2;
        im         = 0.5 - th2 / 48.0 + th4 / 3840.0;
        re         = 1.0 - th2 / 8.0 + th4 / 384.0;
        a          = 0.5;
        bb         = 1.0 / 6.0;
    }
    else
    {
        im = sin(0.5 * th) / th;
        re = cos(0.5 * th);
        a  = (1.0 - cos(th)) / th2;
        bb = (th - sin(th)) / (th2 * th);
    }
    double ex = im * wx, ey = im * wy, ez = im * wz, ew = re;
    double c1x = wy * uz - wz * uy, c1y = wz * ux - wx * uz, c1z = wx * uy - wy * ux;
    double c2x = wy * c1z - wz * c1y, c2y = wz * c1x - wx * c1z, c2z = wx * c1y - wy * c1x;
    double etx = ux + a * c1x + bb * c2x, ety = uy + a * c1y + bb * c2y, etz = uz + a * c1z + bb * c2z;
    double qx = p[0], qy = p[1], qz = p[2], qw = p[3];
    double nx = ew * qx + ex * qw + ey * qz - ez * qy;
    double ny = ew * qy - ex * qz + ey * qw + ez * qx;
    double nz = ew * qz + ex * qy - ey * qx + ez * qw;
    double nw = ew * qw - ex * qx - ey * qy - ez * qz;
    double tx = p[4], ty = p[5], tz = p[6];
    double uvx = 2 * (ey * tz - ez * ty), uvy = 2 * (ez * tx - ex * tz), uvz = 2 * (ex * ty - ey * tx);
    double rx = tx + ew * uvx + (ey * uvz - ez * uvy);
    double ry = ty + ew * uvy + (ez * uvx - ex * uvz);
    double rz = tz + ew * uvz + (ex * uvy - ey * uvx);
    double qn = sqrt(nx * nx + ny * ny + nz * nz + nw * nw);
    p[0]      = nx / qn;
    p[1]      = ny / qn;
    p[2]      = nz / qn;
    p[3]      = nw / qn;
    p[4]      = rx + etx;
    p[5]      = ry + ety;
    p[6]      = rz + etz;
    for (int k = 0; k < 6; ++k) t[k] = 0;
}

// ------------------------------------------------------------------------------------------------
// host side of the C-ABI
// ------------------------------------------------------------------------------------------------

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
thread_local bool g_profile = false;
thread_local std::vector<StageEvent> g_stage_events;
thread_local std::vector<hipEvent_t> g_event_pool;

hipEvent_t take_event()
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

struct WorkspaceLayout
{
    size_t views;       // ViewConst[B]
    size_t bg_partial;  // double[kPartialBlocks * kMaxChannels]
    size_t pt_partial;  // double[B * kPartialBlocks * kPartialStride]
    size_t scratch;     // double[num_poses*7 + num_cameras*(cols+1)]
    size_t total;
};

size_t align_up(size_t v, size_t a)
{
    return (v + a - 1) / a * a;
}

WorkspaceLayout layout(const adop_scene* s, int B)
{
    WorkspaceLayout w;
    size_t o     = 0;
    w.views      = o;
    o            = align_up(o + sizeof(ViewConst) * (size_t)B, 256);
    w.bg_partial = o;
    o            = align_up(o + sizeof(double) * kPartialBlocks * kMaxChannels, 256);
    w.pt_partial = o;
    o            = align_up(o + sizeof(double) * (size_t)B * kPartialBlocks * kPartialStride, 256);
    w.scratch    = o;
    o = align_up(o + sizeof(double) * ((size_t)s->num_poses * 7 + (size_t)s->num_cameras * (s->intrinsics_cols + 1)),
                 256);
    w.total = o;
    return w;
}

adop_status validate(const adop_scene* s, const adop_view* views, int B, const adop_render_params* rp,
                     const adop_forward_buffers* fb)
{
    if (!s || !views || !rp || !fb) return fail(ADOP_INVALID_ARG, "null argument");
    if (B < 1) return fail(ADOP_INVALID_ARG, "num_views must be >= 1");  // SAIGA_ASSERT(num_batches > 0), :909
    if (fb->num_layers < 1 || fb->num_layers > ADOP_MAX_LAYERS)
        return fail(ADOP_UNSUPPORTED_LAYERS, "invalid number of layers");  // :1199
    if (s->num_points < 0 || !s->position || !s->index) return fail(ADOP_INVALID_ARG, "point cloud missing");
    if (rp->check_normal && !s->normal)
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

adop_status upload_views(const adop_scene* s, const adop_view* views, int B, ViewConst* dst, hipStream_t st)
{
    for (int first = 0; first < B; first += 32)
    {
        ViewChunk ch;
        memset(&ch, 0, sizeof(ch));
        int count = B - first < 32 ? B - first : 32;
        for (int k = 0; k < count; ++k) ch.v[k] = views[first + k];
        hipLaunchKernelGGL(prepare_views_kernel, dim3(1), dim3(32), 0, st, ch, first, count, s->poses_se3,
                           s->intrinsics, s->intrinsics_cols, dst);
    }
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

adop_status fill_async(void* p, size_t bytes, uint32_t v, hipStream_t st)
{
    if (!p || bytes == 0) return ADOP_OK;
    size_t n    = bytes / 4;
    size_t want = (n + kBlock - 1) / kBlock;
    int grid    = (int)(want < 8192 ? (want ? want : 1) : 8192);
    hipLaunchKernelGGL(fill_u32_kernel, dim3(grid), dim3(kBlock), 0, st, (uint32_t*)p, n, v);
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

int pixel_grid(const Levels& lv)
{
    size_t total = (size_t)lv.pix_prefix[lv.num] * lv.B;
    size_t want  = (total + kBlock - 1) / kBlock;
    return (int)(want < 16384 ? (want ? want : 1) : 16384);
}

}  // namespace adop

using namespace adop;

extern "C"
{
size_t adop_workspace_size(const adop_scene* scene, int32_t num_views, int32_t num_layers, int32_t w, int32_t h)
{
    (void)num_layers;
    (void)w;
    (void)h;
    if (!scene || num_views < 1) return 0;
    return layout(scene, num_views).total;
}

adop_status adop_forward(const adop_scene* scene, const adop_view* views, int32_t num_views,
                         const adop_render_params* params, const adop_forward_buffers* buffers, void* workspace,
                         size_t workspace_bytes, adop_stats* stats, void* hip_stream)
{
    adop_status st = validate(scene, views, num_views, params, buffers);
    if (st != ADOP_OK) return st;
    WorkspaceLayout wl = layout(scene, num_views);
    if (!workspace || workspace_bytes < wl.total) return fail(ADOP_WORKSPACE_TOO_SMALL, "workspace too small");
    hipStream_t stream = (hipStream_t)hip_stream;
    ViewConst* dviews  = (ViewConst*)((char*)workspace + wl.views);

    st = upload_views(scene, views, num_views, dviews, stream);
    if (st != ADOP_OK) return st;
    Levels lv   = make_levels(scene, num_views, buffers, nullptr);
    CloudArg pc = make_cloud(scene, buffers);
    ParamArg rp = make_params(params);

    if (stats)
    {
        st = fill_async(stats, sizeof(adop_stats), 0, stream);
        if (st != ADOP_OK) return st;
    }
    {
        StageScope sc("Initialize", stream);
        hipLaunchKernelGGL(clear_kernel, dim3(pixel_grid(lv)), dim3(kBlock), 0, stream, lv);
    }

    int grid = (scene->num_points + kBlock - 1) / kBlock;
    if (grid > 0)
    {
        {
            StageScope sc("DepthPrepass", stream);
            if (stats)
                hipLaunchKernelGGL((prepass_kernel<true>), dim3(grid), dim3(kBlock), 0, stream, pc, dviews, lv, rp,
                                   stats);
            else
                hipLaunchKernelGGL((prepass_kernel<false>), dim3(grid), dim3(kBlock), 0, stream, pc, dviews, lv, rp,
                                   stats);
        }
        StageScope sc("RenderForward", stream);
        bool half = scene->texture_dtype == ADOP_TEXTURE_F16;
        if (half && stats)
            hipLaunchKernelGGL((blend_kernel<true, true>), dim3(grid), dim3(kBlock), 0, stream, pc, dviews, lv, rp,
                               stats);
        else if (half)
            hipLaunchKernelGGL((blend_kernel<true, false>), dim3(grid), dim3(kBlock), 0, stream, pc, dviews, lv, rp,
                               stats);
        else if (stats)
            hipLaunchKernelGGL((blend_kernel<false, true>), dim3(grid), dim3(kBlock), 0, stream, pc, dviews, lv, rp,
                               stats);
        else
            hipLaunchKernelGGL((blend_kernel<false, false>), dim3(grid), dim3(kBlock), 0, stream, pc, dviews, lv, rp,
                               stats);
    }
    {
        StageScope sc("CombineAndFill", stream);
        hipLaunchKernelGGL(resolve_kernel, dim3(pixel_grid(lv)), dim3(kBlock), 0, stream, lv, scene->background_color,
                           params->output_background_mask, params->output_background_mask_value);
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
    WorkspaceLayout wl = layout(scene, num_views);
    if (!workspace || workspace_bytes < wl.total) return fail(ADOP_WORKSPACE_TOO_SMALL, "workspace too small");
    hipStream_t stream = (hipStream_t)hip_stream;
    ViewConst* dviews  = (ViewConst*)((char*)workspace + wl.views);
    double* bg_partial = (double*)((char*)workspace + wl.bg_partial);
    double* pt_partial = (double*)((char*)workspace + wl.pt_partial);
    double* scratch    = (double*)((char*)workspace + wl.scratch);

    st = upload_views(scene, views, num_views, dviews, stream);
    if (st != ADOP_OK) return st;
    Levels lv   = make_levels(scene, num_views, fwd, grads);
    CloudArg pc = make_cloud(scene, fwd);
    ParamArg rp = make_params(params);
    const int C = scene->num_channels;
    const int N = scene->num_points;

    // Build(info,false): zero the gradient tensors (:922-949)
    {
        StageScope sc("Prepare Backward", stream);
        if ((st = fill_async(grads->grad_texture, sizeof(float) * (size_t)C * scene->num_texels, 0, stream)) != ADOP_OK)
            return st;
        if (grads->grad_points)
        {
            if ((st = fill_async(grads->grad_points, sizeof(float) * 4 * (size_t)N, 0, stream)) != ADOP_OK) return st;
            if ((st = fill_async(grads->grad_points_count, sizeof(float) * (size_t)N, 0, stream)) != ADOP_OK)
                return st;
        }
        if (stats)
        {
            // keep the forward counters, clear only the backward ones
            if ((st = fill_async(stats->spatial, sizeof(uint64_t) * ADOP_MAX_LAYERS, 0, stream)) != ADOP_OK)
                return st;
        }
    }

    int bg_blocks = pixel_grid(lv) < kPartialBlocks ? pixel_grid(lv) : kPartialBlocks;
    {
        StageScope sc("CombineAndFillBackward", stream);
        hipLaunchKernelGGL(background_grad_kernel, dim3(bg_blocks), dim3(kBlock), 0, stream, lv, bg_partial);
    }

    int want_pose = grads->grad_pose != nullptr;
    int want_intr = grads->grad_intrinsics != nullptr;
    int pt_blocks = (N + kBlock - 1) / kBlock;
    if (pt_blocks > kPartialBlocks) pt_blocks = kPartialBlocks;
    if (pt_blocks < 1) pt_blocks = 1;
    bool half = scene->texture_dtype == ADOP_TEXTURE_F16;
    for (int b = 0; b < num_views; ++b)
    {
        StageScope sc("RenderBackward", stream);
#define ADOP_LAUNCH_BWD(H, S)                                                                                       \
    hipLaunchKernelGGL((render_backward_kernel<H, S>), dim3(pt_blocks), dim3(kBlock), 0, stream, pc, dviews, lv, rp, \
                       grads->grad_texture, grads->grad_points, grads->grad_points_count, want_pose, want_intr, b,   \
                       pt_partial, stats)
        if (half && stats)
            ADOP_LAUNCH_BWD(true, true);
        else if (half)
            ADOP_LAUNCH_BWD(true, false);
        else if (stats)
            ADOP_LAUNCH_BWD(false, true);
        else
            ADOP_LAUNCH_BWD(false, false);
#undef ADOP_LAUNCH_BWD
    }
    StageScope post("Post Process Gradient", stream);
    hipLaunchKernelGGL(finalize_kernel, dim3(1), dim3(kBlock), 0, stream, dviews, num_views, C, bg_partial, bg_blocks,
                       pt_partial, pt_blocks, grads->grad_background, grads->grad_pose, grads->grad_pose_count,
                       scene->num_poses, grads->grad_intrinsics, grads->grad_intrinsics_count, scene->num_cameras,
                       scene->intrinsics_cols, params->normalize_mode, scratch);
    if (grads->grad_points && N > 0)
        hipLaunchKernelGGL(normalize_points_kernel, dim3((N + kBlock - 1) / kBlock), dim3(kBlock), 0, stream,
                           grads->grad_points, grads->grad_points_count, N, params->normalize_mode);
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
        // SAIGA_ASSERT(cam.camera_model_type == CameraModel::PINHOLE_DISTORTION), EnvironmentMap.cu:129
        if (views[b].camera_model_type != ADOP_CAMERA_PINHOLE_DISTORTION)
            return fail(ADOP_INVALID_ARG, "environment map needs the pinhole model");
        if (views[b].image_index < 0 || views[b].image_index >= scene->num_poses || views[b].camera_index < 0 ||
            views[b].camera_index >= scene->num_cameras)
            return fail(ADOP_INVALID_ARG, "view index out of range");
    }
    if (scene->intrinsics_cols != 13) return fail(ADOP_INVALID_ARG, "pinhole intrinsics need 13 columns");
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
    }
    size_t total = (size_t)lv.pix_prefix[lv.num] * lv.B;
    int grid     = (int)((total + kBlock - 1) / kBlock);
    if (grid > 0)
        hipLaunchKernelGGL(env_sample_kernel, dim3(grid), dim3(kBlock), 0, stream, chunk, scene->poses_se3,
                           scene->intrinsics, lv, ev, env_texture, env_h,
                           env_w, add_to_out);
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

adop_status adop_env_sample_backward(const adop_scene* scene, const adop_view* views, int32_t num_views, int32_t env_h,
                                     int32_t env_w, const adop_forward_buffers* buffers,
                                     const float* const* grad_out_levels, float* grad_env, void* hip_stream)
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
    }
    st = fill_async(grad_env, sizeof(float) * (size_t)scene->num_channels * env_h * env_w, 0, stream);
    if (st != ADOP_OK) return st;
    size_t total = (size_t)lv.pix_prefix[lv.num] * lv.B;
    int grid     = (int)((total + kBlock - 1) / kBlock);
    if (grid > 0)
        hipLaunchKernelGGL(env_backward_kernel, dim3(grid), dim3(kBlock), 0, stream, chunk, scene->poses_se3,
                           scene->intrinsics, lv, ev, grad_env, env_h,
                           env_w);
    ADOP_HIP_CHECK(hipGetLastError());
    return ADOP_OK;
}

adop_status adop_apply_tangent(double* tangent, double* poses_se3, int32_t num_poses, void* hip_stream)
{
    if (!tangent || !poses_se3 || num_poses < 0) return fail(ADOP_INVALID_ARG, "null argument");
    if (num_poses == 0) return ADOP_OK;
    hipLaunchKernelGGL(apply_tangent_kernel, dim3((num_poses + 127) / 128), dim3(128), 0, (hipStream_t)hip_stream,
                       tangent, poses_se3, num_poses);
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
    for (StageEvent& e : g_stage_events)
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
        g_event_pool.push_back(e.start);
        g_event_pool.push_back(e.stop);
    }
    g_stage_events.clear();
    return n;
}

const char* adop_last_error_string(void)
{
    return g_last_error.c_str();
}

const char* adop_version(void)
{
    return "adop_raster 0.1 (gfx950)";
}
}  // extern "C"
