// common.h — kernel argument structs and small device helpers shared by the rasterizer kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/adop_raster.h"
#include "device_math.h"

#pragma clang fp contract(off)

// These kernels are written for gfx950 (CDNA4) alone, and a few places lean on what that hardware does: wave64, the
// LDS and vector instructions named in the comments, and, where partial results travel between workgroups through
// agent-scope atomic stores and loads around a ticket (backward_kernels.hip, tile_kernels.hip), on stores being counted
// by vmcnt, so that s_waitcnt(0) before the ticket means they have been acknowledged.  An architecture with a separate
// store counter would need release / acquire on the ticket instead: refuse to build there rather than run wrong.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "adop_raster's kernels are written for gfx950 only (see the comment above)"
#endif

namespace adop
{
constexpr int kBlock         = 256;
constexpr int kMaxChannels   = 16;
constexpr int kPartialBlocks = 1024;  // grid of backward_ghost_kernel: per-block partial sums of the pose / intrinsics gradients
constexpr int kBgBlocks      = 2048;  // grid of interleave_kernel: per-block partial sums of the background gradient
constexpr int kPartialStride = 24;    // doubles per (block, view), 21 used: 6 pose, pose count, intr count, 13 intr
constexpr int kAcc           = 21;
constexpr int kFinalizeParts = 16;    // workgroups of the first stage of the final two-stage reduction
constexpr int kNumQueues     = 2048;  // sub-queues of the backward work queue (multiple of kBlock)
constexpr int kMaxIntrinsicsCols = 24;  // 13 pinhole / 5 affine + up to 19 polynomial coefficients
// Point cache: when a whole run of 64 points (64-aligned) is culled for a view, the record of its first point carries
// this bit pattern in x (its depth is 0 like every culled record's), so that a reader can skip the other 63 records.
constexpr uint32_t kRunCulledBits = 0x7FC0C011u;  // a quiet NaN no projection produces
constexpr uint64_t kClearPacked = (uint64_t(0x47C35000u) << 32) | 0xFFFFFFFFull;  // bits(100000.f), PointRenderer.cu:1045

// The depth kept in the point cache and in the bin entries: 0 = culled, sign bit set = dropped for this image
// (PointRenderer.cu:314-315).  Tested on the bits, so that a NaN depth (a point with NaN coordinates seen through an
// OCam) counts as a depth like any other, as in the reference, where every comparison with it is false and the point
// is blended.
__device__ __forceinline__ float signed_depth(float z, bool dropped)
{
    // (a NaN may come with either sign: only the dropout flag decides the sign bit)
    const uint32_t bits = __float_as_uint(z) & 0x7FFFFFFFu;
    return __uint_as_float(dropped ? bits | 0x80000000u : bits);
}
__device__ __forceinline__ bool depth_is_rendered(float zs)
{
    return (int32_t)__float_as_uint(zs) > 0;
}
__device__ __forceinline__ bool depth_is_dropped(float zs)
{
    return (int32_t)__float_as_uint(zs) < 0;
}

// A kernel that runs only when a flag word in the workspace has a given value (flag == nullptr: always).  The flag is
// written by an earlier launch of the same call: the first binning passes find out on the device whether the bin
// entries of the call fit a workspace with smaller bins; if not, the tile kernels return at once and the kernels of
// the direct path, queued behind them, run instead.
struct Gate
{
    const uint32_t* flag;
    uint32_t run_when;
};
__device__ __forceinline__ bool gate_closed(const Gate& g)
{
    return g.flag != nullptr && *g.flag != g.run_when;  // (kernel-uniform)
}

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
    // The resolved image in pixel-major order, [ws_pixel][C] (what the spatial gradients read at four neighbours of a
    // pixel).  Forward: where the resolve leaves it beside the planar images (the caller's pixel_cache), or null.
    // Backward: where it lies, and whether the forward wrote it (else interleave_kernel transposes `out`).
    float* irec;
    int32_t irec_ready;
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
    float4* cache;         // [B,N] projected points (ip.x, ip.y, depth or 0, LOD radius in pixels) or null
    // Direct forward path without a caller's point cache: the prepass compacts, per wavefront, the points that may
    // still pass a depth test; `cache` then holds their records in the first list_count[b][g][w] slots of the own
    // range of wavefront w of workgroup g (b * list_stride + g * list_span + w * list_span / 4 ...), list_ids the point ids.
    // Null: no lists.
    // The ranges of the last workgroup reach past n: a view's lists take list_stride >= n rounded up to whole
    // workgroups, and in list mode `cache` has B * list_stride records.
    uint32_t* list_ids;    // [B, list_stride]
    uint32_t* list_count;  // [B, number of prepass workgroups, 4]
    int32_t list_span;     // points per prepass workgroup
    size_t list_stride;    // slots per view
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

// Uniform grid of the nearest-neighbour search: cubic cells of edge `cell` from `min`, dim cells per axis.  The grid
// lives in device memory: the second one of a search is sized on the device from sampled neighbour distances.
struct KnnGrid
{
    float min[3];
    float ext[3];  // size of the bounding box
    float cell, inv_cell;
    int32_t dim[3];
    uint32_t cells;  // dim[0] * dim[1] * dim[2]
};

struct ViewChunk
{
    adop_view v[32];
};

// Up to 32 views whose constants the first kernel of a call computes on the side (count = 0: nothing to do, the
// constants were written by prepare_views launches).
struct ViewPrep
{
    ViewChunk chunk;
    int count;
    int cols;
    const double* poses;
    const float* intrinsics;
    ViewConst* out;
};

// Workspace pixel index of pixel p of level l of image b: all levels and images of a call form one array
// (B images of level 0, then B images of level 1, ...).
__device__ __forceinline__ uint32_t ws_pixel(const Levels& lv, int l, int b, uint32_t p)
{
    return (uint32_t)lv.pix_prefix[l] * (uint32_t)lv.B + (uint32_t)b * (uint32_t)(lv.l[l].w * lv.l[l].h) + p;
}

// Backward workspace: the resolved image and the upstream gradient in pixel-major order as two arrays [pixel][C], the
// image first; this is where the gradient array starts (in floats).
__device__ __forceinline__ size_t gradient_array_offset(const Levels& lv, int C)
{
    return (size_t)lv.pix_prefix[lv.num] * (size_t)lv.B * (size_t)C;
}

// Streamed data (read or written once per kernel) goes past the caches with the nontemporal hint, so that the lines
// the gathers of the same kernel reuse stay resident.
typedef float v4f __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 nt_load4(const float4* p)
{
    const v4f r = __builtin_nontemporal_load((const v4f*)p);
    return make_float4(r.x, r.y, r.z, r.w);
}
__device__ __forceinline__ void nt_store4(float4* p, float4 v)
{
    v4f r = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(r, (v4f*)p);
}

// One record of the pixel-major image: C consecutive floats (16-byte stores for C = 4 and 8: the records are aligned).
// Plain stores: with the nontemporal hint tile_blend_kernel, which writes most of them, ran 4 us longer.
template <int CT, bool NT = false>
__device__ __forceinline__ void store_pixel_record(float* __restrict__ dst, const float* v, int C)
{
    if (CT == 8 && NT)
    {
        nt_store4((float4*)dst, make_float4(v[0], v[1], v[2], v[3]));
        nt_store4((float4*)dst + 1, make_float4(v[4], v[5], v[6], v[7]));
    }
    else if (CT == 4 && NT)
        nt_store4((float4*)dst, make_float4(v[0], v[1], v[2], v[3]));
    else if (CT == 8)
    {
        ((float4*)dst)[0] = make_float4(v[0], v[1], v[2], v[3]);
        ((float4*)dst)[1] = make_float4(v[4], v[5], v[6], v[7]);
    }
    else if (CT == 4)
        ((float4*)dst)[0] = make_float4(v[0], v[1], v[2], v[3]);
    else
    {
#pragma unroll
        for (int c = 0; c < kMaxChannels; ++c)  // (unrolled: v stays in registers)
            if (c < C) dst[c] = v[c];
    }
}


template <typename T>
__device__ __forceinline__ T wave_sum(T v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    return v;
}

// counter += number of lanes with pred (one atomic per wavefront; counter passes only)
__device__ __forceinline__ void stat_add(uint64_t* dst, bool pred)
{
    unsigned long long m = __ballot(pred);
    if (m && (threadIdx.x & 63) == (__ffsll((long long)m) - 1))
        atomicAdd((unsigned long long*)dst, (unsigned long long)__popcll(m));
}

template <bool HALF>
__device__ __forceinline__ float tex_fetch(const void* tex, size_t o)
{
    if (HALF) return __half2float(((const __half*)tex)[o]);
    return ((const float*)tex)[o];
}

// the same with the nontemporal hint
template <bool HALF>
__device__ __forceinline__ float tex_fetch_stream(const void* tex, size_t o)
{
    if (HALF)
    {
        const unsigned short h = __builtin_nontemporal_load((const unsigned short*)tex + o);
        return __half2float(__ushort_as_half(h));
    }
    return __builtin_nontemporal_load((const float*)tex + o);
}

// LDS written by some lanes of a wavefront is read by other lanes of the same wavefront: DS operations of one
// wavefront execute in order, so only the compiler has to be kept from moving accesses across this point.
__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Groups the lanes of a wavefront by key.  Lanes with active == false are ignored.  For every distinct key, in
// order of its first lane, writes gkey[g] and the 64-bit lane mask gmask[g]; returns the number of groups.
// *mine (if not null) receives the group of the calling lane (-1 for inactive lanes).
// (gfx950 has no match-any instruction: one ballot per distinct key.)
__device__ __forceinline__ int wave_group_by_key(bool active, uint32_t key, uint32_t* gkey, unsigned long long* gmask,
                                                 int* mine = nullptr)
{
    const int lane               = threadIdx.x & 63;
    unsigned long long remaining = __ballot(active);
    int g                        = 0;
    int my                       = -1;
    while (remaining)
    {
        int leader           = __ffsll((long long)remaining) - 1;
        uint32_t k           = (uint32_t)__builtin_amdgcn_readlane((int)key, leader);
        bool hit             = active && key == k;
        unsigned long long m = __ballot(hit);
        if (hit) my = g;
        if (lane == leader)
        {
            gkey[g]  = k;
            gmask[g] = m;
        }
        remaining &= ~m;
        ++g;
    }
    if (mine) *mine = my;
    return g;
}

// Is grouping the wavefront's active lanes by key worth its loop (one iteration per distinct key)?  The clouds the
// library is built for are stored in spatial order, so lanes that share a pixel are mostly neighbours: the answer is
// yes when at least an eighth of the active lanes carry the key of the lane before them (a quarter: config 4 1 % faster,
// the blend of 10 M ordered points in 1920 x 1080 6 % slower; a sixteenth: config 4 3 % slower).  A cloud without
// order, or with few points per pixel of the level, says no, and pays one atomic per lane instead of 64 iterations
// for 60 keys (100 k unordered points in 256 x 256: the forward pass 0.060 -> 0.040 ms; config 4, whose level 0 holds
// few neighbours in a pixel: 1.49 -> 1.41 ms).  Wavefront-uniform.
__device__ __forceinline__ bool wave_shares_keys(bool active, uint32_t key)
{
    const uint32_t mine = active ? key : 0xFFFFFFFFu;  // (no pixel index reaches this value)
    const uint32_t prev = (uint32_t)__shfl_up((int)mine, 1, 64);
    const bool same     = active && (threadIdx.x & 63) != 0 && prev == mine;
    return 8 * __popcll(__ballot(same)) >= __popcll(__ballot(active));
}

// The same grouping without tables: every active lane gets the lane mask of its own group (0 for inactive lanes).
// The lowest lane of a mask is the group's leader; the others fetch what it holds with a cross-lane read.
__device__ __forceinline__ unsigned long long wave_group_mask(bool active, uint32_t key)
{
    unsigned long long remaining = __ballot(active);
    unsigned long long mine      = 0;
    while (remaining)
    {
        int leader           = __ffsll((long long)remaining) - 1;
        uint32_t k           = (uint32_t)__builtin_amdgcn_readlane((int)key, leader);
        bool hit             = active && key == k;
        unsigned long long m = __ballot(hit);
        if (hit) mine = m;
        remaining &= ~m;
    }
    return mine;
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
    c.no_distortion = v.camera_model_type == ADOP_CAMERA_PINHOLE_DISTORTION;
    for (int i = 0; i < 8; ++i) c.no_distortion = c.no_distortion && c.d[i] == 0.f;
    return c;
}

// The per-view constants computed inside the first kernel of a call: one block spends its first lanes on it.
__device__ __forceinline__ void prepare_views_inline(const ViewPrep& vp)
{
    if (blockIdx.x == gridDim.x - 1 && (int)threadIdx.x < vp.count)
        vp.out[threadIdx.x] = make_view_const(vp.chunk.v[threadIdx.x], vp.poses, vp.intrinsics, vp.cols);
}

// level of flattened per-image pixel index r (pix_prefix is increasing)
__device__ __forceinline__ int level_of(const Levels& lv, int r)
{
    int l = 0;
#pragma unroll
    for (int k = 1; k < ADOP_MAX_LAYERS; ++k)
        if (k < lv.num && r >= lv.pix_prefix[k]) l = k;
    return l;
}

}  // namespace adop
