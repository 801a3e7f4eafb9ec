// forward_kernels.hip — prepare_views, clear, depth prepass, blend, resolve (gfx950).
//
// Measured on MI355X: device-scope atomics (and scattered 4-byte stores) retire at ~21 G cache-line transactions/s
// no matter how many lanes of the instruction fall into the line, while 16 lanes adding into one 64-byte line cost
// one transaction.  Hence:
//   * the blend accumulates into a pixel-major workspace array (S floats per pixel: C sums + the weight, padded to
//     a power of two), so the C+1 adds of one point-level are ONE transaction instead of C+1;
//   * every workgroup first merges its point-levels per pixel in an LDS hash table (ds_add_f32 / ds_min_u64) and
//     flushes each distinct pixel once; clouds stored in Morton-ordered 256-point blocks (the reference's
//     preprocessing order) collide heavily at the coarse levels.
#include "common.h"
#include "launch.h"

#pragma clang fp contract(off)

namespace adop
{
// Once per call: the per-view constants every point kernel reads through uniform loads.
__global__ void prepare_views_kernel(ViewChunk chunk, int first, int count, const double* __restrict__ poses,
                                     const float* __restrict__ intrinsics, int cols, ViewConst* __restrict__ out)
{
    int t = threadIdx.x;
    if (t >= count) return;
    out[first + t] = make_view_const(chunk.v[t], poses, intrinsics, cols);
}

__global__ void fill_u32_kernel(uint32_t* __restrict__ p, size_t n, uint32_t v)
{
    size_t i      = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

// InitializeData (PointRenderer.cu:1039-1090): packed depth|index of every level, and the blend accumulators.
__global__ __launch_bounds__(kBlock) void clear_kernel(Levels lv, float4* __restrict__ accum, size_t accum_vec4)
{
    int per_image = lv.pix_prefix[lv.num];
    size_t total  = (size_t)per_image * lv.B;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t t0     = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (size_t t = t0; t < total; t += stride)
    {
        int b             = (int)(t / per_image);
        int r             = (int)(t - (size_t)b * per_image);
        int l             = level_of(lv, r);
        const LevelArg& L = lv.l[l];
        int p             = r - lv.pix_prefix[l];
        L.depth_index[(size_t)b * L.w * L.h + p] = kClearPacked;
    }
    const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
    for (size_t t = t0; t < accum_vec4; t += stride) accum[t] = z;
}

__device__ __forceinline__ uint64_t* depth_index_ptr(const Levels& lv, int l)
{
    uint64_t* p = lv.l[0].depth_index;
    if (l == 1) p = lv.l[1].depth_index;
    if (l == 2) p = lv.l[2].depth_index;
    if (l == 3) p = lv.l[3].depth_index;
    if (l == 4) p = lv.l[4].depth_index;
    return p;
}

__device__ __forceinline__ void depth_min_global(uint64_t* dst, uint64_t pk)
{
    // early-z (PointRenderer.cu:278): a stale value only costs a redundant atomic
    uint64_t cur = __builtin_nontemporal_load(dst);
    if (pk < cur) atomicMin((unsigned long long*)dst, (unsigned long long)pk);
}

// DepthPrepassMulti (PointRenderer.cu:203-301) on the packed buffer the reference keeps as "old rendering"
// (LayerCuda::depth_index_tensor, PackIndex): min over (depth bits << 32 | point id).
// Key of the LDS table: level << 28 | pixel.
template <int BITS>
__global__ __launch_bounds__(kBlock) void prepass_kernel(CloudArg pc, const ViewConst* __restrict__ views, Levels lv,
                                                         ParamArg rp, adop_stats* stats)
{
    constexpr int T = 1 << BITS;
    __shared__ uint32_t keys[T];
    __shared__ unsigned long long mins[T];
    __shared__ uint16_t used[T];
    __shared__ uint32_t used_count;
    const bool STATS = stats != nullptr;  // counter pass (uniform branch)

    int i      = blockIdx.x * kBlock + threadIdx.x;
    bool valid = i < pc.n;
    float4 P   = valid ? pc.position[i] : make_float4(0, 0, 0, 0);
    V3 pos     = {P.x, P.y, P.z};
    V3 nrm     = {0, 0, 0};
    if (valid && pc.normal) nrm = unpack_normal10(pc.normal[i]);

    for (int b = 0; b < lv.B; ++b)
    {
        for (int k = threadIdx.x; k < T; k += kBlock)
        {
            keys[k] = kEmptyKey;
            mins[k] = ~0ull;
        }
        if (threadIdx.x == 0) used_count = 0;
        __syncthreads();

        const ViewConst& vc = views[b];
        V2 ip;
        V3 view_p;
        float z, radius_pixels;
        bool ok = valid && project_point(vc, pc.intrinsics, pos, nrm, P.w, rp.check_normal != 0, rp.dist_cutoff,
                                         lv.l[0].w, &ip, &z, &radius_pixels, &view_p);
        bool alive = ok;
        if (STATS || ok)
        {
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
                    uint64_t pk  = ((uint64_t)f2u(z) << 32) | (uint32_t)i;
                    uint32_t pix = (uint32_t)py * (uint32_t)L.w + (uint32_t)px;
                    int slot     = table_insert<BITS>(keys, used, &used_count, ((uint32_t)l << 28) | pix);
                    if (slot >= 0)
                        atomicMin(&mins[slot], (unsigned long long)pk);
                    else
                        depth_min_global(L.depth_index + (size_t)b * L.w * L.h + pix, pk);
                }
                radius_pixels *= 0.5f;
                ip.x *= 0.5f;
                ip.y *= 0.5f;
            }
        }
        __syncthreads();
        uint32_t n = used_count;
        for (uint32_t e = threadIdx.x; e < n; e += kBlock)
        {
            uint32_t slot = used[e];
            uint32_t key  = keys[slot];
            int l         = (int)(key >> 28);
            uint32_t pix  = key & 0x0FFFFFFFu;
            size_t hw     = (size_t)lv.l[0].w * lv.l[0].h;
            if (l == 1) hw = (size_t)lv.l[1].w * lv.l[1].h;
            if (l == 2) hw = (size_t)lv.l[2].w * lv.l[2].h;
            if (l == 3) hw = (size_t)lv.l[3].w * lv.l[3].h;
            if (l == 4) hw = (size_t)lv.l[4].w * lv.l[4].h;
            depth_min_global(depth_index_ptr(lv, l) + (size_t)b * hw + pix, (uint64_t)mins[slot]);
        }
        __syncthreads();
    }
}

// RenderForwardMulti (PointRenderer.cu:303-393).  CT = compile-time channel count (0: runtime lv.C <= 16).
// Key of the LDS table: workspace pixel index (ws_pixel).  accum: S floats per workspace pixel.
template <int CT, int BITS, bool HALF>
__global__ __launch_bounds__(kBlock) void blend_kernel(CloudArg pc, const ViewConst* __restrict__ views, Levels lv,
                                                       ParamArg rp, float* __restrict__ accum, int S,
                                                       adop_stats* stats)
{
    constexpr int T    = 1 << BITS;
    constexpr int CMAX = CT ? CT : kMaxChannels;
    __shared__ uint32_t keys[T];
    __shared__ uint16_t used[T];
    __shared__ uint32_t used_count;
    extern __shared__ float vals[];  // T * (C+1)
    const bool STATS = stats != nullptr;  // counter pass (uniform branch)

    const int C  = CT ? CT : lv.C;
    const int C1 = C + 1;

    int i      = blockIdx.x * kBlock + threadIdx.x;
    bool valid = i < pc.n;
    float4 P   = valid ? pc.position[i] : make_float4(0, 0, 0, 0);
    V3 pos     = {P.x, P.y, P.z};
    V3 nrm     = {0, 0, 0};
    if (valid && pc.normal) nrm = unpack_normal10(pc.normal[i]);
    int tex_index = valid ? pc.index[i] : 0;
    bool tex_ok   = (unsigned)tex_index < (unsigned)pc.num_texels;  // device assert :362
    const float accept = rp.depth_accept + 1;

    float t[CMAX];
    bool t_loaded = false;

    for (int b = 0; b < lv.B; ++b)
    {
        for (int k = threadIdx.x; k < T; k += kBlock) keys[k] = kEmptyKey;
        for (int k = threadIdx.x; k < T * C1; k += kBlock) vals[k] = 0.f;
        if (threadIdx.x == 0) used_count = 0;
        __syncthreads();

        bool dropped = valid && pc.dropout && pc.dropout[(size_t)b * pc.n + i] == 1.f;  // :314-315
        const ViewConst& vc = views[b];
        V2 ip;
        V3 view_p;
        float z, radius_pixels;
        bool ok = valid && !dropped &&
                  project_point(vc, pc.intrinsics, pos, nrm, P.w, rp.check_normal != 0, rp.dist_cutoff, lv.l[0].w, &ip,
                                &z, &radius_pixels, &view_p);
        if (STATS) stat_add(&stats->bad_index, ok && !tex_ok);
        ok         = ok && tex_ok;
        bool alive = ok;
        if (STATS || ok)
        {
#pragma unroll
            for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
            {
                if (l >= lv.num) break;
                if (rp.drop_by_radius && radius_pixels < rp.drop_threshold) alive = false;
                const LevelArg& L = lv.l[l];
                int px = f2i_rn(ip.x), py = f2i_rn(ip.y);
                bool in  = alive && (unsigned)px < (unsigned)L.w && (unsigned)py < (unsigned)L.h;
                bool acc = false;
                if (in)
                {
                    size_t hw    = (size_t)L.w * L.h;
                    uint32_t pix = (uint32_t)py * (uint32_t)L.w + (uint32_t)px;
                    // high word of the packed pixel = depth
                    float image_depth = __uint_as_float((uint32_t)(L.depth_index[(size_t)b * hw + pix] >> 32));
                    acc               = !(z > image_depth * accept);  // :380
                    if (acc)
                    {
                        if (!t_loaded)
                        {
#pragma unroll
                            for (int c = 0; c < CMAX; ++c)
                                if (c < C) t[c] = tex_fetch<HALF>(pc.texture, (size_t)c * pc.num_texels + tex_index);
                            t_loaded = true;
                        }
                        uint32_t gp = ws_pixel(lv, l, b, pix);
                        int slot    = table_insert<BITS>(keys, used, &used_count, gp);
                        if (slot >= 0)
                        {
                            float* v = vals + slot * C1;
#pragma unroll
                            for (int c = 0; c < CMAX; ++c)
                                if (c < C) atomicAdd(v + c, t[c]);
                            atomicAdd(v + C, 1.f);
                        }
                        else
                        {
                            float* g = accum + (size_t)gp * S;
#pragma unroll
                            for (int c = 0; c < CMAX; ++c)
                                if (c < C) unsafeAtomicAdd(g + c, t[c]);
                            unsafeAtomicAdd(g + C, 1.f);
                        }
                    }
                }
                if (STATS) stat_add(&stats->accepted[l], acc);
                radius_pixels *= 0.5f;
                ip.x *= 0.5f;
                ip.y *= 0.5f;
            }
        }
        __syncthreads();
        // flush: S consecutive lanes add the C+1 sums of one pixel into one cache line
        uint32_t n    = used_count;
        int lane      = threadIdx.x % S;
        int group     = threadIdx.x / S;
        int groups    = kBlock / S;
        for (uint32_t e = group; e < n; e += groups)
        {
            uint32_t slot = used[e];
            uint32_t gp   = keys[slot];
            if (lane < C1) unsafeAtomicAdd(accum + (size_t)gp * S + lane, vals[slot * C1 + lane]);
        }
        __syncthreads();
    }
}

// CombineAndFill (:726-754) + CreateMask (:828-847) + the f32 depth the reference saves for backward.
// Reads the pixel-major accumulators, writes the planar [B,C,h,w] image, weight, depth and mask.
template <int CT>
__global__ __launch_bounds__(kBlock) void resolve_kernel(Levels lv, const float* __restrict__ accum, int S,
                                                         const float* __restrict__ background, int write_mask,
                                                         float mask_value)
{
    constexpr int CMAX = CT ? CT : kMaxChannels;
    const int C        = CT ? CT : lv.C;
    int per_image      = lv.pix_prefix[lv.num];
    size_t total       = (size_t)per_image * lv.B;
    size_t stride      = (size_t)gridDim.x * blockDim.x;
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride)
    {
        int b             = (int)(t / per_image);
        int r             = (int)(t - (size_t)b * per_image);
        int l             = level_of(lv, r);
        const LevelArg& L = lv.l[l];
        int p             = r - lv.pix_prefix[l];
        size_t hw         = (size_t)L.w * L.h;
        size_t o          = (size_t)b * hw + p;
        const float* a    = accum + (size_t)ws_pixel(lv, l, b, (uint32_t)p) * S;
        float v[CMAX + 1];
        if (CT == 8)
        {
            const float4* a4 = (const float4*)a;
            float4 q0 = a4[0], q1 = a4[1];
            v[0] = q0.x; v[1] = q0.y; v[2] = q0.z; v[3] = q0.w;
            v[4] = q1.x; v[5] = q1.y; v[6] = q1.z; v[7] = q1.w;
            v[8] = a[8];
        }
        else if (CT == 4)
        {
            const float4* a4 = (const float4*)a;
            float4 q0 = a4[0];
            v[0] = q0.x; v[1] = q0.y; v[2] = q0.z; v[3] = q0.w;
            v[4] = a[4];
        }
        else
        {
#pragma unroll
            for (int c = 0; c <= CMAX; ++c)
                if (c <= C) v[c] = a[c];
        }
        float cou   = v[C];
        L.weight[o] = cou;
        L.depth[o]  = __uint_as_float((uint32_t)(L.depth_index[o] >> 32));
        float* out  = L.out + (size_t)b * C * hw + p;
#pragma unroll
        for (int c = 0; c < CMAX; ++c)
            if (c < C) out[(size_t)c * hw] = (cou == 0) ? background[c] : v[c] / cou;
        if (write_mask && L.mask) L.mask[o] = (cou == 0) ? mask_value : 1.f;
    }
}


// ------------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------------
constexpr int kPrepassBits = 10;  // LDS table of the prepass: 1024 slots x 14 B
constexpr int kBlendBits   = 9;   // LDS table of the blend: 512 slots x (6 + 4(C+1)) B

void launch_prepare_views(const ViewChunk& ch, int first, int count, const double* poses, const float* intrinsics,
                          int cols, ViewConst* out, hipStream_t st)
{
    hipLaunchKernelGGL(prepare_views_kernel, dim3(1), dim3(32), 0, st, ch, first, count, poses, intrinsics, cols, out);
}

void launch_fill_u32(uint32_t* p, size_t n, uint32_t v, hipStream_t st)
{
    size_t want = (n + kBlock - 1) / kBlock;
    int grid    = (int)(want < 8192 ? (want ? want : 1) : 8192);
    hipLaunchKernelGGL(fill_u32_kernel, dim3(grid), dim3(kBlock), 0, st, p, n, v);
}

void launch_clear(const Levels& lv, int grid, float* accum, size_t accum_floats, hipStream_t st)
{
    hipLaunchKernelGGL(clear_kernel, dim3(grid), dim3(kBlock), 0, st, lv, (float4*)accum, accum_floats / 4);
}

void launch_prepass(const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp, adop_stats* stats,
                    hipStream_t st)
{
    int grid = (pc.n + kBlock - 1) / kBlock;
    if (grid < 1) return;
    hipLaunchKernelGGL((prepass_kernel<kPrepassBits>), dim3(grid), dim3(kBlock), 0, st, pc, views, lv, rp, stats);
}

template <int CT, bool HALF>
static void launch_blend_t(const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp,
                           float* accum, int S, adop_stats* stats, hipStream_t st)
{
    int grid   = (pc.n + kBlock - 1) / kBlock;
    size_t lds = sizeof(float) * ((size_t)1 << kBlendBits) * (size_t)(lv.C + 1);
    hipLaunchKernelGGL((blend_kernel<CT, kBlendBits, HALF>), dim3(grid), dim3(kBlock), lds, st, pc, views, lv, rp,
                       accum, S, stats);
}

void launch_blend(const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp, bool half,
                  float* accum, int S, adop_stats* stats, hipStream_t st)
{
    if (pc.n < 1) return;
    if (lv.C == 8)
        half ? launch_blend_t<8, true>(pc, views, lv, rp, accum, S, stats, st)
             : launch_blend_t<8, false>(pc, views, lv, rp, accum, S, stats, st);
    else if (lv.C == 4)
        half ? launch_blend_t<4, true>(pc, views, lv, rp, accum, S, stats, st)
             : launch_blend_t<4, false>(pc, views, lv, rp, accum, S, stats, st);
    else
        half ? launch_blend_t<0, true>(pc, views, lv, rp, accum, S, stats, st)
             : launch_blend_t<0, false>(pc, views, lv, rp, accum, S, stats, st);
}

void launch_resolve(const Levels& lv, int grid, const float* accum, int S, const float* background, int write_mask,
                    float mask_value, hipStream_t st)
{
    if (lv.C == 8)
        hipLaunchKernelGGL((resolve_kernel<8>), dim3(grid), dim3(kBlock), 0, st, lv, accum, S, background, write_mask,
                           mask_value);
    else if (lv.C == 4)
        hipLaunchKernelGGL((resolve_kernel<4>), dim3(grid), dim3(kBlock), 0, st, lv, accum, S, background, write_mask,
                           mask_value);
    else
        hipLaunchKernelGGL((resolve_kernel<0>), dim3(grid), dim3(kBlock), 0, st, lv, accum, S, background, write_mask,
                           mask_value);
}

}  // namespace adop
