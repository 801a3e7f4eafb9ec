// forward_kernels.hip — prepare_views, clear, depth prepass, blend, resolve (gfx950).
//
// Measured on MI355X: device-scope atomics (and scattered 4-byte stores) retire at ~21 G cache-line transactions/s
// no matter how many lanes of the instruction fall into the line, while 16 lanes adding into one 64-byte line cost
// one transaction.  Hence:
//   * the blend accumulates into a pixel-major workspace array (S floats per pixel: C sums + the weight, padded to
//     a power of two), so the C+1 adds of one point-level are ONE transaction instead of C+1;
//   * every wavefront first merges its point-levels per pixel (ballot grouping + plain LDS reads, no LDS atomics:
//     two variants built on ds_add_f32 / ds_cmpst - a workgroup hash table and a per-wavefront leader election -
//     were measured 1.8-2.2x slower) and issues one transaction per distinct pixel; clouds stored in Morton-ordered 256-point blocks
//     (the reference's preprocessing order) collide heavily at the coarse levels.
#include <stdlib.h>

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
    for (; i < n; i += stride) __builtin_nontemporal_store(v, p + i);
}

// InitializeData (PointRenderer.cu:1039-1090): packed depth|index of every level, and the blend accumulators.
// Levels below first_level are left alone (the tile path writes them itself).
__global__ __launch_bounds__(kBlock) void clear_kernel(Levels lv, int first_level, float4* __restrict__ accum,
                                                       size_t accum_vec4, uint32_t* __restrict__ zero_u32, int zero_n,
                                                       ViewPrep vp, Gate gate, adop_stats* zero_stats)
{
    if (gate_closed(gate)) return;
    prepare_views_inline(vp);
    // (the direct path taking over from the tile path counts the point-levels again)
    if (zero_stats && blockIdx.x == 0 && threadIdx.x < sizeof(adop_stats) / sizeof(uint64_t))
        ((uint64_t*)zero_stats)[threadIdx.x] = 0;
    // counters of the tile bins (tile path only)
    for (int k = blockIdx.x * blockDim.x + threadIdx.x; k < zero_n; k += gridDim.x * blockDim.x) zero_u32[k] = 0;
    int r0        = lv.pix_prefix[first_level];
    int per_image = lv.pix_prefix[lv.num] - r0;
    size_t total  = (size_t)per_image * lv.B;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t t0     = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (size_t t = t0; t < total; t += stride)
    {
        int b             = (int)(t / per_image);
        int r             = r0 + (int)(t - (size_t)b * per_image);
        int l             = level_of(lv, r);
        const LevelArg& L = lv.l[l];
        int p             = r - lv.pix_prefix[l];
        L.depth_index[(size_t)b * L.w * L.h + p] = kClearPacked;
    }
    const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
    for (size_t t = t0; t < accum_vec4; t += stride) accum[t] = z;
}

// DepthPrepassMulti (PointRenderer.cu:203-301) on the packed buffer the reference keeps as "old rendering"
// (LayerCuda::depth_index_tensor, PackIndex): min over (depth bits << 32 | point id).
// Every thread handles PPT points (all their loads are issued before anything waits: the kernel is bound by memory
// latency, not by arithmetic).  Per level and 64-point run the lanes that survive the early-z read are grouped by
// pixel, one lane per distinct pixel takes the minimum of its group from LDS and issues the 64-bit atomicMin:
// clouds stored in Morton-ordered blocks collide heavily at the coarse levels, and a device-scope atomic costs one
// memory transaction whatever it carries.
template <int PPT>
__global__ __launch_bounds__(kBlock) void prepass_kernel(CloudArg pc, const ViewConst* __restrict__ views, Levels lv,
                                                         ParamArg rp, int group_from, adop_stats* stats, Gate gate)
{
    __shared__ unsigned long long s_pk[kBlock];
    if (gate_closed(gate)) return;
    __shared__ unsigned long long s_gmask[kBlock];
    __shared__ uint32_t s_gkey[kBlock];
    const bool STATS = stats != nullptr;  // counter pass (uniform branch)
    const int lane   = threadIdx.x & 63;
    const int wbase  = threadIdx.x & ~63;
    unsigned long long* pk_w    = s_pk + wbase;
    unsigned long long* gmask_w = s_gmask + wbase;
    uint32_t* gkey_w            = s_gkey + wbase;

    const int base = blockIdx.x * (kBlock * PPT) + threadIdx.x;
    float4 P[PPT];
    int32_t nenc[PPT];
#pragma unroll
    for (int k = 0; k < PPT; ++k)
    {
        int i   = base + k * kBlock;
        P[k]    = i < pc.n ? pc.position[i] : make_float4(0, 0, 0, 0);
        nenc[k] = (i < pc.n && pc.normal) ? pc.normal[i] : 0;
    }

    const ImageBox box = image_box(lv);
    for (int b = 0; b < lv.B; ++b)
    {
        const ViewConst& vc = views[b];
        const bool sparse = lv.B > 1 && b < 64 && !STATS;  // (the cache records of a run outside the view: see below)
        // phase 1: projection, pixel of every level and the early-z read (PointRenderer.cu:278) of the depth word;
        // the loads are independent.  A stale value only costs a redundant atomic.
        uint32_t pix[PPT][ADOP_MAX_LAYERS];
        uint32_t cur[PPT][ADOP_MAX_LAYERS];
        uint32_t inmask[PPT];
        float zz[PPT];
        float4 rec[PPT];  // list mode: the record of a point that may still pass a depth test (depth 0: none)
        bool okk[PPT];
#pragma unroll
        for (int k = 0; k < PPT; ++k)
        {
            int i      = base + k * kBlock;
            bool valid = i < pc.n;
            V3 pos     = {P[k].x, P[k].y, P[k].z};
            V3 nrm     = unpack_normal10(nenc[k]);
            V2 ip = {0.f, 0.f};
            float radius_pixels = 0.f;
            // (keeping the point in the uncropped image from one crop of a frame to the next, as the tile path does,
            // costs this kernel more in registers than it saves: a single view of 100 M points ran 17 % slower)
            V3 view_p;
            V2 frame_p = {0.f, 0.f};
            float z    = 0.f;
            if (valid) project_frame(vc, pc.intrinsics, pos, nrm, rp.check_normal != 0, rp.dist_cutoff, &frame_p, &z, &view_p);
            const bool ok = z != 0;
            if (ok) ip = k_apply(vc.crop, frame_p);
            // a crop sees a small part of the cloud: most runs of 64 points are nowhere near it and skip the levels
            const bool near_image = __ballot(ok && !outside_every_level(box, ip)) != 0;  // wavefront-uniform
            if (ok && rp.drop_by_radius && (near_image || !sparse)) radius_pixels = crop_radius(vc, z, P[k].w, lv.l[0].w);
            zz[k]      = z;
            inmask[k]  = 0;
            rec[k]     = make_float4(ip.x, ip.y, 0.f, radius_pixels);
            okk[k]     = ok;
            bool alive = ok;
#pragma unroll
            for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
            {
                pix[k][l] = 0;
                cur[k][l] = 0;
                if (l < lv.num && near_image)
                {
                    if (rp.drop_by_radius && radius_pixels < rp.drop_threshold) alive = false;  // break, :261-264
                    const LevelArg& L = lv.l[l];
                    int px = f2i_rn(ip.x), py = f2i_rn(ip.y);
                    bool in = alive && (unsigned)px < (unsigned)L.w && (unsigned)py < (unsigned)L.h;
                    if (STATS) stat_add(&stats->visible[l], in);
                    if (in)
                    {
                        inmask[k] |= 1u << l;
                        pix[k][l] = (uint32_t)py * (uint32_t)L.w + (uint32_t)px;
                        size_t o  = (size_t)b * L.w * L.h + pix[k][l];
                        // (a cached read: with the nontemporal hint a dense cloud - 43 points per pixel - fetched 6 GB
                        // per pass for these words and ran 28 % slower)
                        cur[k][l] = ((const uint32_t*)L.depth_index)[2 * o + 1];
                    }
                    radius_pixels *= 0.5f;
                    ip.x *= 0.5f;
                    ip.y *= 0.5f;
                }
            }
        }
        // The blend (and the backward pass, if the caller keeps the buffer) read the projected points from the cache
        // instead of projecting again; the sign of the depth carries the dropout flag (only the flags of points in the
        // image are read; the counter pass reads those of all projected points).  A run of 64 points none of which
        // lands in the image at any level (a crop sees a small part of the cloud): its first record says so
        // (kRunCulledBits).  The readers of a batch of views look at that record first and skip the run, so its other
        // records are not written at all (views 0..63, no counter pass).
        if (pc.cache && !pc.list_ids)
        {
#pragma unroll
            for (int k = 0; k < PPT; ++k)
            {
                const int i       = base + k * kBlock;
                const bool culled = !__ballot(inmask[k] != 0);  // wavefront-uniform
                if (culled && sparse)
                {
                    if (lane == 0 && i < pc.n)
                        pc.cache[(size_t)b * pc.n + i] = make_float4(__uint_as_float(kRunCulledBits), 0, 0, 0);
                }
                else if (i < pc.n)
                {
                    const bool dropped = (inmask[k] != 0 || (STATS && okk[k])) && pc.dropout && pc.dropout[(size_t)b * pc.n + i] == 1.f;
                    float4 r = okk[k] ? make_float4(rec[k].x, rec[k].y, signed_depth(zz[k], dropped), rec[k].w)
                                      : make_float4(0, 0, 0, 0);
                    if (culled && lane == 0) r = make_float4(__uint_as_float(kRunCulledBits), 0, 0, 0);
                    pc.cache[(size_t)b * pc.n + i] = r;
                }
            }
        }
        // List mode: the points of every wavefront that may still pass a depth test, compacted into the first slots of
        // the wavefront's own range (no LDS, no barrier, no atomics).  In a dense cloud they are a few percent,
        // scattered over all wavefronts; the blend packs the four lists of a workgroup and runs on full wavefronts of
        // them instead of on every wavefront of the cloud.
        if (pc.list_ids)  // kernel-uniform
        {
            const int wave     = threadIdx.x >> 6;
            const size_t range = (size_t)b * pc.list_stride + (size_t)blockIdx.x * (kBlock * PPT) + (size_t)wave * (64 * PPT);
            uint32_t before    = 0;
#pragma unroll
            for (int k = 0; k < PPT; ++k)
            {
                // (only here are the early-z words looked at: all their loads were issued before anything waits)
                // The depth only decreases from the value read: a point behind its band is behind the band of the
                // final depth (:380).  The counter pass keeps every projected point: the blend counts texel indices
                // out of range for them.  Dropped points are not blended (:314-315).
                const int i = base + k * kBlock;
                bool cand   = false;
#pragma unroll
                for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
                    if (inmask[k] >> l & 1u) cand |= !(zz[k] > __uint_as_float(cur[k][l]) * (rp.depth_accept + 1));
                if (STATS) cand = okk[k];
                if (cand && pc.dropout && pc.dropout[(size_t)b * pc.n + i] == 1.f) cand = false;
                if (cand) rec[k].z = zz[k];
                const unsigned long long m = __ballot(cand);
                if (cand)
                {
                    const size_t slot = range + before + (uint32_t)__popcll(m & ((1ull << lane) - 1ull));
                    pc.cache[slot]    = rec[k];
                    pc.list_ids[slot] = (uint32_t)i;
                }
                before += (uint32_t)__popcll(m);
            }
            if (lane == 0)
                pc.list_count[((size_t)b * gridDim.x + blockIdx.x) * (kBlock / 64) + wave] = before;
        }
        // phase 2: per 64-point run and level, the surviving lanes are grouped by pixel; one atomicMin per group
#pragma unroll
        for (int k = 0; k < PPT; ++k)
        {
            const uint32_t zbits = f2u(zz[k]);
            uint32_t cmask       = 0;
#pragma unroll
            for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
                if ((inmask[k] >> l & 1u) && zbits <= cur[k][l]) cmask |= 1u << l;  // equal depth: the index decides
            if (!__ballot(cmask != 0)) continue;  // wavefront-uniform
            const uint64_t pk = ((uint64_t)zbits << 32) | (uint32_t)(base + k * kBlock);
            wave_lds_sync();  // readers of the previous run are done
            pk_w[lane] = pk;
#pragma unroll
            for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
            {
                if (l >= lv.num) break;
                const bool cand = cmask >> l & 1u;
                if (!__ballot(cand)) continue;
                const LevelArg& L = lv.l[l];
                uint64_t* dst     = L.depth_index + (size_t)b * L.w * L.h;
                if (l < group_from || !wave_shares_keys(cand, pix[k][l]))
                {
                    // fine levels, or a cloud without order / with few points per pixel: few lanes of the wavefront
                    // share a pixel, grouping would cost more than it saves
                    if (cand) atomicMin((unsigned long long*)(dst + pix[k][l]), (unsigned long long)pk);
                    continue;
                }
                wave_lds_sync();
                int G = wave_group_by_key(cand, pix[k][l], gkey_w, gmask_w);
                wave_lds_sync();
                if (lane < G)
                {
                    unsigned long long m  = gmask_w[lane];
                    unsigned long long mn = ~0ull;
                    while (m)
                    {
                        int bit = __ffsll((long long)m) - 1;
                        m &= m - 1;
                        unsigned long long v = pk_w[bit];
                        mn                   = v < mn ? v : mn;
                    }
                    atomicMin((unsigned long long*)(dst + gkey_w[lane]), mn);
                }
            }
        }
    }
}

// RenderForwardMulti (PointRenderer.cu:303-393).  CT = compile-time channel count (0: runtime lv.C <= 16).
// accum: S floats per workspace pixel (C sums + weight, padded to a power of two).
// Per level every wavefront groups its accepted lanes by pixel; LG = max(S,8) consecutive lanes then sum the
// staged descriptors of one group (lane j = channel j, lane C = the count) and add them with ONE cache-line atomic.
template <int CT, bool HALF>
__global__ __launch_bounds__(kBlock) void blend_kernel(CloudArg pc, const ViewConst* __restrict__ views, Levels lv,
                                                       ParamArg rp, float* __restrict__ accum, int S,
                                                       adop_stats* stats, int group_from, Gate gate)
{
    constexpr int CMAX = CT ? CT : kMaxChannels;
    __shared__ unsigned long long s_gmask[kBlock];
    __shared__ uint32_t s_gkey[kBlock];
    extern __shared__ float s_stage[];  // kBlock * C descriptors of the block's points
    if (gate_closed(gate)) return;
    const bool STATS = stats != nullptr;  // counter pass (uniform branch)
    const int C      = CT ? CT : lv.C;
    const int lane   = threadIdx.x & 63;
    const int wbase  = threadIdx.x & ~63;
    unsigned long long* gmask_w = s_gmask + wbase;
    uint32_t* gkey_w            = s_gkey + wbase;
    float* stage_w              = s_stage + wbase * C;
    const int LG                = S < 8 ? 8 : S;  // lanes per group in the accumulate phase
    const int sub               = lane / LG;
    const int j                 = lane - sub * LG;
    const int subs              = 64 / LG;

    const float accept = rp.depth_accept + 1;

    // phases 1-3 for one projected point of view b in every lane (ok: the lane has one)
    auto blend_point = [&](int b, bool ok, V2 ip, float z, float radius_pixels, int tex_index, bool tex_ok,
                           bool& staged)
    {
        if (STATS) stat_add(&stats->bad_index, ok && !tex_ok);
        ok = ok && tex_ok;
        if (!__ballot(ok) && !STATS) return;  // wavefront-uniform

        // The descriptors are requested together with the depth words (one memory round trip instead of two); points
        // that end up rejected at every level fetch them in vain, which costs less than the extra latency.
        float t[CMAX];
        const bool want_t = ok && !staged;
        if (want_t)
        {
#pragma unroll
            for (int c = 0; c < CMAX; ++c)
                if (c < C) t[c] = tex_fetch<HALF>(pc.texture, (size_t)c * pc.num_texels + tex_index);
        }
        // phase 1: pixel of every level and the depth test (all depth loads are independent)
        uint32_t gp[ADOP_MAX_LAYERS];
        bool acc[ADOP_MAX_LAYERS];
        {
            uint32_t dw[ADOP_MAX_LAYERS];
            bool in[ADOP_MAX_LAYERS];
            bool alive = ok;
#pragma unroll
            for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
            {
                in[l] = false;
                gp[l] = 0;
                dw[l] = 0;
                if (l < lv.num)
                {
                    if (rp.drop_by_radius && radius_pixels < rp.drop_threshold) alive = false;
                    const LevelArg& L = lv.l[l];
                    int px = f2i_rn(ip.x), py = f2i_rn(ip.y);
                    in[l] = alive && (unsigned)px < (unsigned)L.w && (unsigned)py < (unsigned)L.h;
                    if (in[l])
                    {
                        uint32_t pix = (uint32_t)py * (uint32_t)L.w + (uint32_t)px;
                        size_t o     = (size_t)b * L.w * L.h + pix;
                        dw[l]        = ((const uint32_t*)L.depth_index)[2 * o + 1];  // high word = depth bits
                        gp[l]        = ws_pixel(lv, l, b, pix);
                    }
                    radius_pixels *= 0.5f;
                    ip.x *= 0.5f;
                    ip.y *= 0.5f;
                }
            }
#pragma unroll
            for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
            {
                acc[l] = in[l] && !(z > __uint_as_float(dw[l]) * accept);  // :380
                if (STATS && l < lv.num) stat_add(&stats->accepted[l], acc[l]);
            }
        }
        bool any = false;
#pragma unroll
        for (int l = 0; l < ADOP_MAX_LAYERS; ++l) any |= acc[l];
        if (!__ballot(any)) return;  // wavefront-uniform

        // phase 2: stage the descriptors of this point (the same for every level and view)
        if (want_t)
        {
#pragma unroll
            for (int c = 0; c < CMAX; ++c)
                if (c < C) stage_w[lane * C + c] = t[c];
            staged = true;
        }

        // phase 3: per level, one cache-line atomic per distinct pixel of the wavefront
#pragma unroll
        for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
        {
            if (l >= lv.num) break;
            const unsigned long long bal = __ballot(acc[l]);
            if (!bal) continue;
            wave_lds_sync();
            int G;
            if (l < group_from || !wave_shares_keys(acc[l], gp[l]))
            {
                // fine level, or a cloud without order / with few points per pixel: few lanes of the wavefront share a
                // pixel; every accepted lane is its own entry
                G = __popcll(bal);
                if (acc[l])
                {
                    int e      = __popcll(bal & ((1ull << lane) - 1ull));
                    gkey_w[e]  = gp[l];
                    gmask_w[e] = 1ull << lane;
                }
            }
            else
                G = wave_group_by_key(acc[l], gp[l], gkey_w, gmask_w);
            wave_lds_sync();
            for (int g0 = 0; g0 < G; g0 += subs)
            {
                int g = g0 + sub;
                if (g < G && j <= C)
                {
                    unsigned long long m = gmask_w[g];
                    float sum;
                    if (j < C)
                    {
                        sum = 0.f;
                        while (m)
                        {
                            int bit = __ffsll((long long)m) - 1;
                            m &= m - 1;
                            sum += stage_w[bit * C + j];
                        }
                    }
                    else
                        sum = (float)__popcll(m);
                    unsafeAtomicAdd(accum + (size_t)gkey_w[g] * S + j, sum);
                }
            }
        }
    };

    if (pc.list_ids)  // kernel-uniform: the points that survived the prepass, one list per prepass wavefront
    {
        static_assert(kBlock / 64 == 4, "four lists per prepass workgroup");
        const uint32_t per_wave = (uint32_t)pc.list_span / 4;
        for (int b = 0; b < lv.B; ++b)
        {
            const uint4 c = *(const uint4*)(pc.list_count + ((size_t)b * gridDim.x + blockIdx.x) * 4);
            const uint32_t p1 = c.x, p2 = p1 + c.y, p3 = p2 + c.z, n = p3 + c.w;
            const size_t range = (size_t)b * pc.list_stride + (size_t)blockIdx.x * pc.list_span;
            for (uint32_t t0 = 0; t0 < n; t0 += blockDim.x)
            {
                const uint32_t t = t0 + threadIdx.x;
                const bool valid = t < n;
                // the four lists back to back: list w holds the items [p_w, p_{w+1})
                const uint32_t w   = (t >= p1) + (t >= p2) + (t >= p3);
                const uint32_t off = t - (w == 0 ? 0u : (w == 1 ? p1 : (w == 2 ? p2 : p3)));
                const size_t slot  = range + (size_t)w * per_wave + off;
                const float4 R     = valid ? pc.cache[slot] : make_float4(0, 0, 0, 0);
                const int i        = valid ? (int)pc.list_ids[slot] : 0;
                int tex_index      = valid ? pc.index[i] : 0;
                bool tex_ok        = (unsigned)tex_index < (unsigned)pc.num_texels;  // device assert :362
                bool staged        = false;
                wave_lds_sync();  // the staged descriptors of the previous round are no longer read
                blend_point(b, valid && depth_is_rendered(R.z), V2{R.x, R.y}, R.z, R.w, tex_index, tex_ok, staged);
            }
        }
        return;
    }

    int i      = blockIdx.x * kBlock + threadIdx.x;
    bool valid = i < pc.n;
    int tex_index = valid ? pc.index[i] : 0;
    bool tex_ok   = (unsigned)tex_index < (unsigned)pc.num_texels;  // device assert :362
    bool staged = false;
    float4 P    = make_float4(0, 0, 0, 0);
    V3 nrm      = {0, 0, 0};
    if (!pc.cache)  // kernel-uniform: no point cache, project again
    {
        if (valid) P = pc.position[i];
        if (valid && pc.normal) nrm = unpack_normal10(pc.normal[i]);
    }

    // Several views: the prepass marked the runs of 64 points that miss a view entirely in their first record
    // (kRunCulledBits); lane b asks for view b, all at once, and the records of such runs are not read.
    unsigned long long culled_views = 0;
    if (pc.cache && lv.B > 1)
    {
        const int lane  = threadIdx.x & 63;
        const int first = i & ~63;
        bool c          = false;
        if (lane < lv.B && first < pc.n)
        {
            const float4 head = pc.cache[(size_t)lane * pc.n + first];
            c                 = __float_as_uint(head.x) == kRunCulledBits && head.z == 0.f;
        }
        culled_views = __ballot(c);
    }
    for (int b = 0; b < lv.B; ++b)
    {
        if (b < 64 && (culled_views >> b & 1ull) != 0 && !STATS) continue;  // wavefront-uniform
        V2 ip = {0.f, 0.f};
        float z = 0.f, radius_pixels = 0.f;
        bool ok;
        if (pc.cache)
        {
            // projected by the depth prepass of this call; dropped points (:314-315) carry a negative depth
            const float4 R = valid ? pc.cache[(size_t)b * pc.n + i] : make_float4(0, 0, 0, 0);
            ip             = {R.x, R.y};
            z              = R.z;
            radius_pixels  = R.w;
            ok             = valid && depth_is_rendered(z);
        }
        else
        {
            bool dropped = valid && pc.dropout && pc.dropout[(size_t)b * pc.n + i] == 1.f;  // :314-315
            V3 pos = {P.x, P.y, P.z};
            V3 view_p;
            ok = valid && !dropped &&
                 project_point(views[b], pc.intrinsics, pos, nrm, P.w, rp.check_normal != 0, rp.dist_cutoff, lv.l[0].w, &ip,
                               &z, &radius_pixels, &view_p);
        }
        blend_point(b, ok, ip, z, radius_pixels, tex_index, tex_ok, staged);
    }
}

// CombineAndFill (:726-754) + CreateMask (:828-847) + the f32 depth the reference saves for backward.
// Reads the pixel-major accumulators, writes the planar [B,C,h,w] image, weight, depth and mask.
template <int CT>
__global__ __launch_bounds__(kBlock) void resolve_kernel(Levels lv, int first_level, const float* __restrict__ accum,
                                                         int S, const float* __restrict__ background, int write_mask,
                                                         float mask_value, Gate gate)
{
    constexpr int CMAX = CT ? CT : kMaxChannels;
    if (gate_closed(gate)) return;
    const int C        = CT ? CT : lv.C;
    int r0             = lv.pix_prefix[first_level];
    int per_image      = lv.pix_prefix[lv.num] - r0;
    size_t total       = (size_t)per_image * lv.B;
    size_t stride      = (size_t)gridDim.x * blockDim.x;
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride)
    {
        int b             = (int)(t / per_image);
        int r             = r0 + (int)(t - (size_t)b * per_image);
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
            if (c < C)
            {
                v[c]               = (cou == 0) ? background[c] : v[c] / cou;
                out[(size_t)c * hw] = v[c];
            }
        if (write_mask && L.mask) L.mask[o] = (cou == 0) ? mask_value : 1.f;
        if (lv.irec) store_pixel_record<CT, true>(lv.irec + (size_t)ws_pixel(lv, l, b, (uint32_t)p) * C, v, C);
    }
}


// ------------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------------
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

void launch_clear(const Levels& lv, int first_level, int grid, float* accum, size_t accum_floats, uint32_t* zero_u32,
                  int zero_n, const ViewPrep& vp, hipStream_t st, Gate gate, adop_stats* zero_stats)
{
    hipLaunchKernelGGL(clear_kernel, dim3(grid), dim3(kBlock), 0, st, lv, first_level, (float4*)accum, accum_floats / 4,
                       zero_u32, zero_n, vp, gate, zero_stats);
}

// Points per thread of prepass_kernel: two for the clouds of a hundred million points that reach the direct path by
// their density (more loads in flight per wavefront: config 4 1.10 -> 1.04 ms), one below 2^24 points, where the
// launch is a few workgroups per CU and the shorter chain per thread counts (1 M points in 256 x 256, unordered:
// 0.17 -> 0.10 ms; 100 k points: 0.096 -> 0.073 ms).
static int prepass_ppt(int n, int tuned)
{
    const int ppt = tuned ? tuned : (n >= (1 << 24) ? 2 : 1);
    return ppt == 4 ? 4 : (ppt == 2 ? 2 : 1);
}

int prepass_points_per_block(int n, int tuned_ppt) { return kBlock * prepass_ppt(n, tuned_ppt); }

void launch_prepass(const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp, adop_stats* stats,
                    const adop_tuning& tn, hipStream_t st, Gate gate)
{
    if (pc.n < 1) return;
    const int group_from = tn.prepass_group_from;
    const int ppt        = prepass_ppt(pc.n, tn.prepass_ppt);
    if (ppt == 4)
        hipLaunchKernelGGL((prepass_kernel<4>), dim3((pc.n + kBlock * 4 - 1) / (kBlock * 4)), dim3(kBlock), 0, st, pc,
                           views, lv, rp, group_from, stats, gate);
    else if (ppt == 2)
        hipLaunchKernelGGL((prepass_kernel<2>), dim3((pc.n + kBlock * 2 - 1) / (kBlock * 2)), dim3(kBlock), 0, st, pc,
                           views, lv, rp, group_from, stats, gate);
    else
        hipLaunchKernelGGL((prepass_kernel<1>), dim3((pc.n + kBlock - 1) / kBlock), dim3(kBlock), 0, st, pc, views, lv,
                           rp, group_from, stats, gate);
}

template <int CT, bool HALF>
static void launch_blend_t(const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp,
                           float* accum, int S, adop_stats* stats, const adop_tuning& tn, hipStream_t st, Gate gate)
{
    const int group_from = tn.blend_group_from;  // 0: group at every level
    // list mode: one small workgroup per prepass workgroup (a few percent of the points survive in a dense cloud)
    const int list_block = tn.list_block;
    const int block = pc.list_ids ? ((list_block >= 64 && list_block <= kBlock && list_block % 64 == 0) ? list_block : 128)
                                  : kBlock;
    const int grid  = pc.list_ids ? (pc.n + pc.list_span - 1) / pc.list_span : (pc.n + kBlock - 1) / kBlock;
    size_t lds      = sizeof(float) * (size_t)block * (size_t)lv.C;
    hipLaunchKernelGGL((blend_kernel<CT, HALF>), dim3(grid), dim3(block), lds, st, pc, views, lv, rp,
                       accum, S, stats, group_from, gate);
}

void launch_blend(const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp, bool half,
                  float* accum, int S, adop_stats* stats, const adop_tuning& tn, hipStream_t st, Gate gate)
{
    if (pc.n < 1) return;
    if (lv.C == 8)
        half ? launch_blend_t<8, true>(pc, views, lv, rp, accum, S, stats, tn, st, gate)
             : launch_blend_t<8, false>(pc, views, lv, rp, accum, S, stats, tn, st, gate);
    else if (lv.C == 4)
        half ? launch_blend_t<4, true>(pc, views, lv, rp, accum, S, stats, tn, st, gate)
             : launch_blend_t<4, false>(pc, views, lv, rp, accum, S, stats, tn, st, gate);
    else
        half ? launch_blend_t<0, true>(pc, views, lv, rp, accum, S, stats, tn, st, gate)
             : launch_blend_t<0, false>(pc, views, lv, rp, accum, S, stats, tn, st, gate);
}

void launch_resolve(const Levels& lv, int first_level, int grid, const float* accum, int S, const float* background,
                    int write_mask, float mask_value, hipStream_t st, Gate gate)
{
    if (lv.C == 8)
        hipLaunchKernelGGL((resolve_kernel<8>), dim3(grid), dim3(kBlock), 0, st, lv, first_level, accum, S, background,
                           write_mask, mask_value, gate);
    else if (lv.C == 4)
        hipLaunchKernelGGL((resolve_kernel<4>), dim3(grid), dim3(kBlock), 0, st, lv, first_level, accum, S, background,
                           write_mask, mask_value, gate);
    else
        hipLaunchKernelGGL((resolve_kernel<0>), dim3(grid), dim3(kBlock), 0, st, lv, first_level, accum, S, background,
                           write_mask, mask_value, gate);
}

}  // namespace adop
