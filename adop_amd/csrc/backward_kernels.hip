// backward_kernels.hip — background gradient + gradient/image interleave, RenderBackward, finalize, normalise.
//
// The ghost gradient of one point-level reads the image I and the upstream gradient G at four neighbour pixels for
// every channel.  In the planar [B,C,h,w] layout that is 8C scattered 4-byte loads (plus C for the centre); the
// interleave kernel therefore first builds two pixel-major arrays in the workspace, I[pixel][C] and, behind it,
// G[pixel][C] (32 bytes per pixel each for C = 8), while it sums the background gradient in the same pass.  Two arrays
// and not one record [I | G] per pixel: the descriptor pass gathers G alone, and with I in the same 64-byte line it
// fetched twice the bytes it used.
#include "common.h"
#include "launch.h"

#pragma clang fp contract(off)

namespace adop
{
// Work-queue items of one view: point id (32 bits) | level mask (5 bits) | kItemSharedBit.
constexpr int kItemSharedBit = 37;  // set when the point has items in other views of the call too

// CombineAndFillBackward (:851-900) fused with the I/G interleave.  One thread per pixel of every level/image.
// Background gradient: per-thread fp32 partial over a handful of pixels, wave/block reduction in f64, one f64
// partial row per block.
template <int CT>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(8, 8))) void interleave_kernel(Levels lv, float* __restrict__ ig,
                                                            float2* __restrict__ dw, double* __restrict__ partial,
                                                            uint32_t* __restrict__ q_counts, ViewPrep vp)
{
    prepare_views_inline(vp);
    // counters of the backward work queues (one set per view): empty before backward_tex_kernel
    for (int k = blockIdx.x * kBlock + threadIdx.x; k <= lv.B * kNumQueues; k += gridDim.x * kBlock)
        q_counts[k] = 0;  // (the last word is the ticket counter of finalize_normalize_kernel)
    constexpr int CMAX = CT ? CT : kMaxChannels;
    const int C        = CT ? CT : lv.C;
    __shared__ double red[kBlock / 64][kMaxChannels];
    __shared__ float4 s_tr[kBlock / 64][(CT == 8 || CT == 4) ? 64 * (CT / 2) : 1];
    float acc[CMAX];
#pragma unroll
    for (int c = 0; c < CMAX; ++c) acc[c] = 0;
    int per_image = lv.pix_prefix[lv.num];
    size_t total  = (size_t)per_image * lv.B;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride)
    {
        int b             = (int)(t / per_image);
        int r             = (int)(t - (size_t)b * per_image);
        int l             = level_of(lv, r);
        const LevelArg& L = lv.l[l];
        int p             = r - lv.pix_prefix[l];
        size_t hw         = (size_t)L.w * L.h;
        const float wgt   = L.weight[(size_t)b * hw + p];
        bool empty        = wgt == 0;
        // (depth, weight) of the pixel side by side: the descriptor pass fetches both with one 8-byte load
        dw[ws_pixel(lv, l, b, (uint32_t)p)] = make_float2(L.depth[(size_t)b * hw + p], wgt);
        const float* g    = L.gin + (size_t)b * C * hw + p;
        const float* im   = L.out + (size_t)b * C * hw + p;
        float* dst        = ig + (size_t)ws_pixel(lv, l, b, (uint32_t)p) * C;  // I record; the G record at dst + goff
        const size_t goff = total * (size_t)C;
        // (the forward pass may have left the I records with the caller: then only G is transposed here)
        const bool with_I = !lv.irec_ready;  // kernel-uniform
        float I[CMAX], G[CMAX];
#pragma unroll
        for (int c = 0; c < CMAX; ++c)
            if (c < C)
            {
                I[c] = with_I ? __builtin_nontemporal_load(im + (size_t)c * hw) : 0.f;
                G[c] = __builtin_nontemporal_load(g + (size_t)c * hw);
                if (empty) acc[c] += G[c];
            }
        if (CT == 8 || CT == 4)
        {
            // The 64 pixels of a wavefront are 64 consecutive records of the pixel-major array when they lie in one
            // level of one image: transposed through LDS, every store instruction then writes 1 KB of consecutive
            // bytes instead of a quarter (half) of 64 separate lines.
            constexpr int V     = CT / 4;  // float4 per record of either array
            const int lane      = threadIdx.x & 63;
            const size_t t_wave = t - lane;
            const int r_last    = (int)((t_wave + 63) - (size_t)b * per_image);
            const bool whole    = t_wave + 63 < total && (t_wave / per_image) == (size_t)b &&
                               (t_wave + 63) / per_image == (size_t)b && level_of(lv, r_last) == l &&
                               level_of(lv, r - lane) == l;
            if (whole)  // wavefront-uniform
            {
                // s_tr: the I records of the 64 pixels, then their G records
                float4* sw = s_tr[threadIdx.x >> 6];
                wave_lds_sync();
#pragma unroll
                for (int q = 0; q < V; ++q)
                {
                    if (with_I) sw[lane * V + q] = make_float4(I[4 * q], I[4 * q + 1], I[4 * q + 2], I[4 * q + 3]);
                    sw[64 * V + lane * V + q] = make_float4(G[4 * q], G[4 * q + 1], G[4 * q + 2], G[4 * q + 3]);
                }
                wave_lds_sync();
                float* d0 = dst - (size_t)lane * CT;  // I record of the wavefront's first pixel
#pragma unroll
                for (int k = 0; k < V; ++k)
                {
                    if (with_I) __builtin_nontemporal_store(((const v4f*)sw)[k * 64 + lane], (v4f*)d0 + k * 64 + lane);
                    __builtin_nontemporal_store(((const v4f*)sw)[64 * V + k * 64 + lane], (v4f*)(d0 + goff) + k * 64 + lane);
                }
            }
            else
            {
                float4* d4 = (float4*)dst;
                float4* g4 = (float4*)(dst + goff);
                if (with_I)
                {
#pragma unroll
                    for (int q = 0; q < V; ++q) d4[q] = make_float4(I[4 * q], I[4 * q + 1], I[4 * q + 2], I[4 * q + 3]);
                }
#pragma unroll
                for (int q = 0; q < V; ++q) g4[q] = make_float4(G[4 * q], G[4 * q + 1], G[4 * q + 2], G[4 * q + 3]);
            }
        }
        else
        {
#pragma unroll
            for (int c = 0; c < CMAX; ++c)
                if (c < C)
                {
                    if (with_I) dst[c] = I[c];
                    dst[goff + c] = G[c];
                }
        }
    }
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int c = 0; c < CMAX; ++c)
    {
        double v = wave_sum<double>((double)acc[c]);
        if (lane == 0) red[wave][c] = v;
    }
    __syncthreads();
    if (threadIdx.x < kMaxChannels)
    {
        double v = 0;
        if ((int)threadIdx.x < CMAX)
            for (int w = 0; w < kBlock / 64; ++w) v += red[w][threadIdx.x];
        partial[(size_t)blockIdx.x * kMaxChannels + threadIdx.x] = v;
    }
}

template <int CT>
__device__ __forceinline__ void load_channels(const float* __restrict__ src, float* dst)
{
    static_assert(CT == 4 || CT == 8, "vector path");
    const float4* s4 = (const float4*)src;
#pragma unroll
    for (int q = 0; q < CT / 4; ++q)
    {
        float4 v       = s4[q];
        dst[4 * q]     = v.x;
        dst[4 * q + 1] = v.y;
        dst[4 * q + 2] = v.z;
        dst[4 * q + 3] = v.w;
    }
}

// RenderBackward (PointRenderer.cu:396-724) is split in two kernels.
//
// backward_tex_kernel — one thread per point: projection, the per-level depth test (`break` at the first failed
// level, :462), the descriptor gradient (:469-485, summed over the levels in registers) and the decision which
// levels receive a ghost / spatial gradient (:487-489).  Points with at least one such level are appended to a
// work queue as (point id | level mask << 32).  The queue is split in kNumQueues sub-queues with their own counters
// (one returning atomic per workgroup; a single counter would serialise ~40 k same-address atomics).
//
// backward_ghost_kernel — one thread per queue item, all lanes busy: the four-neighbour gather from the
// pixel-major [I|G] array, the approximate image-space gradient (:491-611) and ProjectPoint*Backward.
template <int CT, bool HALF, bool MULTI>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(CT != 0 ? 8 : 4, 8))) void backward_tex_kernel(CloudArg pc, const ViewConst* __restrict__ views,
                                                               Levels lv, ParamArg rp, const float* __restrict__ ig,
                                                               const float2* __restrict__ dw,
                                                               float* __restrict__ gtex,
                                                               float* __restrict__ gpoints,
                                                               float* __restrict__ gpoints_count, int identity_index,
                                                               uint32_t* __restrict__ q_counts,
                                                               unsigned long long* __restrict__ q_items,
                                                               uint32_t q_cap, int concurrent, adop_stats* stats)
{
    constexpr int CMAX = CT ? CT : 1;  // register arrays exist only for compile-time channel counts
    __shared__ uint32_t s_wave_count[kBlock / 64];
    __shared__ uint32_t s_base;
    __shared__ unsigned long long s_culled[kBlock / 64];
    __shared__ unsigned long long s_block_culled;
    static_assert(kBlock / 64 == 4, "four runs per workgroup");
    const bool STATS    = stats != nullptr;  // counter pass (uniform branch)
    const float accept  = rp.depth_accept + 1;
    const int C         = CT ? CT : lv.C;
    const int lane      = threadIdx.x & 63;
    const int wave      = threadIdx.x >> 6;

    const int i     = blockIdx.x * kBlock + threadIdx.x;
    const bool valid = i < pc.n;
    const int tex_index    = identity_index ? i : (valid ? pc.index[i] : 0);
    const bool tex_in_range = (unsigned)tex_index < (unsigned)pc.num_texels;
    // the descriptor gradient of the point, summed over the views and levels in registers and written once
    float gt[CMAX];
#pragma unroll
    for (int c = 0; c < CMAX; ++c) gt[c] = 0.f;
    bool gt_live = false;

    // the views one after the other: view b appends to work queue b (MULTI = false: one view, no loop)
    const int num_views = MULTI ? lv.B : 1;
    unsigned long long masks = 0;
    // `concurrent` (at most kConcurrentViews views): the level masks of all views are kept (5 bits each) and the items
    // are pushed after the loop, when the thread knows whether its point has items in several views; the
    // spatial-gradient kernel then runs all views in one launch, see backward_ghost_kernel
    const bool deferred = MULTI && concurrent != 0;
    unsigned long long kept[2] = {0ull, 0ull};
    // Several views (crops see a small part of the cloud): the first record of the wavefront's run of 64 points says
    // whether the forward pass culled the whole run for a view (kRunCulledBits); lane b asks for view b, all at once,
    // and the records of the runs culled are never read.
    unsigned long long culled_views = 0;
    if (MULTI && pc.cache)
    {
        const int first = i & ~63;
        bool c          = false;
        if (lane < num_views && first < pc.n)
        {
            const float4 head = pc.cache[(size_t)lane * pc.n + first];
            c                 = __float_as_uint(head.x) == kRunCulledBits && head.z == 0.f;
        }
        culled_views = __ballot(c);
        // views culled for all four runs of the workgroup: their whole iteration is skipped below
        if (lane == 0) s_culled[wave] = culled_views;
        __syncthreads();
        if (threadIdx.x == 0) s_block_culled = s_culled[0] & s_culled[1] & s_culled[2] & s_culled[3];
        __syncthreads();
    }
    else if (MULTI)
    {
        if (threadIdx.x == 0) s_block_culled = 0;
        __syncthreads();
    }
    // Views 0..63 for which every run of this workgroup was culled have nothing to test: the loop jumps from one live view
    // to the next (a crop sees a small part of the cloud: 2 to 3 of 16 views are live for a workgroup, and the loop
    // is scalar control flow that the scalar unit of the CU has to issue for every wavefront).
    unsigned long long live_views = ~0ull;
    if (MULTI)
    {
        const unsigned long long bc = s_block_culled;
        live_views = ~(((unsigned long long)(uint32_t)__builtin_amdgcn_readfirstlane((int)(bc >> 32)) << 32) |
                       (unsigned long long)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)bc));
        // view 0 culled for the whole workgroup: its iteration, which clears the point-gradient rows, is skipped
        if (!deferred && (live_views & 1ull) == 0 && gpoints && valid)
        {
            nt_store4((float4*)gpoints + i, make_float4(0, 0, 0, 0));
            __builtin_nontemporal_store(0.f, gpoints_count + i);
        }
    }
    for (int b = 0; b < num_views; ++b)
    {
        if (MULTI && b < 64)
        {
            const unsigned long long rest = live_views >> b;  // (uniform)
            if (rest == 0)
            {
                b = 63;  // the views from 64 on carry no marks
                continue;
            }
            b += __builtin_ctzll(rest);
            if (b >= num_views) break;
        }
        uint32_t mask = 0;
        {
            const ViewConst& vc = views[b];
            bool drop_out;
            V2 ip = {0.f, 0.f};
            float z = 0.f, radius_pixels = 0.f;
            bool ok;
            if (pc.cache)  // kernel-uniform: the forward pass left the projected points with the caller
            {
                // depth 0: culled; negative depth: dropped for this image (:314-315)
                float4 R = make_float4(0, 0, 0, 0);
                // Several views (crops see a small part of the cloud): the first record of the wavefront's run of 64 points
                // says whether the forward pass culled the whole run for this view; the other 63 records are then not read.
                const bool run_culled = MULTI && b < 64 && (culled_views >> b & 1ull) != 0;
                if (valid && !run_culled)
                {
                    const v4f r = __builtin_nontemporal_load((const v4f*)pc.cache + (size_t)b * pc.n + i);
                    R           = make_float4(r.x, r.y, r.z, r.w);
                }
                ip             = {R.x, R.y};
                drop_out       = depth_is_dropped(R.z);
                z              = fabsf(R.z);
                radius_pixels  = R.w;
                ok             = valid && z != 0;
            }
            else
            {
                drop_out = valid && pc.dropout && pc.dropout[(size_t)b * pc.n + i] == 1.f;
                float4 P = valid ? pc.position[i] : make_float4(0, 0, 0, 0);
                V3 pos   = {P.x, P.y, P.z};
                V3 nrm   = {0, 0, 0};
                if (valid && pc.normal) nrm = unpack_normal10(pc.normal[i]);
                V3 view_p;
                ok = valid && project_point(vc, pc.intrinsics, pos, nrm, P.w, rp.check_normal != 0, rp.dist_cutoff, lv.l[0].w,
                                            &ip, &z, &radius_pixels, &view_p);
            }
            ok = ok && tex_in_range;

            // phase 1: pixel of every level, depth loads (independent)
            uint32_t pix[ADOP_MAX_LAYERS];
            bool in[ADOP_MAX_LAYERS];
            bool edge_ok[ADOP_MAX_LAYERS];
            float dep[ADOP_MAX_LAYERS];
            float wgt[ADOP_MAX_LAYERS];
    #pragma unroll
            for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
            {
                in[l]      = false;
                edge_ok[l] = false;
                pix[l]     = 0;
                dep[l]     = 0.f;
                wgt[l]     = 0.f;
                if (l < lv.num)
                {
                    const LevelArg& L = lv.l[l];
                    int px = f2i_rn(ip.x), py = f2i_rn(ip.y);
                    bool lod_skip = rp.drop_by_radius && radius_pixels < rp.drop_threshold;  // continue, :451-454
                    in[l]         = ok && !lod_skip && (unsigned)px < (unsigned)L.w && (unsigned)py < (unsigned)L.h;
                    if (in[l])
                    {
                        pix[l]     = (uint32_t)py * (uint32_t)L.w + (uint32_t)px;
                        const float2 d_w = dw[ws_pixel(lv, l, b, pix[l])];  // (depth, weight) left by interleave_kernel
                        dep[l]           = d_w.x;
                        wgt[l]           = d_w.y;
                        int ex     = min(px, L.w - 1 - px);
                        int ey     = min(py, L.h - 1 - py);
                        edge_ok[l] = min(ex, ey) > 2;  // distanceFromEdge > 2, :489
                    }
                    radius_pixels *= 0.5f;
                    ip.x *= 0.5f;
                    ip.y *= 0.5f;
                }
            }
            // phase 2: depth test in level order, `break` at the first failure (:462)
            bool pass[ADOP_MAX_LAYERS];
            {
                bool alive = true;
    #pragma unroll
                for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
                {
                    pass[l] = false;
                    if (in[l] && alive)
                    {
                        if (z > dep[l] * accept)
                            alive = false;
                        else
                            pass[l] = true;
                    }
                }
            }
            // phase 3: descriptor gradient of the rendered (not dropped) points; spatial-gradient eligibility
            const bool point_grad = (rp.ghost_gradients && drop_out) | (!rp.ghost_gradients && !drop_out);
            mask                  = 0;
    #pragma unroll
            for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
            {
                bool go = pass[l];
                if (pass[l] && !drop_out)
                {
                    if (wgt[l] == 0)
                        go = false;  // continue, :473
                    else
                    {
                        float iw        = 1.f / wgt[l];
                        const float* pg = ig + gradient_array_offset(lv, C) + (size_t)ws_pixel(lv, l, b, pix[l]) * C;  // G of the pixel
                        if (CT == 0)
                        {
                            // any channel count: one atomic per channel and level (:478-484)
    #pragma unroll 1
                            for (int c = 0; c < C; ++c)
                                unsafeAtomicAdd(gtex + (size_t)c * pc.num_texels + tex_index, iw * pg[c]);
                        }
                        else
                        {
                            float G[CMAX];
                            load_channels<CT ? CT : 4>(pg, G);
    #pragma unroll
                            for (int c = 0; c < CMAX; ++c) gt[c] += iw * G[c];
                            gt_live = true;
                        }
                    }
                }
                bool spatial = go && point_grad && edge_ok[l];
                if (spatial) mask |= 1u << l;
                if (STATS && l < lv.num) stat_add(&stats->spatial[l], spatial);
            }
        }
        // Point gradients of the first view: points without a spatial gradient are cleared here (Build(info,false),
        // :922-949), the others are written by backward_ghost_kernel; no separate zero-fill of the two buffers.
        if (deferred)
        {
            kept[b / 12] |= (unsigned long long)mask << (5 * (b % 12));
            continue;
        }
        if (b == 0 && gpoints && valid && (mask == 0 || !MULTI))
        {
            if (mask == 0) nt_store4((float4*)gpoints + i, make_float4(0, 0, 0, 0));
            // One view: the number of contributions of a point is the number of its levels with a spatial gradient, known
            // here for every point; the spatial-gradient kernel then normalises its rows itself (NormalizeGradient,
            // :1534-1547), for which it needs the counts of other points (normalize_mode 0 divides the floats 3t..3t+2 of
            // the [N,4] buffer by count[t]).
            __builtin_nontemporal_store(MULTI ? 0.f : (float)__popc(mask), gpoints_count + i);
        }

        const int set = b;  // queue set the item goes to
        masks         = mask;
        bool has               = masks != 0;
        unsigned long long bal = __ballot(has);
        uint32_t rank_in_wave  = (uint32_t)__popcll(bal & ((1ull << lane) - 1ull));
        if (MULTI)
        {
            // Several views: every wavefront pushes for itself (one returning atomic per wavefront with items, onto the
            // sub-queue of its workgroup), so that the loop over the views has no barrier in it: most views do not see
            // the run at all.
            if (bal)
            {
                const uint32_t q = blockIdx.x % kNumQueues;
                uint32_t base    = 0;
                if (lane == 0) base = atomicAdd(&q_counts[(size_t)set * kNumQueues + q], (uint32_t)__popcll(bal));
                base = (uint32_t)__shfl((int)base, 0, 64);
                if (has)
                {
                    const size_t at = ((size_t)set * kNumQueues + q) * q_cap + base + rank_in_wave;
                    q_items[at]     = (unsigned long long)(uint32_t)i | (masks << 32);
                }
            }
            masks = 0;
            continue;
        }
        // one view: rank inside the workgroup, one returning atomic per workgroup on the sub-queue counter
        if (lane == 0) s_wave_count[wave] = (uint32_t)__popcll(bal);
        __syncthreads();
        uint32_t before = 0, total = 0;
#pragma unroll
        for (int w = 0; w < kBlock / 64; ++w)
        {
            uint32_t c = s_wave_count[w];
            if (w < wave) before += c;
            total += c;
        }
        const uint32_t q = blockIdx.x % kNumQueues;
        if (threadIdx.x == 0) s_base = total ? atomicAdd(&q_counts[(size_t)set * kNumQueues + q], total) : 0u;
        __syncthreads();
        if (has)
        {
            const size_t at = ((size_t)set * kNumQueues + q) * q_cap + s_base + before + rank_in_wave;
            q_items[at]     = (unsigned long long)(uint32_t)i | (masks << 32);
        }
        masks = 0;
        __syncthreads();  // s_wave_count and s_base are reused by the next view
    }  // views

    if (deferred)
    {
        // number of views with an item: the non-zero 5-bit fields of the two words (bit 0 of a field = the OR of its bits)
        constexpr unsigned long long kField0 = 0x0084210842108421ull;  // bits 0, 5, ..., 55: twelve fields
        int nitems = 0;
#pragma unroll
        for (int w = 0; w < 2; ++w)
        {
            const unsigned long long k = kept[w];
            nitems += __popcll((k | k >> 1 | k >> 2 | k >> 3 | k >> 4) & kField0);
        }
        // A point with one item gets its gradient row from that item's thread; a row nobody writes, or one that several
        // views add to with atomics, starts at zero (Build(info,false), :922-949).
        if (gpoints && valid && nitems != 1)
        {
            nt_store4((float4*)gpoints + i, make_float4(0, 0, 0, 0));
            __builtin_nontemporal_store(0.f, gpoints_count + i);
        }
        const unsigned long long shared = nitems > 1 ? 1ull << kItemSharedBit : 0ull;
        for (int b = 0; b < num_views; ++b)
        {
            {
                const unsigned long long rest = live_views >> b;  // (uniform; at most kConcurrentViews < 64 views here)
                if (rest == 0) break;
                b += __builtin_ctzll(rest);
                if (b >= num_views) break;
            }
            const unsigned long long m = kept[b / 12] >> (5 * (b % 12)) & 31ull;
            const unsigned long long bal = __ballot(m != 0);
            if (!bal) continue;  // wavefront-uniform
            const uint32_t q = blockIdx.x % kNumQueues;
            uint32_t base    = 0;
            if (lane == 0) base = atomicAdd(&q_counts[(size_t)b * kNumQueues + q], (uint32_t)__popcll(bal));
            base = (uint32_t)__shfl((int)base, 0, 64);
            if (m != 0)
                q_items[((size_t)b * kNumQueues + q) * q_cap + base + (uint32_t)__popcll(bal & ((1ull << lane) - 1ull))] =
                    (unsigned long long)(uint32_t)i | (m << 32) | shared;
        }
    }

    if (CT != 0)
    {
        if (identity_index)
        {
            // texel i belongs to this thread alone: plain coalesced stores, which also clear the buffer
            if (valid)
            {
#pragma unroll
                for (int c = 0; c < CMAX; ++c)
                {
                    // streamed once: kept out of the caches the gathers of this kernel live in
                    float* dst = gtex + (size_t)c * pc.num_texels + i;
                    __builtin_nontemporal_store(gt[c], dst);
                }
            }
        }
        else if (gt_live)
        {
#pragma unroll
            for (int c = 0; c < CMAX; ++c) unsafeAtomicAdd(gtex + (size_t)c * pc.num_texels + tex_index, gt[c]);
        }
    }
}

// 4 waves per SIMD (<= 128 VGPRs): the grid of kPartialBlocks = 4 workgroups x 256 CUs is then resident at once; with
// the 151 VGPRs the compiler takes by itself only 3 fit and a quarter of the grid runs as a second, mostly idle round.
template <int CT, bool HALF>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(4, 4))) void backward_ghost_kernel(CloudArg pc, const ViewConst* __restrict__ views,
                                                                 Levels lv, ParamArg rp, const float* __restrict__ ig,
                                                                 float* __restrict__ gpoints,
                                                                 float* __restrict__ gpoints_count, int want_pose,
                                                                 int want_intr, int identity_index, int view_b,
                                                                 int first_view, int normalize,
                                                                 const uint32_t* __restrict__ q_counts,
                                                                 const unsigned long long* __restrict__ q_items,
                                                                 uint32_t q_cap, double* __restrict__ partial)
{
    constexpr int CMAX = CT ? CT : 1;
    __shared__ float s_red[kAcc * kBlock];
    __shared__ uint32_t s_prefix[kNumQueues + 1];
    // view_b < 0: all views in one launch, view = blockIdx.y (the queues of the views follow each other); an item's
    // kItemSharedBit then says whether other views add to the same point's gradient row
    const bool concurrent = view_b < 0;
    const int b           = concurrent ? (int)blockIdx.y : view_b;
    if (concurrent)
    {
        q_counts += (size_t)b * kNumQueues;
        q_items += (size_t)b * kNumQueues * q_cap;
    }
    const ViewConst& vc = views[b];
    const float accept  = rp.depth_accept + 1;
    const int C         = CT ? CT : lv.C;

    // Exclusive prefix over the sub-queue counters, by every workgroup for itself (8 KB from the L2; a kernel of its
    // own for it cost more than all these prologues): s_prefix[0..kNumQueues], s_prefix[kNumQueues] = number of items.
    {
        constexpr int PER = kNumQueues / kBlock;
        static_assert(PER == 8, "two 16-byte loads per thread");
        __shared__ uint32_t s_wave[kBlock / 64];
        const uint4 c0 = *(const uint4*)(q_counts + threadIdx.x * PER);
        const uint4 c1 = *(const uint4*)(q_counts + threadIdx.x * PER + 4);
        const uint32_t v[PER] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
        uint32_t sum = 0;
#pragma unroll
        for (int k = 0; k < PER; ++k) sum += v[k];
        uint32_t inc = sum;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1)
        {
            uint32_t u = __shfl_up(inc, off, 64);
            if ((int)(threadIdx.x & 63) >= off) inc += u;
        }
        if ((threadIdx.x & 63) == 63) s_wave[threadIdx.x >> 6] = inc;
        __syncthreads();
        uint32_t run = inc - sum;
        for (int w = 0; w < (int)(threadIdx.x >> 6); ++w) run += s_wave[w];
#pragma unroll
        for (int k = 0; k < PER; ++k)
        {
            s_prefix[threadIdx.x * PER + k] = run;
            run += v[k];
        }
        if (threadIdx.x == kBlock - 1) s_prefix[kNumQueues] = run;
        __syncthreads();
    }
    const uint32_t total = s_prefix[kNumQueues];

    // per-thread sums of the pose / intrinsics gradients: a thread sees a few dozen contributions at most, so fp32
    // here costs ~1e-7 relative; everything beyond the thread (wavefront, block, grid) is summed in f64
    // (they live in LDS, one column per thread: 21 registers less in a kernel whose occupancy is set by registers)
    float* acc = s_red + threadIdx.x;  // acc[k * kBlock]
#pragma unroll
    for (int k = 0; k < kAcc; ++k) acc[k * kBlock] = 0;

    for (uint32_t t = blockIdx.x * kBlock + threadIdx.x; t < total; t += gridDim.x * kBlock)
    {
        // sub-queue of item t: largest q with prefix[q] <= t
        uint32_t lo = 0, hi = kNumQueues;
        while (hi - lo > 1)
        {
            uint32_t mid = (lo + hi) >> 1;
            if (s_prefix[mid] <= t)
                lo = mid;
            else
                hi = mid;
        }
        // (the item and the point record are read once by this kernel: past the caches, which hold the [I|G] lines)
        unsigned long long item = __builtin_nontemporal_load(q_items + (size_t)lo * q_cap + (t - s_prefix[lo]));
        const int i             = (int)(uint32_t)item;
        const uint32_t mask     = (uint32_t)(item >> 32) & 31u;
        const bool shared       = (item >> kItemSharedBit & 1ull) != 0;

        float4 P = nt_load4(pc.position + i);
        V3 pos   = {P.x, P.y, P.z};
        V3 nrm   = {0, 0, 0};
        if (pc.normal) nrm = unpack_normal10(__builtin_nontemporal_load(pc.normal + i));
        V2 ip;
        V3 view_p;
        float z, radius_pixels;
        project_point(vc, pc.intrinsics, pos, nrm, P.w, rp.check_normal != 0, rp.dist_cutoff, lv.l[0].w, &ip, &z,
                      &radius_pixels, &view_p);
        const int tex_index = identity_index ? i : pc.index[i];
        float T[CMAX];
        if (CT != 0)
        {
#pragma unroll
            for (int c = 0; c < CMAX; ++c) T[c] = tex_fetch_stream<HALF>(pc.texture, (size_t)c * pc.num_texels + tex_index);
        }
        // running value of grad_points[i] / count[i]: the additions happen in the reference's order (view after
        // view, level after level); this thread owns point i for this view
        float gp[3] = {0, 0, 0};
        float gp_n  = 0;
        if (gpoints && !first_view && !concurrent)
        {
            const float* g = gpoints + 4 * (size_t)i;
            gp[0]          = g[0];
            gp[1]          = g[1];
            gp[2]          = g[2];
            gp_n           = gpoints_count[i];
        }
        float scale = 1;
#pragma unroll 1
        for (int l = 0; l < lv.num; ++l)
        {
            if (mask & (1u << l))
            {
                const LevelArg& L = lv.l[l];
                int px = f2i_rn(ip.x), py = f2i_rn(ip.y);
                size_t hw             = (size_t)L.w * L.h;
                size_t p              = (size_t)py * L.w + px;
                // I of the pixel (where the forward pass or interleave_kernel left it) and its G at + goff
                const size_t rec      = (size_t)ws_pixel(lv, l, b, (uint32_t)p) * C;
                const float* pg       = lv.irec + rec;
                const float* pgg      = ig + gradient_array_offset(lv, C) + rec;
                const ptrdiff_t nb[4] = {-1, 1, -(ptrdiff_t)L.w, (ptrdiff_t)L.w};
                float Wn[4] = {0, 0, 0, 0}, Dn[4] = {0, 0, 0, 0};
                if (rp.test_backward_mode == 4)
                {
                    const float* Wp = L.weight + (size_t)b * hw + p;
                    const float* Dp = L.depth + (size_t)b * hw + p;
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                    {
                        Wn[k] = Wp[nb[k]];
                        Dn[k] = Dp[nb[k]];
                    }
                }
                auto dI_of = [&](float T_c, float I_x, float W_x, float D_x) -> float
                {
                    if (rp.test_backward_mode == 4)
                    {
                        if (W_x == 0 || z * accept < D_x) return T_c - I_x;          // full override
                        if (z > D_x * accept) return 0.f;                            // discard
                        return (W_x / (W_x + 1) * I_x + 1 / (W_x + 1) * T_c - I_x);  // blend
                    }
                    return T_c - I_x;
                };
                float dR_dpx = 0, dR_dpy = 0;
                if (CT == 0)
                {
#pragma unroll 1
                    for (int c = 0; c < C; ++c)
                    {
                        float T_c = tex_fetch<HALF>(pc.texture, (size_t)c * pc.num_texels + tex_index);
                        float v[4];
#pragma unroll
                        for (int k = 0; k < 4; ++k)
                        {
                            const float* q = pg + nb[k] * C;
                            v[k]           = dI_of(T_c, q[c], Wn[k], Dn[k]) * pgg[nb[k] * C + c];
                        }
                        float a0 = -v[0], a1 = v[1], b0 = -v[2], b1 = v[3];
                        dR_dpx += 0.5f * (a0 + a1);
                        dR_dpy += 0.5f * (b0 + b1);
                    }
                }
                else
                {
                    float v[4][CMAX];  // dI * G per neighbour and channel
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                    {
                        const float* q = pg + nb[k] * C;
                        float In[CMAX], Gn[CMAX];
                        load_channels<CT ? CT : 4>(q, In);
                        load_channels<CT ? CT : 4>(pgg + nb[k] * C, Gn);
#pragma unroll
                        for (int c = 0; c < CMAX; ++c) v[k][c] = dI_of(T[c], In[c], Wn[k], Dn[k]) * Gn[c];
                    }
#pragma unroll
                    for (int c = 0; c < CMAX; ++c)
                    {
                        float a0 = -v[0][c], a1 = v[1][c], b0 = -v[2][c], b1 = v[3][c];
                        dR_dpx += 0.5f * (a0 + a1);
                        dR_dpy += 0.5f * (b0 + b1);
                    }
                }
                V2 dR_dp       = {dR_dpx / (float)C, dR_dpy / (float)C};
                float crop2[5] = {vc.crop[0] * scale, vc.crop[1] * scale, vc.crop[2] * scale, vc.crop[3] * scale,
                                  vc.crop[4] * scale};  // crop.scale(scale), :616
                BackwardOut bo;
                project_point_backward(vc, pc.intrinsics, view_p, dR_dp, crop2, rp.dist_cutoff, &bo);
                gp[0] += bo.g_point[0];
                gp[1] += bo.g_point[1];
                gp[2] += bo.g_point[2];
                gp_n += 1.f;
                if (want_pose)
                {
#pragma unroll
                    for (int k = 0; k < 6; ++k) acc[k * kBlock] += bo.g_pose[k];
                    acc[6 * kBlock] += 1.0f;
                }
                if (want_intr)
                {
                    if (vc.model == 0)
                    {
                        float kf = rp.K_gradient_factor;
                        bo.g_k[4] *= 0;  // the shear gradient is removed, :653-654
#pragma unroll
                        for (int k = 0; k < 5; ++k) acc[(8 + k) * kBlock] += kf * bo.g_k[k];
                        float df = rp.distortion_gradient_factor;
                        // float *= double literal in the reference: the product is formed in double and rounded to
                        // float once (:664-673); 0.25 is exact either way
                        bo.g_dis[2] *= 0.25f;
#pragma unroll
                        for (int k = 3; k < 8; ++k) bo.g_dis[k] = (float)((double)bo.g_dis[k] * 0.1);
#pragma unroll
                        for (int k = 0; k < 8; ++k) acc[(13 + k) * kBlock] += df * bo.g_dis[k];
                        acc[7 * kBlock] += 1.0f / 1024.0f;  // :680-681
                    }
                    else
                    {
#pragma unroll
                        for (int k = 0; k < 5; ++k) acc[(8 + k) * kBlock] += bo.g_k[k];
                        acc[7 * kBlock] += 1.0f;  // :718
                    }
                }
            }
            scale *= 0.5f;
            ip.x *= 0.5f;
            ip.y *= 0.5f;
        }
        if (gpoints)
        {
            float* g = gpoints + 4 * (size_t)i;
            if (concurrent && shared)
            {
                // the point has items in several views, which run side by side: the row was cleared by the descriptor
                // pass and every view adds its part (the order of these float additions is the one thing of the
                // gradients that is not fixed from run to run)
                unsafeAtomicAdd(g + 0, gp[0]);
                unsafeAtomicAdd(g + 1, gp[1]);
                unsafeAtomicAdd(g + 2, gp[2]);
                unsafeAtomicAdd(gpoints_count + i, gp_n);
            }
            else
            {
                if (normalize)
                {
                    // One view: the descriptor pass left the final count of every point, and this thread writes the
                    // normalised row (NormalizeGradient<float,3>, :1534-1547, launched on the [N,4] buffer, :1620-1627).
                    // normalize = 1 (the reference's launch): float f of the buffer belongs to element f / 3 and is
                    // divided by that point's count when it is positive and f / 3 < N; 2: row i by count[i].
                    if (normalize == 2)
                    {
                        gp[0] = gp[0] / gp_n;
                        gp[1] = gp[1] / gp_n;
                        gp[2] = gp[2] / gp_n;
                    }
                    else
                    {
                        const uint32_t f0 = 4u * (uint32_t)i;  // (N <= 2^30)
#pragma unroll
                        for (int k = 0; k < 3; ++k)
                        {
                            const uint32_t t = (f0 + (uint32_t)k) / 3u;
                            if (t < (uint32_t)pc.n)
                            {
                                const float c = t == (uint32_t)i ? gp_n : gpoints_count[t];
                                if (c > 0) gp[k] = gp[k] / c;
                            }
                        }
                    }
                    *(float4*)g = make_float4(gp[0], gp[1], gp[2], 0.f);
                }
                else if (first_view || concurrent)
                {
                    *(float4*)g      = make_float4(gp[0], gp[1], gp[2], 0.f);  // nothing has cleared the row
                    gpoints_count[i] = gp_n;
                }
                else
                {
                    g[0]             = gp[0];
                    g[1]             = gp[1];
                    g[2]             = gp[2];
                    gpoints_count[i] = gp_n;
                }
            }
        }
    }

    if (want_pose || want_intr)
    {
        // block sums in f64 through LDS: 8 threads per value, 32 columns each (21 f64 wavefront reductions with
        // cross-lane permutes took 7 us per workgroup)
        __syncthreads();
        const int k = threadIdx.x >> 3, part = threadIdx.x & 7;
        double v    = 0;
        if (k < kAcc)
            for (int c = part; c < kBlock; c += 8) v += (double)s_red[k * kBlock + c];
        v += __shfl_xor(v, 1, 64);
        v += __shfl_xor(v, 2, 64);
        v += __shfl_xor(v, 4, 64);
        if (k < kAcc && part == 0) partial[((size_t)b * gridDim.x + blockIdx.x) * kPartialStride + k] = v;
    }
}


constexpr int kFinalizeBlock = 1024;  // the reduction as a kernel of its own: one workgroup, 16 loads in flight per thread

// Reduces the per-block partial rows and runs NormalizeGradient (:1534-1547, launches :1611-1636) for the
// background / pose / intrinsics outputs.  One block of NT threads; sh holds NT values.
struct FinalizeArg
{
    const ViewConst* views;
    int B, C;
    const double* bg_partial;
    int bg_blocks;
    const double* pt_partial;
    int pt_blocks;
    float* gbg;
    double* gpose;
    float* gpose_count;
    int num_poses;
    float* gintr;
    float* gintr_count;
    int num_cameras, cols, normalize_mode;
    double* scratch;
    double* mini;      // [kFinalizeParts * kMaxChannels] + [B * kFinalizeParts * kPartialStride]: rows of the first stage
    uint32_t* ticket;  // zero at the start of the kernel
    // one view: its work queue names exactly the points with a spatial gradient (count > 0); null otherwise
    const uint32_t* q_counts;
    const unsigned long long* q_items;
    uint32_t q_cap;
};

constexpr int kFinalizeSmall = 1024;  // pose / intrinsics sums of up to this many f64 stay in LDS

// part: 0 = everything, 1 = the background gradient only, 2 = the pose / intrinsics gradients only (the two are
// independent: two workgroups can share the work)
template <int NT>
__device__ static void finalize_block(const FinalizeArg& a, double* sh, double* s_small, int part = 0)
{
    const ViewConst* __restrict__ views = a.views;
    const int B = a.B, C = a.C, bg_blocks = a.bg_blocks, pt_blocks = a.pt_blocks, num_poses = a.num_poses,
              num_cameras = a.num_cameras, cols = a.cols, normalize_mode = a.normalize_mode;
    const double* __restrict__ bg_partial = a.bg_partial;
    const double* __restrict__ pt_partial = a.pt_partial;
    float* __restrict__ gbg               = a.gbg;
    double* __restrict__ gpose            = a.gpose;
    float* __restrict__ gpose_count       = a.gpose_count;
    float* __restrict__ gintr             = a.gintr;
    float* __restrict__ gintr_count       = a.gintr_count;
    // flat pointer: LDS when the sums fit (every round trip to memory is on this block's critical path)
    double* scratch = (num_poses * 7 + num_cameras * (cols + 1) <= kFinalizeSmall) ? s_small : a.scratch;
    // background: thread t sums channel t%16 over the partial rows t/16, t/16+16, ...
    if (part != 2)
    {
        const int c = threadIdx.x % kMaxChannels, k0 = threadIdx.x / kMaxChannels;
        constexpr int GR = NT / kMaxChannels;
        double v = 0;
#pragma unroll(NT >= 1024 ? 16 : 8)
        for (int k = k0; k < bg_blocks; k += GR) v += bg_partial[(size_t)k * kMaxChannels + c];
        sh[threadIdx.x] = v;
        __syncthreads();
        if (threadIdx.x < kMaxChannels)
        {
            double t = 0;
            for (int g = 0; g < GR; ++g) t += sh[g * kMaxChannels + threadIdx.x];
            if ((int)threadIdx.x < C) gbg[threadIdx.x] = (float)t;
        }
        __syncthreads();
    }
    if ((!gpose && !gintr) || part == 1) return;

    // scratch: [num_poses*7] pose sums + count, then [num_cameras*(cols+1)] intrinsics sums + count
    double* sp = scratch;
    double* si = scratch + (size_t)num_poses * 7;
    for (int k = threadIdx.x; k < num_poses * 7 + num_cameras * (cols + 1); k += NT) scratch[k] = 0;
    __syncthreads();
    for (int b = 0; b < B; ++b)
    {
        // thread t sums value t%32 (21 used) over the partial rows t/32, t/32+8, ...
        const int q = threadIdx.x % 32, k0 = threadIdx.x / 32;
        constexpr int GR = NT / 32;
        double v = 0;
        if (q < kAcc)
#pragma unroll(NT >= 1024 ? 16 : 8)
            for (int k = k0; k < pt_blocks; k += GR) v += pt_partial[((size_t)b * pt_blocks + k) * kPartialStride + q];
        sh[threadIdx.x] = v;
        __syncthreads();
        if (threadIdx.x < kAcc)
        {
            double t = 0;
            for (int g = 0; g < GR; ++g) t += sh[g * 32 + threadIdx.x];
            const ViewConst& vc = views[b];
            const int qq        = threadIdx.x;
            // distinct threads write distinct addresses; views are processed one after another
            if (qq < 6)
                sp[(size_t)vc.image_index * 7 + qq] += t;
            else if (qq == 6)
                sp[(size_t)vc.image_index * 7 + 6] += t;
            else if (qq == 7)
                si[(size_t)vc.camera_index * (cols + 1) + cols] += t;
            else if (qq - 8 < cols)
                si[(size_t)vc.camera_index * (cols + 1) + (qq - 8)] += t;
        }
        __syncthreads();
    }
    if (gpose)
    {
        for (int f = threadIdx.x; f < num_poses; f += NT)
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
        // NormalizeGradient<float,13> on the flat buffer whatever the row width (:1633) in mode 0: element t = floats
        // 13t..13t+12 divided by count[t]; mode 1 normalises row t
        const int total = num_cameras * cols;
        for (int k = threadIdx.x; k < total; k += NT)
        {
            float v     = (float)si[(size_t)(k / cols) * (cols + 1) + (k % cols)];
            const int t = normalize_mode == 0 ? k / 13 : k / cols;
            if (t < num_cameras)
            {
                const float c = (float)si[(size_t)t * (cols + 1) + cols];
                if (c > 0) v = v / c;
            }
            gintr[k] = v;
        }
        for (int k = threadIdx.x; k < num_cameras; k += NT) gintr_count[k] = (float)si[(size_t)k * (cols + 1) + cols];
    }
}

// NormalizeGradient<float,3> on the [N,4] point-gradient buffer (:1620-1627).  mode 0 reproduces the reference's
// vec3 view (element t = floats 3t..3t+2 divided by count[t]); mode 1 normalises row t by count[t].
// Fused with the reduction of the partial rows, which then costs no launch of its own and hides behind the
// normalisation.  One workgroup reads the ~400 KB of partial rows in 16 us when nothing else runs and in ~50 us next
// to the normalisation's traffic, so with point gradients the reduction has two stages: kFinalizeParts workgroups for
// the background sums and as many for every view each reduce a slice of the partial rows to one row (a workgroup
// that walked the views one after the other spent 2 to 3 us on each: 40 us for a batch of 16), and the one that
// finishes last (ticket counter) reduces those rows, in their fixed order, and writes the outputs.  The other
// workgroups normalise.  Without point gradients (n = 0) a single workgroup of NT = kFinalizeBlock threads does the
// whole reduction.
// The rows of the first stage go from their writers to the last workgroup through agent-scope atomic stores and
// loads (past the L2 of the XCD, which is not coherent with the others'), the stores waited for before the ticket is
// taken: a release / acquire pair around the ticket would write back and invalidate the whole L2 of the XCD, once per
// workgroup, under the normalisation's traffic.
constexpr int kNormPer = 4;  // point-gradient rows per thread of the normalisation

__device__ __forceinline__ void mini_store(double* p, double v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ double mini_load(const double* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Second stage: the kFinalizeParts rows of the background sums and of every view -> the outputs (as finalize_block).
template <int NT>
__device__ static void finalize_last(const FinalizeArg& a, const double* bg_m, const double* pt_m, double* sh,
                                     double* s_small)
{
    const int B = a.B, C = a.C, num_poses = a.num_poses, num_cameras = a.num_cameras, cols = a.cols;
    double* scratch = (num_poses * 7 + num_cameras * (cols + 1) <= kFinalizeSmall) ? s_small : a.scratch;
    if ((int)threadIdx.x < kMaxChannels)
    {
        double t = 0;
        for (int r = 0; r < kFinalizeParts; ++r) t += mini_load(bg_m + r * kMaxChannels + threadIdx.x);
        if ((int)threadIdx.x < C) a.gbg[threadIdx.x] = (float)t;
    }
    if (!a.gpose && !a.gintr) return;
    double* sp = scratch;
    double* si = scratch + (size_t)num_poses * 7;
    for (int k = threadIdx.x; k < num_poses * 7 + num_cameras * (cols + 1); k += NT) scratch[k] = 0;
    __syncthreads();
    constexpr int VIEWS = NT / 32;  // views summed side by side: thread = (view, value)
    for (int b0 = 0; b0 < B; b0 += VIEWS)
    {
        const int b = b0 + (int)threadIdx.x / 32, q = threadIdx.x % 32;
        double t = 0;
        if (b < B && q < kAcc)
            for (int r = 0; r < kFinalizeParts; ++r) t += mini_load(pt_m + ((size_t)b * kFinalizeParts + r) * kPartialStride + q);
        sh[threadIdx.x] = t;
        __syncthreads();
        // the views of the chunk one after the other: distinct threads write distinct addresses, the order of the
        // additions to a pose or camera shared by views is that of the views
        if ((int)threadIdx.x < kAcc)
        {
            const int qq = threadIdx.x;
            for (int v = 0; v < VIEWS && b0 + v < B; ++v)
            {
                const double tv     = sh[v * 32 + qq];
                const ViewConst& vc = a.views[b0 + v];
                if (qq < 7)
                    sp[(size_t)vc.image_index * 7 + qq] += tv;
                else if (qq == 7)
                    si[(size_t)vc.camera_index * (cols + 1) + cols] += tv;
                else if (qq - 8 < cols)
                    si[(size_t)vc.camera_index * (cols + 1) + (qq - 8)] += tv;
            }
        }
        __syncthreads();
    }
    if (a.gpose)
    {
        for (int f = threadIdx.x; f < num_poses; f += NT)
        {
            float c          = (float)sp[(size_t)f * 7 + 6];
            a.gpose_count[f] = c;
            for (int k = 0; k < 6; ++k)
            {
                double t                   = sp[(size_t)f * 7 + k];
                a.gpose[(size_t)f * 6 + k] = (c > 0) ? t / (double)c : t;
            }
        }
    }
    if (a.gintr)
    {
        const int total = num_cameras * cols;
        for (int k = threadIdx.x; k < total; k += NT)
        {
            float v     = (float)si[(size_t)(k / cols) * (cols + 1) + (k % cols)];
            const int t = a.normalize_mode == 0 ? k / 13 : k / cols;
            if (t < num_cameras)
            {
                const float c = (float)si[(size_t)t * (cols + 1) + cols];
                if (c > 0) v = v / c;
            }
            a.gintr[k] = v;
        }
        for (int k = threadIdx.x; k < num_cameras; k += NT) a.gintr_count[k] = (float)si[(size_t)k * (cols + 1) + cols];
    }
}

// workgroups of the first stage of finalize_body for a batch of B views
static int finalize_first_stage(int B) { return kFinalizeParts * (1 + B); }

template <int NT>
__device__ __forceinline__ void finalize_body(FinalizeArg a, float* __restrict__ g, const float* __restrict__ count, int n,
                                              int mode)
{
    const int first_stage = n > 0 ? kFinalizeParts * (1 + a.B) : 0;
    if ((int)blockIdx.x < (first_stage ? first_stage : 1))
    {
        __shared__ double sh[NT];
        __shared__ double s_small[kFinalizeSmall];
        __shared__ int s_last;
        if (first_stage)
        {
            const int r     = blockIdx.x % kFinalizeParts;
            const int which = blockIdx.x / kFinalizeParts;  // 0: background sums; 1 + b: view b
            double* bg_m    = a.mini;
            double* pt_m    = a.mini + kFinalizeParts * kMaxChannels;
            if (which == 0)
            {
                const int c = threadIdx.x % kMaxChannels, k0 = threadIdx.x / kMaxChannels;
                constexpr int GR = NT / kMaxChannels;
                const int lo = (int)((long long)a.bg_blocks * r / kFinalizeParts);
                const int hi = (int)((long long)a.bg_blocks * (r + 1) / kFinalizeParts);
                double v     = 0;
#pragma unroll 8
                for (int k = lo + k0; k < hi; k += GR) v += a.bg_partial[(size_t)k * kMaxChannels + c];
                sh[threadIdx.x] = v;
                __syncthreads();
                if (threadIdx.x < kMaxChannels)
                {
                    double t = 0;
                    for (int q = 0; q < GR; ++q) t += sh[q * kMaxChannels + threadIdx.x];
                    mini_store(bg_m + r * kMaxChannels + threadIdx.x, t);
                }
            }
            else
            {
                const int b = which - 1;
                const int q = threadIdx.x % 32, k0 = threadIdx.x / 32;
                constexpr int GR = NT / 32;
                const int lo = (int)((long long)a.pt_blocks * r / kFinalizeParts);
                const int hi = (int)((long long)a.pt_blocks * (r + 1) / kFinalizeParts);
                double v     = 0;
                if (q < kAcc)
#pragma unroll 8
                    for (int k = lo + k0; k < hi; k += GR)
                        v += a.pt_partial[((size_t)b * a.pt_blocks + k) * kPartialStride + q];
                sh[threadIdx.x] = v;
                __syncthreads();
                if (threadIdx.x < kAcc)
                {
                    double t = 0;
                    for (int w = 0; w < GR; ++w) t += sh[w * 32 + threadIdx.x];
                    mini_store(pt_m + ((size_t)b * kFinalizeParts + r) * kPartialStride + threadIdx.x, t);
                }
            }
            __builtin_amdgcn_s_waitcnt(0);  // the stores of this lane have been acknowledged ...
            __syncthreads();                // ... and those of the workgroup, before its ticket is taken
            if (threadIdx.x == 0) s_last = atomicAdd(a.ticket, 1u) == (uint32_t)(first_stage - 1);
            __syncthreads();
            if (!s_last) return;
            finalize_last<NT>(a, bg_m, pt_m, sh, s_small);
            return;
        }
        finalize_block<NT>(a, sh, s_small);
        return;
    }
    // kNormPer elements per thread, kNormPer wavefront-strided count loads in flight (the chain count -> row -> store is
    // two dependent round trips and most counts are zero)
    const int t0 = (blockIdx.x - first_stage) * (NT * kNormPer) + threadIdx.x;
    float c[kNormPer];
#pragma unroll
    for (int k = 0; k < kNormPer; ++k)
    {
        const int t = t0 + k * NT;
        c[k]        = t < n ? __builtin_nontemporal_load(count + t) : 0.f;
    }
    float v[kNormPer][3];
#pragma unroll
    for (int k = 0; k < kNormPer; ++k)
    {
        const int t    = t0 + k * NT;
        const size_t o = (mode == 0) ? 3 * (size_t)t : 4 * (size_t)t;
        if (c[k] > 0)
        {
            v[k][0] = g[o + 0];
            v[k][1] = g[o + 1];
            v[k][2] = g[o + 2];
        }
    }
#pragma unroll
    for (int k = 0; k < kNormPer; ++k)
    {
        const int t    = t0 + k * NT;
        const size_t o = (mode == 0) ? 3 * (size_t)t : 4 * (size_t)t;
        if (c[k] > 0)
        {
            g[o + 0] = v[k][0] / c[k];
            g[o + 1] = v[k][1] / c[k];
            g[o + 2] = v[k][2] / c[k];
        }
    }
}

__global__ __launch_bounds__(kFinalizeBlock) void finalize_kernel(FinalizeArg a)
{
    finalize_body<kFinalizeBlock>(a, nullptr, nullptr, 0, 0);
}

// One view: the rows to normalise are the items of its work queue (a few percent of the points), which costs so
// little that the reduction is the whole duration of the kernel; it then runs in one stage (one workgroup of 1024
// threads: half the dependent round trips of the two stages with their ticket) beside the workgroups that normalise,
// four sub-queues each.  Element t of the normalisation is point t in either mode.
constexpr int kQueuesPerBlock = 2;  // 512 threads per sub-queue: about one item per thread

__global__ __launch_bounds__(kFinalizeBlock) void finalize_queue_kernel(FinalizeArg a, float* __restrict__ g,
                                                                        const float* __restrict__ count, int mode)
{
    if (blockIdx.x < 2)
    {
        __shared__ double sh[kFinalizeBlock];
        __shared__ double s_small[kFinalizeSmall];
        finalize_block<kFinalizeBlock>(a, sh, s_small, 1 + (int)blockIdx.x);
        return;
    }
    constexpr int TPQ = kFinalizeBlock / kQueuesPerBlock;  // threads per sub-queue
    const int q       = (blockIdx.x - 2) * kQueuesPerBlock + (threadIdx.x / TPQ);
    if (q >= kNumQueues) return;
    const uint32_t items = a.q_counts[q];
    for (uint32_t e = threadIdx.x % TPQ; e < items; e += TPQ)
    {
        const uint32_t t = (uint32_t)__builtin_nontemporal_load(a.q_items + (size_t)q * a.q_cap + e);
        const float c    = count[t];
        const size_t o   = (mode == 0) ? 3 * (size_t)t : 4 * (size_t)t;
        if (c > 0)
        {
            const float v0 = g[o + 0], v1 = g[o + 1], v2 = g[o + 2];
            g[o + 0] = v0 / c;
            g[o + 1] = v1 / c;
            g[o + 2] = v2 / c;
        }
    }
}

// 8 waves per SIMD (<= 64 VGPRs): the normalisation lives on memory latency; the registers the reduction would like
// to take (104) halve its occupancy and cost it 40%.
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(8, 8))) void finalize_normalize_kernel(
    FinalizeArg a, float* __restrict__ g, const float* __restrict__ count, int n, int mode)
{
    finalize_body<kBlock>(a, g, count, n, mode);
}

// ------------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------------
void launch_interleave(const Levels& lv, int blocks, float* ig, float2* dw, double* partial, uint32_t* q_counts,
                       const ViewPrep& vp, hipStream_t st)
{
    if (lv.C == 8)
        hipLaunchKernelGGL((interleave_kernel<8>), dim3(blocks), dim3(kBlock), 0, st, lv, ig, dw, partial, q_counts, vp);
    else if (lv.C == 4)
        hipLaunchKernelGGL((interleave_kernel<4>), dim3(blocks), dim3(kBlock), 0, st, lv, ig, dw, partial, q_counts, vp);
    else
        hipLaunchKernelGGL((interleave_kernel<0>), dim3(blocks), dim3(kBlock), 0, st, lv, ig, dw, partial, q_counts, vp);
}

template <int CT, bool HALF>
static void launch_bwd_tex_t(const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp,
                             const float* ig, const float2* dw, const adop_backward_buffers* g, int identity_index,
                             const QueueArg& q, adop_stats* stats, hipStream_t st)
{
    int grid = (pc.n + kBlock - 1) / kBlock;
    if (lv.B > 1)
        hipLaunchKernelGGL((backward_tex_kernel<CT, HALF, true>), dim3(grid), dim3(kBlock), 0, st, pc, views, lv, rp, ig,
                           dw, g->grad_texture, g->grad_points, g->grad_points_count, identity_index, q.counts, q.items,
                           q.cap, q.concurrent, stats);
    else
        hipLaunchKernelGGL((backward_tex_kernel<CT, HALF, false>), dim3(grid), dim3(kBlock), 0, st, pc, views, lv, rp, ig,
                           dw, g->grad_texture, g->grad_points, g->grad_points_count, identity_index, q.counts, q.items,
                           q.cap, 0, stats);
}

template <int CT, bool HALF>
static void launch_bwd_ghost_t(const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp,
                               const float* ig, const adop_backward_buffers* g, int want_pose, int want_intr,
                               int identity_index, int b, const QueueArg& q, int ghost_blocks, double* partial,
                               hipStream_t st)
{
    if (b < 0)  // every view at once: view = blockIdx.y
        hipLaunchKernelGGL((backward_ghost_kernel<CT, HALF>), dim3(ghost_blocks, lv.B), dim3(kBlock), 0, st, pc, views, lv,
                           rp, ig, g->grad_points, g->grad_points_count, want_pose, want_intr, identity_index, -1, 0, 0,
                           q.counts, q.items, q.cap, partial);
    else
        hipLaunchKernelGGL((backward_ghost_kernel<CT, HALF>), dim3(ghost_blocks), dim3(kBlock), 0, st, pc, views, lv, rp,
                           ig, g->grad_points, g->grad_points_count, want_pose, want_intr, identity_index, b, b == 0,
                           q.normalize, q.counts + (size_t)b * kNumQueues, q.items + (size_t)b * kNumQueues * q.cap, q.cap,
                           partial);
}

#define ADOP_DISPATCH_C_HALF(FN, ...)                                   \
    do                                                                  \
    {                                                                   \
        if (lv.C == 8)                                                  \
            half ? FN<8, true>(__VA_ARGS__) : FN<8, false>(__VA_ARGS__); \
        else if (lv.C == 4)                                             \
            half ? FN<4, true>(__VA_ARGS__) : FN<4, false>(__VA_ARGS__); \
        else                                                            \
            half ? FN<0, true>(__VA_ARGS__) : FN<0, false>(__VA_ARGS__); \
    } while (0)

// descriptor gradient of one view + the work queue of its ghost / spatial gradients
void launch_backward_tex(const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp, bool half,
                         const float* ig, const float2* dw, const adop_backward_buffers* g, int identity_index,
                         const QueueArg& q, adop_stats* stats, hipStream_t st)
{
    if (pc.n < 1) return;
    ADOP_DISPATCH_C_HALF(launch_bwd_tex_t, pc, views, lv, rp, ig, dw, g, identity_index, q, stats, st);
}

// ghost / spatial gradients of the queued points of one view
void launch_backward_ghost(const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp, bool half,
                           const float* ig, const adop_backward_buffers* g, int want_pose, int want_intr,
                           int identity_index, int b, const QueueArg& q, int ghost_blocks, double* partial,
                           hipStream_t st)
{
    if (pc.n < 1) return;
    ADOP_DISPATCH_C_HALF(launch_bwd_ghost_t, pc, views, lv, rp, ig, g, want_pose, want_intr, identity_index, b, q,
                         ghost_blocks, partial, st);
}

#undef ADOP_DISPATCH_C_HALF

void launch_finalize(const ViewConst* views, int B, int C, const double* bg_partial, int bg_blocks,
                     const double* pt_partial, int pt_blocks, const adop_backward_buffers* g, int num_poses,
                     int num_cameras, int cols, int normalize_mode, double* scratch, double* mini, uint32_t* ticket, int n,
                     const QueueArg& q, const adop_tuning& tn, hipStream_t st)
{
    FinalizeArg a{views, B, C, bg_partial, bg_blocks, pt_partial, pt_blocks, g->grad_background, g->grad_pose,
                  g->grad_pose_count, num_poses, g->grad_intrinsics, g->grad_intrinsics_count, num_cameras, cols,
                  normalize_mode, scratch, mini, ticket, nullptr, nullptr, 0};
    if (!g->grad_points || n < 1) n = 0;
    const int by_queue = tn.normalize_by_queue;
    if (n == 0)
        hipLaunchKernelGGL(finalize_kernel, dim3(1), dim3(kFinalizeBlock), 0, st, a);
    else if (q.normalize)
        // one view: the spatial-gradient kernel has normalised the rows; two workgroups reduce the partial sums
        hipLaunchKernelGGL(finalize_queue_kernel, dim3(2), dim3(kFinalizeBlock), 0, st, a, g->grad_points,
                           g->grad_points_count, normalize_mode);
    else if (B == 1 && by_queue)
    {
        // (with several views a point sits in several queues and would be divided more than once)
        a.q_counts = q.counts;
        a.q_items  = q.items;
        a.q_cap    = q.cap;
        hipLaunchKernelGGL(finalize_queue_kernel, dim3(2 + kNumQueues / kQueuesPerBlock), dim3(kFinalizeBlock), 0, st, a,
                           g->grad_points, g->grad_points_count, normalize_mode);
    }
    else
        hipLaunchKernelGGL(finalize_normalize_kernel, dim3(finalize_first_stage(B) + (n + kBlock * kNormPer - 1) / (kBlock * kNormPer)), dim3(kBlock), 0, st, a,
                           g->grad_points, g->grad_points_count, n, normalize_mode);
}

}  // namespace adop
