// tile_kernels.hip — the two per-tile kernels of the binned forward pass (gfx950).
//
// One workgroup owns one screen tile of 16 x 16 level-0 pixels and the bin of 16-byte entries bin_kernel<1> wrote for
// it.  Counters on MI355X show the direct forward (prepass_kernel, blend_kernel) to be bound by vector instruction
// issue — the per-wavefront ballot loops that merge lanes by pixel — not by memory.  Here the merge needs no ballots and
// no float atomics: integer LDS atomics run at 12-25 clocks per wavefront instruction and tolerate lanes that share
// an address (the native LDS float add takes ~200 clocks, a compare-and-swap add 34 and up).
//
//   tile_depth_kernel   ds_min_u64 of (depth bits | point id) into the tile's pixels of every level; the levels < lt
//                       (owned by the tile) are stored to depth_index, the coarse levels (a window of a few pixels
//                       shared with the neighbouring tiles) are merged with one global atomicMin per touched pixel
//   tile_blend_kernel   per batch of entries: fuzzy depth test against the final depth; every accepted (entry, level)
//                       is pushed on the linked list of its pixel (one LDS exchange), the descriptors are staged in
//                       LDS, then one thread per pixel walks its list and sums in registers; the levels < lt are
//                       resolved straight to the output tensors, the coarse windows are added to the global
//                       pixel-major accumulators (one cache-line atomic per pixel) and resolved by resolve_kernel
#include <stdlib.h>

#include "common.h"
#include "launch.h"

#pragma clang fp contract(off)

namespace adop
{
// Local layout of the pixels a tile touches: levels < lt are the tile's own (32 >> l) x (8 >> l) rectangles; a coarser
// level is the window of ((extent - 1) >> l) + 2 pixels per axis that rint(ip * 0.5^l) can reach from the tile.
struct TileLayout
{
    int ox[ADOP_MAX_LAYERS], oy[ADOP_MAX_LAYERS], wx[ADOP_MAX_LAYERS], wy[ADOP_MAX_LAYERS], base[ADOP_MAX_LAYERS + 1];
    int cwx[ADOP_MAX_LAYERS], cwy[ADOP_MAX_LAYERS];  // extents clipped to the image: a local pixel inside them is in the image
};

__host__ __device__ inline int tile_extent(int shift, int l, int lt)
{
    return l < lt ? 1 << (shift - l) : (((1 << shift) - 1) >> l) + 2;
}

__device__ __forceinline__ TileLayout tile_layout(const Levels& lv, int tx, int ty, int lt, int num)
{
    TileLayout t;
    int base = 0;
#pragma unroll
    for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
    {
        t.ox[l] = t.oy[l] = t.wx[l] = t.wy[l] = t.cwx[l] = t.cwy[l] = 0;
        t.base[l]                             = base;
        if (l < num)
        {
            t.ox[l] = l < lt ? tx << (kTileShiftX - l) : (tx << kTileShiftX) >> l;
            t.oy[l] = l < lt ? ty << (kTileShiftY - l) : (ty << kTileShiftY) >> l;
            t.wx[l] = tile_extent(kTileShiftX, l, lt);
            t.wy[l] = tile_extent(kTileShiftY, l, lt);
            int rx = lv.l[l].w - t.ox[l], ry = lv.l[l].h - t.oy[l];
            t.cwx[l] = rx < 0 ? 0 : (rx < t.wx[l] ? rx : t.wx[l]);
            t.cwy[l] = ry < 0 ? 0 : (ry < t.wy[l] ? ry : t.wy[l]);
            base += t.wx[l] * t.wy[l];
        }
    }
    t.base[ADOP_MAX_LAYERS] = base;
    return t;
}

// number of local pixels of the levels [0, upto)
__host__ __device__ inline int tile_pixels(int lt, int upto)
{
    int n = 0;
    for (int l = 0; l < upto; ++l) n += tile_extent(kTileShiftX, l, lt) * tile_extent(kTileShiftY, l, lt);
    return n;
}

constexpr int kTileMaxPixels = 512;  // 256 + 64 own pixels and the coarse windows (9x3 + 5x2 + 3x2)

// LT = LT as a compile-time constant: the extents and offsets of the tile's pixel windows are then constants instead
// of scalar registers (the kernel is short: a tile's set-up is a third of it).
// 8 waves per SIMD: the kernel is a chain of round trips per tile (bin range, entries, stores) with little arithmetic,
// and its 100 scalar registers allow only 6.
template <int LT>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(8, 8))) void tile_depth_kernel(Levels lv, BinArg bin, int num_tiles)
{
    __shared__ unsigned long long s_depth[kTileMaxPixels];
    if (bin.overflow && *bin.overflow) return;  // the bins of this workspace were too small for the call
    const int tiles_per_view = bin.tiles_x * bin.tiles_y;
    // the first max_rows workgroups take the further slices of the bins that are split (they are the longest pieces of
    // work of the launch: first, so that they do not form its tail); most calls have none
    const bool extra = (int)blockIdx.x < bin.max_rows;
    if (extra && blockIdx.x >= *bin.row_count) return;
    // (tile, first entry, end, slice word): the tiles fullest bin first, behind them the places of the slices
    const uint4 mine = bin.order[extra ? (uint32_t)num_tiles + blockIdx.x : blockIdx.x - (uint32_t)bin.max_rows];
    const int slices         = (int)(mine.w & 1023u);  // K > 1: this workgroup has slice `slice` of K of the tile's bin
    const int slice          = (int)(mine.w >> 10 & 1023u);
    const int row0           = (int)(mine.w >> 20);
    if (extra && slices == 0) return;  // (the place of a slice 0, which sits among the tiles)
    const int tile           = (int)mine.x;
    const int b              = tile / tiles_per_view;
    const int tr             = tile - b * tiles_per_view;
    const int ty             = tr / bin.tiles_x;
    const int tx             = tr - ty * bin.tiles_x;
    const uint32_t start     = mine.y;
    const uint32_t end       = mine.z;
    if (end == start && slices <= 1)  // (workgroup-uniform) an empty bin, four tiles in ten of a typical view: the tile's own pixels are
    {                  // cleared and nothing else happens
#pragma unroll
        for (int l = 0; l < LT; ++l)
        {
            if (l < lv.num)
            {
                const LevelArg& L = lv.l[l];
                const int W       = 1 << (kTileShiftX - l);
                const int q       = threadIdx.x;
                const int cy = q / W, cx = q - cy * W;
                const int px = (tx << (kTileShiftX - l)) + cx, py = (ty << (kTileShiftY - l)) + cy;
                if (q < W * (1 << (kTileShiftY - l)) && px < L.w && py < L.h)
                    L.depth_index[(size_t)b * L.w * L.h + (size_t)py * L.w + px] = kClearPacked;
            }
        }
        return;
    }
    const TileLayout T       = tile_layout(lv, tx, ty, LT, lv.num);
    const int npix           = T.base[ADOP_MAX_LAYERS];

    for (int p = threadIdx.x; p < npix; p += kBlock) s_depth[p] = kClearPacked;
    __syncthreads();

    for (uint32_t e = start + threadIdx.x; e < end; e += kBlock)
    {
        const float4 E       = bin.entries[e];
        const uint32_t word  = __float_as_uint(E.w);
        const uint32_t id    = word & kEntryIdMask;
        const int nlev       = (int)(word >> 28 & 7u);
        const bool primary   = (word & kEntryPrimary) != 0;
        const uint32_t zbits = f2u(E.z) & 0x7FFFFFFFu;  // the sign carries the dropout flag
        const uint64_t pk    = ((uint64_t)zbits << 32) | id;
        float x = E.x, y = E.y;
        uint32_t miss = 0;  // coarse levels whose pixel is not in the tile's window (does not happen for in-image points)
#pragma unroll
        for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
        {
            if (l < lv.num)
            {
                const int px = f2i_rn(x), py = f2i_rn(y);
                const int cx = px - T.ox[l], cy = py - T.oy[l];
                const bool live = l < nlev && (l < LT || primary);
                const bool hit  = live && (unsigned)cx < (unsigned)T.cwx[l] && (unsigned)cy < (unsigned)T.cwy[l];
                if (hit)
                {
                    // Early depth test on the LDS copy from level 1 on: the entries of a tile share few coarse pixels,
                    // LDS atomics of one instruction on one address run one after the other, and after the first
                    // batches most entries lose against the value already there (a plain read is a broadcast).
                    // (builtins that keep the LDS address space: with the register limit of 8 waves per SIMD the
                    // compiler fails on the generic-pointer forms)
                    unsigned long long* dst = &s_depth[T.base[l] + cy * T.wx[l] + cx];
                    if (l == 0 || pk < __hip_atomic_load(dst, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP))
                        __hip_atomic_fetch_min(dst, (unsigned long long)pk, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
                if (l >= LT && live && !hit) miss |= 1u << l;
                x *= 0.5f;
                y *= 0.5f;
            }
        }
        if (miss)  // straight to memory
        {
            x = E.x;
            y = E.y;
            for (int l = 0; l < lv.num; ++l)
            {
                const LevelArg& L = lv.l[l];
                const int px = f2i_rn(x), py = f2i_rn(y);
                if ((miss >> l & 1u) && (unsigned)px < (unsigned)L.w && (unsigned)py < (unsigned)L.h)
                    atomicMin((unsigned long long*)(L.depth_index + (size_t)b * L.w * L.h + (size_t)py * L.w + px),
                              (unsigned long long)pk);
                x *= 0.5f;
                y *= 0.5f;
            }
        }
    }
    __syncthreads();

    // A slice of a split bin leaves the minima of the tile's own pixels in its row; the slice that finishes last takes
    // the minimum over the K rows and stores it (the coarse windows go through atomics anyway).
    bool store_own = true;
    if (slices > 1)  // (workgroup-uniform)
    {
        __shared__ uint32_t s_ticket;
        const int own = T.base[LT];  // local pixels of the levels the tile owns (LT <= lv.num)
        unsigned long long* rows = (unsigned long long*)bin.rows;
        const size_t kRow        = (size_t)bin.row_floats / 2;  // 64-bit words per row
        for (int p = threadIdx.x; p < own; p += kBlock) rows[(size_t)(row0 + slice) * kRow + p] = s_depth[p];
        __threadfence();
        __syncthreads();
        if (threadIdx.x == 0) s_ticket = atomicAdd(&bin.tickets[row0], 1u);
        __syncthreads();
        store_own = s_ticket == (uint32_t)(slices - 1);
        if (store_own)
        {
            __threadfence();
            for (int p = threadIdx.x; p < own; p += kBlock)
            {
                unsigned long long v = kClearPacked;
                for (int sl = 0; sl < slices; ++sl)
                {
                    const unsigned long long u = __builtin_nontemporal_load(&rows[(size_t)(row0 + sl) * kRow + p]);
                    v                          = u < v ? u : v;
                }
                s_depth[p] = v;
            }
            __syncthreads();
        }
    }

#pragma unroll
    for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
    {
        if (l < lv.num)
        {
            const LevelArg& L = lv.l[l];
            const int W       = T.wx[l];
            for (int q = threadIdx.x; q < W * T.wy[l]; q += kBlock)
            {
                const int cy = q / W, cx = q - cy * W;
                const int px = T.ox[l] + cx, py = T.oy[l] + cy;
                if (px < L.w && py < L.h)
                {
                    unsigned long long v = s_depth[T.base[l] + q];
                    uint64_t* dst        = L.depth_index + (size_t)b * L.w * L.h + (size_t)py * L.w + px;
                    if (l < LT)
                    {
                        if (store_own) *dst = v;  // the tile owns the pixel
                    }
                    else if (v != kClearPacked)
                        atomicMin((unsigned long long*)dst, v);
                }
            }
        }
    }
}

// Buckets of the gather (a tile has kBlock level-0 pixels): bucket p < 256 is level-0 pixel p; the level-1 pixels and
// the pixels of the coarse windows collect many more entries each, so their lists are split in 2 and up to 3 parts
// (an entry picks the part by its batch slot): buckets 256 + 2*q + part and 384 + parts*c + part.
constexpr int kL1Parts       = 2;
constexpr int kMaxCoarseParts = 3;
constexpr int kL1Bucket0     = 256;
constexpr int kCoarseBucket0 = 384;
constexpr uint32_t kListEnd = 0xFFFFu;

template <int CT, int BATCH>
__device__ __forceinline__ void add_staged(float* acc, const float* s_stage, int slot, int C)
{
    constexpr int CMAX = CT ? CT : kMaxChannels;
    if (CT == 8)
    {
        // (two planes of float4, [half][slot]: the lanes of a wavefront store consecutive 16-byte words)
        const float4* d = (const float4*)s_stage + slot;
        float4 u = d[0], v = d[BATCH];
        acc[0] += u.x; acc[1] += u.y; acc[2] += u.z; acc[3] += u.w;
        acc[4] += v.x; acc[5] += v.y; acc[6] += v.z; acc[7] += v.w;
    }
    else if (CT == 4)
    {
        float4 u = *(const float4*)(s_stage + slot * 4);
        acc[0] += u.x; acc[1] += u.y; acc[2] += u.z; acc[3] += u.w;
    }
    else
    {
#pragma unroll
        for (int c = 0; c < CMAX; ++c)
            if (c < C) acc[c] += s_stage[slot * C + c];
    }
}

// K entries per thread and batch (BATCH = K * kBlock, a power of two).
template <int CT, bool HALF, int K>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu((CT != 0 && K == 1) ? 8 : 4, 8))) void tile_blend_kernel(CloudArg pc, Levels lv, ParamArg rp, BinArg bin,
                                                            float* __restrict__ accum, int S,
                                                            const float* __restrict__ background, int write_mask,
                                                            float mask_value, int identity_index, adop_stats* stats, int num_tiles)
{
    constexpr int CMAX  = CT ? CT : kMaxChannels;
    constexpr int BATCH = K * kBlock;
    constexpr int TX    = 1 << kTileShiftX;  // level-0 extent of the tile; TX * TY = kBlock
    constexpr int TY    = 1 << kTileShiftY;
    extern __shared__ __align__(16) unsigned char smem[];
    if (bin.overflow && *bin.overflow) return;  // the bins of this workspace were too small for the call
    const bool STATS = stats != nullptr;
    const int C      = CT ? CT : lv.C;
    const int tid    = threadIdx.x;

    const int tiles_per_view = bin.tiles_x * bin.tiles_y;
    // the first max_rows workgroups take the further slices of the bins that are split (they are the longest pieces of
    // work of the launch: first, so that they do not form its tail); most calls have none
    const bool extra = (int)blockIdx.x < bin.max_rows;
    if (extra && blockIdx.x >= *bin.row_count) return;
    // (tile, first entry, end, slice word): the tiles fullest bin first, behind them the places of the slices
    const uint4 mine = bin.order[extra ? (uint32_t)num_tiles + blockIdx.x : blockIdx.x - (uint32_t)bin.max_rows];
    const int slices         = (int)(mine.w & 1023u);  // > 1: this workgroup has slice `slice` of the tile's bin
    if (extra && slices == 0) return;  // (the place of a slice 0, which sits among the tiles)
    const int tile           = (int)mine.x;
    const int b              = tile / tiles_per_view;
    const int tr             = tile - b * tiles_per_view;
    const int ty             = tr / bin.tiles_x;
    const int tx             = tr - ty * bin.tiles_x;
    const uint32_t start     = mine.y;
    const uint32_t end       = mine.z;
    const int lt             = bin.lt;
    const TileLayout T       = tile_layout(lv, tx, ty, lt, lv.num);
    const int npix           = T.base[ADOP_MAX_LAYERS];
    const int first_coarse   = lt > 1 ? TX * TY + TX * TY / 4 : TX * TY;  // local pixel index of the first coarse pixel
    const int ncoarse        = npix - first_coarse;
    // parts per coarse pixel: the coarse buckets are the second buckets of the threads kBlock/2 .. kBlock-1
    const int cparts = ncoarse * kMaxCoarseParts <= kBlock / 2 ? kMaxCoarseParts : (ncoarse * 2 <= kBlock / 2 ? 2 : 1);

    float* s_stage   = (float*)smem;                     // [BATCH * C]
    float* s_depth   = s_stage + BATCH * C;              // [npix] f32 depth of the local pixels
    uint32_t* s_head = (uint32_t*)(s_depth + npix);      // [2 * kBlock] list heads of the buckets
    uint16_t* s_next = (uint16_t*)(s_head + 2 * kBlock); // [BATCH * num levels] node = level * BATCH + slot

    float acc0[CMAX + 1], acc1[CMAX + 1];  // bucket tid, bucket kBlock + tid
#pragma unroll
    for (int c = 0; c <= CMAX; ++c) acc0[c] = acc1[c] = 0.f;

    if (end > start)  // workgroup-uniform
    {
        // entries of the first batch: requested together with the depth values below
        float4 Enext[K];
#pragma unroll
        for (int k = 0; k < K; ++k)
        {
            const uint32_t e = start + k * kBlock + tid;
            Enext[k]         = e < end ? nt_load4(bin.entries + e) : make_float4(0, 0, -1.f, 0);  // last use of the entry
        }
        // final depth of the local pixels (tile_depth_kernel has completed)
#pragma unroll
        for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
        {
            if (l < lv.num)
            {
                const LevelArg& L = lv.l[l];
                const int W       = T.wx[l];
                for (int q = tid; q < W * T.wy[l]; q += kBlock)
                {
                    const int cy = q / W, cx = q - cy * W;
                    const int px = T.ox[l] + cx, py = T.oy[l] + cy;
                    float d = 0.f;
                    if (px < L.w && py < L.h)
                        d = __uint_as_float(
                            ((const uint32_t*)(L.depth_index + (size_t)b * L.w * L.h + (size_t)py * L.w + px))[1]);
                    s_depth[T.base[l] + q] = d;
                }
            }
        }
        s_head[tid]          = kListEnd;
        s_head[kBlock + tid] = kListEnd;
        __syncthreads();

        const float accept = rp.depth_accept + 1;
        for (uint32_t b0 = start; b0 < end; b0 += BATCH)  // workgroup-uniform
        {
            // -- entries of this thread, their descriptors, and the entries of the next batch (all requested before
            //    anything waits: a batch is a chain of dependent memory round trips) --------------------------------
            float4 E[K];
            float t[K][CMAX];
            bool ok[K];
#pragma unroll
            for (int k = 0; k < K; ++k) E[k] = Enext[k];
#pragma unroll
            for (int k = 0; k < K; ++k)
            {
                const uint32_t id = __float_as_uint(E[k].w) & kEntryIdMask;
                ok[k]             = depth_is_rendered(E[k].z);  // dropped points carry -z (:314-315), padding too
                int tex_index     = 0;
                if (ok[k]) tex_index = identity_index ? (int)id : pc.index[id];
                ok[k] = ok[k] && (unsigned)tex_index < (unsigned)pc.num_texels;  // device assert :362
#pragma unroll
                for (int c = 0; c < CMAX; ++c) t[k][c] = 0.f;
                if (ok[k])
                {
#pragma unroll
                    for (int c = 0; c < CMAX; ++c)
                        if (c < C) t[k][c] = tex_fetch<HALF>(pc.texture, (size_t)c * pc.num_texels + tex_index);
                }
            }
#pragma unroll
            for (int k = 0; k < K; ++k)
            {
                const uint32_t e = b0 + BATCH + k * kBlock + tid;
                Enext[k]         = e < end ? nt_load4(bin.entries + e) : make_float4(0, 0, -1.f, 0);  // last use of the entry
            }
            // -- fuzzy depth test per level (:380); an accepted (entry, level) is pushed on the list of its bucket ----
#pragma unroll
            for (int k = 0; k < K; ++k)
            {
                const int slot      = k * kBlock + tid;
                const uint32_t word = __float_as_uint(E[k].w);
                const int nlev      = (int)(word >> 28 & 7u);
                const bool primary  = (word & kEntryPrimary) != 0;
                const float z       = E[k].z;
                float x = E[k].x, y = E[k].y;
                uint32_t miss = 0, accepted_mask = 0;
#pragma unroll
                for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
                {
                    if (l < lv.num)
                    {
                        const int px = f2i_rn(x), py = f2i_rn(y);
                        const int cx = px - T.ox[l], cy = py - T.oy[l];
                        const bool live = ok[k] && l < nlev && (l < lt || primary);
                        const bool hit  = live && (unsigned)cx < (unsigned)T.cwx[l] && (unsigned)cy < (unsigned)T.cwy[l];
                        const int q     = hit ? cy * T.wx[l] + cx : 0;
                        const bool accepted = hit && !(z > s_depth[T.base[l] + q] * accept);
                        if (accepted)
                        {
                            int bucket;
                            if (l == 0)
                                bucket = q;
                            else if (l < lt)
                                bucket = kL1Bucket0 + q * kL1Parts + (slot & (kL1Parts - 1));
                            else
                                bucket = kCoarseBucket0 + (T.base[l] - first_coarse + q) * cparts + slot % cparts;
                            const uint32_t node = (uint32_t)(l * BATCH + slot);
                            uint32_t old = atomicExch(s_head + bucket, node);
                            s_next[node] = (uint16_t)old;
                            accepted_mask |= 1u << l;
                        }
                        if (l >= lt && live && !hit) miss |= 1u << l;
                        x *= 0.5f;
                        y *= 0.5f;
                    }
                }
                if (miss)
                {
                    // coarse pixel outside the tile's window (does not happen for in-image points): blend straight to memory
                    x = E[k].x;
                    y = E[k].y;
                    for (int l = 0; l < lv.num; ++l)
                    {
                        const LevelArg& L = lv.l[l];
                        const int px = f2i_rn(x), py = f2i_rn(y);
                        if ((miss >> l & 1u) && (unsigned)px < (unsigned)L.w && (unsigned)py < (unsigned)L.h)
                        {
                            size_t pix = (size_t)py * L.w + px;
                            float d    = __uint_as_float(((const uint32_t*)(L.depth_index + (size_t)b * L.w * L.h + pix))[1]);
                            if (!(z > d * accept))
                            {
                                float* a = accum + (size_t)ws_pixel(lv, l, b, (uint32_t)pix) * S;
#pragma unroll
                                for (int c = 0; c < CMAX; ++c)
                                    if (c < C) unsafeAtomicAdd(a + c, t[k][c]);
                                unsafeAtomicAdd(a + C, 1.f);
                                accepted_mask |= 1u << l;
                            }
                        }
                        x *= 0.5f;
                        y *= 0.5f;
                    }
                }
                if (STATS)
                {
#pragma unroll
                    for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
                        if (l < lv.num) stat_add(&stats->accepted[l], (accepted_mask >> l & 1u) != 0);
                }
            }
            // -- descriptors staged by batch slot ----------------------------------------------------------------
#pragma unroll
            for (int k = 0; k < K; ++k)
            {
                const int slot = k * kBlock + tid;
                if (ok[k])
                {
                    if (CT == 8)
                    {
                        float4* d = (float4*)s_stage + slot;
                        d[0]      = make_float4(t[k][0], t[k][1], t[k][2], t[k][3]);
                        d[BATCH]  = make_float4(t[k][4], t[k][5], t[k][6], t[k][7]);
                    }
                    else if (CT == 4)
                        *(float4*)(s_stage + slot * 4) = make_float4(t[k][0], t[k][1], t[k][2], t[k][3]);
                    else
                    {
#pragma unroll
                        for (int c = 0; c < CMAX; ++c)
                            if (c < C) s_stage[slot * C + c] = t[k][c];
                    }
                }
            }
            __syncthreads();
            // -- gather: every thread walks the lists of its two buckets and empties them ------------------------------
            {
                uint32_t node = s_head[tid];
                float n       = 0.f;
                while (node != kListEnd)
                {
                    add_staged<CT, BATCH>(acc0, s_stage, (int)(node & (BATCH - 1)), C);
                    n += 1.f;
                    node = s_next[node];
                }
                acc0[CMAX] += n;
                s_head[tid] = kListEnd;
                node        = s_head[kBlock + tid];
                n           = 0.f;
                while (node != kListEnd)
                {
                    add_staged<CT, BATCH>(acc1, s_stage, (int)(node & (BATCH - 1)), C);
                    n += 1.f;
                    node = s_next[node];
                }
                acc1[CMAX] += n;
                s_head[kBlock + tid] = kListEnd;
            }
            __syncthreads();
        }
    }

    // A slice of a split bin leaves its sums for the tile's own pixels in its row; the slice that finishes last adds the
    // K rows in their order and resolves the pixels (the coarse windows go through the global accumulators anyway).
    // Row: per thread the C sums and the count of its first accumulator, then of its second.
    bool resolve_own = true;
    if (slices > 1)  // (workgroup-uniform)
    {
        const int slice = (int)(mine.w >> 10 & 1023u), row0 = (int)(mine.w >> 20);
        const bool l1   = tid < kCoarseBucket0 - kL1Bucket0;  // second accumulator: a part of a level-1 pixel
        const int W     = C + 1;
        float* mine_row = bin.rows + (size_t)(row0 + slice) * bin.row_floats + (size_t)tid * 2 * W;
#pragma unroll
        for (int c = 0; c < CMAX; ++c)
            if (c < C) mine_row[c] = acc0[c];
        mine_row[C] = acc0[CMAX];
        if (l1)
        {
#pragma unroll
            for (int c = 0; c < CMAX; ++c)
                if (c < C) mine_row[W + c] = acc1[c];
            mine_row[W + C] = acc1[CMAX];
        }
        __threadfence();
        __syncthreads();
        if (tid == 0) s_head[0] = atomicAdd(&bin.tickets[bin.max_rows + row0], 1u);  // (the lists are empty by now)
        __syncthreads();
        resolve_own = s_head[0] == (uint32_t)(slices - 1);
        if (resolve_own)
        {
            __threadfence();
#pragma unroll
            for (int c = 0; c <= CMAX; ++c) acc0[c] = 0.f;
            if (l1)
            {
#pragma unroll
                for (int c = 0; c <= CMAX; ++c) acc1[c] = 0.f;
            }
            for (int sl = 0; sl < slices; ++sl)
            {
                const float* r = bin.rows + (size_t)(row0 + sl) * bin.row_floats + (size_t)tid * 2 * W;
#pragma unroll
                for (int c = 0; c < CMAX; ++c)
                    if (c < C) acc0[c] += __builtin_nontemporal_load(r + c);
                acc0[CMAX] += __builtin_nontemporal_load(r + C);
                if (l1)
                {
#pragma unroll
                    for (int c = 0; c < CMAX; ++c)
                        if (c < C) acc1[c] += __builtin_nontemporal_load(r + W + c);
                    acc1[CMAX] += __builtin_nontemporal_load(r + W + C);
                }
            }
        }
        __syncthreads();  // (s_head[0] is read by all before anything else may use the LDS)
    }

    // -- resolve (CombineAndFill :726-754, CreateMask :828-847) ----------------------------------------------------
    // level 0: bucket tid is pixel tid of the tile
    if (resolve_own)
    {
        const LevelArg& L = lv.l[0];
        const int px = T.ox[0] + (tid & (TX - 1)), py = T.oy[0] + (tid >> kTileShiftX);
        if (px < L.w && py < L.h)
        {
            const float cou  = acc0[CMAX];
            const size_t hw  = (size_t)L.w * L.h;
            const size_t pix = (size_t)py * L.w + px;
            const size_t o   = (size_t)b * hw + pix;
            // the outputs are not read again by this pass: stored past the caches
            __builtin_nontemporal_store(cou, L.weight + o);
            __builtin_nontemporal_store(end > start ? s_depth[tid] : 100000.f, L.depth + o);  // high word of the packed pixel
            float* out = L.out + (size_t)b * C * hw + pix;
#pragma unroll
            for (int c = 0; c < CMAX; ++c)
                if (c < C)
                {
                    acc0[c] = (cou == 0) ? background[c] : acc0[c] / cou;
                    __builtin_nontemporal_store(acc0[c], out + (size_t)c * hw);
                }
            if (write_mask && L.mask) __builtin_nontemporal_store((cou == 0) ? mask_value : 1.f, L.mask + o);
            if (lv.irec) store_pixel_record<CT>(lv.irec + (size_t)ws_pixel(lv, 0, b, (uint32_t)pix) * C, acc0, C);
        }
    }
    // level 1: buckets kBlock + 2*q and kBlock + 2*q + 1 (adjacent lanes) are the two parts of pixel q
    if (lt > 1)
    {
#pragma unroll
        for (int c = 0; c <= CMAX; ++c) acc1[c] += (tid < kCoarseBucket0 - kL1Bucket0) ? __shfl_xor(acc1[c], 1, 64) : 0.f;
        if (resolve_own && tid < kCoarseBucket0 - kL1Bucket0 && (tid & 1) == 0)
        {
            constexpr int T1  = TX / 2;
            const LevelArg& L = lv.l[1];
            const int q       = tid >> 1;
            const int px = T.ox[1] + (q & (T1 - 1)), py = T.oy[1] + q / T1;
            if (px < L.w && py < L.h)
            {
                const float cou  = acc1[CMAX];
                const size_t hw  = (size_t)L.w * L.h;
                const size_t pix = (size_t)py * L.w + px;
                const size_t o   = (size_t)b * hw + pix;
                L.weight[o]      = cou;
                L.depth[o]       = end > start ? s_depth[TX * TY + q] : 100000.f;
                float* out       = L.out + (size_t)b * C * hw + pix;
#pragma unroll
                for (int c = 0; c < CMAX; ++c)
                    if (c < C)
                    {
                        acc1[c]            = (cou == 0) ? background[c] : acc1[c] / cou;
                        out[(size_t)c * hw] = acc1[c];
                    }
                if (write_mask && L.mask) L.mask[o] = (cou == 0) ? mask_value : 1.f;
                if (lv.irec) store_pixel_record<CT>(lv.irec + (size_t)ws_pixel(lv, 1, b, (uint32_t)pix) * C, acc1, C);
            }
        }
    }
    // coarse windows: the parts of a pixel are summed through LDS, then S consecutive lanes add the C sums and the
    // weight of one pixel to the global accumulators with ONE cache-line atomic
    if (lt < lv.num && end > start)
    {
        float* s_flush = (float*)smem;  // [ncoarse * cparts * S], reuses the stage: all threads are past the gather
        const int u    = tid - (kCoarseBucket0 - kL1Bucket0);
        if (u >= 0 && u < ncoarse * cparts)
        {
            float* f = s_flush + u * S;
#pragma unroll
            for (int c = 0; c < CMAX; ++c)
                if (c < C) f[c] = acc1[c];
            f[C] = acc1[CMAX];
        }
        __syncthreads();
        for (int i = tid; i < ncoarse * S; i += kBlock)
        {
            const int cp = i / S, j = i - cp * S;
            if (j <= C)
            {
                const float* f = s_flush + cp * cparts * S;
                float cou = f[C], v = f[j];
                for (int part = 1; part < cparts; ++part)
                {
                    cou += f[part * S + C];
                    v += f[part * S + j];
                }
                if (cou != 0.f)
                {
                    // level and pixel of coarse pixel cp
                    int l = lt, r = cp;
#pragma unroll
                    for (int k = 2; k < ADOP_MAX_LAYERS; ++k)
                        if (k > lt && k < lv.num && cp >= T.base[k] - first_coarse)
                        {
                            l = k;
                            r = cp - (T.base[k] - first_coarse);
                        }
                    int W = 0, ox = 0, oy = 0, Lw = 0;
#pragma unroll
                    for (int k = 1; k < ADOP_MAX_LAYERS; ++k)
                        if (k == l)
                        {
                            W  = T.wx[k];
                            ox = T.ox[k];
                            oy = T.oy[k];
                            Lw = lv.l[k].w;
                        }
                    const int cy = r / W, cx = r - cy * W;
                    const uint32_t pix = (uint32_t)((oy + cy) * Lw + (ox + cx));  // in the image: something was blended
                    unsafeAtomicAdd(accum + (size_t)ws_pixel(lv, l, b, pix) * S + j, v);
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------------
void launch_tile_depth(const Levels& lv, const BinArg& bin, int num_tiles, hipStream_t st)
{
    if (bin.lt == 1)
        hipLaunchKernelGGL(tile_depth_kernel<1>, dim3(num_tiles + bin.max_rows), dim3(kBlock), 0, st, lv, bin, num_tiles);
    else
        hipLaunchKernelGGL(tile_depth_kernel<2>, dim3(num_tiles + bin.max_rows), dim3(kBlock), 0, st, lv, bin, num_tiles);
}

template <int K>
static size_t tile_blend_lds(const Levels& lv, const BinArg& bin, int S)
{
    size_t npix    = (size_t)tile_pixels(bin.lt, lv.num);
    size_t ncoarse = npix - (size_t)tile_pixels(bin.lt, bin.lt < lv.num ? bin.lt : lv.num);
    size_t stage   = (size_t)K * kBlock * lv.C * 4;
    size_t rest    = npix * 4 + 2 * kBlock * 4 + (size_t)K * kBlock * lv.num * 2 + 16;
    size_t flush   = ncoarse * kMaxCoarseParts * (size_t)S * 4;  // the flush area reuses the LDS from its start
    return stage + rest > flush ? stage + rest : flush;
}

template <int CT, bool HALF, int K>
static hipError_t launch_tile_blend_k(const CloudArg& pc, const Levels& lv, const ParamArg& rp, const BinArg& bin,
                                      int num_tiles, float* accum, int S, const float* background, int write_mask,
                                      float mask_value, int identity_index, adop_stats* stats, hipStream_t st)
{
    if (bin.lt > 2 || tile_pixels(bin.lt, lv.num) > kTileMaxPixels) return hipErrorInvalidValue;
    size_t lds = tile_blend_lds<K>(lv, bin, S);
    static size_t allowed = 0;  // largest dynamic LDS size this instantiation has been enabled for
    if (lds > 65536 && lds > allowed)
    {
        hipError_t e = hipFuncSetAttribute((const void*)tile_blend_kernel<CT, HALF, K>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        allowed = lds;
    }
    hipLaunchKernelGGL((tile_blend_kernel<CT, HALF, K>), dim3(num_tiles + bin.max_rows), dim3(kBlock), lds, st, pc, lv, rp, bin,
                       accum, S, background, write_mask, mask_value, identity_index, stats, num_tiles);
    return hipSuccess;
}

template <int CT, bool HALF>
static hipError_t launch_tile_blend_t(const CloudArg& pc, const Levels& lv, const ParamArg& rp, const BinArg& bin,
                                      int num_tiles, float* accum, int S, const float* background, int write_mask,
                                      float mask_value, int identity_index, adop_stats* stats, int k, hipStream_t st)
{
    if (k == 1)
        return launch_tile_blend_k<CT, HALF, 1>(pc, lv, rp, bin, num_tiles, accum, S, background, write_mask, mask_value,
                                                identity_index, stats, st);
    if (k == 4)
        return launch_tile_blend_k<CT, HALF, 4>(pc, lv, rp, bin, num_tiles, accum, S, background, write_mask, mask_value,
                                                identity_index, stats, st);
    return launch_tile_blend_k<CT, HALF, 2>(pc, lv, rp, bin, num_tiles, accum, S, background, write_mask, mask_value,
                                            identity_index, stats, st);
}

hipError_t launch_tile_blend(const CloudArg& pc, const Levels& lv, const ParamArg& rp, const BinArg& bin, int num_tiles,
                             bool half, float* accum, int S, const float* background, int write_mask,
                             float mask_value, int identity_index, adop_stats* stats, const adop_tuning& tn,
                             hipStream_t st)
{
#define ADOP_TILE(CT, H) \
    launch_tile_blend_t<CT, H>(pc, lv, rp, bin, num_tiles, accum, S, background, write_mask, mask_value, identity_index, stats, tn.tile_k, st)
    if (lv.C == 8) return half ? ADOP_TILE(8, true) : ADOP_TILE(8, false);
    if (lv.C == 4) return half ? ADOP_TILE(4, true) : ADOP_TILE(4, false);
    return half ? ADOP_TILE(0, true) : ADOP_TILE(0, false);
#undef ADOP_TILE
}

}  // namespace adop
