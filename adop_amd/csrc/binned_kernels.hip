// binned_kernels.hip — forward pass through screen-space tile bins (gfx950).
//
// The direct forward (prepass_kernel + blend_kernel) issues ~5 M device-scope atomics per 10 M-point frame and spends
// most of its vector instructions merging lanes by pixel.  Here every point is first sorted into the bin of the
// screen tile it falls in; the per-tile kernels (tile_kernels.hip) then work in LDS.
//
//   bin_count       per point: projection (kept in the point cache), number of bin entries per screen tile
//   tile_scan       exclusive prefix sum of the tile counts
//   bin_scatter     per point: reads the point cache, writes a 16-byte entry (level-0 image point, depth, point id |
//                   flags) into the bin of the tile that owns its level-0 pixel, and into the tile that owns its
//                   level-1 pixel when that is another one (levels are not nested: pixel = rint(ip * 0.5^l))
// The entries of a wavefront are appended with one returning atomic per distinct tile (Morton-ordered clouds put a
// wavefront's points into one to three tiles), so the bins hold runs of consecutive point ids.
#include <stdlib.h>

#include "common.h"
#include "launch.h"

#pragma clang fp contract(off)

namespace adop
{
constexpr uint32_t kNoTile       = 0xFFFFFFFFu;
constexpr uint32_t kInfoTileMask = 0x00FFFFFFu;
constexpr uint32_t kInfoRight    = 1u << 27;
constexpr uint32_t kInfoBelow    = 1u << 28;
constexpr uint32_t kInfoValid    = 1u << 31;

// Pixels of every level -> does the point touch the image at all, how many levels precede the LOD break, the tile
// of its primary entry (tile of the level-0 pixel, clamped into the image; the primary entry also carries the
// coarse levels) and the tile of a second entry when the level-1 pixel belongs to another tile.
__device__ __forceinline__ void entry_tiles(const Levels& lv, const ParamArg& rp, const BinArg& bin, int b, bool ok,
                                            V2 ip, float radius_pixels, bool* in_out, bool* any_in, uint32_t* nlev,
                                            uint32_t* ptile, uint32_t* xtile)
{
    int px[ADOP_MAX_LAYERS], py[ADOP_MAX_LAYERS];
    bool in[ADOP_MAX_LAYERS];
    bool alive = ok;
    *any_in    = false;
    *nlev      = 0;
#pragma unroll
    for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
    {
        px[l] = py[l] = 0;
        in[l]         = false;
        if (l < lv.num)
        {
            if (rp.drop_by_radius && radius_pixels < rp.drop_threshold) alive = false;  // break, :261-264
            if (alive) *nlev = l + 1;
            const LevelArg& L = lv.l[l];
            px[l]             = f2i_rn(ip.x);
            py[l]             = f2i_rn(ip.y);
            in[l] = alive && (unsigned)px[l] < (unsigned)L.w && (unsigned)py[l] < (unsigned)L.h;
            *any_in |= in[l];
            radius_pixels *= 0.5f;
            ip.x *= 0.5f;
            ip.y *= 0.5f;
        }
        if (in_out) in_out[l] = in[l];
    }
    const int tiles_per_view = bin.tiles_x * bin.tiles_y;
    int cx = px[0] < 0 ? 0 : (px[0] >= lv.l[0].w ? lv.l[0].w - 1 : px[0]);
    int cy = py[0] < 0 ? 0 : (py[0] >= lv.l[0].h ? lv.l[0].h - 1 : py[0]);
    *ptile = (uint32_t)(b * tiles_per_view + (cy >> kTileShiftY) * bin.tiles_x + (cx >> kTileShiftX));
    *xtile = kNoTile;
    if (bin.lt > 1 && in[1])
    {
        uint32_t t1 = (uint32_t)(b * tiles_per_view + (py[1] >> (kTileShiftY - 1)) * bin.tiles_x + (px[1] >> (kTileShiftX - 1)));
        if (t1 != *ptile) *xtile = t1;
    }
}

__device__ __forceinline__ uint32_t shard_of(uint32_t point, int shard_shift)
{
    return (point >> 8) & ((1u << shard_shift) - 1u);  // as bin_shard_of(): runs of 256 points take the shards in turn
}

// First pass over the points: projection (kept in the point cache) and the number of entries per tile.  A thread
// handles PPT points whose loads are all issued before anything waits.
template <int PPT>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(PPT > 2 ? 5 : 8, PPT > 2 ? 5 : 8))) void bin_count_kernel(CloudArg pc, const ViewConst* __restrict__ views, Levels lv,
                                                           ParamArg rp, BinArg bin, adop_stats* stats)
{
    const bool STATS = stats != nullptr;  // counter pass (uniform branch)
    const int lane   = threadIdx.x & 63;
    const int base   = blockIdx.x * (kBlock * PPT) + threadIdx.x;

    float4 P[PPT];
    int32_t nenc[PPT];
    bool tex_ok[PPT];
#pragma unroll
    for (int k = 0; k < PPT; ++k)
    {
        const int i      = base + k * kBlock;
        const bool valid = i < pc.n;
        P[k]             = valid ? nt_load4(pc.position + i) : make_float4(0, 0, 0, 0);
        nenc[k]          = (valid && pc.normal) ? __builtin_nontemporal_load(pc.normal + i) : 0;
        tex_ok[k]        = true;
        if (STATS)
        {
            int tex_index = valid ? pc.index[i] : 0;
            tex_ok[k]     = (unsigned)tex_index < (unsigned)pc.num_texels;
        }
    }

    // (the crops of one frame follow each other in a training batch: the point in the uncropped image is kept from
    // one view to the next, only the crop transform and the radius are computed per view)
    V2 frame_p[PPT];
    float frame_z[PPT];
    const ImageBox box = image_box(lv);
    for (int b = 0; b < lv.B; ++b)
    {
        const ViewConst& vc = views[b];
        const bool same_frame = b > 0 && vc.image_index == views[b - 1].image_index &&
                                vc.camera_index == views[b - 1].camera_index && vc.model == views[b - 1].model;  // uniform
#pragma unroll
        for (int k = 0; k < PPT; ++k)
        {
            const int i      = base + k * kBlock;
            const bool valid = i < pc.n;
            V2 ip            = {0.f, 0.f};
            float radius_pixels = 0.f;
            if (!same_frame)
            {
                V3 pos = {P[k].x, P[k].y, P[k].z};
                V3 nrm = unpack_normal10(nenc[k]);
                V3 view_p;
                frame_p[k] = {0.f, 0.f};
                frame_z[k] = 0.f;
                if (valid)
                    project_frame(vc, pc.intrinsics, pos, nrm, rp.check_normal != 0, rp.dist_cutoff, &frame_p[k], &frame_z[k],
                                  &view_p);
            }
            const float z = frame_z[k];
            const bool ok = z != 0;
            if (ok) ip = k_apply(vc.crop, frame_p[k]);
            // The second pass (and the backward pass, if the caller keeps the buffer) read the cache instead of
            // projecting.  A run of 64 points none of which lands in the image at any level is marked in its first
            // record, see kRunCulledBits.  The readers of a batch of views look at that record first and skip the run:
            // its other records are not written at all (views 0..63, no counter pass).
            const bool sparse = lv.B > 1 && b < 64 && !STATS;
            const float4 mark = make_float4(__uint_as_float(kRunCulledBits), 0, 0, 0);
            // a crop sees a small part of the cloud: most runs are nowhere near it (or not projected at all)
            const bool near_image = __ballot(ok && !outside_every_level(box, ip)) != 0;  // wavefront-uniform
            if (!near_image && !STATS)
            {
                if (sparse)
                {
                    // (the second pass sees the mark and reads no tile words of the run)
                    if (valid && lane == 0) nt_store4(pc.cache + (size_t)b * pc.n + i, mark);
                }
                else if (valid)
                {
                    const bool dropped = ok && pc.dropout && __builtin_nontemporal_load(pc.dropout + (size_t)b * pc.n + i) == 1.f;
                    const float4 far   = ok ? make_float4(ip.x, ip.y, signed_depth(z, dropped), rp.drop_by_radius ? crop_radius(vc, z, P[k].w, lv.l[0].w) : 0.f)
                                            : make_float4(0, 0, 0, 0);
                    nt_store4(pc.cache + (size_t)b * pc.n + i, lane == 0 ? mark : far);
                    __builtin_nontemporal_store(0u, bin.info + (size_t)b * pc.n + i);
                }
                continue;
            }
            // (the LOD radius costs a correctly rounded division: computed only when the LOD test reads it)
            if (ok && rp.drop_by_radius) radius_pixels = crop_radius(vc, z, P[k].w, lv.l[0].w);
            // (the sign of the depth carries the dropout flag: the readers need no second array; only the projected
            // points' flags are read)
            const bool dropped = ok && pc.dropout && __builtin_nontemporal_load(pc.dropout + (size_t)b * pc.n + i) == 1.f;  // :314-315
            const float4 rec   = ok ? make_float4(ip.x, ip.y, signed_depth(z, dropped), radius_pixels) : make_float4(0, 0, 0, 0);
            if (STATS) stat_add(&stats->bad_index, ok && !dropped && !tex_ok[k]);

            bool in[ADOP_MAX_LAYERS];
            bool any_in;
            uint32_t nlev, ptile, xtile;
            entry_tiles(lv, rp, bin, b, ok, ip, radius_pixels, in, &any_in, &nlev, &ptile, &xtile);
            if (valid)
            {
                uint32_t word = 0;
                if (any_in)
                {
                    word = kInfoValid | ptile | (nlev << 24);
                    if (xtile != kNoTile)
                    {
                        const uint32_t d = xtile - ptile;  // 1, tiles_x or tiles_x + 1
                        const bool below = d >= (uint32_t)bin.tiles_x;
                        if (below) word |= kInfoBelow;
                        if (d - (below ? (uint32_t)bin.tiles_x : 0u) == 1u) word |= kInfoRight;
                    }
                }
                __builtin_nontemporal_store(word, bin.info + (size_t)b * pc.n + i);
            }
            if (STATS)
            {
#pragma unroll
                for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
                    if (l < lv.num) stat_add(&stats->visible[l], in[l]);
            }
            if (!__ballot(any_in))
            {
                // projected, but all outside the image (a crop): the run counts as culled all the same
                if (valid && (lane == 0 || !sparse)) nt_store4(pc.cache + (size_t)b * pc.n + i, lane == 0 ? mark : rec);
                continue;
            }
            if (valid) nt_store4(pc.cache + (size_t)b * pc.n + i, rec);
            // one atomic per distinct tile of the wavefront, for the primary and for the second entries
            const unsigned long long below = (1ull << lane) - 1ull;
            const unsigned long long pm    = wave_group_mask(any_in, ptile);
            const unsigned long long xm    = wave_group_mask(xtile != kNoTile, xtile);
            const uint32_t shard = shard_of((uint32_t)i, bin.shard_shift);  // (wavefront-uniform)
            if (any_in && (pm & below) == 0) atomicAdd(&bin.count[shard * bin.num_tiles + ptile], (uint32_t)__popcll(pm));
            if (xtile != kNoTile && (xm & below) == 0) atomicAdd(&bin.count[shard * bin.num_tiles + xtile], (uint32_t)__popcll(xm));
        }
    }
}

// The order in which the tile kernels take the tiles: order[i] = (tile, first entry, end, 0), the fullest bins first.
// The bins of a view differ by two orders of magnitude (a surface seen at a grazing angle beside empty sky), a tile is one
// workgroup from its first entry to its last, and the hardware starts workgroups in the order of their index: with the
// tiles in image order a full bin may start late and run on alone (config 3: tile_blend_kernel 129 -> 102 us).
// Computed by the first order_groups(T) workgroups of the bin_scatter launch, beside the scatter (nothing waits for it
// before the tile kernels): workgroup g classes the tiles g, g + G, g + 2G, ... by entries / 128 (classes of equal cost
// in batches of the tile kernels) and puts the r-th of them, fullest class first, at order[g + G * r].  Inside a class the
// order is whatever the LDS atomics make it, which changes no result.
constexpr int kOrderClasses       = 64;
constexpr int kOrderTilesPerGroup = 1024;

static int order_groups(int T) { return T > 0 ? (T + kOrderTilesPerGroup - 1) / kOrderTilesPerGroup : 0; }

__device__ __forceinline__ void order_tiles(const BinArg& bin, int T, int g, int G)
{
    __shared__ uint32_t s_class[kOrderClasses];  // tiles per class, then the next free rank of the class
    static_assert(kOrderClasses == 64, "one wavefront scans the classes");
    const int tid = threadIdx.x;
    if (tid < kOrderClasses) s_class[tid] = 0;
    __syncthreads();
    auto class_of = [](uint32_t entries) -> uint32_t
    {
        const uint32_t c = entries >> 7;
        return (uint32_t)(kOrderClasses - 1) - (c < (uint32_t)(kOrderClasses - 1) ? c : (uint32_t)(kOrderClasses - 1));  // 0 = fullest
    };
    const int sh = bin.shard_shift;  // (a bin: the parts of the tile's shards, one behind the other)
    for (int t = g + G * tid; t < T; t += G * kBlock) atomicAdd(&s_class[class_of(bin.offset[(t + 1) << sh] - bin.offset[t << sh])], 1u);
    __syncthreads();
    if (tid < 64)
    {
        const uint32_t h = s_class[tid];
        uint32_t inc     = h;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1)
        {
            uint32_t u = __shfl_up(inc, off, 64);
            if (tid >= off) inc += u;
        }
        s_class[tid] = inc - h;
    }
    __syncthreads();
    for (int t = g + G * tid; t < T; t += G * kBlock)
    {
        const uint32_t start = bin.offset[t << sh], end = bin.offset[(t + 1) << sh];
        const uint32_t rank  = atomicAdd(&s_class[class_of(end - start)], 1u);
        uint32_t first_end = end, word = 0;
        const uint32_t n   = end - start;
        if (n > (uint32_t)kSplitFrom * bin.slice_entries)
        {
            // a bin too full for one workgroup: K slices (at most 1023, and as many as rows are left)
            uint32_t K = (n + bin.slice_entries - 1) / bin.slice_entries;
            if (K > 1023u) K = 1023u;
            const uint32_t row = atomicAdd(bin.row_count, K);
            if (row >= (uint32_t)bin.max_rows)
                K = 1;
            else if (row + K > (uint32_t)bin.max_rows)
                K = (uint32_t)bin.max_rows - row;
            // (every row below max_rows that was handed out has a workgroup that reads its place of the order)
            if (row < (uint32_t)bin.max_rows && K == 1) bin.order[(size_t)T + row] = make_uint4(0u, 0u, 0u, 0u);
            if (K > 1)
            {
                // slice sl = entries [n * sl / K, n * (sl + 1) / K) of the bin: none is empty (K <= n)
                auto cut = [&](uint32_t sl) { return start + (uint32_t)((unsigned long long)n * sl / K); };
                bin.order[(size_t)T + row] = make_uint4(0u, 0u, 0u, 0u);  // (slice 0 sits in the tile's own place)
                for (uint32_t sl = 1; sl < K; ++sl)
                    bin.order[(size_t)T + row + sl] = make_uint4((uint32_t)t, cut(sl), cut(sl + 1), K | sl << 10 | row << 20);
                first_end = cut(1);
                word      = K | row << 20;
            }
        }
        bin.order[(size_t)g + (size_t)G * rank] = make_uint4((uint32_t)t, start, first_end, word);
    }
}

// Second pass: PPT points per thread, so that the cache loads, the slot reservations (one returning atomic per
// distinct tile of a wavefront, for the primary entries and for the second entries alike) and the entry stores of PPT
// runs of 64 points are in flight together — the kernel is a chain of three dependent memory round trips.
template <int PPT>
__global__ __launch_bounds__(kBlock) void bin_scatter_kernel(CloudArg pc, Levels lv, ParamArg rp, BinArg bin, int T, int G)
{
    if (bin.overflow && *bin.overflow) return;  // more entries than the bins hold: the direct path renders the call
    if ((int)blockIdx.x < G)  // the first G workgroups order the T tiles for the tile kernels
    {
        order_tiles(bin, T, (int)blockIdx.x, G);
        return;
    }
    const int lane = threadIdx.x & 63;
    const int base = ((int)blockIdx.x - G) * (kBlock * PPT) + threadIdx.x;
    const unsigned long long below = (1ull << lane) - 1ull;

    // Several views: the first pass marked the runs of 64 points that miss a view entirely in the first record of the
    // run (kRunCulledBits) and wrote no tile words for them; lane b asks for view b, for all views at once.
    unsigned long long culled_views[PPT];
#pragma unroll
    for (int k = 0; k < PPT; ++k)
    {
        culled_views[k] = 0;
        if (lv.B > 1)  // kernel-uniform
        {
            const int first = (base + k * kBlock) & ~63;
            bool c          = false;
            if (lane < lv.B && first < pc.n)
            {
                const float4 head = pc.cache[(size_t)lane * pc.n + first];
                c                 = __float_as_uint(head.x) == kRunCulledBits && head.z == 0.f;
            }
            culled_views[k] = __ballot(c);
        }
    }

    // (views 0..63 that every run of this wavefront missed are jumped over: the loop is scalar control flow, and a crop
    // sees a small part of the cloud)
    unsigned long long all_culled = ~0ull;
#pragma unroll
    for (int k = 0; k < PPT; ++k) all_culled &= culled_views[k];
    for (int b = 0; b < lv.B; ++b)
    {
        if (b < 64)
        {
            const unsigned long long rest = ~all_culled >> b;  // (wavefront-uniform)
            if (rest == 0)
            {
                b = 63;  // the views from 64 on carry no marks
                continue;
            }
            b += __builtin_ctzll(rest);
            if (b >= lv.B) break;
        }
        uint32_t info[PPT];
        bool any = false;
#pragma unroll
        for (int k = 0; k < PPT; ++k)
        {
            const int i       = base + k * kBlock;
            const bool culled = b < 64 && (culled_views[k] >> b & 1ull) != 0;  // wavefront-uniform
            info[k]           = (i < pc.n && !culled) ? __builtin_nontemporal_load(bin.info + (size_t)b * pc.n + i) : 0u;
            any |= !culled;
        }
        if (!any) continue;  // wavefront-uniform
        float4 R[PPT];
#pragma unroll
        for (int k = 0; k < PPT; ++k)
        {
            const int i = base + k * kBlock;
            R[k]        = make_float4(0, 0, 0, 0);
            if (info[k] & kInfoValid) R[k] = nt_load4(pc.cache + (size_t)b * pc.n + i);
        }
        // groups of equal tile inside the wavefront: the lowest lane of a group reserves the slots of all its lanes
        // (slots are handed out from the end of the bin: the tile's counter runs down from its count to zero)
        unsigned long long pm[PPT], xm[PPT];
        uint32_t pbase[PPT], xbase[PPT];
#pragma unroll
        for (int k = 0; k < PPT; ++k)
        {
            const bool any_in    = (info[k] & kInfoValid) != 0;
            const uint32_t ptile = info[k] & kInfoTileMask;
            const bool has_x     = (info[k] & (kInfoRight | kInfoBelow)) != 0;
            const uint32_t xtile = ptile + ((info[k] & kInfoRight) ? 1u : 0u) + ((info[k] & kInfoBelow) ? (uint32_t)bin.tiles_x : 0u);
            pm[k]                = wave_group_mask(any_in, ptile);
            xm[k]                = wave_group_mask(has_x, xtile);
            pbase[k] = xbase[k] = 0;
            if (any_in && (pm[k] & below) == 0)
            {
                const uint32_t n = (uint32_t)__popcll(pm[k]);
                const uint32_t sd = shard_of((uint32_t)(base + k * kBlock), bin.shard_shift);
                pbase[k] = bin.offset[(ptile << bin.shard_shift) + sd] + atomicSub(&bin.count[sd * bin.num_tiles + ptile], n) - n;
            }
            if (has_x && (xm[k] & below) == 0)
            {
                const uint32_t n = (uint32_t)__popcll(xm[k]);
                const uint32_t sd = shard_of((uint32_t)(base + k * kBlock), bin.shard_shift);
                xbase[k] = bin.offset[(xtile << bin.shard_shift) + sd] + atomicSub(&bin.count[sd * bin.num_tiles + xtile], n) - n;
            }
        }
#pragma unroll
        for (int k = 0; k < PPT; ++k)
        {
            const int i         = base + k * kBlock;
            const float zs      = R[k].z;  // the sign carries the dropout flag (:314-315)
            const uint32_t word = (uint32_t)i | ((info[k] >> 24 & 7u) << 28);
            // every lane asks its group's leader for the base (inactive lanes ask lane 0 for nothing)
            const int pl      = pm[k] ? __ffsll((long long)pm[k]) - 1 : 0;
            const int xl      = xm[k] ? __ffsll((long long)xm[k]) - 1 : 0;
            const uint32_t pb = (uint32_t)__shfl((int)pbase[k], pl, 64);
            const uint32_t xb = (uint32_t)__shfl((int)xbase[k], xl, 64);
            if (pm[k])
                bin.entries[pb + (uint32_t)__popcll(pm[k] & below)] =
                    make_float4(R[k].x, R[k].y, zs, __uint_as_float(word | kEntryPrimary));
            if (xm[k])
                bin.entries[xb + (uint32_t)__popcll(xm[k] & below)] = make_float4(R[k].x, R[k].y, zs, __uint_as_float(word));
        }
    }
}

// Exclusive prefix sum of the tile counts (one workgroup): offset[0..T].  Chunks of 1024 * PER tiles; the PER counts of
// a thread are consecutive (16-byte loads, one memory round trip per chunk).  PER = 8 covers one view of 1920 x 1080 in
// one chunk; batches of views take PER = 32 (a chunk costs three barriers and a round trip whatever its size).
// The counters lie shard by shard (count[shard * tiles + tile]), the offsets tile by tile with a tile's shards side by
// side (k = (tile << shard_shift) + shard): T = tiles << shard_shift logical counters.
template <int PER>
__global__ __launch_bounds__(1024) void tile_scan_kernel(const uint32_t* __restrict__ count, uint32_t* __restrict__ offset,
                                                         int T, int shard_shift, int tiles, uint32_t* __restrict__ overflow,
                                                         uint32_t cap)
{
    __shared__ uint32_t s_wave[16];
    __shared__ uint32_t s_carry;
    const int tid = threadIdx.x;
    if (tid == 0) s_carry = 0;
    __syncthreads();
    for (int c0 = 0; c0 < T; c0 += 1024 * PER)
    {
        const int t0 = c0 + tid * PER;
        uint32_t v[PER];
        if (shard_shift > 0)
        {
            // (unconditional loads of clamped indices, all in flight at once; what lies past the end counts as zero)
#pragma unroll
            for (int k = 0; k < PER; ++k)
            {
                const int q = min(t0 + k, T - 1);
                v[k]        = __builtin_nontemporal_load(count + (q & ((1 << shard_shift) - 1)) * tiles + (q >> shard_shift));
            }
#pragma unroll
            for (int k = 0; k < PER; ++k)
                if (t0 + k >= T) v[k] = 0u;
        }
        else if (t0 + PER <= T)  // (count is 256-byte aligned and t0 a multiple of PER)
        {
#pragma unroll
            for (int k = 0; k < PER; k += 4)
            {
                const uint4 q = *(const uint4*)(count + t0 + k);
                v[k] = q.x, v[k + 1] = q.y, v[k + 2] = q.z, v[k + 3] = q.w;
            }
        }
        else
        {
#pragma unroll
            for (int k = 0; k < PER; ++k) v[k] = t0 + k < T ? count[t0 + k] : 0u;
        }
        uint32_t sum = 0;
#pragma unroll
        for (int k = 0; k < PER; ++k) sum += v[k];
        // inclusive scan inside the wavefront, then over the 16 wavefronts
        uint32_t inc = sum;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1)
        {
            uint32_t u = __shfl_up(inc, off, 64);
            if ((tid & 63) >= off) inc += u;
        }
        if ((tid & 63) == 63) s_wave[tid >> 6] = inc;
        __syncthreads();
        uint32_t run = s_carry + inc - sum;
        for (int w = 0; w < (tid >> 6); ++w) run += s_wave[w];
        // (offset is 256-byte aligned and t0 a multiple of PER: 16-byte stores, a quarter of the store instructions)
#pragma unroll
        for (int k = 0; k < PER; k += 4)
        {
            uint4 o;
            o.x = run, run += v[k];
            o.y = run, run += v[k + 1];
            o.z = run, run += v[k + 2];
            o.w = run, run += v[k + 3];
            if (t0 + k + 3 < T)
                *(uint4*)(offset + t0 + k) = o;
            else
            {
                if (t0 + k < T) offset[t0 + k] = o.x;
                if (t0 + k + 1 < T) offset[t0 + k + 1] = o.y;
                if (t0 + k + 2 < T) offset[t0 + k + 2] = o.z;
            }
        }
        __syncthreads();
        if (tid == 1023) s_carry = run;  // the last thread ends at the chunk total
        __syncthreads();
    }
    if (tid == 0)
    {
        offset[T] = s_carry;
        if (overflow) *overflow = s_carry > cap ? 1u : 0u;  // (the bins of this workspace hold `cap` entries)
    }
}

// ------------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------------
void launch_bin(int pass, const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp,
                const BinArg& bin, adop_stats* stats, const adop_tuning& tn, hipStream_t st)
{
    if (pc.n < 1) return;
    if (pass == 0)
    {
        // (one point per thread while the grid is small: twice the workgroups in flight; config 2 0.038 -> 0.033 ms,
        // 10 M points 0.079 against 0.082 ms the other way round)
        const int cppt = tn.count_ppt ? tn.count_ppt : (pc.n <= (1 << 22) ? 1 : 2);
        if (cppt == 2)
            hipLaunchKernelGGL((bin_count_kernel<2>), dim3((pc.n + kBlock * 2 - 1) / (kBlock * 2)), dim3(kBlock), 0, st,
                               pc, views, lv, rp, bin, stats);
        else if (cppt == 4)
            hipLaunchKernelGGL((bin_count_kernel<4>), dim3((pc.n + kBlock * 4 - 1) / (kBlock * 4)), dim3(kBlock), 0, st,
                               pc, views, lv, rp, bin, stats);
        else
            hipLaunchKernelGGL((bin_count_kernel<1>), dim3((pc.n + kBlock - 1) / kBlock), dim3(kBlock), 0, st, pc, views,
                               lv, rp, bin, stats);
        return;
    }
    const int T = bin.tiles_x * bin.tiles_y * lv.B;
    const int G = order_groups(T);
    const int ppt = tn.scatter_ppt;
    if (ppt == 1)
        hipLaunchKernelGGL((bin_scatter_kernel<1>), dim3(G + (pc.n + kBlock - 1) / kBlock), dim3(kBlock), 0, st, pc, lv, rp, bin, T, G);
    else if (ppt == 2)
        hipLaunchKernelGGL((bin_scatter_kernel<2>), dim3(G + (pc.n + kBlock * 2 - 1) / (kBlock * 2)), dim3(kBlock), 0, st, pc,
                           lv, rp, bin, T, G);
    else
        hipLaunchKernelGGL((bin_scatter_kernel<4>), dim3(G + (pc.n + kBlock * 4 - 1) / (kBlock * 4)), dim3(kBlock), 0, st, pc,
                           lv, rp, bin, T, G);
}

void launch_tile_scan(const BinArg& bin, int num_tiles, hipStream_t st)
{
    if (num_tiles <= 8192)
        hipLaunchKernelGGL(tile_scan_kernel<8>, dim3(1), dim3(1024), 0, st, bin.count, bin.offset, num_tiles, bin.shard_shift, bin.num_tiles, bin.overflow, bin.cap);
    else if (num_tiles <= 16384)  // (the sharded counters of a call: one chunk)
        hipLaunchKernelGGL(tile_scan_kernel<16>, dim3(1), dim3(1024), 0, st, bin.count, bin.offset, num_tiles, bin.shard_shift, bin.num_tiles, bin.overflow, bin.cap);
    else
        hipLaunchKernelGGL(tile_scan_kernel<32>, dim3(1), dim3(1024), 0, st, bin.count, bin.offset, num_tiles, bin.shard_shift, bin.num_tiles, bin.overflow, bin.cap);
}

}  // namespace adop
