// preprocess_kernels.hip — point-cloud preprocessing that decides how well the rasterizer runs (gfx950):
// the distance of every point to its n-th nearest neighbour (SceneData::ComputeRadius, SceneData.cpp:441-484: a
// kd-tree k-nearest-neighbour search per point on the host) and the Morton code of every point (the key of
// ReorderMorton64, SceneData.cpp:101).
//
// Nearest neighbours: the points are binned into a uniform grid (count, prefix sum, scatter: the structure of the
// rasterizer's tile bins), stored cell after cell, and every point then walks the shells of cells around its own
// until the n-th best distance cannot be beaten from outside the cube searched so far.  The distances are formed as
// sqrt((dx*dx + dy*dy) + dz*dz) in fp32; the result is the n-th smallest of them over all other points, whatever the
// search order and whatever the grid, so a brute-force search over the same arithmetic gives the same bits.
// The cost is the number of candidates, which the cell size decides, and the right cell size depends on how the cloud
// fills space (scans are surfaces: a grid sized by volume puts hundreds of points into the few cells that have any).
// So there are two grids, both sized on the device (no host round trip): a first one sized by volume, on which 2048
// sample points are searched, and a second one with cells of twice the median distance those found.  All points are
// searched on the second grid (2 shells at most), what that leaves on the first (4 shells), and the stray points
// neither settles against all points.
#include "common.h"
#include "launch.h"

#pragma clang fp contract(off)

namespace adop
{
// Cell of a point; points outside the grid's box (the box leaves the far tails of the cloud out) belong to the nearest
// boundary cell.
__device__ __forceinline__ int3 grid_cell(const KnnGrid& g, float x, float y, float z)
{
    const float fx = fminf(fmaxf((x - g.min[0]) * g.inv_cell, 0.f), (float)(g.dim[0] - 1));
    const float fy = fminf(fmaxf((y - g.min[1]) * g.inv_cell, 0.f), (float)(g.dim[1] - 1));
    const float fz = fminf(fmaxf((z - g.min[2]) * g.inv_cell, 0.f), (float)(g.dim[2] - 1));
    return make_int3((int)fx, (int)fy, (int)fz);
}

__device__ __forceinline__ uint32_t grid_index(const KnnGrid& g, int cx, int cy, int cz)
{
    return ((uint32_t)cz * (uint32_t)g.dim[1] + (uint32_t)cy) * (uint32_t)g.dim[0] + (uint32_t)cx;
}

// pass 0: points per cell; pass 1: the points cell after cell, (x, y, z, bits of the point id)
__global__ __launch_bounds__(kBlock) void knn_bin_kernel(int pass, const float4* __restrict__ position, int n,
                                                         const KnnGrid* __restrict__ gp, uint32_t* __restrict__ count,
                                                         const uint32_t* __restrict__ offset, float4* __restrict__ sorted)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const KnnGrid g = *gp;
    const float4 p    = nt_load4(position + i);
    const int3 c      = grid_cell(g, p.x, p.y, p.z);
    const uint32_t ci = grid_index(g, c.x, c.y, c.z);
    if (pass == 0)
        atomicAdd(&count[ci], 1u);
    else  // the counter runs down to zero: slots are handed out from the end of the cell's range
        sorted[offset[ci] + atomicSub(&count[ci], 1u) - 1u] = make_float4(p.x, p.y, p.z, __uint_as_float((uint32_t)i));
}

// The search of one point by one thread: the cube of cells around the point's cell grows until the K-th best distance
// cannot be beaten from outside it; a row of cells along x is one contiguous run of the cell-ordered array, so a cube
// of (2r+1)^3 cells is (2r+1)^2 runs.  A larger cube is searched from scratch (the first cube, r = 1, settles nearly
// every point).  Gives up after rmax shells: false, and the caller hands the point to the next, coarser stage.
template <int K>  // K = n + 1 best squared distances are kept (the point itself is one of them)
__device__ __forceinline__ bool knn_cubes(const float4 p, const KnnGrid& g, const float4* __restrict__ sorted,
                                          const uint32_t* __restrict__ offset, int rmax, float* kth)
{
    const int3 c = grid_cell(g, p.x, p.y, p.z);
    float best[K];
    for (int r = 1; r <= rmax; ++r)
    {
#pragma unroll
        for (int k = 0; k < K; ++k) best[k] = 3.0e38f;
        const int z0 = max(c.z - r, 0), z1 = min(c.z + r, g.dim[2] - 1);
        const int y0 = max(c.y - r, 0), y1 = min(c.y + r, g.dim[1] - 1);
        const int x0 = max(c.x - r, 0), x1 = min(c.x + r, g.dim[0] - 1);
        for (int cz = z0; cz <= z1; ++cz)
            for (int cy = y0; cy <= y1; ++cy)
            {
                const uint32_t row = grid_index(g, 0, cy, cz);
                const uint32_t e   = offset[row + x1 + 1];
                for (uint32_t q = offset[row + x0]; q < e; ++q)
                {
                    const float4 o = sorted[q];
                    const float dx = p.x - o.x, dy = p.y - o.y, dz = p.z - o.z;
                    float d2 = (dx * dx + dy * dy) + dz * dz;
                    if (d2 < best[K - 1])
                    {
#pragma unroll
                        for (int k = 0; k < K; ++k)  // insertion into the ascending list
                        {
                            const float b = best[k];
                            const bool lt = d2 < b;
                            best[k]       = lt ? d2 : b;
                            d2            = lt ? b : d2;
                        }
                    }
                }
            }
        // Nothing outside the cube is closer than the nearest face of the cube that has cells behind it (slightly
        // shrunk: the cell of a point and the faces are computed in fp32).  No such face: the cube is the whole grid.
        float bound = 3.0e38f;
        if (c.x - r > 0) bound = fminf(bound, p.x - (g.min[0] + (float)(c.x - r) * g.cell));
        if (c.y - r > 0) bound = fminf(bound, p.y - (g.min[1] + (float)(c.y - r) * g.cell));
        if (c.z - r > 0) bound = fminf(bound, p.z - (g.min[2] + (float)(c.z - r) * g.cell));
        if (c.x + r < g.dim[0] - 1) bound = fminf(bound, (g.min[0] + (float)(c.x + r + 1) * g.cell) - p.x);
        if (c.y + r < g.dim[1] - 1) bound = fminf(bound, (g.min[1] + (float)(c.y + r + 1) * g.cell) - p.y);
        if (c.z + r < g.dim[2] - 1) bound = fminf(bound, (g.min[2] + (float)(c.z + r + 1) * g.cell) - p.z);
        bound = fmaxf(bound, 0.f) * 0.999f;
        if (bound >= 1.0e38f || best[K - 1] <= bound * bound)
        {
            *kth = best[K - 1];
            return true;
        }
    }
    return false;
}

// Appends `value` of the lanes with `push` to a list (one atomic per wavefront).  Called by all lanes of a wavefront.
__device__ __forceinline__ void wave_push(bool push, uint32_t value, uint32_t* __restrict__ list, uint32_t* count)
{
    const unsigned long long m = __ballot(push);
    if (!m) return;
    const int lane   = threadIdx.x & 63;
    const int leader = __ffsll((long long)m) - 1;
    uint32_t base    = 0;
    if (lane == leader) base = atomicAdd(count, (uint32_t)__popcll(m));
    base = (uint32_t)__shfl((int)base, leader, 64);
    if (push) list[base + (uint32_t)__popcll(m & ((1ull << lane) - 1ull))] = value;
}

// Stage 1: every point, one thread each in cell order of the second grid (the lanes of a wavefront search nearly the
// same cells), at most 2 shells; what is left (points in sparse parts of the cloud) goes to list.
template <int K>
__global__ __launch_bounds__(kBlock) void knn_search_kernel(const float4* __restrict__ sorted, int n,
                                                            const KnnGrid* __restrict__ gp,
                                                            const uint32_t* __restrict__ offset, float* __restrict__ out,
                                                            uint32_t* __restrict__ list, uint32_t* list_count)
{
    const int t = blockIdx.x * kBlock + threadIdx.x;
    bool left   = false;
    if (t < n)
    {
        const KnnGrid g = *gp;
        const float4 p  = sorted[t];
        float kth;
        if (knn_cubes<K>(p, g, sorted, offset, 2, &kth))
            out[__float_as_uint(p.w)] = sqrtf(kth);
        else
            left = true;
    }
    wave_push(left, (uint32_t)t, list, list_count);
}

// Stage 2: the points stage 1 left, on the first (coarser) grid, at most 4 shells; the rest goes to list2.
template <int K>
__global__ __launch_bounds__(kBlock) void knn_list_kernel(const float4* __restrict__ points,
                                                          const uint32_t* __restrict__ list,
                                                          const uint32_t* __restrict__ list_count,
                                                          const float4* __restrict__ sorted0,
                                                          const KnnGrid* __restrict__ gp0,
                                                          const uint32_t* __restrict__ offset0, float* __restrict__ out,
                                                          uint32_t* __restrict__ list2, uint32_t* list2_count)
{
    const uint32_t count = *list_count;
    const KnnGrid g      = *gp0;
    const uint32_t lane  = threadIdx.x & 63;
    for (uint32_t e0 = blockIdx.x * kBlock + (threadIdx.x & ~63u); e0 < count; e0 += gridDim.x * kBlock)  // wavefront-uniform
    {
        const uint32_t e = e0 + lane;
        bool left        = false;
        uint32_t t       = 0;
        if (e < count)
        {
            t              = list[e];
            const float4 p = points[t];
            float kth;
            if (knn_cubes<K>(p, g, sorted0, offset0, 4, &kth))
                out[__float_as_uint(p.w)] = sqrtf(kth);
            else
                left = true;
        }
        wave_push(left, t, list2, list2_count);
    }
}

// K-th smallest of the union of the lanes' ascending lists (destroys them): K rounds of taking the smallest head.
template <int K>
__device__ __forceinline__ float wave_kth(float* best)
{
    const int lane = threadIdx.x & 63;
    float kth      = 3.0e38f;
#pragma unroll
    for (int k = 0; k < K; ++k)
    {
        float m = best[0];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) m = fminf(m, __shfl_xor(m, off, 64));
        kth = m;
        const unsigned long long holders = __ballot(best[0] == m);
        if (lane == __ffsll((long long)holders) - 1)
        {
#pragma unroll
            for (int j = 0; j + 1 < K; ++j) best[j] = best[j + 1];
            best[K - 1] = 3.0e38f;
        }
    }
    return kth;
}

// Stage 3: stray points far from everything (no cube of a few shells of either grid settles them): one wavefront
// per point goes through all points.
template <int K>
__global__ __launch_bounds__(kBlock) void knn_brute_kernel(const float4* __restrict__ points, int n,
                                                           const uint32_t* __restrict__ list,
                                                           const uint32_t* __restrict__ list_count,
                                                           float* __restrict__ out)
{
    const uint32_t count = *list_count;
    const int lane       = threadIdx.x & 63;
    for (uint32_t e = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6); e < count; e += gridDim.x * (kBlock / 64))
    {
        const float4 p = points[list[e]];
        float best[K];
#pragma unroll
        for (int k = 0; k < K; ++k) best[k] = 3.0e38f;
        for (int q = lane; q < n; q += 64)
        {
            const float4 o = points[q];
            const float dx = p.x - o.x, dy = p.y - o.y, dz = p.z - o.z;
            float d2 = (dx * dx + dy * dy) + dz * dz;
            if (d2 < best[K - 1])
            {
#pragma unroll
                for (int k = 0; k < K; ++k)
                {
                    const float b = best[k];
                    const bool lt = d2 < b;
                    best[k]       = lt ? d2 : b;
                    d2            = lt ? b : d2;
                }
            }
        }
        const float kth = wave_kth<K>(best);
        if (lane == 0) out[__float_as_uint(p.w)] = sqrtf(kth);
    }
}

// The search of stage 1 for `samples` points evenly spaced in cell order, one wavefront per point (on the first grid a
// point has thousands of candidates: the lanes share them, every lane keeps the K best of its share).  out[s] =
// distance of sample s, 3e38 for a sample that 4 shells do not settle (a stray point: it shall not size the grid).
// All branches on r, the bound and the result are uniform over the wavefront.
template <int K>
__global__ __launch_bounds__(kBlock) void knn_sample_kernel(const float4* __restrict__ sorted, int n,
                                                            const KnnGrid* __restrict__ gp,
                                                            const uint32_t* __restrict__ offset, float* __restrict__ out,
                                                            int samples)
{
    const int slot = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (slot >= samples) return;
    const int t     = (int)((long long)slot * n / samples);
    const KnnGrid g = *gp;
    const float4 p  = sorted[t];
    const int3 c    = grid_cell(g, p.x, p.y, p.z);
    float result    = 3.0e38f;
    for (int r = 1; r <= 4; ++r)
    {
        float best[K];
#pragma unroll
        for (int k = 0; k < K; ++k) best[k] = 3.0e38f;
        const int z0 = max(c.z - r, 0), z1 = min(c.z + r, g.dim[2] - 1);
        const int y0 = max(c.y - r, 0), y1 = min(c.y + r, g.dim[1] - 1);
        const int x0 = max(c.x - r, 0), x1 = min(c.x + r, g.dim[0] - 1);
        for (int cz = z0; cz <= z1; ++cz)
            for (int cy = y0; cy <= y1; ++cy)
            {
                const uint32_t row = grid_index(g, 0, cy, cz);
                const uint32_t e   = offset[row + x1 + 1];
                for (uint32_t q = offset[row + x0] + lane; q < e; q += 64)
                {
                    const float4 o = sorted[q];
                    const float dx = p.x - o.x, dy = p.y - o.y, dz = p.z - o.z;
                    float d2 = (dx * dx + dy * dy) + dz * dz;
                    if (d2 < best[K - 1])
                    {
#pragma unroll
                        for (int k = 0; k < K; ++k)
                        {
                            const float b = best[k];
                            const bool lt = d2 < b;
                            best[k]       = lt ? d2 : b;
                            d2            = lt ? b : d2;
                        }
                    }
                }
            }
        const float kth = wave_kth<K>(best);
        float bound = 3.0e38f;
        if (c.x - r > 0) bound = fminf(bound, p.x - (g.min[0] + (float)(c.x - r) * g.cell));
        if (c.y - r > 0) bound = fminf(bound, p.y - (g.min[1] + (float)(c.y - r) * g.cell));
        if (c.z - r > 0) bound = fminf(bound, p.z - (g.min[2] + (float)(c.z - r) * g.cell));
        if (c.x + r < g.dim[0] - 1) bound = fminf(bound, (g.min[0] + (float)(c.x + r + 1) * g.cell) - p.x);
        if (c.y + r < g.dim[1] - 1) bound = fminf(bound, (g.min[1] + (float)(c.y + r + 1) * g.cell) - p.y);
        if (c.z + r < g.dim[2] - 1) bound = fminf(bound, (g.min[2] + (float)(c.z + r + 1) * g.cell) - p.z);
        bound = fmaxf(bound, 0.f) * 0.999f;
        if (bound >= 1.0e38f || kth <= bound * bound)
        {
            result = sqrtf(kth);
            break;
        }
    }
    if (lane == 0) out[slot] = result;
}

constexpr int kKnnSamples   = 2048;
constexpr int kKnnMaxDim    = 2048;
constexpr int kKnnCoarseDim = 160;

// ascending bitonic sort of kKnnSamples floats in LDS by a workgroup of 1024 threads
__device__ __forceinline__ void sort_samples(float* s)
{
    for (int k = 2; k <= kKnnSamples; k <<= 1)
        for (int j = k >> 1; j > 0; j >>= 1)
        {
            for (int i = threadIdx.x; i < kKnnSamples; i += 1024)
            {
                const int o = i ^ j;
                if (o > i)
                {
                    const float a = s[i], b = s[o];
                    const bool up = (i & k) == 0;
                    if ((a > b) == up)
                    {
                        s[i] = b;
                        s[o] = a;
                    }
                }
            }
            __syncthreads();
        }
}

// First grid.  Its box is not the bounding box of the cloud (one far outlier would stretch that until all other points
// share a cell) but, per axis, the 1st to 99th percentile of 2048 points taken at equal steps through the array,
// widened by 5 % of that range on either side and cut to the caller's box; the points outside it go to the boundary
// cells, which keeps the search exact (a cube of cells then stands for a region open to the outside).  Cells for ~8
// points each if the cloud filled the box, at most kKnnCoarseDim per axis.  One workgroup.
__global__ __launch_bounds__(1024) void knn_first_grid_kernel(const float4* __restrict__ position, int n, KnnGrid box,
                                                              KnnGrid* __restrict__ dst)
{
    __shared__ float s[kKnnSamples];
    const int samples = n < kKnnSamples ? n : kKnnSamples;
    float lo[3], hi[3];
#pragma unroll
    for (int axis = 0; axis < 3; ++axis)
    {
        for (int i = threadIdx.x; i < kKnnSamples; i += 1024)
        {
            float v = 3.0e38f;
            if (i < samples)
            {
                const float4 p = position[(size_t)((long long)i * n / samples)];
                v              = axis == 0 ? p.x : (axis == 1 ? p.y : p.z);
            }
            s[i] = v;
        }
        __syncthreads();
        sort_samples(s);
        const float a = s[samples / 100], b = s[samples - 1 - samples / 100];
        const float box_hi = box.min[axis] + box.ext[axis];
        lo[axis] = fmaxf(a - 0.05f * (b - a), box.min[axis]);
        hi[axis] = fminf(b + 0.05f * (b - a), box_hi);
        if (!(hi[axis] >= lo[axis]))  // not a number among the samples
        {
            lo[axis] = box.min[axis];
            hi[axis] = box_hi;
        }
        __syncthreads();
    }
    if (threadIdx.x != 0) return;
    KnnGrid g;
    for (int k = 0; k < 3; ++k)
    {
        g.min[k] = lo[k];
        g.ext[k] = hi[k] - lo[k];
    }
    const float longest = fmaxf(g.ext[0], fmaxf(g.ext[1], g.ext[2]));
    float volume        = 1.f;  // thin axes count as a millionth of the longest one
    for (int k = 0; k < 3; ++k) volume *= g.ext[k] > 1e-6f * longest ? g.ext[k] : (longest > 0.f ? 1e-6f * longest : 1.f);
    float cell = cbrtf(volume * 8.0f / (float)n);
    if (!(cell > longest / kKnnCoarseDim)) cell = longest / kKnnCoarseDim;
    if (!(cell > 0.f)) cell = 1.f;  // all samples coincide
    g.cell     = cell;
    g.inv_cell = 1.0f / cell;
    g.cells    = 1;
    for (int k = 0; k < 3; ++k)
    {
        int d    = (int)(g.ext[k] / cell) + 1;
        g.dim[k] = d < 1 ? 1 : (d > kKnnCoarseDim ? kKnnCoarseDim : d);
        g.cells *= (uint32_t)g.dim[k];
    }
    *dst = g;
}

// Second grid: cells of twice the median sampled neighbour distance (a cube of 3 cells then settles every point whose
// own distance is below twice the median, with ~60 candidates on a surface, ~260 in a volume), never coarser than the
// first grid, at most kKnnMaxDim cells per axis and `budget` cells in all, over the same box.  One workgroup.
__global__ __launch_bounds__(1024) void knn_refine_grid_kernel(const float* __restrict__ sample, int samples,
                                                               const KnnGrid* __restrict__ first,
                                                               KnnGrid* __restrict__ gp, uint32_t budget)
{
    __shared__ float s[kKnnSamples];
    for (int i = threadIdx.x; i < kKnnSamples; i += 1024) s[i] = i < samples ? sample[i] : 3.0e38f;
    __syncthreads();
    sort_samples(s);
    if (threadIdx.x != 0) return;
    KnnGrid g          = *first;
    const float median = s[samples / 2];
    const float longest = fmaxf(g.ext[0], fmaxf(g.ext[1], g.ext[2]));
    float cell = 2.0f * median;
    if (!(cell < g.cell)) cell = g.cell;  // also NaN / the 3e38 of a cloud with fewer points than neighbours asked for
    if (!(cell > longest / (float)(kKnnMaxDim - 1))) cell = longest / (float)(kKnnMaxDim - 1);
    if (!(cell > 0.f)) cell = g.cell;
    for (;;)
    {
        unsigned long long cells = 1;
        for (int k = 0; k < 3; ++k)
        {
            int d    = (int)(g.ext[k] / cell) + 1;
            g.dim[k] = d < 1 ? 1 : (d > kKnnMaxDim ? kKnnMaxDim : d);
            cells *= (unsigned long long)g.dim[k];
        }
        if (cells <= budget)
        {
            g.cells = (uint32_t)cells;
            break;
        }
        cell *= 1.26f;
    }
    g.cell     = cell;
    g.inv_cell = 1.0f / cell;
    *gp        = g;
}

// Zeroes the cell counters of the grid.
__global__ __launch_bounds__(kBlock) void knn_clear_kernel(uint32_t* __restrict__ count, const KnnGrid* __restrict__ gp)
{
    const uint32_t cells = gp->cells;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < cells; i += (size_t)gridDim.x * kBlock)
        __builtin_nontemporal_store(0u, count + i);
}

// Exclusive prefix sum over the cell counters (offset[0..cells]) in three launches: sums of chunks of 8192 cells,
// their prefix sum (one workgroup: at most 16384 chunks), the prefix sum inside every chunk.
constexpr int kScanChunk = 8192;

__device__ __forceinline__ uint32_t block_exclusive_scan_1024(uint32_t sum, uint32_t* s_wave, uint32_t* total)
{
    const int tid = threadIdx.x;
    uint32_t inc  = sum;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1)
    {
        const uint32_t u = __shfl_up(inc, off, 64);
        if ((tid & 63) >= off) inc += u;
    }
    __syncthreads();  // s_wave of the last call has been read
    if ((tid & 63) == 63) s_wave[tid >> 6] = inc;
    __syncthreads();
    uint32_t run = inc - sum, all = 0;
    for (int w = 0; w < 16; ++w)
    {
        if (w < (tid >> 6)) run += s_wave[w];
        all += s_wave[w];
    }
    *total = all;
    return run;
}

__global__ __launch_bounds__(1024) void knn_scan_reduce_kernel(const uint32_t* __restrict__ count,
                                                               const KnnGrid* __restrict__ gp,
                                                               uint32_t* __restrict__ chunk_sum)
{
    __shared__ uint32_t s_wave[16];
    const uint32_t cells = gp->cells;
    const uint32_t nb    = (cells + kScanChunk - 1) / kScanChunk;
    for (uint32_t b = blockIdx.x; b < nb; b += gridDim.x)
    {
        const size_t t0 = (size_t)b * kScanChunk + (size_t)threadIdx.x * 8;
        uint32_t sum    = 0;
        if (t0 + 8 <= cells)
        {
            const uint4 a = ((const uint4*)(count + t0))[0], c = ((const uint4*)(count + t0))[1];
            sum = a.x + a.y + a.z + a.w + c.x + c.y + c.z + c.w;
        }
        else
            for (int k = 0; k < 8; ++k) sum += t0 + k < cells ? count[t0 + k] : 0u;
        uint32_t total;
        block_exclusive_scan_1024(sum, s_wave, &total);
        if (threadIdx.x == 0) chunk_sum[b] = total;
    }
}

__global__ __launch_bounds__(1024) void knn_scan_chunks_kernel(const uint32_t* __restrict__ chunk_sum,
                                                               const KnnGrid* __restrict__ gp,
                                                               uint32_t* __restrict__ chunk_offset)
{
    __shared__ uint32_t s_wave[16];
    const uint32_t nb = (gp->cells + kScanChunk - 1) / kScanChunk;
    uint32_t carry    = 0;
    for (uint32_t c0 = 0; c0 < nb; c0 += 1024)
    {
        const uint32_t i = c0 + threadIdx.x;
        const uint32_t v = i < nb ? chunk_sum[i] : 0u;
        uint32_t total;
        const uint32_t run = block_exclusive_scan_1024(v, s_wave, &total);
        if (i < nb) chunk_offset[i] = carry + run;
        carry += total;
    }
    if (threadIdx.x == 0) chunk_offset[nb] = carry;
}

__global__ __launch_bounds__(1024) void knn_scan_apply_kernel(const uint32_t* __restrict__ count,
                                                              const KnnGrid* __restrict__ gp,
                                                              const uint32_t* __restrict__ chunk_offset,
                                                              uint32_t* __restrict__ offset)
{
    __shared__ uint32_t s_wave[16];
    const uint32_t cells = gp->cells;
    const uint32_t nb    = (cells + kScanChunk - 1) / kScanChunk;
    for (uint32_t b = blockIdx.x; b < nb; b += gridDim.x)
    {
        const size_t t0 = (size_t)b * kScanChunk + (size_t)threadIdx.x * 8;
        uint32_t v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = t0 + k < cells ? count[t0 + k] : 0u;
        uint32_t sum = 0;
#pragma unroll
        for (int k = 0; k < 8; ++k) sum += v[k];
        uint32_t total;
        uint32_t run = chunk_offset[b] + block_exclusive_scan_1024(sum, s_wave, &total);
#pragma unroll
        for (int k = 0; k < 8; ++k)
            if (t0 + k < cells)
            {
                offset[t0 + k] = run;
                run += v[k];
            }
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) offset[cells] = chunk_offset[nb];
}

// SceneData::PointDistanceToCamera (SceneData.cpp:645-669): distance from every point to the nearest camera that sees
// it (in front of the camera, projected inside the image with the frame's pinhole + distortion model), 10258.4 (the
// root of the reference's start value 105235545) where no frame does.  The distance is taken in camera space
// (|V p| = |p - c| for the camera centre c).  The frames are read through uniform loads.
__global__ __launch_bounds__(kBlock) void camera_distance_kernel(const float4* __restrict__ position, int n,
                                                                 const ViewConst* __restrict__ views, int num_frames,
                                                                 float* __restrict__ out)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const float4 P = nt_load4(position + i);
    const V3 pos   = {P.x, P.y, P.z};
    float best     = 105235545.f;
    for (int f = 0; f < num_frames; ++f)
    {
        const ViewConst& vc = views[f];
        const V3 r          = quat_rotate(vc.qx, vc.qy, vc.qz, vc.qw, pos);
        const V3 v          = {r.x + vc.tx, r.y + vc.ty, r.z + vc.tz};
        if (!(v.z > 0.f)) continue;
        const V2 np   = {v.x / v.z, v.y / v.z};
        const V2 dp   = distort<false>(np, vc.d, 3.0e38f, nullptr, nullptr);
        const V2 ip   = k_apply(vc.k, dp);
        const bool in = ip.x >= 0.f && ip.y >= 0.f && ip.x < (float)vc.w && ip.y < (float)vc.h;
        const float d = (v.x * v.x + v.y * v.y) + v.z * v.z;
        if (in && d < best) best = d;
    }
    out[i] = sqrtf(best);
}

// SceneData::RemoveClosePoints (SceneData.cpp:598-642) walks the points in order and erases point i when a point it
// has kept before lies within radius[i] of it: state[i] = kept unless a kept j < i is that close.  Here the points
// are decided in rounds: a point whose earlier neighbours are all decided is decided; states only ever go from
// undecided to kept / erased, so reading a neighbour's state of this round instead of the last one is as good.
// One thread per point in cell order; count[round] receives the points still undecided after this round, and a round
// that finds count[round - 1] == 0 has nothing to do.
constexpr int kStateUndecided = 0, kStateKept = 1, kStateErased = 2;

__global__ __launch_bounds__(kBlock) void close_points_kernel(const float4* __restrict__ sorted, int n,
                                                              const KnnGrid* __restrict__ gp,
                                                              const uint32_t* __restrict__ offset,
                                                              const float* __restrict__ radius, int32_t* state,
                                                              uint32_t* round_count, int round)
{
    if (round > 0 && *(volatile uint32_t*)(round_count + round - 1) == 0) return;
    const int t = blockIdx.x * kBlock + threadIdx.x;
    bool pending = false;
    if (t < n)
    {
        const KnnGrid g  = *gp;
        const float4 p   = sorted[t];
        const uint32_t i = __float_as_uint(p.w);
        if (__atomic_load_n(&state[i], __ATOMIC_RELAXED) == kStateUndecided)
        {
            const float rad = radius[i];
            const float r2  = rad * rad;
            const int3 c    = grid_cell(g, p.x, p.y, p.z);
            // cells the ball can reach (the cell of a point is computed in fp32: one cell of slack)
            const float reach = fminf(fmaxf(rad, 0.f) * g.inv_cell, 1.0e6f);
            const int rc      = (int)reach + 1;
            const int z0 = max(c.z - rc, 0), z1 = min(c.z + rc, g.dim[2] - 1);
            const int y0 = max(c.y - rc, 0), y1 = min(c.y + rc, g.dim[1] - 1);
            const int x0 = max(c.x - rc, 0), x1 = min(c.x + rc, g.dim[0] - 1);
            int result = kStateKept;
            for (int cz = z0; cz <= z1 && result != kStateErased; ++cz)
                for (int cy = y0; cy <= y1 && result != kStateErased; ++cy)
                {
                    const uint32_t row = grid_index(g, 0, cy, cz);
                    const uint32_t e   = offset[row + x1 + 1];
                    for (uint32_t q = offset[row + x0]; q < e; ++q)
                    {
                        const float4 o   = sorted[q];
                        const uint32_t j = __float_as_uint(o.w);
                        if (j >= i) continue;
                        const float dx = p.x - o.x, dy = p.y - o.y, dz = p.z - o.z;
                        const float d2 = (dx * dx + dy * dy) + dz * dz;
                        if (!(d2 < r2)) continue;
                        const int sj = __atomic_load_n(&state[j], __ATOMIC_RELAXED);
                        if (sj == kStateKept)
                        {
                            result = kStateErased;
                            break;
                        }
                        if (sj == kStateUndecided) result = kStateUndecided;
                    }
                }
            if (result != kStateUndecided) __atomic_store_n(&state[i], result, __ATOMIC_RELAXED);
            pending = result == kStateUndecided;
        }
    }
    const unsigned long long m = __ballot(pending);
    if (m && (threadIdx.x & 63) == (__ffsll((long long)m) - 1)) atomicAdd(round_count + round, (uint32_t)__popcll(m));
}

// Morton code of every point: 21 bits per axis of the position inside the bounding box, x in the lowest bit.
__device__ __forceinline__ unsigned long long spread21(unsigned long long v)
{
    v &= 0x1FFFFFull;
    v = (v | v << 32) & 0x1F00000000FFFFull;
    v = (v | v << 16) & 0x1F0000FF0000FFull;
    v = (v | v << 8) & 0x100F00F00F00F00Full;
    v = (v | v << 4) & 0x10C30C30C30C30C3ull;
    v = (v | v << 2) & 0x1249249249249249ull;
    return v;
}

__global__ __launch_bounds__(kBlock) void morton_kernel(const float4* __restrict__ position, int n, float min_x,
                                                        float min_y, float min_z, float scale_x, float scale_y,
                                                        float scale_z, unsigned long long* __restrict__ code)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const float4 p = nt_load4(position + i);
    const float m  = 2097151.f;  // 2^21 - 1
    const float fx = fminf(fmaxf((p.x - min_x) * scale_x, 0.f), m);
    const float fy = fminf(fmaxf((p.y - min_y) * scale_y, 0.f), m);
    const float fz = fminf(fmaxf((p.z - min_z) * scale_z, 0.f), m);
    code[i] = spread21((unsigned long long)fx) | spread21((unsigned long long)fy) << 1 | spread21((unsigned long long)fz) << 2;
}

// ------------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------------
void launch_knn_first_grid(const float4* position, int n, const KnnGrid& box, KnnGrid* dst, hipStream_t st)
{
    hipLaunchKernelGGL(knn_first_grid_kernel, dim3(1), dim3(1024), 0, st, position, n, box, dst);
}

void launch_knn_refine_grid(const float* sample, int samples, const KnnGrid* first, KnnGrid* g, uint32_t budget,
                            hipStream_t st)
{
    hipLaunchKernelGGL(knn_refine_grid_kernel, dim3(1), dim3(1024), 0, st, sample, samples, first, g, budget);
}

int knn_num_samples(int n) { return n < kKnnSamples ? n : kKnnSamples; }

// count, prefix sum and scatter of the points into the cells of *g (device)
void launch_knn_build(const float4* position, int n, const KnnGrid* g, uint32_t max_cells, uint32_t* count,
                      uint32_t* offset, uint32_t* chunk_sum, float4* sorted, hipStream_t st)
{
    const int chunks = (int)((max_cells + kScanChunk - 1) / kScanChunk);
    const int blocks = chunks < 1024 ? chunks : 1024;
    const int clear  = (int)((max_cells / 4 + kBlock - 1) / kBlock);
    hipLaunchKernelGGL(knn_clear_kernel, dim3(clear < 4096 ? (clear ? clear : 1) : 4096), dim3(kBlock), 0, st, count, g);
    hipLaunchKernelGGL(knn_bin_kernel, dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0, st, 0, position, n, g, count,
                       offset, sorted);
    // chunk sums and their offsets share one array: [chunks] sums, [chunks + 1] offsets
    hipLaunchKernelGGL(knn_scan_reduce_kernel, dim3(blocks), dim3(1024), 0, st, count, g, chunk_sum);
    hipLaunchKernelGGL(knn_scan_chunks_kernel, dim3(1), dim3(1024), 0, st, chunk_sum, g, chunk_sum + chunks);
    hipLaunchKernelGGL(knn_scan_apply_kernel, dim3(blocks), dim3(1024), 0, st, count, g, chunk_sum + chunks, offset);
    hipLaunchKernelGGL(knn_bin_kernel, dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0, st, 1, position, n, g, count,
                       offset, sorted);
}

size_t knn_chunk_words(uint32_t max_cells)
{
    const size_t chunks = (max_cells + kScanChunk - 1) / kScanChunk;
    return 2 * chunks + 1;
}

bool launch_knn_sample(int rank, const float4* sorted, int n, const KnnGrid* g, const uint32_t* offset, float* out,
                       int samples, hipStream_t st)
{
    const dim3 block(kBlock), grid((samples + kBlock / 64 - 1) / (kBlock / 64));
#define ADOP_KNN_CASE(R) \
    case R: hipLaunchKernelGGL(knn_sample_kernel<R + 1>, grid, block, 0, st, sorted, n, g, offset, out, samples); return true;
    switch (rank)
    {
        ADOP_KNN_CASE(1) ADOP_KNN_CASE(2) ADOP_KNN_CASE(3) ADOP_KNN_CASE(4)
        ADOP_KNN_CASE(5) ADOP_KNN_CASE(6) ADOP_KNN_CASE(7) ADOP_KNN_CASE(8)
    }
#undef ADOP_KNN_CASE
    return false;
}

// The three stages of the search: second grid (all points), first grid (what that left), all points (strays).
bool launch_knn_search(int rank, int n, const KnnSearchArg& a, float* out, hipStream_t st)
{
    const dim3 block(kBlock), grid((n + kBlock - 1) / kBlock), grid2(512), grid3(1024);
#define ADOP_KNN_CASE(R)                                                                                              \
    case R:                                                                                                           \
        hipLaunchKernelGGL(knn_search_kernel<R + 1>, grid, block, 0, st, a.sorted, n, a.grid, a.offset, out, a.list,   \
                           a.counts);                                                                                 \
        hipLaunchKernelGGL(knn_list_kernel<R + 1>, grid2, block, 0, st, a.sorted, a.list, a.counts, a.sorted0, a.grid0, \
                           a.offset0, out, a.list2, a.counts + 1);                                                    \
        hipLaunchKernelGGL(knn_brute_kernel<R + 1>, grid3, block, 0, st, a.sorted, n, a.list2, a.counts + 1, out);     \
        return true;
    switch (rank)
    {
        ADOP_KNN_CASE(1) ADOP_KNN_CASE(2) ADOP_KNN_CASE(3) ADOP_KNN_CASE(4)
        ADOP_KNN_CASE(5) ADOP_KNN_CASE(6) ADOP_KNN_CASE(7) ADOP_KNN_CASE(8)
    }
#undef ADOP_KNN_CASE
    return false;
}

void launch_camera_distance(const float4* position, int n, const ViewConst* views, int num_frames, float* out,
                            hipStream_t st)
{
    hipLaunchKernelGGL(camera_distance_kernel, dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0, st, position, n, views,
                       num_frames, out);
}

void launch_close_points(const float4* sorted, int n, const KnnGrid* g, const uint32_t* offset, const float* radius,
                         int32_t* state, uint32_t* round_count, int round, hipStream_t st)
{
    hipLaunchKernelGGL(close_points_kernel, dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0, st, sorted, n, g, offset,
                       radius, state, round_count, round);
}

void launch_morton(const float4* position, int n, const float* mn, const float* scale, unsigned long long* code,
                   hipStream_t st)
{
    hipLaunchKernelGGL(morton_kernel, dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0, st, position, n, mn[0], mn[1],
                       mn[2], scale[0], scale[1], scale[2], code);
}

}  // namespace adop
