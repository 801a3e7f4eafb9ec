// launch.h — host-callable launchers of the kernels (one translation unit per kernel family).
#pragma once
#include <stdlib.h>
#include "common.h"

namespace adop
{
// The process's tuning switches as they are now (adop_set_tuning / adop_get_tuning; defined in adop_raster.hip).
adop_tuning tuning_now();

struct EnvLevels
{
    float* uv[ADOP_MAX_LAYERS];
    float* env[ADOP_MAX_LAYERS];
    const float* gout[ADOP_MAX_LAYERS];
};

void launch_prepare_views(const ViewChunk& ch, int first, int count, const double* poses, const float* intrinsics,
                          int cols, ViewConst* out, hipStream_t st);
void launch_fill_u32(uint32_t* p, size_t n, uint32_t v, hipStream_t st);
void launch_clear(const Levels& lv, int first_level, int grid, float* accum, size_t accum_floats, uint32_t* zero_u32,
                  int zero_n, const ViewPrep& vp, hipStream_t st, Gate gate = {nullptr, 0}, adop_stats* zero_stats = nullptr);
void launch_knn_first_grid(const float4* position, int n, const KnnGrid& box, KnnGrid* dst, hipStream_t st);
void launch_knn_refine_grid(const float* sample, int samples, const KnnGrid* first, KnnGrid* g, uint32_t budget,
                            hipStream_t st);
int knn_num_samples(int n);
size_t knn_chunk_words(uint32_t max_cells);  // uint32 words of the scan's scratch array
void launch_knn_build(const float4* position, int n, const KnnGrid* g, uint32_t max_cells, uint32_t* count,
                      uint32_t* offset, uint32_t* chunk_sum, float4* sorted, hipStream_t st);
bool launch_knn_sample(int rank, const float4* sorted, int n, const KnnGrid* g, const uint32_t* offset, float* out,
                       int samples, hipStream_t st);
struct KnnSearchArg
{
    const KnnGrid *grid, *grid0;          // second / first grid (device)
    const float4 *sorted, *sorted0;       // the points in cell order of either grid
    const uint32_t *offset, *offset0;
    uint32_t *list, *list2;               // [n] points left over by the first / second stage
    uint32_t* counts;                     // [2] their numbers, zero at the start
};
bool launch_knn_search(int rank, int n, const KnnSearchArg& a, float* out, hipStream_t st);
void launch_camera_distance(const float4* position, int n, const ViewConst* views, int num_frames, float* out,
                            hipStream_t st);
void launch_close_points(const float4* sorted, int n, const KnnGrid* g, const uint32_t* offset, const float* radius,
                         int32_t* state, uint32_t* round_count, int round, hipStream_t st);
void launch_morton(const float4* position, int n, const float* mn, const float* scale, unsigned long long* code,
                   hipStream_t st);
// The launchers take the tuning switches of the call as an argument (one snapshot per call: adop_forward / adop_backward).
// points per workgroup of prepass_kernel on a cloud of n points (the unit of its candidate lists)
int prepass_points_per_block(int n, int tuned_ppt);
void launch_prepass(const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp, adop_stats* stats,
                    const adop_tuning& tn, hipStream_t st, Gate gate = {nullptr, 0});
void launch_blend(const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp, bool half,
                  float* accum, int S, adop_stats* stats, const adop_tuning& tn, hipStream_t st, Gate gate = {nullptr, 0});
void launch_resolve(const Levels& lv, int first_level, int grid, const float* accum, int S, const float* background,
                    int write_mask, float mask_value, hipStream_t st, Gate gate = {nullptr, 0});

// Forward pass through screen-space tile bins (binned_kernels.hip, tile_kernels.hip).  A tile has kBlock level-0 pixels,
// one per thread of a workgroup: 16 x 16 (32 x 8, with 128-byte rows in the output tensors, measured 5 % slower: more
// points have their level-1 pixel in another tile).
constexpr int kTileShiftX = 4;
constexpr int kTileShiftY = 4;
struct BinArg
{
    uint32_t* count;   // [T] entries per tile after the first pass; the second pass counts it down to zero to hand
                       // out the slots of a bin
    uint32_t* offset;  // [T + 1] exclusive prefix sum
    uint4* order;      // [T + max_rows] (tile, first entry, end, slice word): the tiles as the tile kernels take them,
                       // the fullest bins first; behind them the further slices of the bins that are split
    // A bin with more than slice_entries entries (a cloud that covers a few tiles only) is split in K slices that as
    // many workgroups take: slice 0 in the tile's own place of the order, the others in order[T + row + s].  The slices
    // leave their partial results of the tile's own pixels in rows[row + s]; the one that finishes last (ticket) merges
    // the K rows in their fixed order and writes the pixels.  Slice word: K | s << 10 | row << 20 (0: not split).
    uint32_t* row_count;   // rows handed out (zero at the start of the call; may run past max_rows: bins that get no
                           // rows stay whole)
    uint32_t* tickets;     // [2][max_rows] depth pass, blend pass (zero at the start of the call)
    float* rows;           // [max_rows][row_floats]
    uint32_t slice_entries;
    int32_t max_rows;      // 16 .. kMaxSlices, by the size of the cloud (slice_rows())
    int32_t row_floats;    // two accumulators of C + 1 floats per thread (slice_row_floats())
    float4* entries;   // (ip.x, ip.y, +-depth, point id | flags), at most lt per point and view
    uint32_t* info;    // [B * N] written by the first pass for the second: tile of the primary entry (bits 0..23),
                       // levels before the LOD break (24..26), second entry one tile to the right / below (27, 28),
                       // point has entries (31)
    int32_t tiles_x, tiles_y;  // tiles of one view
    int32_t lt;                // levels rendered in the tile's LDS (1 or 2); the others go through global atomics
    // A tile has 1 << shard_shift counters and offsets.  Runs of 256 consecutive points take the shards in turn, in
    // both binning passes alike, so a bin is the concatenation of its shards' parts: offset[(tile << shard_shift) +
    // shard].  Atomics on one cache line run one after the other (~0.1 us each): a view whose cloud piles up in a few
    // tiles waits for the chains on their counters' lines, and every shard shortens them, which is why the counters
    // lie shard by shard, count[shard * num_tiles + tile], the shards of a tile (and of its neighbours) in lines of
    // their own.
    int32_t shard_shift;
    int32_t num_tiles;  // tiles of all views of the call
    // A workspace with smaller bins (ADOP_WORKSPACE_SMALL_BINS): `entries` holds `cap` entries, fewer than the call can
    // have.  The prefix sum writes *overflow = 1 when the call has more (else 0); the second binning pass and the tile
    // kernels then return at once.  nullptr: the bins hold every entry the call can have.
    uint32_t* overflow;
    uint32_t cap;
};
// Shards per tile: as many as keep the counters of a call within 16 384 (the prefix sum over them is one workgroup), at
// most 8, and none above 4 096 tiles: the second pass then looks up two lines per entry group instead of one, which a
// view of 1920 x 1080 without hot tiles pays with 7 us (config 3), while 4 views of 512 x 512 of a cloud that piles up
// in the image centre gain 15 us (config 2: 0.270 -> 0.256 ms).  `tuned` >= 0 (adop_tuning.bin_shard_shift) asks for a
// shift, which is lowered while the call would need more counters than the workspace holds.
constexpr size_t kMaxShardedCounters = 65536;  // counters a call may have through an explicit shard shift
inline int bin_shard_shift(size_t tiles, int tuned)
{
    if (tuned >= 0)
    {
        int s = tuned > 3 ? 3 : tuned;
        while (s > 0 && (tiles << s) > kMaxShardedCounters) --s;
        return s;
    }
    int s = 0;
    while (tiles <= 4096 && s < 3 && (tiles << (s + 1)) <= 16384) ++s;
    return s;
}
// counters the workspace holds for a call of `tiles` tiles: enough for every shard shift bin_shard_shift() can return
inline size_t bin_counter_capacity(size_t tiles)
{
    size_t c = tiles;
    for (int s = 1; s <= 3; ++s)
        if ((tiles << s) <= kMaxShardedCounters) c = tiles << s;
    return c;
}
inline uint32_t bin_shard_of(uint32_t point, int shard_shift) { return (point >> 8) & ((1u << shard_shift) - 1u); }
constexpr int kMaxSlices = 1024;  // (10 bits of the slice word)
// A bin with more than kSplitFrom slices' worth of entries is split in slices of kSliceEntries.  Splitting a bin that is
// not by far the longest piece of work of its launch only costs (a tile's set-up per slice, and the release / acquire
// around its ticket, which writes back and invalidates the L2 of its XCD: config 5, whose fullest bins hold 10 to 30
// thousand entries, lost 0.3 ms per tile kernel when they were split), and the rows are handed out as the bins come:
// those bins would take them from the ones that need them.
constexpr int kSliceEntries = 8192;
constexpr int kSplitFrom    = 4;
inline int slice_row_floats(int C) { return (1 << (kTileShiftX + kTileShiftY)) * 2 * (C + 1); }
// rows for the slices of split bins: what a cloud of n points in B views can fill at the default slice size
inline int slice_rows(long long n, int B)
{
    const long long r = (2 * n * B + kSliceEntries - 1) / kSliceEntries;
    return (int)(r < 16 ? 16 : (r > kMaxSlices ? kMaxSlices : r));
}
constexpr uint32_t kEntryIdMask  = 0x0FFFFFFFu;  // entry word: point id; bits 28..30: levels before the LOD break;
constexpr uint32_t kEntryPrimary = 0x80000000u;  // bit 31: entry of the tile that owns the (clamped) level-0 pixel
void launch_bin(int pass, const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp,
                const BinArg& bin, adop_stats* stats, const adop_tuning& tn, hipStream_t st);
void launch_tile_scan(const BinArg& bin, int num_tiles, hipStream_t st);
void launch_tile_depth(const Levels& lv, const BinArg& bin, int num_tiles, hipStream_t st);
hipError_t launch_tile_blend(const CloudArg& pc, const Levels& lv, const ParamArg& rp, const BinArg& bin, int num_tiles,
                             bool half, float* accum, int S, const float* background, int write_mask,
                             float mask_value, int identity_index, adop_stats* stats, const adop_tuning& tn,
                             hipStream_t st);

void launch_interleave(const Levels& lv, int blocks, float* ig, float2* dw, double* partial, uint32_t* q_counts,
                       const ViewPrep& vp, hipStream_t st);
// Work queue of the backward pass (points that receive a ghost / spatial gradient), split in kNumQueues sub-queues
// of `cap` items each.
struct QueueArg
{
    uint32_t* counts;           // [B][kNumQueues]: one set per view
    unsigned long long* items;  // [B][kNumQueues * cap]
    uint32_t cap;
    int normalize;              // one view: 0 = the point gradients are normalised by the finalize kernel; 1, 2 = by the
                                // spatial-gradient kernel, as normalize_mode 0 / 1 (the descriptor pass then writes
                                // the final count of every point)
    int concurrent;             // several views: 1 = the items of all views are pushed when the descriptor pass knows
                                // which points several views share, and the spatial-gradient kernel runs every view
                                // in one launch; 0 = items pushed view by view, one spatial-gradient launch per view
};
void launch_backward_tex(const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp, bool half,
                         const float* ig, const float2* dw, const adop_backward_buffers* g, int identity_index,
                         const QueueArg& q, adop_stats* stats, hipStream_t st);
void launch_backward_ghost(const CloudArg& pc, const ViewConst* views, const Levels& lv, const ParamArg& rp, bool half,
                           const float* ig, const adop_backward_buffers* g, int want_pose, int want_intr,
                           int identity_index, int b, const QueueArg& q, int ghost_blocks, double* partial,
                           hipStream_t st);
constexpr int kConcurrentViews = 24;  // views whose level masks a descriptor-pass thread can keep (2 x 12 x 5 bits)
void launch_finalize(const ViewConst* views, int B, int C, const double* bg_partial, int bg_blocks,
                     const double* pt_partial, int pt_blocks, const adop_backward_buffers* g, int num_poses,
                     int num_cameras, int cols, int normalize_mode, double* scratch, double* mini, uint32_t* ticket, int n,
                     const QueueArg& q, const adop_tuning& tn, hipStream_t st);

void launch_env_sample(const ViewChunk& chunk, const double* poses, const float* intrinsics, const Levels& lv,
                       const EnvLevels& ev, const float* tex, int eh, int ew, int add_to_out, int cols, hipStream_t st);
void launch_env_backward(const ViewChunk& chunk, const double* poses, const float* intrinsics, const Levels& lv,
                         const EnvLevels& ev, float* genv, int eh, int ew, int cols, hipStream_t st);
void launch_apply_tangent(double* tangent, double* poses, int n, hipStream_t st);
}  // namespace adop
