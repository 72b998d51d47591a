// Work partition and copy/wait schedule of the grouped GEMM, shared by the kernel (device) and by the host-side
// replay that checks the schedule (dpep_megamoe_schedule_check).  Everything here is plain integer arithmetic.
#pragma once
#include <stdint.h>

#ifndef __HIPCC__
#define __host__
#define __device__
#endif

namespace dpep {

constexpr int kSpanItems = 4;    // k tiles (items) per span: the unit scales are copied in and work is dealt out in
constexpr int kZeroPerItem = 4;  // 1 KiB zero stores a wave issues per item while it still has output rows to zero

// Per tile height (64 * RT rows): LDS stages, how many items the copies run ahead, 16-byte copies per thread and item.
template <int RT>
struct GemmRing {
    static constexpr int kStages = RT == 1 ? 5 : RT == 2 ? 4 : 3;
    static constexpr int kAhead = kStages;
    static constexpr int kCopies = 2 * RT + 4;
    // Vector-memory operations that may still be in flight at an item's wait such that the NEXT item's copies
    // (and the scale / index copies that followed them) have landed: the copies of the kAhead - 2 items after it.
    // Zero stores sit between those copy groups when every one of those items issued kZeroPerItem of them.
    static constexpr int kWaitPlain = (kAhead - 2) * kCopies;
    static constexpr int kWaitZeroing = (kAhead - 2) * (kCopies + kZeroPerItem);
};

// ---- who works on what ---------------------------------------------------------------------------------------
// The launch's work is the flat stream of (tile, k tile) items, tile-major, measured in spans of kSpanItems items
// (a tile's last span is short when its k tiles are not a multiple of four).  `workers` workgroups take
// consecutive ranges of it.  When whole tiles deal out evenly enough the ranges end on tile boundaries;
// otherwise they are equal shares of the span stream, a tile's k range is then summed by several workers and the
// last of them to finish adds the others' partial sums.
struct WorkSplit {
    int split;       // 1: ranges may end inside a tile
    int workers;     // workgroups that get a range (the others have none)
    int spans_per_tile;
    long long total_spans;
};

__host__ __device__ inline WorkSplit choose_split(int total_tiles, int ktiles, int grid)
{
    WorkSplit s;
    s.spans_per_tile = (ktiles + kSpanItems - 1) / kSpanItems;
    s.total_spans = static_cast<long long>(total_tiles) * s.spans_per_tile;
    const long long rounds = (total_tiles + grid - 1) / grid;
    const long long idle = rounds * grid - total_tiles;  // tile slots nobody fills in the last round
    s.split = total_tiles > 0 && idle * 8 > rounds * grid;
    if (s.split) {
        // nobody gets less than one span, and a tile is cut into at most about four pieces
        long long workers = grid;
        if (workers > s.total_spans) workers = s.total_spans;
        if (workers > 4ll * total_tiles) workers = 4ll * total_tiles;
        s.workers = static_cast<int>(workers);
    } else {
        s.workers = total_tiles < grid ? total_tiles : grid;
    }
    return s;
}

struct WorkRange {
    long long begin, end;  // spans
};

__host__ __device__ inline WorkRange worker_range(const WorkSplit& s, int worker)
{
    WorkRange r = {0, 0};
    if (worker >= s.workers) return r;
    if (s.split) {
        r.begin = s.total_spans * worker / s.workers;
        r.end = s.total_spans * (worker + 1) / s.workers;
    } else {
        const long long tiles = s.total_spans / s.spans_per_tile;
        r.begin = tiles * worker / s.workers * s.spans_per_tile;
        r.end = tiles * (worker + 1) / s.workers * s.spans_per_tile;
    }
    return r;
}

// The worker whose range holds `span` (split ranges only).
__host__ __device__ inline int span_owner(const WorkSplit& s, long long span)
{
    return static_cast<int>(((span + 1) * s.workers - 1) / s.total_spans);
}

// Items in [begin, end): four per span, less what the short last span of each tile that ends inside lacks.
__host__ __device__ inline long long range_items(const WorkSplit& s, const WorkRange& r, int ktiles)
{
    const long long tile_ends = r.end / s.spans_per_tile - r.begin / s.spans_per_tile;
    return (r.end - r.begin) * kSpanItems - tile_ends * (static_cast<long long>(s.spans_per_tile) * kSpanItems - ktiles);
}

// ---- when the copy cursor may trust the next tile's gather indices ---------------------------------------------
// The indices of a worker's next tile are fetched (asynchronously, into LDS) together with the first item the
// worker issues of the current tile, and read when the cursor moves on to that next tile, right after it has
// issued the current tile's last item.  Waits only happen in the main loop, one per consumed item, and the wait of
// consumed item m guarantees everything issued with items <= m + 1.  The cursor is kAhead items ahead of the
// consumer, so the fetch is covered iff the worker issued at least kAhead items of the current tile and the
// switch does not happen in the prologue (which issues kAhead items before the first wait).  Otherwise the
// cursor has to drain its copies (wait for all of them, then a workgroup barrier) before it reads the indices.
__host__ __device__ inline bool switch_needs_drain(bool in_prologue, int tile_items_issued, int ahead)
{
    return in_prologue || tile_items_issued < ahead;
}

// Items of a worker that carry zero stores: the first zero_blocks / kZeroPerItem of them.  The wait of item i may
// count those stores as in flight only if every item whose stores sit between the copy groups still in flight did
// issue them: items i - (kAhead - 2) ... i - 1.
__host__ __device__ inline bool wait_counts_zero_stores(int item, int zero_items, int ahead)
{
    return item >= ahead - 2 && item - 1 < zero_items;
}

}  // namespace dpep
