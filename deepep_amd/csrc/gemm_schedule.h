// Copy/wait schedule of the grouped GEMM, shared by the kernel (device) and by the host-side replay that checks it
// (dpep_megamoe_schedule_check).  Everything here is plain integer arithmetic.
#pragma once
#include <stdint.h>

#ifndef __HIPCC__
#define __host__
#define __device__
#endif

namespace dpep {

// Per tile height (64 * RT rows): LDS stages, how many items (k tiles of 128) the copies run ahead, 16-byte copies
// per thread and item (A and B).
template <int RT>
struct GemmRing {
    static constexpr int kStages = RT == 1 ? 5 : RT == 2 ? 4 : 3;
    // Copies run a full ring ahead: a stage is refilled in the very item that consumes it, right after the
    // barrier that follows the last LDS read of it.
    static constexpr int kAhead = kStages;
    static constexpr int kCopies = 2 * RT + 4;
    // Vector-memory operations that may still be in flight at an item's wait such that the NEXT item's copies
    // (and the scale / index copies that followed them) have landed: the copies of the kAhead - 2 items after it.
    static constexpr int kWaitPlain = (kAhead - 2) * kCopies;
};

// The column-wave kernel (weights straight to registers): per tile height the ring of four stages that is also the unroll of
// its item loop, the asynchronous requests per thread and item (activation copies + four weight loads; a span's first item
// adds two scale copies, a tile's first item the fetch of the next tile's gather indices), and what may still be in flight at
// an item's wait such that the NEXT item's operands have arrived: the requests of the two items after it.
template <int RT>
struct ColumnRing {
    static constexpr int kStages = 4;
    static constexpr int kRequests = 2 * RT + 4;
    static constexpr int kWait = 2 * kRequests;
    static constexpr int kPrologueWait = (kStages - 1) * kRequests;  // behind the prologue's four items: item 0 has arrived
};

// When the copy cursor may trust the next tile's gather indices.  They are fetched (asynchronously, into LDS)
// together with the first item of the current tile, and read when the cursor moves on to that next tile, right after
// it has issued the current tile's last item.  Waits only happen in the main loop, one per consumed item, and the
// wait of consumed item m guarantees everything issued with items <= m + 1.  The cursor is kAhead items ahead of the
// consumer, so the fetch is covered iff the tile has at least kAhead items and the switch does not happen in the
// prologue (which issues kAhead items before the first wait).  Otherwise the cursor has to drain its copies (wait
// for all of them, then a workgroup barrier) before it reads the indices.
__host__ __device__ inline bool switch_needs_drain(bool in_prologue, int tile_items, int ahead)
{
    return in_prologue || tile_items < ahead;
}

}  // namespace dpep
