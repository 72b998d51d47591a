// Device code of the routing layout (see layout.hip for the decomposition and the contract), shared by the layout
// kernels and by the kernel that runs the layout and the payload dispatch of a large batch in one launch.
#pragma once

#include "common.h"

namespace dpep {
namespace layout_device {


constexpr int kWaves = 4;             // wavefronts (= chunks) per workgroup
constexpr int kThreads = kWaves * kWave;
constexpr int kHistInts = 16384;      // chunks * padded experts never exceeds this
constexpr int kBlockHistInts = kHistInts / kWaves + DPEP_MAX_LOCAL_EXPERTS;  // workgroups * experts, rounded up
constexpr int kMinChunk = 256;        // routes per wavefront, lower bound (multiple of 64)
constexpr int kPrefetch = 8;          // 64-route steps whose ids are fetched at once
constexpr int kKeep = 16;             // 64-route steps of a chunk that the one-launch kernel holds in registers
constexpr int kColumnBatch = 16;      // histogram loads in flight per thread
static_assert(kSyncTaggedWords >= static_cast<size_t>(kBlockHistInts), "the tagged histograms need a word per (workgroup, expert)");

__device__ __forceinline__ uint64_t lanes_below()
{
    return (1ull << (threadIdx.x & 63)) - 1ull;
}

// Orders this wave's LDS accesses before the call against those after it, for all its lanes.
__device__ __forceinline__ void wave_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Local experts of kSteps consecutive 64-route steps from `base` on.  All loads are issued before the first is
// used (a route past the end reads the last id instead of branching around the load), so that the wave pays
// one memory latency for the batch, not one per step.  Needs n_routes > 0.
template <int kSteps, typename IdxT>
__device__ __forceinline__ void fetch_experts(int (&experts)[kSteps], const IdxT* __restrict__ idx, int base, int end,
                                              int n_routes, int num_experts, int expert_begin, int num_local)
{
    const int lane = threadIdx.x & 63;
    IdxT raw[kSteps];
#pragma unroll
    for (int i = 0; i < kSteps; ++i) raw[i] = idx[min(base + i * kWave + lane, n_routes - 1)];
#pragma unroll
    for (int i = 0; i < kSteps; ++i)
        experts[i] = local_expert(static_cast<long long>(raw[i]), base + i * kWave + lane, end, num_experts, expert_begin,
                                  num_local);
}

// LDS of one workgroup.  running[w][e]: wave w's histogram, later its next free row of expert e; match[w][e]: bit
// per lane of wave w whose route in the current step goes to expert e (all zero between steps); totals[e]: rows
// of expert e.
template <int kMaxExperts>
struct LayoutLdsT {
    int totals[kMaxExperts];
    int running[kWaves][kMaxExperts];
    unsigned long long match[kWaves][kMaxExperts];
    int partial[kThreads * 2];
    int wave_sums[kWaves];
    int timed_out;  // one-launch kernel: some thread's wait for another workgroup's histogram ran out
    unsigned long long tag;  // one-launch kernel: the tag of this launch, read once per workgroup
};
using LayoutLds = LayoutLdsT<DPEP_MAX_LOCAL_EXPERTS>;  // any number of local experts the library takes

template <typename Lds>
__device__ __forceinline__ void clear_wave_lds(Lds& lds, int num_local)
{
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int e = lane; e < num_local; e += kWave) {
        lds.running[wave][e] = 0;
        lds.match[wave][e] = 0ull;
    }
    wave_sync();
}

__device__ __forceinline__ void count_step(int e, int* __restrict__ mine)
{
    if (e >= 0) __hip_atomic_fetch_add(mine + e, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
}

// The waves' histograms (lds.running) out to wave_hist, and their sum to block_hist.  Called by all threads.
template <typename Lds>
__device__ __forceinline__ void publish_histograms(Lds& lds, int num_local, int num_chunks,
                                                   int* __restrict__ wave_hist, int* __restrict__ block_hist)
{
    __syncthreads();
    for (int e = threadIdx.x; e < num_local; e += kThreads) {
        int sum = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const int g = blockIdx.x * kWaves + w;
            const int count = lds.running[w][e];
            sum += count;
            if (g < num_chunks) wave_hist[static_cast<size_t>(g) * num_local + e] = count;
        }
        block_hist[static_cast<size_t>(blockIdx.x) * num_local + e] = sum;
    }
}

// One 64-route step of the ordered replay.  kThrough: route_to_row is written through the caches (device scope), for
// readers in the same launch.
template <bool kThrough = false>
__device__ __forceinline__ void assign_step(int e, int route, int end, unsigned long long* __restrict__ match,
                                            int* __restrict__ next_row, int* __restrict__ route_to_row,
                                            int* __restrict__ row_to_route)
{
    if (e >= 0)
        __hip_atomic_fetch_or(match + e, 1ull << (threadIdx.x & 63), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
    wave_sync();
    int row = -1, ahead = 0, group = 0;
    if (e >= 0) {
        const unsigned long long mask = match[e];
        ahead = __popcll(mask & lanes_below());
        group = __popcll(mask);
        row = next_row[e] + ahead;
    }
    wave_sync();  // every lane has read its expert's mask and next row before the first lane of the group moves them
    if (e >= 0 && ahead == 0) {
        next_row[e] = row + group;
        match[e] = 0ull;
    }
    wave_sync();
    if (route < end) {
        if (kThrough) __hip_atomic_store(route_to_row + route, row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else route_to_row[route] = row;
        if (row >= 0) row_to_route[row] = route;
    }
}

// For one expert, over the workgroups {first, first+stride, ...}: the sum of all block_hist rows and of those
// of workgroups before this one.
struct ColumnSums {
    int total;
    int before;
};

__device__ __forceinline__ ColumnSums column_sums(const int* __restrict__ block_hist, int num_local, int e, int first,
                                                  int stride, int num_blocks)
{
    ColumnSums sums = {0, 0};
    for (int b0 = first; b0 < num_blocks; b0 += kColumnBatch * stride) {
        int v[kColumnBatch];
#pragma unroll
        for (int j = 0; j < kColumnBatch; ++j) {
            const int b = b0 + j * stride;
            v[j] = b < num_blocks ? block_hist[static_cast<size_t>(b) * num_local + e] : 0;
        }
#pragma unroll
        for (int j = 0; j < kColumnBatch; ++j) {
            sums.total += v[j];
            sums.before += b0 + j * stride < static_cast<int>(blockIdx.x) ? v[j] : 0;
        }
    }
    return sums;
}

// Words of the one-launch kernel's exchange (see "one launch" below): tag above kCountBits, count below.
constexpr int kCountBits = 24;
constexpr unsigned long long kCountMask = (1ull << kCountBits) - 1ull;

__device__ __forceinline__ unsigned long long load_word(const unsigned long long* src)
{
    return __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The workgroup's histogram (sum of its waves') out to its row of `tagged`.  Called by all threads, after a workgroup
// barrier behind the counting.
template <typename Lds>
__device__ __forceinline__ void publish_tagged(Lds& lds, int num_local, unsigned long long* __restrict__ tagged,
                                               unsigned long long tag)
{
    for (int e = threadIdx.x; e < num_local; e += kThreads) {
        int sum = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) sum += lds.running[w][e];
        __hip_atomic_store(tagged + static_cast<size_t>(blockIdx.x) * num_local + e,
                           (tag << kCountBits) | static_cast<unsigned long long>(sum), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
}

// column_sums over tagged rows {first, first+stride, ...} below `rows`: every word is re-read until it carries `tag`.
// Sets lds_timed_out and gives up when that takes longer than limit_ticks.
__device__ __forceinline__ ColumnSums tagged_column_sums(const unsigned long long* __restrict__ tagged, int num_local, int e,
                                                         int first, int stride, int rows, unsigned long long tag,
                                                         long long limit_ticks, int* lds_timed_out)
{
    ColumnSums sums = {0, 0};
    long long start = 0;
    for (int b0 = first; b0 < rows; b0 += kColumnBatch * stride) {
        unsigned long long v[kColumnBatch];
        for (int spins = 0;; ++spins) {
            bool all = true;
#pragma unroll
            for (int j = 0; j < kColumnBatch; ++j) {
                const int b = b0 + j * stride;
                v[j] = b < rows ? load_word(tagged + static_cast<size_t>(b) * num_local + e) : tag << kCountBits;
            }
#pragma unroll
            for (int j = 0; j < kColumnBatch; ++j) all = all && (v[j] >> kCountBits) == tag;
            if (all) break;
            if ((spins & 15) == 15) {
                const long long now = wall_clock64();
                if (start == 0) start = now;
                if (now - start > limit_ticks) {
                    *lds_timed_out = 1;
                    return sums;
                }
            }
            __builtin_amdgcn_s_sleep(1);
        }
#pragma unroll
        for (int j = 0; j < kColumnBatch; ++j) {
            const int count = static_cast<int>(v[j] & kCountMask);
            sums.total += count;
            sums.before += b0 + j * stride < static_cast<int>(blockIdx.x) ? count : 0;
        }
    }
    return sums;
}

// Where the one-launch kernel's workgroups find each other's histograms.
struct TaggedSource {
    const unsigned long long* tagged;
    unsigned long long tag;
    int rows;
    long long limit_ticks;
    uint32_t* timeouts;  // host mailbox word that receives launch_id when the wait runs out
    uint32_t launch_id;
};

// From the histograms to every wave's first row per expert (lds.running).  The launch's last workgroup owns no
// chunk: it is the reporter, which writes the per-expert outputs and reports to the host, so that the wait for the
// host stores (a PCIe round trip) delays no workgroup that still has routes to assign.  Called by all threads.
// num_blocks = workgroups that own chunks.  kTagged: the one-launch kernel (the workgroup's own wave histograms are
// still in lds.running, the others' arrive as tagged words from `source`); else the count launch left everything in
// wave_hist / block_hist.  Returns false if the wait for the tagged words ran out: every count is then reported as zero.
template <bool kTagged, typename Lds>
__device__ __forceinline__ bool expert_bases(Lds& lds, const int* __restrict__ wave_hist,
                                             const int* __restrict__ block_hist, int num_local, int padded_local,
                                             int num_chunks, int num_blocks, int* __restrict__ counts,
                                             int* __restrict__ psum, int* __restrict__ offsets, int* __restrict__ num_rows,
                                             uint32_t* __restrict__ mailbox, uint32_t sequence,
                                             const TaggedSource* source = nullptr)
{
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const bool reporter = static_cast<int>(blockIdx.x) == num_blocks;  // the workgroup after those that own chunks
    // This workgroup's own rows are asked for before the column sums, so that all loads are in flight together.
    auto own_rows = [&](int e, int (&own)[kWaves]) {
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const int g = blockIdx.x * kWaves + w;
            if (kTagged) own[w] = lds.running[w][e];  // (the reporter's are zero: it counted nothing)
            else own[w] = g < num_chunks ? wave_hist[static_cast<size_t>(g) * num_local + e] : 0;
        }
    };
    auto sums_of = [&](int e, int first, int stride) {
        if (kTagged)
            return tagged_column_sums(source->tagged, num_local, e, first, stride, source->rows, source->tag,
                                      source->limit_ticks, &lds.timed_out);
        return column_sums(block_hist, num_local, e, first, stride, num_blocks);
    };
    auto finish = [&](int e, int total, int before, const int (&own)[kWaves]) {  // the waves one after the other
        lds.totals[e] = total;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            lds.running[w][e] = before;
            before += own[w];
        }
    };
    if (padded_local >= kThreads) {
        for (int e = tid; e < num_local; e += kThreads) {
            int own[kWaves];
            own_rows(e, own);
            const ColumnSums sums = sums_of(e, 0, 1);
            finish(e, sums.total, sums.before, own);
        }
    } else {
        // Few experts: split the workgroups' rows over `parts` thread groups (at most 16), then reduce through LDS.
        int parts = kThreads / padded_local;
        if (parts > 16) parts = 16;
        const int p = tid / padded_local, e = tid % padded_local;
        int own[kWaves] = {0, 0, 0, 0};
        if (tid < num_local) own_rows(tid, own);
        if (p < parts && e < num_local) {
            const ColumnSums sums = sums_of(e, p, parts);
            lds.partial[tid * 2] = sums.total;
            lds.partial[tid * 2 + 1] = sums.before;
        }
        __syncthreads();
        if (tid < num_local) {
            int total = 0, before = 0;
            for (int q = 0; q < parts; ++q) {
                total += lds.partial[(q * padded_local + tid) * 2];
                before += lds.partial[(q * padded_local + tid) * 2 + 1];
            }
            finish(tid, total, before, own);
        }
    }
    __syncthreads();
    const bool valid = !kTagged || lds.timed_out == 0;
    if (!valid) {
        // A histogram is missing: every count is reported as zero, and the host is told (this store is acknowledged
        // before the reporter publishes the mailbox's sequence word below, so the host never sees one without the other).
        if (tid == 0) __hip_atomic_store(source->timeouts, source->launch_id, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        for (int e = tid; e < num_local; e += kThreads) {
            lds.totals[e] = 0;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) lds.running[w][e] = 0;
        }
        __syncthreads();
    }

    // Exclusive scan of totals over experts: four consecutive experts per thread, then a workgroup scan.
    int mine[4], local_sum = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = tid * 4 + j;
        mine[j] = e < num_local ? lds.totals[e] : 0;
        local_sum += mine[j];
    }
    int incl = local_sum;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int up = __shfl_up(incl, d);
        if (lane >= d) incl += up;
    }
    if (lane == kWave - 1) lds.wave_sums[wave] = incl;
    __syncthreads();
    int offset = incl - local_sum;
    for (int w = 0; w < wave; ++w) offset += lds.wave_sums[w];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = tid * 4 + j;
        if (e < num_local) {
#pragma unroll
            for (int w = 0; w < kWaves; ++w) lds.running[w][e] += offset;
            if (reporter) {
                counts[e] = mine[j];
                psum[e] = offset + mine[j];
                offsets[e + 1] = offset + mine[j];
            }
        }
        offset += mine[j];
    }
    if (reporter && tid == kThreads - 1) {
        offsets[0] = 0;
        num_rows[0] = offset;
    }
    if (reporter && mailbox != nullptr && tid * 4 < num_local) mailbox_store_counts(mailbox, tid * 4, mine);
    // The host polls the mailbox's sequence word: publish it (with the row count, one 8-byte store) after
    // every per-expert count of this workgroup has reached host memory.  The counts went out as write-through
    // stores, so each thread only has to wait until its own are acknowledged: no cache needs writing back, which
    // is what a system-scope release fence would spend microseconds on after a kernel that left the L2 dirty.
    if (reporter && mailbox != nullptr) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (reporter && mailbox != nullptr && tid == kThreads - 1) {
        const unsigned long long word = (static_cast<unsigned long long>(sequence) << 32) | static_cast<uint32_t>(offset);
        __hip_atomic_store(reinterpret_cast<unsigned long long*>(mailbox), word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    return valid;
}

// ---- one launch: histograms exchanged as tagged words -------------------------------------------------------------
// A published histogram entry is one 64-bit word: the launch's tag in the upper kTagBits, the count below.  A reader
// knows from the word itself whether it belongs to this launch, so there is nothing to wait for but the data, and
// nothing to clear afterwards.  Tags only grow: a launch uses epoch + 1, where the epoch (device memory) is the highest
// tag any launch on this workspace has used, read by every workgroup before it publishes and raised with an atomic max
// when the workgroup ends.  No workgroup can end before every workgroup has read the epoch: it ends only after it has
// seen the words of everybody who owns a chunk, which are published after that read, and the tag of the reporter, which
// owns none, in a word of its own (the reporter stores it right after its read; the others look for it as the last
// thing they do, when it has long been there).  So all workgroups of a launch agree on the tag; a launch that ran
// out of time may use two tags, and the atomic max still leaves the epoch above both.  Replays of a captured launch
// therefore get fresh tags without any host involvement.  40 tag bits last 10^12 launches.
// Count, exchange, assign in one launch; every wave keeps the ids of its chunk (at most kKeep steps) in registers.
// `rows` = histogram rows to wait for (the workgroups that own chunks; one more in a test that wants the wait to run out),
// `limit_ticks` the bound of that wait (100 MHz ticks); `layout_blocks` = the workgroups that run this body (those that own
// chunks, then the reporter): the first ones of the launch.
template <bool kThrough, typename IdxT, typename Lds>
__device__ __forceinline__ void layout_fused_body(
    Lds& lds, int layout_blocks, const IdxT* __restrict__ idx, int n_routes, int num_experts, int expert_begin, int num_local, int padded_local,
    int chunk, int num_chunks, int* __restrict__ counts, int* __restrict__ psum, int* __restrict__ offsets,
    int* __restrict__ num_rows, int* __restrict__ route_to_row, int* __restrict__ row_to_route,
    uint32_t* __restrict__ mailbox, uint32_t sequence, unsigned long long* __restrict__ epoch,
    unsigned long long* __restrict__ tagged, int rows, long long limit_ticks, uint32_t* __restrict__ timeouts,
    uint32_t launch_id)
{
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int g = blockIdx.x * kWaves + wave;
    const int begin = g < num_chunks ? g * chunk : 0;
    const int end = g < num_chunks ? min(begin + chunk, n_routes) : 0;
    // One thread reads the epoch for the whole workgroup (asked for together with the ids): every thread must use the
    // same tag, and the tag must be final before anything this workgroup publishes can be seen.
    unsigned long long* reporter_tag = epoch + kSyncReporterTag / sizeof(unsigned long long);
    const bool reporter = static_cast<int>(blockIdx.x) == layout_blocks - 1;
    if (threadIdx.x == 0) {
        lds.tag = load_word(epoch) + 1ull;
        lds.timed_out = 0;
        if (reporter) __hip_atomic_store(reporter_tag, lds.tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    int experts[kKeep];
    fetch_experts(experts, idx, begin, end, n_routes, num_experts, expert_begin, num_local);
    clear_wave_lds(lds, num_local);
#pragma unroll
    for (int i = 0; i < kKeep; ++i) count_step(experts[i], lds.running[wave]);
    __syncthreads();
    const unsigned long long tag = lds.tag;
    // (the reporter owns no chunk and publishes nothing: row layout_blocks - 1 is only ever waited for by a test that wants
    // the wait to run out)
    if (!reporter) publish_tagged(lds, num_local, tagged, tag);
    const TaggedSource source = {tagged, tag, rows, limit_ticks, timeouts, launch_id};
    const bool in_time = expert_bases<true>(lds, nullptr, nullptr, num_local, padded_local, num_chunks, layout_blocks - 1, counts,
                                            psum, offsets, num_rows, mailbox, sequence, &source);
    // (asked for here, needed only at the very end: the load travels while the routes are assigned)
    unsigned long long reporter_seen = threadIdx.x == 0 && !reporter ? load_word(reporter_tag) : 0ull;
    if (in_time) {
#pragma unroll
        for (int i = 0; i < kKeep; ++i)
            if (begin + i * kWave < end)
                assign_step<kThrough>(experts[i], begin + i * kWave + lane, end, lds.match[wave], lds.running[wave], route_to_row,
                                      row_to_route);
    } else {
        // Some workgroup's histogram is missing: rows computed without it could lie anywhere.  No route gets a row
        // (and the counts above are all zero).
        for (int route = begin + lane; route < end; route += kWave) {
            if (kThrough) __hip_atomic_store(route_to_row + route, -1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else route_to_row[route] = -1;
        }
    }
    if (threadIdx.x == 0) {
        // The epoch may only move once the reporter has read it (a reporter that read the raised epoch would wait for
        // words nobody publishes).  Tags only grow, so any value from this launch's tag on means that it has; the wait
        // is bounded like the others, and a reporter that comes later still reports the launch as failed.
        if (!reporter) {
            long long start = 0;
            for (int spins = 0; reporter_seen < tag; ++spins) {
                if ((spins & 15) == 15) {
                    const long long now = wall_clock64();
                    if (start == 0) start = now;
                    if (now - start > limit_ticks) break;
                }
                __builtin_amdgcn_s_sleep(1);
                reporter_seen = load_word(reporter_tag);
            }
        }
        __hip_atomic_fetch_max(epoch, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}


}  // namespace layout_device
}  // namespace dpep
