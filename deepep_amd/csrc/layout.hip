// Routing layout for one rank: per-expert counts, prefix sums and the stable expert-major
// permutation of the T*K routes (a stable counting sort); no atomic decides the order of rows.
//
// Observable contract (reference: tests/utils/reference.py:39-73, tests/clos/common.py:248-287,
// tests/elastic/test_dispatch.py:538-548): rows are ordered (local expert, token, slot); every valid
// slot gets its own row (duplicates included); invalid ids produce no row.
//
// Decomposition: the flat route stream is cut into chunks, one wavefront each, four per workgroup.
//   count  : each wave histograms its chunk in LDS (atomic adds: a count does not depend on order)
//            -> wave_hist[chunk][expert] and the workgroup's sum block_hist[workgroup][expert]
//   assign : each workgroup sums block_hist over the workgroups (expert totals and their exclusive scan; the
//            workgroups before it -> its own base) and adds its waves' rows, then every wave replays its chunk in
//            order.  Inside a 64-route step the lanes with the same expert find each other through a 64-bit
//            mask per expert in LDS (each lane ORs its bit in, then all read the mask back): a route's row is
//            its expert's next free row plus the number of lower lanes in the mask.  The carry between steps
//            lives in LDS.  There is no separate scan launch.
// Inputs whose chunks fit a wave's registers (at most kKeep steps of 64 routes) take ONE launch: the workgroups
// (at most 65, far fewer than there are CUs, so all are resident together) count, publish their histograms as
// self-validating words (count + the launch's tag in one 64-bit store), read each other's as soon as they appear, and
// assign from the ids they still hold: no barrier, no counter that anybody has to reset.  The wait for the others'
// words is bounded; a launch whose wait runs out assigns nothing (a histogram is missing): it reports no rows, marks
// every route as having none, and leaves its number in the workspace's mailbox, where the host finds it; later layouts
// on that workspace take two launches.  Larger inputs take two launches anyway.
#include <mutex>

#include "common.h"

namespace dpep {
namespace {

constexpr int kWaves = 4;             // wavefronts (= chunks) per workgroup
constexpr int kThreads = kWaves * kWave;
constexpr int kHistInts = 16384;      // chunks * padded experts never exceeds this
constexpr int kBlockHistInts = kHistInts / kWaves + DPEP_MAX_LOCAL_EXPERTS;  // workgroups * experts, rounded up
constexpr int kLargeHistInts = 65536;  // the two-launch form of large inputs, where the workspace has the room
constexpr int kLargeBlockHistInts = kLargeHistInts / kWaves + DPEP_MAX_LOCAL_EXPERTS;
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
struct LayoutLds {
    int totals[DPEP_MAX_LOCAL_EXPERTS];
    int running[kWaves][DPEP_MAX_LOCAL_EXPERTS];
    unsigned long long match[kWaves][DPEP_MAX_LOCAL_EXPERTS];
    int partial[kThreads * 2];
    int wave_sums[kWaves];
    int timed_out;  // one-launch kernel: some thread's wait for another workgroup's histogram ran out
    unsigned long long tag;  // one-launch kernel: the tag of this launch, read once per workgroup
};

__device__ __forceinline__ void clear_wave_lds(LayoutLds& lds, int num_local)
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
__device__ __forceinline__ void publish_histograms(LayoutLds& lds, int num_local, int num_chunks,
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

// One 64-route step of the ordered replay.
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
        route_to_row[route] = row;
        if (row >= 0) row_to_route[row] = route;
    }
}

template <typename IdxT>
__global__ __launch_bounds__(kThreads) void layout_count_kernel(const IdxT* __restrict__ idx, int n_routes,
                                                                int num_experts, int expert_begin, int num_local,
                                                                int chunk, int num_chunks, int* __restrict__ wave_hist,
                                                                int* __restrict__ block_hist)
{
    __shared__ LayoutLds lds;
    const int wave = threadIdx.x >> 6;
    const int g = blockIdx.x * kWaves + wave;
    const int begin = g < num_chunks ? g * chunk : 0;
    const int end = g < num_chunks ? min(begin + chunk, n_routes) : 0;
    clear_wave_lds(lds, num_local);
    for (int base = begin; base < end; base += kPrefetch * kWave) {
        int experts[kPrefetch];
        fetch_experts(experts, idx, base, end, n_routes, num_experts, expert_begin, num_local);
#pragma unroll
        for (int i = 0; i < kPrefetch; ++i) count_step(experts[i], lds.running[wave]);
    }
    publish_histograms(lds, num_local, num_chunks, wave_hist, block_hist);
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
__device__ __forceinline__ void publish_tagged(LayoutLds& lds, int num_local, unsigned long long* __restrict__ tagged,
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
template <bool kTagged>
__device__ __forceinline__ bool expert_bases(LayoutLds& lds, const int* __restrict__ wave_hist,
                                             const int* __restrict__ block_hist, int num_local, int padded_local,
                                             int num_chunks, int num_blocks, int* __restrict__ counts,
                                             int* __restrict__ psum, int* __restrict__ offsets, int* __restrict__ num_rows,
                                             uint32_t* __restrict__ mailbox, uint32_t sequence,
                                             const TaggedSource* source = nullptr)
{
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const bool reporter = blockIdx.x == gridDim.x - 1;
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
        // A histogram is missing: every count is reported as zero, and the host is told.  (The reporter's own store is
        // acknowledged before it publishes the mailbox's sequence word below, so the host never sees a reporter's
        // time-out later than its report; another workgroup's time-out may reach the host after the report, and is
        // then found by the next call on the workspace.)
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

template <typename IdxT>
__global__ __launch_bounds__(kThreads) void layout_assign_kernel(
    const IdxT* __restrict__ idx, int n_routes, int num_experts, int expert_begin, int num_local, int padded_local,
    int chunk, int num_chunks, const int* __restrict__ wave_hist, const int* __restrict__ block_hist,
    int* __restrict__ counts, int* __restrict__ psum, int* __restrict__ offsets, int* __restrict__ num_rows,
    int* __restrict__ route_to_row, int* __restrict__ row_to_route, uint32_t* __restrict__ mailbox, uint32_t sequence)
{
    __shared__ LayoutLds lds;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int g = blockIdx.x * kWaves + wave;
    const int begin = g < num_chunks ? g * chunk : 0;
    const int end = g < num_chunks ? min(begin + chunk, n_routes) : 0;
    int experts[kPrefetch];  // the first ids travel while the histograms are summed
    if (begin < end) fetch_experts(experts, idx, begin, end, n_routes, num_experts, expert_begin, num_local);
    clear_wave_lds(lds, num_local);
    __syncthreads();  // expert_bases writes the rows of all waves
    expert_bases<false>(lds, wave_hist, block_hist, num_local, padded_local, num_chunks, gridDim.x - 1, counts, psum,
                        offsets, num_rows, mailbox, sequence);
    for (int base = begin; base < end; base += kPrefetch * kWave) {
        if (base != begin) fetch_experts(experts, idx, base, end, n_routes, num_experts, expert_begin, num_local);
#pragma unroll
        for (int i = 0; i < kPrefetch; ++i)
            assign_step(experts[i], base + i * kWave + lane, end, lds.match[wave], lds.running[wave], route_to_row,
                        row_to_route);
    }
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
// `limit_ticks` the bound of that wait (100 MHz ticks).
template <typename IdxT>
__global__ __launch_bounds__(kThreads) void layout_fused_kernel(
    const IdxT* __restrict__ idx, int n_routes, int num_experts, int expert_begin, int num_local, int padded_local,
    int chunk, int num_chunks, int* __restrict__ counts, int* __restrict__ psum, int* __restrict__ offsets,
    int* __restrict__ num_rows, int* __restrict__ route_to_row, int* __restrict__ row_to_route,
    uint32_t* __restrict__ mailbox, uint32_t sequence, unsigned long long* __restrict__ epoch,
    unsigned long long* __restrict__ tagged, int rows, long long limit_ticks, uint32_t* __restrict__ timeouts,
    uint32_t launch_id)
{
    __shared__ LayoutLds lds;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int g = blockIdx.x * kWaves + wave;
    const int begin = g < num_chunks ? g * chunk : 0;
    const int end = g < num_chunks ? min(begin + chunk, n_routes) : 0;
    // One thread reads the epoch for the whole workgroup (asked for together with the ids): every thread must use the
    // same tag, and the tag must be final before anything this workgroup publishes can be seen.
    unsigned long long* reporter_tag = epoch + kSyncReporterTag / sizeof(unsigned long long);
    const bool reporter = blockIdx.x == gridDim.x - 1;
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
    // (the reporter owns no chunk and publishes nothing: row gridDim.x - 1 is only ever waited for by a test that wants
    // the wait to run out)
    if (!reporter) publish_tagged(lds, num_local, tagged, tag);
    // The reporter gives up first (the others wait twice as long): a launch that the reporter passes as valid is then
    // one in which every histogram arrived within the reporter's bound, so another workgroup can only have run out of
    // time if its own wait began more than a whole bound before the reporter's.  What remains of that window is closed
    // on the consumers' side: such a workgroup marks its routes as having no row, and the kernels that read
    // row_to_route clamp what they find there.
    const TaggedSource source = {tagged, tag, rows, reporter ? limit_ticks : 2 * limit_ticks, timeouts, launch_id};
    const bool in_time = expert_bases<true>(lds, nullptr, nullptr, num_local, padded_local, num_chunks, gridDim.x - 1, counts,
                                            psum, offsets, num_rows, mailbox, sequence, &source);
    // (asked for here, needed only at the very end: the load travels while the routes are assigned)
    unsigned long long reporter_seen = threadIdx.x == 0 && !reporter ? load_word(reporter_tag) : 0ull;
    if (in_time) {
#pragma unroll
        for (int i = 0; i < kKeep; ++i)
            if (begin + i * kWave < end)
                assign_step(experts[i], begin + i * kWave + lane, end, lds.match[wave], lds.running[wave], route_to_row,
                            row_to_route);
    } else {
        // Some workgroup's histogram is missing: rows computed without it could lie anywhere.  No route gets a row
        // (and the counts above are all zero).
        for (int route = begin + lane; route < end; route += kWave) route_to_row[route] = -1;
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

int padded_experts(int num_local)
{
    int padded = 1;
    while (padded < num_local) padded <<= 1;
    return padded;
}

// Chunk length: as many chunks as the histogram budget allows (16..256), at least kMinChunk routes each.
int chunk_routes(int n_routes, int padded_local, int hist_ints = kHistInts)
{
    int max_chunks = hist_ints / padded_local;
    max_chunks = max_chunks > 256 ? 256 : (max_chunks < 16 ? 16 : max_chunks);
    int chunk = (n_routes + max_chunks - 1) / max_chunks;
    chunk = (chunk + kWave - 1) / kWave * kWave;
    return chunk < kMinChunk ? kMinChunk : chunk;
}

int check_layout_arguments(const void* idx, int num_tokens, int num_topk, int num_experts, int expert_begin, int num_local,
                           const int32_t* counts, const int32_t* psum, const int32_t* offsets, const int32_t* route_to_row,
                           const int32_t* row_to_route, const int32_t* num_rows)
{
    DPEP_REQUIRE(num_tokens >= 0 && num_topk >= 1 && num_topk <= DPEP_MAX_TOPK, "layout: bad T=%d K=%d", num_tokens,
                 num_topk);
    DPEP_REQUIRE(num_experts >= 1 && expert_begin >= 0 && num_local >= 1 && num_local <= DPEP_MAX_LOCAL_EXPERTS &&
                     expert_begin + num_local <= num_experts,
                 "layout: bad expert range E=%d begin=%d L=%d (at most %d local experts)", num_experts, expert_begin, num_local,
                 DPEP_MAX_LOCAL_EXPERTS);
    DPEP_REQUIRE(static_cast<long long>(num_tokens) * num_topk < (1ll << 31), "layout: T*K must fit int32");
    DPEP_REQUIRE(counts && psum && offsets && num_rows, "layout: NULL output");
    DPEP_REQUIRE(static_cast<long long>(num_tokens) * num_topk == 0 || (idx && route_to_row && row_to_route),
                 "layout: NULL routing buffer");
    return DPEP_OK;
}

// The two-launch form: count, then assign.  The count launch writes every histogram entry the assign launch reads, so
// the scratch needs no clearing and holds nothing between calls.
template <typename IdxT>
int enqueue_count_and_assign(const IdxT* idx, int n_routes, int num_experts, int expert_begin, int num_local, int padded, int chunk,
                             int num_chunks, int* wave_hist, int* block_hist, int32_t* counts, int32_t* psum, int32_t* offsets,
                             int32_t* num_rows, int32_t* route_to_row, int32_t* row_to_route, uint32_t* mailbox, uint32_t sequence,
                             hipStream_t stream)
{
    const int blocks = (num_chunks + kWaves - 1) / kWaves;
    if (blocks > 0) {
        hipLaunchKernelGGL(layout_count_kernel<IdxT>, dim3(blocks), dim3(kThreads), 0, stream, idx, n_routes, num_experts,
                           expert_begin, num_local, chunk, num_chunks, wave_hist, block_hist);
        if (int rc = launch_status("layout_count")) return rc;
    }
    // One workgroup more than there are chunks to assign: the reporter (with no routes, it alone publishes the
    // all-zero counts and prefix sums).
    hipLaunchKernelGGL(layout_assign_kernel<IdxT>, dim3(blocks + 1), dim3(kThreads), 0, stream, idx,
                       n_routes, num_experts, expert_begin, num_local, padded, chunk, num_chunks, wave_hist, block_hist, counts,
                       psum, offsets, num_rows, route_to_row, row_to_route, mailbox, sequence);
    return launch_status("layout_assign");
}

template <typename IdxT>
int launch_layout(void* ws, const IdxT* idx, int num_tokens, int num_topk, int num_experts, int expert_begin,
                  int num_local, int32_t* counts, int32_t* psum, int32_t* offsets, int32_t* route_to_row,
                  int32_t* row_to_route, int32_t* num_rows, bool report_to_host, hipStream_t stream)
{
    Workspace* w = as_workspace(ws);
    DPEP_REQUIRE(w != nullptr, "layout: not a live workspace");
    if (int rc = check_layout_arguments(idx, num_tokens, num_topk, num_experts, expert_begin, num_local, counts, psum, offsets,
                                        route_to_row, row_to_route, num_rows))
        return rc;
    const int n_routes = num_tokens * num_topk;
    const size_t need = dpep_layout_workspace_bytes(num_tokens, num_topk, num_local);
    DPEP_REQUIRE(need <= w->bytes, "layout: workspace too small (%zu needed, %zu available)", need, w->bytes);
    // A one-launch layout whose wait for the other workgroups' histograms ran out left its number in the mailbox.  If nobody has been told yet
    // (the launch reported to no host wait: MegaMoE's internal layout), this call is; either way the workspace
    // takes two launches from then on.
    if (const uint32_t timed_out = w->mailbox_host[kMailboxTimeout]; timed_out != w->timeout_seen) {
        w->timeout_seen = timed_out;
        w->layout_one_launch = 0;
        return fail(DPEP_ERUNTIME, "layout: an earlier layout kernel on this workspace ran out of time waiting for the "
                                   "other workgroups' histograms and reported no rows; layouts on this workspace take two launches from now on");
    }
    w->layout_launches = w->layout_launches == 0xffffffffu ? 1u : w->layout_launches + 1u;  // never 0
    const int padded = padded_experts(num_local);
    int chunk = chunk_routes(n_routes, padded);
    const bool one_launch = n_routes > 0 && chunk <= kKeep * kWave && w->layout_one_launch;
    // Inputs that take two launches anyway get shorter chunks (more waves at work), with the larger histograms the
    // workspace has room for: 131 072 routes over 256 local experts 16 -> 64 workgroups.
    int hist_ints = kHistInts;
    if (!one_launch) {
        hist_ints = kLargeHistInts;
        chunk = chunk_routes(n_routes, padded, kLargeHistInts);
    }
    const int num_chunks = (n_routes + chunk - 1) / chunk;
    int* wave_hist = static_cast<int*>(w->base);
    int* block_hist = wave_hist + hist_ints;
    const int blocks = (num_chunks + kWaves - 1) / kWaves;
    if (report_to_host) {
        w->sequence = w->sequence == 0xffffffffu ? 1u : w->sequence + 1u;  // never 0: that is "nothing launched"
        w->mailbox_local = num_local;
    }
    uint32_t* mailbox = report_to_host ? w->mailbox_device : nullptr;
    if (one_launch) {
        char* sync = static_cast<char*>(w->sync);
        hipLaunchKernelGGL(layout_fused_kernel<IdxT>, dim3(blocks + 1), dim3(kThreads), 0, stream, idx, n_routes, num_experts,
                           expert_begin, num_local, padded, chunk, num_chunks, counts, psum, offsets, num_rows, route_to_row,
                           row_to_route, mailbox, w->sequence, reinterpret_cast<unsigned long long*>(sync),
                           reinterpret_cast<unsigned long long*>(sync + kSyncTagged), blocks + w->exchange_extra_rows,
                           w->exchange_ticks, w->mailbox_device + kMailboxTimeout, w->layout_launches);
        return launch_status("layout_fused");
    }
    return enqueue_count_and_assign<IdxT>(idx, n_routes, num_experts, expert_begin, num_local, padded, chunk, num_chunks, wave_hist,
                                          block_hist, counts, psum, offsets, num_rows, route_to_row, row_to_route, mailbox,
                                          w->sequence, stream);
}

}  // namespace

// Shared with the MegaMoE forward, which routes on int32 ids.
int layout_i32(void* ws, const int32_t* idx, int num_tokens, int num_topk, int num_experts, int expert_begin,
               int num_local, int32_t* counts, int32_t* psum, int32_t* offsets, int32_t* route_to_row,
               int32_t* row_to_route, int32_t* num_rows, hipStream_t stream)
{
    return launch_layout<int32_t>(ws, idx, num_tokens, num_topk, num_experts, expert_begin, num_local, counts, psum,
                                  offsets, route_to_row, row_to_route, num_rows, /*report_to_host=*/false, stream);
}

}  // namespace dpep

// ---- the layout for callers that cannot allocate -------------------------------------------------------------
// Scratch of dpep_layout_static: the histograms a workspace would hold, in a device array of this library instead.
// Every GPU the library runs on has its own copy, at its own address, for the life of the process.
namespace dpep {
namespace {
constexpr size_t kStaticScratchInts = kHistInts + kBlockHistInts;  // 21 504 ints = 84 KiB
}
}
static __device__ __align__(256) int scratch[dpep::kStaticScratchInts];

namespace dpep {
namespace {

constexpr int kMaxDevices = 64;
int* g_scratch_of_device[kMaxDevices];  // device address of `scratch` on each GPU, looked up on first use
std::mutex g_scratch_mutex;

// The address of this GPU's copy of `scratch` (the current device's).  In host code the array's name is only a
// handle for the runtime, not a device address: kernels and memory calls get the looked-up pointer, never the name.
int scratch_of_current_device(int** out)
{
    int device = -1;
    DPEP_HIP(hipGetDevice(&device));
    DPEP_REQUIRE(device >= 0 && device < kMaxDevices, "layout_static: device %d outside [0, %d)", device, kMaxDevices);
    std::lock_guard<std::mutex> guard(g_scratch_mutex);
    if (g_scratch_of_device[device] == nullptr) {
        int* ptr = nullptr;
        DPEP_HIP(hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)));
        DPEP_REQUIRE(ptr != nullptr, "layout_static: the scratch array has no address on device %d", device);
        g_scratch_of_device[device] = ptr;
    }
    *out = g_scratch_of_device[device];
    return DPEP_OK;
}

}  // namespace
}  // namespace dpep

extern "C" {

size_t dpep_layout_workspace_bytes(int num_tokens, int num_topk, int num_local_experts)
{
    if (num_tokens < 0 || num_topk < 1 || num_local_experts < 1) return 0;
    return static_cast<size_t>(dpep::kLargeHistInts + dpep::kLargeBlockHistInts) * sizeof(int);
}

int dpep_layout(void* ws, const int64_t* topk_idx, int num_tokens, int num_topk, int num_experts, int expert_begin,
                int num_local, int32_t* counts, int32_t* psum, int32_t* offsets, int32_t* route_to_row,
                int32_t* row_to_route, int32_t* num_rows, void* stream)
{
    return dpep::launch_layout<int64_t>(ws, topk_idx, num_tokens, num_topk, num_experts, expert_begin, num_local,
                                        counts, psum, offsets, route_to_row, row_to_route, num_rows,
                                        /*report_to_host=*/true, static_cast<hipStream_t>(stream));
}

int dpep_layout_static(const int64_t* topk_idx, int num_tokens, int num_topk, int num_experts, int expert_begin,
                       int num_local, int32_t* counts, int32_t* psum, int32_t* offsets, int32_t* route_to_row,
                       int32_t* row_to_route, int32_t* num_rows, void* stream)
{
    using namespace dpep;
    if (int rc = check_layout_arguments(topk_idx, num_tokens, num_topk, num_experts, expert_begin, num_local, counts, psum,
                                        offsets, route_to_row, row_to_route, num_rows))
        return rc;
    const int n_routes = num_tokens * num_topk;
    const int padded = padded_experts(num_local);
    const int chunk = chunk_routes(n_routes, padded);
    const int num_chunks = (n_routes + chunk - 1) / chunk;
    const int blocks = (num_chunks + kWaves - 1) / kWaves;
    // what the two launches address: num_chunks rows of wave histograms, blocks rows of workgroup histograms
    DPEP_REQUIRE(static_cast<size_t>(num_chunks) * num_local <= static_cast<size_t>(kHistInts) &&
                     static_cast<size_t>(blocks) * num_local <= static_cast<size_t>(kBlockHistInts),
                 "layout_static: %d chunks x %d local experts exceed the static scratch of %zu bytes", num_chunks, num_local,
                 kStaticScratchInts * sizeof(int));
    int* base = nullptr;
    if (int rc = scratch_of_current_device(&base)) return rc;
    return enqueue_count_and_assign<int64_t>(topk_idx, n_routes, num_experts, expert_begin, num_local, padded, chunk, num_chunks,
                                             base, base + kHistInts, counts, psum, offsets, num_rows, route_to_row, row_to_route,
                                             /*mailbox=*/nullptr, 0u, static_cast<hipStream_t>(stream));
}

}  // extern "C"
