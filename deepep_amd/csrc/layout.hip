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

#include "layout_device.h"

namespace dpep {
namespace {

using namespace layout_device;

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
    layout_fused_body<false>(lds, static_cast<int>(gridDim.x), idx, n_routes, num_experts, expert_begin, num_local, padded_local, chunk, num_chunks, counts, psum, offsets, num_rows, route_to_row, row_to_route, mailbox, sequence, epoch, tagged, rows, limit_ticks, timeouts, launch_id);
}

int padded_experts(int num_local)
{
    int padded = 1;
    while (padded < num_local) padded <<= 1;
    return padded;
}

// Chunk length: as many chunks as the histogram budget allows (16..256), at least kMinChunk routes each.
int chunk_routes(int n_routes, int padded_local)
{
    int max_chunks = kHistInts / padded_local;
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
    const int chunk = chunk_routes(n_routes, padded);
    const int num_chunks = (n_routes + chunk - 1) / chunk;
    int* wave_hist = static_cast<int*>(w->base);
    int* block_hist = wave_hist + kHistInts;
    const int blocks = (num_chunks + kWaves - 1) / kWaves;
    if (report_to_host) {
        w->sequence = w->sequence == 0xffffffffu ? 1u : w->sequence + 1u;  // never 0: that is "nothing launched"
        w->mailbox_local = num_local;
    }
    uint32_t* mailbox = report_to_host ? w->mailbox_device : nullptr;
    if (blocks > 0 && chunk <= kKeep * kWave && w->layout_one_launch) {
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
    return static_cast<size_t>(dpep::kHistInts + dpep::kBlockHistInts) * sizeof(int);
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
