// Routing layout for one rank: per-expert counts, prefix sums and the stable expert-major
// permutation of the T*K routes (a stable counting sort), without atomics that would reorder rows.
//
// Observable contract (reference: tests/utils/reference.py:39-73, tests/clos/common.py:248-287,
// tests/elastic/test_dispatch.py:538-548): rows are ordered (local expert, token, slot); every valid
// slot gets its own row (duplicates included); invalid ids produce no row.
//
// Decomposition: the flat route stream is cut into chunks, one wavefront each, four per workgroup.
//   count  : each wave histograms its chunk                    -> hist[chunk][expert]   (<= 64 KiB, L2-resident)
//   assign : each workgroup sums the histogram columns (all chunks -> expert totals and their exclusive
//            scan; chunks before each of its waves -> that wave's base), then every wave replays its
//            chunk in order.  The rank of a route among equal experts inside a 64-route step comes from
//            ballot/popcount, the carry between steps lives in LDS.  There is no separate scan launch.
#include "common.h"

namespace dpep {
namespace {

constexpr int kWaves = 4;             // wavefronts (= chunks) per workgroup
constexpr int kThreads = kWaves * kWave;
constexpr int kHistInts = 16384;      // chunks * padded experts never exceeds this
constexpr int kMinChunk = 256;        // routes per wavefront, lower bound (multiple of 64)
constexpr int kPrefetch = 8;          // 64-route steps whose ids are fetched before the ordered replay
constexpr int kColumnBatch = 16;      // histogram loads in flight per thread

__device__ __forceinline__ uint64_t lanes_below()
{
    return (1ull << (threadIdx.x & 63)) - 1ull;
}

// Mask of lanes in this wave whose (valid) expert equals mine.  nbits = bits needed for L-1.
__device__ __forceinline__ uint64_t match_expert(int e, bool valid, int nbits)
{
    uint64_t mask = __ballot(valid);
    for (int b = 0; b < nbits; ++b) {
        const bool bit = (e >> b) & 1;
        const uint64_t vote = __ballot(valid && bit);
        mask &= bit ? vote : ~vote;
    }
    return valid ? mask : 0ull;
}

template <typename IdxT>
__device__ __forceinline__ int local_expert(const IdxT* __restrict__ idx, int route, int end, int num_experts,
                                            int expert_begin, int num_local)
{
    if (route >= end) return -1;
    const long long e = static_cast<long long>(idx[route]);
    if (e < 0 || e >= num_experts) return -1;
    const long long local = e - expert_begin;
    return (local >= 0 && local < num_local) ? static_cast<int>(local) : -1;
}

template <typename IdxT>
__global__ __launch_bounds__(kThreads) void layout_count_kernel(const IdxT* __restrict__ idx, int n_routes,
                                                                int num_experts, int expert_begin, int num_local,
                                                                int nbits, int chunk, int num_chunks,
                                                                int* __restrict__ hist)
{
    extern __shared__ int lds[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int g = blockIdx.x * kWaves + wave;
    if (g >= num_chunks) return;
    int* mine = lds + wave * num_local;
    for (int e = lane; e < num_local; e += kWave) mine[e] = 0;
    __builtin_amdgcn_wave_barrier();
    const int begin = g * chunk;
    const int end = min(begin + chunk, n_routes);
    for (int base = begin; base < end; base += kPrefetch * kWave) {
        int experts[kPrefetch];
#pragma unroll
        for (int i = 0; i < kPrefetch; ++i)
            experts[i] = local_expert(idx, base + i * kWave + lane, end, num_experts, expert_begin, num_local);
#pragma unroll
        for (int i = 0; i < kPrefetch; ++i) {
            const int e = experts[i];
            const uint64_t mask = match_expert(e, e >= 0, nbits);
            if (e >= 0 && (mask & lanes_below()) == 0) mine[e] += __popcll(mask);
            __builtin_amdgcn_wave_barrier();
        }
    }
    int* out = hist + static_cast<size_t>(g) * num_local;
    for (int e = lane; e < num_local; e += kWave) out[e] = mine[e];
}

// Column sums of hist for one expert over the chunks {first, first+stride, ...}: the total, and for
// each wave w of this workgroup the part that lies in chunks before chunk0 + w.
struct ColumnSums {
    int total;
    int before[kWaves];
};

__device__ __forceinline__ ColumnSums column_sums(const int* __restrict__ hist, int num_local, int e, int first,
                                                  int stride, int num_chunks, int chunk0)
{
    ColumnSums sums;
    sums.total = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) sums.before[w] = 0;
    for (int c0 = first; c0 < num_chunks; c0 += kColumnBatch * stride) {
        int v[kColumnBatch];
#pragma unroll
        for (int j = 0; j < kColumnBatch; ++j) {
            const int c = c0 + j * stride;
            v[j] = c < num_chunks ? hist[static_cast<size_t>(c) * num_local + e] : 0;
        }
#pragma unroll
        for (int j = 0; j < kColumnBatch; ++j) {
            const int c = c0 + j * stride;
            sums.total += v[j];
#pragma unroll
            for (int w = 0; w < kWaves; ++w) sums.before[w] += c < chunk0 + w ? v[j] : 0;
        }
    }
    return sums;
}

template <typename IdxT>
__global__ __launch_bounds__(kThreads) void layout_assign_kernel(
    const IdxT* __restrict__ idx, int n_routes, int num_experts, int expert_begin, int num_local, int padded_local,
    int nbits, int chunk, int num_chunks, const int* __restrict__ hist, int* __restrict__ counts,
    int* __restrict__ psum, int* __restrict__ offsets, int* __restrict__ num_rows, int* __restrict__ route_to_row,
    int* __restrict__ row_to_route, uint32_t* __restrict__ mailbox, uint32_t sequence)
{
    // totals[e]: rows of expert e (later its exclusive offset); running[w][e]: next row of expert e for wave w.
    __shared__ int totals[DPEP_MAX_LOCAL_EXPERTS];
    __shared__ int running[kWaves][DPEP_MAX_LOCAL_EXPERTS];
    __shared__ int partial[kThreads * (kWaves + 1)];
    __shared__ int wave_sums[kWaves];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int chunk0 = blockIdx.x * kWaves;

    if (padded_local >= kThreads) {
        for (int e = tid; e < num_local; e += kThreads) {
            const ColumnSums sums = column_sums(hist, num_local, e, 0, 1, num_chunks, chunk0);
            totals[e] = sums.total;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) running[w][e] = sums.before[w];
        }
    } else {
        // Few experts: split the chunks over `parts` thread groups (at most 16), then reduce through LDS.
        int parts = kThreads / padded_local;
        if (parts > 16) parts = 16;
        const int p = tid / padded_local, e = tid % padded_local;
        const bool active = p < parts && e < num_local;
        if (active) {
            const ColumnSums sums = column_sums(hist, num_local, e, p, parts, num_chunks, chunk0);
            partial[tid * (kWaves + 1)] = sums.total;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) partial[tid * (kWaves + 1) + 1 + w] = sums.before[w];
        }
        __syncthreads();
        if (tid < num_local) {
            int total = 0, before[kWaves] = {0, 0, 0, 0};
            for (int q = 0; q < parts; ++q) {
                const int* src = partial + (q * padded_local + tid) * (kWaves + 1);
                total += src[0];
#pragma unroll
                for (int w = 0; w < kWaves; ++w) before[w] += src[1 + w];
            }
            totals[tid] = total;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) running[w][tid] = before[w];
        }
    }
    __syncthreads();

    // Exclusive scan of totals over experts: four consecutive experts per thread, then a workgroup scan.
    int mine[4], local_sum = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = tid * 4 + j;
        mine[j] = e < num_local ? totals[e] : 0;
        local_sum += mine[j];
    }
    int incl = local_sum;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int up = __shfl_up(incl, d);
        if (lane >= d) incl += up;
    }
    if (lane == kWave - 1) wave_sums[wave] = incl;
    __syncthreads();
    int offset = incl - local_sum;
    for (int w = 0; w < wave; ++w) offset += wave_sums[w];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = tid * 4 + j;
        if (e < num_local) {
#pragma unroll
            for (int w = 0; w < kWaves; ++w) running[w][e] += offset;
            if (blockIdx.x == 0) {
                counts[e] = mine[j];
                if (mailbox != nullptr) mailbox[2 + e] = static_cast<uint32_t>(mine[j]);  // pinned host memory
                psum[e] = offset + mine[j];
                offsets[e + 1] = offset + mine[j];
            }
        }
        offset += mine[j];
    }
    if (blockIdx.x == 0 && tid == kThreads - 1) {
        offsets[0] = 0;
        num_rows[0] = offset;
    }
    // The host polls the mailbox's sequence word: publish it (with the row count, one 8-byte store) after
    // every per-expert count of this workgroup has reached host memory.
    if (blockIdx.x == 0 && mailbox != nullptr) __threadfence_system();
    __syncthreads();
    if (blockIdx.x == 0 && mailbox != nullptr && tid == kThreads - 1) {
        const unsigned long long word = (static_cast<unsigned long long>(sequence) << 32) | static_cast<uint32_t>(offset);
        __hip_atomic_store(reinterpret_cast<unsigned long long*>(mailbox), word, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }

    const int g = chunk0 + wave;
    if (g >= num_chunks) return;
    int* next_row = running[wave];
    const int begin = g * chunk;
    const int end = min(begin + chunk, n_routes);
    for (int base = begin; base < end; base += kPrefetch * kWave) {
        int experts[kPrefetch];
#pragma unroll
        for (int i = 0; i < kPrefetch; ++i)
            experts[i] = local_expert(idx, base + i * kWave + lane, end, num_experts, expert_begin, num_local);
#pragma unroll
        for (int i = 0; i < kPrefetch; ++i) {
            const int route = base + i * kWave + lane;
            const int e = experts[i];
            const uint64_t mask = match_expert(e, e >= 0, nbits);
            const int ahead = __popcll(mask & lanes_below());
            int row = -1;
            if (e >= 0) row = next_row[e] + ahead;
            __builtin_amdgcn_wave_barrier();
            if (e >= 0 && ahead == 0) next_row[e] = row + __popcll(mask);
            __builtin_amdgcn_wave_barrier();
            if (route < end) {
                route_to_row[route] = row;
                if (row >= 0) row_to_route[row] = route;
            }
        }
    }
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

template <typename IdxT>
int launch_layout(void* ws, const IdxT* idx, int num_tokens, int num_topk, int num_experts, int expert_begin,
                  int num_local, int32_t* counts, int32_t* psum, int32_t* offsets, int32_t* route_to_row,
                  int32_t* row_to_route, int32_t* num_rows, bool report_to_host, hipStream_t stream)
{
    Workspace* w = as_workspace(ws);
    DPEP_REQUIRE(w != nullptr, "layout: not a live workspace");
    DPEP_REQUIRE(num_tokens >= 0 && num_topk >= 1 && num_topk <= DPEP_MAX_TOPK, "layout: bad T=%d K=%d", num_tokens,
                 num_topk);
    DPEP_REQUIRE(num_experts >= 1 && expert_begin >= 0 && num_local >= 1 && num_local <= DPEP_MAX_LOCAL_EXPERTS &&
                     expert_begin + num_local <= num_experts,
                 "layout: bad expert range E=%d begin=%d L=%d", num_experts, expert_begin, num_local);
    DPEP_REQUIRE(static_cast<long long>(num_tokens) * num_topk < (1ll << 31), "layout: T*K must fit int32");
    DPEP_REQUIRE(counts && psum && offsets && num_rows, "layout: NULL output");
    const int n_routes = num_tokens * num_topk;
    DPEP_REQUIRE(n_routes == 0 || (idx && route_to_row && row_to_route), "layout: NULL routing buffer");
    const size_t need = dpep_layout_workspace_bytes(num_tokens, num_topk, num_local);
    DPEP_REQUIRE(need <= w->bytes, "layout: workspace too small (%zu needed, %zu available)", need, w->bytes);
    const int padded = padded_experts(num_local);
    const int chunk = chunk_routes(n_routes, padded);
    const int num_chunks = (n_routes + chunk - 1) / chunk;
    int nbits = 0;
    while ((1 << nbits) < num_local) ++nbits;
    int* hist = static_cast<int*>(w->base);
    const int blocks = (num_chunks + kWaves - 1) / kWaves;
    if (blocks > 0) {
        hipLaunchKernelGGL(layout_count_kernel<IdxT>, dim3(blocks), dim3(kThreads),
                           static_cast<size_t>(kWaves) * num_local * sizeof(int), stream, idx, n_routes, num_experts,
                           expert_begin, num_local, nbits, chunk, num_chunks, hist);
        if (int rc = launch_status("layout_count")) return rc;
    }
    // With no routes one workgroup still publishes the all-zero counts and prefix sums.
    if (report_to_host) {
        w->sequence = w->sequence == 0xffffffffu ? 1u : w->sequence + 1u;  // never 0: that is "nothing launched"
        w->mailbox_local = num_local;
    }
    hipLaunchKernelGGL(layout_assign_kernel<IdxT>, dim3(blocks > 0 ? blocks : 1), dim3(kThreads), 0, stream, idx,
                       n_routes, num_experts, expert_begin, num_local, padded, nbits, chunk, num_chunks, hist, counts,
                       psum, offsets, num_rows, route_to_row, row_to_route, report_to_host ? w->mailbox_device : nullptr,
                       w->sequence);
    return launch_status("layout_assign");
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

extern "C" {

size_t dpep_layout_workspace_bytes(int num_tokens, int num_topk, int num_local_experts)
{
    if (num_tokens < 0 || num_topk < 1 || num_local_experts < 1) return 0;
    return static_cast<size_t>(dpep::kHistInts) * sizeof(int);
}

int dpep_layout(void* ws, const int64_t* topk_idx, int num_tokens, int num_topk, int num_experts, int expert_begin,
                int num_local, int32_t* counts, int32_t* psum, int32_t* offsets, int32_t* route_to_row,
                int32_t* row_to_route, int32_t* num_rows, void* stream)
{
    return dpep::launch_layout<int64_t>(ws, topk_idx, num_tokens, num_topk, num_experts, expert_begin, num_local,
                                        counts, psum, offsets, route_to_row, row_to_route, num_rows,
                                        /*report_to_host=*/true, static_cast<hipStream_t>(stream));
}

}  // extern "C"
