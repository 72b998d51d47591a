// Routing layout for one rank: per-expert counts, prefix sums and the stable expert-major
// permutation of the T*K routes (a stable counting sort), without atomics that would reorder rows.
//
// Observable contract (reference: tests/utils/reference.py:39-73, tests/clos/common.py:248-287,
// tests/elastic/test_dispatch.py:538-548): rows are ordered (local expert, token, slot); every valid
// slot gets its own row (duplicates included); invalid ids produce no row.
//
// Decomposition: the flat route stream is cut into chunks of kChunk routes, one wavefront each.
//   count  : each wave histograms its chunk              -> hist[chunk][expert]
//   scan   : one workgroup turns hist into exclusive bases (over chunks, then over experts)
//   assign : each wave replays its chunk in order; the rank of a route among equal experts inside a
//            64-route step comes from ballot/popcount, the carry between steps lives in LDS.
#include "common.h"

namespace dpep {
namespace {

constexpr int kChunk = 256;        // routes per wavefront
constexpr int kWavesPerBlock = 4;  // wavefronts per workgroup in count/assign
constexpr int kScanThreads = 1024;

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
__device__ __forceinline__ int local_expert(const IdxT* __restrict__ idx, int route, int n_routes, int num_experts,
                                            int expert_begin, int num_local)
{
    if (route >= n_routes) return -1;
    const long long e = static_cast<long long>(idx[route]);
    if (e < 0 || e >= num_experts) return -1;
    const long long local = e - expert_begin;
    return (local >= 0 && local < num_local) ? static_cast<int>(local) : -1;
}

template <typename IdxT>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void layout_count_kernel(
    const IdxT* __restrict__ idx, int n_routes, int num_experts, int expert_begin, int num_local, int nbits,
    int num_chunks, int* __restrict__ hist)
{
    extern __shared__ int lds[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int chunk = blockIdx.x * kWavesPerBlock + wave;
    int* mine = lds + wave * num_local;
    for (int e = lane; e < num_local; e += kWave) mine[e] = 0;
    __builtin_amdgcn_wave_barrier();
    if (chunk >= num_chunks) return;
    const int begin = chunk * kChunk;
    for (int step = 0; step < kChunk; step += kWave) {
        const int e = local_expert(idx, begin + step + lane, n_routes, num_experts, expert_begin, num_local);
        const uint64_t mask = match_expert(e, e >= 0, nbits);
        if (e >= 0 && (mask & lanes_below()) == 0) mine[e] += __popcll(mask);
        __builtin_amdgcn_wave_barrier();
    }
    int* out = hist + static_cast<size_t>(chunk) * num_local;
    for (int e = lane; e < num_local; e += kWave) out[e] = mine[e];
}

// hist[chunk][e] (counts) -> exclusive base of chunk `chunk` for expert e, including the expert's
// own offset; also emits counts / psum / offsets / num_rows.
__global__ __launch_bounds__(kScanThreads) void layout_scan_kernel(int* __restrict__ hist, int num_chunks,
                                                                   int num_local, int ex, int* __restrict__ counts,
                                                                   int* __restrict__ psum, int* __restrict__ offsets,
                                                                   int* __restrict__ num_rows)
{
    __shared__ int partial[kScanThreads];
    __shared__ int scan_a[DPEP_MAX_LOCAL_EXPERTS];
    __shared__ int scan_b[DPEP_MAX_LOCAL_EXPERTS];
    const int tid = threadIdx.x;
    const int parts = kScanThreads / ex;
    const int p = tid / ex, e = tid % ex;
    const int per_part = (num_chunks + parts - 1) / parts;
    const int g0 = min(p * per_part, num_chunks), g1 = min(g0 + per_part, num_chunks);
    int sum = 0;
    if (e < num_local)
        for (int g = g0; g < g1; ++g) sum += hist[static_cast<size_t>(g) * num_local + e];
    partial[tid] = sum;
    __syncthreads();
    int before = 0;
    for (int q = 0; q < p; ++q) before += partial[q * ex + e];
    if (p == parts - 1 && e < num_local) scan_a[e] = before + sum;  // total rows of expert e
    __syncthreads();
    // Inclusive Hillis-Steele scan over experts (num_local <= 1024 == blockDim).
    int* src = scan_a;
    int* dst = scan_b;
    for (int stride = 1; stride < num_local; stride <<= 1) {
        if (tid < num_local) dst[tid] = src[tid] + (tid >= stride ? src[tid - stride] : 0);
        __syncthreads();
        int* t = src;
        src = dst;
        dst = t;
    }
    if (tid < num_local) {
        const int incl = src[tid];
        const int total = incl - (tid > 0 ? src[tid - 1] : 0);
        counts[tid] = total;
        psum[tid] = incl;
        offsets[tid + 1] = incl;
        if (tid == 0) offsets[0] = 0;
        if (tid == num_local - 1) num_rows[0] = incl;
    }
    if (e < num_local) {
        int running = before + (e > 0 ? src[e - 1] : 0);
        for (int g = g0; g < g1; ++g) {
            const size_t at = static_cast<size_t>(g) * num_local + e;
            const int v = hist[at];
            hist[at] = running;
            running += v;
        }
    }
}

template <typename IdxT>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void layout_assign_kernel(
    const IdxT* __restrict__ idx, int n_routes, int num_experts, int expert_begin, int num_local, int nbits,
    int num_chunks, const int* __restrict__ base, int* __restrict__ route_to_row, int* __restrict__ row_to_route)
{
    extern __shared__ int lds[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int chunk = blockIdx.x * kWavesPerBlock + wave;
    if (chunk >= num_chunks) return;
    int* running = lds + wave * num_local;
    const int* mine = base + static_cast<size_t>(chunk) * num_local;
    for (int e = lane; e < num_local; e += kWave) running[e] = mine[e];
    __builtin_amdgcn_wave_barrier();
    const int begin = chunk * kChunk;
    for (int step = 0; step < kChunk; step += kWave) {
        const int route = begin + step + lane;
        const int e = local_expert(idx, route, n_routes, num_experts, expert_begin, num_local);
        const uint64_t mask = match_expert(e, e >= 0, nbits);
        const int ahead = __popcll(mask & lanes_below());
        int row = -1;
        if (e >= 0) row = running[e] + ahead;
        __builtin_amdgcn_wave_barrier();
        if (e >= 0 && ahead == 0) running[e] = row + __popcll(mask);
        __builtin_amdgcn_wave_barrier();
        if (route < n_routes) {
            route_to_row[route] = row;
            if (row >= 0) row_to_route[row] = route;
        }
    }
}

template <typename IdxT>
int launch_layout(void* ws, const IdxT* idx, int num_tokens, int num_topk, int num_experts, int expert_begin,
                  int num_local, int32_t* counts, int32_t* psum, int32_t* offsets, int32_t* route_to_row,
                  int32_t* row_to_route, int32_t* num_rows, hipStream_t stream)
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
    const int num_chunks = (n_routes + kChunk - 1) / kChunk;
    int nbits = 0;
    while ((1 << nbits) < num_local) ++nbits;
    int ex = 1;
    while (ex < num_local) ex <<= 1;
    int* hist = static_cast<int*>(w->base);
    const int blocks = (num_chunks + kWavesPerBlock - 1) / kWavesPerBlock;
    const size_t lds = static_cast<size_t>(kWavesPerBlock) * num_local * sizeof(int);
    if (blocks > 0) {
        hipLaunchKernelGGL(layout_count_kernel<IdxT>, dim3(blocks), dim3(kWavesPerBlock * kWave), lds, stream, idx,
                           n_routes, num_experts, expert_begin, num_local, nbits, num_chunks, hist);
        if (int rc = launch_status("layout_count")) return rc;
    }
    hipLaunchKernelGGL(layout_scan_kernel, dim3(1), dim3(kScanThreads), 0, stream, hist, num_chunks, num_local, ex,
                       counts, psum, offsets, num_rows);
    if (int rc = launch_status("layout_scan")) return rc;
    if (blocks > 0) {
        hipLaunchKernelGGL(layout_assign_kernel<IdxT>, dim3(blocks), dim3(kWavesPerBlock * kWave), lds, stream, idx,
                           n_routes, num_experts, expert_begin, num_local, nbits, num_chunks, hist, route_to_row,
                           row_to_route);
        if (int rc = launch_status("layout_assign")) return rc;
    }
    return DPEP_OK;
}

}  // namespace

// Shared with the MegaMoE forward, which routes on int32 ids.
int layout_i32(void* ws, const int32_t* idx, int num_tokens, int num_topk, int num_experts, int expert_begin,
               int num_local, int32_t* counts, int32_t* psum, int32_t* offsets, int32_t* route_to_row,
               int32_t* row_to_route, int32_t* num_rows, hipStream_t stream)
{
    return launch_layout<int32_t>(ws, idx, num_tokens, num_topk, num_experts, expert_begin, num_local, counts, psum,
                                  offsets, route_to_row, row_to_route, num_rows, stream);
}

}  // namespace dpep

extern "C" {

size_t dpep_layout_workspace_bytes(int num_tokens, int num_topk, int num_local_experts)
{
    if (num_tokens < 0 || num_topk < 1 || num_local_experts < 1) return 0;
    const size_t routes = static_cast<size_t>(num_tokens) * num_topk;
    const size_t chunks = (routes + dpep::kChunk - 1) / dpep::kChunk;
    const size_t bytes = (chunks > 0 ? chunks : 1) * num_local_experts * sizeof(int);
    return (bytes + 255) / 256 * 256;
}

int dpep_layout(void* ws, const int64_t* topk_idx, int num_tokens, int num_topk, int num_experts, int expert_begin,
                int num_local, int32_t* counts, int32_t* psum, int32_t* offsets, int32_t* route_to_row,
                int32_t* row_to_route, int32_t* num_rows, void* stream)
{
    return dpep::launch_layout<int64_t>(ws, topk_idx, num_tokens, num_topk, num_experts, expert_begin, num_local,
                                        counts, psum, offsets, route_to_row, row_to_route, num_rows,
                                        static_cast<hipStream_t>(stream));
}

}  // extern "C"
