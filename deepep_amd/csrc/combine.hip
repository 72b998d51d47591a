// Combine: every token gathers its expert rows and reduces them in fp32, in slot order, with an
// optional per-row weight, then rounds once to BF16.  A token (column part) is owned by exactly one
// workgroup, so there are no atomics and the summation order is fixed.
//
// Operation order follows the reference's aggregate kernel
// (csrc/direct/kernels/aggregate/aggregate_impl.h:166-226): acc = +0; per valid slot
// tmp = float(y); tmp = tmp * w; acc = acc + tmp (separate multiply and add); final cast RNE.
// Unweighted form: tests/elastic/test_combine.py:504-515; weighted form:
// tests/elastic/test_ep_low_latency.py:449-463; weight-return channel: docs/elastic.md:71.
#include "common.h"

#pragma clang fp contract(off)

namespace dpep {
namespace {

constexpr int kMaxThreads = 256;
constexpr int kDenseTargetBlocks = 1000000;  // dense routing: always split the token rows
constexpr int kDenseVec = 64;                // ... into parts of 64 16-byte vectors
constexpr int kSparseTargetBlocks = 2048;    // sparse shares: a workgroup per token while that fills the chip
constexpr int kBatch = 8;  // rows fetched per thread before the dependent adds start

// kWeights: 0 = plain sum, 1 = weight per expert row (w[row]), 2 = weight per route (w[t*K + s]).
// kHalf: rows and output are IEEE half instead of BF16.
template <int kWeights, bool kHalf = false>
__global__ __launch_bounds__(kMaxThreads) void combine_kernel(
    const u32x4* __restrict__ y, const float* __restrict__ row_weights, const int* __restrict__ route_to_row,
    int num_topk, int vec_per_row, int vec_per_part, int parts, u32x4* __restrict__ out,
    const float* __restrict__ return_in, float* __restrict__ return_out, const int* __restrict__ shared_first_row,
    int num_shared, int num_tokens, const int* __restrict__ fill_state, int num_rows, int leave_unserved)
{
    __shared__ int rows[DPEP_MAX_TOPK + kBatch];
    __shared__ float wts[DPEP_MAX_TOPK + kBatch];
    const int token = blockIdx.x / parts, part = blockIdx.x % parts;
    if (threadIdx.x < DPEP_MAX_TOPK + kBatch) {
        int row = -1;
        if (threadIdx.x < num_topk) row = route_to_row[static_cast<size_t>(token) * num_topk + threadIdx.x];
        if (row >= num_rows) row = -1;  // a row the caller's y does not hold (capacity layouts drop surplus rows)
        rows[threadIdx.x] = row;
        if (kWeights == 1) wts[threadIdx.x] = row >= 0 ? row_weights[row] : 0.0f;
        if (kWeights == 2)
            wts[threadIdx.x] = row >= 0 ? row_weights[static_cast<size_t>(token) * num_topk + threadIdx.x] : 0.0f;
        if (part == 0 && return_out != nullptr && threadIdx.x < num_topk)
            return_out[static_cast<size_t>(token) * num_topk + threadIdx.x] = row >= 0 ? return_in[row] : 0.0f;
        // Shared experts (MegaMoE): slot K + j is row first + j * B + token with weight 1, summed after the routes.
        if (kWeights == 2 && threadIdx.x >= num_topk && threadIdx.x < num_topk + num_shared) {
            rows[threadIdx.x] = shared_first_row[0] + (threadIdx.x - num_topk) * num_tokens + token;
            wts[threadIdx.x] = 1.0f;
        }
    }
    const int num_slots = num_topk + (kWeights == 2 ? num_shared : 0);
    // Tokens without any row (the common case of a sparse receive share) are plain zero fill.  Streaming
    // stores: cached ones would push the rows read next, and the caller's other data, out of the caches.
    const bool any_row = __syncthreads_or(threadIdx.x < num_slots && rows[threadIdx.x] >= 0) != 0;
    const int v_begin = part * vec_per_part;
    const int v_end = min(v_begin + vec_per_part, vec_per_row);
    if (!any_row) {
        if (leave_unserved) return;  // the caller wants only the tokens that own a row written
        // (MegaMoE) rows that idle workgroups of the first GEMM have already zeroed: filler f of n took tokens
        // f, f + n, ... and got through fill_state[1 + f] of them
        if (kWeights == 2 && fill_state != nullptr) {
            const int fillers = fill_state[0];
            if (fillers > 0 && token / fillers < fill_state[1 + token % fillers]) return;
        }
        const u32x4 zero = {0u, 0u, 0u, 0u};
        for (int v = v_begin + threadIdx.x; v < v_end; v += blockDim.x)
            store16_nt(out + static_cast<size_t>(token) * vec_per_row + v, zero);
        return;
    }
    for (int v = v_begin + threadIdx.x; v < v_end; v += blockDim.x) {
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
        for (int s0 = 0; s0 < num_slots; s0 += kBatch) {
            u32x4 val[kBatch];
#pragma unroll
            for (int j = 0; j < kBatch; ++j) {
                const int row = rows[s0 + j];
                if (row >= 0) val[j] = load16_nt(y + static_cast<size_t>(row) * vec_per_row + v);
            }
#pragma unroll
            for (int j = 0; j < kBatch; ++j) {
                if (rows[s0 + j] < 0) continue;
                const float w = kWeights != 0 ? wts[s0 + j] : 1.0f;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float lo = kHalf ? f16_to_f32(val[j][i] & 0xffffu) : bf16_to_f32(val[j][i] & 0xffffu);
                    float hi = kHalf ? f16_to_f32(val[j][i] >> 16) : bf16_to_f32(val[j][i] >> 16);
                    if (kWeights != 0) {
                        lo = __fmul_rn(lo, w);
                        hi = __fmul_rn(hi, w);
                    }
                    acc[2 * i] = __fadd_rn(acc[2 * i], lo);
                    acc[2 * i + 1] = __fadd_rn(acc[2 * i + 1], hi);
                }
            }
        }
        u32x4 packed;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            packed[i] = kHalf ? pack_f16x2(acc[2 * i], acc[2 * i + 1]) : pack_bf16x2(acc[2 * i], acc[2 * i + 1]);
        store16_through(out + static_cast<size_t>(token) * vec_per_row + v, packed);
    }
}

// One wave reduces the 16-byte vectors [vec_begin, vec_end) of one token: lane s holds the row and weight of the
// token's slot s (row < 0: no row), valid = the lanes that hold a row; rows are row_stride vectors apart.  Slots ascending, separate fp32 multiply and add, one
// rounding to BF16.  kSparseBatch = 16-byte vectors per lane in flight per slot.
template <int kWeights, bool kCached, int kSparseBatch>
__device__ __forceinline__ void reduce_token_rows(const u32x4* __restrict__ y, int row, float weight, uint64_t valid,
                                                  int row_stride, int vec_begin, int vec_end, u32x4* __restrict__ dst, int lane)
{
    for (int v0 = vec_begin; v0 < vec_end; v0 += 64 * kSparseBatch) {
        float acc[kSparseBatch][8];
#pragma unroll
        for (int b = 0; b < kSparseBatch; ++b)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[b][i] = 0.0f;
        for (uint64_t rest = valid; rest != 0ull; rest &= rest - 1ull) {
            const int slot = __builtin_ctzll(rest);
            const int r = __builtin_amdgcn_readlane(row, slot);
            const float w = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, weight), slot));
            const u32x4* src = y + static_cast<size_t>(r) * row_stride;
            u32x4 val[kSparseBatch];
#pragma unroll
            for (int b = 0; b < kSparseBatch; ++b) {
                const int v = v0 + b * 64 + lane;
                if (v < vec_end) val[b] = kCached ? load16(src + v) : load16_nt(src + v);
            }
#pragma unroll
            for (int b = 0; b < kSparseBatch; ++b) {
                if (v0 + b * 64 + lane >= vec_end) continue;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float lo = bf16_to_f32(val[b][i] & 0xffffu);
                    float hi = bf16_to_f32(val[b][i] >> 16);
                    if (kWeights != 0) {
                        lo = __fmul_rn(lo, w);
                        hi = __fmul_rn(hi, w);
                    }
                    acc[b][2 * i] = __fadd_rn(acc[b][2 * i], lo);
                    acc[b][2 * i + 1] = __fadd_rn(acc[b][2 * i + 1], hi);
                }
            }
        }
#pragma unroll
        for (int b = 0; b < kSparseBatch; ++b) {
            const int v = v0 + b * 64 + lane;
            if (v >= vec_end) continue;
            u32x4 packed;
#pragma unroll
            for (int i = 0; i < 4; ++i) packed[i] = pack_bf16x2(acc[b][2 * i], acc[b][2 * i + 1]);
            store16_nt(dst + v, packed);
        }
    }
}

// The reduce for sparse shares (most tokens own no row, none owns a shared expert's): one WAVE per token, so that a
// token without rows costs one short-lived wave instead of a workgroup with a barrier, and four times as many tokens
// are in flight per CU (the kernel above spends its time on the chain of dependent loads each of its workgroups
// starts with).  Same arithmetic in the same order as combine_kernel: slots ascending, separate fp32 multiply and
// add (no multiply at all without weights), one RNE rounding to BF16.  kWeights as above; kCached: the rows were
// written by the kernel right before this one (the second GEMM) and are read through the caches.
constexpr int kSparseWaves = 4;  // tokens (= waves) per workgroup
template <int kWeights, bool kCached>
__global__ __launch_bounds__(64 * kSparseWaves) void combine_sparse_kernel(
    const u32x4* __restrict__ y, const float* __restrict__ weights, const int* __restrict__ route_to_row, int num_topk,
    int vec_per_row, u32x4* __restrict__ out, int num_tokens, const int* __restrict__ fill_state,
    const float* __restrict__ return_in, float* __restrict__ return_out, int num_rows)
{
    const int lane = threadIdx.x & 63;
    const int token = blockIdx.x * kSparseWaves + (threadIdx.x >> 6);
    if (token >= num_tokens) return;
    int row = -1;
    float weight = 0.0f;
    if (lane < num_topk) {
        const size_t route = static_cast<size_t>(token) * num_topk + lane;
        row = route_to_row[route];
        if (row >= num_rows) row = -1;  // a row the caller's y does not hold
        if (kWeights == 1) weight = row >= 0 ? weights[row] : 0.0f;
        if (kWeights == 2) weight = weights[route];
        if (return_out != nullptr) return_out[route] = row >= 0 ? return_in[row] : 0.0f;
    }
    const uint64_t valid = __ballot(row >= 0);
    u32x4* dst = out + static_cast<size_t>(token) * vec_per_row;
    if (valid == 0ull) {
        if (fill_state != nullptr) {  // rows that idle workgroups of the first GEMM have already zeroed
            const int fillers = fill_state[0];
            if (fillers > 0 && token / fillers < fill_state[1 + token % fillers]) return;
        }
        const u32x4 zero = {0u, 0u, 0u, 0u};
        for (int v = lane; v < vec_per_row; v += 64) store16_nt(dst + v, zero);
        return;
    }
    reduce_token_rows<kWeights, kCached, 8>(y, row, weight, valid, vec_per_row, 0, vec_per_row, dst, lane);
}

// Sparse shares whose unserved tokens are left alone (one rank's part of an EP job: the rows of tokens it does not
// serve belong to other ranks).  A workgroup takes 64 / top-k consecutive tokens: every wave loads their (at most 64)
// routes itself, one per lane, so that the tokens without a row (most of them) cost a lane of one load instead of a wave
// each, and nothing goes through LDS or a barrier.  The four waves share every row, a quarter of its vectors each, and walk
// the block's rows (set bits of the ballot, i.e. tokens ascending, slots ascending) with the loads of the next row in
// flight while the current one is accumulated: a workgroup with several rows pays one memory round trip, not one per row.
// Same arithmetic as combine_kernel: slots ascending, separate fp32 multiply and add, one rounding to BF16.
constexpr int kServedWaves = 4;
constexpr int kServedBatch = 4;  // 16-byte vectors per lane and row in flight
template <int kWeights, bool kCached>
__global__ __launch_bounds__(64 * kServedWaves) void combine_served_kernel(
    const u32x4* __restrict__ y, const float* __restrict__ weights, const int* __restrict__ route_to_row, int num_topk,
    int tokens_per_block, int vec_per_row, u32x4* __restrict__ out, int num_tokens, const float* __restrict__ return_in,
    float* __restrict__ return_out, int num_rows)
{
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int token0 = blockIdx.x * tokens_per_block;
    const int tokens = min(tokens_per_block, num_tokens - token0);
    int row = -1;
    float weight = 0.0f;
    if (lane < tokens * num_topk) {
        const size_t route = static_cast<size_t>(token0) * num_topk + lane;
        row = route_to_row[route];
        if (row >= num_rows) row = -1;  // a row the caller's y does not hold
        if (kWeights == 1) weight = row >= 0 ? weights[row] : 0.0f;
        if (kWeights == 2) weight = weights[route];
        if (return_out != nullptr && wave == 0) return_out[route] = row >= 0 ? return_in[row] : 0.0f;
    }
    const uint64_t valid = __ballot(row >= 0);
    if (valid == 0ull) return;
    const int token_of_lane = lane / num_topk;
    const int quarter = (vec_per_row + kServedWaves - 1) / kServedWaves;
    const int vec_begin = wave * quarter, vec_end = min(vec_begin + quarter, vec_per_row);
    for (int v0 = vec_begin; v0 < vec_end; v0 += 64 * kServedBatch) {
        u32x4 buffer[2][kServedBatch];
        float acc[kServedBatch][8];
        auto clear = [&]() {
#pragma unroll
            for (int b = 0; b < kServedBatch; ++b)
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[b][i] = 0.0f;
        };
        auto issue = [&](u32x4 (&into)[kServedBatch], int at) {
            const u32x4* src = y + static_cast<size_t>(__builtin_amdgcn_readlane(row, at)) * vec_per_row;
#pragma unroll
            for (int b = 0; b < kServedBatch; ++b) {
                const int v = v0 + b * 64 + lane;
                if (v < vec_end) into[b] = kCached ? load16(src + v) : load16_nt(src + v);
            }
        };
        // accumulates the row of lane `at`; stores the token when `next` (-1: none) belongs to another one
        auto consume = [&](const u32x4 (&from)[kServedBatch], int at, int next) {
            const float w = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, weight), at));
#pragma unroll
            for (int b = 0; b < kServedBatch; ++b) {
                if (v0 + b * 64 + lane >= vec_end) continue;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float lo = bf16_to_f32(from[b][i] & 0xffffu);
                    float hi = bf16_to_f32(from[b][i] >> 16);
                    if (kWeights != 0) {
                        lo = __fmul_rn(lo, w);
                        hi = __fmul_rn(hi, w);
                    }
                    acc[b][2 * i] = __fadd_rn(acc[b][2 * i], lo);
                    acc[b][2 * i + 1] = __fadd_rn(acc[b][2 * i + 1], hi);
                }
            }
            const int token = __builtin_amdgcn_readlane(token_of_lane, at);
            if (next >= 0 && __builtin_amdgcn_readlane(token_of_lane, next) == token) return;
            u32x4* dst = out + static_cast<size_t>(token0 + token) * vec_per_row;
#pragma unroll
            for (int b = 0; b < kServedBatch; ++b) {
                const int v = v0 + b * 64 + lane;
                if (v >= vec_end) continue;
                u32x4 packed;
#pragma unroll
                for (int i = 0; i < 4; ++i) packed[i] = pack_bf16x2(acc[b][2 * i], acc[b][2 * i + 1]);
                store16_nt(dst + v, packed);
            }
            clear();
        };
        clear();
        uint64_t rest = valid;
        int at = __builtin_ctzll(rest);
        rest &= rest - 1ull;
        issue(buffer[0], at);
        for (;;) {
            int next = rest != 0ull ? __builtin_ctzll(rest) : -1;
            rest &= rest - 1ull;
            if (next >= 0) issue(buffer[1], next);
            consume(buffer[0], at, next);
            if (next < 0) break;
            at = next;
            next = rest != 0ull ? __builtin_ctzll(rest) : -1;
            rest &= rest - 1ull;
            if (next >= 0) issue(buffer[0], next);
            consume(buffer[1], at, next);
            if (next < 0) break;
            at = next;
        }
    }
}

template <int kWeights, bool kCached>
void launch_combine_served(hipStream_t stream, const void* y, const float* weights, const int32_t* route_to_row, int num_tokens,
                           int num_topk, int vec, void* out, const float* return_in, float* return_out, int num_rows)
{
    const int tokens_per_block = 64 / num_topk;  // top-k is at most 32
    hipLaunchKernelGGL((combine_served_kernel<kWeights, kCached>), dim3((num_tokens + tokens_per_block - 1) / tokens_per_block),
                       dim3(64 * kServedWaves), 0, stream, static_cast<const u32x4*>(y), weights, route_to_row, num_topk,
                       tokens_per_block, vec, static_cast<u32x4*>(out), num_tokens, return_in, return_out, num_rows);
}

struct CombineGrid {
    int parts, per_part, threads, blocks;
};


// Dense routing (at least one row per token on average): split every token row into 1-2 KiB parts.
// Sparse receive shares (most tokens own no row and only get zero-filled): one workgroup per token
// while that still fills the chip.
CombineGrid combine_grid(int num_tokens, int num_rows, int vec)
{
    CombineGrid g;
    const int target = num_rows >= num_tokens ? kDenseTargetBlocks : kSparseTargetBlocks;
    int parts = 1;
    while (num_tokens * parts < target && vec / (parts * 2) >= 64 && parts < 16) parts *= 2;
    g.per_part = (vec + parts - 1) / parts;
    // Dense routing: 1 KiB parts, one full wave each (at 4096 tokens x top-8 x 14 KiB rows 84 us, against 87 us for parts of
    // 0.875 or 3.5 KiB, 90 us for 1.75 KiB on two waves and 125 us for 0.5 KiB).
    if (num_rows >= num_tokens && vec >= kDenseVec) g.per_part = kDenseVec;
    g.parts = (vec + g.per_part - 1) / g.per_part;
    int threads = (g.per_part + 63) / 64 * 64;
    g.threads = threads > kMaxThreads ? kMaxThreads : (threads < 64 ? 64 : threads);
    g.blocks = num_tokens * g.parts;
    return g;
}

template <int kWeights, bool kHalf = false>
void launch_combine(const CombineGrid& g, hipStream_t stream, const void* y, const float* weights, const int32_t* route_to_row,
                    int num_topk, int vec, void* out, const float* return_in, float* return_out,
                    int num_rows, const int32_t* shared_first_row = nullptr, int num_shared = 0, int num_tokens = 0,
                    const int32_t* fill_state = nullptr, int leave_unserved = 0)
{
    hipLaunchKernelGGL((combine_kernel<kWeights, kHalf>), dim3(g.blocks), dim3(g.threads), 0, stream, static_cast<const u32x4*>(y),
                       weights, route_to_row, num_topk, vec, g.per_part, g.parts, static_cast<u32x4*>(out), return_in,
                       return_out, shared_first_row, num_shared, num_tokens, fill_state, num_rows, leave_unserved);
}

}  // namespace

// Route-weighted reduce used by the MegaMoE forward: out[t] = bf16( sum_s w[t,s] * float(y[row(t,s)]) ).
int combine_routes(const void* y, const float* route_weights, const int32_t* route_to_row, int num_tokens, int num_topk,
                   int num_rows_hint, int hidden, void* out, const int32_t* shared_first_row, int num_shared,
                   const int32_t* fill_state, int leave_unserved, hipStream_t stream)
{
    const int vec = hidden / 8;
    if (num_shared == 0 && leave_unserved && 2LL * num_rows_hint < num_tokens) {
        launch_combine_served<2, true>(stream, y, route_weights, route_to_row, num_tokens, num_topk, vec, out, nullptr, nullptr,
                                       0x7fffffff);
        return launch_status("combine_routes_served");
    }
    if (num_shared == 0 && 2LL * num_rows_hint < num_tokens) {  // a sparse share: most tokens own no row
        hipLaunchKernelGGL((combine_sparse_kernel<2, true>), dim3((num_tokens + kSparseWaves - 1) / kSparseWaves),
                           dim3(64 * kSparseWaves), 0, stream, static_cast<const u32x4*>(y), route_weights, route_to_row, num_topk,
                           vec, static_cast<u32x4*>(out), num_tokens, fill_state, nullptr, nullptr, 0x7fffffff);
        return launch_status("combine_routes_sparse");
    }
    const CombineGrid g = combine_grid(num_tokens, num_rows_hint, vec);
    launch_combine<2>(g, stream, y, route_weights, route_to_row, num_topk, vec, out, nullptr, nullptr, 0x7fffffff,
                      shared_first_row, num_shared, num_tokens, fill_state, leave_unserved);
    return launch_status("combine_routes");
}

}  // namespace dpep

namespace dpep {
namespace {

template <bool kHalf>
int combine_entry(const char* what, const void* y, const float* row_weights, const int32_t* route_to_row, int num_tokens,
                  int num_topk, int num_rows, int hidden, void* out, const float* return_in, float* return_out, void* stream,
                  int leave_unserved = 0)
{
    DPEP_REQUIRE(num_tokens >= 0 && num_topk >= 1 && num_topk <= DPEP_MAX_TOPK, "%s: bad T=%d K=%d", what, num_tokens,
                 num_topk);
    // (num_rows may exceed T*K: a capacity layout holds more rows than the batch has routes; rows of route_to_row
    // at or beyond num_rows are treated as absent)
    DPEP_REQUIRE(num_rows >= 0, "%s: num_rows=%d is negative", what, num_rows);
    DPEP_REQUIRE(hidden > 0 && hidden % 8 == 0, "%s: hidden=%d must be a positive multiple of 8", what, hidden);
    // (with no rows at all the channel's input is an empty buffer, which may well be a null pointer)
    DPEP_REQUIRE(return_in == nullptr ? (return_out == nullptr || num_rows == 0) : return_out != nullptr,
                 "%s: return_in and return_out go together", what);
    if (num_tokens == 0) return DPEP_OK;
    DPEP_REQUIRE(route_to_row != nullptr && out != nullptr && aligned16(out), "%s: NULL or misaligned buffer", what);
    DPEP_REQUIRE(num_rows == 0 || (y != nullptr && aligned16(y)), "%s: y must be 16-byte aligned", what);
    const int vec = hidden / 8;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (!kHalf && leave_unserved && 2LL * num_rows < num_tokens) {
        // a sparse share whose unserved tokens are skipped (with the zero rows to write as well, the workgroup-per-part
        // kernel below measured faster than a wave per token: 53 against 56 us at 16384 tokens of which 2000 own rows)
        if (row_weights != nullptr)
            launch_combine_served<1, false>(s, y, row_weights, route_to_row, num_tokens, num_topk, vec, out, return_in, return_out,
                                            num_rows);
        else
            launch_combine_served<0, false>(s, y, nullptr, route_to_row, num_tokens, num_topk, vec, out, return_in, return_out,
                                            num_rows);
        return launch_status(what);
    }
    const CombineGrid g = combine_grid(num_tokens, num_rows, vec);
    if (row_weights != nullptr)
        launch_combine<1, kHalf>(g, s, y, row_weights, route_to_row, num_topk, vec, out, return_in, return_out, num_rows, nullptr, 0,
                                 0, nullptr, leave_unserved);
    else
        launch_combine<0, kHalf>(g, s, y, nullptr, route_to_row, num_topk, vec, out, return_in, return_out, num_rows, nullptr, 0, 0,
                                 nullptr, leave_unserved);
    return launch_status(what);
}

}  // namespace
}  // namespace dpep

extern "C" {

int dpep_combine(const void* y, const float* row_weights, const int32_t* route_to_row, int num_tokens, int num_topk,
                 int num_rows, int hidden, void* out, const float* return_in, float* return_out, void* stream)
{
    return dpep::combine_entry<false>("combine", y, row_weights, route_to_row, num_tokens, num_topk, num_rows, hidden, out,
                                      return_in, return_out, stream);
}

int dpep_combine_served(const void* y, const float* row_weights, const int32_t* route_to_row, int num_tokens, int num_topk,
                        int num_rows, int hidden, void* out, const float* return_in, float* return_out, void* stream)
{
    return dpep::combine_entry<false>("combine_served", y, row_weights, route_to_row, num_tokens, num_topk, num_rows, hidden,
                                      out, return_in, return_out, stream, /*leave_unserved=*/1);
}

int dpep_combine_fp16(const void* y, const float* row_weights, const int32_t* route_to_row, int num_tokens, int num_topk,
                      int num_rows, int hidden, void* out, const float* return_in, float* return_out, void* stream)
{
    return dpep::combine_entry<true>("combine_fp16", y, row_weights, route_to_row, num_tokens, num_topk, num_rows, hidden,
                                     out, return_in, return_out, stream);
}

}  // extern "C"
