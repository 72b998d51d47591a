// Expand-permute payload dispatch: out[row(t,s)] = x[t] for every route that owns a row, optionally
// fused with the per-128-element FP8 e4m3fn block quantiser.  HBM-bound: 16-byte coalesced loads,
// 16-byte stores, each input row read once and written to its K destinations.  How the token-major kernels store
// is a process-wide policy (dpep_dispatch_store_policy): streaming by default, write-through or cached on request.
//
// Observable contract: tests/elastic/test_dispatch.py:1391-1416 (payload, scales and weights arrive
// bit-exactly in row order), tests/clos/common.py:276-279; quantiser deep_ep/utils/math.py:45-61.
#include <type_traits>

#include "common.h"

#pragma clang fp contract(off)

namespace dpep {
namespace {

constexpr int kMaxThreads = 256;
constexpr int kTargetBlocks = 8192;  // rows are split into column parts until a launch has about this many workgroups (4096 rows: two parts each measured 3-6 % faster than one, four no better)
constexpr int kMaxScaleCols = 1024;  // hidden <= 131072 for the fused quantiser
constexpr int kRowMajorRatio = 1;  // row-major kernels when rows <= ratio * tokens

// Store policy of the payload rows.  Streaming (non-temporal, the default): the rows go to HBM past the caches at the
// streaming-write rate, and the kernel's time is the time of its traffic.  Write-through (device-scope `sc1`) and cached
// stores let the 256 MiB memory-side cache take the rows first: the kernel itself ends sooner when that cache holds clean
// lines at launch, but the rows still have to reach HBM, and whatever runs next pays for it (measured at T=4096, H=7168,
// top-8: the fused FP8 dispatch after a read-only sweep of 256 MiB takes 59.6 us streaming and 49.5 us write-through; with
// the sweep that follows charged to it, 60.9 against 85.9 us; inside a dispatch + combine loop 49.6 against 69.8 us, and the
// combine behind it 88.3 against 101.6 us).  A caller whose next kernel reads the rows while they are still in the
// memory-side cache may still prefer write-through, hence the knob.
int g_store_policy = DPEP_STORE_STREAMING;

template <int kPolicy>
__device__ __forceinline__ void store16_as(void* p, u32x4 v)
{
    if (kPolicy == DPEP_STORE_THROUGH) store16_through(p, v);
    else if (kPolicy == DPEP_STORE_STREAMING) store16_nt(p, v);
    else *reinterpret_cast<u32x4*>(p) = v;
}

// Calls launch(std::integral_constant<int, policy>) for the current policy.
template <typename Launch>
void with_store_policy(Launch&& launch)
{
    switch (__atomic_load_n(&g_store_policy, __ATOMIC_RELAXED)) {
    case DPEP_STORE_THROUGH: launch(std::integral_constant<int, DPEP_STORE_THROUGH>{}); break;
    case DPEP_STORE_CACHED: launch(std::integral_constant<int, DPEP_STORE_CACHED>{}); break;
    default: launch(std::integral_constant<int, DPEP_STORE_STREAMING>{}); break;
    }
}

// ---- token-major copy: one workgroup per (token, column part); read once, write K times -----------
template <int kPolicy>
__global__ __launch_bounds__(kMaxThreads) void dispatch_copy_token_kernel(
    const u32x4* __restrict__ x, const float* __restrict__ scales, const float* __restrict__ weights,
    const int* __restrict__ route_to_row, int num_topk, int vec_per_row, int vec_per_part, int parts, int scale_cols,
    u32x4* __restrict__ out, float* __restrict__ out_scales, float* __restrict__ out_weights)
{
    __shared__ int rows[DPEP_MAX_TOPK];
    __shared__ int any_valid;
    const int token = blockIdx.x / parts, part = blockIdx.x % parts;
    const int v_begin = part * vec_per_part;
    const int v_end = min(v_begin + vec_per_part, vec_per_row);
    const u32x4* src = x + static_cast<size_t>(token) * vec_per_row;
    // The token's first values are asked for before its routes are known (see the quantising kernel below).
    const int v_first = v_begin + threadIdx.x;
    u32x4 first = {0u, 0u, 0u, 0u};
    if (v_first < v_end) first = load16(src + v_first);
    if (threadIdx.x == 0) any_valid = 0;
    __syncthreads();
    if (threadIdx.x < num_topk) {
        const int row = route_to_row[static_cast<size_t>(token) * num_topk + threadIdx.x];
        rows[threadIdx.x] = row;
        if (row >= 0) any_valid = 1;
    }
    __syncthreads();
    if (!any_valid) return;
    for (int v = v_first; v < v_end; v += blockDim.x) {
        const u32x4 value = v == v_first ? first : load16(src + v);
        for (int s = 0; s < num_topk; ++s) {
            const int row = rows[s];
            if (row >= 0) store16_as<kPolicy>(out + static_cast<size_t>(row) * vec_per_row + v, value);
        }
    }
    if (part == 0) {
        if (scales != nullptr) {
            for (int c = threadIdx.x; c < scale_cols; c += blockDim.x) {
                const float value = scales[static_cast<size_t>(token) * scale_cols + c];
                for (int s = 0; s < num_topk; ++s) {
                    const int row = rows[s];
                    if (row >= 0) out_scales[static_cast<size_t>(row) * scale_cols + c] = value;
                }
            }
        }
        if (weights != nullptr && threadIdx.x < num_topk && rows[threadIdx.x] >= 0)
            out_weights[rows[threadIdx.x]] = weights[static_cast<size_t>(token) * num_topk + threadIdx.x];
    }
}

// ---- row-major copy: one workgroup per (output row, column part); for sparse receive shares -------
template <int kPolicy>
__global__ __launch_bounds__(kMaxThreads) void dispatch_copy_row_kernel(
    const u32x4* __restrict__ x, const float* __restrict__ scales, const float* __restrict__ weights,
    const int* __restrict__ row_to_route, int num_tokens, int num_topk, int vec_per_row, int vec_per_part, int parts,
    int scale_cols, u32x4* __restrict__ out, float* __restrict__ out_scales, float* __restrict__ out_weights)
{
    const int row = blockIdx.x / parts, part = blockIdx.x % parts;
    // (clamped: a map left incomplete by a layout launch that reported a time-out must not become a wild address)
    const int route = min(max(row_to_route[row], 0), num_tokens * num_topk - 1);
    const int token = route / num_topk;
    const int v_begin = part * vec_per_part;
    const int v_end = min(v_begin + vec_per_part, vec_per_row);
    const u32x4* src = x + static_cast<size_t>(token) * vec_per_row;
    u32x4* dst = out + static_cast<size_t>(row) * vec_per_row;
    for (int v = v_begin + threadIdx.x; v < v_end; v += blockDim.x) store16_as<kPolicy>(dst + v, load16(src + v));
    if (part == 0) {
        if (scales != nullptr)
            for (int c = threadIdx.x; c < scale_cols; c += blockDim.x)
                out_scales[static_cast<size_t>(row) * scale_cols + c] = scales[static_cast<size_t>(token) * scale_cols + c];
        if (weights != nullptr && threadIdx.x == 0) out_weights[row] = weights[route];
    }
}

// ---- per-128 FP8 quantiser ------------------------------------------------------------------------
// One lane owns 16 consecutive BF16 values (two 16-byte loads), so 8 adjacent lanes own one
// 128-element block.  amax is reduced over those 8 lanes with DPP-free xor shuffles inside the wave.
struct Quant16 {
    u32x4 codes;  // 16 e4m3fn bytes
    float scale;  // amax / 448
};

// Largest of a value over the 8 lanes that share a 128-element block.
__device__ __forceinline__ uint32_t max8(uint32_t v)
{
    v = max(v, static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), 1)));
    v = max(v, static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), 2)));
    v = max(v, static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), 4)));
    return v;
}

// fp32 -> e4m3fn byte pair, round-to-nearest-even, on the gfx950 converter (OCP FP8).
__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d)
{
    int packed = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    packed = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, packed, true);
    return static_cast<uint32_t>(packed);
}

__device__ __forceinline__ Quant16 quantize16(u32x4 lo, u32x4 hi)
{
    float v[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = bf16_to_f32(lo[i] & 0xffffu);
        v[2 * i + 1] = bf16_to_f32(lo[i] >> 16);
        v[8 + 2 * i] = bf16_to_f32(hi[i] & 0xffffu);
        v[8 + 2 * i + 1] = bf16_to_f32(hi[i] >> 16);
    }
    // amax as the largest magnitude BIT PATTERN (two BF16 magnitudes per word, v_pk_max_u16): for finite values that is
    // the largest magnitude, and a NaN, whose pattern lies above infinity's, wins over everything, as it does in the
    // reference's amax() and clamp() (torch propagates NaN through both, deep_ep/utils/math.py:52-53): a block that
    // holds a NaN gets a NaN scale and the NaN code 0x7F for every value, whatever the others are.
    typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
    u16x2 both = {0, 0};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        both = __builtin_elementwise_max(both, __builtin_bit_cast(u16x2, lo[i] & 0x7fff7fffu));
        both = __builtin_elementwise_max(both, __builtin_bit_cast(u16x2, hi[i] & 0x7fff7fffu));
    }
    const uint32_t mine = max(static_cast<uint32_t>(both[0]), static_cast<uint32_t>(both[1]));
    const uint32_t amax_bits = max(max8(mine) << 16, __float_as_uint(1e-4f));
    const float amax = __uint_as_float(amax_bits);
    const bool poisoned = amax_bits > 0x7f800000u;
    // The reference writes 448.0 / amax, which torch evaluates as reciprocal(amax) * 448:
    // two correctly rounded fp32 operations, reproduced here.
    const float inv = __fmul_rn(__fdiv_rn(1.0f, amax), 448.0f);
    Quant16 q;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t codes = pack4_e4m3(__fmul_rn(v[4 * i], inv), __fmul_rn(v[4 * i + 1], inv), __fmul_rn(v[4 * i + 2], inv),
                                          __fmul_rn(v[4 * i + 3], inv));
        q.codes[i] = poisoned ? 0x7f7f7f7fu : codes;
    }
    q.scale = __fdiv_rn(amax, 448.0f);
    return q;
}

// token-major: one workgroup per (token, column part); units = 16-element groups per row (H/16).
template <int kPolicy>
__global__ __launch_bounds__(kMaxThreads) void dispatch_quant_token_kernel(
    const u32x4* __restrict__ x, const float* __restrict__ weights, const int* __restrict__ route_to_row, int num_topk,
    int units_per_row, int units_per_part, int parts, u32x4* __restrict__ out, float* __restrict__ out_scales,
    float* __restrict__ out_weights)
{
    __shared__ int rows[DPEP_MAX_TOPK];
    __shared__ int any_valid;
    __shared__ float part_scales[kMaxScaleCols];
    const int token = blockIdx.x / parts, part = blockIdx.x % parts;
    const int u_begin = part * units_per_part;
    const int u_end = min(u_begin + units_per_part, units_per_row);
    const u32x4* src = x + static_cast<size_t>(token) * units_per_row * 2;
    // The token's first values are asked for before its routes are known: this grid is only used where most tokens own
    // rows, and the row lookup and the payload then travel together instead of one after the other.
    const int u_first = u_begin + threadIdx.x;
    constexpr int kEarly = 2;  // units per thread fetched up front (all of a 7168-wide row with 256 threads)
    u32x4 lo[kEarly], hi[kEarly];
#pragma unroll
    for (int j = 0; j < kEarly; ++j) {
        const int u = u_first + j * static_cast<int>(blockDim.x);
        if (u < u_end) {
            lo[j] = load16(src + 2 * u);
            hi[j] = load16(src + 2 * u + 1);
        }
    }
    if (threadIdx.x == 0) any_valid = 0;
    __syncthreads();
    if (threadIdx.x < num_topk) {
        const int row = route_to_row[static_cast<size_t>(token) * num_topk + threadIdx.x];
        rows[threadIdx.x] = row;
        if (row >= 0) any_valid = 1;
    }
    __syncthreads();
    if (!any_valid) return;
    const int scale_cols = units_per_row / 8;
    // units_per_part is a multiple of 8 and blockDim of 64, so the 8 lanes of a block stay together.
    // Quantise first, then write row by row: at any moment the workgroup's stores run along ONE output row.
    u32x4 codes[kEarly];
#pragma unroll
    for (int j = 0; j < kEarly; ++j) {
        const int u = u_first + j * static_cast<int>(blockDim.x);
        if (u < u_end) {
            const Quant16 q = quantize16(lo[j], hi[j]);
            codes[j] = q.codes;
            if ((u & 7) == 0) part_scales[(u - u_begin) >> 3] = q.scale;
        }
    }
    for (int s = 0; s < num_topk; ++s) {
        const int row = rows[s];
        if (row < 0) continue;
#pragma unroll
        for (int j = 0; j < kEarly; ++j) {
            const int u = u_first + j * static_cast<int>(blockDim.x);
            if (u < u_end) store16_as<kPolicy>(out + static_cast<size_t>(row) * units_per_row + u, codes[j]);
        }
    }
    for (int u = u_first + kEarly * static_cast<int>(blockDim.x); u < u_end; u += blockDim.x) {  // rows wider than that
        const Quant16 q = quantize16(load16(src + 2 * u), load16(src + 2 * u + 1));
        for (int s = 0; s < num_topk; ++s) {
            const int row = rows[s];
            if (row >= 0) store16_as<kPolicy>(out + static_cast<size_t>(row) * units_per_row + u, q.codes);
        }
        if ((u & 7) == 0) part_scales[(u - u_begin) >> 3] = q.scale;
    }
    __syncthreads();
    // The part's scales leave as contiguous runs (consecutive lanes, consecutive floats) instead of one
    // 4-byte store per block of 128, which would turn every scale row into read-modify-write traffic.
    const int part_cols = (u_end - u_begin) >> 3, col0 = u_begin >> 3;
    for (int i = threadIdx.x; i < num_topk * part_cols; i += blockDim.x) {
        const int s = i / part_cols, c = i - s * part_cols;
        const int row = rows[s];
        if (row >= 0) out_scales[static_cast<size_t>(row) * scale_cols + col0 + c] = part_scales[c];
    }
    if (part == 0 && weights != nullptr && threadIdx.x < num_topk && rows[threadIdx.x] >= 0)
        out_weights[rows[threadIdx.x]] = weights[static_cast<size_t>(token) * num_topk + threadIdx.x];
}

// row-major: one workgroup per (output row, column part); row_to_route == nullptr means identity
// (row == token), which is the stand-alone quantiser.
template <int kPolicy>
__global__ __launch_bounds__(kMaxThreads) void dispatch_quant_row_kernel(
    const u32x4* __restrict__ x, const float* __restrict__ weights, const int* __restrict__ row_to_route, int num_tokens,
    int num_topk, int units_per_row, int units_per_part, int parts, u32x4* __restrict__ out, float* __restrict__ out_scales,
    float* __restrict__ out_weights)
{
    const int row = blockIdx.x / parts, part = blockIdx.x % parts;
    const int route = row_to_route != nullptr ? min(max(row_to_route[row], 0), num_tokens * num_topk - 1) : row;
    const int token = row_to_route != nullptr ? route / num_topk : row;
    const int u_begin = part * units_per_part;
    const int u_end = min(u_begin + units_per_part, units_per_row);
    const int scale_cols = units_per_row / 8;
    const u32x4* src = x + static_cast<size_t>(token) * units_per_row * 2;
    for (int u = u_begin + threadIdx.x; u < u_end; u += blockDim.x) {
        const Quant16 q = quantize16(load16(src + 2 * u), load16(src + 2 * u + 1));
        store16_as<kPolicy>(out + static_cast<size_t>(row) * units_per_row + u, q.codes);
        if ((u & 7) == 0) out_scales[static_cast<size_t>(row) * scale_cols + (u >> 3)] = q.scale;
    }
    if (part == 0 && weights != nullptr && threadIdx.x == 0) out_weights[row] = weights[route];
}

// Stand-alone quantiser for rows whose width is not a multiple of 128: the last block of a row is short and is
// quantised as if padded with zeros (per_token_cast_to_fp8 pads, deep_ep/utils/math.py:52-53).  One thread per 16 values
// of the padded row, so the eight lanes of a block are always all present; padding units load and store nothing.
__global__ __launch_bounds__(256) void cast_to_fp8_short_block_kernel(const u32x4* __restrict__ x, int units_per_row,
                                                                      int blocks_per_row, long long padded_units,
                                                                      u32x4* __restrict__ out, float* __restrict__ out_scales)
{
    const long long id = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= padded_units) return;  // padded_units is a multiple of 8: whole blocks leave together
    const long long row = id / (blocks_per_row * 8);
    const int unit = static_cast<int>(id % (blocks_per_row * 8));
    const bool real = unit < units_per_row;
    const u32x4 zero = {0u, 0u, 0u, 0u};
    const u32x4* src = x + (row * units_per_row + unit) * 2;
    const Quant16 q = quantize16(real ? load16(src) : zero, real ? load16(src + 1) : zero);
    if (real) store16_nt(out + row * units_per_row + unit, q.codes);
    if ((unit & 7) == 0) out_scales[row * blocks_per_row + (unit >> 3)] = q.scale;
}

// ---- dequantiser: bf16(fp32(code) * scale) per block of 128 columns ---------------------------------------------
// One thread per 8 codes (8 bytes in, 16 bytes out), so that consecutive lanes write consecutive 16-byte vectors: with 16
// codes per thread a lane's two output vectors sat 32 bytes apart and every store instruction filled only half of each
// 64 bytes it touched (187 us for 32768 x 7168 codes; this way 5 TB/s and more).  kByteScales: the scales are e8m0 bytes
// (four to an int32 in the caller's tensor), value 2^(byte - 127) built by moving the byte into the exponent field; else
// fp32.  The last block of a row may be short (hidden need only be a multiple of 16).
template <bool kByteScales>
__global__ __launch_bounds__(256) void cast_back_kernel(const unsigned long long* __restrict__ codes, const void* __restrict__ scales,
                                                        int halves_per_row, int scales_per_row, long long total_halves,
                                                        u32x4* __restrict__ out)
{
    const long long id = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total_halves) return;
    long long row;
    int half;
    if (total_halves < (1ll << 31)) {  // 32-bit division where it suffices
        row = static_cast<unsigned>(id) / static_cast<unsigned>(halves_per_row);
        half = static_cast<int>(static_cast<unsigned>(id) - static_cast<unsigned>(row) * static_cast<unsigned>(halves_per_row));
    } else {
        row = id / halves_per_row;
        half = static_cast<int>(id - row * halves_per_row);
    }
    const long long at = row * scales_per_row + (half >> 4);
    const float scale = kByteScales ? __uint_as_float(static_cast<uint32_t>(static_cast<const uint8_t*>(scales)[at]) << 23)
                                    : static_cast<const float*>(scales)[at];
    const unsigned long long q = __builtin_nontemporal_load(codes + id);
    u32x4 value;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int word = static_cast<int>(static_cast<uint32_t>(q >> (32 * i)));
        const float a = __fmul_rn(__builtin_amdgcn_cvt_f32_fp8(word, 0), scale);
        const float b = __fmul_rn(__builtin_amdgcn_cvt_f32_fp8(word, 1), scale);
        const float c = __fmul_rn(__builtin_amdgcn_cvt_f32_fp8(word, 2), scale);
        const float d = __fmul_rn(__builtin_amdgcn_cvt_f32_fp8(word, 3), scale);
        value[2 * i] = pack_bf16x2(a, b);
        value[2 * i + 1] = pack_bf16x2(c, d);
    }
    store16_nt(out + id, value);
}

// ---- small batches: routing layout and payload in ONE launch -------------------------------------------------
// With at most kSmallRoutes routes (a decode step) the whole routing table fits a workgroup's LDS, and a workgroup
// gets the rows of its own token faster by working them out itself than by waiting for a layout kernel: every
// workgroup (one per token and column part) reads all ids, histograms them (LDS atomics: a count does not depend on
// order), scans the histogram over the experts, and counts, for each of its token's routes, the earlier routes with
// the same expert.  row = first row of the expert + that count: the same stable permutation the layout kernels
// produce.  Nothing travels between workgroups.  Part 0 of each token writes the token's entries of route_to_row and
// row_to_route, workgroup 0 the per-expert outputs and the host mailbox.
constexpr int kSmallRoutes = 2048;

template <bool kQuant, int kSlots>  // kSlots: compile-time bound of top-k (8 or DPEP_MAX_TOPK)
__global__ __launch_bounds__(kMaxThreads) void layout_dispatch_small_kernel(
    const long long* __restrict__ idx, int n_routes, int num_experts, int expert_begin, int num_local, int num_topk,
    const u32x4* __restrict__ x, const float* __restrict__ scales, const float* __restrict__ weights, int units_per_row,
    int units_per_part, int parts, int scale_cols, int* __restrict__ counts, int* __restrict__ psum, int* __restrict__ offsets,
    int* __restrict__ num_rows, int* __restrict__ route_to_row, int* __restrict__ row_to_route, u32x4* __restrict__ out,
    float* __restrict__ out_scales, float* __restrict__ out_weights, uint32_t* __restrict__ mailbox, uint32_t sequence)
{
    __shared__ short local_id[kSmallRoutes];
    __shared__ int first_row[DPEP_MAX_LOCAL_EXPERTS];  // per expert: count, then exclusive prefix
    __shared__ int before[DPEP_MAX_TOPK];
    __shared__ int rows[DPEP_MAX_TOPK];
    __shared__ int wave_sums[kMaxThreads / kWave];
    __shared__ float part_scales[kMaxScaleCols];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int token = blockIdx.x / parts, part = blockIdx.x % parts;
    // in units of 16 bytes of input (kQuant: 32 bytes = 16 BF16 values = 16 bytes of output)
    const int u_begin = part * units_per_part, u_end = min(u_begin + units_per_part, units_per_row);
    constexpr int kIn = kQuant ? 2 : 1;
    const u32x4* src = x + static_cast<size_t>(token) * units_per_row * kIn;
    // the payload is asked for first: it does not depend on the routing
    constexpr int kEarly = 2;
    u32x4 early[kEarly][kIn];
#pragma unroll
    for (int j = 0; j < kEarly; ++j) {
        const int u = u_begin + tid + j * kMaxThreads;
        if (u < u_end) {
#pragma unroll
            for (int h = 0; h < kIn; ++h) early[j][h] = load16(src + kIn * u + h);
        }
    }
    for (int e = tid; e < num_local; e += kMaxThreads) first_row[e] = 0;
    if (tid < DPEP_MAX_TOPK) before[tid] = 0;
    __syncthreads();
    for (int j = tid; j < n_routes; j += kMaxThreads) {
        const int e = local_expert(idx[j], j, n_routes, num_experts, expert_begin, num_local);
        local_id[j] = static_cast<short>(e);
        if (e >= 0) atomicAdd(&first_row[e], 1);
    }
    __syncthreads();
    // exclusive scan over the experts: four consecutive experts per thread, wave scan, then the waves' sums
    int mine[4], sum = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = tid * 4 + j;
        mine[j] = e < num_local ? first_row[e] : 0;
        sum += mine[j];
    }
    int incl = sum;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int up = __shfl_up(incl, d);
        if (lane >= d) incl += up;
    }
    if (lane == kWave - 1) wave_sums[wave] = incl;
    __syncthreads();
    int offset = incl - sum;
    for (int w = 0; w < wave; ++w) offset += wave_sums[w];
    const bool reporter = blockIdx.x == 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = tid * 4 + j;
        if (e < num_local) {
            first_row[e] = offset;
            if (reporter) {
                counts[e] = mine[j];
                psum[e] = offset + mine[j];
                offsets[e + 1] = offset + mine[j];
            }
        }
        offset += mine[j];
    }
    if (reporter && tid == kMaxThreads - 1) {
        offsets[0] = 0;
        num_rows[0] = offset;  // the last thread's running offset is the total
    }
    if (reporter && mailbox != nullptr && tid * 4 < num_local) mailbox_store_counts(mailbox, tid * 4, mine);
    if (reporter && mailbox != nullptr) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this thread's counts have reached the host
    __syncthreads();
    if (reporter && mailbox != nullptr && tid == kMaxThreads - 1) {
        const unsigned long long word = (static_cast<unsigned long long>(sequence) << 32) | static_cast<uint32_t>(offset);
        __hip_atomic_store(reinterpret_cast<unsigned long long*>(mailbox), word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    // earlier routes with the same expert, for each route of this token
    const int my_first = token * num_topk;
    int want[kSlots], seen[kSlots];
#pragma unroll
    for (int s = 0; s < kSlots; ++s) {
        want[s] = s < num_topk ? local_id[my_first + s] : -2;  // -2 matches nothing
        seen[s] = 0;
    }
    for (int j = tid; j < my_first + num_topk; j += kMaxThreads) {
        const int e = local_id[j];
#pragma unroll
        for (int s = 0; s < kSlots; ++s) seen[s] += (e == want[s] && j < my_first + s) ? 1 : 0;
    }
#pragma unroll
    for (int s = 0; s < kSlots; ++s)
        if (seen[s] != 0 && want[s] >= 0) atomicAdd(&before[s], seen[s]);
    __syncthreads();
    if (tid < num_topk) {
        const int e = local_id[my_first + tid];
        const int row = e >= 0 ? first_row[e] + before[tid] : -1;
        rows[tid] = row;
        if (part == 0) {
            route_to_row[my_first + tid] = row;
            if (row >= 0) {
                row_to_route[row] = my_first + tid;
                if (weights != nullptr) out_weights[row] = weights[my_first + tid];
            }
        }
    }
    __syncthreads();
    // payload: read once, write to every row of the token
    auto emit = [&](int u, const u32x4 (&in)[kIn]) {
        u32x4 value = in[0];
        if (kQuant) {
            const Quant16 q = quantize16(in[0], in[kIn - 1]);
            value = q.codes;
            if ((u & 7) == 0) part_scales[(u - u_begin) >> 3] = q.scale;
        }
        for (int s = 0; s < num_topk; ++s) {
            const int row = rows[s];
            if (row >= 0) store16_nt(out + static_cast<size_t>(row) * units_per_row + u, value);
        }
    };
#pragma unroll
    for (int j = 0; j < kEarly; ++j) {
        const int u = u_begin + tid + j * kMaxThreads;
        if (u < u_end) emit(u, early[j]);
    }
    for (int u = u_begin + tid + kEarly * kMaxThreads; u < u_end; u += kMaxThreads) {
        u32x4 in[kIn];
#pragma unroll
        for (int h = 0; h < kIn; ++h) in[h] = load16(src + kIn * u + h);
        emit(u, in);
    }
    if (kQuant) {
        __syncthreads();
        const int part_cols = (u_end - u_begin) >> 3, col0 = u_begin >> 3, out_cols = units_per_row / 8;
        for (int i = tid; i < num_topk * part_cols; i += kMaxThreads) {
            const int s = i / part_cols, c = i - s * part_cols;
            const int row = rows[s];
            if (row >= 0) out_scales[static_cast<size_t>(row) * out_cols + col0 + c] = part_scales[c];
        }
    } else if (part == 0 && scales != nullptr) {
        for (int c = tid; c < scale_cols; c += kMaxThreads) {
            const float value = scales[static_cast<size_t>(token) * scale_cols + c];
            for (int s = 0; s < num_topk; ++s) {
                const int row = rows[s];
                if (row >= 0) out_scales[static_cast<size_t>(row) * scale_cols + c] = value;
            }
        }
    }
}

// Split a row of `units` work items over `parts` workgroups so that a launch of `rows` rows has
// enough workgroups to fill 256 CUs; each part is a multiple of `granule` units.
struct Split {
    int parts, per_part, threads;
};

Split choose_split(int rows, int units, int granule)
{
    Split s;
    const int target_blocks = kTargetBlocks;
    int parts = 1;
    while (rows * parts < target_blocks && units / (parts * 2) >= 64 && parts < 16) parts *= 2;
    int per_part = (units + parts - 1) / parts;
    per_part = (per_part + granule - 1) / granule * granule;
    s.parts = (units + per_part - 1) / per_part;
    s.per_part = per_part;
    int threads = (per_part + 63) / 64 * 64;
    s.threads = threads > kMaxThreads ? kMaxThreads : threads;
    return s;
}

int check_common(const char* what, int num_tokens, int num_topk, int num_rows, const int32_t* route_to_row,
                 const int32_t* row_to_route)
{
    DPEP_REQUIRE(num_tokens >= 0 && num_topk >= 1 && num_topk <= DPEP_MAX_TOPK, "%s: bad T=%d K=%d", what, num_tokens,
                 num_topk);
    DPEP_REQUIRE(num_rows >= -1 && static_cast<long long>(num_rows) <= static_cast<long long>(num_tokens) * num_topk,
                 "%s: num_rows=%d outside [0, T*K] (or -1: not known yet)", what, num_rows);
    DPEP_REQUIRE(num_rows == 0 || route_to_row != nullptr, "%s: NULL routing maps", what);
    DPEP_REQUIRE(num_rows <= 0 || row_to_route != nullptr, "%s: NULL routing maps", what);
    return DPEP_OK;
}

}  // namespace
}  // namespace dpep

extern "C" {

int dpep_dispatch_store_policy(int policy)
{
    using namespace dpep;
    const int before = __atomic_load_n(&g_store_policy, __ATOMIC_RELAXED);
    if (policy == DPEP_STORE_QUERY) return before;
    DPEP_REQUIRE(policy == DPEP_STORE_THROUGH || policy == DPEP_STORE_STREAMING || policy == DPEP_STORE_CACHED,
                 "dispatch_store_policy: %d is not DPEP_STORE_THROUGH, _STREAMING, _CACHED or _QUERY", policy);
    __atomic_store_n(&g_store_policy, policy, __ATOMIC_RELAXED);
    return before;
}

int dpep_dispatch_copy(const void* x, const float* scales, const float* topk_weights, const int32_t* route_to_row,
                       const int32_t* row_to_route, int num_tokens, int num_topk, int num_rows, int row_bytes,
                       int scale_cols, void* out, float* out_scales, float* out_weights, void* stream)
{
    using namespace dpep;
    if (int rc = check_common("dispatch_copy", num_tokens, num_topk, num_rows, route_to_row, row_to_route)) return rc;
    DPEP_REQUIRE(row_bytes > 0 && row_bytes % 16 == 0, "dispatch_copy: row_bytes=%d must be a positive multiple of 16",
                 row_bytes);
    // (a share without rows or a batch without tokens: the outputs are empty buffers, which may well be null pointers)
    if (num_rows == 0 || num_tokens == 0) return DPEP_OK;
    DPEP_REQUIRE((scales == nullptr) == (out_scales == nullptr), "dispatch_copy: scales and out_scales go together");
    DPEP_REQUIRE(scales == nullptr || scale_cols > 0, "dispatch_copy: scale_cols must be positive with scales");
    DPEP_REQUIRE((topk_weights == nullptr) == (out_weights == nullptr), "dispatch_copy: weights and out_weights go together");
    DPEP_REQUIRE(x != nullptr && out != nullptr && aligned16(x) && aligned16(out), "dispatch_copy: x/out must be 16-byte aligned");
    const int vec = row_bytes / 16;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // the token-major grid does not depend on R, so a launch that does not know R yet takes it
    if (num_rows < 0 || static_cast<long long>(num_rows) > static_cast<long long>(kRowMajorRatio) * num_tokens) {
        const Split sp = choose_split(num_tokens, vec, 1);
        with_store_policy([&](auto policy) {
            hipLaunchKernelGGL(dispatch_copy_token_kernel<decltype(policy)::value>, dim3(num_tokens * sp.parts),
                               dim3(sp.threads), 0, s, static_cast<const u32x4*>(x), scales, topk_weights, route_to_row,
                               num_topk, vec, sp.per_part, sp.parts, scale_cols, static_cast<u32x4*>(out), out_scales,
                               out_weights);
        });
        return launch_status("dispatch_copy_token");
    }
    const Split sp = choose_split(num_rows, vec, 1);
    with_store_policy([&](auto policy) {
        hipLaunchKernelGGL(dispatch_copy_row_kernel<decltype(policy)::value>, dim3(num_rows * sp.parts), dim3(sp.threads), 0,
                           s, static_cast<const u32x4*>(x), scales, topk_weights, row_to_route, num_tokens, num_topk, vec,
                           sp.per_part, sp.parts, scale_cols, static_cast<u32x4*>(out), out_scales, out_weights);
    });
    return launch_status("dispatch_copy_row");
}

int dpep_dispatch_quant_fp8(const void* x, const float* topk_weights, const int32_t* route_to_row,
                            const int32_t* row_to_route, int num_tokens, int num_topk, int num_rows, int hidden,
                            void* out, float* out_scales, float* out_weights, void* stream)
{
    using namespace dpep;
    if (int rc = check_common("dispatch_quant_fp8", num_tokens, num_topk, num_rows, route_to_row, row_to_route)) return rc;
    DPEP_REQUIRE(hidden > 0 && hidden % 128 == 0 && hidden / 128 <= kMaxScaleCols,
                 "dispatch_quant_fp8: hidden=%d must be a positive multiple of 128, at most %d", hidden, 128 * kMaxScaleCols);
    if (num_rows == 0 || num_tokens == 0) return DPEP_OK;  // (empty outputs may be null pointers)
    DPEP_REQUIRE((topk_weights == nullptr) == (out_weights == nullptr), "dispatch_quant_fp8: weights and out_weights go together");
    DPEP_REQUIRE(x && out && out_scales && aligned16(x) && aligned16(out), "dispatch_quant_fp8: x/out must be 16-byte aligned");
    const int units = hidden / 16;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // the token-major grid does not depend on R, so a launch that does not know R yet takes it
    if (num_rows < 0 || static_cast<long long>(num_rows) > static_cast<long long>(kRowMajorRatio) * num_tokens) {
        const Split sp = choose_split(num_tokens, units, 8);
        with_store_policy([&](auto policy) {
            hipLaunchKernelGGL(dispatch_quant_token_kernel<decltype(policy)::value>, dim3(num_tokens * sp.parts),
                               dim3(sp.threads), 0, s, static_cast<const u32x4*>(x), topk_weights, route_to_row, num_topk,
                               units, sp.per_part, sp.parts, static_cast<u32x4*>(out), out_scales, out_weights);
        });
        return launch_status("dispatch_quant_token");
    }
    const Split sp = choose_split(num_rows, units, 8);
    with_store_policy([&](auto policy) {
        hipLaunchKernelGGL(dispatch_quant_row_kernel<decltype(policy)::value>, dim3(num_rows * sp.parts), dim3(sp.threads),
                           0, s, static_cast<const u32x4*>(x), topk_weights, row_to_route, num_tokens, num_topk, units,
                           sp.per_part, sp.parts, static_cast<u32x4*>(out), out_scales, out_weights);
    });
    return launch_status("dispatch_quant_row");
}

int dpep_layout_dispatch_small(void* ws, const int64_t* topk_idx, const void* x, const float* scales,
                               const float* topk_weights, int num_tokens, int num_topk, int num_experts, int expert_begin,
                               int num_local, int row_bytes, int scale_cols, int quantize, int32_t* counts, int32_t* psum,
                               int32_t* offsets, int32_t* route_to_row, int32_t* row_to_route, int32_t* num_rows, void* out,
                               float* out_scales, float* out_weights, void* stream)
{
    using namespace dpep;
    Workspace* w = as_workspace(ws);
    DPEP_REQUIRE(w != nullptr, "layout_dispatch_small: not a live workspace");
    DPEP_REQUIRE(num_tokens >= 1 && num_topk >= 1 && num_topk <= DPEP_MAX_TOPK &&
                     static_cast<long long>(num_tokens) * num_topk <= kSmallRoutes,
                 "layout_dispatch_small: T=%d K=%d: needs 1 <= T*K <= %d routes (larger batches take dpep_layout and a "
                 "dispatch call)", num_tokens, num_topk, kSmallRoutes);
    DPEP_REQUIRE(num_experts >= 1 && expert_begin >= 0 && num_local >= 1 && num_local <= DPEP_MAX_LOCAL_EXPERTS &&
                     expert_begin + num_local <= num_experts,
                 "layout_dispatch_small: bad expert range E=%d begin=%d L=%d", num_experts, expert_begin, num_local);
    DPEP_REQUIRE(topk_idx && counts && psum && offsets && route_to_row && row_to_route && num_rows, "layout_dispatch_small: NULL routing buffer");
    DPEP_REQUIRE(x && out && aligned16(x) && aligned16(out), "layout_dispatch_small: x/out must be 16-byte aligned");
    DPEP_REQUIRE((topk_weights == nullptr) == (out_weights == nullptr), "layout_dispatch_small: weights and out_weights go together");
    int units = 0;
    if (quantize) {
        DPEP_REQUIRE(row_bytes > 0 && row_bytes % 256 == 0 && row_bytes / 256 <= kMaxScaleCols,
                     "layout_dispatch_small: a quantised row needs a BF16 width that is a multiple of 128 (row_bytes=%d)", row_bytes);
        DPEP_REQUIRE(scales == nullptr && out_scales != nullptr, "layout_dispatch_small: the fused quantiser takes no input scales and needs out_scales");
        units = row_bytes / 32;
    } else {
        DPEP_REQUIRE(row_bytes > 0 && row_bytes % 16 == 0, "layout_dispatch_small: row_bytes=%d must be a positive multiple of 16", row_bytes);
        DPEP_REQUIRE((scales == nullptr) == (out_scales == nullptr), "layout_dispatch_small: scales and out_scales go together");
        DPEP_REQUIRE(scales == nullptr || scale_cols > 0, "layout_dispatch_small: scale_cols must be positive with scales");
        units = row_bytes / 16;
    }
    w->sequence = w->sequence == 0xffffffffu ? 1u : w->sequence + 1u;  // never 0: that is "nothing launched"
    w->mailbox_local = num_local;
    const Split sp = choose_split(num_tokens, units, 8);
    const int n_routes = num_tokens * num_topk;
    hipStream_t s = static_cast<hipStream_t>(stream);
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(num_tokens * sp.parts), dim3(kMaxThreads), 0, s,
                           reinterpret_cast<const long long*>(topk_idx), n_routes, num_experts, expert_begin, num_local, num_topk,
                           static_cast<const u32x4*>(x), quantize ? nullptr : scales, topk_weights, units, sp.per_part, sp.parts,
                           quantize ? 0 : scale_cols, counts, psum, offsets, num_rows, route_to_row, row_to_route,
                           static_cast<u32x4*>(out), out_scales, out_weights, w->mailbox_device, w->sequence);
    };
    if (num_topk <= 8) {
        if (quantize) launch(layout_dispatch_small_kernel<true, 8>);
        else launch(layout_dispatch_small_kernel<false, 8>);
    } else {
        if (quantize) launch(layout_dispatch_small_kernel<true, DPEP_MAX_TOPK>);
        else launch(layout_dispatch_small_kernel<false, DPEP_MAX_TOPK>);
    }
    return launch_status("layout_dispatch_small");
}

int dpep_cast_to_fp8(const void* x, int num_tokens, int hidden, void* out, float* out_scales, void* stream)
{
    using namespace dpep;
    DPEP_REQUIRE(num_tokens >= 0, "cast_to_fp8: bad T=%d", num_tokens);
    DPEP_REQUIRE(hidden > 0 && hidden % 16 == 0, "cast_to_fp8: hidden=%d must be a positive multiple of 16", hidden);
    if (num_tokens == 0) return DPEP_OK;
    DPEP_REQUIRE(x && out && out_scales && aligned16(x) && aligned16(out), "cast_to_fp8: x/out must be 16-byte aligned");
    const int units = hidden / 16;
    if (hidden % 128 != 0) {
        const int blocks = (hidden + 127) / 128;
        const long long padded = static_cast<long long>(num_tokens) * blocks * 8;
        hipLaunchKernelGGL(cast_to_fp8_short_block_kernel, dim3(static_cast<unsigned>((padded + 255) / 256)), dim3(256), 0,
                           static_cast<hipStream_t>(stream), static_cast<const u32x4*>(x), units, blocks, padded,
                           static_cast<u32x4*>(out), out_scales);
        return launch_status("cast_to_fp8");
    }
    const Split sp = choose_split(num_tokens, units, 8);
    with_store_policy([&](auto policy) {
        hipLaunchKernelGGL(dispatch_quant_row_kernel<decltype(policy)::value>, dim3(num_tokens * sp.parts),
                           dim3(sp.threads), 0, static_cast<hipStream_t>(stream), static_cast<const u32x4*>(x), nullptr,
                           nullptr, num_tokens, 1, units, sp.per_part, sp.parts, static_cast<u32x4*>(out), out_scales,
                           nullptr);
    });
    return launch_status("cast_to_fp8");
}

int dpep_cast_back(const void* codes, const void* scales, int scales_are_e8m0_bytes, int num_tokens, int hidden, void* out,
                   void* stream)
{
    using namespace dpep;
    DPEP_REQUIRE(num_tokens >= 0, "cast_back: bad T=%d", num_tokens);
    DPEP_REQUIRE(hidden > 0 && hidden % 16 == 0, "cast_back: hidden=%d must be a positive multiple of 16", hidden);
    if (num_tokens == 0) return DPEP_OK;
    DPEP_REQUIRE(codes && scales && out && aligned16(codes) && aligned16(out), "cast_back: codes/out must be 16-byte aligned");
    const int halves = hidden / 8, blocks_per_row = (hidden + 127) / 128;
    const long long total = static_cast<long long>(num_tokens) * halves;
    DPEP_REQUIRE((total + 255) / 256 < (1ll << 31), "cast_back: %d x %d codes are more than one launch takes", num_tokens, hidden);
    const unsigned grid = static_cast<unsigned>((total + 255) / 256);
    if (scales_are_e8m0_bytes)
        hipLaunchKernelGGL(cast_back_kernel<true>, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                           static_cast<const unsigned long long*>(codes), scales, halves, blocks_per_row, total, static_cast<u32x4*>(out));
    else
        hipLaunchKernelGGL(cast_back_kernel<false>, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                           static_cast<const unsigned long long*>(codes), scales, halves, blocks_per_row, total, static_cast<u32x4*>(out));
    return launch_status("cast_back");
}

}  // extern "C"
