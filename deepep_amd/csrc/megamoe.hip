// W4A8 expert FFN for one rank's local experts: MXFP8 (e4m3 + e8m0 per 32) activations times MXFP4
// (e2m1 + e8m0 per 32) weights on the gfx950 block-scaled MFMA, with a fused SwiGLU + MXFP8 requant
// epilogue after the first GEMM, grouped over ragged per-expert row counts.
//
// Numerics follow experiments/megamoe/python/deep_ep_experimental/megamoe/reference.py:44-100:
//   first = bf16(x @ w1^T); act = bf16(silu(gate) * up); qa = mx_quant(act); out = bf16(qa @ w2^T);
//   y[t] = bf16( sum_s w[t,s] * out[row(t,s)] )  (route weight applied after the second GEMM).
//
// Operand layout of v_mfma_scale_f32_32x32x64_f8f6f4 (fp8 A, fp4 B), as measured on gfx950:
//   A: lane l holds row l%32; VGPR 0-3 = k in [16g, 16g+16), VGPR 4-7 = k in [32+16g, 32+16g+16), g = l/32
//   B: lane l holds column l%32; 4 VGPRs = 32 nibbles k in [32g, 32g+32), low nibble first
//   scales: lane l supplies the e8m0 byte of (row or column l%32, 32-wide k block l/32)
//   D: acc[j] is row (j/4)*8 + (l/32)*4 + j%4, column l%32
#include <atomic>
#include <type_traits>
#include <utility>

#include "common.h"
#include "gemm_schedule.h"

#pragma clang fp contract(off)

namespace dpep {

int layout_i32(void* ws, const int32_t* idx, int num_tokens, int num_topk, int num_experts, int expert_begin,
               int num_local, int32_t* counts, int32_t* psum, int32_t* offsets, int32_t* route_to_row,
               int32_t* row_to_route, int32_t* num_rows, hipStream_t stream);
int combine_routes(const void* y, const float* route_weights, const int32_t* route_to_row, int num_tokens, int num_topk,
                   int num_rows_hint, int hidden, void* out, const int32_t* shared_first_row, int num_shared,
                   const int32_t* fill_state, int leave_unserved, hipStream_t stream);

namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose counter is a compile-time constant in
// the body (register arrays and instruction immediates are indexed by it).
template <typename F, int... I>
__device__ __forceinline__ void static_for_each(F&& f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    static_for_each(f, std::make_integer_sequence<int, N>{});
}

// =====================================================================================================
// MXFP8 activation quantiser (block 32 along the row)
// =====================================================================================================
// e8m0 byte of a block with maximum magnitude amax: biased_exponent(max(amax, 2^-119)) - 8.
__device__ __forceinline__ int mx_scale_byte(float amax)
{
    const float floored = fmaxf(amax, 0x1p-119f);
    return static_cast<int>(__float_as_uint(floored) >> 23) - 8;
}

// v * 2^(127 - byte), magnitude clamped to 448, rounded to e4m3fn (nearest even).
__device__ __forceinline__ float mx_scaled(float v, int byte)
{
    const float scaled = ldexpf(v, 127 - byte);
    return fminf(fmaxf(scaled, -448.0f), 448.0f);
}

__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d)
{
    int packed = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    packed = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, packed, true);
    return static_cast<uint32_t>(packed);
}

// One lane owns 16 consecutive BF16 values (32 bytes in, one 16-byte vector of codes out, consecutive lanes writing
// consecutive vectors); two adjacent lanes own one 32-element block.  The workgroup's 128 scale bytes are staged in LDS
// and leave as eight 16-byte stores instead of one byte-wide store per block, which turned every scale row into
// read-modify-write traffic.  The tensors are treated as flat arrays: hidden is a multiple of 32, so blocks never
// straddle rows.  Input and codes stream past the caches (the input is read once; with cached loads the kernel's time
// depended on what the caches held before: 48 us back to back, 89 us behind a 256 MiB fill, against 58-63 us this way
// under every protocol).  kVectorScales: the scale pointer is 16-byte aligned.
constexpr int kMxThreads = 256;

template <bool kVectorScales>
__global__ __launch_bounds__(kMxThreads) void mx_quant_kernel(const u32x4* __restrict__ x, long long num_units,
                                                              u32x4* __restrict__ codes, uint8_t* __restrict__ scales)
{
    __shared__ __attribute__((aligned(16))) uint8_t staged[kMxThreads / 2];
    const long long u = static_cast<long long>(blockIdx.x) * kMxThreads + threadIdx.x;
    const bool live = u < num_units;
    u32x4 raw[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
    if (live) {
        raw[0] = load16_nt(x + 2 * u);
        raw[1] = load16_nt(x + 2 * u + 1);
    }
    float v[16];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        v[2 * i] = bf16_to_f32(raw[i >> 2][i & 3] & 0xffffu);
        v[2 * i + 1] = bf16_to_f32(raw[i >> 2][i & 3] >> 16);
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(v[i]));
    amax = fmaxf(amax, __shfl_xor(amax, 1));
    const int byte = mx_scale_byte(amax);
    if (live) {
        u32x4 out;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            out[i] = pack4_e4m3(mx_scaled(v[4 * i], byte), mx_scaled(v[4 * i + 1], byte), mx_scaled(v[4 * i + 2], byte),
                                mx_scaled(v[4 * i + 3], byte));
        store16_nt(codes + u, out);
    }
    if ((threadIdx.x & 1) == 0) staged[threadIdx.x >> 1] = static_cast<uint8_t>(byte);
    __syncthreads();
    // blocks (= scale bytes) of this workgroup: [first, first + 128) clipped to the end
    const long long first = static_cast<long long>(blockIdx.x) * (kMxThreads / 2);
    const long long num_blocks = num_units >> 1;
    const int present = static_cast<int>(min(static_cast<long long>(kMxThreads / 2), num_blocks - first));
    if (kVectorScales && present == kMxThreads / 2) {
        if (threadIdx.x < kMxThreads / 32)
            store16_through(scales + first + threadIdx.x * 16, *reinterpret_cast<const u32x4*>(staged + threadIdx.x * 16));
    } else if (static_cast<int>(threadIdx.x) < present) {
        scales[first + threadIdx.x] = staged[threadIdx.x];
    }
}

// =====================================================================================================
// Weight re-layout: raw [L][N][K/2] + [L][N][K/32]  ->  1 KiB blocks holding every lane's 16-byte B fragment of
// one (column tile of 32, k step of 64), ordered [expert][256 columns][k tile of 128][column tile][k step] so
// that a workgroup's 16 KiB per item are contiguous; scales as 2 bytes per lane per k=128.
// =====================================================================================================
__device__ __forceinline__ int source_row(int physical_col, int n, int gate_up)
{
    if (!gate_up) return physical_col;
    // column tiles alternate gate / up for the same 32 activation columns
    const int tile = physical_col >> 5, j = physical_col & 31;
    const int act_col = (tile >> 1) * 32 + j;
    return (tile & 1) * (n >> 1) + act_col;
}

// n, k: the raw matrix; np, kp: what the GEMM works on (padded_dim of each; for gate/up both halves are padded, so
// np = 2 * padded_dim(n / 2)).  Padding columns and k blocks get zero codes (FP4 0.0) and the scale byte of 1.0.
__global__ __launch_bounds__(256) void prepare_weights_kernel(const uint8_t* __restrict__ w,
                                                              const uint8_t* __restrict__ s, int n, int k, int np, int kp,
                                                              int gate_up, uint8_t* __restrict__ w_out,
                                                              uint8_t* __restrict__ s_out, long long packed_chunks,
                                                              long long scale_pairs)
{
    const long long id = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int ktiles = kp / 128;
    // raw row of a physical (padded, interleaved) column, or -1 for a padding column
    auto raw_row = [&](int physical_col) {
        const int row = source_row(physical_col, np, gate_up);
        if (!gate_up) return row < n ? row : -1;
        const int half = np >> 1, in_half = row % half;
        return in_half < (n >> 1) ? (row / half) * (n >> 1) + in_half : -1;
    };
    if (id < packed_chunks) {
        // one 16-byte fragment; order [expert][block of 8 column tiles][k tile][column tile][k step][lane]: the
        // 16 KiB a workgroup copies per item are contiguous and its items follow each other in memory
        const int lane = id & 63, q = (id >> 6) & 15;
        long long rest = id >> 10;
        const int kt = rest % ktiles;
        rest /= ktiles;
        const int nb = rest % (np / 256);
        const long long e = rest / (np / 256);
        const int c = nb * 8 + (q >> 1), ks = kt * 2 + (q & 1);
        const int row = raw_row(c * 32 + (lane & 31));
        const int byte = ks * 32 + (lane >> 5) * 16;  // 16 bytes = 32 values of k, all inside the raw matrix or none
        u32x4 fragment = {0u, 0u, 0u, 0u};
        if (row >= 0 && byte * 2 < k) fragment = *reinterpret_cast<const u32x4*>(w + (e * n + row) * (k / 2) + byte);
        reinterpret_cast<u32x4*>(w_out)[id] = fragment;
    }
    if (id < scale_pairs) {
        // Scales: per (expert, block of 8 column tiles, span of 4 k tiles) one 4 KiB block
        // [column tile 8][lane 64][k tile 4][2 bytes = k blocks (2*kb + g) of that k tile]; a span is what
        // the GEMM copies in one go.  The last span is padded when kp % 512 != 0.
        const int spans = (ktiles + 3) / 4;
        const int kq = id & 3, lane = (id >> 2) & 63, c8 = (id >> 8) & 7;
        long long rest = id >> 11;
        const int span = rest % spans;
        rest /= spans;
        const int nb = rest % (np / 256);
        const long long e = rest / (np / 256);
        const int kt = span * 4 + kq;
        uint8_t lo = 127, hi = 127;
        const int row = raw_row((nb * 8 + c8) * 32 + (lane & 31));
        if (kt < ktiles && row >= 0) {
            const int block = kt * 4 + (lane >> 5);  // k blocks of 32: this lane half's two of the k tile
            const uint8_t* src = s + (e * n + row) * (k / 32);
            if (block < k / 32) lo = src[block];
            if (block + 2 < k / 32) hi = src[block + 2];
        }
        s_out[id * 2] = lo;
        s_out[id * 2 + 1] = hi;
    }
}

// Rows [T, h] of e4m3 codes with [T, h/32] scale bytes -> [T, hp] and [T, hp/32]: zero codes and the scale byte of
// 1.0 behind column h.  One thread per 16 output bytes (codes), then per scale byte.
__global__ __launch_bounds__(256) void pad_activations_kernel(const uint8_t* __restrict__ codes,
                                                              const uint8_t* __restrict__ scales, int h, int hp,
                                                              uint8_t* __restrict__ codes_out,
                                                              uint8_t* __restrict__ scales_out, long long code_units,
                                                              long long scale_bytes)
{
    const long long id = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id < code_units) {
        const long long row = id / (hp / 16);
        const int unit = static_cast<int>(id % (hp / 16));
        u32x4 v = {0u, 0u, 0u, 0u};
        if (unit * 16 < h) v = *reinterpret_cast<const u32x4*>(codes + row * h + unit * 16);
        reinterpret_cast<u32x4*>(codes_out)[id] = v;
    }
    if (id < scale_bytes) {
        const long long row = id / (hp / 32);
        const int block = static_cast<int>(id % (hp / 32));
        scales_out[id] = block < h / 32 ? scales[row * (h / 32) + block] : static_cast<uint8_t>(127);
    }
}

// =====================================================================================================
// Grouped GEMM
// =====================================================================================================
// Workgroup = 4 waves (2 row halves x 2 column halves), tile (64*RT) rows x 256 columns, k tile 128
// (two MFMA k steps) per LDS stage.  Workgroups are persistent (one per CU) and treat their tiles as ONE
// flat stream of (tile, k tile) items: asynchronous global->LDS copies run kAhead items ahead of the
// MFMAs and roll straight into the next tile, so a tile's epilogue overlaps the next tile's first copies.
// Per item there is one vmcnt wait + one barrier; the fragments of the next k step leave LDS while the
// MFMAs of the current one run.  A wave owns its SIMD alone and issues in order, so everything that is not
// an MFMA is placed in the shadow of one: the MFMAs are volatile asm statements (they keep source order;
// builtin MFMAs get gathered into bursts) and the item's copies are dealt out one after each MFMA.
// Scales and gather indices do not travel with every item (a 4-byte copy costs more per instruction than
// a 16-byte one): row scales (16 B per row = k 512), column scales (4 KiB per k 512) and
// the next tile's gather indices (once per tile) are fetched per span of four items.
// Rows are fetched 128 bytes at a time (full cache lines): the texture path handles about one line per
// cycle and CU, which a 64-byte k tile would saturate.
constexpr int kBK = 128;           // k per LDS stage = two MFMA k steps
constexpr int kCT = 4;             // 32-column MFMA tiles per wave
constexpr int kBN = 2 * kCT * 32;  // columns per workgroup tile
constexpr int kGemmThreads = 256;
constexpr int kGemmWaves = kGemmThreads / 64;
constexpr int kMaxMoeExperts = 128;
constexpr int kStagingRowStride = 80;  // 32 BF16 + 16 B pad: conflict-free 16-byte reads

template <int RT, bool kGather>
struct GemmCfg : GemmRing<RT> {
    using GemmRing<RT>::kStages;
    static constexpr int kBM = 64 * RT;
    static constexpr int kOffA = 0;                    // kBM rows x 128 B, 16-byte chunks XOR-swizzled
    static constexpr int kOffB = kBM * kBK;            // 8 column tiles x 2 k steps x 1 KiB fragments
    static constexpr int kStageBytes = kOffB + 16384;
    // Scales travel apart, once per span of four items, into three-slot rings: 16 bytes per row cover
    // k = 512 of row scales, and one 4 KiB block holds the column scales of the span.  (4-byte copies
    // are several times slower per instruction than 16-byte ones, and a 4-byte copy per row costs a
    // cache-line lookup per lane.)  Three slots, not two: a tile whose k is not a multiple of 512 ends with a span of
    // two items, and in a workgroup that goes on to another tile the copies, up to five items ahead, then reach the
    // span after next (two items + one: three items on) while the scales of the span before the short one are still
    // being read; with three slots the span that reuses a slot starts at least seven items behind the last read.
    static constexpr int kScaleSlots = 3;
    static constexpr int kRowScaleSlot = kBM * 16;
    static constexpr int kColScaleSlot = 4096;
    static constexpr int kOffRowScales = kStages * kStageBytes;
    static constexpr int kOffColScales = kOffRowScales + kScaleSlots * kRowScaleSlot;
    static constexpr int kStagingWave = 32 * kStagingRowStride;  // the epilogue handles one 32-row tile at a time
    static constexpr int kOffStaging = kOffColScales + kScaleSlots * kColScaleSlot;
    static constexpr int kLdsBytes = kOffStaging + 4 * kStagingWave;
};

struct GemmParams {
    const uint8_t* a_codes;    // [*, K] e4m3
    const uint8_t* a_scales;   // [*, K/32] e8m0
    const int* row_to_route;   // first GEMM: source row = row_to_route[r] / topk
    int topk;
    int a_rows;                // rows of a_codes (the gather clamps to them)
    const int* offsets;        // [L+1] exclusive row prefix per expert
    int num_local;
    const uint8_t* w;          // prepared fragments, expert stride N*K/2
    const uint8_t* ws;         // prepared scales, expert stride N*K/32
    int num_routed;            // experts >= num_routed are shared experts with weights of their own:
    const uint8_t* w_shared;   //   expert e reads w_shared / ws_shared at index e - num_routed
    const uint8_t* ws_shared;
    int n, k;
    uint8_t* act_codes;        // first GEMM: [rows, N/2] e4m3
    uint8_t* act_scales;       //             [rows, N/64] e8m0
    uint16_t* out;             // second GEMM: [rows, out_cols] bf16
    int out_cols;              //   columns that exist (<= N, a multiple of 8; the padding columns of N are not stored)
    // Zero rows of the final output.  When a launch has fewer tiles than workgroups, the workgroups left
    // without a tile stream zeros into the output rows of the tokens that no local expert serves (most tokens of a
    // rank's share), which the weighted reduce would otherwise have to write after the GEMMs: the stores cost the
    // matrix pipes nothing.  Every wave of such a workgroup is a filler f and takes tokens f, f + fillers, ...
    // until a workgroup with a tile reaches its epilogue and raises *fill_stop.  The word is a counter that only ever
    // grows (device memory of the workspace): a filler remembers the value it found when it started and stops when
    // the word differs, so nothing has to clear it, no value comes from the host, and every replay of a captured
    // launch stops its own fillers.  (Launches on a workspace run one after the other, so a filler's first read sees
    // every increment of the launches before it and none of its own launch: the first increment is a whole tile away.)
    // fill_state[0] = number of fillers, fill_state[1 + f] = tokens filler f got through.  All of it is null / zero in
    // launches that do not fill.
    u32x4* fill_out;                // [fill_tokens, fill_vec] or nullptr
    const int* fill_route_to_row;   // [fill_tokens, fill_topk]
    int fill_tokens, fill_vec, fill_topk;
    int* fill_state;
    int* fill_stop;
    int forced_rt;                  // 1..3: tile height 64 * forced_rt whatever the cost model says (tests); 0: the model decides
    int column_waves;               // 1: the kernel whose waves split the tile's columns and load their weights straight into registers
};

// gate / (1 + exp(-gate)) * up with the hardware exponential and reciprocal (v_exp_f32, v_rcp_f32: about 1 ulp each; the
// result is rounded to BF16 right after).  The clamp keeps exp finite, like the reference's clip(+-80).  (The
// reciprocal is the instruction itself: a correctly rounded 1 / x is a ten-instruction sequence per value, a third of the
// first GEMM's epilogue, for a last bit that the rounding to BF16 drops.)
__device__ __forceinline__ float silu_mul(float gate, float up)
{
    const float clipped = fminf(fmaxf(-gate, -80.0f), 80.0f);
    return gate * __builtin_amdgcn_rcpf(1.0f + __expf(clipped)) * up;
}

// Asynchronous copy global -> LDS: lane l's bytes land at lds_base + l * size.  lds_base is wave-uniform.
// Written as assembly so that the compiler's own wait-count bookkeeping does not serialise the ring;
// completion is awaited explicitly with wait_copies_then_barrier<N>().
__device__ __forceinline__ void copy16_to_lds(const void* src, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(base), "v"(src) : "memory");
}
// The same with the address split into a wave-uniform 64-bit base (SGPR pair) and a 32-bit lane offset.
__device__ __forceinline__ void copy16_to_lds(const void* uniform_base, uint32_t lane_offset, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(base), "v"(lane_offset),
                 "s"(uniform_base)
                 : "memory");
}
// The weight copies carry a cache hint chosen by how often a launch reads a weight tile.  kStreamed (64-row tiles: few
// rows per expert, every weight byte is read once or twice): non-temporal, which measured 10 % faster for the first GEMM
// of a decode-like share (32 local experts x 16 rows: 98 -> 88 us) and costs large batches 1.6 % (their row tiles
// re-read the weights from the L2); otherwise device-scope (`sc1`): 2 % faster at an EP64 rank's share, neutral for
// large batches.
template <bool kStreamed>
__device__ __forceinline__ void copy16_weights_to_lds(const void* uniform_base, uint32_t lane_offset, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    if (kStreamed)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(base), "v"(lane_offset),
                     "s"(uniform_base)
                     : "memory");
    else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 sc1" ::"s"(base), "v"(lane_offset),
                     "s"(uniform_base)
                     : "memory");
}
__device__ __forceinline__ void copy4_to_lds(const void* uniform_base, uint32_t lane_offset, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(base), "v"(lane_offset), "s"(uniform_base) : "memory");
}
__device__ __forceinline__ void copy4_to_lds(const void* src, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(base), "v"(src) : "memory");
}
// The same 16-byte copy, skipped when the (wave-uniform) value skip is not zero.  The jump stays inside
// the asm statement so that the loop body around it remains straight-line code.
__device__ __forceinline__ void copy16_to_lds_unless(const void* src, uint32_t lds_base, int skip)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    const int flag = __builtin_amdgcn_readfirstlane(skip);
    asm volatile(
        "s_mov_b32 m0, %0\n\ts_cmp_lg_u32 %2, 0\n\ts_cbranch_scc1 .Lskip_copy_%=\n\t"
        "global_load_lds_dwordx4 %1, off\n.Lskip_copy_%=:" ::"s"(base),
        "v"(src), "s"(flag)
        : "memory", "scc");
}
__device__ __forceinline__ void copy4_to_lds_unless(const void* uniform_base, uint32_t lane_offset, uint32_t lds_base, int skip)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    const int flag = __builtin_amdgcn_readfirstlane(skip);
    asm volatile(
        "s_mov_b32 m0, %0\n\ts_cmp_lg_u32 %3, 0\n\ts_cbranch_scc1 .Lskip_copy_%=\n\t"
        "global_load_lds_dword %1, %2\n.Lskip_copy_%=:" ::"s"(base),
        "v"(lane_offset), "s"(uniform_base), "s"(flag)
        : "memory", "scc");
}
__device__ __forceinline__ void copy4_to_lds_unless(const void* src, uint32_t lds_base, int skip)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    const int flag = __builtin_amdgcn_readfirstlane(skip);
    asm volatile(
        "s_mov_b32 m0, %0\n\ts_cmp_lg_u32 %2, 0\n\ts_cbranch_scc1 .Lskip_copy_%=\n\t"
        "global_load_lds_dword %1, off\n.Lskip_copy_%=:" ::"s"(base),
        "v"(src), "s"(flag)
        : "memory", "scc");
}
// Also waits for the wave's own LDS reads: past the barrier nothing reads the stage that is refilled next.
template <int kOutstanding>
__device__ __forceinline__ void wait_copies_then_barrier()
{
    // (Never weaken this for a timing experiment: the gather indices of the next tile travel through LDS too, so a
    // wave that runs ahead of a copy reads a stale index and fetches from a wild address.)
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(kOutstanding) : "memory");
}

// One scaled MFMA (FP8 A, FP4 B) as a volatile asm statement: volatile statements keep their source order,
// which is what lets the copies and the barrier be placed between individual MFMAs (builtin MFMAs are pure
// and the compiler gathers them into bursts).  kSecond selects scale bytes 2|3 of A and byte 1 of B.
// The compiler cannot see an MFMA in here, so the code that reads an accumulator afterwards has to
// provide the wait states itself (settle_accumulators).  For the same reason these statements must stay in
// straight-line code: with a branch around one the register allocator splits the accumulator's live range
// and copies it out of the AGPRs right behind the instruction, before its last passes have written
// (measured: accumulator registers 10-15 of every tile stale).
template <bool kSecond>
__device__ __forceinline__ void mfma_fp8_fp4(v16f& acc, const v8i& a, const u32x4& b, int scale_a, int scale_b)
{
    if (!kSecond)
        asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] blgp:4"
                     : "+a"(acc)
                     : "v"(a), "v"(b), "v"(scale_a), "v"(scale_b));
    else
        asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[0,1,0] op_sel_hi:[1,0,0] blgp:4"
                     : "+a"(acc)
                     : "v"(a), "v"(b), "v"(scale_a), "v"(scale_b));
}
// 16-pass MFMA results may be read by other instruction types 19 wait states after issue at the earliest.
__device__ __forceinline__ void settle_accumulators() { asm volatile("s_nop 15\n\ts_nop 7" ::: "memory"); }

struct TileInfo {
    int expert, nt, row0, valid;  // row0 = first row of the tile in the expanded layout; valid rows <= kBM
};

template <int RT, bool kGateUp>
__global__ __launch_bounds__(kGemmThreads, 1) void grouped_gemm_kernel(GemmParams p)
{
    constexpr bool kGather = kGateUp;
    using Cfg = GemmCfg<RT, kGather>;
    constexpr int kBM = Cfg::kBM, kStages = Cfg::kStages, kAhead = Cfg::kAhead, kStageBytes = Cfg::kStageBytes;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    __shared__ int tile_base[kMaxMoeExperts + 1];
    __shared__ int row_offsets[kMaxMoeExperts + 1];
    __shared__ int tile_index[2][kGemmThreads];  // row_to_route of a tile's rows; slots alternate per tile

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps LDS copy targets in SGPRs
    const int wm = wave >> 1, wn = wave & 1;
    const int g = lane >> 5, lr = lane & 31;
    const int n_tiles = p.n / kBN;
    const int ktiles = p.k / kBK;
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));
    const uint32_t lds_index = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(&tile_index[0][0]));

    // Tiles per expert: ceil(rows/kBM) row tiles x n_tiles column tiles, expert-major, row tile fastest.
    // (The offsets are fetched by one thread each, in parallel; only the tiny scan is serial.)
    if (tid <= p.num_local) row_offsets[tid] = p.offsets[tid];
    __syncthreads();
    if (tid == 0) {
        int total = 0;
        for (int e = 0; e < p.num_local; ++e) {
            tile_base[e] = total;
            const int rows = row_offsets[e + 1] - row_offsets[e];
            total += (rows + kBM - 1) / kBM * n_tiles;
        }
        tile_base[p.num_local] = total;
    }
    __syncthreads();
    const int total_tiles = tile_base[p.num_local];

    // Consecutive tile ids share weights; give each XCD (workgroups are dealt round-robin over 8 XCDs)
    // a contiguous range of tiles so that its L2 sees each weight tile from one place.  With fewer tiles than
    // workgroups: a launch that fills keeps the ranges whole, so that the first XCDs are full and the workgroups
    // without a tile, the fillers, sit together on the XCDs left over (their stores then stay out of the L2s the
    // GEMM works from: fillers on every XCD fill faster but cost the GEMM three times as much); a launch that
    // does not fill shrinks the ranges evenly (about 4 % faster than leaving two XCDs idle).
    const bool one_round = total_tiles < static_cast<int>(gridDim.x);
    const int fillers = one_round && p.fill_out != nullptr ? (static_cast<int>(gridDim.x) - total_tiles) * kGemmWaves : 0;
    const bool spread = one_round && fillers == 0 && (gridDim.x & 7) == 0;
    const int per_xcd = spread ? (total_tiles + 7) / 8 : (gridDim.x + 7) / 8;
    const int first = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    const int stride = one_round ? total_tiles + 1 : per_xcd * 8;  // one round: a single tile each
    const bool has_tile = first < total_tiles && (!spread || static_cast<int>(blockIdx.x >> 3) < per_xcd);
    if (blockIdx.x == 0 && tid == 0 && p.fill_state != nullptr) p.fill_state[0] = fillers;  // workgroup 0 always has tile 0
    if (!has_tile) {
        if (fillers == 0) return;
        const int filler = (first - total_tiles) * kGemmWaves + wave;
        const u32x4 zero = {0u, 0u, 0u, 0u};
        int done = 0;
        const int stop_at_start = __hip_atomic_load(p.fill_stop, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int token = filler; token < p.fill_tokens; token += fillers, ++done) {
            if (__hip_atomic_load(p.fill_stop, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != stop_at_start) break;
            const bool mine = lane < p.fill_topk && p.fill_route_to_row[static_cast<size_t>(token) * p.fill_topk + lane] >= 0;
            if (__ballot(mine) != 0ull) continue;  // some local expert serves the token: the reduce writes its row
            u32x4* row = p.fill_out + static_cast<size_t>(token) * p.fill_vec;
            for (int v = lane; v < p.fill_vec; v += 64) store16_nt(row + v, zero);
        }
        if (lane == 0) p.fill_state[1 + filler] = done;
        return;
    }
    const int my_tiles = one_round ? 1 : (total_tiles - first + stride - 1) / stride;

    auto decode = [&](int tile) {
        int e = 0;
        while (tile >= tile_base[e + 1]) ++e;
        const int row_begin = row_offsets[e], rows = row_offsets[e + 1] - row_begin;
        const int m_tiles = (rows + kBM - 1) / kBM;
        const int local = tile - tile_base[e];
        TileInfo info;
        info.expert = e;
        info.nt = local / m_tiles;
        const int m0 = (local % m_tiles) * kBM;
        info.row0 = row_begin + m0;
        info.valid = min(kBM, rows - m0);
        return info;
    };

    // ---- copy cursor -------------------------------------------------------------------------------
    // copy i of wave w fills LDS rows i*32 + w*8 + lane/8; chunk (lane%8) ^ ((row>>1)&7) of the 128-byte row
    const int a_chunk = ((lane & 7) ^ ((wave * 4 + (lane >> 4)) & 7)) * 16;
    uint32_t a_off[2 * RT];  // lane offsets from p.a_codes: source row * K + chunk
    const uint8_t* sa_src;
    uint32_t b_off[4];       // lane offsets from the tile's first weight fragment
    const uint8_t* b_base = p.w;
    const uint8_t* sb_src;
    const int* index_src = p.row_to_route;
    int copy_tile = first, copy_kt = 0, copy_stage = 0, copy_span = -1, copy_ordinal = 0;
    const int scale_bytes = p.k / 32;  // per row
    const int spans = (ktiles + 3) / 4;
    TileInfo next_info = decode(first);

    // Tile number j of this workgroup keeps its gather indices in tile_index[j & 1].
    auto point_at_tile = [&](const TileInfo& info) {
        const int* index = tile_index[copy_ordinal & 1];
        // rows past the tile's end repeat its last row
#pragma unroll
        for (int i = 0; i < 2 * RT; ++i) {
            const int r = min(i * 32 + wave * 8 + (lane >> 3), info.valid - 1);
            // (clamped: a map left incomplete by a layout launch that ran out of time must not become a wild address)
            const int src = kGather ? min(max(index[r] / p.topk, 0), p.a_rows - 1) : info.row0 + r;
            a_off[i] = static_cast<uint32_t>(src) * static_cast<uint32_t>(p.k) + a_chunk;
        }
        {
            // thread t serves row t % kBM (surplus waves repeat rows, which keeps every wave's copy count equal)
            const int r = min(tid % kBM, info.valid - 1);
            const int src = kGather ? min(max(index[r] / p.topk, 0), p.a_rows - 1) : info.row0 + r;
            sa_src = p.a_scales + static_cast<size_t>(src) * scale_bytes;
        }
        const bool shared = info.expert >= p.num_routed;
        const size_t weight_index = shared ? info.expert - p.num_routed : info.expert;
        b_base = (shared ? p.w_shared : p.w) + weight_index * p.n * (p.k / 2) +
                 static_cast<size_t>(info.nt) * ktiles * 16384;
        // fragment q = copy*4 + wave of the 16 (column tile, k step) fragments of one k tile
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int q = j * 4 + wave;
            b_off[j] = static_cast<uint32_t>(q * 1024 + lane * 16);
        }
        sb_src = (shared ? p.ws_shared : p.ws) + (weight_index * n_tiles + info.nt) * spans * Cfg::kColScaleSlot + tid * 16;
    };
    auto aim_index_prefetch = [&](const TileInfo& info) {
        if (kGather) index_src = p.row_to_route + info.row0 + min(tid, info.valid - 1);
    };

    // Copy number c (compile-time) of the item under the copy cursor; the pieces are issued between MFMAs.
    auto issue_copy = [&](int c) {
        const uint32_t stage = lds0 + copy_stage * kStageBytes;
        if (c < 2 * RT)
            copy16_to_lds(p.a_codes + static_cast<size_t>(copy_kt) * kBK, a_off[c], stage + Cfg::kOffA + c * 4096 + wave * 1024);
        else
            copy16_weights_to_lds<RT == 1>(b_base + static_cast<size_t>(copy_kt) * 16384, b_off[c - 2 * RT],
                          stage + Cfg::kOffB + ((c - 2 * RT) * 4 + wave) * 1024);
    };
    // Every fourth item starts a new span: a 16-byte window of row scales per row (clamped so that it never
    // leaves the row: k % 512 may be 256) and the span's 4 KiB of column scales.  A tile's first item also
    // fetches the gather indices of the workgroup's next tile.  These extra copies only make the counted
    // waits stricter.
    auto issue_span_copies = [&]() {
        if ((copy_kt & 3) == 0) copy_span = copy_span + 1 == Cfg::kScaleSlots ? 0 : copy_span + 1;
        const int window = min((copy_kt & ~3) * 4, scale_bytes - 16);
        const int slot = copy_span;
        copy16_to_lds_unless(sa_src + window, lds0 + Cfg::kOffRowScales + slot * Cfg::kRowScaleSlot + ((wave * 64) % kBM) * 16,
                             copy_kt & 3);
        copy16_to_lds_unless(sb_src + static_cast<size_t>(copy_kt >> 2) * Cfg::kColScaleSlot,
                             lds0 + Cfg::kOffColScales + slot * Cfg::kColScaleSlot + wave * 1024, copy_kt & 3);
        if (kGather) copy4_to_lds_unless(index_src, lds_index + ((copy_ordinal + 1) & 1) * (kGemmThreads * 4) + wave * 256, copy_kt);
    };
    // The cursor moves on after an item's copies: the next ring stage (advance_copy_stage), then the next k tile or tile.
    auto finish_copy_cursor = [&](bool in_prologue = false) {
        if (++copy_kt == ktiles) {
            if (copy_tile + stride < total_tiles) {
                // The next tile's indices were fetched with this tile's first item, so switching needs no global
                // load; they have landed unless the tile is too short for any counted wait to have covered that
                // fetch (gemm_schedule.h), in which case the cursor lets everything land first.
                if (kGather && switch_needs_drain(in_prologue, ktiles, kAhead)) wait_copies_then_barrier<0>();
                copy_tile += stride;
                copy_kt = 0;
                ++copy_ordinal;
                point_at_tile(next_info);
                if (copy_tile + stride < total_tiles) next_info = decode(copy_tile + stride);
                aim_index_prefetch(next_info);
            } else {
                copy_kt = ktiles - 1;  // past the last tile: keep re-copying its last item (never read)
            }
        }
    };
    auto advance_copy_cursor = [&](bool in_prologue) {
        copy_stage = copy_stage + 1 == kStages ? 0 : copy_stage + 1;
        finish_copy_cursor(in_prologue);
    };
    auto issue_item = [&]() {
#pragma unroll
        for (int c = 0; c < Cfg::kCopies; ++c) issue_copy(c);
        issue_span_copies();
        advance_copy_cursor(true);
    };

    // First tile: fetch its gather indices synchronously, then aim the prefetch at the second tile.
    if (kGather) {
        aim_index_prefetch(next_info);
        copy4_to_lds(index_src, lds_index + wave * 256);
        wait_copies_then_barrier<0>();
    }
    point_at_tile(next_info);
    if (first + stride < total_tiles) next_info = decode(first + stride);
    aim_index_prefetch(next_info);

    // ---- fragment addresses inside a stage ---------------------------------------------------------
    // Row tile i of a lane sits 32 rows = 4096 bytes below row tile 0 and has the same swizzle (32 rows is a multiple
    // of the swizzle period), so one set of lane addresses serves all row tiles with compile-time offsets.
    int a_addr[2][2];  // [k step][lo/hi 16 bytes] of row tile 0
    const int row_in_wave = wm * 32 * RT + lr;
    {
        const int sw = (row_in_wave >> 1) & 7;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            a_addr[kb][0] = Cfg::kOffA + row_in_wave * kBK + (((kb * 4 + g) ^ sw) << 4);
            a_addr[kb][1] = Cfg::kOffA + row_in_wave * kBK + (((kb * 4 + 2 + g) ^ sw) << 4);
        }
    }
    const int sa_addr = Cfg::kOffRowScales + row_in_wave * 16;  // row tile i: + i * 512
    const int b_addr = Cfg::kOffB + wn * kCT * 2048 + lane * 16;
    const int sb_addr = Cfg::kOffColScales + wn * kCT * 512 + lane * 8;

    v8i afrag[2][RT];     // [k step][row tile]
    u32x4 bfrag[2][kCT];  // [k step][column tile]
    int ascale[2][RT];    // [item parity][row tile]
    int bscale[2][kCT];
    // Fragment reads of one k step come in kGroups pieces (row tiles first, then column tiles) so that they can
    // be dealt out between MFMAs; the scale reads of an item likewise.
    constexpr int kGroups = RT + kCT;
    auto read_group = [&](int stage_index, int kb, int group) {
        const uint8_t* stage = lds + stage_index * kStageBytes;
        if (group < RT) {
            const int i = group;
            const u32x4 lo = *reinterpret_cast<const u32x4*>(stage + a_addr[kb][0] + i * (32 * kBK));
            const u32x4 hi = *reinterpret_cast<const u32x4*>(stage + a_addr[kb][1] + i * (32 * kBK));
            afrag[kb][i] = v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
        } else {
            const int c = group - RT;
            bfrag[kb][c] = *reinterpret_cast<const u32x4*>(stage + b_addr + (c * 2 + kb) * 1024);
        }
    };
    // row_at / col_at = byte offsets of the item's scales: ring slot + position inside the span
    auto read_scale_group = [&](int slot, int row_at, int col_at, int group) {
        if (group < RT)
            ascale[slot][group] = static_cast<int>(*reinterpret_cast<const uint32_t*>(lds + sa_addr + group * 512 + row_at));
        else
            bscale[slot][group - RT] =
                static_cast<int>(*reinterpret_cast<const uint16_t*>(lds + sb_addr + (group - RT) * 512 + col_at));
    };

    v16f acc[RT][kCT];
    auto clear_acc = [&]() {
#pragma unroll
        for (int i = 0; i < RT; ++i)
#pragma unroll
            for (int c = 0; c < kCT; ++c)
#pragma unroll
                for (int j = 0; j < 16; ++j) acc[i][c][j] = 0.0f;
    };
    // The row-scale word holds the four k blocks of the k tile; the upper lane half owns the odd ones
    // (shifted at use, not at the read, so that the read does not have to be waited for early).
    constexpr int kMfmas = RT * kCT;  // per k step
    int ashift[2][RT];  // row scale word moved so that this lane half's first k block is byte 0
    auto mfma_one = [&](int kb, int slot, int n) {
        const int c = n / RT, i = n % RT;
        if (kb == 0) mfma_fp8_fp4<false>(acc[i][c], afrag[0][i], bfrag[0][c], ashift[slot][i], bscale[slot][c]);
        else mfma_fp8_fp4<true>(acc[i][c], afrag[1][i], bfrag[1][c], ashift[slot][i], bscale[slot][c]);
    };
    auto shift_scales = [&](int slot) {
#pragma unroll
        for (int i = 0; i < RT; ++i) ashift[slot][i] = ascale[slot][i] >> (8 * g);
    };

    // ---- epilogue of one tile (per-wave staging region, no workgroup synchronisation) ----------------
    uint8_t* region = lds + Cfg::kOffStaging + wave * Cfg::kStagingWave;
    auto epilogue = [&](const TileInfo& info) {
        constexpr int kPasses = kGateUp ? kCT / 2 : kCT;
        // The staging region holds one 32 x 32 tile as BF16 rows.
#pragma unroll
        for (int i = 0; i < RT; ++i) {
            // The last row tile of the epilogue is about what a filler needs to finish the row it is on: tell them to
            // stop (the first workgroup to get here does; the others are at most a few microseconds behind).
            if (i == RT - 1 && fillers != 0 && tid == 0)
                __hip_atomic_fetch_add(p.fill_stop, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const int tile_rows = min(32, info.valid - wm * 32 * RT - 32 * i);  // may be <= 0
            const size_t out_row0 = static_cast<size_t>(info.row0) + wm * 32 * RT + 32 * i;
#pragma unroll
            for (int pass = 0; pass < kPasses; ++pass) {
#pragma unroll
                for (int j = 0; j < 16; j += 2) {
                    float value[2];
#pragma unroll
                    for (int d = 0; d < 2; ++d) {
                        if (kGateUp) {
                            // column tiles alternate gate / up for the same 32 activation columns
                            const uint32_t rounded = pack_bf16x2(acc[i][2 * pass][j + d], acc[i][2 * pass + 1][j + d]);
                            value[d] = silu_mul(__uint_as_float(rounded << 16), __uint_as_float(rounded & 0xffff0000u));
                        } else {
                            value[d] = acc[i][pass][j + d];
                        }
                    }
                    const uint32_t pair = pack_bf16x2(value[0], value[1]);  // rows r and r + 1 of this lane's column
                    const int r = (j >> 2) * 8 + g * 4 + (j & 3);
                    uint8_t* cell = region + r * kStagingRowStride + lr * 2;
                    *reinterpret_cast<uint16_t*>(cell) = static_cast<uint16_t>(pair);
                    *reinterpret_cast<uint16_t*>(cell + kStagingRowStride) = static_cast<uint16_t>(pair >> 16);
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                if (kGateUp) {
                    // two lanes requantise one row: 2 x 16 BF16 -> e8m0 byte + 32 e4m3 codes
                    const int act_width = p.n / 2;
                    const int act_col = (info.nt * kCT + wn * (kCT / 2) + pass) * 32;
                    const int r = lane >> 1, half = lane & 1;
                    float v[16];
#pragma unroll
                    for (int q = 0; q < 2; ++q) {
                        const u32x4 raw = *reinterpret_cast<const u32x4*>(region + r * kStagingRowStride + half * 32 + q * 16);
#pragma unroll
                        for (int t = 0; t < 4; ++t) {
                            v[q * 8 + 2 * t] = bf16_to_f32(raw[t] & 0xffffu);
                            v[q * 8 + 2 * t + 1] = bf16_to_f32(raw[t] >> 16);
                        }
                    }
                    float amax = 0.0f;
#pragma unroll
                    for (int t = 0; t < 16; ++t) amax = fmaxf(amax, fabsf(v[t]));
                    amax = fmaxf(amax, __shfl_xor(amax, 1));
                    const int byte = mx_scale_byte(amax);
                    u32x4 codes;
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        codes[t] = pack4_e4m3(mx_scaled(v[4 * t], byte), mx_scaled(v[4 * t + 1], byte),
                                              mx_scaled(v[4 * t + 2], byte), mx_scaled(v[4 * t + 3], byte));
                    if (r < tile_rows) {
                        *reinterpret_cast<u32x4*>(p.act_codes + (out_row0 + r) * act_width + act_col + half * 16) = codes;
                        if (half == 0)
                            p.act_scales[(out_row0 + r) * (act_width / 32) + (act_col >> 5)] = static_cast<uint8_t>(byte);
                    }
                } else {
                    // 4 lanes carry one 64-byte row segment
                    const int col = info.nt * kBN + (wn * kCT + pass) * 32 + (lane & 3) * 8;
#pragma unroll
                    for (int it = 0; it < 2; ++it) {
                        const int r = it * 16 + (lane >> 2);
                        if (r < tile_rows && col < p.out_cols) {
                            const u32x4 chunk = *reinterpret_cast<const u32x4*>(region + r * kStagingRowStride + (lane & 3) * 16);
                            // cached store: the weighted reduce that follows reads these rows back at once
                            *reinterpret_cast<u32x4*>(p.out + (out_row0 + r) * p.out_cols + col) = chunk;
                        }
                    }
                }
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
        }
    };

    // ---- the flat item stream --------------------------------------------------------------------------
#pragma unroll
    for (int j = 0; j < kAhead; ++j) issue_item();
    wait_copies_then_barrier<(kAhead - 1) * Cfg::kCopies>();  // item 0 has landed
    // Scale bookkeeping of the item whose fragments are read next: span counter (ring slot) and k tile.
    int read_span = -1, read_kt = 0;
    int row_at = 0, col_at = 0;
    auto next_scale_offsets = [&]() {
        if ((read_kt & 3) == 0) read_span = read_span + 1 == Cfg::kScaleSlots ? 0 : read_span + 1;
        const int window = min((read_kt & ~3) * 4, scale_bytes - 16);
        const int ring = read_span;
        row_at = ring * Cfg::kRowScaleSlot + (read_kt * 4 - window);
        col_at = ring * Cfg::kColScaleSlot + (read_kt & 3) * 2;
        read_kt = read_kt + 1 == ktiles ? 0 : read_kt + 1;
    };
    next_scale_offsets();
#pragma unroll
    for (int group = 0; group < kGroups; ++group) {
        read_scale_group(0, row_at, col_at, group);
        read_group(0, 0, group);
    }
    clear_acc();
    asm volatile("s_nop 3");
    int stage_now = 0;  // stage of the item whose MFMAs run
    int tile = first, kt = 0;
    TileInfo info = decode(first);
    const long long total_items = static_cast<long long>(my_tiles) * ktiles;
    for (long long item = 0; item < total_items; item += 2) {
#pragma unroll
        for (int parity = 0; parity < 2; ++parity) {  // ktiles is even, so tiles start on even items
            const int stage_next = stage_now + 1 == kStages ? 0 : stage_now + 1;
            // A wave issues in order and owns its SIMD alone, so whatever is not an MFMA should sit in the
            // shadow of one.  First k step: its MFMAs are followed, one piece each, by the LDS reads of the
            // second k step's fragments and, once the barrier has passed, by the copies of the item kAhead
            // ahead.  Second k step: the remaining copies in its first half, then the item's scale / index copies and
            // the copy cursor's arithmetic, and all along the reads of the next item's scales and first fragments
            // (whose registers the first k step has released).
            shift_scales(parity);
            constexpr int kSlots = kMfmas;  // MFMAs behind the barrier that deal out the item's copies
            // enough read groups per MFMA that the second k step's fragments have all left LDS before the barrier
            constexpr int kReadsPerMfma = (kGroups + kMfmas / 2 - 1) / (kMfmas / 2);
#pragma unroll
            for (int n = 0; n < kMfmas; ++n) {
                mfma_one(0, parity, n);
#pragma unroll
                for (int group = kReadsPerMfma * n; group < kReadsPerMfma * (n + 1); ++group)
                    if (group < kGroups) read_group(stage_now, 1, group);
                if (n == kMfmas / 2 - 1) {
                    // item+1 has landed for every thread once each has at most kAhead-2 items of its own copies
                    // in flight; past the barrier every wave has also finished reading the stage refilled next.
                    wait_copies_then_barrier<Cfg::kWaitPlain>();
                }
                if (n >= kMfmas / 2) {
                    const int slot = n - kMfmas / 2;
#pragma unroll
                    for (int c = slot * Cfg::kCopies / kSlots; c < (slot + 1) * Cfg::kCopies / kSlots; ++c) issue_copy(c);
                }
            }
            next_scale_offsets();
#pragma unroll
            for (int n = 0; n < kMfmas; ++n) {
                mfma_one(1, parity, n);
                const int slot = n + kMfmas / 2;
                if (slot < kSlots) {
#pragma unroll
                    for (int c = slot * Cfg::kCopies / kSlots; c < (slot + 1) * Cfg::kCopies / kSlots; ++c) issue_copy(c);
                }
                // 2*kGroups read pieces for the next item: its scales first (they are shifted first), then fragments
#pragma unroll
                for (int piece = n * 2 * kGroups / kMfmas; piece < (n + 1) * 2 * kGroups / kMfmas; ++piece) {
                    if (piece < kGroups) read_scale_group(parity ^ 1, row_at, col_at, piece);
                    else read_group(stage_next, 0, piece - kGroups);
                }
                if (n == kMfmas / 2) {
                    // Every regular copy of the item is out: its scale / index copies and the cursor's stage arithmetic go
                    // under the remaining MFMAs instead of behind the last one, where the matrix pipe would drain
                    // meanwhile (45 scalar instructions used to sit there).  The counted waits only get stricter by it.
                    issue_span_copies();
                    copy_stage = copy_stage + 1 == kStages ? 0 : copy_stage + 1;
                    asm volatile("" : "+s"(copy_stage));  // computed here, not sunk to the end of the item
                }
            }
            finish_copy_cursor();
            stage_now = stage_next;
        }
        kt += 2;
        // (marked unlikely: the register allocator then keeps the loop's values in place and does its shuffling around the
        // epilogue, once per tile, instead of at the head of the item loop)
        if (__builtin_expect(kt == ktiles, 0)) {
                    settle_accumulators();
            // tie every accumulator to a statement behind the wait, so that no read of it can be moved above
#pragma unroll
            for (int i = 0; i < RT; ++i)
#pragma unroll
                for (int c = 0; c < kCT; ++c) asm volatile("" : "+a"(acc[i][c]));
            epilogue(info);
                    clear_acc();
            asm volatile("s_nop 3");  // accumulator writes settle before the next MFMA reads them
            kt = 0;
            tile += stride;
            if (tile < total_tiles) info = decode(tile);
        }
    }
    // No copy may still be in flight into this workgroup's LDS when it retires.
    wait_copies_then_barrier<0>();
}

// =====================================================================================================
// Grouped GEMM, column-wave form: the weights go straight from memory to registers
// =====================================================================================================
// The prepared weight layout already is the per-lane B operand of the scaled MFMA, so a wave that owns whole
// 32-column tiles can load its weight fragments with plain 16-byte loads and never share them.  Here the four waves
// split the tile's 256 columns (64 each: two column tiles; for the first GEMM one gate / up pair) and every wave covers
// ALL the tile's rows (2 * RT row tiles of 32): the same RT * 4 accumulator tiles per wave as the 2 x 2 form, but the
// weights need no LDS write, no LDS read and no barrier, and the LDS ring holds activations only (8 KiB * RT per
// stage), which buys a fourth stage at 192 rows.  The ring has exactly as many stages as the item loop is unrolled
// (4): an item's stage, its weight registers and the selection of its scale bytes are all compile-time constants,
// the LDS target of a copy is one scalar add away from a per-wave base, and a tile ends only behind the fourth body
// (k is a multiple of 512 here).  Everything of item i + 4 is requested in the body of item i, so the one counted wait
// per item lets two whole items of copies and loads stay in flight.
// The weight fragments of the four items in flight live in the 64 accumulation registers behind the accumulators (a[192:255]
// at 192 rows), which the loads and the
// MFMAs name themselves: the compiler never sees them as values.  It could not be trusted with them: a register that
// an asynchronous load has been told to fill counts as defined right behind the load, and a register allocator that moves
// such a value (it parked weight fragments in spare registers when they were ordinary operands) copies what the register
// held BEFORE the load landed.  Every weight load declares all 64 clobbered, so nothing the compiler keeps alive in
// the loop can sit there (the accumulators end up below); that it also puts no short-lived value
// there is checked on the generated code by tests/test_gemm_registers.py.  Column scales travel through LDS like the row
// scales (each wave copies and reads only the 1 KiB of its own two column tiles).
template <int RT>
struct ColCfg : ColumnRing<RT> {
    using ColumnRing<RT>::kStages;                     // LDS stages = items the requests run ahead = unroll of the item loop
    static constexpr int kBM = 64 * RT;
    static constexpr int kRowTiles = 2 * RT;           // 32-row MFMA tiles per workgroup tile, all of them on every wave
    static constexpr int kColTiles = 2;                // 32-column MFMA tiles per wave
    static constexpr int kStageBytes = kBM * kBK;      // activations only
    static constexpr int kRowScaleSlot = kBM * 16;
    static constexpr int kOffRowScales = kStages * kStageBytes;
    static constexpr int kColScaleSlot = 4096;
    static constexpr int kOffColScales = kOffRowScales + 2 * kRowScaleSlot;
    static constexpr int kLdsBytes = kOffColScales + 2 * kColScaleSlot;
    static_assert(ColumnRing<RT>::kRequests == kRowTiles + 2 * kColTiles, "per thread and item: activation copies + weight loads");
    // 64-row tiles leave room (200 registers per lane, 53 KiB of LDS) for two workgroups on a CU: launches of that height are
    // bound by streaming their weights, and a second workgroup doubles the requests in flight
    static constexpr int kWorkgroupsPerCu = RT == 1 ? 2 : 1;
    static constexpr int kWeightRegs = 64 * RT;  // first of the 64 accumulation registers that hold weight fragments: right behind the accumulators
};

// Asynchronous 16-byte copy global -> LDS whose LDS address is a per-wave base (SGPR) plus a compile-time constant.
template <int kLdsConst>
__device__ __forceinline__ void copy16_to_lds_at(const void* uniform_base, uint32_t lane_offset, uint32_t wave_lds_base)
{
    asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3" ::"s"(wave_lds_base), "n"(kLdsConst),
                 "v"(lane_offset), "s"(uniform_base)
                 : "memory", "scc");
}
// The 64 registers of the weight fragments, as clobber lists: they follow the accumulators (64 * RT registers), so that a
// kernel with few accumulators also needs few registers in all.
#define DPEP_WEIGHT_REGS_64 \
    "a64", "a65", "a66", "a67", "a68", "a69", "a70", "a71", "a72", "a73", "a74", "a75", "a76", "a77", "a78", "a79",    \
        "a80", "a81", "a82", "a83", "a84", "a85", "a86", "a87", "a88", "a89", "a90", "a91", "a92", "a93", "a94",       \
        "a95", "a96", "a97", "a98", "a99", "a100", "a101", "a102", "a103", "a104", "a105", "a106", "a107", "a108",     \
        "a109", "a110", "a111", "a112", "a113", "a114", "a115", "a116", "a117", "a118", "a119", "a120", "a121",        \
        "a122", "a123", "a124", "a125", "a126", "a127"
#define DPEP_WEIGHT_REGS_128 \
    "a128", "a129", "a130", "a131", "a132", "a133", "a134", "a135", "a136", "a137", "a138", "a139", "a140", "a141",    \
        "a142", "a143", "a144", "a145", "a146", "a147", "a148", "a149", "a150", "a151", "a152", "a153", "a154",        \
        "a155", "a156", "a157", "a158", "a159", "a160", "a161", "a162", "a163", "a164", "a165", "a166", "a167",        \
        "a168", "a169", "a170", "a171", "a172", "a173", "a174", "a175", "a176", "a177", "a178", "a179", "a180",        \
        "a181", "a182", "a183", "a184", "a185", "a186", "a187", "a188", "a189", "a190", "a191"
#define DPEP_WEIGHT_REGS_V192 \
    "v192", "v193", "v194", "v195", "v196", "v197", "v198", "v199", "v200", "v201", "v202", "v203", "v204", "v205",    \
        "v206", "v207", "v208", "v209", "v210", "v211", "v212", "v213", "v214", "v215", "v216", "v217", "v218",        \
        "v219", "v220", "v221", "v222", "v223", "v224", "v225", "v226", "v227", "v228", "v229", "v230", "v231",        \
        "v232", "v233", "v234", "v235", "v236", "v237", "v238", "v239", "v240", "v241", "v242", "v243", "v244",        \
        "v245", "v246", "v247", "v248", "v249", "v250", "v251", "v252", "v253", "v254", "v255"
// Asynchronous 16-byte load into the weight registers kReg .. kReg + 3.  Nothing is an output as far as the compiler knows.
// kFirst: the first of the kernel's 64 weight registers (all of them are declared clobbered, whichever four are loaded).
// At 64 and 128 rows they are accumulation registers right behind the accumulators (a64.. / a128..); at 192 rows, where the
// accumulators fill 192 of the 256 accumulation registers, they are the ordinary registers v192..v255 (the kernel's own
// values need fewer than 150, and with every accumulation register taken the register allocator started to put
// loop-carried values on the stack).
#define DPEP_WEIGHT_LOAD(file, hint, clobbers)                                                                                  \
    asm volatile("global_load_dwordx4 " file "[%3:%4], %0, %1 offset:%2 " hint ::"v"(lane_offset), "s"(uniform_base), "n"(kImm), \
                 "n"(kReg), "n"(kReg + 3)                                                                                       \
                 : "memory", clobbers)
template <int kFirst, int kReg, int kImm, bool kStreamed>
__device__ __forceinline__ void load16_to_weight_regs(const void* uniform_base, uint32_t lane_offset)
{
    static_assert(kFirst == 64 || kFirst == 128 || kFirst == 192, "weight registers start at a64, a128 or a192");
    static_assert(kReg >= kFirst && kReg + 3 < kFirst + 64, "not one of the kernel's weight registers");
    if constexpr (kFirst == 64) {
        if (kStreamed) DPEP_WEIGHT_LOAD("a", "nt", DPEP_WEIGHT_REGS_64);
        else DPEP_WEIGHT_LOAD("a", "sc1", DPEP_WEIGHT_REGS_64);
    } else if constexpr (kFirst == 128) {
        if (kStreamed) DPEP_WEIGHT_LOAD("a", "nt", DPEP_WEIGHT_REGS_128);
        else DPEP_WEIGHT_LOAD("a", "sc1", DPEP_WEIGHT_REGS_128);
    } else {
        if (kStreamed) DPEP_WEIGHT_LOAD("v", "nt", DPEP_WEIGHT_REGS_V192);
        else DPEP_WEIGHT_LOAD("v", "sc1", DPEP_WEIGHT_REGS_V192);
    }
}
// Scaled MFMA with the operands the other way round: the weights (FP4, a[kReg : kReg + 3]) are the instruction's A
// operand and the activations (FP8) its B operand, so the result comes out transposed: lane l holds activation row
// l % 32, and acc[j] is weight column (j/4)*8 + (l/32)*4 + j%4 of the tile: four consecutive columns per group of
// four registers.  A lane's results are then pieces of ONE output row, which the epilogue can store from registers (the
// other way round a lane holds sixteen rows of one column, and the tile has to be transposed through LDS).  The scale bytes
// are chosen at compile time: byte kByteW of scale_w, byte kByteX of scale_x.
template <int kReg, int kByteW, int kByteX>
__device__ __forceinline__ void mfma_fp4_fp8_regs(v16f& acc, const v8i& x, int scale_w, int scale_x)
{
    if constexpr (kReg >= 192)  // (192-row kernels keep their weights in v192..v255, the others behind their accumulators)
        asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, v[%8:%9], %1, %0, %2, %3 op_sel:[%4,%5,0] op_sel_hi:[%6,%7,0] cbsz:4"
                     : "+a"(acc)
                     : "v"(x), "v"(scale_w), "v"(scale_x), "n"(kByteW & 1), "n"(kByteX & 1), "n"(kByteW >> 1), "n"(kByteX >> 1),
                       "n"(kReg), "n"(kReg + 3));
    else
        asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, a[%8:%9], %1, %0, %2, %3 op_sel:[%4,%5,0] op_sel_hi:[%6,%7,0] cbsz:4"
                     : "+a"(acc)
                     : "v"(x), "v"(scale_w), "v"(scale_x), "n"(kByteW & 1), "n"(kByteX & 1), "n"(kByteW >> 1), "n"(kByteX >> 1),
                       "n"(kReg), "n"(kReg + 3));
}

// The lane's number, worked out on the spot (two instructions) instead of kept in a register: the code that runs once
// per tile or span (tile switches, scale requests, the epilogue) takes its lane-dependent addresses from this, so that the
// item loop does not have to carry them.
__device__ __forceinline__ int lane_now()
{
    int lane;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane));
    return lane;
}

template <int RT, bool kGateUp>
__global__ __launch_bounds__(kGemmThreads, ColCfg<RT>::kWorkgroupsPerCu) void grouped_gemm_colwave_kernel(GemmParams p)
{
    constexpr bool kGather = kGateUp;
    using Cfg = ColCfg<RT>;
    constexpr int kBM = Cfg::kBM, kStages = Cfg::kStages, kStageBytes = Cfg::kStageBytes, kRowTiles = Cfg::kRowTiles;
    constexpr int kCols = Cfg::kColTiles;
    constexpr bool kStreamed = RT == 1;  // few rows per expert: every weight byte is read once or twice
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    __shared__ int tile_base[kMaxMoeExperts + 1];
    __shared__ int row_offsets[kMaxMoeExperts + 1];
    __shared__ int tile_index[2][kGemmThreads];  // row_to_route of a tile's rows; slots alternate per tile
    // Where each thread's copies of the tile under the cursor start: [0 .. kRowTiles-1] byte offsets of its activation rows
    // from a_codes, [kRowTiles] of its row of scale bytes from a_scales.  Written at tile switches, read back right before
    // each copy: kept in registers instead, they are values that live across the whole item loop, and the register
    // allocator has put such values on the stack (every reload from there waits for all the copies in flight).
    __shared__ uint32_t copy_offsets[ColCfg<RT>::kRowTiles + 1][kGemmThreads];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 5, lr = lane & 31;
    const int n_tiles = p.n / kBN;
    const int ktiles = p.k / kBK;  // a multiple of 4
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));
    const uint32_t lds_index = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(&tile_index[0][0]));
    const uint32_t wave_lds = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);

    if (tid <= p.num_local) row_offsets[tid] = p.offsets[tid];
    __syncthreads();
    if (tid == 0) {
        int total = 0;
        for (int e = 0; e < p.num_local; ++e) {
            tile_base[e] = total;
            const int rows = row_offsets[e + 1] - row_offsets[e];
            total += (rows + kBM - 1) / kBM * n_tiles;
        }
        tile_base[p.num_local] = total;
    }
    __syncthreads();
    const int total_tiles = tile_base[p.num_local];

    // Tiles to workgroups, and what the workgroups without a tile do: as in grouped_gemm_kernel.
    const bool one_round = total_tiles < static_cast<int>(gridDim.x);
    const int fillers = one_round && p.fill_out != nullptr ? (static_cast<int>(gridDim.x) - total_tiles) * kGemmWaves : 0;
    const bool spread = one_round && fillers == 0 && (gridDim.x & 7) == 0;
    const int per_xcd = spread ? (total_tiles + 7) / 8 : (gridDim.x + 7) / 8;
    const int first = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    const int stride = one_round ? total_tiles + 1 : per_xcd * 8;
    const bool has_tile = first < total_tiles && (!spread || static_cast<int>(blockIdx.x >> 3) < per_xcd);
    if (blockIdx.x == 0 && tid == 0 && p.fill_state != nullptr) p.fill_state[0] = fillers;
    if (!has_tile) {
        if (fillers == 0) return;
        const int filler = (first - total_tiles) * kGemmWaves + wave;
        const u32x4 zero = {0u, 0u, 0u, 0u};
        int done = 0;
        const int stop_at_start = __hip_atomic_load(p.fill_stop, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int token = filler; token < p.fill_tokens; token += fillers, ++done) {
            if (__hip_atomic_load(p.fill_stop, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != stop_at_start) break;
            const bool mine = lane < p.fill_topk && p.fill_route_to_row[static_cast<size_t>(token) * p.fill_topk + lane] >= 0;
            if (__ballot(mine) != 0ull) continue;
            u32x4* row = p.fill_out + static_cast<size_t>(token) * p.fill_vec;
            for (int v = lane; v < p.fill_vec; v += 64) store16_nt(row + v, zero);
        }
        if (lane == 0) p.fill_state[1 + filler] = done;
        return;
    }
    const int my_tiles = one_round ? 1 : (total_tiles - first + stride - 1) / stride;

    auto decode = [&](int tile) {
        int e = 0;
        while (tile >= tile_base[e + 1]) ++e;
        const int row_begin = row_offsets[e], rows = row_offsets[e + 1] - row_begin;
        const int m_tiles = (rows + kBM - 1) / kBM;
        const int local = tile - tile_base[e];
        // Inside an expert the tiles are numbered panel by panel: kPanel column tiles wide (the last panel may be
        // narrower), all row tiles high, row by row.  The 32 consecutive tiles an XCD works on at a time are then a block of
        // about 4 row tiles x 8 column tiles, whose activation rows and weight columns that XCD's L2 fetches once, instead
        // of every row tile of a few column tiles (which made each of the eight XCDs fetch all the rows of a large expert).
        constexpr int kPanel = 8;
        const int panel = local / (m_tiles * kPanel), in_panel = local - panel * (m_tiles * kPanel);
        const int width = min(kPanel, n_tiles - panel * kPanel);
        TileInfo info;
        info.expert = e;
        info.nt = panel * kPanel + in_panel % width;
        const int m0 = (in_panel / width) * kBM;
        info.row0 = row_begin + m0;
        info.valid = min(kBM, rows - m0);
        return info;
    };

    // ---- request cursor: what is asked for next (activation copies, weight loads, scales, gather indices) ----------
    // activation copy c of wave w fills LDS rows c*32 + w*8 + lane/8; chunk (lane%8) ^ ((row>>1)&7) of the 128-byte row
    auto a_chunk_of = [&](int l) { return ((l & 7) ^ ((wave * 4 + (l >> 4)) & 7)) * 16; };
    const uint32_t* my_offsets = &copy_offsets[0][tid];  // entry i: + i * kGemmThreads
    const uint32_t b_lane = static_cast<uint32_t>(wave * 4096 + lane * 16);  // this wave's four fragments of an item are contiguous
    const uint8_t* b_base = p.w;
    const uint8_t* sb_base = p.ws;  // column scales of the tile under the cursor (thread t copies bytes 16 t .. 16 t + 15 of a span)
    int index_row0 = 0, index_valid = 1;  // rows whose gather indices are fetched next
    int copy_tile = first, copy_kt = 0, copy_span = -1, copy_ordinal = 0;
    const int scale_bytes = p.k / 32;  // per row
    const int spans = ktiles / 4;
    TileInfo next_info = decode(first);

    auto point_at_tile = [&](const TileInfo& info) {
        const int* index = tile_index[copy_ordinal & 1];
        // (the lane's row numbers are worked out afresh at every tile switch: kept in registers across the item loop
        // they cost the loop a register each, or a place on the stack)
        const int lane_here = lane_now(), tid_here = wave * 64 + lane_here;
#pragma unroll
        for (int i = 0; i < kRowTiles; ++i) {
            const int r = min(i * 32 + wave * 8 + (lane_here >> 3), info.valid - 1);  // rows past the tile's end repeat its last row
            const int src = kGather ? min(max(index[r] / p.topk, 0), p.a_rows - 1) : info.row0 + r;
            copy_offsets[i][tid_here] = static_cast<uint32_t>(src) * static_cast<uint32_t>(p.k) + a_chunk_of(lane_here);
        }
        {
            const int r = min(tid_here % kBM, info.valid - 1);
            const int src = kGather ? min(max(index[r] / p.topk, 0), p.a_rows - 1) : info.row0 + r;
            copy_offsets[kRowTiles][tid_here] = static_cast<uint32_t>(src) * static_cast<uint32_t>(scale_bytes);
        }
        const bool shared = info.expert >= p.num_routed;
        const size_t weight_index = shared ? info.expert - p.num_routed : info.expert;
        b_base = (shared ? p.w_shared : p.w) + weight_index * p.n * (p.k / 2) + static_cast<size_t>(info.nt) * ktiles * 16384;
        sb_base = (shared ? p.ws_shared : p.ws) + (weight_index * n_tiles + info.nt) * spans * Cfg::kColScaleSlot;
    };
    auto aim_index_prefetch = [&](const TileInfo& info) {
        index_row0 = info.row0;
        index_valid = info.valid;
    };
    auto index_offset = [&]() {  // this thread's entry of row_to_route, in bytes
        return static_cast<uint32_t>(index_row0 + min(wave * 64 + lane_now(), index_valid - 1)) * 4u;
    };

    // Column scales of the current span and of the next one: [column tile] x 8 bytes = k tiles 0..3 x k steps 0..1.
    u32x2 bscale_now[kCols], bscale_next[kCols];

    // The requests of the item under the cursor, which goes to ring position kPos; issued in pieces between MFMAs.
    auto request_activations_at = [&](auto pos, auto piece, uint32_t offset) {
        constexpr int kPos = decltype(pos)::value, kPiece = decltype(piece)::value;
        copy16_to_lds_at<kPos * kStageBytes + kPiece * 4096>(p.a_codes + static_cast<size_t>(copy_kt) * kBK, offset, wave_lds);
    };
    auto request_activations = [&](auto pos, auto piece) {
        request_activations_at(pos, piece, my_offsets[decltype(piece)::value * kGemmThreads]);
    };
    auto request_weights = [&](auto pos, auto step) {
        constexpr int kPos = decltype(pos)::value, kStep = decltype(step)::value;
        const uint8_t* item = b_base + static_cast<size_t>(copy_kt) * 16384;
        // fragment (column tile c, k step) of the wave's four: 2048 c + 1024 step bytes in; registers 16 pos + 8 step + 4 c
        constexpr int kReg = Cfg::kWeightRegs + 16 * kPos + 8 * kStep;
        load16_to_weight_regs<Cfg::kWeightRegs, kReg, kStep * 1024, kStreamed>(item, b_lane);
        load16_to_weight_regs<Cfg::kWeightRegs, kReg + 4, 2048 + kStep * 1024, kStreamed>(item, b_lane);
    };
    // A span's first item (ring position 0) also asks for the span's scales, into the LDS slots of the span's parity: 16
    // bytes of row scales per row and the span's 4 KiB of column scales.  A tile's first item asks for the gather indices of
    // the workgroup's next tile.
    auto request_span = [&]() {
        ++copy_span;
        const int window = min(copy_kt * 4, scale_bytes - 16);
        copy16_to_lds(p.a_scales + window, my_offsets[kRowTiles * kGemmThreads], lds0 + Cfg::kOffRowScales + (copy_span & 1) * Cfg::kRowScaleSlot + ((wave * 64) % kBM) * 16);
        copy16_to_lds(sb_base + static_cast<size_t>(copy_kt >> 2) * Cfg::kColScaleSlot, static_cast<uint32_t>(wave * 1024 + lane_now() * 16),
                      lds0 + Cfg::kOffColScales + (copy_span & 1) * Cfg::kColScaleSlot + wave * 1024);
        if (kGather)
            copy4_to_lds_unless(p.row_to_route, index_offset(), lds_index + ((copy_ordinal + 1) & 1) * (kGemmThreads * 4) + wave * 256, copy_kt);
    };
    // (k tiles come in fours, so a tile can only end behind ring position 3)
    auto advance_cursor = [&](bool in_prologue, bool last_of_four) {
        ++copy_kt;
        if (last_of_four && copy_kt == ktiles) {
            if (copy_tile + stride < total_tiles) {
                // (a tile has at least four items, so only a switch inside the prologue can come before a counted wait
                // has covered the fetch of the next tile's indices)
                if (kGather && switch_needs_drain(in_prologue, ktiles, kStages)) wait_copies_then_barrier<0>();
                copy_tile += stride;
                copy_kt = 0;
                ++copy_ordinal;
                point_at_tile(next_info);
                if (copy_tile + stride < total_tiles) next_info = decode(copy_tile + stride);
                aim_index_prefetch(next_info);
            } else {
                copy_kt = ktiles - 4;  // past the last tile: keep asking for its last span (never used)
            }
        }
    };

    if (kGather) {
        aim_index_prefetch(next_info);
        copy4_to_lds(p.row_to_route, index_offset(), lds_index + wave * 256);
        wait_copies_then_barrier<0>();
    }
    point_at_tile(next_info);
    if (first + stride < total_tiles) next_info = decode(first + stride);
    aim_index_prefetch(next_info);

    // ---- fragment addresses inside a stage ---------------------------------------------------------
    int a_addr[2][2];  // [k step][lo/hi 16 bytes] of row tile 0; row tile i lies i * 4096 bytes further (same swizzle)
    {
        const int sw = (lr >> 1) & 7;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            a_addr[kb][0] = lr * kBK + (((kb * 4 + g) ^ sw) << 4);
            a_addr[kb][1] = lr * kBK + (((kb * 4 + 2 + g) ^ sw) << 4);
        }
    }
    // LDS address of this lane's row-scale entry in the slot of the span being read; row tile i lies i * 512 bytes further,
    // k tile q of the span 4 q bytes (one register and instruction offsets, not a register per row tile)
    int row_scale_at = Cfg::kOffRowScales + lr * 16;

    v8i afrag[2][kRowTiles];   // [k step][row tile]
    int ascale[2][kRowTiles];  // [item parity][row tile]: the row-scale word of the k tile, moved so that this lane half's
                               // first k block is byte 0 (its second is byte 2)
    auto read_fragment = [&](int stage, int kb, int i) {
        const uint8_t* at = lds + stage * kStageBytes + i * 4096;
        const u32x4 lo = *reinterpret_cast<const u32x4*>(at + a_addr[kb][0]);
        const u32x4 hi = *reinterpret_cast<const u32x4*>(at + a_addr[kb][1]);
        afrag[kb][i] = v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
    };
    int col_scale_slot = 0;  // byte offset of the LDS slot whose span's column scales are read next
    auto read_row_scale = [&](int parity, int pos, int i) {
        ascale[parity][i] = static_cast<int>(*reinterpret_cast<const uint32_t*>(lds + row_scale_at + (i * 512 + pos * 4)));
    };
    auto read_col_scales = [&]() {
        const int sb_addr = Cfg::kOffColScales + wave * 1024 + lane_now() * 8;  // this wave's column tile c: + c * 512
#pragma unroll
        for (int c = 0; c < kCols; ++c) bscale_next[c] = *reinterpret_cast<const u32x2*>(lds + sb_addr + c * 512 + col_scale_slot);
    };

    v16f acc[kRowTiles][kCols];
    auto clear_acc = [&]() {
#pragma unroll
        for (int i = 0; i < kRowTiles; ++i)
#pragma unroll
            for (int c = 0; c < kCols; ++c)
#pragma unroll
                for (int j = 0; j < 16; ++j) acc[i][c][j] = 0.0f;
    };

    // ---- epilogue of one tile: straight from the accumulators (see mfma_fp4_fp8_regs) ----------------------------------
    // A lane holds, for its row, columns q*8 + g*4 .. + 3 (q = 0..3) of a column tile, its partner lane (l ^ 32) the four
    // columns in between.  Two register swaps between the lane halves give the lower lane columns 0..15 and the upper lane
    // columns 16..31 of the row as consecutive bytes, which leave as 16-byte stores.
    auto swap_halves = [](uint32_t lower_q, uint32_t upper_q, uint32_t (&out)[2]) {
        // lanes 0..31 get (their own lower_q, the partner's lower_q), lanes 32..63 (the partner's upper_q, their own upper_q)
        const auto swapped = __builtin_amdgcn_permlane32_swap(lower_q, upper_q, false, false);
        out[0] = swapped[0];
        out[1] = swapped[1];
    };
    auto epilogue = [&](const TileInfo& info) {
        const int lane = lane_now(), g = lane >> 5, lr = lane & 31;  // (the epilogue's own copies: see lane_now)
#pragma unroll
        for (int i = 0; i < kRowTiles; ++i) {
            if (i == kRowTiles - 1 && fillers != 0 && wave == 0 && lane == 0)
                __hip_atomic_fetch_add(p.fill_stop, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const bool row_exists = lr < info.valid - 32 * i;
            const size_t row = static_cast<size_t>(info.row0) + 32 * i + lr;
            // (a row tile's accumulators leave their registers here, not earlier: read all at once at the head of the
            // epilogue, the twelve tiles would need 192 more registers than the loop's own state leaves free)
#pragma unroll
            for (int c = 0; c < kCols; ++c) asm volatile("" : "+a"(acc[i][c]));
            if (kGateUp) {
                // column tile 0 = gate, 1 = up of the same 32 activation columns
                float v[16];
                float amax = 0.0f;
#pragma unroll
                for (int j = 0; j < 16; j += 2) {
                    const uint32_t gate = pack_bf16x2(acc[i][0][j], acc[i][0][j + 1]), up = pack_bf16x2(acc[i][1][j], acc[i][1][j + 1]);
                    const uint32_t act = pack_bf16x2(silu_mul(__uint_as_float(gate << 16), __uint_as_float(up << 16)),
                                                     silu_mul(__uint_as_float(gate & 0xffff0000u), __uint_as_float(up & 0xffff0000u)));
                    v[j] = bf16_to_f32(act & 0xffffu);
                    v[j + 1] = bf16_to_f32(act >> 16);
                    amax = fmaxf(amax, fmaxf(fabsf(v[j]), fabsf(v[j + 1])));
                }
                amax = fmaxf(amax, __shfl_xor(amax, 32));  // the row's other sixteen columns
                const int byte = mx_scale_byte(amax);
                uint32_t code[4];
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    code[q] = pack4_e4m3(mx_scaled(v[4 * q], byte), mx_scaled(v[4 * q + 1], byte), mx_scaled(v[4 * q + 2], byte),
                                         mx_scaled(v[4 * q + 3], byte));
                uint32_t first[2], second[2];
                swap_halves(code[0], code[2], first);
                swap_halves(code[1], code[3], second);
                const u32x4 codes = {first[0], first[1], second[0], second[1]};
                const int act_width = p.n / 2;
                const int act_col = (info.nt * (kBN / 64) + wave) * 32;
                if (row_exists) {
                    *reinterpret_cast<u32x4*>(p.act_codes + row * act_width + act_col + g * 16) = codes;
                    if (g == 0) p.act_scales[row * (act_width / 32) + (act_col >> 5)] = static_cast<uint8_t>(byte);
                }
            } else {
#pragma unroll
                for (int c = 0; c < kCols; ++c) {
                    uint32_t pairs[4][2];  // [q][columns +0,1 | +2,3]
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        pairs[q][0] = pack_bf16x2(acc[i][c][4 * q], acc[i][c][4 * q + 1]);
                        pairs[q][1] = pack_bf16x2(acc[i][c][4 * q + 2], acc[i][c][4 * q + 3]);
                    }
                    uint32_t s00[2], s01[2], s10[2], s11[2];
                    swap_halves(pairs[0][0], pairs[2][0], s00);
                    swap_halves(pairs[0][1], pairs[2][1], s01);
                    swap_halves(pairs[1][0], pairs[3][0], s10);
                    swap_halves(pairs[1][1], pairs[3][1], s11);
                    const u32x4 lower = {s00[0], s01[0], s00[1], s01[1]}, upper = {s10[0], s11[0], s10[1], s11[1]};
                    const int col = info.nt * kBN + (wave * kCols + c) * 32 + g * 16;
                    if (row_exists) {
                        // cached stores: the weighted reduce that follows reads these rows back at once
                        if (col < p.out_cols) *reinterpret_cast<u32x4*>(p.out + row * p.out_cols + col) = lower;
                        if (col + 8 < p.out_cols) *reinterpret_cast<u32x4*>(p.out + row * p.out_cols + col + 8) = upper;
                    }
                }
            }
        }
    };

    // ---- prologue: everything of items 0..3, then item 0's first fragments -------------------------------
    auto request_item = [&](auto pos) {
        if (decltype(pos)::value == 0) request_span();
        static_for<kRowTiles>([&](auto piece) { request_activations(pos, piece); });
        request_weights(pos, std::integral_constant<int, 0>{});
        request_weights(pos, std::integral_constant<int, 1>{});
        advance_cursor(true, decltype(pos)::value == 3);
    };
    request_item(std::integral_constant<int, 0>{});
    request_item(std::integral_constant<int, 1>{});
    request_item(std::integral_constant<int, 2>{});
    request_item(std::integral_constant<int, 3>{});
    wait_copies_then_barrier<Cfg::kPrologueWait>();  // item 0 and its span have arrived
    int read_span = 0;
    read_col_scales();
#pragma unroll
    for (int i = 0; i < kRowTiles; ++i) {
        read_row_scale(0, 0, i);
        read_fragment(0, 0, i);
    }
    clear_acc();
    asm volatile("s_nop 3");
    int tile = first, kt = 0;
    TileInfo info = decode(first);
    const long long total_items = static_cast<long long>(my_tiles) * ktiles;
    constexpr int kMfmas = kRowTiles * kCols;  // per k step; MFMA n works on row tile n % kRowTiles, column tile n / kRowTiles

    // One item at ring position kPos.  First k step: its MFMAs, with the LDS reads of the second k step's fragments dealt
    // out between them; then the wait + barrier, after which the item's own stage may be refilled.  Second k step: its
    // MFMAs, with the activation copies of the item four ahead, and the reads of the next item's row scales and first
    // fragments, dealt out between them.  Behind the last MFMA of a k step its weight registers are free: the weight loads
    // of the item four ahead follow.
    auto item_body = [&](auto pos) {
        constexpr int kPos = decltype(pos)::value;
        constexpr int kParity = kPos & 1, kNextPos = (kPos + 1) & 3;
        if (kPos == 0) {
            // the span's column scales were read from LDS under the previous item's last MFMAs
#pragma unroll
            for (int c = 0; c < kCols; ++c) bscale_now[c] = bscale_next[c];
        }
        const int scale_b0 = static_cast<int>(bscale_now[0][kPos >> 1]), scale_b1 = static_cast<int>(bscale_now[1][kPos >> 1]);
        int shifted[kRowTiles];
#pragma unroll
        for (int i = 0; i < kRowTiles; ++i) shifted[i] = ascale[kParity][i] >> (8 * g);
        // MFMA number n of a k step works on row tile n / kCols, column tile n % kCols.
        auto mfma = [&](auto step, auto number) {
            constexpr int kStep = decltype(step)::value, kN = decltype(number)::value;
            constexpr int kI = kN / kCols, kC = kN % kCols;
            mfma_fp4_fp8_regs<Cfg::kWeightRegs + 16 * kPos + 8 * kStep + 4 * kC, 2 * (kPos & 1) + kStep, 2 * kStep>(
                acc[kI][kC], afrag[kStep][kI], kC == 0 ? scale_b0 : scale_b1, shifted[kI]);
        };
        // First k step.  Behind MFMA kBarrierAt comes the wait + barrier: the second step's fragments were all asked for under
        // the first kRowTiles MFMAs and have had kBarrierAt - kRowTiles more to arrive.  The activation copies of the item four
        // ahead (into this item's own stage, free from the barrier on) are dealt out one per kCopyEvery MFMAs over what
        // is left of the item.
        constexpr int kBarrierAt = kRowTiles + 1;
        constexpr int kSlotsLeft = 2 * kMfmas - kBarrierAt - 1, kCopyEvery = kSlotsLeft / kRowTiles;
        // (the copies' offsets are read from LDS in one go right behind the barrier: read one by one in front of each copy,
        // every copy waited for its own read behind whatever fragment reads were queued before it)
        uint32_t copy_from[kRowTiles];
        auto copies_behind = [&](auto slot) {  // slot = MFMAs issued since the barrier, 1-based
            constexpr int kSlot = decltype(slot)::value;
            if constexpr (kSlot >= 1 && (kSlot - 1) % kCopyEvery == 0 && (kSlot - 1) / kCopyEvery < kRowTiles)
                request_activations_at(pos, std::integral_constant<int, (kSlot - 1) / kCopyEvery>{}, copy_from[(kSlot - 1) / kCopyEvery]);
        };
        static_for<kMfmas>([&](auto n) {
            constexpr int kN = decltype(n)::value;
            mfma(std::integral_constant<int, 0>{}, n);
            if constexpr (kN < kRowTiles) read_fragment(kPos, 1, kN);
            if constexpr (kN == kBarrierAt) {
                // The next item's operands have arrived once each thread has at most the requests of the two items after it
                // in flight; past the barrier every wave has also read the last fragment of this item's stage.
                wait_copies_then_barrier<Cfg::kWait>();
#pragma unroll
                for (int i = 0; i < kRowTiles; ++i) copy_from[i] = my_offsets[i * kGemmThreads];
                if (kPos == 0) request_span();
            }
            if constexpr (kN > kBarrierAt) copies_behind(std::integral_constant<int, kN - kBarrierAt>{});
        });
        request_weights(pos, std::integral_constant<int, 0>{});
        if (kPos == 3) {
            // the next item opens a span: its scales sit in the other LDS slots
            ++read_span;
            row_scale_at += (read_span & 1) ? Cfg::kRowScaleSlot : -Cfg::kRowScaleSlot;
            asm volatile("" : "+v"(row_scale_at));  // (kept as one value: see its declaration)
            col_scale_slot = (read_span & 1) * Cfg::kColScaleSlot;
            read_col_scales();
        }
        static_for<kMfmas>([&](auto n) {
            constexpr int kN = decltype(n)::value;
            mfma(std::integral_constant<int, 1>{}, n);
            copies_behind(std::integral_constant<int, kMfmas - 1 - kBarrierAt + kN + 1>{});
            // the next item's row scale and first fragment of the row tile just finished
            if constexpr (kN % kCols == kCols - 1) {
                read_row_scale(kParity ^ 1, kNextPos, kN / kCols);
                read_fragment(kNextPos, 0, kN / kCols);
            }
        });
        request_weights(pos, std::integral_constant<int, 1>{});
        advance_cursor(false, kPos == 3);
    };

    for (long long item = 0; item < total_items; item += 4) {
        item_body(std::integral_constant<int, 0>{});
        item_body(std::integral_constant<int, 1>{});
        item_body(std::integral_constant<int, 2>{});
        item_body(std::integral_constant<int, 3>{});
        kt += 4;
        if (__builtin_expect(kt == ktiles, 0)) {
            settle_accumulators();
#pragma unroll
            for (int i = 0; i < kRowTiles; ++i)
#pragma unroll
                for (int c = 0; c < kCols; ++c) asm volatile("" : "+a"(acc[i][c]));
            epilogue(info);
            clear_acc();
            asm volatile("s_nop 3");
            kt = 0;
            tile += stride;
            if (tile < total_tiles) info = decode(tile);
        }
    }
    // Nothing may still be in flight into this workgroup's LDS or registers when it retires.
    wait_copies_then_barrier<0>();
}

// Shared experts take every token: their rows follow the routed ones, expert-major, token order.
// offsets[num_routed + 1 + s] = R + (s + 1) * B and row_to_route[R + s * B + t] = t * topk (so that the gather's
// route / topk is t), with R read from the device.
__global__ __launch_bounds__(256) void shared_rows_kernel(const int* __restrict__ num_rows, int num_tokens, int num_topk,
                                                          int num_routed, int num_shared, int* __restrict__ offsets,
                                                          int* __restrict__ row_to_route)
{
    const int first = num_rows[0];
    const long long id = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id < num_shared) offsets[num_routed + 1 + id] = first + static_cast<int>(id + 1) * num_tokens;
    if (id < static_cast<long long>(num_shared) * num_tokens)
        row_to_route[first + id] = static_cast<int>(id % num_tokens) * num_topk;
}

// What the GEMM works on for a logical dimension (hidden or intermediate): whole 256-column tiles and whole spans of
// scales, at least 512 (a row's scale bytes fill one 16-byte copy).  Weights are padded when they are prepared,
// activations by a copy of their own before the first GEMM; padding multiplies zero codes.
int padded_dim(int dim) { return dim <= 512 ? 512 : (dim + 255) / 256 * 256; }

int check_gemm(const char* what, int n, int k, int num_local)
{
    DPEP_REQUIRE(num_local >= 1 && num_local <= kMaxMoeExperts, "%s: number of local experts %d outside [1, %d]", what,
                 num_local, kMaxMoeExperts);
    DPEP_REQUIRE(k >= 512 && k % 256 == 0, "%s: K=%d must be a multiple of 256, at least 512", what, k);
    DPEP_REQUIRE(n > 0 && n % kBN == 0, "%s: N=%d must be a positive multiple of %d", what, n, kBN);
    return DPEP_OK;
}

int gemm_grid()
{
    int device = 0, cus = 256;
    if (hipGetDevice(&device) == hipSuccess) {
        int value = 0;
        if (hipDeviceGetAttribute(&value, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && value > 0) cus = value;
    }
    return cus / 8 * 8;  // one resident workgroup per CU (the LDS ring takes most of the 160 KiB)
}

// Raising the dynamic LDS limit is a setting per function and per device (each device holds its own copy of the code
// object).  One flag per device; two threads that both find it clear both make the (idempotent) call.
template <typename Kernel>
int allow_lds(Kernel kernel, int bytes, std::atomic<bool>* configured, int max_devices)
{
    int device = 0;
    DPEP_HIP(hipGetDevice(&device));
    const bool tracked = device >= 0 && device < max_devices;
    if (!tracked || !configured[device].load(std::memory_order_acquire)) {
        DPEP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
        if (tracked) configured[device].store(true, std::memory_order_release);
    }
    return DPEP_OK;
}

template <int RT, bool kGateUp>
int launch_gemm_rt(const GemmParams& p, double expected_tiles, hipStream_t stream, const char* what)
{
    constexpr int kMaxDevices = 64;
    if (p.column_waves && p.k % 512 == 0) {
        constexpr int kLds = ColCfg<RT>::kLdsBytes;
        static std::atomic<bool> configured[kMaxDevices];
        if (int rc = allow_lds(&grouped_gemm_colwave_kernel<RT, kGateUp>, kLds, configured, kMaxDevices)) return rc;
        // Two workgroups on a CU each run at about half speed: worth it where that does not add rounds (512 tiles on
        // 256 CUs: one round of 512 instead of two of 256, with twice the requests in flight; 700 tiles: two slow rounds
        // would replace three fast ones).
        const int cus = gemm_grid();
        int per_cu = 1;
        if (ColCfg<RT>::kWorkgroupsPerCu == 2 && 2.0 * ceil(expected_tiles / (2.0 * cus)) <= ceil(expected_tiles / cus)) per_cu = 2;
        hipLaunchKernelGGL((grouped_gemm_colwave_kernel<RT, kGateUp>), dim3(cus * per_cu), dim3(kGemmThreads), kLds, stream, p);
        return launch_status(what);
    }
    constexpr int kLds = GemmCfg<RT, kGateUp>::kLdsBytes;
    static std::atomic<bool> configured[kMaxDevices];
    if (int rc = allow_lds(&grouped_gemm_kernel<RT, kGateUp>, kLds, configured, kMaxDevices)) return rc;
    hipLaunchKernelGGL((grouped_gemm_kernel<RT, kGateUp>), dim3(gemm_grid()), dim3(kGemmThreads), kLds, stream, p);
    return launch_status(what);
}

// Row-tile height: the cheapest of 64 / 128 / 192 rows by a small cost model, judged from the expected rows per expert (the true counts
// stay on the device).  Routing scatters the counts around that mean (about +-sqrt(mean)), and one expert a few
// rows over a multiple of the tile height costs a whole extra row tile each: the tile count is therefore the
// expectation of ceil(rows / height) under a normal spread, not ceil(mean / height).  (Mean 256 over 8 experts:
// 128-row tiles need 2.5 row tiles per expert on average = 320 tiles = two rounds on 256 CUs, 192-row tiles need
// 2 = one round; measured 103 vs 80 us.)
template <bool kGateUp>
int launch_gemm(const GemmParams& p, int expected_rows_per_expert, hipStream_t stream, const char* what)
{
    const int cus = gemm_grid();
    const int n_tiles = p.n / kBN;
    const double mean = expected_rows_per_expert > 1 ? expected_rows_per_expert : 1;
    const double sigma = sqrt(mean);
    int best = 2;
    double best_cost = 1e30, tiles_of[4] = {0.0, 0.0, 0.0, 0.0};
    for (int rt = 1; rt <= 3; ++rt) {
        const int bm = 64 * rt;
        double m_tiles = 1.0;  // E[ceil(X / bm)] = sum over j >= 0 of P(X > j * bm)
        for (int j = 1; j * bm < mean + 6.0 * sigma; ++j) m_tiles += 0.5 * erfc((j * bm - mean) / (sigma * 1.4142135623730951));
        const double tiles = p.num_local * m_tiles * n_tiles;
        tiles_of[rt] = tiles;
        const double rounds = ceil(tiles / cus - 0.02);  // a stray tile in one launch out of fifty does not count
        // Microseconds, fitted to kernel traces on an MI355X over shares from 32 to 2048 rows per expert, 4 to 32
        // experts and two problem sizes (it reproduced the measured order of the three heights in 14 of 16 small cases,
        // was within 7 % in the other two, and in the many-round cases of a large batch): once per launch the part of the
        // first tile that nothing overlaps (the 192-row kernel's three-stage ring starts slowly), per tile its epilogue
        // and switch, per k tile the main loop; an expert with a single row tile streams its weight tile from HBM with
        // nobody to share it with, which adds about 0.3 us per k tile whatever the height.
        // (These figures are the column-wave kernel's; how to refit them: force each height with the workspace setting
        // "gemm_tile_rows" on a many-round launch, take a kernel trace, and solve time = rounds * (per tile + k tiles * per
        // item) over two k lengths: the two GEMMs of one forward give them.)
        constexpr double kFirst[3] = {0.0, 0.0, 4.7}, kPerTile[3] = {4.0, 3.0, 3.4}, kPerItem[3] = {0.50, 0.83, 1.15};
        const double per_item = kPerItem[rt - 1] + (m_tiles <= 1.2 ? 0.3 : 0.0);
        const double cost = kFirst[rt - 1] + (rounds < 1.0 ? 1.0 : rounds) * (kPerTile[rt - 1] + (p.k / kBK) * per_item);
        if (cost < best_cost - 1e-9) {
            best_cost = cost;
            best = rt;
        }
    }
    if (p.forced_rt >= 1 && p.forced_rt <= 3) best = p.forced_rt;
    if (best == 1) return launch_gemm_rt<1, kGateUp>(p, tiles_of[1], stream, what);
    if (best == 2) return launch_gemm_rt<2, kGateUp>(p, tiles_of[2], stream, what);
    return launch_gemm_rt<3, kGateUp>(p, tiles_of[3], stream, what);
}

}  // namespace

// ---- host replay of one workgroup's schedule ---------------------------------------------------------------
// Vector-memory operations complete in issue order, and a wait for "at most N in flight" guarantees no more than
// that all but the newest N have completed.  The replay issues what the kernel issues, in the kernel's order (the
// prologue's kAhead items; per item: the counted wait, the copies of the item kAhead ahead with their scale and index
// copies, the cursor's tile switch; epilogue stores at tile ends), lets nothing complete that a wait has not
// forced, and checks that every item's copies have completed when its fragments are read and that the gather
// indices of a tile have when the cursor reads them.
struct ScheduleFault {
    int item, what;  // what: 1 = an item's copies, 2 = gather indices
};

// The rings of scale slots: a span's scales (the scales of item x are read during the body of item x - 1) must all have
// been read when the copies of a later span go into the same slot; the copies are issued behind the barrier of the body
// that is running (-1: the prologue, before anything is read).
struct ScaleSlots {
    long long last_item[4] = {-1, -1, -1, -1};  // of the span each slot holds
    int slots, next = 0;
    explicit ScaleSlots(int n) : slots(n) {}
    bool take(long long span_last_item, long long body)  // false: the slot's present span is still being read
    {
        const long long held = last_item[next];
        last_item[next] = span_last_item;
        next = next + 1 == slots ? 0 : next + 1;
        return held < 0 || held <= body;
    }
};

template <int RT>
bool replay_workgroup(int my_tiles, int ktiles, int epilogue_stores, bool drain_at_switches, int scale_slots, ScheduleFault* fault)
{
    using Ring = GemmRing<RT>;
    constexpr int kAhead = Ring::kAhead, kCopies = Ring::kCopies;
    ScaleSlots scales(scale_slots);
    long long body = -1;
    const long long n_items = static_cast<long long>(my_tiles) * ktiles;
    if (n_items == 0) return true;
    long long issued = 0, done = 0;  // operations [0, done) have certainly completed
    auto wait = [&](long long in_flight) {
        if (issued - in_flight > done) done = issued - in_flight;
    };
    int copy_kt = 0, copy_tile = 0;
    long long copy_item = 0;   // ordinal of the item under the cursor
    long long index_op = -1;   // operation that fetches the indices of the cursor's next tile
    static thread_local long long item_last_op[1 << 16];
    if (n_items >= (1 << 16)) return true;  // not replayed (far beyond any real workgroup's share)
    bool ok = true, past_end = false;
    auto issue_copies = [&]() {
        issued += kCopies;
        if ((copy_kt & 3) == 0) {
            issued += 2;  // row and column scales of the span
            if (!scales.take(copy_item + (ktiles - 1 - copy_kt < 3 ? ktiles - 1 - copy_kt : 3), body) && ok) {
                ok = false;
                *fault = {static_cast<int>(body), 3};
            }
        }
        if (copy_kt == 0) index_op = issued++;    // (re-copies past the end sit on the last k tile, never 0)
        if (!past_end) item_last_op[copy_item] = issued - 1;
    };
    auto advance = [&](bool in_prologue, int item) {
        if (++copy_kt == ktiles) {
            if (copy_tile + 1 < my_tiles) {
                if (drain_at_switches && switch_needs_drain(in_prologue, ktiles, kAhead)) wait(0);
                if (index_op >= done && ok) {
                    ok = false;
                    *fault = {item, 2};
                }
                ++copy_tile;
                copy_kt = 0;
                ++copy_item;
            } else {
                copy_kt = ktiles - 1;  // past the last tile: keep re-copying its last item (never read)
                past_end = true;
            }
        } else if (!past_end) {
            ++copy_item;
        }
    };
    auto check_item = [&](long long item) {
        if (item < n_items && item_last_op[item] >= done && ok) {
            ok = false;
            *fault = {static_cast<int>(item), 1};
        }
    };
    ++issued;  // the first tile's own indices, fetched synchronously
    wait(0);
    for (int j = 0; j < kAhead; ++j) {
        issue_copies();
        advance(true, -1);
    }
    wait((kAhead - 1) * kCopies);
    check_item(0);
    int kt = 0;
    for (long long item = 0; item < n_items; ++item) {
        wait(Ring::kWaitPlain);
        check_item(item + 1);  // its first fragments leave LDS during this item's second k step
        body = item;
        issue_copies();
        advance(false, static_cast<int>(item));
        if (++kt == ktiles) {
            issued += epilogue_stores;
            kt = 0;
        }
    }
    return ok;
}

// The same replay for the column-wave kernel: the prologue requests items 0..3 (each: its span's scales and the next tile's
// gather indices where it opens a span / a tile, its activation copies, its weight loads), then waits; every item's body
// waits (kWait + slack in flight), then requests the item four ahead in the same order; tiles end behind every ktiles-th
// item with the epilogue's stores.  slack > 0 replays a kernel whose wait is laxer than the real one.
template <int RT>
bool replay_column_waves(int my_tiles, int ktiles, int epilogue_stores, int slack, ScheduleFault* fault)
{
    using Ring = ColumnRing<RT>;
    const long long n_items = static_cast<long long>(my_tiles) * ktiles;
    if (n_items == 0) return true;
    static thread_local long long item_last_op[1 << 16];
    if (n_items >= (1 << 16)) return true;  // not replayed (far beyond any real workgroup's share)
    long long issued = 0, done = 0;
    auto wait = [&](long long in_flight) {
        if (issued - in_flight > done) done = issued - in_flight;
    };
    int copy_kt = 0, copy_tile = 0;
    long long copy_item = 0, index_op = -1;
    bool ok = true, past_end = false;
    ScaleSlots scales(2);
    long long body = -1;
    auto request_item = [&]() {
        if ((copy_kt & 3) == 0) {
            issued += 2;                            // row and column scales of the span
            if (!past_end && !scales.take(copy_item + 3, body) && ok) {
                ok = false;
                *fault = {static_cast<int>(body), 3};
            }
            if (copy_kt == 0) index_op = issued++;  // gather indices of the tile after the cursor's
        }
        issued += Ring::kRequests;
        if (!past_end) item_last_op[copy_item] = issued - 1;
    };
    auto advance = [&](bool in_prologue, int item) {
        ++copy_kt;
        if (!past_end) ++copy_item;
        if (copy_kt == ktiles) {
            if (copy_tile + 1 < my_tiles) {
                if (switch_needs_drain(in_prologue, ktiles, Ring::kStages)) wait(0);
                if (index_op >= done && ok) {
                    ok = false;
                    *fault = {item, 2};
                }
                ++copy_tile;
                copy_kt = 0;
            } else {
                copy_kt = ktiles - 4;  // past the last tile: its last span again (never used)
                if (!past_end) --copy_item;
                past_end = true;
            }
        }
    };
    auto check_item = [&](long long item) {
        if (item < n_items && item_last_op[item] >= done && ok) {
            ok = false;
            *fault = {static_cast<int>(item), 1};
        }
    };
    ++issued;  // the first tile's own indices, fetched synchronously
    wait(0);
    for (int j = 0; j < Ring::kStages; ++j) {
        request_item();
        advance(true, -1);
    }
    wait(Ring::kPrologueWait);
    check_item(0);
    int kt = 0;
    for (long long item = 0; item < n_items; ++item) {
        wait(Ring::kWait + slack);
        check_item(item + 1);  // its first fragments leave LDS during this item's second k step, its weights right after
        body = item;
        request_item();
        advance(false, static_cast<int>(item));
        if (++kt == ktiles) {
            issued += epilogue_stores;
            kt = 0;
        }
    }
    return ok;
}

int launch_gemm1(const GemmParams& p, int expected_rows_per_expert, hipStream_t stream)
{
    if (int rc = check_gemm("gemm1", p.n, p.k, p.num_local)) return rc;
    DPEP_REQUIRE(p.row_to_route != nullptr && p.topk >= 1, "gemm1: needs the row -> route map");
    return launch_gemm<true>(p, expected_rows_per_expert, stream, "grouped_gemm1");
}

int launch_gemm2(const GemmParams& p, int expected_rows_per_expert, hipStream_t stream)
{
    if (int rc = check_gemm("gemm2", p.n, p.k, p.num_local)) return rc;
    return launch_gemm<false>(p, expected_rows_per_expert, stream, "grouped_gemm2");
}

}  // namespace dpep

extern "C" {

int dpep_mx_quant(const void* x, int rows, int hidden, void* codes, uint8_t* scales, void* stream)
{
    using namespace dpep;
    DPEP_REQUIRE(rows >= 0, "mx_quant: bad row count %d", rows);
    DPEP_REQUIRE(hidden > 0 && hidden % 32 == 0, "mx_quant: hidden=%d must be a positive multiple of 32", hidden);
    if (rows == 0) return DPEP_OK;
    DPEP_REQUIRE(x && codes && scales && aligned16(x) && aligned16(codes), "mx_quant: NULL or misaligned buffer");
    const long long units = static_cast<long long>(rows) * (hidden / 16);
    DPEP_REQUIRE((units + kMxThreads - 1) / kMxThreads < (1ll << 31), "mx_quant: %d x %d values are more than one launch takes",
                 rows, hidden);
    const unsigned blocks = static_cast<unsigned>((units + kMxThreads - 1) / kMxThreads);
    if (aligned16(scales))
        hipLaunchKernelGGL(mx_quant_kernel<true>, dim3(blocks), dim3(kMxThreads), 0, static_cast<hipStream_t>(stream),
                           static_cast<const u32x4*>(x), units, static_cast<u32x4*>(codes), scales);
    else
        hipLaunchKernelGGL(mx_quant_kernel<false>, dim3(blocks), dim3(kMxThreads), 0, static_cast<hipStream_t>(stream),
                           static_cast<const u32x4*>(x), units, static_cast<u32x4*>(codes), scales);
    return launch_status("mx_quant");
}

int dpep_megamoe_schedule_check(int tile_rows, int tiles_per_workgroup, int ktiles, int epilogue_stores, int without_drain)
{
    using namespace dpep;
    DPEP_REQUIRE(tile_rows == 64 || tile_rows == 128 || tile_rows == 192, "schedule_check: tile_rows is 64, 128 or 192");
    DPEP_REQUIRE(tiles_per_workgroup >= 0 && ktiles >= 2 && ktiles % 2 == 0 && epilogue_stores >= 0,
                 "schedule_check: bad arguments");
    ScheduleFault fault = {0, 0};
    const bool drain = (without_drain & 1) == 0;
    const int slots = (without_drain & 2) != 0 ? 2 : GemmCfg<1, false>::kScaleSlots;  // (bit 1: the rings as they were, two slots)
    const bool ok = tile_rows == 64    ? replay_workgroup<1>(tiles_per_workgroup, ktiles, epilogue_stores, drain, slots, &fault)
                    : tile_rows == 128 ? replay_workgroup<2>(tiles_per_workgroup, ktiles, epilogue_stores, drain, slots, &fault)
                                       : replay_workgroup<3>(tiles_per_workgroup, ktiles, epilogue_stores, drain, slots, &fault);
    if (!ok && fault.what == 3)
        return fail(DPEP_EINVAL, "schedule_check: a span's scales are overwritten while they are still being read (behind item %d)",
                    fault.item);
    if (!ok)
        return fail(DPEP_EINVAL, "schedule_check: %s read before any wait covers them (item %d)",
                    fault.what == 1 ? "an item's copies are" : "the next tile's gather indices are", fault.item);
    return DPEP_OK;
}

int dpep_megamoe_schedule_check_column_waves(int tile_rows, int tiles_per_workgroup, int ktiles, int epilogue_stores, int slack)
{
    using namespace dpep;
    DPEP_REQUIRE(tile_rows == 64 || tile_rows == 128 || tile_rows == 192, "schedule_check: tile_rows is 64, 128 or 192");
    DPEP_REQUIRE(tiles_per_workgroup >= 0 && ktiles >= 4 && ktiles % 4 == 0 && epilogue_stores >= 0 && slack >= 0,
                 "schedule_check: bad arguments (the column-wave kernel takes k tiles in fours)");
    ScheduleFault fault = {0, 0};
    const bool ok = tile_rows == 64    ? replay_column_waves<1>(tiles_per_workgroup, ktiles, epilogue_stores, slack, &fault)
                    : tile_rows == 128 ? replay_column_waves<2>(tiles_per_workgroup, ktiles, epilogue_stores, slack, &fault)
                                       : replay_column_waves<3>(tiles_per_workgroup, ktiles, epilogue_stores, slack, &fault);
    if (!ok && fault.what == 3)
        return fail(DPEP_EINVAL, "schedule_check: a span's scales are overwritten while they are still being read (behind item %d)",
                    fault.item);
    if (!ok)
        return fail(DPEP_EINVAL, "schedule_check: %s read before any wait covers them (item %d)",
                    fault.what == 1 ? "an item's operands are" : "the next tile's gather indices are", fault.item);
    return DPEP_OK;
}

int dpep_megamoe_padded_dim(int dim) { return dim < 1 ? 0 : dpep::padded_dim(dim); }

int dpep_megamoe_prepared_shape(int n, int k, int gate_up, int* padded_n, int* padded_k, int* scale_cols)
{
    using namespace dpep;
    DPEP_REQUIRE(padded_n && padded_k && scale_cols, "prepared_shape: NULL output");
    DPEP_REQUIRE(k > 0 && k % 64 == 0, "prepared_shape: K=%d must be a positive multiple of 64", k);
    DPEP_REQUIRE(n > 0 && n % (gate_up ? 256 : 64) == 0, "prepared_shape: N=%d must be a positive multiple of %d", n,
                 gate_up ? 256 : 64);
    *padded_n = gate_up ? 2 * padded_dim(n / 2) : padded_dim(n);
    *padded_k = padded_dim(k);
    *scale_cols = (*padded_k / 128 + 3) / 4 * 16;  // groups of four k tiles, the last one padded
    return DPEP_OK;
}

int dpep_megamoe_prepare_weights(const uint8_t* w_packed, const uint8_t* w_scales, int num_local, int n, int k,
                                 int gate_up, uint8_t* out_packed, uint8_t* out_scales, void* stream)
{
    using namespace dpep;
    DPEP_REQUIRE(num_local >= 1, "prepare_weights: bad expert count %d", num_local);
    int np = 0, kp = 0, scale_cols = 0;
    if (int rc = dpep_megamoe_prepared_shape(n, k, gate_up, &np, &kp, &scale_cols)) return rc;
    DPEP_REQUIRE(w_packed && w_scales && out_packed && out_scales && aligned16(w_packed) && aligned16(out_packed),
                 "prepare_weights: NULL or misaligned buffer");
    DPEP_REQUIRE(w_packed != out_packed && w_scales != out_scales, "prepare_weights: cannot run in place");
    const long long chunks = static_cast<long long>(num_local) * np * (kp / 2) / 16;
    const long long pairs = static_cast<long long>(num_local) * np * scale_cols / 2;
    const long long threads = chunks > pairs ? chunks : pairs;
    const unsigned blocks = static_cast<unsigned>((threads + 255) / 256);
    hipLaunchKernelGGL(prepare_weights_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), w_packed,
                       w_scales, n, k, np, kp, gate_up, out_packed, out_scales, chunks, pairs);
    return launch_status("prepare_weights");
}

// Workspace carve-up shared by workspace_bytes and forward.
struct MegaLayout {
    size_t hist, meta, fill_state, route_to_row, row_to_route, x_codes, x_scales, act_codes, act_scales, out2, total;
};

static MegaLayout mega_layout(int num_tokens, int num_topk, int hidden, int intermediate, int num_local, int num_shared)
{
    auto up = [](size_t v) { return (v + 255) / 256 * 256; };
    const size_t routes = static_cast<size_t>(num_tokens) * num_topk;
    const size_t shared_rows = static_cast<size_t>(num_tokens) * num_shared;
    const size_t max_rows = static_cast<size_t>(num_tokens) * (num_topk < num_local ? num_topk : num_local) + shared_rows;
    MegaLayout l;
    size_t at = 0;
    l.hist = at;         at += up(dpep_layout_workspace_bytes(num_tokens, num_topk, num_local));
    l.meta = at;         at += up((3 * static_cast<size_t>(num_local) + num_shared + 2) * 4);
    l.fill_state = at;   at += up((1 + 4096) * 4);  // fillers of the first GEMM: count + progress of each (<= 1024 CUs x 4 waves)
    l.route_to_row = at; at += up(routes * 4);
    l.row_to_route = at; at += up((routes + shared_rows) * 4);
    const size_t hp = dpep::padded_dim(hidden), ip = dpep::padded_dim(intermediate);
    // padded copy of the input rows, only when hidden is not already what the GEMM works on
    l.x_codes = at;      at += hp != static_cast<size_t>(hidden) ? up(static_cast<size_t>(num_tokens) * hp) : 0;
    l.x_scales = at;     at += hp != static_cast<size_t>(hidden) ? up(static_cast<size_t>(num_tokens) * (hp / 32)) : 0;
    l.act_codes = at;    at += up(max_rows * ip);
    l.act_scales = at;   at += up(max_rows * (ip / 32));
    l.out2 = at;         at += up(max_rows * hidden * 2);
    l.total = at;
    return l;
}

size_t dpep_megamoe_workspace_bytes(int num_tokens, int num_topk, int hidden, int intermediate, int num_local,
                                    int num_shared)
{
    if (num_tokens < 1 || num_topk < 1 || hidden < 1 || intermediate < 1 || num_local < 1 || num_shared < 0) return 0;
    return mega_layout(num_tokens, num_topk, hidden, intermediate, num_local, num_shared).total;
}

int dpep_megamoe_fill_report(void* ws, int num_tokens, int num_topk, int hidden, int intermediate, int num_local,
                             int num_shared, int32_t* fillers_host, int64_t* tokens_filled_host, void* stream)
{
    using namespace dpep;
    Workspace* w = as_workspace(ws);
    DPEP_REQUIRE(w != nullptr && fillers_host != nullptr && tokens_filled_host != nullptr,
                 "megamoe_fill_report: not a live workspace, or NULL output");
    DPEP_REQUIRE(num_tokens >= 1 && num_topk >= 1 && hidden >= 1 && intermediate >= 1 && num_local >= 1 && num_shared >= 0,
                 "megamoe_fill_report: bad sizes");
    const MegaLayout l = mega_layout(num_tokens, num_topk, hidden, intermediate, num_local, num_shared);
    DPEP_REQUIRE(l.total <= w->bytes, "megamoe_fill_report: these are not the sizes of a forward on this workspace");
    static thread_local int32_t state[1 + 4096];
    DPEP_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    DPEP_HIP(hipMemcpy(state, static_cast<uint8_t*>(w->base) + l.fill_state, sizeof(state), hipMemcpyDeviceToHost));
    const int fillers = state[0] < 0 ? 0 : state[0] > 4096 ? 4096 : state[0];
    int64_t filled = 0;
    for (int f = 0; f < fillers; ++f) filled += state[1 + f];
    *fillers_host = fillers;
    *tokens_filled_host = filled;
    return DPEP_OK;
}

int dpep_megamoe_forward(void* ws, const void* x_codes, const uint8_t* x_scales, const int32_t* topk_idx,
                         const float* topk_weights, const uint8_t* w1, const uint8_t* s1, const uint8_t* w2,
                         const uint8_t* s2, const uint8_t* shared_w1, const uint8_t* shared_s1,
                         const uint8_t* shared_w2, const uint8_t* shared_s2, int num_shared, int num_tokens, int hidden,
                         int intermediate, int num_topk, int num_experts, int expert_begin, int num_local, void* y,
                         int32_t* expert_token_nums, void* stream)
{
    using namespace dpep;
    Workspace* w = as_workspace(ws);
    DPEP_REQUIRE(w != nullptr, "megamoe_forward: not a live workspace");
    DPEP_REQUIRE(num_tokens >= 1 && num_topk >= 1 && num_topk <= DPEP_MAX_TOPK, "megamoe_forward: bad B=%d K=%d",
                 num_tokens, num_topk);
    DPEP_REQUIRE(hidden >= 64 && hidden % 64 == 0 && intermediate >= 128 && intermediate % 128 == 0,
                 "megamoe_forward: hidden=%d must be a positive multiple of 64, intermediate=%d of 128", hidden,
                 intermediate);
    const int hp = padded_dim(hidden), ip = padded_dim(intermediate);
    DPEP_REQUIRE(num_local >= 1 && num_local <= kMaxMoeExperts && expert_begin >= 0 &&
                     expert_begin + num_local <= num_experts,
                 "megamoe_forward: bad expert range E=%d begin=%d L=%d (at most %d local experts)", num_experts,
                 expert_begin, num_local, kMaxMoeExperts);
    DPEP_REQUIRE(num_shared >= 0 && num_shared <= 8 && num_topk + num_shared <= DPEP_MAX_TOPK &&
                     num_local + num_shared <= kMaxMoeExperts,
                 "megamoe_forward: %d shared experts with K=%d, L=%d (at most 8, K+S <= %d, L+S <= %d)", num_shared,
                 num_topk, num_local, DPEP_MAX_TOPK, kMaxMoeExperts);
    DPEP_REQUIRE(x_codes && x_scales && topk_idx && topk_weights && w1 && s1 && w2 && s2 && y && expert_token_nums,
                 "megamoe_forward: NULL buffer");
    DPEP_REQUIRE(num_shared == 0 || (shared_w1 && shared_s1 && shared_w2 && shared_s2 && aligned16(shared_w1) &&
                                     aligned16(shared_w2) && aligned16(shared_s1) && aligned16(shared_s2)),
                 "megamoe_forward: shared experts need their four prepared weight buffers, 16-byte aligned");
    DPEP_REQUIRE(aligned16(x_codes) && aligned16(w1) && aligned16(w2) && aligned16(s1) && aligned16(s2) && aligned16(y),
                 "megamoe_forward: misaligned buffer");
    // the GEMM's copies address activation rows with 32-bit byte offsets
    const long long max_rows = static_cast<long long>(num_tokens) * ((num_topk < num_local ? num_topk : num_local) + num_shared);
    DPEP_REQUIRE(static_cast<long long>(num_tokens) * hp < (1LL << 32) && max_rows * ip < (1LL << 32),
                 "megamoe_forward: activation tensors of B=%d tokens exceed 4 GiB", num_tokens);
    const MegaLayout l = mega_layout(num_tokens, num_topk, hidden, intermediate, num_local, num_shared);
    DPEP_REQUIRE(l.total <= w->bytes, "megamoe_forward: workspace too small (%zu needed, %zu available)", l.total, w->bytes);
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint8_t* base = static_cast<uint8_t*>(w->base);
    int32_t* meta = reinterpret_cast<int32_t*>(base + l.meta);
    int32_t* psum = meta;
    int32_t* offsets = meta + num_local;                          // [L + S + 1]
    int32_t* num_rows = meta + 2 * num_local + num_shared + 1;    // rows of the routed experts
    int32_t* route_to_row = reinterpret_cast<int32_t*>(base + l.route_to_row);
    int32_t* row_to_route = reinterpret_cast<int32_t*>(base + l.row_to_route);
    if (int rc = layout_i32(ws, topk_idx, num_tokens, num_topk, num_experts, expert_begin, num_local, expert_token_nums,
                            psum, offsets, route_to_row, row_to_route, num_rows, s))
        return rc;
    if (num_shared > 0) {
        const long long shared_rows = static_cast<long long>(num_tokens) * num_shared;
        hipLaunchKernelGGL(shared_rows_kernel, dim3(static_cast<unsigned>((shared_rows + 255) / 256)), dim3(256), 0, s,
                           num_rows, num_tokens, num_topk, num_local, num_shared, offsets, row_to_route);
        if (int rc = launch_status("shared_rows")) return rc;
    }
    GemmParams g1{};
    g1.a_codes = static_cast<const uint8_t*>(x_codes);
    g1.a_scales = x_scales;
    if (hp != hidden) {
        const long long units = static_cast<long long>(num_tokens) * (hp / 16), bytes = static_cast<long long>(num_tokens) * (hp / 32);
        hipLaunchKernelGGL(pad_activations_kernel, dim3(static_cast<unsigned>((units + 255) / 256)), dim3(256), 0, s,
                           static_cast<const uint8_t*>(x_codes), x_scales, hidden, hp, base + l.x_codes, base + l.x_scales, units,
                           bytes);
        if (int rc = launch_status("pad_activations")) return rc;
        g1.a_codes = base + l.x_codes;
        g1.a_scales = base + l.x_scales;
    }
    g1.row_to_route = row_to_route;
    g1.topk = num_topk;
    g1.a_rows = num_tokens;
    g1.offsets = offsets;
    g1.num_local = num_local + num_shared;
    g1.num_routed = num_local;
    g1.w = w1;
    g1.ws = s1;
    g1.w_shared = shared_w1;
    g1.ws_shared = shared_s1;
    g1.n = 2 * ip;
    g1.k = hp;
    g1.act_codes = base + l.act_codes;
    g1.act_scales = base + l.act_scales;
    // Expected rows (the true counts stay on the device): tokens * topk / experts per routed expert, every
    // token for a shared one.
    const long long expected_routed = static_cast<long long>(num_tokens) * num_topk * num_local / num_experts;
    const long long expected_rows = expected_routed + static_cast<long long>(num_tokens) * num_shared;
    const int per_expert = static_cast<int>((expected_rows + g1.num_local - 1) / g1.num_local);
    // Without shared experts most tokens of a share have no row: workgroups of the first GEMM that get no tile
    // zero those rows of y meanwhile, and the weighted reduce skips what they got through.
    int* fill_state = reinterpret_cast<int*>(base + l.fill_state);
    int* fill_stop = reinterpret_cast<int*>(static_cast<char*>(w->sync) + kSyncFillStop);
    g1.forced_rt = w->gemm_tile_rows / 64;
    g1.column_waves = w->gemm_column_waves;
    // (served-only: rows of y whose token no local expert serves are nobody's business, neither the fillers' nor the
    // reduce's; with shared experts every token is served)
    const bool served_only = num_shared == 0 && w->megamoe_served_only;
    const bool fill = num_shared == 0 && w->gemm_zero_fill && !served_only;
    if (fill) {
        g1.fill_out = static_cast<u32x4*>(y);
        g1.fill_route_to_row = route_to_row;
        g1.fill_tokens = num_tokens;
        g1.fill_vec = hidden / 8;
        g1.fill_topk = num_topk;
        g1.fill_stop = fill_stop;
    }
    g1.fill_state = fill_state;  // written even when nothing fills (then as "no fillers")
    if (int rc = launch_gemm1(g1, per_expert, s)) return rc;
    GemmParams g2{};
    g2.a_codes = base + l.act_codes;
    g2.a_scales = base + l.act_scales;
    g2.row_to_route = nullptr;
    g2.topk = 1;
    g2.offsets = offsets;
    g2.num_local = num_local + num_shared;
    g2.num_routed = num_local;
    g2.w = w2;
    g2.ws = s2;
    g2.w_shared = shared_w2;
    g2.ws_shared = shared_s2;
    g2.n = hp;
    g2.k = ip;
    g2.out = reinterpret_cast<uint16_t*>(base + l.out2);
    g2.out_cols = hidden;
    g2.forced_rt = g1.forced_rt;
    g2.column_waves = g1.column_waves;
    if (int rc = launch_gemm2(g2, per_expert, s)) return rc;
    return combine_routes(base + l.out2, topk_weights, route_to_row, num_tokens, num_topk,
                          static_cast<int>(expected_rows),
                          hidden, y, num_shared > 0 ? num_rows : nullptr, num_shared, fill ? fill_state : nullptr,
                          served_only ? 1 : 0, s);
}

}  // extern "C"
