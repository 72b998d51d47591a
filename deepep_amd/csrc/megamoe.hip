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
#include "common.h"

#pragma clang fp contract(off)

namespace dpep {

int layout_i32(void* ws, const int32_t* idx, int num_tokens, int num_topk, int num_experts, int expert_begin,
               int num_local, int32_t* counts, int32_t* psum, int32_t* offsets, int32_t* route_to_row,
               int32_t* row_to_route, int32_t* num_rows, hipStream_t stream);
int combine_routes(const void* y, const float* route_weights, const int32_t* route_to_row, int num_tokens, int num_topk,
                   int num_rows_hint, int hidden, void* out, hipStream_t stream);

namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

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

// One lane owns 8 consecutive BF16 values; 4 adjacent lanes own one 32-element block.
__global__ __launch_bounds__(256) void mx_quant_kernel(const u32x4* __restrict__ x, long long num_units,
                                                       int units_per_row, u32x2* __restrict__ codes,
                                                       uint8_t* __restrict__ scales)
{
    const long long u = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    const bool live = u < num_units;
    u32x4 raw = {0, 0, 0, 0};
    if (live) raw = x[u];
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = bf16_to_f32(raw[i] & 0xffffu);
        v[2 * i + 1] = bf16_to_f32(raw[i] >> 16);
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
    amax = fmaxf(amax, __shfl_xor(amax, 1));
    amax = fmaxf(amax, __shfl_xor(amax, 2));
    const int byte = mx_scale_byte(amax);
    if (!live) return;
    u32x2 out;
    out[0] = pack4_e4m3(mx_scaled(v[0], byte), mx_scaled(v[1], byte), mx_scaled(v[2], byte), mx_scaled(v[3], byte));
    out[1] = pack4_e4m3(mx_scaled(v[4], byte), mx_scaled(v[5], byte), mx_scaled(v[6], byte), mx_scaled(v[7], byte));
    codes[u] = out;
    if ((u & 3) == 0) scales[u >> 2] = static_cast<uint8_t>(byte);
    (void)units_per_row;
}

// =====================================================================================================
// Weight re-layout: raw [L][N][K/2] + [L][N][K/32]  ->  per (column tile of 32, k step of 64) one
// contiguous 1 KiB block holding every lane's 16-byte B fragment; scales as 2 bytes per lane per k=128.
// =====================================================================================================
__device__ __forceinline__ int source_row(int physical_col, int n, int gate_up)
{
    if (!gate_up) return physical_col;
    // column tiles alternate gate / up for the same 32 activation columns
    const int tile = physical_col >> 5, j = physical_col & 31;
    const int act_col = (tile >> 1) * 32 + j;
    return (tile & 1) * (n >> 1) + act_col;
}

__global__ __launch_bounds__(256) void prepare_weights_kernel(const uint8_t* __restrict__ w,
                                                              const uint8_t* __restrict__ s, int n, int k, int gate_up,
                                                              uint8_t* __restrict__ w_out, uint8_t* __restrict__ s_out,
                                                              long long packed_chunks, long long scale_pairs)
{
    const long long id = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int ksteps = k / 64, ktiles = k / 128, ctiles = n / 32;
    if (id < packed_chunks) {  // one 16-byte fragment
        const int lane = id & 63;
        long long rest = id >> 6;
        const int ks = rest % ksteps;
        rest /= ksteps;
        const int c = rest % ctiles;
        const long long e = rest / ctiles;
        const int row = source_row(c * 32 + (lane & 31), n, gate_up);
        const uint8_t* src = w + (e * n + row) * (k / 2) + ks * 32 + (lane >> 5) * 16;
        reinterpret_cast<u32x4*>(w_out)[id] = *reinterpret_cast<const u32x4*>(src);
    }
    if (id < scale_pairs) {  // two scale bytes: k blocks (2*kb + g) of one k=128 tile
        const int lane = id & 63;
        long long rest = id >> 6;
        const int kt = rest % ktiles;
        rest /= ktiles;
        const int c = rest % ctiles;
        const long long e = rest / ctiles;
        const int row = source_row(c * 32 + (lane & 31), n, gate_up);
        const uint8_t* src = s + (e * n + row) * (k / 32) + kt * 4 + (lane >> 5);
        s_out[id * 2] = src[0];
        s_out[id * 2 + 1] = src[2];
    }
}

// =====================================================================================================
// Grouped GEMM
// =====================================================================================================
// Workgroup = 4 waves (2 row halves x 2 column halves), tile 128 rows x 256 columns, k tile 128.
// Everything the main loop reads arrives through asynchronous global->LDS copies into a ring of
// kStages k tiles; the only synchronisation per k tile is one vmcnt wait plus one barrier.
constexpr int kBM = 128;           // rows per workgroup tile
constexpr int kBK = 128;           // k per LDS stage (two MFMA k steps of 64)
constexpr int kCT = 4;             // 32-column MFMA tiles per wave
constexpr int kBN = 2 * kCT * 32;  // columns per workgroup tile
constexpr int kGemmThreads = 256;
constexpr int kStages = 4;         // LDS ring depth; copies run kStages-1 k tiles ahead
constexpr int kStageA = 0;                         // 128 rows x 128 B, 16-byte chunks XOR-swizzled
constexpr int kStageB = kBM * kBK;                 // 8 column tiles x 2 k steps x 1 KiB fragments
constexpr int kStageSA = kStageB + kBN * 64;       // 128 row scale words (+128 duplicates)
constexpr int kStageSB = kStageSA + 1024;          // 8 column tiles x 64 lanes x 2 B
constexpr int kStageBytes = kStageSB + 1024;
constexpr int kCopiesPerTile = 10;                 // per thread: 4 A + 4 B + 1 A-scale + 1 B-scale
constexpr int kGemmLdsBytes = kStages * kStageBytes;

struct GemmParams {
    const uint8_t* a_codes;    // [*, K] e4m3
    const uint8_t* a_scales;   // [*, K/32] e8m0
    const int* row_to_route;   // gather: source row = row_to_route[r] / topk; nullptr = identity
    int topk;
    const int* offsets;        // [L+1] exclusive row prefix per expert
    int num_local;
    const uint8_t* w;          // prepared fragments, expert stride N*K/2
    const uint8_t* ws;         // prepared scales, expert stride N*K/32
    int n, k;
    uint8_t* act_codes;        // first GEMM: [rows, N/2] e4m3
    uint8_t* act_scales;       //             [rows, N/64] e8m0
    uint16_t* out;             // second GEMM: [rows, N] bf16
};

// gate / (1 + exp(-gate)) * up with the hardware exponential and reciprocal (about 1 ulp each; the
// result is rounded to BF16 right after).  The clamp keeps exp finite, like the reference's clip(+-80).
__device__ __forceinline__ float silu_mul(float gate, float up)
{
    const float clipped = fminf(fmaxf(-gate, -80.0f), 80.0f);
    return gate * __frcp_rn(1.0f + __expf(clipped)) * up;
}

// Asynchronous copy global -> LDS: lane l's bytes land at lds_base + l * size.  lds_base is wave-uniform.
// Written as assembly so that the compiler's own wait-count bookkeeping does not serialise the ring;
// completion is awaited explicitly with wait_copies<N>().
__device__ __forceinline__ void copy16_to_lds(const void* src, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(base), "v"(src) : "memory");
}
__device__ __forceinline__ void copy4_to_lds(const void* src, uint32_t lds_base)
{
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(base), "v"(src) : "memory");
}
template <int kOutstanding>
__device__ __forceinline__ void wait_copies_then_barrier()
{
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kOutstanding) : "memory");
}

template <bool kGateUp>
__global__ __launch_bounds__(kGemmThreads, 1) void grouped_gemm_kernel(GemmParams p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    __shared__ int tile_base[DPEP_MAX_LOCAL_EXPERTS + 1];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int g = lane >> 5, lr = lane & 31;
    const int n_tiles = p.n / kBN;
    const int ksteps = p.k / 64, ktiles = p.k / kBK;
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));

    // Tiles per expert: ceil(rows/128) row tiles x n_tiles column tiles, expert-major.
    if (tid == 0) {
        int total = 0;
        for (int e = 0; e < p.num_local; ++e) {
            tile_base[e] = total;
            const int rows = p.offsets[e + 1] - p.offsets[e];
            total += (rows + kBM - 1) / kBM * n_tiles;
        }
        tile_base[p.num_local] = total;
    }
    __syncthreads();
    const int total_tiles = tile_base[p.num_local];

    // Consecutive tile ids share weights; give each XCD (workgroups are dealt round-robin over 8 XCDs)
    // a contiguous range of tiles so that its L2 sees each weight tile from one place.
    const int per_xcd = (gridDim.x + 7) / 8;
    const int first = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);

    // Per-thread constants of the copy pattern.
    const int a_swizzle = (wave * 4 + (lane >> 4)) & 7;            // ((row >> 1) & 7) of this thread's A rows
    const int a_chunk = ((lane & 7) ^ a_swizzle) * 16;              // byte offset inside the 128-byte k tile
    const uint32_t lds_wave_a = wave * 1024;                        // + copy * 4096
    const uint32_t lds_wave_s = wave * 256;

    for (int tile = first; tile < total_tiles; tile += per_xcd * 8) {
        int e = 0;
        while (tile >= tile_base[e + 1]) ++e;
        const int row_begin = p.offsets[e], rows = p.offsets[e + 1] - row_begin;
        const int m_tiles = (rows + kBM - 1) / kBM;
        const int local = tile - tile_base[e];
        const int nt = local / m_tiles, mt = local % m_tiles;
        const int m0 = mt * kBM;
        const int valid_rows = min(kBM, rows - m0);

        // A: copy i of wave w fills LDS rows i*32 + w*8 + lane/8.
        const uint8_t* a_src[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = min(i * 32 + wave * 8 + (lane >> 3), valid_rows - 1);
            int src = row_begin + m0 + r;
            if (p.row_to_route != nullptr) src = p.row_to_route[src] / p.topk;
            a_src[i] = p.a_codes + static_cast<size_t>(src) * p.k + a_chunk;
        }
        const uint8_t* sa_src;
        {
            const int r = min(tid & (kBM - 1), valid_rows - 1);
            int src = row_begin + m0 + r;
            if (p.row_to_route != nullptr) src = p.row_to_route[src] / p.topk;
            sa_src = p.a_scales + static_cast<size_t>(src) * (p.k / 32);
        }
        // B: fragment q = copy*4 + wave of the 16 (column tile, k step) fragments of one k tile.
        const uint8_t* w_block = p.w + static_cast<size_t>(e) * p.n * (p.k / 2) +
                                 static_cast<size_t>(nt) * (2 * kCT) * ksteps * 1024 + lane * 16;
        const uint8_t* b_src[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int q = j * 4 + wave;
            b_src[j] = w_block + (static_cast<size_t>(q >> 1) * ksteps + (q & 1)) * 1024;
        }
        const uint8_t* sb_src = p.ws + static_cast<size_t>(e) * p.n * (p.k / 32) +
                                (static_cast<size_t>(nt) * (2 * kCT) + (tid >> 5)) * ktiles * 128 + (tid & 31) * 4;

        auto issue_tile = [&](int kt) {
            const uint32_t stage = lds0 + (kt & (kStages - 1)) * kStageBytes;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                copy16_to_lds(a_src[i] + static_cast<size_t>(kt) * kBK, stage + kStageA + i * 4096 + lds_wave_a);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                copy16_to_lds(b_src[j] + static_cast<size_t>(kt) * 2048, stage + kStageB + (j * 4 + wave) * 1024);
            copy4_to_lds(sa_src + kt * 4, stage + kStageSA + lds_wave_s);
            copy4_to_lds(sb_src + kt * 128, stage + kStageSB + lds_wave_s);
        };

        v16f acc[2][kCT];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int c = 0; c < kCT; ++c)
#pragma unroll
                for (int j = 0; j < 16; ++j) acc[i][c][j] = 0.0f;

#pragma unroll
        for (int kt = 0; kt < kStages - 1; ++kt) issue_tile(min(kt, ktiles - 1));

        // Fragment addresses inside a stage.
        int a_addr[2][2][2];  // [row tile][k step][lo/hi 16 bytes]
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int row = wm * 64 + i * 32 + lr;
            const int sw = (row >> 1) & 7;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                a_addr[i][kb][0] = kStageA + row * kBK + (((kb * 4 + g) ^ sw) << 4);
                a_addr[i][kb][1] = kStageA + row * kBK + (((kb * 4 + 2 + g) ^ sw) << 4);
            }
        }
        const int sa_addr = kStageSA + (wm * 64 + lr) * 4;
        const int b_addr = kStageB + wn * kCT * 2048 + lane * 16;
        const int sb_addr = kStageSB + wn * kCT * 128 + lane * 2;

        // Software pipeline over k steps of 64: while the MFMAs of one k step run, the fragments of the
        // next one are already on their way out of LDS.  Per k tile there is one wait + barrier, placed
        // between the two k steps so that the reads issued right after it have a full k step to land.
        v8i afrag[2][2];     // [k step][row tile]
        u32x4 bfrag[2][kCT]; // [k step][column tile]
        int ascale[2][2];    // [current/next k tile][row tile]
        int bscale[2][kCT];
        auto read_step = [&](const uint8_t* stage, int kb) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const u32x4 lo = *reinterpret_cast<const u32x4*>(stage + a_addr[i][kb][0]);
                const u32x4 hi = *reinterpret_cast<const u32x4*>(stage + a_addr[i][kb][1]);
                afrag[kb][i] = v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
            }
#pragma unroll
            for (int c = 0; c < kCT; ++c) bfrag[kb][c] = *reinterpret_cast<const u32x4*>(stage + b_addr + (c * 2 + kb) * 1024);
        };
        auto read_scales = [&](const uint8_t* stage, int slot) {
#pragma unroll
            for (int i = 0; i < 2; ++i)
                ascale[slot][i] = static_cast<int>(*reinterpret_cast<const uint32_t*>(stage + sa_addr + i * 128));
#pragma unroll
            for (int c = 0; c < kCT; ++c)
                bscale[slot][c] = static_cast<int>(*reinterpret_cast<const uint16_t*>(stage + sb_addr + c * 128));
        };
        auto mfma_step = [&](int kb, int slot) {
            // The row-scale word holds the four k blocks of the tile; the upper lane half owns the odd ones.
            // (Shifted here, not at the read, so that the read does not have to be waited for early.)
            const int sa0 = ascale[slot][0] >> (8 * g), sa1 = ascale[slot][1] >> (8 * g);
#pragma unroll
            for (int c = 0; c < kCT; ++c) {
                const u32x4 b = bfrag[kb][c];
                const v8i bf = v8i{(int)b[0], (int)b[1], (int)b[2], (int)b[3], 0, 0, 0, 0};
#pragma unroll
                for (int i = 0; i < 2; ++i) {
#ifdef DPEP_DEBUG_NO_MFMA
                    acc[i][c][0] += __int_as_float(afrag[kb][i][0] ^ bf[0] ^ (i ? sa1 : sa0) ^ bscale[slot][c]);
#else
                    if (kb == 0)
                        acc[i][c] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(afrag[0][i], bf, acc[i][c], 0, 4, 0,
                                                                                    i ? sa1 : sa0, 0, bscale[slot][c]);
                    else
                        acc[i][c] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(afrag[1][i], bf, acc[i][c], 0, 4, 2,
                                                                                    i ? sa1 : sa0, 1, bscale[slot][c]);
#endif
                }
            }
        };

        // k tile 0 has landed once each thread has at most kStages-2 tiles of its own copies in flight.
        wait_copies_then_barrier<(kStages - 2) * kCopiesPerTile>();
        read_step(lds, 0);
        read_scales(lds, 0);
        for (int kt2 = 0; kt2 < ktiles; kt2 += 2) {
#pragma unroll
            for (int half = 0; half < 2; ++half) {  // unrolled by two so the scale slots are compile-time
                const int kt = kt2 + half;
                const uint8_t* stage = lds + (kt & (kStages - 1)) * kStageBytes;
                const uint8_t* next_stage = lds + ((kt + 1) & (kStages - 1)) * kStageBytes;
#ifndef DPEP_DEBUG_NO_READ
                read_step(stage, 1);
#endif
                __builtin_amdgcn_sched_barrier(0);
                mfma_step(0, half);
                __builtin_amdgcn_sched_barrier(0);
                // k tile kt+1 has landed everywhere, and every wave is past its reads of the stage that
                // the next copies overwrite (the one read during k tile kt-1).
#ifndef DPEP_DEBUG_NO_BARRIER
                wait_copies_then_barrier<(kStages - 3) * kCopiesPerTile>();
#endif
#ifndef DPEP_DEBUG_NO_COPY
                issue_tile(min(kt + kStages - 1, ktiles - 1));
#endif
#ifndef DPEP_DEBUG_NO_READ
                read_step(next_stage, 0);
                read_scales(next_stage, half ^ 1);
#endif
                __builtin_amdgcn_sched_barrier(0);
                mfma_step(1, half);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // Drain the tail copies and make sure every wave has left the ring before it is refilled.
        wait_copies_then_barrier<0>();

        // ---- Epilogue: through LDS (the ring is idle now) so that global stores are 16 bytes wide ----
        const int out_row0 = row_begin + m0 + wm * 64;
        const int wave_rows = min(64, valid_rows - wm * 64);  // may be <= 0 for the lower row half
        if (kGateUp) {
            // Column tiles alternate gate / up for the same 32 activation columns, so SwiGLU is lane-local.
            // The wave's 64 rows x 64 activation columns are staged as BF16 (row stride 144 B), then each
            // lane requantises one row: two blocks of 32 -> e8m0 byte + 32 e4m3 codes each.
            constexpr int kRowStride = 144;
            uint8_t* region = lds + wave * (64 * kRowStride);
#pragma unroll
            for (int pair = 0; pair < kCT / 2; ++pair) {
#pragma unroll
                for (int i = 0; i < 2; ++i) {
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        const int r = i * 32 + (j >> 2) * 8 + g * 4 + (j & 3);
                        const float gate = bf16_to_f32(f32_to_bf16(acc[i][2 * pair][j]));
                        const float up = bf16_to_f32(f32_to_bf16(acc[i][2 * pair + 1][j]));
                        *reinterpret_cast<uint16_t*>(region + r * kRowStride + (pair * 32 + lr) * 2) =
                            static_cast<uint16_t>(f32_to_bf16(silu_mul(gate, up)));
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            const int act_width = p.n / 2;
            const int act_col0 = (nt * kCT + wn * (kCT / 2)) * 32;
            if (lane < wave_rows) {
                const size_t row = static_cast<size_t>(out_row0 + lane);
#pragma unroll
                for (int blk = 0; blk < kCT / 2; ++blk) {
                    float v[32];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const u32x4 raw = *reinterpret_cast<const u32x4*>(region + lane * kRowStride + blk * 64 + q * 16);
#pragma unroll
                        for (int t = 0; t < 4; ++t) {
                            v[q * 8 + 2 * t] = bf16_to_f32(raw[t] & 0xffffu);
                            v[q * 8 + 2 * t + 1] = bf16_to_f32(raw[t] >> 16);
                        }
                    }
                    float amax = 0.0f;
#pragma unroll
                    for (int t = 0; t < 32; ++t) amax = fmaxf(amax, fabsf(v[t]));
                    const int byte = mx_scale_byte(amax);
                    u32x4 codes[2];
#pragma unroll
                    for (int t = 0; t < 8; ++t)
                        codes[t >> 2][t & 3] = pack4_e4m3(mx_scaled(v[4 * t], byte), mx_scaled(v[4 * t + 1], byte),
                                                          mx_scaled(v[4 * t + 2], byte), mx_scaled(v[4 * t + 3], byte));
                    uint8_t* dst = p.act_codes + row * act_width + act_col0 + blk * 32;
                    *reinterpret_cast<u32x4*>(dst) = codes[0];
                    *reinterpret_cast<u32x4*>(dst + 16) = codes[1];
                    p.act_scales[row * (act_width / 32) + (act_col0 >> 5) + blk] = static_cast<uint8_t>(byte);
                }
            }
        } else {
            // The wave's 64 rows x 128 columns are staged as BF16 (row stride 272 B) and leave as 16-byte
            // chunks: 16 lanes cover one 256-byte row segment.
            constexpr int kRowStride = 272;
            uint8_t* region = lds + wave * (64 * kRowStride);
#pragma unroll
            for (int c = 0; c < kCT; ++c) {
#pragma unroll
                for (int i = 0; i < 2; ++i) {
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        const int r = i * 32 + (j >> 2) * 8 + g * 4 + (j & 3);
                        *reinterpret_cast<uint16_t*>(region + r * kRowStride + (c * 32 + lr) * 2) =
                            static_cast<uint16_t>(f32_to_bf16(acc[i][c][j]));
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            const int col0 = nt * kBN + wn * kCT * 32;
#pragma unroll
            for (int it = 0; it < 16; ++it) {
                const int r = it * 4 + (lane >> 4), ch = lane & 15;
                if (r < wave_rows) {
                    const u32x4 chunk = *reinterpret_cast<const u32x4*>(region + r * kRowStride + ch * 16);
                    store16_nt(p.out + static_cast<size_t>(out_row0 + r) * p.n + col0 + ch * 8, chunk);
                }
            }
        }
        __syncthreads();  // the staging regions overlap the ring: finish reading before the next tile refills it
    }
}

int check_gemm(const char* what, int n, int k, int num_local, int block_n)
{
    DPEP_REQUIRE(num_local >= 1 && num_local <= DPEP_MAX_LOCAL_EXPERTS, "%s: bad number of local experts %d", what, num_local);
    DPEP_REQUIRE(k > 0 && k % 256 == 0, "%s: K=%d must be a positive multiple of 256", what, k);
    DPEP_REQUIRE(n > 0 && n % block_n == 0, "%s: N=%d must be a positive multiple of %d", what, n, block_n);
    return DPEP_OK;
}

int gemm_grid()
{
    int device = 0, cus = 256;
    if (hipGetDevice(&device) == hipSuccess) {
        int value = 0;
        if (hipDeviceGetAttribute(&value, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && value > 0) cus = value;
    }
    return cus;  // one resident workgroup per CU (the LDS ring takes most of the 160 KiB)
}

template <bool kGateUp>
int launch_gemm(const GemmParams& p, hipStream_t stream, const char* what)
{
    static bool configured = false;  // raising the dynamic LDS limit is a per-function, per-process setting
    if (!configured) {
        DPEP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&grouped_gemm_kernel<kGateUp>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kGemmLdsBytes));
        configured = true;
    }
    hipLaunchKernelGGL((grouped_gemm_kernel<kGateUp>), dim3(gemm_grid()), dim3(kGemmThreads), kGemmLdsBytes, stream, p);
    return launch_status(what);
}

}  // namespace

int launch_gemm1(const GemmParams& p, hipStream_t stream)
{
    if (int rc = check_gemm("gemm1", p.n, p.k, p.num_local, kBN)) return rc;
    return launch_gemm<true>(p, stream, "grouped_gemm1");
}

int launch_gemm2(const GemmParams& p, hipStream_t stream)
{
    if (int rc = check_gemm("gemm2", p.n, p.k, p.num_local, kBN)) return rc;
    return launch_gemm<false>(p, stream, "grouped_gemm2");
}

}  // namespace dpep

extern "C" {

int dpep_mx_quant(const void* x, int rows, int hidden, void* codes, uint8_t* scales, void* stream)
{
    using namespace dpep;
    DPEP_REQUIRE(rows >= 0, "mx_quant: bad row count %d", rows);
    DPEP_REQUIRE(hidden > 0 && hidden % 32 == 0, "mx_quant: hidden=%d must be a positive multiple of 32", hidden);
    if (rows == 0) return DPEP_OK;
    DPEP_REQUIRE(x && codes && scales && aligned16(x) && (reinterpret_cast<uintptr_t>(codes) & 7u) == 0,
                 "mx_quant: NULL or misaligned buffer");
    const long long units = static_cast<long long>(rows) * (hidden / 8);
    const unsigned blocks = static_cast<unsigned>((units + 255) / 256);
    hipLaunchKernelGGL(mx_quant_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const u32x4*>(x), units, hidden / 8, static_cast<u32x2*>(codes), scales);
    return launch_status("mx_quant");
}

int dpep_megamoe_prepare_weights(const uint8_t* w_packed, const uint8_t* w_scales, int num_local, int n, int k,
                                 int gate_up, uint8_t* out_packed, uint8_t* out_scales, void* stream)
{
    using namespace dpep;
    DPEP_REQUIRE(num_local >= 1, "prepare_weights: bad expert count %d", num_local);
    DPEP_REQUIRE(k > 0 && k % 128 == 0, "prepare_weights: K=%d must be a positive multiple of 128", k);
    DPEP_REQUIRE(n > 0 && n % (gate_up ? 64 : 32) == 0, "prepare_weights: N=%d must be a positive multiple of %d", n,
                 gate_up ? 64 : 32);
    DPEP_REQUIRE(w_packed && w_scales && out_packed && out_scales && aligned16(w_packed) && aligned16(out_packed),
                 "prepare_weights: NULL or misaligned buffer");
    DPEP_REQUIRE(w_packed != out_packed && w_scales != out_scales, "prepare_weights: cannot run in place");
    const long long chunks = static_cast<long long>(num_local) * n * (k / 2) / 16;
    const long long pairs = static_cast<long long>(num_local) * n * (k / 32) / 2;
    const unsigned blocks = static_cast<unsigned>((chunks + 255) / 256);
    hipLaunchKernelGGL(prepare_weights_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), w_packed,
                       w_scales, n, k, gate_up, out_packed, out_scales, chunks, pairs);
    return launch_status("prepare_weights");
}

// Workspace carve-up shared by workspace_bytes and forward.
struct MegaLayout {
    size_t hist, meta, route_to_row, row_to_route, act_codes, act_scales, out2, total;
};

static MegaLayout mega_layout(int num_tokens, int num_topk, int hidden, int intermediate, int num_local)
{
    auto up = [](size_t v) { return (v + 255) / 256 * 256; };
    const size_t routes = static_cast<size_t>(num_tokens) * num_topk;
    const size_t max_rows = static_cast<size_t>(num_tokens) * (num_topk < num_local ? num_topk : num_local);
    MegaLayout l;
    size_t at = 0;
    l.hist = at;         at += up(dpep_layout_workspace_bytes(num_tokens, num_topk, num_local));
    l.meta = at;         at += up((3 * static_cast<size_t>(num_local) + 2) * 4);
    l.route_to_row = at; at += up(routes * 4);
    l.row_to_route = at; at += up(routes * 4);
    l.act_codes = at;    at += up(max_rows * intermediate);
    l.act_scales = at;   at += up(max_rows * (intermediate / 32));
    l.out2 = at;         at += up(max_rows * hidden * 2);
    l.total = at;
    return l;
}

size_t dpep_megamoe_workspace_bytes(int num_tokens, int num_topk, int hidden, int intermediate, int num_local)
{
    if (num_tokens < 1 || num_topk < 1 || hidden < 1 || intermediate < 1 || num_local < 1) return 0;
    return mega_layout(num_tokens, num_topk, hidden, intermediate, num_local).total;
}

int dpep_megamoe_forward(void* ws, const void* x_codes, const uint8_t* x_scales, const int32_t* topk_idx,
                         const float* topk_weights, const uint8_t* w1, const uint8_t* s1, const uint8_t* w2,
                         const uint8_t* s2, int num_tokens, int hidden, int intermediate, int num_topk,
                         int num_experts, int expert_begin, int num_local, void* y, int32_t* expert_token_nums,
                         void* stream)
{
    using namespace dpep;
    Workspace* w = as_workspace(ws);
    DPEP_REQUIRE(w != nullptr, "megamoe_forward: not a live workspace");
    DPEP_REQUIRE(num_tokens >= 1 && num_topk >= 1 && num_topk <= DPEP_MAX_TOPK, "megamoe_forward: bad B=%d K=%d",
                 num_tokens, num_topk);
    DPEP_REQUIRE(hidden % 256 == 0 && intermediate % 256 == 0 && hidden > 0 && intermediate > 0,
                 "megamoe_forward: hidden=%d and intermediate=%d must be positive multiples of 256", hidden, intermediate);
    DPEP_REQUIRE(num_local >= 1 && num_local <= DPEP_MAX_LOCAL_EXPERTS && expert_begin >= 0 &&
                     expert_begin + num_local <= num_experts,
                 "megamoe_forward: bad expert range E=%d begin=%d L=%d", num_experts, expert_begin, num_local);
    DPEP_REQUIRE(x_codes && x_scales && topk_idx && topk_weights && w1 && s1 && w2 && s2 && y && expert_token_nums,
                 "megamoe_forward: NULL buffer");
    DPEP_REQUIRE(aligned16(x_codes) && aligned16(w1) && aligned16(w2) && aligned16(y), "megamoe_forward: misaligned buffer");
    const MegaLayout l = mega_layout(num_tokens, num_topk, hidden, intermediate, num_local);
    DPEP_REQUIRE(l.total <= w->bytes, "megamoe_forward: workspace too small (%zu needed, %zu available)", l.total, w->bytes);
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint8_t* base = static_cast<uint8_t*>(w->base);
    int32_t* meta = reinterpret_cast<int32_t*>(base + l.meta);
    int32_t* psum = meta;
    int32_t* offsets = meta + num_local;
    int32_t* num_rows = meta + 2 * num_local + 1;
    int32_t* route_to_row = reinterpret_cast<int32_t*>(base + l.route_to_row);
    int32_t* row_to_route = reinterpret_cast<int32_t*>(base + l.row_to_route);
    if (int rc = layout_i32(ws, topk_idx, num_tokens, num_topk, num_experts, expert_begin, num_local, expert_token_nums,
                            psum, offsets, route_to_row, row_to_route, num_rows, s))
        return rc;
    GemmParams g1{};
    g1.a_codes = static_cast<const uint8_t*>(x_codes);
    g1.a_scales = x_scales;
    g1.row_to_route = row_to_route;
    g1.topk = num_topk;
    g1.offsets = offsets;
    g1.num_local = num_local;
    g1.w = w1;
    g1.ws = s1;
    g1.n = 2 * intermediate;
    g1.k = hidden;
    g1.act_codes = base + l.act_codes;
    g1.act_scales = base + l.act_scales;
    if (int rc = launch_gemm1(g1, s)) return rc;
    GemmParams g2{};
    g2.a_codes = base + l.act_codes;
    g2.a_scales = base + l.act_scales;
    g2.row_to_route = nullptr;
    g2.topk = 1;
    g2.offsets = offsets;
    g2.num_local = num_local;
    g2.w = w2;
    g2.ws = s2;
    g2.n = hidden;
    g2.k = intermediate;
    g2.out = reinterpret_cast<uint16_t*>(base + l.out2);
    if (int rc = launch_gemm2(g2, s)) return rc;
    // Expected rows (the true count stays on the device): tokens * topk * local / experts.
    const long long expected_rows = static_cast<long long>(num_tokens) * num_topk * num_local / num_experts;
    return combine_routes(base + l.out2, topk_weights, route_to_row, num_tokens, num_topk,
                          static_cast<int>(expected_rows), hidden, y, s);
}

}  // extern "C"
