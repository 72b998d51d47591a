// Shared host/device helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/deepep_amd.h"

namespace dpep {

int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define DPEP_REQUIRE(cond, ...)                              \
    do {                                                     \
        if (!(cond)) return ::dpep::fail(DPEP_EINVAL, __VA_ARGS__); \
    } while (0)

#define DPEP_HIP(expr)                                                                          \
    do {                                                                                        \
        hipError_t err_ = (expr);                                                               \
        if (err_ != hipSuccess)                                                                 \
            return ::dpep::fail(DPEP_ERUNTIME, "%s failed: %s", #expr, hipGetErrorString(err_)); \
    } while (0)

inline int launch_status(const char* what)
{
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return fail(DPEP_ERUNTIME, "launch of %s failed: %s", what, hipGetErrorString(err));
    return DPEP_OK;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

struct Workspace {
    uint32_t magic;
    void* base;
    size_t bytes;
    // Host mailbox of the routing layout: pinned host memory the layout kernel writes straight into
    // (word 0 = rows, word 1 = sequence number of the launch, words 2.. = rows per local expert), so that
    // the host learns the output sizes by polling instead of a device-to-host copy plus a stream wait.
    uint32_t* mailbox_host;
    uint32_t* mailbox_device;  // the same memory as the kernels address it
    uint32_t sequence;         // of the most recent layout launch
    int mailbox_local;         // its number of local experts
    // One-launch layout: the memory its workgroups exchange histograms through, the bound of a workgroup's wait for the
    // others' histograms in 100 MHz ticks, and two switches for tests (take two launches instead; expect more
    // histogram rows than there are workgroups, so that the wait runs out).
    void* sync;  // kSyncBytes of device memory behind the caller's bytes, see below
    long long exchange_ticks;
    int exchange_extra_rows;
    int layout_one_launch;
    uint32_t layout_launches;  // number of the most recent layout launch (never 0)
    uint32_t timeout_seen;     // number of the last timed-out launch the host has been told about
    int gemm_zero_fill;        // 1 (default): idle workgroups of the first GEMM zero rows of unserved tokens; 0: the reduce does
    int megamoe_served_only;   // 1: rows of y whose token no local expert serves are left untouched; 0 (default): zeroed
    int gemm_tile_rows;  // 0: the grouped GEMM chooses its tile height; 64 / 128 / 192: forced (tests)
    int gemm_column_waves;  // which grouped GEMM kernel runs: 1 = waves split the columns, weights straight to registers; 0 = 2 x 2 waves, weights through LDS
};
// Device memory the kernels synchronise through, behind the caller's bytes, zero when the workspace is created:
// at offset 0 the one-launch layout's epoch (64 bits: the highest tag any launch has used; a launch tags what it
// publishes with epoch + 1 and raises the epoch when it ends, so a replayed HIP graph gets a fresh tag too); at
// kSyncFillStop the word through which the MegaMoE fillers are told to stop (a counter that only grows: a filler stops when
// it differs from what the filler found at its start, so it needs no clearing and no value from the host); at kSyncReporterTag the tag the one-launch layout's reporter workgroup has settled on
// (64 bits; it publishes no histogram, so this is how the others know that it has read the epoch); from kSyncTagged on the
// tagged per-workgroup histograms of the one-launch layout.
constexpr size_t kSyncFillStop = 64;
constexpr size_t kSyncReporterTag = 128;
constexpr size_t kSyncTagged = 256;
constexpr size_t kSyncTaggedWords = 4096 + DPEP_MAX_LOCAL_EXPERTS;  // (workgroups + 1) * experts never exceeds this
constexpr size_t kSyncBytes = kSyncTagged + kSyncTaggedWords * 8;
// The host mailbox (pinned memory, 32-bit words): word 0 = number of rows and word 1 = sequence number of the layout
// that reported last (one 8-byte store); word kMailboxTimeout = launch number of a layout kernel whose wait for the
// other workgroups' histograms ran out; from word kMailboxCounts on, 16-byte aligned, the per-expert counts.
constexpr int kMailboxTimeout = 2;
constexpr int kMailboxCounts = 4;
constexpr int kMailboxWords = kMailboxCounts + (DPEP_MAX_LOCAL_EXPERTS + 3) / 4 * 4;
constexpr long long kLayoutExchangeTicks = 200000000;  // 2 s
constexpr uint32_t kWorkspaceMagic = 0x44504550u;  // "DPEP"
Workspace* as_workspace(void* ws);

constexpr int kWave = 64;

// ---- device helpers -------------------------------------------------------------------------
__device__ __forceinline__ float bf16_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// Round-to-nearest-even fp32 -> bf16 bits, two at a time: lo in bits 0-15, hi in bits 16-31
// (v_cvt_pk_bf16_f32; NaN stays a quiet NaN).
typedef float dpep_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 dpep_bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi)
{
    const dpep_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, dpep_bf16x2));
}
__device__ __forceinline__ uint32_t f32_to_bf16(float v) { return pack_bf16x2(v, 0.0f) & 0xffffu; }

// The same pair of helpers for IEEE half (low-latency payloads): exact widening, round-to-nearest-even narrowing.
typedef _Float16 dpep_f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float f16_to_f32(uint32_t bits16)
{
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits16)));
}
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi)
{
    const dpep_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, dpep_f16x2));
}

// Local expert of a raw id, -1 if the route is past `end` or its expert is not one of this rank's.
__device__ __forceinline__ int local_expert(long long e, int route, int end, int num_experts, int expert_begin,
                                            int num_local)
{
    const long long local = e - expert_begin;
    const bool valid = route < end && e >= 0 && e < num_experts && local >= 0 && local < num_local;
    return valid ? static_cast<int>(local) : -1;
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ u32x4 load16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
// Streaming (non-temporal) 16-byte accesses: the byte movers write rows nobody reads again soon, and combine reads
// rows once.
__device__ __forceinline__ void store16_nt(void* p, u32x4 v) { __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p)); }
// Write-through 16-byte store (device scope): the line goes to memory without waiting in the L2 for an eviction.  For
// the combine's output, which shares HBM with eight times as many reads, this measured 1 % faster than the streaming store.
__device__ __forceinline__ void store16_through(void* p, u32x4 v)
{
    asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ u32x4 load16_nt(const void* p) { return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)); }

// Counts of four consecutive local experts, first of them `first` (a multiple of 4), into the host mailbox as one
// 16-byte store that goes through every cache (system scope).  One store per four experts instead of four: the
// stores cross PCIe one by one, and a layout over 256 experts that sent a word at a time left the next launch
// waiting behind them.  The caller waits with s_waitcnt vmcnt(0) before it publishes the sequence word.
__device__ __forceinline__ void mailbox_store_counts(uint32_t* mailbox, int first, const int (&four)[4])
{
    const u32x4 v = {static_cast<uint32_t>(four[0]), static_cast<uint32_t>(four[1]), static_cast<uint32_t>(four[2]),
                     static_cast<uint32_t>(four[3])};
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(mailbox + kMailboxCounts + first), "v"(v) : "memory");
}

}  // namespace dpep
