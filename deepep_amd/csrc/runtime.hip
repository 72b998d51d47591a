// Error reporting and the HBM workspace (the single-GPU stand-in for the reference's symmetric
// SHMEM workspace, csrc/runtime/session.cpp:40-140).
#include <stdarg.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "common.h"

namespace dpep {

static thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...)
{
    va_list args;
    va_start(args, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, args);
    va_end(args);
    return code;
}

Workspace* as_workspace(void* ws)
{
    Workspace* w = static_cast<Workspace*>(ws);
    return (w != nullptr && w->magic == kWorkspaceMagic) ? w : nullptr;
}

}  // namespace dpep

extern "C" {

const char* dpep_last_error(void) { return dpep::g_error; }

int dpep_version(void) { return 1; }

int dpep_workspace_create(size_t bytes, void** ws)
{
    DPEP_REQUIRE(ws != nullptr, "workspace_create: ws is NULL");
    DPEP_REQUIRE(bytes > 0, "workspace_create: bytes must be positive");
    *ws = nullptr;
    void* base = nullptr;
    const size_t sync_at = (bytes + 255) / 256 * 256;  // the kernels' synchronisation memory follows the caller's bytes
    DPEP_HIP(hipMalloc(&base, sync_at + dpep::kSyncBytes));
    if (hipError_t cleared = hipMemset(static_cast<char*>(base) + sync_at, 0, dpep::kSyncBytes); cleared != hipSuccess) {
        (void)hipFree(base);
        return dpep::fail(DPEP_ERUNTIME, "workspace_create: %s", hipGetErrorString(cleared));
    }
    dpep::Workspace* w = static_cast<dpep::Workspace*>(malloc(sizeof(dpep::Workspace)));
    if (w == nullptr) {
        (void)hipFree(base);
        return dpep::fail(DPEP_ERUNTIME, "workspace_create: host allocation failed");
    }
    void* mailbox = nullptr;
    void* mailbox_device = nullptr;
    hipError_t err = hipHostMalloc(&mailbox, dpep::kMailboxWords * sizeof(uint32_t), hipHostMallocMapped);
    if (err == hipSuccess) err = hipHostGetDevicePointer(&mailbox_device, mailbox, 0);
    if (err != hipSuccess) {
        if (mailbox != nullptr) (void)hipHostFree(mailbox);
        (void)hipFree(base);
        free(w);
        return dpep::fail(DPEP_ERUNTIME, "workspace_create: pinned host mailbox: %s", hipGetErrorString(err));
    }
    memset(mailbox, 0, dpep::kMailboxWords * sizeof(uint32_t));
    w->magic = dpep::kWorkspaceMagic;
    w->base = base;
    w->bytes = bytes;
    w->mailbox_host = static_cast<uint32_t*>(mailbox);
    w->mailbox_device = static_cast<uint32_t*>(mailbox_device);
    w->sequence = 0;
    w->mailbox_local = 0;
    w->sync = static_cast<char*>(base) + sync_at;
    w->exchange_ticks = dpep::kLayoutExchangeTicks;
    w->exchange_extra_rows = 0;
    w->layout_one_launch = 1;
    w->gemm_tile_rows = 0;
    w->gemm_column_waves = 1;
    w->gemm_zero_fill = 1;
    w->megamoe_served_only = 0;
    w->layout_launches = 0;
    w->timeout_seen = 0;
    *ws = w;
    return DPEP_OK;
}

int dpep_workspace_destroy(void* ws)
{
    dpep::Workspace* w = dpep::as_workspace(ws);
    DPEP_REQUIRE(w != nullptr, "workspace_destroy: not a live workspace");
    hipError_t err = hipFree(w->base);
    const hipError_t err_host = hipHostFree(w->mailbox_host);
    if (err == hipSuccess) err = err_host;
    w->magic = 0;
    free(w);
    if (err != hipSuccess) return dpep::fail(DPEP_ERUNTIME, "hipFree failed: %s", hipGetErrorString(err));
    return DPEP_OK;
}

int dpep_layout_wait(void* ws, int32_t* counts_host, int num_local, int32_t* num_rows_host, long long timeout_us)
{
    dpep::Workspace* w = dpep::as_workspace(ws);
    DPEP_REQUIRE(w != nullptr, "layout_wait: not a live workspace");
    DPEP_REQUIRE(w->sequence != 0, "layout_wait: no layout was launched on this workspace");
    DPEP_REQUIRE(num_rows_host != nullptr, "layout_wait: num_rows_host is NULL");
    DPEP_REQUIRE(counts_host == nullptr || num_local == w->mailbox_local,
                 "layout_wait: num_local=%d does not match the launched layout (%d)", num_local, w->mailbox_local);
    volatile uint32_t* box = w->mailbox_host;
    timespec start;
    clock_gettime(CLOCK_MONOTONIC, &start);
    for (long long spins = 0; box[1] != w->sequence; ++spins) {
        if ((spins & 1023) == 1023) {
            timespec now;
            clock_gettime(CLOCK_MONOTONIC, &now);
            const long long waited = (now.tv_sec - start.tv_sec) * 1000000ll + (now.tv_nsec - start.tv_nsec) / 1000;
            if (waited > timeout_us)
                return dpep::fail(DPEP_ERUNTIME, "layout_wait: the layout kernel did not report within %lld us", timeout_us);
        }
        __builtin_ia32_pause();
    }
    __atomic_thread_fence(__ATOMIC_ACQUIRE);
    if (const uint32_t timed_out = box[dpep::kMailboxTimeout]; timed_out != w->timeout_seen) {
        w->timeout_seen = timed_out;
        w->layout_one_launch = 0;
        return dpep::fail(DPEP_ERUNTIME, "layout_wait: the layout kernel ran out of time waiting for the other workgroups' histograms "
                                         "and reported no rows; layouts on this workspace take two launches from now on");
    }
    *num_rows_host = static_cast<int32_t>(box[0]);
    if (counts_host != nullptr)
        for (int e = 0; e < num_local; ++e) counts_host[e] = static_cast<int32_t>(box[dpep::kMailboxCounts + e]);
    return DPEP_OK;
}

int dpep_workspace_tune(void* ws, const char* key, long long value)
{
    dpep::Workspace* w = dpep::as_workspace(ws);
    DPEP_REQUIRE(w != nullptr && key != nullptr, "workspace_tune: not a live workspace");
    if (strcmp(key, "layout_one_launch") == 0) {
        w->layout_one_launch = value != 0;
    } else if (strcmp(key, "layout_exchange_ticks") == 0) {
        DPEP_REQUIRE(value > 0, "workspace_tune: layout_exchange_ticks must be positive");
        w->exchange_ticks = value;
    } else if (strcmp(key, "layout_exchange_extra_rows") == 0) {
        DPEP_REQUIRE(value >= 0 && value <= 1, "workspace_tune: layout_exchange_extra_rows is 0 or 1");
        w->exchange_extra_rows = static_cast<int>(value);
    } else if (strcmp(key, "gemm_zero_fill") == 0) {
        w->gemm_zero_fill = value != 0;
    } else if (strcmp(key, "megamoe_served_only") == 0) {
        w->megamoe_served_only = value != 0;
    } else if (strcmp(key, "gemm_column_waves") == 0) {
        w->gemm_column_waves = value != 0;
    } else if (strcmp(key, "gemm_tile_rows") == 0) {
        DPEP_REQUIRE(value == 0 || value == 64 || value == 128 || value == 192,
                     "workspace_tune: gemm_tile_rows is 0 (automatic), 64, 128 or 192");
        w->gemm_tile_rows = static_cast<int>(value);
    } else {
        return dpep::fail(DPEP_EINVAL, "workspace_tune: unknown key '%s'", key);
    }
    return DPEP_OK;
}

int dpep_workspace_capacity(void* ws, size_t* bytes)
{
    dpep::Workspace* w = dpep::as_workspace(ws);
    DPEP_REQUIRE(w != nullptr && bytes != nullptr, "workspace_capacity: not a live workspace");
    *bytes = w->bytes;
    return DPEP_OK;
}

}  // extern "C"
