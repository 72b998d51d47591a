// Error reporting and the HBM workspace (the single-GPU stand-in for the reference's symmetric
// SHMEM workspace, csrc/runtime/session.cpp:40-140).
#include <stdarg.h>
#include <stdlib.h>

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
    DPEP_HIP(hipMalloc(&base, bytes));
    dpep::Workspace* w = static_cast<dpep::Workspace*>(malloc(sizeof(dpep::Workspace)));
    if (w == nullptr) {
        (void)hipFree(base);
        return dpep::fail(DPEP_ERUNTIME, "workspace_create: host allocation failed");
    }
    w->magic = dpep::kWorkspaceMagic;
    w->base = base;
    w->bytes = bytes;
    *ws = w;
    return DPEP_OK;
}

int dpep_workspace_destroy(void* ws)
{
    dpep::Workspace* w = dpep::as_workspace(ws);
    DPEP_REQUIRE(w != nullptr, "workspace_destroy: not a live workspace");
    hipError_t err = hipFree(w->base);
    w->magic = 0;
    free(w);
    if (err != hipSuccess) return dpep::fail(DPEP_ERUNTIME, "hipFree failed: %s", hipGetErrorString(err));
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
