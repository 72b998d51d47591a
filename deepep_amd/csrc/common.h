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
};
constexpr uint32_t kWorkspaceMagic = 0x44504550u;  // "DPEP"
Workspace* as_workspace(void* ws);

constexpr int kWave = 64;

// ---- device helpers -------------------------------------------------------------------------
__device__ __forceinline__ float bf16_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// Round-to-nearest-even fp32 -> bf16 bits (finite inputs; NaN keeps a quiet payload).
__device__ __forceinline__ uint32_t f32_to_bf16(float v)
{
    uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7fffffffu) > 0x7f800000u) return (bits >> 16) | 0x40u;
    return (bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16;
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ u32x4 load16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ void store16_nt(void* p, u32x4 v)
{
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}
__device__ __forceinline__ u32x4 load16_nt(const void* p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}

}  // namespace dpep
