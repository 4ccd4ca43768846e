// Shared by the kernel translation units: error reporting for the C ABI and small device
// helpers.
#ifndef NIXL_AMD_KERNELS_COMMON_H
#define NIXL_AMD_KERNELS_COMMON_H

#include <hip/hip_runtime.h>

#include <string>

#include "nixl_amd_hip.h"

// Records `msg` as the calling thread's last error and returns `code`.
int
nixl_amd_fail(int code, const std::string &msg);

#define HIP_TRY(expr)                                                                        \
    do {                                                                                     \
        hipError_t e_ = (expr);                                                              \
        if (e_ != hipSuccess)                                                                \
            return nixl_amd_fail(NIXL_AMD_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(e_)); \
    } while (0)

constexpr int kWaveSize = 64;

__device__ __forceinline__ uint32_t
uniform(uint32_t v) {
    return __builtin_amdgcn_readfirstlane(v);
}

__device__ __forceinline__ uint64_t
uniform64(uint64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

#endif
