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

// Makes `device` current for the calling thread for the lifetime of the object and puts the
// thread's previous device back afterwards: a library call must not leave the application on
// another GPU than it was on.
class DeviceScope {
public:
    explicit DeviceScope(int device) {
        int current = -1;
        if (hipGetDevice(&current) != hipSuccess) current = -1;
        if (current == device) {
            status_ = hipSuccess;
            return;
        }
        status_ = hipSetDevice(device);
        if (status_ == hipSuccess && current >= 0) previous_ = current;
    }

    ~DeviceScope() {
        if (previous_ >= 0) (void)hipSetDevice(previous_);
    }

    DeviceScope(const DeviceScope &) = delete;
    DeviceScope &
    operator=(const DeviceScope &) = delete;

    hipError_t
    status() const {
        return status_;
    }

private:
    int previous_ = -1;
    hipError_t status_ = hipSuccess;
};

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
