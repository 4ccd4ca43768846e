#include "common.h"

namespace {
thread_local std::string g_last_error;
}

int
nixl_amd_fail(int code, const std::string &msg) {
    g_last_error = msg;
    return code;
}

extern "C" {

const char *
nixl_amd_last_error(void) {
    return g_last_error.c_str();
}

int
nixl_amd_device_count(void) {
    int n = 0;
    const hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) return nixl_amd_fail(NIXL_AMD_ERR_NO_DEVICE, hipGetErrorString(e));
    return n;
}

} // extern "C"
