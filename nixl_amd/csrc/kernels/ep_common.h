// Device helpers shared by the expert-parallel kernels: bf16 / e4m3 conversions written at
// bit level (so that results do not depend on which conversion instructions a GPU has),
// the per-128-channel scale rule, and 16-byte non-temporal accesses.
#ifndef NIXL_AMD_EP_COMMON_H
#define NIXL_AMD_EP_COMMON_H

#include <hip/hip_runtime.h>

#include <cstdint>

__device__ __forceinline__ float
bf16_lo_to_f32(uint32_t pair) {
    return __uint_as_float(pair << 16);
}

__device__ __forceinline__ float
bf16_hi_to_f32(uint32_t pair) {
    return __uint_as_float(pair & 0xffff0000u);
}

// fp32 -> bf16 bits, round to nearest even; NaN stays a quiet NaN.
__device__ __forceinline__ uint32_t
f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x0040u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

// fp32 -> OCP FP8 E4M3 code (bias 7, no infinity, NaN = S.1111.111, largest finite 448),
// round to nearest even, saturating to +-448: the conversion the reference requests with
// __NV_SATFINITE / __NV_E4M3 (examples/device/ep/csrc/kernels/nixl_ep_ll.cu:175).
__device__ __forceinline__ uint32_t
f32_to_e4m3(float f) {
    const uint32_t u = __float_as_uint(f);
    const uint32_t sign = (u >> 24) & 0x80u;
    const uint32_t a = u & 0x7fffffffu;
    uint32_t code;
    if (a > 0x7f800000u) {
        code = 0x7fu; // NaN
    } else if (a >= 0x43e00000u) { // 448.0f and above, infinity included
        code = 0x7eu;
    } else if (a < 0x3c800000u) { // below 2^-6: multiples of 2^-9, 8 is the code of 2^-6
        code = static_cast<uint32_t>(__float2int_rn(__uint_as_float(a) * 512.0f));
    } else {
        const uint32_t r = a + 0x7ffffu + ((a >> 20) & 1u);
        code = (((r >> 23) - 120u) << 3) | ((r >> 20) & 7u);
    }
    return sign | code;
}

// examples/device/ep/csrc/kernels/utils.cuh:430-456: scale = 448 / amax (IEEE division),
// scale_inv = amax * (1/448.0f); with round_scale both become powers of two,
// scale_inv = 2^ceil(log2(amax / 448)).
__device__ __forceinline__ void
fp8_scales(float amax, bool round_scale, float &scale, float &scale_inv) {
    constexpr float kAmaxInv = 1 / 448.0f;
    if (round_scale) {
        const uint32_t b = __float_as_uint(amax * kAmaxInv);
        const int e = static_cast<int>((b >> 23) & 0xffu) - 127 + ((b & 0x7fffffu) != 0);
        scale = __uint_as_float(static_cast<uint32_t>(127 - e) << 23);
        scale_inv = __uint_as_float(static_cast<uint32_t>(127 + e) << 23);
    } else {
        scale_inv = amax * kAmaxInv;
        scale = 448.0f / amax;
    }
}

using ep_v4u = __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned;

__device__ __forceinline__ uint4
ld16_nt(const void *p) {
    const ep_v4u v = __builtin_nontemporal_load(
        (const __attribute__((address_space(1))) ep_v4u *)(reinterpret_cast<uintptr_t>(p)));
    return make_uint4(v[0], v[1], v[2], v[3]);
}

__device__ __forceinline__ void
st16_nt(void *p, const uint4 &x) {
    const ep_v4u v = {x.x, x.y, x.z, x.w};
    __builtin_nontemporal_store(v, (__attribute__((address_space(1))) ep_v4u *)(reinterpret_cast<uintptr_t>(p)));
}

#endif
