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

// Four fp32 values -> four E4M3 codes (first value in the low byte), same results as
// f32_to_e4m3.  gfx950 converts fp32 to OCP E4M3 in hardware, two values per instruction,
// round to nearest even; values beyond +-448 are clamped first (the reference's saturating
// conversion), and a group that holds a NaN (or whose sum is one) takes the bit-level
// routine, which keeps the NaN's sign.
__device__ __forceinline__ uint32_t
e4m3_pack4(float a, float b, float c, float d) {
    const float s = (a + b) + (c + d);
    if (s != s) return f32_to_e4m3(a) | (f32_to_e4m3(b) << 8) | (f32_to_e4m3(c) << 16) | (f32_to_e4m3(d) << 24);
    a = __builtin_amdgcn_fmed3f(a, -448.0f, 448.0f);
    b = __builtin_amdgcn_fmed3f(b, -448.0f, 448.0f);
    c = __builtin_amdgcn_fmed3f(c, -448.0f, 448.0f);
    d = __builtin_amdgcn_fmed3f(d, -448.0f, 448.0f);
    int pk = 0;
    pk = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, pk, false);
    pk = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, pk, true);
    return static_cast<uint32_t>(pk);
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

// Streaming store with device scope ("sc1 nt"): measured a little faster than the plain
// non-temporal store for rows that are written once and read by a later kernel.
__device__ __forceinline__ void
st16_stream(void *p, const uint4 &x) {
    const ep_v4u v = {x.x, x.y, x.z, x.w};
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt"
                 :
                 : "v"((__attribute__((address_space(1))) ep_v4u *)(reinterpret_cast<uintptr_t>(p))), "v"(v)
                 : "memory");
}

// ---- wave-wide reductions on the DPP data path ------------------------------------------------

constexpr int kEpWaveSize = 64;

template<int CTRL, int ROW_MASK>
__device__ __forceinline__ int
dpp_move(int x) {
    // lanes whose row is masked out, or whose source lane does not exist, keep x
    return __builtin_amdgcn_update_dpp(x, x, CTRL, ROW_MASK, 0xf, false);
}

// Reduction of one 32-bit value per lane over the wave; every lane of the last row (and so
// lane 63) holds the result.  op must be idempotent (max, min).
template<typename Op>
__device__ __forceinline__ int
wave_reduce_dpp(int x, Op op) {
    x = op(x, dpp_move<0xb1, 0xf>(x));  // quad_perm [1,0,3,2]
    x = op(x, dpp_move<0x4e, 0xf>(x));  // quad_perm [2,3,0,1]
    x = op(x, dpp_move<0x124, 0xf>(x)); // row_ror 4
    x = op(x, dpp_move<0x128, 0xf>(x)); // row_ror 8
    x = op(x, dpp_move<0x142, 0xa>(x)); // row_bcast 15 into rows 1 and 3
    x = op(x, dpp_move<0x143, 0xc>(x)); // row_bcast 31 into rows 2 and 3
    return __builtin_amdgcn_readlane(x, kEpWaveSize - 1);
}

// Order-preserving map of a float onto a signed integer (negative floats reversed), so that
// integer max is float max; -0.0 and +0.0 stay distinct neighbours, which the tie rule of the
// values below undoes by comparing the floats themselves.
__device__ __forceinline__ int
float_order_key(float f) {
    const int b = __float_as_int(f);
    return b >= 0 ? b : b ^ 0x7fffffff;
}


// One router round for a wave that holds one token's logits, PL per lane (lane l holds experts
// l, l + 64, ...): the largest value not taken yet, ties to the lower expert index, NaNs
// last in index order.  Marks the winner taken in its lane and returns it in every lane.
template<int PL>
__device__ __forceinline__ void
router_round(const float (&v)[PL], unsigned &taken, int lane, float &top, int &win) {
    float best = 0.f;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < PL; ++j) {
        const int e = j * kEpWaveSize + lane;
        if (!((taken >> j) & 1u) && (best_e == 0x7fffffff || v[j] > best)) {
            best = v[j];
            best_e = e;
        }
    }
    const bool have = best_e != 0x7fffffff;
    // largest value among the lanes that still have one
    const int key = have ? float_order_key(best) : static_cast<int>(0x80000000);
    const int top_key = wave_reduce_dpp(key, [](int a, int b) { return a > b ? a : b; });
    top = __int_as_float(top_key >= 0 ? top_key : top_key ^ 0x7fffffff);
    // lowest expert index among the lanes that hold a value equal to it (0.0 == -0.0)
    const int cand = (have && best == top) ? best_e : 0x7fffffff;
    win = wave_reduce_dpp(cand, [](int a, int b) { return a < b ? a : b; });
    if (win == 0x7fffffff) // only NaNs are left: take them in index order
        win = wave_reduce_dpp(have ? best_e : 0x7fffffff, [](int a, int b) { return a < b ? a : b; });
    if ((win & (kEpWaveSize - 1)) == lane) taken |= 1u << (win / kEpWaveSize);
}

#endif
