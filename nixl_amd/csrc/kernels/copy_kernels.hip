// Gather/scatter copy kernels for descriptor lists and the C ABI that plans and launches
// them (declared in include/nixl_amd_hip.h).
//
// Data layout of a plan in HBM
//   The 16-byte-aligned descriptors of a request are concatenated, in request order, into
//   one virtual stream measured in 16-byte units.  The plan keeps, per descriptor j,
//   src[j], dst[j] (byte addresses) and prefix[j] (first unit of j in the stream;
//   prefix[n] = total units).  The stream is cut into chunks of 64*UPL units; one
//   wavefront moves one chunk: lane l moves units chunk*64*UPL + k*64 + l, k < UPL, so
//   every load/store instruction of a wave touches 1 KiB of consecutive bytes unless a
//   descriptor boundary falls inside it.  span[c] = {first, last} descriptor touched by
//   chunk c, computed on the host, so a wave never searches the whole prefix array.
//   Descriptors that are not 16-byte aligned in src, dst and len are cut into byte-range
//   work items handled by a second, byte-exact kernel.
//
// What is equal to the reference: the bytes.  For every descriptor, in list order,
// dst[0..len) = src[0..len), the result of the per-descriptor put/get loop at
// src/plugins/ucx/ucx_backend.cpp:1216-1244.  Descriptors of one request must not
// overlap each other's destination ranges (the reference's puts are unordered too).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "nixl_amd_hip.h"

namespace {

thread_local std::string g_last_error;

int
fail(int code, const std::string &msg) {
    g_last_error = msg;
    return code;
}

#define HIP_TRY(expr)                                                                      \
    do {                                                                                   \
        hipError_t e_ = (expr);                                                            \
        if (e_ != hipSuccess)                                                              \
            return fail(NIXL_AMD_ERR_HIP,                                                  \
                        std::string(#expr) + ": " + hipGetErrorString(e_));                \
    } while (0)

constexpr int kWaveSize = 64;
constexpr int kWavesPerWg = 4;
constexpr int kThreadsPerWg = kWaveSize * kWavesPerWg;
constexpr uint32_t kGenericItemBytes = 16384; // byte-path work item size
constexpr int kMaxLdsDescs = 64; // descriptors a wave stages in LDS for one chunk

struct StreamArgs {
    const uint64_t *src; // [n]
    const uint64_t *dst; // [n]
    const uint64_t *prefix; // [n + 1], units
    const uint2 *span; // [n_chunks], {first desc, last desc}
    uint64_t total_units;
    uint32_t n_chunks;
};

struct GenericItem {
    uint64_t src;
    uint64_t dst;
    uint32_t len; // <= kGenericItemBytes
    uint32_t pad;
};

// 16-byte vector in the global address space, so that accesses compile to
// global_load/store_dwordx4 rather than flat instructions.
using v4u = __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned;
using gv4_ptr = __attribute__((address_space(1))) v4u *;
using gv4_cptr = const __attribute__((address_space(1))) v4u *;

template<bool NT>
__device__ __forceinline__ uint4
load16(const uint4 *p) {
    gv4_cptr g = (gv4_cptr)(reinterpret_cast<uintptr_t>(p));
    const v4u v = NT ? __builtin_nontemporal_load(g) : *g;
    return make_uint4(v[0], v[1], v[2], v[3]);
}

template<bool NT>
__device__ __forceinline__ void
store16(uint4 *p, const uint4 &x) {
    gv4_ptr g = (gv4_ptr)(reinterpret_cast<uintptr_t>(p));
    const v4u v = {x.x, x.y, x.z, x.w};
    if constexpr (NT)
        __builtin_nontemporal_store(v, g);
    else
        *g = v;
}

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

// One wavefront per chunk of the virtual stream, 128-bit loads and stores.
template<int UPL, bool NT>
__global__ void __launch_bounds__(kThreadsPerWg)
copy_stream_kernel(StreamArgs a) {
    constexpr uint32_t kChunkUnits = kWaveSize * UPL;
    __shared__ uint64_t lds_prefix[kWavesPerWg][kMaxLdsDescs + 1];
    __shared__ uint64_t lds_src[kWavesPerWg][kMaxLdsDescs];
    __shared__ uint64_t lds_dst[kWavesPerWg][kMaxLdsDescs];

    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const uint32_t wave = threadIdx.x / kWaveSize;
    const uint32_t n_waves = gridDim.x * kWavesPerWg;

    for (uint32_t c = uniform(blockIdx.x * kWavesPerWg + wave); c < a.n_chunks; c += n_waves) {
        const uint2 sp = a.span[c];
        const uint32_t j0 = uniform(sp.x);
        const uint32_t j1 = uniform(sp.y);
        const uint64_t u0 = static_cast<uint64_t>(c) * kChunkUnits;
        const uint64_t remaining = a.total_units - u0; // > 0 because c < n_chunks
        const uint32_t n_units =
            remaining < kChunkUnits ? static_cast<uint32_t>(remaining) : kChunkUnits;

        if (j0 == j1) {
            // The whole chunk lies inside one descriptor: wave-uniform base addresses.
            const uint64_t off = (u0 - uniform64(a.prefix[j0])) * 16u;
            const uint4 *s = reinterpret_cast<const uint4 *>(uniform64(a.src[j0]) + off);
            uint4 *d = reinterpret_cast<uint4 *>(uniform64(a.dst[j0]) + off);
            if (n_units == kChunkUnits) {
                uint4 v[UPL];
#pragma unroll
                for (int k = 0; k < UPL; ++k)
                    v[k] = load16<NT>(s + k * kWaveSize + lane);
#pragma unroll
                for (int k = 0; k < UPL; ++k)
                    store16<NT>(d + k * kWaveSize + lane, v[k]);
            } else {
                for (uint32_t i = lane; i < n_units; i += kWaveSize)
                    store16<NT>(d + i, load16<NT>(s + i));
            }
            continue;
        }

        const uint32_t nd = j1 - j0 + 1;
        if (nd <= kMaxLdsDescs) {
            // Stage this chunk's descriptors in the wave's LDS slice, then each lane walks
            // forward through them as its unit index grows by 64 per step.
            __builtin_amdgcn_wave_barrier();
            if (lane < nd) {
                lds_prefix[wave][lane] = a.prefix[j0 + lane];
                lds_src[wave][lane] = a.src[j0 + lane];
                lds_dst[wave][lane] = a.dst[j0 + lane];
            }
            if (lane == 0) lds_prefix[wave][nd] = a.prefix[j0 + nd];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

            uint32_t jj = 0;
            const uint4 *sp_[UPL];
            uint4 *dp_[UPL];
            uint4 v[UPL];
#pragma unroll
            for (int k = 0; k < UPL; ++k) {
                const uint32_t i = k * kWaveSize + lane;
                sp_[k] = nullptr;
                dp_[k] = nullptr;
                if (i < n_units) {
                    const uint64_t u = u0 + i;
                    while (jj + 1 < nd && lds_prefix[wave][jj + 1] <= u)
                        ++jj;
                    const uint64_t off = (u - lds_prefix[wave][jj]) * 16u;
                    sp_[k] = reinterpret_cast<const uint4 *>(lds_src[wave][jj] + off);
                    dp_[k] = reinterpret_cast<uint4 *>(lds_dst[wave][jj] + off);
                }
            }
#pragma unroll
            for (int k = 0; k < UPL; ++k)
                if (sp_[k]) v[k] = load16<NT>(sp_[k]);
#pragma unroll
            for (int k = 0; k < UPL; ++k)
                if (dp_[k]) store16<NT>(dp_[k], v[k]);
            __builtin_amdgcn_wave_barrier();
        } else {
            // Many tiny descriptors in one chunk: bisect the global prefix array per unit.
            for (uint32_t i = lane; i < n_units; i += kWaveSize) {
                const uint64_t u = u0 + i;
                uint32_t lo = j0, hi = j1;
                while (lo < hi) {
                    const uint32_t mid = lo + (hi - lo + 1) / 2;
                    if (a.prefix[mid] <= u)
                        lo = mid;
                    else
                        hi = mid - 1;
                }
                const uint64_t off = (u - a.prefix[lo]) * 16u;
                const uint4 *s = reinterpret_cast<const uint4 *>(a.src[lo] + off);
                uint4 *d = reinterpret_cast<uint4 *>(a.dst[lo] + off);
                store16<NT>(d, load16<NT>(s));
            }
        }
    }
}

struct __attribute__((packed, aligned(1))) unaligned16 {
    uint32_t w[4];
};

// One wavefront per byte-range work item; correct for any alignment and length.
__global__ void __launch_bounds__(kThreadsPerWg)
copy_generic_kernel(const GenericItem *items, uint32_t n_items) {
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const uint32_t wave = threadIdx.x / kWaveSize;
    const uint32_t n_waves = gridDim.x * kWavesPerWg;
    for (uint32_t it = uniform(blockIdx.x * kWavesPerWg + wave); it < n_items; it += n_waves) {
        const uint64_t src = uniform64(items[it].src);
        const uint64_t dst = uniform64(items[it].dst);
        const uint32_t len = uniform(items[it].len);
        const uint8_t *s = reinterpret_cast<const uint8_t *>(src);
        uint8_t *d = reinterpret_cast<uint8_t *>(dst);

        // Head: bytes until dst is 16-byte aligned (at most 15).
        uint32_t head = static_cast<uint32_t>((16u - (dst & 15u)) & 15u);
        if (head > len) head = len;
        if (lane < head) d[lane] = s[lane];
        const uint32_t body = (len - head) / 16u;
        const uint8_t *sb = s + head;
        uint4 *db = reinterpret_cast<uint4 *>(d + head);
        if (((src + head) & 15u) == 0) {
            const uint4 *sv = reinterpret_cast<const uint4 *>(sb);
            for (uint32_t i = lane; i < body; i += kWaveSize)
                db[i] = sv[i];
        } else {
            const unaligned16 *sv = reinterpret_cast<const unaligned16 *>(sb);
            for (uint32_t i = lane; i < body; i += kWaveSize) {
                const unaligned16 t = sv[i];
                db[i] = make_uint4(t.w[0], t.w[1], t.w[2], t.w[3]);
            }
        }
        const uint32_t done = head + body * 16u;
        const uint32_t tail = len - done; // < 16
        if (lane < tail) d[done + lane] = s[done + lane];
    }
}

} // namespace

struct nixl_amd_copy_plan {
    int device = 0;
    int upl = 8;
    bool nt = true;
    uint32_t max_wgs = 0;
    // device arrays
    void *arena = nullptr;
    size_t arena_bytes = 0;
    StreamArgs stream_args{};
    const GenericItem *generic_items = nullptr;
    uint32_t n_generic = 0;
    uint32_t vec_wgs = 0;
    uint32_t generic_wgs = 0;
    // facts
    nixl_amd_copy_plan_info_t info{};
    // timing events (lazily created)
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
};

extern "C" {

const char *
nixl_amd_last_error(void) {
    return g_last_error.c_str();
}

int
nixl_amd_device_count(void) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) return fail(NIXL_AMD_ERR_NO_DEVICE, hipGetErrorString(e));
    return n;
}

int
nixl_amd_copy_plan_create(const nixl_amd_copy_desc_t *descs,
                          size_t n,
                          int device,
                          const nixl_amd_copy_tuning_t *tuning,
                          nixl_amd_copy_plan_t **out) {
    if (!out) return fail(NIXL_AMD_ERR_INVALID, "plan_create: out is null");
    *out = nullptr;
    if (!descs && n) return fail(NIXL_AMD_ERR_INVALID, "plan_create: descs is null");
    if (n >= (1ull << 32)) return fail(NIXL_AMD_ERR_TOO_LARGE, "plan_create: more than 2^32-1 descriptors");

    int upl = 8, nt = 1;
    uint32_t max_wgs = 0;
    if (tuning) {
        if (tuning->units_per_lane) upl = tuning->units_per_lane;
        if (tuning->nontemporal) nt = tuning->nontemporal;
        if (tuning->max_workgroups > 0) max_wgs = static_cast<uint32_t>(tuning->max_workgroups);
    }
    if (upl != 4 && upl != 8 && upl != 16)
        return fail(NIXL_AMD_ERR_INVALID, "plan_create: units_per_lane must be 4, 8 or 16");
    if (nt != 1 && nt != 2) return fail(NIXL_AMD_ERR_INVALID, "plan_create: nontemporal must be 0, 1 or 2");

    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev <= 0)
        return fail(NIXL_AMD_ERR_NO_DEVICE, "plan_create: no HIP device");
    if (device < 0 || device >= ndev) return fail(NIXL_AMD_ERR_INVALID, "plan_create: bad device index");
    HIP_TRY(hipSetDevice(device));

    // ---- host-side lowering ------------------------------------------------------
    std::vector<uint64_t> vsrc, vdst, vprefix;
    std::vector<GenericItem> items;
    vsrc.reserve(n);
    vdst.reserve(n);
    vprefix.reserve(n + 1);
    uint64_t units = 0, payload = 0, n_generic_descs = 0;
    for (size_t i = 0; i < n; ++i) {
        const nixl_amd_copy_desc_t &d = descs[i];
        if (d.len == 0) continue;
        if (d.src == 0 || d.dst == 0)
            return fail(NIXL_AMD_ERR_INVALID, "plan_create: null address in descriptor " + std::to_string(i));
        if (d.src + d.len < d.src || d.dst + d.len < d.dst)
            return fail(NIXL_AMD_ERR_INVALID, "plan_create: address range wraps in descriptor " + std::to_string(i));
        payload += d.len;
        if (((d.src | d.dst | d.len) & 15u) == 0) {
            vsrc.push_back(d.src);
            vdst.push_back(d.dst);
            vprefix.push_back(units);
            units += d.len / 16u;
        } else {
            ++n_generic_descs;
            for (uint64_t off = 0; off < d.len; off += kGenericItemBytes) {
                GenericItem it{};
                it.src = d.src + off;
                it.dst = d.dst + off;
                it.len = static_cast<uint32_t>(std::min<uint64_t>(kGenericItemBytes, d.len - off));
                items.push_back(it);
            }
        }
    }
    vprefix.push_back(units);
    const size_t nv = vsrc.size();
    const uint64_t chunk_units = static_cast<uint64_t>(kWaveSize) * upl;
    const uint64_t n_chunks64 = (units + chunk_units - 1) / chunk_units;
    if (n_chunks64 >= (1ull << 32) || items.size() >= (1ull << 32))
        return fail(NIXL_AMD_ERR_TOO_LARGE, "plan_create: request too large for 32-bit chunk index");
    const uint32_t n_chunks = static_cast<uint32_t>(n_chunks64);

    std::vector<uint2> span(n_chunks);
    {
        size_t j = 0;
        for (uint32_t c = 0; c < n_chunks; ++c) {
            const uint64_t first = static_cast<uint64_t>(c) * chunk_units;
            const uint64_t last = std::min(units, first + chunk_units) - 1;
            while (vprefix[j + 1] <= first)
                ++j;
            size_t jl = j;
            while (vprefix[jl + 1] <= last)
                ++jl;
            span[c] = make_uint2(static_cast<uint32_t>(j), static_cast<uint32_t>(jl));
        }
    }

    // ---- one device arena for all plan arrays --------------------------------------
    auto align256 = [](size_t x) { return (x + 255) & ~size_t(255); };
    const size_t off_src = 0;
    const size_t off_dst = off_src + align256(nv * 8);
    const size_t off_prefix = off_dst + align256(nv * 8);
    const size_t off_span = off_prefix + align256((nv + 1) * 8);
    const size_t off_items = off_span + align256(size_t(n_chunks) * sizeof(uint2));
    const size_t total = off_items + align256(items.size() * sizeof(GenericItem));

    auto *plan = new nixl_amd_copy_plan();
    plan->device = device;
    plan->upl = upl;
    plan->nt = (nt == 1);
    plan->max_wgs = max_wgs;

    if (total > 0 && (nv > 0 || !items.empty())) {
        std::vector<uint8_t> host(total, 0);
        if (nv) {
            std::memcpy(host.data() + off_src, vsrc.data(), nv * 8);
            std::memcpy(host.data() + off_dst, vdst.data(), nv * 8);
        }
        std::memcpy(host.data() + off_prefix, vprefix.data(), (nv + 1) * 8);
        if (n_chunks) std::memcpy(host.data() + off_span, span.data(), size_t(n_chunks) * sizeof(uint2));
        if (!items.empty())
            std::memcpy(host.data() + off_items, items.data(), items.size() * sizeof(GenericItem));
        hipError_t e = hipMalloc(&plan->arena, total);
        if (e != hipSuccess) {
            delete plan;
            return fail(NIXL_AMD_ERR_HIP, std::string("hipMalloc(plan arena): ") + hipGetErrorString(e));
        }
        e = hipMemcpy(plan->arena, host.data(), total, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            (void)hipFree(plan->arena);
            delete plan;
            return fail(NIXL_AMD_ERR_HIP, std::string("hipMemcpy(plan arena): ") + hipGetErrorString(e));
        }
        plan->arena_bytes = total;
        auto *base = static_cast<uint8_t *>(plan->arena);
        plan->stream_args.src = reinterpret_cast<const uint64_t *>(base + off_src);
        plan->stream_args.dst = reinterpret_cast<const uint64_t *>(base + off_dst);
        plan->stream_args.prefix = reinterpret_cast<const uint64_t *>(base + off_prefix);
        plan->stream_args.span = reinterpret_cast<const uint2 *>(base + off_span);
        plan->generic_items = reinterpret_cast<const GenericItem *>(base + off_items);
    }
    plan->stream_args.total_units = units;
    plan->stream_args.n_chunks = n_chunks;
    plan->n_generic = static_cast<uint32_t>(items.size());

    auto wgs_for = [&](uint32_t waves) {
        uint32_t w = (waves + kWavesPerWg - 1) / kWavesPerWg;
        if (plan->max_wgs && w > plan->max_wgs) w = plan->max_wgs;
        return w;
    };
    plan->vec_wgs = wgs_for(n_chunks);
    plan->generic_wgs = wgs_for(plan->n_generic);

    plan->info.payload_bytes = payload;
    plan->info.vec_descs = nv;
    plan->info.generic_descs = n_generic_descs;
    plan->info.plan_device_bytes = plan->arena_bytes;
    plan->info.vec_chunks = n_chunks;
    plan->info.vec_workgroups = plan->vec_wgs;
    plan->info.generic_items = plan->n_generic;
    plan->info.units_per_lane = static_cast<uint32_t>(upl);
    *out = plan;
    return NIXL_AMD_OK;
}

int
nixl_amd_copy_plan_launch(nixl_amd_copy_plan_t *plan, void *stream) {
    if (!plan) return fail(NIXL_AMD_ERR_INVALID, "plan_launch: plan is null");
    HIP_TRY(hipSetDevice(plan->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (plan->vec_wgs) {
        const dim3 grid(plan->vec_wgs), block(kThreadsPerWg);
        const StreamArgs &a = plan->stream_args;
#define LAUNCH_STREAM(UPL_, NT_) hipLaunchKernelGGL((copy_stream_kernel<UPL_, NT_>), grid, block, 0, s, a)
        if (plan->nt) {
            if (plan->upl == 4) LAUNCH_STREAM(4, true);
            else if (plan->upl == 8) LAUNCH_STREAM(8, true);
            else LAUNCH_STREAM(16, true);
        } else {
            if (plan->upl == 4) LAUNCH_STREAM(4, false);
            else if (plan->upl == 8) LAUNCH_STREAM(8, false);
            else LAUNCH_STREAM(16, false);
        }
#undef LAUNCH_STREAM
        HIP_TRY(hipGetLastError());
    }
    if (plan->generic_wgs) {
        hipLaunchKernelGGL(copy_generic_kernel, dim3(plan->generic_wgs), dim3(kThreadsPerWg), 0, s,
                           plan->generic_items, plan->n_generic);
        HIP_TRY(hipGetLastError());
    }
    return NIXL_AMD_OK;
}

int
nixl_amd_copy_plan_destroy(nixl_amd_copy_plan_t *plan) {
    if (!plan) return NIXL_AMD_OK;
    (void)hipSetDevice(plan->device);
    if (plan->ev0) (void)hipEventDestroy(plan->ev0);
    if (plan->ev1) (void)hipEventDestroy(plan->ev1);
    hipError_t e = plan->arena ? hipFree(plan->arena) : hipSuccess;
    delete plan;
    if (e != hipSuccess) return fail(NIXL_AMD_ERR_HIP, std::string("hipFree(plan arena): ") + hipGetErrorString(e));
    return NIXL_AMD_OK;
}

int
nixl_amd_copy_plan_query(const nixl_amd_copy_plan_t *plan, nixl_amd_copy_plan_info_t *info) {
    if (!plan || !info) return fail(NIXL_AMD_ERR_INVALID, "plan_query: null argument");
    *info = plan->info;
    return NIXL_AMD_OK;
}

int
nixl_amd_copy_plan_time(nixl_amd_copy_plan_t *plan, void *stream, int iters, float *ms_per_launch) {
    if (!plan || !ms_per_launch || iters <= 0)
        return fail(NIXL_AMD_ERR_INVALID, "plan_time: bad argument");
    HIP_TRY(hipSetDevice(plan->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (!plan->ev0) HIP_TRY(hipEventCreate(&plan->ev0));
    if (!plan->ev1) HIP_TRY(hipEventCreate(&plan->ev1));
    HIP_TRY(hipEventRecord(plan->ev0, s));
    for (int i = 0; i < iters; ++i) {
        int rc = nixl_amd_copy_plan_launch(plan, stream);
        if (rc) return rc;
    }
    HIP_TRY(hipEventRecord(plan->ev1, s));
    HIP_TRY(hipEventSynchronize(plan->ev1));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, plan->ev0, plan->ev1));
    *ms_per_launch = ms / static_cast<float>(iters);
    return NIXL_AMD_OK;
}

} // extern "C"
