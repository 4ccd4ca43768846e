/* Device-side memory-view API for kernels that move data themselves, for HIP on gfx950.
 *
 * Host side: nixlAgent::prepMemView (local or remote descriptor list) returns a
 * nixlMemViewH.  With the HIP backend that handle is a device pointer to the table laid
 * out below; a kernel receives it by value, inside nixlMemViewElem{mvh, index, offset}.
 * The table lives until nixlAgent::releaseMemView.
 *
 * The names, argument order and status codes are the ones of the reference's device
 * header (src/api/gpu/ucx/nixl_device.cuh:25-197), which forwards every call to a network
 * library's device queue.  Here every view entry is memory that the calling GPU can address
 * itself, so a put is a cooperative copy by the calling lanes and a counter increment is
 * one release-ordered atomic:
 *
 *   nixlPut<level>(src, dst, size, channel, flags, status)   src.mvh local, dst.mvh remote
 *   nixlAtomicAdd<level>(value, counter, channel, flags, status)
 *   nixlGetPtr(mvh, index)                                   nullptr for a placeholder entry
 *   nixlGpuGetXferStatus<level>(status)                      NIXL_SUCCESS once data is visible
 *
 * level says which lanes make the call together, with identical arguments:
 *   THREAD  the calling lane alone
 *   WARP    all 64 lanes of the calling wavefront
 *   BLOCK   all threads of the workgroup (the call contains workgroup barriers)
 *   GRID    not offered: returns NIXL_ERR_NOT_SUPPORTED
 *
 * Ordering, as in the reference (nixl_device.cuh:147-149): a counter increment becomes
 * visible only after the writes of earlier puts by the same lanes at the same level.  A put
 * without a following increment is made visible to other workgroups and later kernels by
 * nixlGpuGetXferStatus, or by the end of the kernel.
 *
 * Every call checks index, offset and size against the table and returns
 * NIXL_ERR_INVALID_PARAM instead of touching memory outside an entry.
 */
#ifndef NIXL_AMD_DEVICE_H
#define NIXL_AMD_DEVICE_H

#include <stddef.h>
#include <stdint.h>

/* ---- table layout (host code fills it, device code reads it) ------------------------ */

#define NIXL_AMD_MEM_VIEW_MAGIC 0x5649584cu /* "LXIV" */
#define NIXL_AMD_MEM_VIEW_LOCAL 0u
#define NIXL_AMD_MEM_VIEW_REMOTE 1u

typedef struct nixl_amd_mem_view_entry {
    uint64_t addr; /* 0 for a placeholder (the reference's null-agent entry) */
    uint64_t len;
} nixl_amd_mem_view_entry_t;

typedef struct nixl_amd_mem_view {
    uint32_t magic;
    uint32_t kind; /* NIXL_AMD_MEM_VIEW_LOCAL or _REMOTE */
    uint64_t count;
    /* count entries follow */
} nixl_amd_mem_view_t;

#if defined(__HIPCC__)

#include <hip/hip_runtime.h>

/* nixl_status_t and nixlMemViewH, shared with host code (src/api/cpp/nixl_types.h). */
#include "nixl/nixl_types.h"

enum class nixl_gpu_level_t : uint64_t { THREAD = 0, WARP = 1, BLOCK = 2, GRID = 3 };

namespace nixl_gpu_flags {
/* The caller will post more before it needs this one seen: skip the visibility fence. */
constexpr uint64_t defer = 1;
} // namespace nixl_gpu_flags

/* Nothing stays in flight after a put here; the handle only remembers that one was made. */
struct nixlGpuXferStatusH {
    uint32_t posted;
    int32_t status;
};

struct nixlMemViewElem {
    nixlMemViewH mvh;
    size_t index;  /* entry of the view */
    size_t offset; /* bytes into that entry */
};

namespace nixl_amd_device_detail {

template<nixl_gpu_level_t level>
__device__ inline unsigned
laneOf() {
    if constexpr (level == nixl_gpu_level_t::THREAD) return 0u;
    if constexpr (level == nixl_gpu_level_t::WARP) return __lane_id();
    return (threadIdx.z * blockDim.y + threadIdx.y) * blockDim.x + threadIdx.x;
}

template<nixl_gpu_level_t level>
__device__ inline unsigned
lanesOf() {
    if constexpr (level == nixl_gpu_level_t::THREAD) return 1u;
    if constexpr (level == nixl_gpu_level_t::WARP) return 64u;
    return blockDim.x * blockDim.y * blockDim.z;
}

/* Address of `size` bytes at `offset` in entry `index`, or 0. */
__device__ inline uint64_t
resolve(const void *mvh, size_t index, size_t offset, size_t size, uint32_t kind) {
    const nixl_amd_mem_view_t *v = static_cast<const nixl_amd_mem_view_t *>(mvh);
    if (!v || v->magic != NIXL_AMD_MEM_VIEW_MAGIC || v->kind != kind || index >= v->count) return 0;
    const nixl_amd_mem_view_entry_t e = reinterpret_cast<const nixl_amd_mem_view_entry_t *>(v + 1)[index];
    if (e.addr == 0 || size > e.len || offset > e.len - size) return 0;
    return e.addr + offset;
}

template<nixl_gpu_level_t level>
__device__ inline void
releaseToAgent() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    if constexpr (level == nixl_gpu_level_t::BLOCK) __syncthreads();
}

/* Copies size bytes with the lanes of the level: 16-byte units where source and
 * destination share their alignment modulo 16, single bytes for the ragged ends and for
 * pairs that do not. */
template<nixl_gpu_level_t level>
__device__ inline void
copyBytes(uint64_t dst, uint64_t src, size_t size) {
    const unsigned lane = laneOf<level>();
    const unsigned lanes = lanesOf<level>();
    if (((dst ^ src) & 15u) != 0) {
        for (size_t i = lane; i < size; i += lanes)
            reinterpret_cast<uint8_t *>(dst)[i] = reinterpret_cast<const uint8_t *>(src)[i];
        return;
    }
    size_t head = (16u - (dst & 15u)) & 15u;
    if (head > size) head = size;
    const size_t units = (size - head) >> 4;
    const size_t tail = size - head - (units << 4);
    for (size_t i = lane; i < head; i += lanes)
        reinterpret_cast<uint8_t *>(dst)[i] = reinterpret_cast<const uint8_t *>(src)[i];
    const uint4 *s = reinterpret_cast<const uint4 *>(src + head);
    uint4 *d = reinterpret_cast<uint4 *>(dst + head);
    for (size_t i = lane; i < units; i += lanes)
        d[i] = s[i];
    const size_t done = head + (units << 4);
    for (size_t i = lane; i < tail; i += lanes)
        reinterpret_cast<uint8_t *>(dst)[done + i] = reinterpret_cast<const uint8_t *>(src)[done + i];
}

} // namespace nixl_amd_device_detail

/* reference: src/api/gpu/ucx/nixl_device.cuh:88-103 */
template<nixl_gpu_level_t level = nixl_gpu_level_t::THREAD>
__device__ inline nixl_status_t
nixlGpuGetXferStatus(nixlGpuXferStatusH &xfer_status) {
    if constexpr (level == nixl_gpu_level_t::GRID) return NIXL_ERR_NOT_SUPPORTED;
    if (xfer_status.status < 0) return static_cast<nixl_status_t>(xfer_status.status);
    if (!xfer_status.posted) return NIXL_ERR_NOT_POSTED;
    nixl_amd_device_detail::releaseToAgent<level>();
    return NIXL_SUCCESS;
}

/* reference: src/api/gpu/ucx/nixl_device.cuh:119-142.  Returns NIXL_IN_PROG when the copy
 * was made, as the reference does for a posted put. */
template<nixl_gpu_level_t level = nixl_gpu_level_t::THREAD>
__device__ inline nixl_status_t
nixlPut(const nixlMemViewElem &src,
        const nixlMemViewElem &dst,
        size_t size,
        unsigned channel_id = 0,
        uint64_t flags = 0,
        nixlGpuXferStatusH *xfer_status = nullptr) {
    (void)channel_id; /* channels separate network queues; there is one memory system here */
    if constexpr (level == nixl_gpu_level_t::GRID) return NIXL_ERR_NOT_SUPPORTED;
    namespace d = nixl_amd_device_detail;
    nixl_status_t st = NIXL_IN_PROG;
    if ((flags & ~nixl_gpu_flags::defer) != 0) {
        st = NIXL_ERR_INVALID_PARAM;
    } else {
        const uint64_t s = d::resolve(src.mvh, src.index, src.offset, size, NIXL_AMD_MEM_VIEW_LOCAL);
        const uint64_t t = d::resolve(dst.mvh, dst.index, dst.offset, size, NIXL_AMD_MEM_VIEW_REMOTE);
        if (!s || !t)
            st = NIXL_ERR_INVALID_PARAM;
        else
            d::copyBytes<level>(t, s, size);
    }
    if (xfer_status) {
        xfer_status->posted = 1;
        xfer_status->status = st < 0 ? st : 0;
    }
    return st;
}

/* reference: src/api/gpu/ucx/nixl_device.cuh:159-178.  The counter is a 64-bit word,
 * 8-byte aligned, in a remote view. */
template<nixl_gpu_level_t level = nixl_gpu_level_t::THREAD>
__device__ inline nixl_status_t
nixlAtomicAdd(uint64_t value,
              const nixlMemViewElem &counter,
              unsigned channel_id = 0,
              uint64_t flags = 0,
              nixlGpuXferStatusH *xfer_status = nullptr) {
    (void)channel_id;
    if constexpr (level == nixl_gpu_level_t::GRID) return NIXL_ERR_NOT_SUPPORTED;
    namespace d = nixl_amd_device_detail;
    nixl_status_t st = NIXL_IN_PROG;
    const uint64_t c =
        d::resolve(counter.mvh, counter.index, counter.offset, sizeof(uint64_t), NIXL_AMD_MEM_VIEW_REMOTE);
    if ((flags & ~nixl_gpu_flags::defer) != 0 || !c || (c & 7u) != 0) {
        st = NIXL_ERR_INVALID_PARAM;
    } else {
        /* Every lane of the level publishes its earlier writes; then one lane adds. */
        d::releaseToAgent<level>();
        if (d::laneOf<level>() == 0)
            __hip_atomic_fetch_add(reinterpret_cast<uint64_t *>(c), value, __ATOMIC_RELEASE,
                                   __HIP_MEMORY_SCOPE_AGENT);
    }
    if (xfer_status) {
        xfer_status->posted = 1;
        xfer_status->status = st < 0 ? st : 0;
    }
    return st;
}

/* reference: src/api/gpu/ucx/nixl_device.cuh:191-197 */
__device__ inline void *
nixlGetPtr(nixlMemViewH mvh, size_t index) {
    return reinterpret_cast<void *>(
        nixl_amd_device_detail::resolve(mvh, index, 0, 0, NIXL_AMD_MEM_VIEW_REMOTE));
}

#endif /* __HIPCC__ */
#endif /* NIXL_AMD_DEVICE_H */
