// Memory views and the device-side calls over them, through nixlAgent and the HIP backend.
// The scenarios are the ones of the reference's device API test
// (test/gtest/device_api/single_write_test.cu: one 4 KiB put with a 0xDEADBEEF first word
// at thread, wave and block level, polled with nixlGpuGetXferStatus, :375-421; several
// workers, each with its own pair of views, :424-499; a remote list with a null-agent
// placeholder and nixlGetPtr, :502-556), followed by what a loopback implementation has to
// get right on its own: ragged and misaligned spans against memcpy on the host, counter
// increments ordered after puts, refusals that leave memory untouched, and the reference's
// own arrangement of a sender and a receiver agent that exchange metadata.
//
// usage: mem_view_device_api; prints "OK" and exits 0 on success.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "nixl.h"
#include "nixl_amd_device.h"

#define REQUIRE(cond)                                                              \
    do {                                                                           \
        if (!(cond)) {                                                             \
            std::fprintf(stderr, "%s:%d: %s failed\n", __FILE__, __LINE__, #cond); \
            std::exit(1);                                                          \
        }                                                                          \
    } while (0)

#define HIP_OK(call) REQUIRE((call) == hipSuccess)

namespace {

struct putParams {
    nixlMemViewElem src;
    nixlMemViewElem dst;
    size_t size;
};

// out[0] = status of the last put, out[1] = status after polling.
template<nixl_gpu_level_t level>
__global__ void
putKernel(putParams p, int iters, int *out) {
    nixlGpuXferStatusH status{};
    nixl_status_t st = NIXL_ERR_NOT_POSTED;
    for (int i = 0; i < iters; ++i) {
        st = nixlPut<level>(p.src, p.dst, p.size, 0, 0, &status);
        if (st != NIXL_IN_PROG) break;
        nixl_status_t polled;
        int spins = 0;
        do {
            polled = nixlGpuGetXferStatus<level>(status);
        } while (polled == NIXL_IN_PROG && ++spins < 1000);
        if (threadIdx.x == 0) out[1] = polled;
    }
    if (threadIdx.x == 0) out[0] = st;
}

__global__ void
getPtrKernel(nixlMemViewH mvh, size_t index, void **out) {
    *out = nixlGetPtr(mvh, index);
}

// Each workgroup puts its own slice, then bumps the counter once; the counter entry is the
// last one of the remote view.
__global__ void
putThenCountKernel(nixlMemViewH src, nixlMemViewH dst, size_t slice, size_t counter_index, int *out) {
    const size_t off = blockIdx.x * slice;
    const nixl_status_t a =
        nixlPut<nixl_gpu_level_t::BLOCK>({src, 0, off}, {dst, 0, off}, slice, 0, nixl_gpu_flags::defer);
    const nixl_status_t b = nixlAtomicAdd<nixl_gpu_level_t::BLOCK>(1, {dst, counter_index, 0});
    if (threadIdx.x == 0 && (a != NIXL_IN_PROG || b != NIXL_IN_PROG)) atomicAdd(out, 1);
}

// A consumer that trusts the counter: once it reads `expected`, every slice must be there.
__global__ void
checkAfterCountKernel(const uint64_t *counter, uint64_t expected, const uint32_t *dst, const uint32_t *src,
                      size_t words, int *mismatches) {
    if (__hip_atomic_load(counter, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) != expected) {
        if (threadIdx.x == 0 && blockIdx.x == 0) atomicAdd(mismatches, 1 << 20);
        return;
    }
    for (size_t i = blockIdx.x * blockDim.x + threadIdx.x; i < words; i += size_t(gridDim.x) * blockDim.x)
        if (dst[i] != src[i]) atomicAdd(mismatches, 1);
}

// The same consumer, started before the producers on a stream of its own: one workgroup
// polls the counter a bounded number of times, then checks.  out[0] = polls used, or -1
// if the count never arrived within the bound; out[1] = words that differ.
__global__ void
pollThenCheckKernel(const uint64_t *counter, uint64_t expected, const uint32_t *dst, const uint32_t *src,
                    size_t words, int max_polls, int *out) {
    __shared__ int seen;
    if (threadIdx.x == 0) {
        int polls = 0;
        while (__hip_atomic_load(counter, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) != expected &&
               polls < max_polls) {
            ++polls;
            __builtin_amdgcn_s_sleep(32);
        }
        seen = (polls < max_polls) ? polls : -1;
        out[0] = seen;
    }
    __syncthreads();
    if (seen < 0) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    int bad = 0;
    for (size_t i = threadIdx.x; i < words; i += blockDim.x)
        bad += (__builtin_nontemporal_load(dst + i) != src[i]);
    if (bad) atomicAdd(out + 1, bad);
}

__global__ void
refusalKernel(nixlMemViewH src, nixlMemViewH dst, size_t len, int *out) {
    int i = 0;
    out[i++] = nixlPut({src, 1, 0}, {dst, 0, 0}, 16);           // source index past the table
    out[i++] = nixlPut({src, 0, 0}, {dst, 7, 0}, 16);           // destination index past the table
    out[i++] = nixlPut({src, 0, len - 8}, {dst, 0, 0}, 16);     // source span runs past the entry
    out[i++] = nixlPut({src, 0, 0}, {dst, 0, len}, 1);          // destination offset at the end
    out[i++] = nixlPut({src, 0, 0}, {dst, 1, 0}, 16);           // placeholder entry
    out[i++] = nixlPut({dst, 0, 0}, {src, 0, 0}, 16);           // views swapped
    out[i++] = nixlPut({src, 0, 0}, {dst, 0, 0}, 16, 0, 2);     // unknown flag
    out[i++] = nixlPut({nullptr, 0, 0}, {dst, 0, 0}, 16);       // no view
    out[i++] = nixlAtomicAdd(1, {dst, 0, 4});                   // counter not 8-byte aligned
    out[i++] = nixlAtomicAdd(1, {dst, 0, len - 4});             // counter runs past the entry
    out[i++] = nixlPut<nixl_gpu_level_t::GRID>({src, 0, 0}, {dst, 0, 0}, 16);
    nixlGpuXferStatusH never{};
    out[i++] = nixlGpuGetXferStatus(never);                     // nothing posted on this handle
    nixlGpuXferStatusH failed{};
    (void)nixlPut({src, 1, 0}, {dst, 0, 0}, 16, 0, 0, &failed);
    out[i++] = nixlGpuGetXferStatus(failed);                    // the failure is remembered
    out[i++] = nixlPut({src, 0, 0}, {dst, 0, 0}, 0);            // empty put is fine
}

template<nixl_gpu_level_t level>
__global__ void
raggedKernel(nixlMemViewH src, nixlMemViewH dst, size_t src_off, size_t dst_off, size_t size, int *out) {
    const nixl_status_t st = nixlPut<level>({src, 0, src_off}, {dst, 0, dst_off}, size);
    if (threadIdx.x == 0) *out = st;
}

struct Buffer {
    void *ptr = nullptr;
    size_t len = 0;
};

Buffer
makeRegistered(nixlAgent &agent, size_t len) {
    Buffer b;
    b.len = len;
    HIP_OK(hipMalloc(&b.ptr, len));
    HIP_OK(hipMemset(b.ptr, 0, len));
    nixl_reg_dlist_t reg(VRAM_SEG);
    reg.addDesc(nixlBlobDesc(reinterpret_cast<uintptr_t>(b.ptr), len, 0, ""));
    REQUIRE(agent.registerMem(reg) == NIXL_SUCCESS);
    return b;
}

void
dropRegistered(nixlAgent &agent, Buffer &b) {
    nixl_reg_dlist_t reg(VRAM_SEG);
    reg.addDesc(nixlBlobDesc(reinterpret_cast<uintptr_t>(b.ptr), b.len, 0, ""));
    REQUIRE(agent.deregisterMem(reg) == NIXL_SUCCESS);
    HIP_OK(hipFree(b.ptr));
    b.ptr = nullptr;
}

nixl_local_dlist_t
localList(const std::vector<Buffer> &bufs) {
    nixl_local_dlist_t l(VRAM_SEG);
    for (const Buffer &b : bufs)
        l.addDesc(nixlBasicDesc(reinterpret_cast<uintptr_t>(b.ptr), b.len, 0));
    return l;
}

nixl_remote_dlist_t
remoteList(const std::vector<Buffer> &bufs, const std::string &agent) {
    nixl_remote_dlist_t l(VRAM_SEG);
    for (const Buffer &b : bufs)
        l.addDesc(nixlRemoteDesc(reinterpret_cast<uintptr_t>(b.ptr), b.len, 0, agent));
    return l;
}

template<nixl_gpu_level_t level>
void
singlePut(nixlAgent &agent, const std::string &name, unsigned threads, int *dev_out) {
    constexpr size_t size = 4 * 1024;
    Buffer src = makeRegistered(agent, size), dst = makeRegistered(agent, size);
    const uint32_t pattern = 0xDEADBEEF;
    HIP_OK(hipMemcpy(src.ptr, &pattern, sizeof(pattern), hipMemcpyHostToDevice));

    nixlMemViewH src_mvh = nullptr, dst_mvh = nullptr;
    REQUIRE(agent.prepMemView(localList({src}), src_mvh) == NIXL_SUCCESS && src_mvh);
    REQUIRE(agent.prepMemView(remoteList({dst}, name), dst_mvh) == NIXL_SUCCESS && dst_mvh);

    HIP_OK(hipMemset(dev_out, 0xff, 2 * sizeof(int)));
    HIP_OK(hipDeviceSynchronize());
    putKernel<level><<<1, threads>>>(putParams{{src_mvh, 0, 0}, {dst_mvh, 0, 0}, size}, 100, dev_out);
    HIP_OK(hipGetLastError());
    HIP_OK(hipDeviceSynchronize());
    int out[2];
    HIP_OK(hipMemcpy(out, dev_out, sizeof(out), hipMemcpyDeviceToHost));
    REQUIRE(out[0] == NIXL_IN_PROG && out[1] == NIXL_SUCCESS);

    std::vector<uint32_t> got(size / 4);
    HIP_OK(hipMemcpy(got.data(), dst.ptr, size, hipMemcpyDeviceToHost));
    REQUIRE(got[0] == pattern);
    for (size_t i = 1; i < got.size(); ++i)
        REQUIRE(got[i] == 0);

    agent.releaseMemView(dst_mvh);
    agent.releaseMemView(src_mvh);
    dropRegistered(agent, src);
    dropRegistered(agent, dst);
}

template<nixl_gpu_level_t level>
void
raggedPuts(nixlAgent &agent, const std::string &name, unsigned threads, int *dev_out) {
    constexpr size_t len = 64 * 1024;
    Buffer src = makeRegistered(agent, len), dst = makeRegistered(agent, len);
    std::vector<uint8_t> host_src(len), expect(len), got(len);
    uint32_t x = 12345;
    for (auto &b : host_src) {
        x = x * 1664525u + 1013904223u;
        b = static_cast<uint8_t>(x >> 24);
    }
    HIP_OK(hipMemcpy(src.ptr, host_src.data(), len, hipMemcpyHostToDevice));
    nixlMemViewH src_mvh = nullptr, dst_mvh = nullptr;
    REQUIRE(agent.prepMemView(localList({src}), src_mvh) == NIXL_SUCCESS);
    REQUIRE(agent.prepMemView(remoteList({dst}, name), dst_mvh) == NIXL_SUCCESS);

    // {source offset, destination offset, size}: equal and unequal alignment modulo 16,
    // spans shorter than one unit, spans whose head swallows everything, a long one.
    const size_t cases[][3] = {{0, 0, 4096},   {3, 3, 1000},  {5, 21, 777},  {1, 2, 333},   {16, 16, 1},
                               {15, 31, 1},    {7, 7, 5},     {9, 9, 7},     {32, 48, 15},  {100, 4100, 33000},
                               {13, 14, 33001}, {0, 8, 16},    {8, 0, 17},    {40000, 50000, 15536}};
    for (const auto &c : cases) {
        std::memset(expect.data(), 0xA5, len);
        HIP_OK(hipMemset(dst.ptr, 0xA5, len));
        HIP_OK(hipDeviceSynchronize());
        std::memcpy(expect.data() + c[1], host_src.data() + c[0], c[2]);
        raggedKernel<level><<<1, threads>>>(src_mvh, dst_mvh, c[0], c[1], c[2], dev_out);
        HIP_OK(hipGetLastError());
        HIP_OK(hipDeviceSynchronize());
        int st = 0;
        HIP_OK(hipMemcpy(&st, dev_out, sizeof(st), hipMemcpyDeviceToHost));
        REQUIRE(st == NIXL_IN_PROG);
        HIP_OK(hipMemcpy(got.data(), dst.ptr, len, hipMemcpyDeviceToHost));
        if (std::memcmp(got.data(), expect.data(), len) != 0) {
            std::fprintf(stderr, "ragged put {%zu, %zu, %zu} at level %d differs from memcpy\n", c[0], c[1], c[2],
                         static_cast<int>(level));
            std::exit(1);
        }
    }
    agent.releaseMemView(dst_mvh);
    agent.releaseMemView(src_mvh);
    dropRegistered(agent, src);
    dropRegistered(agent, dst);
}

} // namespace

int
main() {
    int n_dev = 0;
    if (hipGetDeviceCount(&n_dev) != hipSuccess || n_dev < 1) {
        std::fprintf(stderr, "no HIP device\n");
        return 2;
    }
    HIP_OK(hipSetDevice(0));

    const std::string name = "views";
    nixlAgent agent(name, nixlAgentConfig(false));
    nixlBackendH *backend = nullptr;
    nixl_b_params_t params;
    nixl_mem_list_t mems;
    REQUIRE(agent.getPluginParams("HIP", mems, params) == NIXL_SUCCESS);
    REQUIRE(agent.createBackend("HIP", params, backend) == NIXL_SUCCESS && backend);

    int *dev_out = nullptr;
    HIP_OK(hipMalloc(&dev_out, 64 * sizeof(int)));

    // 1. one 4 KiB put per level
    singlePut<nixl_gpu_level_t::THREAD>(agent, name, 1, dev_out);
    singlePut<nixl_gpu_level_t::WARP>(agent, name, 64, dev_out);
    singlePut<nixl_gpu_level_t::BLOCK>(agent, name, 256, dev_out);
    std::printf("single put: thread, wave, block\n");

    // 2. several workers, each with its own buffers and views, all kernels in flight together
    {
        constexpr int workers = 4;
        constexpr size_t size = 4 * 1024;
        std::vector<Buffer> src(workers), dst(workers);
        std::vector<nixlMemViewH> sv(workers), dv(workers);
        std::vector<hipStream_t> streams(workers);
        for (int w = 0; w < workers; ++w) {
            src[w] = makeRegistered(agent, size);
            dst[w] = makeRegistered(agent, size);
            const uint32_t pattern = 0xDEADBEEF + w;
            HIP_OK(hipMemcpy(src[w].ptr, &pattern, sizeof(pattern), hipMemcpyHostToDevice));
            REQUIRE(agent.prepMemView(localList({src[w]}), sv[w]) == NIXL_SUCCESS);
            REQUIRE(agent.prepMemView(remoteList({dst[w]}, name), dv[w]) == NIXL_SUCCESS);
            HIP_OK(hipStreamCreateWithFlags(&streams[w], hipStreamNonBlocking));
        }
        HIP_OK(hipMemset(dev_out, 0xff, 2 * workers * sizeof(int)));
        HIP_OK(hipDeviceSynchronize());
        for (int w = 0; w < workers; ++w) {
            putKernel<nixl_gpu_level_t::WARP><<<1, 64, 0, streams[w]>>>(
                putParams{{sv[w], 0, 0}, {dv[w], 0, 0}, size}, 50, dev_out + 2 * w);
            HIP_OK(hipGetLastError());
        }
        HIP_OK(hipDeviceSynchronize());
        for (int w = 0; w < workers; ++w) {
            uint32_t got = 0;
            HIP_OK(hipMemcpy(&got, dst[w].ptr, sizeof(got), hipMemcpyDeviceToHost));
            REQUIRE(got == 0xDEADBEEF + static_cast<uint32_t>(w));
            agent.releaseMemView(dv[w]);
            agent.releaseMemView(sv[w]);
            HIP_OK(hipStreamDestroy(streams[w]));
            dropRegistered(agent, src[w]);
            dropRegistered(agent, dst[w]);
        }
        std::printf("several workers\n");
    }

    // 3. placeholder entry, nixlGetPtr
    {
        constexpr size_t size = 4 * 1024;
        Buffer src = makeRegistered(agent, size), dst = makeRegistered(agent, size);
        const uint32_t pattern = 0xDEADBEEF;
        HIP_OK(hipMemcpy(src.ptr, &pattern, sizeof(pattern), hipMemcpyHostToDevice));
        nixlMemViewH src_mvh = nullptr, dst_mvh = nullptr;
        REQUIRE(agent.prepMemView(localList({src}), src_mvh) == NIXL_SUCCESS);
        nixl_remote_dlist_t remote = remoteList({dst}, name);
        remote.addDesc(nixlRemoteDesc(nixlBasicDesc(), nixl_null_agent));
        REQUIRE(agent.prepMemView(remote, dst_mvh) == NIXL_SUCCESS);

        HIP_OK(hipDeviceSynchronize());
        putKernel<nixl_gpu_level_t::THREAD><<<1, 1>>>(putParams{{src_mvh, 0, 0}, {dst_mvh, 0, 0}, size}, 10, dev_out);
        HIP_OK(hipGetLastError());
        void **dev_ptr = nullptr;
        HIP_OK(hipMalloc(&dev_ptr, 2 * sizeof(void *)));
        getPtrKernel<<<1, 1>>>(dst_mvh, 0, dev_ptr);
        getPtrKernel<<<1, 1>>>(dst_mvh, 1, dev_ptr + 1);
        HIP_OK(hipGetLastError());
        HIP_OK(hipDeviceSynchronize());
        void *ptrs[2];
        HIP_OK(hipMemcpy(ptrs, dev_ptr, sizeof(ptrs), hipMemcpyDeviceToHost));
        REQUIRE(ptrs[0] == dst.ptr);
        REQUIRE(ptrs[1] == nullptr);
        uint32_t got = 0;
        HIP_OK(hipMemcpy(&got, dst.ptr, sizeof(got), hipMemcpyDeviceToHost));
        REQUIRE(got == pattern);

        // 4. refusals: statuses, and both buffers exactly as they were
        std::vector<uint8_t> before_src(size), before_dst(size), after(size);
        HIP_OK(hipMemcpy(before_src.data(), src.ptr, size, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(before_dst.data(), dst.ptr, size, hipMemcpyDeviceToHost));
        HIP_OK(hipMemset(dev_out, 0x7f, 16 * sizeof(int)));
        HIP_OK(hipDeviceSynchronize());
        refusalKernel<<<1, 1>>>(src_mvh, dst_mvh, size, dev_out);
        HIP_OK(hipGetLastError());
        HIP_OK(hipDeviceSynchronize());
        int out[14];
        HIP_OK(hipMemcpy(out, dev_out, sizeof(out), hipMemcpyDeviceToHost));
        for (int i = 0; i < 10; ++i)
            REQUIRE(out[i] == NIXL_ERR_INVALID_PARAM);
        REQUIRE(out[10] == NIXL_ERR_NOT_SUPPORTED);
        REQUIRE(out[11] == NIXL_ERR_NOT_POSTED);
        REQUIRE(out[12] == NIXL_ERR_INVALID_PARAM);
        REQUIRE(out[13] == NIXL_IN_PROG);
        HIP_OK(hipMemcpy(after.data(), src.ptr, size, hipMemcpyDeviceToHost));
        REQUIRE(after == before_src);
        HIP_OK(hipMemcpy(after.data(), dst.ptr, size, hipMemcpyDeviceToHost));
        REQUIRE(after == before_dst);

        HIP_OK(hipFree(dev_ptr));
        agent.releaseMemView(dst_mvh);
        agent.releaseMemView(src_mvh);
        dropRegistered(agent, src);
        dropRegistered(agent, dst);
        std::printf("placeholder, getPtr, refusals\n");
    }

    // 5. ragged and misaligned spans against memcpy
    raggedPuts<nixl_gpu_level_t::THREAD>(agent, name, 1, dev_out);
    raggedPuts<nixl_gpu_level_t::WARP>(agent, name, 64, dev_out);
    raggedPuts<nixl_gpu_level_t::BLOCK>(agent, name, 256, dev_out);
    std::printf("ragged spans\n");

    // 6. puts by many workgroups, one counter increment each; a later kernel that reads the
    //    full count must see every slice
    {
        constexpr size_t slice = 16 * 1024;
        constexpr unsigned groups = 512;
        constexpr size_t len = slice * groups;
        Buffer src = makeRegistered(agent, len), dst = makeRegistered(agent, len), counter = makeRegistered(agent, 64);
        std::vector<uint32_t> host(len / 4);
        uint32_t x = 99;
        for (auto &w : host) {
            x = x * 1664525u + 1013904223u;
            w = x;
        }
        HIP_OK(hipMemcpy(src.ptr, host.data(), len, hipMemcpyHostToDevice));
        nixlMemViewH src_mvh = nullptr, dst_mvh = nullptr;
        REQUIRE(agent.prepMemView(localList({src}), src_mvh) == NIXL_SUCCESS);
        REQUIRE(agent.prepMemView(remoteList({dst, counter}, name), dst_mvh) == NIXL_SUCCESS);
        HIP_OK(hipMemset(dev_out, 0, 2 * sizeof(int)));
        HIP_OK(hipDeviceSynchronize());
        putThenCountKernel<<<groups, 256>>>(src_mvh, dst_mvh, slice, 1, dev_out);
        HIP_OK(hipGetLastError());
        checkAfterCountKernel<<<256, 256>>>(static_cast<const uint64_t *>(counter.ptr), groups,
                                            static_cast<const uint32_t *>(dst.ptr),
                                            static_cast<const uint32_t *>(src.ptr), len / 4, dev_out + 1);
        HIP_OK(hipGetLastError());
        HIP_OK(hipDeviceSynchronize());
        int out[2];
        HIP_OK(hipMemcpy(out, dev_out, sizeof(out), hipMemcpyDeviceToHost));
        REQUIRE(out[0] == 0);
        REQUIRE(out[1] == 0);
        uint64_t count = 0;
        HIP_OK(hipMemcpy(&count, counter.ptr, sizeof(count), hipMemcpyDeviceToHost));
        REQUIRE(count == groups);
        std::vector<uint32_t> got(len / 4);
        HIP_OK(hipMemcpy(got.data(), dst.ptr, len, hipMemcpyDeviceToHost));
        REQUIRE(got == host);

        // Again with the consumer already polling while the producers run.
        hipStream_t producer = nullptr, consumer = nullptr;
        HIP_OK(hipStreamCreateWithFlags(&producer, hipStreamNonBlocking));
        HIP_OK(hipStreamCreateWithFlags(&consumer, hipStreamNonBlocking));
        HIP_OK(hipMemset(dst.ptr, 0, len));
        HIP_OK(hipMemset(counter.ptr, 0, 64));
        HIP_OK(hipMemset(dev_out, 0, 4 * sizeof(int)));
        HIP_OK(hipDeviceSynchronize());
        pollThenCheckKernel<<<1, 1024, 0, consumer>>>(static_cast<const uint64_t *>(counter.ptr), groups,
                                                      static_cast<const uint32_t *>(dst.ptr),
                                                      static_cast<const uint32_t *>(src.ptr), len / 4, 1 << 20,
                                                      dev_out + 2);
        HIP_OK(hipGetLastError());
        putThenCountKernel<<<groups, 256, 0, producer>>>(src_mvh, dst_mvh, slice, 1, dev_out);
        HIP_OK(hipGetLastError());
        HIP_OK(hipDeviceSynchronize());
        int conc[4];
        HIP_OK(hipMemcpy(conc, dev_out, sizeof(conc), hipMemcpyDeviceToHost));
        REQUIRE(conc[0] == 0);
        REQUIRE(conc[2] >= 0); // the count arrived within the bound
        REQUIRE(conc[3] == 0); // and every slice was there when it did
        std::printf("puts then counter (consumer polled %d times)\n", conc[2]);
        HIP_OK(hipStreamDestroy(producer));
        HIP_OK(hipStreamDestroy(consumer));

        agent.releaseMemView(dst_mvh);
        agent.releaseMemView(src_mvh);
        dropRegistered(agent, src);
        dropRegistered(agent, dst);
        dropRegistered(agent, counter);
    }

    // 7. what the host refuses
    {
        Buffer reg = makeRegistered(agent, 4096);
        void *stray = nullptr;
        HIP_OK(hipMalloc(&stray, 4096));
        nixlMemViewH mvh = nullptr;
        nixl_local_dlist_t unregistered(VRAM_SEG);
        unregistered.addDesc(nixlBasicDesc(reinterpret_cast<uintptr_t>(stray), 4096, 0));
        REQUIRE(agent.prepMemView(unregistered, mvh) == NIXL_ERR_NOT_FOUND && !mvh);
        nixl_local_dlist_t too_long(VRAM_SEG);
        too_long.addDesc(nixlBasicDesc(reinterpret_cast<uintptr_t>(reg.ptr), 8192, 0));
        REQUIRE(agent.prepMemView(too_long, mvh) == NIXL_ERR_NOT_FOUND && !mvh);
        REQUIRE(agent.prepMemView(remoteList({reg}, "stranger"), mvh) == NIXL_ERR_NOT_FOUND && !mvh);
        Buffer fake{stray, 4096};
        REQUIRE(agent.prepMemView(remoteList({fake}, name), mvh) == NIXL_ERR_NOT_FOUND && !mvh);
        // a list of placeholders alone names no backend
        nixl_remote_dlist_t only_null(VRAM_SEG);
        only_null.addDesc(nixlRemoteDesc(nixlBasicDesc(), nixl_null_agent));
        REQUIRE(agent.prepMemView(only_null, mvh) == NIXL_ERR_NOT_FOUND && !mvh);
        // a handle the agent never made is ignored
        agent.releaseMemView(stray);
        // a view left unreleased is freed with the agent
        REQUIRE(agent.prepMemView(localList({reg}), mvh) == NIXL_SUCCESS && mvh);
        HIP_OK(hipFree(stray));
        std::printf("host refusals\n");
    }

    // 8. sender and receiver as two agents of this process, as in the reference's fixture
    //    (single_write_test.cu:170-265: a backend each, metadata exchanged both ways); the
    //    remote view names the receiver, the put lands in the receiver's registration, and a
    //    counter in the receiver's memory tells it so
    {
        const std::string sender_name = "sender", receiver_name = "receiver";
        nixlAgent sender(sender_name, nixlAgentConfig(false)), receiver(receiver_name, nixlAgentConfig(false));
        nixlBackendH *sb = nullptr, *rb = nullptr;
        REQUIRE(sender.createBackend("HIP", params, sb) == NIXL_SUCCESS);
        REQUIRE(receiver.createBackend("HIP", params, rb) == NIXL_SUCCESS);
        constexpr size_t size = 64 * 1024;
        Buffer src = makeRegistered(sender, size), dst = makeRegistered(receiver, size), flag = makeRegistered(receiver, 64);
        std::vector<uint32_t> host(size / 4);
        for (size_t i = 0; i < host.size(); ++i)
            host[i] = 0xDEADBEEF ^ static_cast<uint32_t>(i * 2654435761u);
        HIP_OK(hipMemcpy(src.ptr, host.data(), size, hipMemcpyHostToDevice));

        nixlMemViewH dst_mvh = nullptr;
        // before the metadata is loaded the receiver is unknown to the sender
        REQUIRE(sender.prepMemView(remoteList({dst, flag}, receiver_name), dst_mvh) == NIXL_ERR_NOT_FOUND);
        nixl_blob_t md;
        std::string loaded;
        REQUIRE(receiver.getLocalMD(md) == NIXL_SUCCESS);
        REQUIRE(sender.loadRemoteMD(md, loaded) == NIXL_SUCCESS && loaded == receiver_name);
        REQUIRE(sender.getLocalMD(md) == NIXL_SUCCESS);
        REQUIRE(receiver.loadRemoteMD(md, loaded) == NIXL_SUCCESS && loaded == sender_name);

        nixlMemViewH src_mvh = nullptr;
        REQUIRE(sender.prepMemView(localList({src}), src_mvh) == NIXL_SUCCESS);
        REQUIRE(sender.prepMemView(remoteList({dst, flag}, receiver_name), dst_mvh) == NIXL_SUCCESS);
        // the receiver's buffers are not the sender's own registrations
        nixlMemViewH wrong = nullptr;
        REQUIRE(sender.prepMemView(localList({dst}), wrong) == NIXL_ERR_NOT_FOUND);
        REQUIRE(sender.prepMemView(remoteList({dst}, sender_name), wrong) == NIXL_ERR_NOT_FOUND);

        HIP_OK(hipMemset(dev_out, 0, 2 * sizeof(int)));
        HIP_OK(hipDeviceSynchronize());
        constexpr unsigned groups = 4;
        putThenCountKernel<<<groups, 256>>>(src_mvh, dst_mvh, size / groups, 1, dev_out);
        HIP_OK(hipGetLastError());
        HIP_OK(hipDeviceSynchronize());
        int bad = -1;
        HIP_OK(hipMemcpy(&bad, dev_out, sizeof(bad), hipMemcpyDeviceToHost));
        REQUIRE(bad == 0);
        uint64_t count = 0;
        HIP_OK(hipMemcpy(&count, flag.ptr, sizeof(count), hipMemcpyDeviceToHost));
        REQUIRE(count == groups);
        std::vector<uint32_t> got(size / 4);
        HIP_OK(hipMemcpy(got.data(), dst.ptr, size, hipMemcpyDeviceToHost));
        REQUIRE(got == host);

        // host-initiated transfer between the same two agents, with a notification
        HIP_OK(hipMemset(dst.ptr, 0, size));
        HIP_OK(hipDeviceSynchronize());
        nixl_xfer_dlist_t l(VRAM_SEG), r(VRAM_SEG);
        l.addDesc(nixlBasicDesc(reinterpret_cast<uintptr_t>(src.ptr), size, 0));
        r.addDesc(nixlBasicDesc(reinterpret_cast<uintptr_t>(dst.ptr), size, 0));
        nixl_opt_args_t with_notif;
        with_notif.notifMsg = "landed";
        with_notif.hasNotif = true;
        nixlXferReqH *req = nullptr;
        REQUIRE(sender.createXferReq(NIXL_WRITE, l, r, receiver_name, req, &with_notif) == NIXL_SUCCESS);
        nixl_status_t st = sender.postXferReq(req);
        while (st == NIXL_IN_PROG)
            st = sender.getXferStatus(req);
        REQUIRE(st == NIXL_SUCCESS);
        nixl_notifs_t notifs;
        REQUIRE(receiver.getNotifs(notifs) == NIXL_SUCCESS);
        REQUIRE(notifs.size() == 1 && notifs[sender_name].size() == 1 && notifs[sender_name][0] == "landed");
        HIP_OK(hipMemcpy(got.data(), dst.ptr, size, hipMemcpyDeviceToHost));
        REQUIRE(got == host);
        REQUIRE(sender.releaseXferReq(req) == NIXL_SUCCESS);

        // once the receiver is invalidated, no new view of it can be made
        sender.releaseMemView(dst_mvh);
        sender.releaseMemView(src_mvh);
        REQUIRE(sender.invalidateRemoteMD(receiver_name) == NIXL_SUCCESS);
        REQUIRE(sender.prepMemView(remoteList({dst}, receiver_name), dst_mvh) == NIXL_ERR_NOT_FOUND);
        dropRegistered(sender, src);
        dropRegistered(receiver, dst);
        dropRegistered(receiver, flag);
        std::printf("two agents\n");
    }

    HIP_OK(hipFree(dev_out));
    std::printf("OK\n");
    return 0;
}
