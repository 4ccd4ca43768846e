// Drives the HIP backend plugin through the raw south-bound API, the way the reference's
// plugin tests drive a backend without an agent (test/gtest/plugins/transfer_handler.h:
// 125-209; round trip "WRITE, reset the source, READ, check the pattern",
// test/gtest/plugins/obj/obj_plugin.cpp:93-101 with the increasing-byte pattern of
// test/gtest/plugins/memory_handler.h:42-58; handle reuse, test/unit/plugins/ucx/
// ucx_backend_test.cpp:28-92).  The plugin is opened with the flags the reference's plugin
// manager uses (src/core/nixl_plugin_manager.cpp:342).
//
// usage: sb_api_roundtrip <path to libplugin_HIP.so>; prints "OK" and exits 0 on success.
#include <dlfcn.h>
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "backend/backend_engine.h"
#include "backend/backend_plugin.h"

#define REQUIRE(cond)                                                          \
    do {                                                                       \
        if (!(cond)) {                                                         \
            std::fprintf(stderr, "%s:%d: %s failed\n", __FILE__, __LINE__, #cond); \
            std::exit(1);                                                      \
        }                                                                      \
    } while (0)

namespace {

void
fillIncreasing(std::vector<uint8_t> &v, uint8_t start) {
    for (size_t i = 0; i < v.size(); ++i)
        v[i] = static_cast<uint8_t>(start + i);
}

bool
checkIncreasing(const std::vector<uint8_t> &v, uint8_t start) {
    for (size_t i = 0; i < v.size(); ++i)
        if (v[i] != static_cast<uint8_t>(start + i)) return false;
    return true;
}

nixl_status_t
runToCompletion(nixlBackendEngine *engine,
                nixl_xfer_op_t op,
                const nixl_meta_dlist_t &local,
                const nixl_meta_dlist_t &remote,
                const std::string &agent,
                nixlBackendReqH *&handle) {
    nixl_status_t st = engine->postXfer(op, local, remote, agent, handle);
    while (st == NIXL_IN_PROG)
        st = engine->checkXfer(handle);
    return st;
}

} // namespace

int
main(int argc, char **argv) {
    REQUIRE(argc == 2);
    void *lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL | RTLD_NODELETE);
    if (!lib) {
        std::fprintf(stderr, "dlopen: %s\n", dlerror());
        return 1;
    }
    using init_fn = nixlBackendPlugin *(*)();
    using fini_fn = void (*)();
    auto init = reinterpret_cast<init_fn>(dlsym(lib, "nixl_plugin_init"));
    auto fini = reinterpret_cast<fini_fn>(dlsym(lib, "nixl_plugin_fini"));
    REQUIRE(init && fini);
    nixlBackendPlugin *plugin = init();
    REQUIRE(plugin && plugin->api_version == NIXL_PLUGIN_API_VERSION);
    REQUIRE(std::string(plugin->get_plugin_name()) == "HIP");
    const nixl_mem_list_t mems = plugin->get_backend_mems();
    REQUIRE(std::find(mems.begin(), mems.end(), VRAM_SEG) != mems.end());

    const std::string agent = "sb-tester";
    nixl_b_params_t custom;
    nixlBackendInitParams params;
    params.localAgent = agent;
    params.type = "HIP";
    params.customParams = &custom;
    params.enableProgTh = false;
    params.pthrDelay = 0;
    params.syncMode = nixl_thread_sync_t::NIXL_THREAD_SYNC_NONE;
    nixlBackendEngine *engine = plugin->create_engine(&params);
    REQUIRE(engine && !engine->getInitErr());
    // remote = other agents of this process; a remote-capable backend must carry notifications
    REQUIRE(engine->supportsLocal() && engine->supportsRemote() && engine->supportsNotif());
    std::string conn;
    REQUIRE(engine->getConnInfo(conn) == NIXL_SUCCESS && !conn.empty());
    REQUIRE(engine->connect("stranger") == NIXL_ERR_NOT_FOUND);
    REQUIRE(engine->connect(agent) == NIXL_SUCCESS);

    // 48 descriptors of 20 KiB + one of 4 KiB + 16 B + one odd-sized one, local -> remote
    const size_t n_big = 48, big = 20480;
    const std::vector<size_t> lens = [&] {
        std::vector<size_t> l(n_big, big);
        l.push_back(4096 + 16);
        l.push_back(1001);
        return l;
    }();
    size_t total = 0;
    for (size_t l : lens)
        total += l;
    uint8_t *src = nullptr, *dst = nullptr;
    REQUIRE(hipSetDevice(0) == hipSuccess);
    REQUIRE(hipMalloc(reinterpret_cast<void **>(&src), total) == hipSuccess);
    REQUIRE(hipMalloc(reinterpret_cast<void **>(&dst), 2 * total) == hipSuccess);
    std::vector<uint8_t> host(total), back(total);
    fillIncreasing(host, 7);
    REQUIRE(hipMemcpy(src, host.data(), total, hipMemcpyHostToDevice) == hipSuccess);
    REQUIRE(hipMemset(dst, 0xda, 2 * total) == hipSuccess);
    REQUIRE(hipDeviceSynchronize() == hipSuccess); // hipMemset returns before the fill has run

    nixlBackendMD *src_md = nullptr, *dst_md = nullptr, *dst_remote_md = nullptr;
    REQUIRE(engine->registerMem(nixlBlobDesc(reinterpret_cast<uintptr_t>(src), total, 0, ""), VRAM_SEG, src_md) == NIXL_SUCCESS);
    REQUIRE(engine->registerMem(nixlBlobDesc(reinterpret_cast<uintptr_t>(dst), 2 * total, 0, ""), VRAM_SEG, dst_md) == NIXL_SUCCESS);
    REQUIRE(engine->loadLocalMD(dst_md, dst_remote_md) == NIXL_SUCCESS);

    nixl_meta_dlist_t local(VRAM_SEG), remote(VRAM_SEG);
    std::vector<size_t> dst_off(lens.size());
    {
        // destination blocks in reverse order, one gap of `total` bytes in the middle
        size_t s_off = 0, d_off = 2 * total;
        for (size_t i = 0; i < lens.size(); ++i) {
            d_off -= lens[i];
            if (i == lens.size() / 2) d_off -= total;
            dst_off[i] = d_off;
            nixlMetaDesc l(reinterpret_cast<uintptr_t>(src) + s_off, lens[i], 0);
            l.metadataP = src_md;
            nixlMetaDesc r(reinterpret_cast<uintptr_t>(dst) + d_off, lens[i], 0);
            r.metadataP = dst_remote_md;
            local.addDesc(l);
            remote.addDesc(r);
            s_off += lens[i];
        }
    }

    // WRITE: local -> remote
    nixlBackendReqH *wr = nullptr;
    REQUIRE(engine->prepXfer(NIXL_WRITE, local, remote, agent, wr) == NIXL_SUCCESS && wr);
    REQUIRE(engine->checkXfer(wr) == NIXL_SUCCESS); // harmless before any post
    REQUIRE(runToCompletion(engine, NIXL_WRITE, local, remote, agent, wr) == NIXL_SUCCESS);
    std::vector<uint8_t> image(2 * total);
    REQUIRE(hipMemcpy(image.data(), dst, 2 * total, hipMemcpyDeviceToHost) == hipSuccess);
    {
        std::vector<uint8_t> expect(2 * total, 0xda);
        size_t s_off = 0;
        for (size_t i = 0; i < lens.size(); ++i) {
            std::memcpy(expect.data() + dst_off[i], host.data() + s_off, lens[i]);
            s_off += lens[i];
        }
        REQUIRE(image == expect); // every byte outside the destination ranges kept its fill
    }

    // reset the source, READ it back: remote -> local
    REQUIRE(hipMemset(src, 0, total) == hipSuccess);
    REQUIRE(hipDeviceSynchronize() == hipSuccess);
    nixlBackendReqH *rd = nullptr;
    REQUIRE(engine->prepXfer(NIXL_READ, local, remote, agent, rd) == NIXL_SUCCESS && rd);
    REQUIRE(runToCompletion(engine, NIXL_READ, local, remote, agent, rd) == NIXL_SUCCESS);
    REQUIRE(hipMemcpy(back.data(), src, total, hipMemcpyDeviceToHost) == hipSuccess);
    REQUIRE(checkIncreasing(back, 7));

    // the same WRITE handle posted again delivers the source's current bytes
    fillIncreasing(host, 101);
    REQUIRE(hipMemcpy(src, host.data(), total, hipMemcpyHostToDevice) == hipSuccess);
    REQUIRE(runToCompletion(engine, NIXL_WRITE, local, remote, agent, wr) == NIXL_SUCCESS);
    REQUIRE(hipMemset(src, 0, total) == hipSuccess);
    REQUIRE(hipDeviceSynchronize() == hipSuccess);
    REQUIRE(runToCompletion(engine, NIXL_READ, local, remote, agent, rd) == NIXL_SUCCESS);
    REQUIRE(hipMemcpy(back.data(), src, total, hipMemcpyDeviceToHost) == hipSuccess);
    REQUIRE(checkIncreasing(back, 101));

    // what the engine must refuse: another agent, lists that disagree
    nixlBackendReqH *bad = nullptr;
    REQUIRE(engine->prepXfer(NIXL_WRITE, local, remote, "someone-else", bad) < 0 && bad == nullptr);
    nixl_meta_dlist_t shorter(VRAM_SEG);
    shorter.addDesc(remote[0]);
    REQUIRE(engine->prepXfer(NIXL_WRITE, local, shorter, agent, bad) < 0 && bad == nullptr);

    REQUIRE(engine->releaseReqH(wr) == NIXL_SUCCESS);
    REQUIRE(engine->releaseReqH(rd) == NIXL_SUCCESS);
    REQUIRE(engine->unloadMD(dst_remote_md) == NIXL_SUCCESS);
    REQUIRE(engine->deregisterMem(src_md) == NIXL_SUCCESS);
    REQUIRE(engine->deregisterMem(dst_md) == NIXL_SUCCESS);
    REQUIRE(engine->disconnect(agent) == NIXL_SUCCESS);
    plugin->destroy_engine(engine);
    fini();
    REQUIRE(hipFree(src) == hipSuccess && hipFree(dst) == hipSuccess);
    std::puts("OK");
    return 0;
}
