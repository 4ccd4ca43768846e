// Drives the HIP backend plugin through the raw south-bound API, the way the reference's
// plugin tests drive a backend without an agent (test/gtest/plugins/transfer_handler.h:
// 125-209; round trip "WRITE, reset the source, READ, check the pattern",
// test/gtest/plugins/obj/obj_plugin.cpp:93-101 with the increasing-byte pattern of
// test/gtest/plugins/memory_handler.h:42-58; handle reuse, test/unit/plugins/ucx/
// ucx_backend_test.cpp:28-92; a second engine as the target of remote transfers and
// notifications, as that test's two-engine set-up).  The plugin is opened with the flags the reference's plugin
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

    // A second engine under another agent name: initiator and target of one process, wired
    // the way the agent wires two backends (connection info, public data of a registration,
    // loadRemoteMD, connect), then a WRITE with a notification and a READ
    // (shape of test/unit/plugins/ucx/ucx_backend_test.cpp: two engines, :383-389 data check,
    // notification seen by the target once the transfer is complete).
    {
        const std::string peer = "sb-peer";
        nixlBackendInitParams peer_params = params;
        peer_params.localAgent = peer;
        nixlBackendEngine *target = plugin->create_engine(&peer_params);
        REQUIRE(target && !target->getInitErr());
        uint8_t *tbuf = nullptr;
        REQUIRE(hipMalloc(reinterpret_cast<void **>(&tbuf), total) == hipSuccess);
        REQUIRE(hipMemset(tbuf, 0, total) == hipSuccess);
        REQUIRE(hipDeviceSynchronize() == hipSuccess);
        nixlBackendMD *t_md = nullptr, *t_at_initiator = nullptr;
        const nixlBlobDesc t_region(reinterpret_cast<uintptr_t>(tbuf), total, 0, "");
        REQUIRE(target->registerMem(t_region, VRAM_SEG, t_md) == NIXL_SUCCESS);

        std::string t_conn, t_public;
        REQUIRE(target->getConnInfo(t_conn) == NIXL_SUCCESS);
        REQUIRE(target->getPublicData(t_md, t_public) == NIXL_SUCCESS && !t_public.empty());
        // nothing of the peer is usable before its connection info is loaded
        REQUIRE(engine->loadRemoteMD(nixlBlobDesc(t_region, t_public), VRAM_SEG, peer, t_at_initiator) < 0);
        REQUIRE(engine->loadRemoteConnInfo(peer, "HIP1:pid=1") < 0); // an older format
        // another process whose mailbox does not exist cannot be connected to
        REQUIRE(engine->loadRemoteConnInfo(peer, "HIP2:pid=1;mbox=/nixl_amd_hip_no_such_mailbox") == NIXL_ERR_NOT_FOUND);
        REQUIRE(engine->loadRemoteConnInfo(peer, "HIP2:pid=1;mbox=") < 0);
        REQUIRE(engine->loadRemoteConnInfo(peer, "garbage") < 0);
        REQUIRE(engine->loadRemoteConnInfo(peer, t_conn) == NIXL_SUCCESS);
        REQUIRE(engine->connect(peer) == NIXL_SUCCESS);
        // public data that does not belong to the descriptor it arrives with is refused
        REQUIRE(engine->loadRemoteMD(nixlBlobDesc(reinterpret_cast<uintptr_t>(tbuf), total / 2, 0, t_public), VRAM_SEG, peer,
                                     t_at_initiator) < 0);
        REQUIRE(engine->loadRemoteMD(nixlBlobDesc(t_region, t_public.substr(1)), VRAM_SEG, peer, t_at_initiator) < 0);
        {
            // a blob that names memory the runtime does not know (a region freed since it was
            // published, a forged record) is refused on the host: no kernel may ever see it
            std::string stale = t_public;
            const uint64_t nowhere = 0x7f0000001000ull;
            std::memcpy(&stale[8], &nowhere, sizeof(nowhere)); // the record's address field
            REQUIRE(engine->loadRemoteMD(nixlBlobDesc(nowhere, total, 0, stale), VRAM_SEG, peer, t_at_initiator) ==
                    NIXL_ERR_INVALID_PARAM);
            REQUIRE(t_at_initiator == nullptr);
            // live memory of the wrong kind: a host buffer published as VRAM
            void *pinned = nullptr;
            REQUIRE(hipHostMalloc(&pinned, 4096, hipHostMallocDefault) == hipSuccess);
            const uint64_t host_addr = reinterpret_cast<uint64_t>(pinned), host_len = 4096;
            std::memcpy(&stale[8], &host_addr, sizeof(host_addr));
            std::memcpy(&stale[16], &host_len, sizeof(host_len));
            REQUIRE(engine->loadRemoteMD(nixlBlobDesc(host_addr, host_len, 0, stale), VRAM_SEG, peer, t_at_initiator) ==
                    NIXL_ERR_INVALID_PARAM);
            REQUIRE(hipHostFree(pinned) == hipSuccess);
        }
        REQUIRE(engine->loadRemoteMD(nixlBlobDesc(t_region, t_public), VRAM_SEG, peer, t_at_initiator) == NIXL_SUCCESS);
        REQUIRE(t_at_initiator && t_at_initiator != t_md);

        nixl_meta_dlist_t l2(VRAM_SEG), r2(VRAM_SEG);
        nixlMetaDesc le(reinterpret_cast<uintptr_t>(src), total, 0), re(reinterpret_cast<uintptr_t>(tbuf), total, 0);
        le.metadataP = src_md;
        re.metadataP = t_at_initiator;
        l2.addDesc(le);
        r2.addDesc(re);
        fillIncreasing(host, 33);
        REQUIRE(hipMemcpy(src, host.data(), total, hipMemcpyHostToDevice) == hipSuccess);
        nixl_opt_b_args_t with_notif;
        with_notif.notifMsg = "block landed";
        with_notif.hasNotif = true;
        nixlBackendReqH *w2 = nullptr;
        REQUIRE(engine->prepXfer(NIXL_WRITE, l2, r2, peer, w2, &with_notif) == NIXL_SUCCESS && w2);
        nixl_status_t st = engine->postXfer(NIXL_WRITE, l2, r2, peer, w2, &with_notif);
        REQUIRE(st == NIXL_IN_PROG || st == NIXL_SUCCESS);
        while (st == NIXL_IN_PROG)
            st = engine->checkXfer(w2);
        REQUIRE(st == NIXL_SUCCESS);
        notif_list_t seen;
        REQUIRE(target->getNotifs(seen) == NIXL_SUCCESS);
        REQUIRE(seen.size() == 1 && seen[0].first == agent && seen[0].second == "block landed");
        REQUIRE(hipMemcpy(back.data(), tbuf, total, hipMemcpyDeviceToHost) == hipSuccess);
        REQUIRE(checkIncreasing(back, 33));
        seen.clear();
        REQUIRE(engine->getNotifs(seen) == NIXL_SUCCESS && seen.empty()); // none for the initiator

        // READ from the peer, no notification
        REQUIRE(hipMemset(src, 0, total) == hipSuccess);
        REQUIRE(hipDeviceSynchronize() == hipSuccess);
        nixlBackendReqH *r2h = nullptr;
        REQUIRE(engine->prepXfer(NIXL_READ, l2, r2, peer, r2h) == NIXL_SUCCESS);
        REQUIRE(runToCompletion(engine, NIXL_READ, l2, r2, peer, r2h) == NIXL_SUCCESS);
        REQUIRE(hipMemcpy(back.data(), src, total, hipMemcpyDeviceToHost) == hipSuccess);
        REQUIRE(checkIncreasing(back, 33));
        REQUIRE(target->getNotifs(seen) == NIXL_SUCCESS && seen.empty());

        // stand-alone messages, both ways and to oneself
        REQUIRE(engine->genNotif(peer, "ping") == NIXL_SUCCESS && target->genNotif(agent, "pong") == NIXL_SUCCESS);
        REQUIRE(engine->genNotif(agent, "self") == NIXL_SUCCESS);
        REQUIRE(engine->genNotif("nobody", "lost") == NIXL_ERR_NOT_FOUND);
        REQUIRE(target->getNotifs(seen) == NIXL_SUCCESS && seen.size() == 1 && seen[0].second == "ping");
        seen.clear();
        REQUIRE(engine->getNotifs(seen) == NIXL_SUCCESS && seen.size() == 2);

        REQUIRE(engine->releaseReqH(w2) == NIXL_SUCCESS && engine->releaseReqH(r2h) == NIXL_SUCCESS);
        REQUIRE(engine->unloadMD(t_at_initiator) == NIXL_SUCCESS); // frees the initiator's copy
        REQUIRE(engine->disconnect(peer) == NIXL_SUCCESS);
        REQUIRE(engine->prepXfer(NIXL_WRITE, l2, r2, peer, bad) < 0 && bad == nullptr); // no longer a peer
        REQUIRE(target->deregisterMem(t_md) == NIXL_SUCCESS);
        plugin->destroy_engine(target);
        REQUIRE(engine->genNotif(peer, "too late") == NIXL_ERR_NOT_FOUND); // its queue went with it
        REQUIRE(hipFree(tbuf) == hipSuccess);
    }

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
