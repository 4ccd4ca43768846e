// Several threads on one pair of agents, on the CPU: four threads create, post, poll and
// release their own transfer requests with notifications and make and release memory views,
// while one thread registers and deregisters memory and reads the metadata and another drains
// the target's notifications (the reference drives one request per thread the same way,
// benchmark/nixlbench/src/worker/nixl/nixl_worker.cpp:1847-1879).  Every notification must
// arrive exactly once.  The agent sources are compiled in, so that the program can also be
// built with -fsanitize=thread (make SANITIZE=...).
//
// usage: agent_threads_check <directory holding libplugin_MEMCPY.so>; prints "OK".
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>
#include "nixl.h"
#define REQUIRE(c) do { if (!(c)) { std::fprintf(stderr, "%s:%d: %s failed\n", __FILE__, __LINE__, #c); std::exit(1);} } while (0)
int main(int argc, char **argv) {
    setenv("NIXL_PLUGIN_DIR", argv[1], 1);
    nixlAgent a("A", nixlAgentConfig(false)), b("B", nixlAgentConfig(false));
    nixl_b_params_t params{{"peer_agents", "1"}};
    nixlBackendH *ba, *bb;
    REQUIRE(a.createBackend("MEMCPY", params, ba) == NIXL_SUCCESS);
    REQUIRE(b.createBackend("MEMCPY", params, bb) == NIXL_SUCCESS);
    const int T = 4;
    std::vector<std::vector<uint8_t>> src(T, std::vector<uint8_t>(1 << 16, 7)), dst(T, std::vector<uint8_t>(1 << 16, 0));
    for (int t = 0; t < T; ++t) {
        nixl_reg_dlist_t ra(DRAM_SEG), rb(DRAM_SEG);
        ra.addDesc(nixlBlobDesc((uintptr_t)src[t].data(), src[t].size(), 0, ""));
        rb.addDesc(nixlBlobDesc((uintptr_t)dst[t].data(), dst[t].size(), 0, ""));
        REQUIRE(a.registerMem(ra) == NIXL_SUCCESS && b.registerMem(rb) == NIXL_SUCCESS);
    }
    nixl_blob_t md; std::string name;
    REQUIRE(b.getLocalMD(md) == NIXL_SUCCESS && a.loadRemoteMD(md, name) == NIXL_SUCCESS);
    std::atomic<bool> stop{false};
    std::atomic<int> got{0};
    std::thread poller([&] {
        while (!stop) { nixl_notifs_t n; b.getNotifs(n); for (auto &kv : n) got += kv.second.size(); }
        nixl_notifs_t n; b.getNotifs(n); for (auto &kv : n) got += kv.second.size();
    });
    std::thread registrar([&] {   // registration traffic while transfers run
        std::vector<uint8_t> tmp(4096);
        for (int i = 0; i < 200; ++i) {
            nixl_reg_dlist_t r(DRAM_SEG); r.addDesc(nixlBlobDesc((uintptr_t)tmp.data(), tmp.size(), 0, ""));
            REQUIRE(a.registerMem(r) == NIXL_SUCCESS); REQUIRE(a.deregisterMem(r) == NIXL_SUCCESS);
            nixl_blob_t m; a.getLocalMD(m);
        }
    });
    std::vector<std::thread> workers;
    const int rounds = 200;
    for (int t = 0; t < T; ++t)
        workers.emplace_back([&, t] {
            for (int i = 0; i < rounds; ++i) {
                nixl_xfer_dlist_t l(DRAM_SEG), r(DRAM_SEG);
                l.addDesc(nixlBasicDesc((uintptr_t)src[t].data() + 64 * (i % 100), 4096, 0));
                r.addDesc(nixlBasicDesc((uintptr_t)dst[t].data() + 64 * (i % 100), 4096, 0));
                nixl_opt_args_t o; o.notifMsg = "n"; o.hasNotif = true;
                nixlXferReqH *req = nullptr;
                REQUIRE(a.createXferReq(NIXL_WRITE, l, r, "B", req, &o) == NIXL_SUCCESS);
                nixl_status_t st = a.postXferReq(req);
                while (st == NIXL_IN_PROG) st = a.getXferStatus(req);
                REQUIRE(st == NIXL_SUCCESS);
                REQUIRE(a.releaseXferReq(req) == NIXL_SUCCESS);
                nixlMemViewH v = nullptr;
                nixl_local_dlist_t ll(DRAM_SEG); ll.addDesc(nixlBasicDesc((uintptr_t)src[t].data(), 64, 0));
                REQUIRE(a.prepMemView(ll, v) == NIXL_SUCCESS); a.releaseMemView(v);
            }
        });
    for (auto &w : workers) w.join();
    registrar.join();
    stop = true; poller.join();
    REQUIRE(got == T * rounds);
    std::puts("OK");
}
