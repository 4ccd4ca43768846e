// Two agents of one process through the C++ north-bound API, on the CPU: metadata by hand,
// WRITE with a notification, READ, prepared lists, partial metadata, invalidation and the
// refusals around them.  The flow is the reference's two-agent example
// (examples/cpp/nixl_example.cpp: createBackend on both, registerMem, getLocalMD /
// loadRemoteMD both ways, createXferReq with a notification, postXferReq / getXferStatus,
// getNotifs on the target, invalidateRemoteMD) with the memcpy test backend standing in for
// a network backend.  The agent sources are compiled into this program, so that it can also
// be built with the host sanitizers.
//
// usage: agent_two_peers_check <directory holding libplugin_MEMCPY.so>; prints "OK".
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <string>
#include <vector>

#include "nixl.h"

#define REQUIRE(cond)                                                              \
    do {                                                                           \
        if (!(cond)) {                                                             \
            std::fprintf(stderr, "%s:%d: %s failed\n", __FILE__, __LINE__, #cond); \
            std::exit(1);                                                          \
        }                                                                          \
    } while (0)

namespace {

nixl_status_t
runToCompletion(nixlAgent &agent, nixlXferReqH *req, const nixl_opt_args_t *extra = nullptr) {
    nixl_status_t st = agent.postXferReq(req, extra);
    while (st == NIXL_IN_PROG)
        st = agent.getXferStatus(req);
    return st;
}

nixl_reg_dlist_t
regList(const std::vector<uint8_t> &buf) {
    nixl_reg_dlist_t l(DRAM_SEG);
    l.addDesc(nixlBlobDesc(reinterpret_cast<uintptr_t>(buf.data()), buf.size(), 0, ""));
    return l;
}

nixl_xfer_dlist_t
spans(const std::vector<uint8_t> &buf, const std::vector<std::pair<size_t, size_t>> &pieces) {
    nixl_xfer_dlist_t l(DRAM_SEG);
    for (const auto &[off, len] : pieces)
        l.addDesc(nixlBasicDesc(reinterpret_cast<uintptr_t>(buf.data()) + off, len, 0));
    return l;
}

} // namespace

int
main(int argc, char **argv) {
    if (argc != 2) {
        std::fprintf(stderr, "usage: %s <plugin dir>\n", argv[0]);
        return 2;
    }
    setenv("NIXL_PLUGIN_DIR", argv[1], 1);

    for (int round = 0; round < 3; ++round) { // agents come and go; nothing may be left behind
        nixlAgent a("A", nixlAgentConfig(false)), b("B", nixlAgentConfig(false));
        nixl_b_params_t params{{"peer_agents", "1"}};
        nixlBackendH *ba = nullptr, *bb = nullptr;
        REQUIRE(a.createBackend("MEMCPY", params, ba) == NIXL_SUCCESS);
        REQUIRE(b.createBackend("MEMCPY", params, bb) == NIXL_SUCCESS);

        if (round == 2) {
            // metadata of agents that have registered nothing yet loads, and is dropped again
            // (test/gtest/unit/agent/agent.cpp:353-380)
            nixl_blob_t bare;
            std::string who;
            REQUIRE(b.getLocalMD(bare) == NIXL_SUCCESS && !bare.empty());
            REQUIRE(a.loadRemoteMD(bare, who) == NIXL_SUCCESS && who == "B");
            REQUIRE(a.genNotif("B", "early bird") == NIXL_SUCCESS); // agent.cpp:517-542
            nixl_notifs_t early;
            REQUIRE(b.getNotifs(early) == NIXL_SUCCESS && early["A"] == std::vector<nixl_blob_t>{"early bird"});
            REQUIRE(a.invalidateRemoteMD("B") == NIXL_SUCCESS);
        }

        std::vector<uint8_t> src(1 << 16), dst(1 << 16, 0), extra(4096, 0);
        std::iota(src.begin(), src.end(), static_cast<uint8_t>(round));
        REQUIRE(a.registerMem(regList(src)) == NIXL_SUCCESS);
        REQUIRE(b.registerMem(regList(dst)) == NIXL_SUCCESS);

        // nothing is known of B yet
        nixlXferReqH *req = nullptr;
        REQUIRE(a.createXferReq(NIXL_WRITE, spans(src, {{0, 64}}), spans(dst, {{0, 64}}), "B", req) == NIXL_ERR_NOT_FOUND);
        REQUIRE(a.checkRemoteMD("B", nixl_xfer_dlist_t(DRAM_SEG)) == NIXL_ERR_NOT_FOUND);
        REQUIRE(a.genNotif("B", "too early") == NIXL_ERR_NOT_FOUND);

        nixl_blob_t md_a, md_b;
        std::string name;
        REQUIRE(a.getLocalMD(md_a) == NIXL_SUCCESS && b.getLocalMD(md_b) == NIXL_SUCCESS);
        REQUIRE(a.loadRemoteMD(md_a, name) == NIXL_ERR_INVALID_PARAM); // its own
        REQUIRE(a.loadRemoteMD(md_b.substr(0, md_b.size() / 2), name) != NIXL_SUCCESS);
        REQUIRE(a.checkRemoteMD("B", nixl_xfer_dlist_t(DRAM_SEG)) == NIXL_ERR_NOT_FOUND);
        REQUIRE(a.loadRemoteMD(md_b, name) == NIXL_SUCCESS && name == "B");
        REQUIRE(b.loadRemoteMD(md_a, name) == NIXL_SUCCESS && name == "A");
        REQUIRE(a.loadRemoteMD(md_b, name) == NIXL_SUCCESS); // again: unchanged, accepted
        REQUIRE(a.makeConnection("B") == NIXL_SUCCESS);
        REQUIRE(a.checkRemoteMD("B", spans(dst, {{100, 200}})) == NIXL_SUCCESS);
        REQUIRE(a.checkRemoteMD("B", spans(src, {{100, 200}})) == NIXL_ERR_NOT_FOUND);

        // WRITE with a notification
        nixl_opt_args_t with_notif;
        with_notif.notifMsg = "written";
        with_notif.hasNotif = true;
        const std::vector<std::pair<size_t, size_t>> from = {{0, 1000}, {4096, 4096}, {60000, 5536}};
        const std::vector<std::pair<size_t, size_t>> to = {{6000, 1000}, {20000, 4096}, {0, 5536}};
        REQUIRE(a.createXferReq(NIXL_WRITE, spans(src, from), spans(dst, to), "B", req, &with_notif) == NIXL_SUCCESS);
        nixlBackendH *used = nullptr;
        REQUIRE(a.queryXferBackend(req, used) == NIXL_SUCCESS && used == ba); // agent.cpp:544-584
        nixl_notifs_t notifs;
        REQUIRE(b.getNotifs(notifs) == NIXL_SUCCESS && notifs.empty());
        REQUIRE(runToCompletion(a, req) == NIXL_SUCCESS);
        for (size_t i = 0; i < from.size(); ++i)
            REQUIRE(std::memcmp(dst.data() + to[i].first, src.data() + from[i].first, from[i].second) == 0);
        REQUIRE(b.getNotifs(notifs) == NIXL_SUCCESS);
        REQUIRE(notifs.size() == 1 && notifs["A"] == std::vector<nixl_blob_t>{"written"});
        // a repost repeats the message; one passed to the post replaces it
        nixl_opt_args_t other;
        other.notif = std::string("bin\0ary", 7); // the optional form, as agent.cpp:413 sets it
        REQUIRE(runToCompletion(a, req) == NIXL_SUCCESS);
        REQUIRE(runToCompletion(a, req, &other) == NIXL_SUCCESS);
        REQUIRE(b.getNotifs(notifs) == NIXL_SUCCESS);
        REQUIRE((notifs["A"] == std::vector<nixl_blob_t>{"written", "written", std::string("bin\0ary", 7)}));
        REQUIRE(a.releaseXferReq(req) == NIXL_SUCCESS);

        // READ
        std::fill(src.begin(), src.begin() + 4096, 0);
        REQUIRE(a.createXferReq(NIXL_READ, spans(src, {{0, 4096}}), spans(dst, {{20000, 4096}}), "B", req) == NIXL_SUCCESS);
        REQUIRE(runToCompletion(a, req) == NIXL_SUCCESS);
        REQUIRE(std::memcmp(src.data(), dst.data() + 20000, 4096) == 0);
        REQUIRE(a.releaseXferReq(req) == NIXL_SUCCESS);

        // prepared lists on both sides
        nixlDlistH *local = nullptr, *remote = nullptr;
        REQUIRE(a.prepXferDlist(spans(src, {{0, 512}, {512, 512}, {1024, 512}, {1536, 512}}), local) == NIXL_SUCCESS);
        REQUIRE(a.prepXferDlist("B", spans(dst, {{30000, 512}, {30512, 512}, {31024, 512}, {31536, 512}}), remote) == NIXL_SUCCESS);
        REQUIRE(a.makeXferReq(NIXL_WRITE, local, {3, 2, 1, 0}, remote, {0, 1, 2, 3}, req) == NIXL_SUCCESS);
        REQUIRE(runToCompletion(a, req) == NIXL_SUCCESS);
        for (int i = 0; i < 4; ++i)
            REQUIRE(std::memcmp(dst.data() + 30000 + 512 * i, src.data() + 512 * (3 - i), 512) == 0);
        REQUIRE(a.releaseXferReq(req) == NIXL_SUCCESS);
        REQUIRE(a.releasedDlistH(local) == NIXL_SUCCESS && a.releasedDlistH(remote) == NIXL_SUCCESS);

        // partial metadata: a region registered later is unknown to A until it is published
        REQUIRE(b.registerMem(regList(extra)) == NIXL_SUCCESS);
        REQUIRE(a.createXferReq(NIXL_WRITE, spans(src, {{0, 4096}}), spans(extra, {{0, 4096}}), "B", req) == NIXL_ERR_NOT_FOUND);
        nixl_blob_t part;
        REQUIRE(b.getLocalPartialMD(regList(extra), part) == NIXL_SUCCESS);
        REQUIRE(a.loadRemoteMD(part, name) == NIXL_SUCCESS && name == "B");
        REQUIRE(a.createXferReq(NIXL_WRITE, spans(src, {{0, 4096}}), spans(extra, {{0, 4096}}), "B", req) == NIXL_SUCCESS);
        REQUIRE(runToCompletion(a, req) == NIXL_SUCCESS);
        REQUIRE(std::memcmp(extra.data(), src.data(), 4096) == 0);

        // standalone messages, also to oneself
        REQUIRE(a.genNotif("B", "hello") == NIXL_SUCCESS && a.genNotif("A", "self") == NIXL_SUCCESS);
        notifs.clear();
        REQUIRE(b.getNotifs(notifs) == NIXL_SUCCESS && notifs["A"] == std::vector<nixl_blob_t>{"hello"});
        notifs.clear();
        REQUIRE(a.getNotifs(notifs) == NIXL_SUCCESS && notifs["A"] == std::vector<nixl_blob_t>{"self"});

        // invalidation: the live request can no longer be posted, the peer is gone
        REQUIRE(a.invalidateRemoteMD("A") == NIXL_ERR_INVALID_PARAM);
        REQUIRE(a.invalidateRemoteMD("B") == NIXL_SUCCESS);
        REQUIRE(a.invalidateRemoteMD("B") == NIXL_ERR_NOT_FOUND);
        REQUIRE(a.postXferReq(req) == NIXL_ERR_NOT_FOUND);
        REQUIRE(a.releaseXferReq(req) == NIXL_SUCCESS);
        REQUIRE(a.makeConnection("B") == NIXL_ERR_NOT_FOUND);
        REQUIRE(a.genNotif("B", "gone") == NIXL_ERR_NOT_FOUND);
        // registering and deregistering a pool of regions over and over neither fails nor slows
        // down (agent.cpp:273-336: 128 regions, 64 cycles between two timed ones, ratio <= 2;
        // the bound here is looser because the test machine is shared)
        if (round == 0) {
            constexpr size_t kPool = 128;
            std::vector<std::vector<uint8_t>> pool(kPool, std::vector<uint8_t>(256));
            auto cycle = [&](int times) {
                for (int r = 0; r < times; ++r) {
                    for (auto &p : pool)
                        REQUIRE(a.registerMem(regList(p)) == NIXL_SUCCESS);
                    for (auto &p : pool)
                        REQUIRE(a.deregisterMem(regList(p)) == NIXL_SUCCESS);
                }
            };
            auto timed = [&]() {
                const auto t0 = std::chrono::steady_clock::now();
                cycle(1);
                return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
            };
            cycle(3);
            double first = timed();
            for (int i = 0; i < 4; ++i)
                first = std::min(first, timed());
            cycle(64);
            double second = timed();
            for (int i = 0; i < 4; ++i)
                second = std::min(second, timed());
            REQUIRE(second <= 5.0 * first && first <= 5.0 * second);
            nixl_blob_t after;
            REQUIRE(a.getLocalMD(after) == NIXL_SUCCESS);
            REQUIRE(a.deregisterMem(regList(pool[0])) == NIXL_ERR_NOT_FOUND); // nothing of the pool is left
        }
        // B still knows A and leaves it to its destructor to unload A's regions
        if (round == 1) REQUIRE(b.deregisterMem(regList(extra)) == NIXL_SUCCESS);
    }
    std::printf("OK\n");
    return 0;
}
