// TEST INFRASTRUCTURE — CPU oracle for the descriptor-transfer half, packaged as a NIXL
// backend plugin ("MEMCPY", DRAM_SEG only) so that it is driven through exactly the same
// agent calls as the HIP backend.  Only tests and the CPU-baseline leg of the benchmark
// load it; no product library links or falls back to it.
//
// Semantics restated from the reference's loopback path: for every descriptor pair, in
// list order, one put (NIXL_WRITE: local -> remote) or one get (NIXL_READ: remote ->
// local) of len bytes (src/plugins/ucx/ucx_backend.cpp:1216-1244, direction at
// :1227-1229), all complete before the request reports success (:1246-1262).  On one
// host that is memcpy(dst, src, len) per descriptor.  Pinned by: byte compare after
// WRITE and READ (test/unit/plugins/ucx/ucx_backend_test.cpp:383-389), repost re-reads
// current bytes (test/unit/plugins/posix/nixl_posix_test.cpp:714-770), and a canary
// check that bytes outside every destination range are untouched.
//
// Memory views (prepMemView) are tables in host memory, for tests of the agent's resolution.
//
// With the parameter peer_agents=1 the backend also reports supportsRemote() and
// supportsNotif(): "remote" agents are other agents of the same process, whose registrations
// are plain addresses here, and a notification is a push into the target engine's queue.
// That lets the agent's metadata exchange (getLocalMD / loadRemoteMD), remote descriptor
// lists and notification calls be tested on the CPU.  The message of a transfer is queued
// after the copy has finished (the reference sends it behind the data,
// src/plugins/ucx/ucx_backend.cpp:1246-1262).
#include <unistd.h>

#include <algorithm>
#include <cstring>
#include <mutex>
#include <thread>
#include <unordered_map>
#include <vector>

#include "backend/backend_engine.h"
#include "backend/backend_plugin.h"

namespace {

class memcpyMD : public nixlBackendMD {
public:
    memcpyMD(uintptr_t a, size_t l, bool of_peer = false) : nixlBackendMD(!of_peer), addr(a), len(l), ofPeer(of_peer) {}
    uintptr_t addr;
    size_t len;
    bool ofPeer; // made by loadRemoteMD; unloadMD frees it
};

class memcpyReqH : public nixlBackendReqH {};

class memcpyEngine;
std::mutex g_registryMutex;
std::unordered_map<std::string, const memcpyEngine *> g_registry;

class memcpyEngine : public nixlBackendEngine {
public:
    explicit memcpyEngine(const nixlBackendInitParams *p) : nixlBackendEngine(p) {
        const auto it = p->customParams->find("threads");
        threads_ = it == p->customParams->end() ? 1 : std::max(1, std::atoi(it->second.c_str()));
        const auto peers = p->customParams->find("peer_agents");
        peerAgents_ = peers != p->customParams->end() && std::atoi(peers->second.c_str()) != 0;
        std::lock_guard<std::mutex> lock(g_registryMutex);
        g_registry[localAgent] = this;
    }

    ~memcpyEngine() override {
        std::lock_guard<std::mutex> lock(g_registryMutex);
        const auto it = g_registry.find(localAgent);
        if (it != g_registry.end() && it->second == this) g_registry.erase(it);
    }

    bool supportsRemote() const override { return peerAgents_; }
    bool supportsLocal() const override { return true; }
    bool supportsNotif() const override { return peerAgents_; }
    nixl_mem_list_t getSupportedMems() const override { return {DRAM_SEG}; }

    nixl_status_t
    registerMem(const nixlBlobDesc &mem, const nixl_mem_t &nixl_mem, nixlBackendMD *&out) override {
        if (nixl_mem != DRAM_SEG) return NIXL_ERR_NOT_SUPPORTED;
        out = new memcpyMD(mem.addr, mem.len);
        return NIXL_SUCCESS;
    }
    nixl_status_t deregisterMem(nixlBackendMD *meta) override {
        delete meta;
        return NIXL_SUCCESS;
    }
    nixl_status_t connect(const std::string &a) override { return known(a) ? NIXL_SUCCESS : NIXL_ERR_NOT_FOUND; }
    nixl_status_t disconnect(const std::string &a) override {
        std::lock_guard<std::mutex> lock(mutex_);
        peers_.erase(std::remove(peers_.begin(), peers_.end(), a), peers_.end());
        return NIXL_SUCCESS;
    }
    nixl_status_t unloadMD(nixlBackendMD *md) override {
        if (md && static_cast<memcpyMD *>(md)->ofPeer) delete md;
        return NIXL_SUCCESS;
    }

    nixl_status_t getConnInfo(std::string &str) const override {
        str = "MEMCPY1:pid=" + std::to_string(static_cast<long long>(getpid()));
        return NIXL_SUCCESS;
    }
    nixl_status_t loadRemoteConnInfo(const std::string &agent, const std::string &info) override {
        std::string mine;
        getConnInfo(mine);
        if (info != mine) return NIXL_ERR_NOT_SUPPORTED; // another process
        std::lock_guard<std::mutex> lock(mutex_);
        if (std::find(peers_.begin(), peers_.end(), agent) == peers_.end()) peers_.push_back(agent);
        return NIXL_SUCCESS;
    }
    nixl_status_t getPublicData(const nixlBackendMD *meta, std::string &str) const override {
        const auto *md = static_cast<const memcpyMD *>(meta);
        const uint64_t words[2] = {md->addr, md->len};
        str.assign(reinterpret_cast<const char *>(words), sizeof(words));
        return NIXL_SUCCESS;
    }
    nixl_status_t loadRemoteMD(const nixlBlobDesc &in, const nixl_mem_t &mem, const std::string &agent,
                               nixlBackendMD *&out) override {
        uint64_t words[2];
        if (mem != DRAM_SEG || !known(agent) || in.metaInfo.size() != sizeof(words)) return NIXL_ERR_MISMATCH;
        std::memcpy(words, in.metaInfo.data(), sizeof(words));
        if (words[0] != in.addr || words[1] != in.len) return NIXL_ERR_MISMATCH;
        out = new memcpyMD(in.addr, in.len, /*of_peer=*/true);
        return NIXL_SUCCESS;
    }
    // Memory views in host memory, in the layout the HIP backend builds on the device
    // (include/nixl_amd_device.h: {magic, kind, count, (addr, len)...}), so that the agent's
    // resolution of local and remote view lists can be checked on the CPU.
    nixl_status_t prepMemView(const nixl_meta_dlist_t &descs, nixlMemViewH &mvh, const nixl_opt_b_args_t *) const override {
        std::vector<std::pair<uint64_t, uint64_t>> entries;
        for (const nixlMetaDesc &d : descs) {
            if (!d.metadataP) return NIXL_ERR_INVALID_PARAM;
            entries.emplace_back(d.addr, d.len);
        }
        return buildView(entries, 0, mvh);
    }
    nixl_status_t prepMemView(const nixl_remote_meta_dlist_t &descs, nixlMemViewH &mvh,
                              const nixl_opt_b_args_t *) const override {
        std::vector<std::pair<uint64_t, uint64_t>> entries;
        for (const nixlRemoteMetaDesc &d : descs)
            entries.emplace_back(d.metadataP ? d.addr : 0, d.metadataP ? d.len : 0); // placeholder: no registration
        return buildView(entries, 1, mvh);
    }
    void releaseMemView(nixlMemViewH mvh) const override { delete[] static_cast<uint64_t *>(mvh); }

    nixl_status_t genNotif(const std::string &agent, const std::string &msg) const override {
        std::lock_guard<std::mutex> registry(g_registryMutex);
        const auto it = g_registry.find(agent);
        if (it == g_registry.end()) return NIXL_ERR_NOT_FOUND;
        std::lock_guard<std::mutex> lock(it->second->mutex_);
        it->second->notifs_.emplace_back(localAgent, msg);
        return NIXL_SUCCESS;
    }
    nixl_status_t getNotifs(notif_list_t &out) override {
        std::lock_guard<std::mutex> lock(mutex_);
        for (auto &n : notifs_)
            out.push_back(std::move(n));
        notifs_.clear();
        return NIXL_SUCCESS;
    }
    nixl_status_t loadLocalMD(nixlBackendMD *in, nixlBackendMD *&out) override {
        out = in;
        return NIXL_SUCCESS;
    }

    nixl_status_t
    prepXfer(const nixl_xfer_op_t &, const nixl_meta_dlist_t &local, const nixl_meta_dlist_t &remote,
             const std::string &remote_agent, nixlBackendReqH *&handle, const nixl_opt_b_args_t *) const override {
        if (!known(remote_agent) || local.descCount() != remote.descCount()) return NIXL_ERR_INVALID_PARAM;
        for (int i = 0; i < local.descCount(); ++i)
            if (local[i].len != remote[i].len) return NIXL_ERR_INVALID_PARAM;
        handle = new memcpyReqH();
        return NIXL_SUCCESS;
    }

    nixl_status_t
    postXfer(const nixl_xfer_op_t &op, const nixl_meta_dlist_t &local, const nixl_meta_dlist_t &remote,
             const std::string &remote_agent, nixlBackendReqH *&, const nixl_opt_b_args_t *opt) const override {
        const int n = local.descCount();
        auto run = [&](int lo, int hi) {
            for (int i = lo; i < hi; ++i) {
                void *l = reinterpret_cast<void *>(local[i].addr);
                void *r = reinterpret_cast<void *>(remote[i].addr);
                if (op == NIXL_WRITE)
                    std::memcpy(r, l, local[i].len);
                else
                    std::memcpy(l, r, local[i].len);
            }
        };
        if (threads_ <= 1 || n < 2 * threads_) {
            run(0, n);
        } else {
            std::vector<std::thread> pool;
            for (int t = 0; t < threads_; ++t)
                pool.emplace_back(run, static_cast<int>(static_cast<long>(n) * t / threads_),
                                  static_cast<int>(static_cast<long>(n) * (t + 1) / threads_));
            for (auto &t : pool)
                t.join();
        }
        if (opt && opt->hasNotif) return genNotif(remote_agent, opt->notifMsg);
        return NIXL_SUCCESS;
    }

    nixl_status_t checkXfer(nixlBackendReqH *) const override { return NIXL_SUCCESS; }
    nixl_status_t releaseReqH(nixlBackendReqH *h) const override {
        delete h;
        return NIXL_SUCCESS;
    }

private:
    static nixl_status_t buildView(const std::vector<std::pair<uint64_t, uint64_t>> &entries, uint32_t kind,
                                   nixlMemViewH &mvh) {
        if (entries.empty()) return NIXL_ERR_INVALID_PARAM;
        auto *words = new uint64_t[2 + 2 * entries.size()];
        words[0] = 0x5649584cull | (static_cast<uint64_t>(kind) << 32);
        words[1] = entries.size();
        for (size_t i = 0; i < entries.size(); ++i) {
            words[2 + 2 * i] = entries[i].first;
            words[3 + 2 * i] = entries[i].second;
        }
        mvh = words;
        return NIXL_SUCCESS;
    }

    bool known(const std::string &agent) const {
        if (agent == localAgent) return true;
        std::lock_guard<std::mutex> lock(mutex_);
        return std::find(peers_.begin(), peers_.end(), agent) != peers_.end();
    }

    int threads_ = 1;
    bool peerAgents_ = false;
    mutable std::mutex mutex_;
    std::vector<std::string> peers_;
    mutable notif_list_t notifs_;
};

} // namespace

extern "C" NIXL_PLUGIN_EXPORT nixlBackendPlugin *
nixl_plugin_init() {
    return nixlBackendPluginCreator<memcpyEngine>::create(NIXL_PLUGIN_API_VERSION, "MEMCPY", "0.1.0",
                                                          {{"threads", "1"}, {"peer_agents", "0"}}, {DRAM_SEG});
}

extern "C" NIXL_PLUGIN_EXPORT void
nixl_plugin_fini() {}
