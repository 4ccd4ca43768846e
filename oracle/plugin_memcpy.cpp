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
#include <cstring>
#include <thread>
#include <vector>

#include "backend/backend_engine.h"
#include "backend/backend_plugin.h"

namespace {

class memcpyMD : public nixlBackendMD {
public:
    memcpyMD(uintptr_t a, size_t l) : nixlBackendMD(true), addr(a), len(l) {}
    uintptr_t addr;
    size_t len;
};

class memcpyReqH : public nixlBackendReqH {};

class memcpyEngine : public nixlBackendEngine {
public:
    explicit memcpyEngine(const nixlBackendInitParams *p) : nixlBackendEngine(p) {
        const auto it = p->customParams->find("threads");
        threads_ = it == p->customParams->end() ? 1 : std::max(1, std::atoi(it->second.c_str()));
    }

    bool supportsRemote() const override { return false; }
    bool supportsLocal() const override { return true; }
    bool supportsNotif() const override { return false; }
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
    nixl_status_t connect(const std::string &) override { return NIXL_SUCCESS; }
    nixl_status_t disconnect(const std::string &) override { return NIXL_SUCCESS; }
    nixl_status_t unloadMD(nixlBackendMD *) override { return NIXL_SUCCESS; }
    nixl_status_t loadLocalMD(nixlBackendMD *in, nixlBackendMD *&out) override {
        out = in;
        return NIXL_SUCCESS;
    }

    nixl_status_t
    prepXfer(const nixl_xfer_op_t &, const nixl_meta_dlist_t &local, const nixl_meta_dlist_t &remote,
             const std::string &remote_agent, nixlBackendReqH *&handle, const nixl_opt_b_args_t *) const override {
        if (remote_agent != localAgent || local.descCount() != remote.descCount()) return NIXL_ERR_INVALID_PARAM;
        for (int i = 0; i < local.descCount(); ++i)
            if (local[i].len != remote[i].len) return NIXL_ERR_INVALID_PARAM;
        handle = new memcpyReqH();
        return NIXL_SUCCESS;
    }

    nixl_status_t
    postXfer(const nixl_xfer_op_t &op, const nixl_meta_dlist_t &local, const nixl_meta_dlist_t &remote,
             const std::string &, nixlBackendReqH *&, const nixl_opt_b_args_t *) const override {
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
        return NIXL_SUCCESS;
    }

    nixl_status_t checkXfer(nixlBackendReqH *) const override { return NIXL_SUCCESS; }
    nixl_status_t releaseReqH(nixlBackendReqH *h) const override {
        delete h;
        return NIXL_SUCCESS;
    }

private:
    int threads_ = 1;
};

} // namespace

extern "C" NIXL_PLUGIN_EXPORT nixlBackendPlugin *
nixl_plugin_init() {
    return nixlBackendPluginCreator<memcpyEngine>::create(NIXL_PLUGIN_API_VERSION, "MEMCPY", "0.1.0",
                                                          {{"threads", "1"}}, {DRAM_SEG});
}

extern "C" NIXL_PLUGIN_EXPORT void
nixl_plugin_fini() {}
