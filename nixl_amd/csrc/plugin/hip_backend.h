// nixlHipEngine: a NIXL backend for VRAM<->VRAM descriptor transfers on one AMD GPU, between
// the regions of one agent (loopback), of several agents that live in the same process, or of
// agents in other processes on the same GPU (their memory is mapped through HIP IPC handles,
// their notifications travel through a shared-memory mailbox).  It fills the same slot as the
// reference's local backends (shape of
// src/plugins/posix/posix_backend.h:78-158; request life-cycle split of
// src/plugins/cuda_gds/gds_backend.cpp:159-391): prepXfer lowers the two descriptor
// lists once into a device-resident copy plan, postXfer enqueues one kernel launch and
// records an event, checkXfer polls the event, releaseReqH frees (or defers freeing if
// the kernel is still running).
#ifndef NIXL_AMD_HIP_BACKEND_H
#define NIXL_AMD_HIP_BACKEND_H

#include <hip/hip_runtime_api.h>

#include <atomic>
#include <condition_variable>
#include <memory>
#include <mutex>
#include <thread>
#include <string>
#include <unordered_map>
#include <vector>

#include "backend/backend_engine.h"
#include "nixl_amd_hip.h"
#include "mailbox.h"
#include "worker_pool.h"

// Registration record returned by registerMem and handed back in nixlMetaDesc::metadataP.
// `addr` is the region's address in its OWNER's address space, which is the space the
// descriptors of that agent are written in; `delta` takes such an address to where the region
// is mapped in this process (0 for this process's own memory, the offset of the opened IPC
// mapping for a region of another process).
class nixlHipMD : public nixlBackendMD {
public:
    nixlHipMD(uintptr_t addr_, size_t len_, int device_, nixl_mem_t mem_, bool of_peer = false, intptr_t delta_ = 0)
        : nixlBackendMD(!of_peer),
          addr(addr_),
          len(len_),
          device(device_),
          mem(mem_),
          ofPeer(of_peer),
          delta(delta_) {}

    const uintptr_t addr;
    const size_t len;
    const int device; // HIP device whose kernels may touch the region
    const nixl_mem_t mem;
    const bool ofPeer; // made by loadRemoteMD from a peer's published data; unloadMD frees it
    const intptr_t delta;
    // What another process needs to map the allocation the region lies in (own VRAM regions
    // whose allocation is small enough to be shared).
    bool hasIpc = false;
    hipIpcMemHandle_t ipc{};
    uintptr_t allocBase = 0;
    size_t allocSize = 0;
    // For a region of another process: the key of the opened mapping, released by unloadMD.
    std::string ipcKey;

    bool
    contains(uintptr_t a, size_t l) const noexcept {
        return a >= addr && l <= len && (a - addr) <= (len - l);
    }

    // Address in this process of the owner's address `a`.
    uintptr_t
    here(uintptr_t a) const noexcept {
        return static_cast<uintptr_t>(static_cast<intptr_t>(a) + delta);
    }
};

class nixlHipReqH : public nixlBackendReqH {
public:
    nixl_amd_copy_plan_t *plan = nullptr;
    hipStream_t stream = nullptr;
    int device = 0;
    bool posted = false;
    size_t bytes = 0;
    // A notification that is due once the posted transfer has finished.  Guarded by the
    // engine's pendingMutex_, because the progress thread looks at it too.
    bool notifPending = false;
    std::string notifTarget;
    std::string notifMsg;

    ~nixlHipReqH() override;
    nixl_status_t
    state(bool wait) const;
};

class nixlHipEngine : public nixlBackendEngine {
public:
    explicit nixlHipEngine(const nixlBackendInitParams *init_params);
    ~nixlHipEngine() override;

    // "Remote" means another agent on the same GPU: of this process (its regions are plain
    // addresses here) or of another one (its allocations are opened through IPC handles).
    bool
    supportsRemote() const override {
        return true;
    }

    bool
    supportsLocal() const override {
        return true;
    }

    bool
    supportsNotif() const override {
        return true;
    }

    nixl_mem_list_t
    getSupportedMems() const override {
        return {VRAM_SEG, DRAM_SEG};
    }

    nixl_status_t
    registerMem(const nixlBlobDesc &mem, const nixl_mem_t &nixl_mem, nixlBackendMD *&out) override;
    nixl_status_t
    deregisterMem(nixlBackendMD *meta) override;

    nixl_status_t
    connect(const std::string &remote_agent) override;
    nixl_status_t
    disconnect(const std::string &remote_agent) override;
    nixl_status_t
    unloadMD(nixlBackendMD *input) override;

    nixl_status_t
    getPublicData(const nixlBackendMD *meta, std::string &str) const override;
    nixl_status_t
    getConnInfo(std::string &str) const override;
    nixl_status_t
    loadRemoteConnInfo(const std::string &remote_agent, const std::string &remote_conn_info) override;
    nixl_status_t
    loadRemoteMD(const nixlBlobDesc &input,
                 const nixl_mem_t &nixl_mem,
                 const std::string &remote_agent,
                 nixlBackendMD *&output) override;

    nixl_status_t
    getNotifs(notif_list_t &notif_list) override;
    nixl_status_t
    genNotif(const std::string &remote_agent, const std::string &msg) const override;

    nixl_status_t
    loadLocalMD(nixlBackendMD *input, nixlBackendMD *&output) override {
        output = input;
        return NIXL_SUCCESS;
    }

    nixl_status_t
    prepXfer(const nixl_xfer_op_t &operation,
             const nixl_meta_dlist_t &local,
             const nixl_meta_dlist_t &remote,
             const std::string &remote_agent,
             nixlBackendReqH *&handle,
             const nixl_opt_b_args_t *opt_args = nullptr) const override;
    nixl_status_t
    postXfer(const nixl_xfer_op_t &operation,
             const nixl_meta_dlist_t &local,
             const nixl_meta_dlist_t &remote,
             const std::string &remote_agent,
             nixlBackendReqH *&handle,
             const nixl_opt_b_args_t *opt_args = nullptr) const override;
    nixl_status_t
    checkXfer(nixlBackendReqH *handle) const override;
    nixl_status_t
    releaseReqH(nixlBackendReqH *handle) const override;

    // prepXfer for a request given as two index vectors into two prepared lists, each list
    // given as its stride runs (address, block length, stride, block count, first index; at
    // most 256 runs a list, one block length throughout): the descriptors are never written
    // out on the host; the records of the copy plan are built on the device from the index
    // vectors and the run tables.  No reference counterpart: the reference's agent
    // expands the indices on the host (src/core/nixl_agent.cpp:799-857) before any backend sees
    // them.  NIXL_ERR_NOT_SUPPORTED means "take the ordinary path" (alignment, direction or
    // shape outside what the device lowering handles).  Reached through the C symbol
    // nixl_hip_prep_xfer_indexed, which an agent looks up in the plugin library.
    nixl_status_t
    prepXferIndexed(const nixl_xfer_op_t &operation,
                    const nixlStrideDesc *local_runs,
                    size_t n_local_runs,
                    const int *local_indices,
                    const nixlStrideDesc *remote_runs,
                    size_t n_remote_runs,
                    const int *remote_indices,
                    size_t count,
                    const std::string &remote_agent,
                    nixlBackendReqH *&handle) const;

    // Memory views for kernels that move data themselves: the handle is a device pointer
    // to a table of {address, length} entries (layout in nixl_amd_device.h), checked here
    // against the registrations (shape of src/plugins/ucx/ucx_backend.cpp prepMemView).
    nixl_status_t
    prepMemView(const nixl_remote_meta_dlist_t &descs,
                nixlMemViewH &mvh,
                const nixl_opt_b_args_t *opt_args = nullptr) const override;
    nixl_status_t
    prepMemView(const nixl_meta_dlist_t &descs,
                nixlMemViewH &mvh,
                const nixl_opt_b_args_t *opt_args = nullptr) const override;
    void
    releaseMemView(nixlMemViewH mvh) const override;

    // Per descriptor: what the HIP runtime knows of the address range, or no value if it
    // does not know it (the reference's storage backends answer "does it exist" the same way,
    // src/plugins/posix/posix_backend.cpp queryMem).
    nixl_status_t
    queryMem(const nixl_reg_dlist_t &descs, std::vector<nixl_query_resp_t> &resp) const override;

    nixl_status_t
    estimateXferCost(const nixl_xfer_op_t &operation,
                     const nixl_meta_dlist_t &local,
                     const nixl_meta_dlist_t &remote,
                     const std::string &remote_agent,
                     nixlBackendReqH *const &handle,
                     std::chrono::microseconds &duration,
                     std::chrono::microseconds &err_margin,
                     nixl_cost_t &method,
                     const nixl_opt_args_t *extra_params = nullptr) const override;

private:
    // The two passes of prepXfer over a request's descriptor lists (hip_backend.cpp).
    struct blockPass {
        nixl_status_t status;
        bool blocks; // every pair a whole number of equal blocks and the records fit
    };
    struct blockSlice;
    blockPass
    lowerBlocks(bool write,
                const nixl_meta_dlist_t &local,
                const nixl_meta_dlist_t &remote,
                nixl_amd_copy_record_t *records,
                size_t room,
                size_t &n_records,
                int &device,
                size_t &bytes,
                nixl_amd_copy_record_facts_t &facts) const;
    void
    lowerBlockSlice(bool write,
                    const nixlMetaDesc *L,
                    const nixlMetaDesc *R,
                    size_t begin,
                    size_t end,
                    size_t len0,
                    nixl_amd_copy_record_t *records,
                    blockSlice &out) const;
    using WorkerPool = nixl_amd_hip::WorkerPool;
    WorkerPool *
    prepPool() const; // made on first use
    nixl_status_t
    lowerGeneral(bool write,
                 const nixl_meta_dlist_t &local,
                 const nixl_meta_dlist_t &remote,
                 nixl_amd_copy_desc_t *lowered,
                 int &device,
                 size_t &bytes) const;
    hipStream_t
    pickStream(int device) const;
    void
    reapRetired(bool wait) const;
    bool
    knowsAgent(const std::string &name) const;
    void
    deliverPending(nixlHipReqH *req, bool completed) const;
    void
    progressLoop();
    struct viewEntry {
        uintptr_t addr;
        size_t len;
        const nixlHipMD *md; // null for a placeholder entry
    };
    nixl_status_t
    buildMemView(const std::vector<viewEntry> &entries, uint32_t kind, nixlMemViewH &mvh) const;

    int numDevices_ = 0;
    int streamsPerDevice_ = 1;
    // prep_threads: threads that share the pass over a long request's descriptor lists (the
    // caller included; 1 = the caller alone).
    int prepThreads_ = 1;
    mutable std::once_flag prepPoolOnce_;
    mutable std::unique_ptr<WorkerPool> prepPool_;
    bool indexedPrep_ = true; // backend parameter indexed_prep: 0 makes prepXferIndexed decline every request
    bool useExternalStream_ = false; // launches go to the application's stream (may be the null stream)
    hipStream_t externalStream_ = nullptr;
    nixl_amd_copy_tuning_t tuning_{};
    // streams_[device * streamsPerDevice_ + i]; created lazily under streamsMutex_.
    mutable std::vector<hipStream_t> streams_;
    mutable std::mutex streamsMutex_;
    mutable std::atomic<unsigned> nextStream_{0};
    // Requests released while their kernel was still running; freed once it has finished.
    mutable std::vector<nixlHipReqH *> retired_;
    mutable std::mutex retiredMutex_;
    // Notifications of posted transfers.  With a progress thread (enableProgTh of the init
    // parameters, the agent's useProgThread) the requests that carry one are watched and the
    // message is queued at the target as soon as the copy has finished; without it, when the
    // initiator next looks at the request.
    mutable std::mutex pendingMutex_;
    mutable std::condition_variable pendingCv_;
    mutable std::vector<nixlHipReqH *> watched_;
    bool stopProgress_ = false;
    bool progressOn_ = false;
    uint64_t progressDelayUs_ = 0;
    std::thread progress_;
    // Peers whose connection info was loaded: agents of this process (no mailbox: their
    // engine is found in the process-wide registry) or of another one.
    using Mailbox = nixl_amd_hip::Mailbox; // shared-memory ring of notifications
    struct peerInfo {
        long long pid = 0;
        std::string mailboxName;
        Mailbox *mailbox = nullptr; // null for an agent of this process
        nixl_amd_hip::MailboxSender sender; // messages that found the peer's ring full wait here
    };
    // Set while some peer's sender holds waiting messages: the calls that an initiator makes
    // anyway (checkXfer, getNotifs, genNotif, the progress thread) then try to move them on.
    mutable std::atomic<bool> backlog_{false};
    void
    flushBacklog() const;
    mutable std::mutex peersMutex_;
    mutable std::unordered_map<std::string, peerInfo> peers_;
    // This engine's own mailbox, where agents of other processes leave notifications.
    std::string mailboxName_;
    Mailbox *mailbox_ = nullptr;
    // Allocations of other processes opened here: "<pid>:<allocation base>" -> mapping.
    struct ipcMapping {
        void *base = nullptr;
        int device = 0;
        int refs = 0;
    };
    mutable std::mutex ipcMutex_;
    mutable std::unordered_map<std::string, ipcMapping> ipcMaps_;
    static Mailbox *
    mapMailbox(const std::string &name, bool create);
    static void
    unmapMailbox(Mailbox *m);
    // Notifications other agents (or this one) left for this agent.
    mutable std::mutex notifMutex_;
    mutable notif_list_t notifs_;
    // Live memory-view tables: device pointer -> owning device.
    mutable std::unordered_map<void *, int> memViews_;
    mutable std::mutex memViewsMutex_;
};

#endif
