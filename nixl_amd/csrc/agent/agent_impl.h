// Private state of the single-process agent: loaded plugins, registered-memory sections,
// prepared descriptor lists and transfer request handles.
//
// What is kept equal to the reference, because it decides which descriptors a backend
// receives:
//   * registered regions are kept sorted per (memory type, backend); a transfer descriptor
//     is resolved to the region that covers it by bisection for the first element and
//     after any decrease, by a forward walk otherwise
//     (src/infra/nixl_memory_section.cpp:56-104, src/infra/nixl_descriptors.cpp:490-503);
//   * a prepared list stores stride runs (src/infra/nixl_memory_section.cpp:106-184);
//   * a local-capable backend's registrations are mirrored into a "remote" section under
//     the agent's own name, which is what makes loopback work
//     (src/core/nixl_agent.cpp:476-479).
#ifndef NIXL_AMD_AGENT_IMPL_H
#define NIXL_AMD_AGENT_IMPL_H

#include <array>
#include <map>
#include <memory>
#include <mutex>
#include <set>
#include <shared_mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "backend/backend_engine.h"
#include "backend/backend_plugin.h"
#include "nixl.h"

// ---- plugin loading ------------------------------------------------------------------

struct nixlLoadedPlugin {
    void *dl = nullptr;
    nixlBackendPlugin *table = nullptr;
    std::string path;
};

// Process-wide cache of dlopen'ed backend plugins, keyed by backend type name.
class nixlPluginCache {
public:
    static nixlPluginCache &
    instance();

    // Finds libplugin_<type>.so in NIXL_PLUGIN_DIR (colon-separated) or in
    // <directory of this library>/plugins; null if absent or rejected.
    const nixlLoadedPlugin *
    load(const std::string &type);

    std::vector<std::string>
    discover() const;

private:
    std::vector<std::string>
    searchDirs() const;

    mutable std::mutex mutex_;
    std::unordered_map<std::string, nixlLoadedPlugin> loaded_;
};

// ---- handles -------------------------------------------------------------------------

class nixlBackendH {
public:
    explicit nixlBackendH(nixlBackendEngine *e) noexcept : engine(e) {}

    nixl_backend_t
    getType() const noexcept {
        return engine->getType();
    }

    nixlBackendEngine *engine;
};

// A registered region as the agent stores it.
class nixlSectionDesc : public nixlMetaDesc {
public:
    nixl_blob_t metaBlob;
    using nixlMetaDesc::nixlMetaDesc;
};

// Registered regions of one (memory type, backend), sorted by (devId, addr, len).
class nixlSecDescList {
public:
    void
    add(std::vector<nixlSectionDesc> batch);
    // Index of the element equal to `query`, or -1.
    int
    indexOf(const nixlBasicDesc &query) const;
    // Index of an element whose range covers `query`, or -1.
    int
    coveringIndex(const nixlBasicDesc &query) const;
    void
    removeAt(std::vector<size_t> indices);

    size_t
    size() const {
        return descs_.size();
    }

    bool
    empty() const {
        return descs_.empty();
    }

    const nixlSectionDesc &
    operator[](size_t i) const {
        return descs_[i];
    }

private:
    std::vector<nixlSectionDesc> descs_;
};

using nixl_section_key_t = std::pair<nixl_mem_t, nixlBackendEngine *>;

class nixlMemSection {
public:
    const std::set<nixlBackendEngine *> *
    backendsFor(nixl_mem_t mem) const;

    // Resolve every query descriptor to its covering registration.
    nixl_status_t
    populate(const nixl_xfer_dlist_t &query, nixlBackendEngine *backend, nixl_meta_dlist_t &resp) const;
    // Same, compressed into stride runs.
    nixl_status_t
    populate(const nixl_xfer_dlist_t &query, nixlBackendEngine *backend, nixl_stride_dlist_t &resp) const;
    // Resolve one remote descriptor and append it (memory views).
    nixl_status_t
    addElement(const nixlRemoteDesc &query, nixlBackendEngine *backend, nixl_remote_meta_dlist_t &resp) const;

    std::map<nixl_section_key_t, nixlSecDescList> sections;
    std::array<std::set<nixlBackendEngine *>, FILE_SEG + 1> memToBackend;
};

class nixlDlistH {
public:
    using descs_t = std::unordered_map<nixlBackendEngine *, std::unique_ptr<nixl_stride_dlist_t>>;

    nixlDlistH(const std::string &remote_agent, descs_t &&d) : remoteAgent(remote_agent), descs(std::move(d)) {}

    const std::string remoteAgent; // empty = initiator side
    const descs_t descs;
};

// Storage of the descriptor lists a request made from index vectors carries.  A paged-KV
// request names tens of thousands of blocks, so its two lists are a few MiB that would be
// allocated, faulted in page by page, filled and freed once per request; instead the
// element vectors of released requests are kept (a few, up to a byte limit) and handed to
// the next request with their pages already resident.
class nixlDescStoragePool {
public:
    using storage_t = std::vector<nixlMetaDesc>;

    static nixlDescStoragePool &
    instance();

    // Gives `list` element storage of exactly `count` entries, contents unspecified.
    void
    adopt(nixl_meta_dlist_t &list, size_t count);
    // Takes the element storage of `list` back (the list is left empty).
    void
    surrender(nixl_meta_dlist_t &list);

    static nixlMetaDesc *
    data(nixl_meta_dlist_t &list) {
        return storageOf(list).data();
    }

    static void
    shrink(nixl_meta_dlist_t &list, size_t count) {
        storageOf(list).resize(count);
    }

private:
    // The element vector is a protected member of the list class (the reference's layout).
    struct opened : nixl_meta_dlist_t {
        static storage_t nixl_meta_dlist_t::*
        member() {
            return &opened::descs;
        }
    };

    static storage_t &
    storageOf(nixl_meta_dlist_t &list) {
        return list.*opened::member();
    }

    static constexpr size_t kMaxKept = 8;
    static constexpr size_t kMaxKeptBytes = size_t{64} << 20;
    static constexpr size_t kMinPooled = 1024; // smaller lists are cheaper to allocate than to share
    std::mutex mutex_;
    std::vector<storage_t> kept_;
    size_t keptBytes_ = 0;
};

class nixlXferReqH {
public:
    nixlXferReqH(const std::string &remote_agent, nixl_xfer_op_t op, nixl_mem_t local_type, nixl_mem_t remote_type)
        : initiatorDescs(local_type),
          targetDescs(remote_type),
          remoteAgent(remote_agent),
          backendOp(op) {}

    nixlXferReqH(const nixlXferReqH &) = delete;
    void
    operator=(const nixlXferReqH &) = delete;

    ~nixlXferReqH() {
        if (backendHandle && engine) engine->releaseReqH(backendHandle);
        // only after the backend let go of the request: it may keep references to the lists
        nixlDescStoragePool::instance().surrender(initiatorDescs);
        nixlDescStoragePool::instance().surrender(targetDescs);
    }

    nixlBackendEngine *engine = nullptr;
    nixlBackendReqH *backendHandle = nullptr;
    nixl_meta_dlist_t initiatorDescs;
    nixl_meta_dlist_t targetDescs;
    const std::string remoteAgent;
    nixl_blob_t notifMsg;
    bool hasNotif = false;
    const nixl_xfer_op_t backendOp;
    nixl_status_t status = NIXL_ERR_NOT_POSTED;
    nixl_xfer_telem_t telemetry{};
    chrono_point_t postEnd{};
};

class nixlAgentData {
public:
    nixlAgentData(const std::string &name, const nixlAgentConfig &cfg) : name_(name), config_(cfg) {}
    ~nixlAgentData();

    // Shared for the transfer path, exclusive for registration and backend creation
    // (the reference's nixlLock in RW mode, src/core/sync.h:24-97).
    mutable std::shared_mutex lock;

    const std::string name_;
    const nixlAgentConfig config_;

    // Optional entry of a backend plugin ("nixl_hip_prep_xfer_indexed" in the HIP plugin): a
    // request given as two index vectors into two prepared lists (passed as their stride runs),
    // lowered by the backend itself.  Null for plugins that do not export it.
    using prepIndexedFn = int (*)(nixlBackendEngine *, int, const nixlStrideDesc *, size_t, const int *,
                                  const nixlStrideDesc *, size_t, const int *, size_t, const char *, nixlBackendReqH **);
    struct engineSlot {
        nixlBackendEngine *engine = nullptr;
        const nixlLoadedPlugin *plugin = nullptr;
        std::unique_ptr<nixlBackendH> handle;
        nixl_b_params_t params;
        prepIndexedFn prepIndexed = nullptr;
    };
    // Creation order is preference order.
    std::vector<std::unique_ptr<engineSlot>> engines_;
    std::array<std::vector<nixlBackendEngine *>, FILE_SEG + 1> memToBackend;

    nixlMemSection localSection_;
    // The agent itself (loopback, filled at registration) and every peer whose metadata
    // was loaded.
    std::unordered_map<std::string, nixlMemSection> remoteSections_;
    // Connection info of every remote-capable backend of this agent, by backend type
    // (what getLocalMD publishes), and what each peer published, as loaded
    // (src/core/agent_data.h:57-66).
    std::unordered_map<nixl_backend_t, nixl_blob_t> connMd_;
    std::unordered_map<std::string, std::unordered_map<nixl_backend_t, nixl_blob_t>> remoteBackends_;
    std::vector<nixlBackendEngine *> notifEngines;

    // Drops a peer's sections (unloading every descriptor from its backend) and
    // disconnects its backends.  The caller holds the lock exclusively.
    nixl_status_t
    dropRemote(const std::string &remote_name);

    // Which engine made each live memory view (src/core/agent_data.h mvhToEngine).
    std::unordered_map<nixlMemViewH, nixlBackendEngine *> mvhToEngine;
    // Guards mvhToEngine alone, so that views can be made under the shared lock.
    std::mutex mvhLock;

    engineSlot *
    slotOf(const nixl_backend_t &type) const;
    // Candidate engines for a section and memory type: the caller's choice, else every
    // engine that holds registrations of that type (src/core/nixl_agent.cpp getBackends).
    std::vector<nixlBackendEngine *>
    backendsFor(const nixl_opt_args_t *extra, const nixlMemSection &section, nixl_mem_t mem) const;
};

#endif
