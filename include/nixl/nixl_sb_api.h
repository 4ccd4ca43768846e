// South-bound NIXL API: what a backend plugin derives from and what the agent hands
// to it.  This is the drop-in boundary of the HIP backend.  Class names, data-member
// order and virtual-member order follow the reference so that the object and vtable
// layouts agree with a plugin compiled against the reference tree (C++20, libstdc++):
//   nixlBackendOptionalArgs, nixlBackendInitParams   src/api/cpp/backend/backend_aux.h:33-57
//   nixlBackendReqH, nixlBackendMD, nixlBackendConnMD src/api/cpp/backend/backend_aux.h:60-89
//   nixlMetaDesc, nixlRemoteMetaDesc                  src/api/cpp/backend/backend_aux.h:92-136
//   nixlStrideDesc, nixlStrideDescList                src/api/cpp/backend/backend_aux.h:140-208
//   nixlTelemetryEvent, event type enum               src/core/telemetry/telemetry_event.h:36-58,256-266
//   nixlBackendEngine                                 src/api/cpp/backend/backend_engine.h:33-251
//   nixlBackendPlugin, creator, nixl_plugin_init/fini src/api/cpp/backend/backend_plugin.h:33-127
#ifndef NIXL_AMD_SB_API_H
#define NIXL_AMD_SB_API_H

#include <cassert>
#include <chrono>
#include <cstdint>
#include <exception>
#include <memory>
#include <mutex>
#include <string>
#include <type_traits>
#include <vector>

#include "nixl_nb_api.h"

namespace nixlTime {
using us_t = uint64_t;
} // namespace nixlTime

// ---- telemetry events a backend may queue for the agent ----------------------------

enum class nixl_telemetry_event_type_t : uint32_t {
    AGENT_TX_BYTES = 0,
    AGENT_RX_BYTES = 1,
    AGENT_TX_REQUESTS_NUM = 2,
    AGENT_RX_REQUESTS_NUM = 3,
    AGENT_MEMORY_REGISTERED = 4,
    AGENT_MEMORY_DEREGISTERED = 5,
    AGENT_XFER_TIME = 6,
    AGENT_XFER_POST_TIME = 7,
    AGENT_ERR_NOT_POSTED = 8,
    AGENT_ERR_INVALID_PARAM = 9,
    AGENT_ERR_BACKEND = 10,
    AGENT_ERR_NOT_FOUND = 11,
    AGENT_ERR_MISMATCH = 12,
    AGENT_ERR_NOT_ALLOWED = 13,
    AGENT_ERR_REPOST_ACTIVE = 14,
    AGENT_ERR_UNKNOWN = 15,
    AGENT_ERR_NOT_SUPPORTED = 16,
    AGENT_ERR_REMOTE_DISCONNECT = 17,
    AGENT_ERR_CANCELED = 18,
    AGENT_ERR_NO_TELEMETRY = 19,
    AGENT_TELEMETRY_EVENTS_DROPPED = 20,
};

struct nixlTelemetryEvent {
    nixl_telemetry_event_type_t eventType_;
    uint64_t value_;

    nixlTelemetryEvent() noexcept = default;

    nixlTelemetryEvent(nixl_telemetry_event_type_t event_type, uint64_t value) noexcept
        : eventType_(event_type),
          value_(value) {}
};

// ---- auxiliary types ---------------------------------------------------------------

typedef std::vector<std::pair<std::string, std::string>> notif_list_t;

struct nixlBackendOptionalArgs {
    nixl_blob_t notifMsg;
    bool hasNotif = false;
    nixl_blob_t customParam;
};
using nixl_opt_b_args_t = nixlBackendOptionalArgs;

// Filled by the agent in createBackend and passed to the engine constructor.
class nixlBackendInitParams {
public:
    std::string localAgent;
    nixl_backend_t type;
    nixl_b_params_t *customParams = nullptr;
    bool enableProgTh = false;
    nixlTime::us_t pthrDelay = 0;
    nixl_thread_sync_t syncMode;
    bool enableTelemetry_ = false;
};

// Opaque per-request state owned by the backend.
class nixlBackendReqH {
public:
    nixlBackendReqH() {}
    virtual ~nixlBackendReqH() {}
};

// Opaque per-registration state owned by the backend.
class nixlBackendMD {
protected:
    bool isPrivateMD;

public:
    nixlBackendMD(bool isPrivate) { isPrivateMD = isPrivate; }
    virtual ~nixlBackendMD() {}
};

class nixlBackendConnMD {
public:
    std::string dstIpAddress;
    uint16_t dstPort;
};

// A span annotated with the registration that covers it (32 bytes, no vtable).
class nixlMetaDesc : public nixlBasicDesc {
public:
    nixlBackendMD *metadataP;

    using nixlBasicDesc::nixlBasicDesc;

    nixlMetaDesc() : nixlBasicDesc() { metadataP = nullptr; }

    nixlMetaDesc(uintptr_t addr_, size_t len_, uint64_t dev_id, nixlBackendMD *metadata)
        : nixlBasicDesc(addr_, len_, dev_id),
          metadataP(metadata) {}

    inline friend bool
    operator==(const nixlMetaDesc &a, const nixlMetaDesc &b) {
        return static_cast<const nixlBasicDesc &>(a) == static_cast<const nixlBasicDesc &>(b) &&
            a.metadataP == b.metadataP;
    }

    inline void
    print(const std::string &suffix) const {
        nixlBasicDesc::print(", Backend ptr val: " +
                             std::to_string(reinterpret_cast<uintptr_t>(metadataP)) + suffix);
    }
};

struct nixlRemoteMetaDesc : public nixlMetaDesc {
    std::string remoteAgent;

    using nixlMetaDesc::nixlMetaDesc;

    explicit nixlRemoteMetaDesc(const std::string &remote_agent)
        : nixlMetaDesc(),
          remoteAgent(remote_agent) {}
};

inline bool
operator==(const nixlRemoteMetaDesc &a, const nixlRemoteMetaDesc &b) {
    return static_cast<const nixlMetaDesc &>(a) == static_cast<const nixlMetaDesc &>(b) &&
        a.remoteAgent == b.remoteAgent;
}

typedef nixlDescList<nixlMetaDesc> nixl_meta_dlist_t;
using nixl_remote_meta_dlist_t = nixlDescList<nixlRemoteMetaDesc>;

// Run-length form kept by a prepared descriptor list: `count` equal-length blocks whose
// starts are `stride` bytes apart; the first block has flat index `start_idx`.
class nixlStrideDesc : public nixlMetaDesc {
public:
    size_t stride = 0;
    size_t count = 0;
    size_t start_idx = 0;

    nixlStrideDesc() = default;

    using nixlMetaDesc::nixlMetaDesc;

    nixlStrideDesc(uintptr_t addr_,
                   size_t len_,
                   uint64_t dev_id,
                   nixlBackendMD *metadata,
                   size_t stride_,
                   size_t count_)
        : nixlMetaDesc(addr_, len_, dev_id, metadata),
          stride(stride_),
          count(count_),
          start_idx(0) {}

    // Block `idx` of the run, widened to `size` consecutive blocks.
    [[nodiscard]] nixlMetaDesc
    getMetaDesc(size_t idx, size_t size) const noexcept {
        return nixlMetaDesc(
            addr + static_cast<uintptr_t>(idx - start_idx) * stride, len * size, devId, metadataP);
    }
};

class nixlStrideDescList : public nixlDescList<nixlStrideDesc> {
public:
    using nixlDescList<nixlStrideDesc>::nixlDescList;

    [[nodiscard]] size_t
    flatSize() const {
        if (descs.empty()) return 0;
        return descs.back().start_idx + descs.back().count;
    }

    // Run holding flat block `flat_idx`: first guess assumes runs of `run_size` blocks
    // each, then falls back to bisection on start_idx.
    const nixlStrideDesc &
    find(size_t flat_idx, size_t run_size) const noexcept {
        assert(run_size > 0);
        size_t mid = flat_idx / run_size;
        if (flat_idx - descs[mid].start_idx < descs[mid].count) [[likely]]
            return descs[mid];
        size_t lo = 0;
        size_t hi = descs.size() - 1;
        while (lo < hi) {
            if (descs[mid].start_idx <= flat_idx)
                lo = mid;
            else
                hi = mid - 1;
            mid = (lo + hi + 1) >> 1;
        }
        return descs[lo];
    }
};
using nixl_stride_dlist_t = nixlStrideDescList;

// ---- the engine base class ---------------------------------------------------------

constexpr size_t MAX_TELEMETRY_QUEUE_SIZE = 1000;

class nixlBackendEngine {
private:
    nixl_backend_t backendType;
    nixl_b_params_t customParams;
    std::vector<nixlTelemetryEvent> telemetryEvents_;
    std::mutex telemetryEventsMutex_;

protected:
    bool initErr = false;
    const std::string localAgent;
    const bool enableTelemetry_;

    [[nodiscard]] nixl_status_t
    setInitParam(const std::string &key, const std::string &value) {
        return customParams.emplace(key, value).second ? NIXL_SUCCESS : NIXL_ERR_NOT_ALLOWED;
    }

    [[nodiscard]] nixl_status_t
    getInitParam(const std::string &key, std::string &value) const {
        const auto it = customParams.find(key);
        if (it == customParams.end()) return NIXL_ERR_INVALID_PARAM;
        value = it->second;
        return NIXL_SUCCESS;
    }

    void
    addTelemetryEvent(nixl_telemetry_event_type_t event_type, uint64_t value) {
        if (!enableTelemetry_) return;
        std::lock_guard<std::mutex> lock(telemetryEventsMutex_);
        if (telemetryEvents_.size() < MAX_TELEMETRY_QUEUE_SIZE)
            telemetryEvents_.emplace_back(event_type, value);
    }

public:
    explicit nixlBackendEngine(const nixlBackendInitParams *init_params)
        : backendType(init_params->type),
          customParams(*init_params->customParams),
          localAgent(init_params->localAgent),
          enableTelemetry_(init_params->enableTelemetry_) {}

    nixlBackendEngine(nixlBackendEngine &&) = delete;
    nixlBackendEngine(const nixlBackendEngine &) = delete;
    void
    operator=(nixlBackendEngine &&) = delete;
    void
    operator=(const nixlBackendEngine &) = delete;

    virtual ~nixlBackendEngine() = default;

    std::vector<nixlTelemetryEvent>
    getTelemetryEvents() {
        std::lock_guard<std::mutex> lock(telemetryEventsMutex_);
        return std::move(telemetryEvents_);
    }

    bool
    getInitErr() const noexcept {
        return initErr;
    }

    const nixl_backend_t &
    getType() const noexcept {
        return backendType;
    }

    const nixl_b_params_t &
    getCustomParams() const noexcept {
        return customParams;
    }

    // Capability queries; they decide which of the optional groups below the agent calls.
    virtual bool
    supportsRemote() const = 0;
    virtual bool
    supportsLocal() const = 0;
    virtual bool
    supportsNotif() const = 0;
    virtual nixl_mem_list_t
    getSupportedMems() const = 0;

    // Required by every backend.
    virtual nixl_status_t
    registerMem(const nixlBlobDesc &mem, const nixl_mem_t &nixl_mem, nixlBackendMD *&out) = 0;
    virtual nixl_status_t
    deregisterMem(nixlBackendMD *meta) = 0;
    virtual nixl_status_t
    connect(const std::string &remote_agent) = 0;
    virtual nixl_status_t
    disconnect(const std::string &remote_agent) = 0;
    virtual nixl_status_t
    unloadMD(nixlBackendMD *input) = 0;
    virtual nixl_status_t
    prepXfer(const nixl_xfer_op_t &operation,
             const nixl_meta_dlist_t &local,
             const nixl_meta_dlist_t &remote,
             const std::string &remote_agent,
             nixlBackendReqH *&handle,
             const nixl_opt_b_args_t *opt_args = nullptr) const = 0;
    virtual nixl_status_t
    postXfer(const nixl_xfer_op_t &operation,
             const nixl_meta_dlist_t &local,
             const nixl_meta_dlist_t &remote,
             const std::string &remote_agent,
             nixlBackendReqH *&handle,
             const nixl_opt_b_args_t *opt_args = nullptr) const = 0;
    virtual nixl_status_t
    checkXfer(nixlBackendReqH *handle) const = 0;
    virtual nixl_status_t
    releaseReqH(nixlBackendReqH *handle) const = 0;

    // Memory views for device-initiated transfers.
    virtual nixl_status_t
    prepMemView(const nixl_remote_meta_dlist_t &,
                nixlMemViewH &,
                const nixl_opt_b_args_t * = nullptr) const {
        return NIXL_ERR_NOT_SUPPORTED;
    }
    virtual nixl_status_t
    prepMemView(const nixl_meta_dlist_t &, nixlMemViewH &, const nixl_opt_b_args_t * = nullptr) const {
        return NIXL_ERR_NOT_SUPPORTED;
    }
    virtual void releaseMemView(nixlMemViewH) const {}

    // Needed when supportsRemote().
    virtual nixl_status_t
    getPublicData(const nixlBackendMD *, std::string &) const {
        return NIXL_ERR_BACKEND;
    }
    virtual nixl_status_t
    getConnInfo(std::string &) const {
        return NIXL_ERR_BACKEND;
    }
    virtual nixl_status_t
    loadRemoteConnInfo(const std::string &, const std::string &) {
        return NIXL_ERR_BACKEND;
    }
    virtual nixl_status_t
    loadRemoteMD(const nixlBlobDesc &, const nixl_mem_t &, const std::string &, nixlBackendMD *&) {
        return NIXL_ERR_BACKEND;
    }

    // Needed when supportsLocal().
    virtual nixl_status_t
    loadLocalMD(nixlBackendMD *, nixlBackendMD *&) {
        return NIXL_ERR_BACKEND;
    }

    // Needed when supportsNotif().
    virtual nixl_status_t
    getNotifs(notif_list_t &) {
        return NIXL_ERR_BACKEND;
    }
    virtual nixl_status_t
    genNotif(const std::string &, const std::string &) const {
        return NIXL_ERR_BACKEND;
    }

    // Optional.
    virtual nixl_status_t
    queryMem(const nixl_reg_dlist_t &, std::vector<nixl_query_resp_t> &) const {
        return NIXL_ERR_NOT_SUPPORTED;
    }
    virtual nixl_status_t
    estimateXferCost(const nixl_xfer_op_t &,
                     const nixl_meta_dlist_t &,
                     const nixl_meta_dlist_t &,
                     const std::string &,
                     nixlBackendReqH *const &,
                     std::chrono::microseconds &,
                     std::chrono::microseconds &,
                     nixl_cost_t &,
                     const nixl_opt_args_t * = nullptr) const {
        return NIXL_ERR_NOT_SUPPORTED;
    }
};

// ---- the plugin table a shared object exports ---------------------------------------

#define NIXL_PLUGIN_API_VERSION 1
#define NIXL_PLUGIN_EXPORT __attribute__((visibility("default")))

class nixlBackendPlugin {
public:
    int api_version;
    nixlBackendEngine *(*create_engine)(const nixlBackendInitParams *init_params);
    void (*destroy_engine)(nixlBackendEngine *engine);
    const char *(*get_plugin_name)();
    const char *(*get_plugin_version)();
    nixl_b_params_t (*get_backend_options)();
    nixl_mem_list_t (*get_backend_mems)();
};

// Builds the static plugin table for an engine type whose constructor takes
// `const nixlBackendInitParams *`.  A throwing constructor yields a null engine.
template<typename EngineType> class nixlBackendPluginCreator {
public:
    static nixlBackendPlugin *
    create(int api_version,
           const char *name,
           const char *version,
           const nixl_b_params_t &params,
           const nixl_mem_list_t &mem_list) {
        static const std::string plugin_name = name;
        static const std::string plugin_version = version;
        static const nixl_b_params_t plugin_params = params;
        static const nixl_mem_list_t plugin_mems = mem_list;
        static nixlBackendPlugin table = {api_version,
                                          makeEngine,
                                          dropEngine,
                                          []() { return plugin_name.c_str(); },
                                          []() { return plugin_version.c_str(); },
                                          []() { return plugin_params; },
                                          []() { return plugin_mems; }};
        return &table;
    }

private:
    [[nodiscard]] static nixlBackendEngine *
    makeEngine(const nixlBackendInitParams *init_params) {
        try {
            return new EngineType(init_params);
        }
        catch (const std::exception &e) {
            std::cerr << "nixl plugin: engine construction failed: " << e.what() << std::endl;
            return nullptr;
        }
    }

    static void
    dropEngine(nixlBackendEngine *engine) {
        delete engine;
    }
};

typedef nixlBackendPlugin *(*nixlStaticPluginCreatorFunc)();

extern "C" {
NIXL_PLUGIN_EXPORT nixlBackendPlugin *
nixl_plugin_init();
NIXL_PLUGIN_EXPORT void
nixl_plugin_fini();
}

#endif // NIXL_AMD_SB_API_H
