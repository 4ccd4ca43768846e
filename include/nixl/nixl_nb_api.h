// North-bound NIXL vocabulary used on the descriptor-transfer path: status / memory /
// operation enums, descriptor classes, descriptor lists and the optional-argument
// structs.  Declarations (names, enumerator values, data-member order, virtual-member
// order) follow the reference so that a backend plugin built against this tree is
// source compatible with one built against the reference tree:
//   enums and aliases      src/api/cpp/nixl_types.h:41-68,75-80,101-137,153-232,238-301
//   nixlBasicDesc          src/api/cpp/nixl_descriptors.h:32-139, src/infra/nixl_descriptors.cpp:37-86
//   nixlBlobDesc           src/api/cpp/nixl_descriptors.h:146-204
//   nixlRemoteDesc         src/api/cpp/nixl_descriptors.h:211-251
//   nixlDescList<T>        src/api/cpp/nixl_descriptors.h:261-463
//   nixlAgentConfig        src/api/cpp/nixl_params.h:29-108
// Everything is header-only here (the reference keeps the member definitions in
// libnixl); serialisation to the metadata wire format is not part of this path.
#ifndef NIXL_AMD_NB_API_H
#define NIXL_AMD_NB_API_H

#include <algorithm>
#include <chrono>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <iostream>
#include <optional>
#include <sstream>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

class nixlSerDes;
class nixlDlistH;
class nixlBackendH;
class nixlXferReqH;
class nixlAgentData;

// ---- enums -----------------------------------------------------------------------

enum nixl_mem_t { DRAM_SEG, VRAM_SEG, BLK_SEG, OBJ_SEG, FILE_SEG };

enum nixl_xfer_op_t { NIXL_READ, NIXL_WRITE };

enum nixl_status_t {
    NIXL_IN_PROG = 1,
    NIXL_SUCCESS = 0,
    NIXL_ERR_NOT_POSTED = -1,
    NIXL_ERR_INVALID_PARAM = -2,
    NIXL_ERR_BACKEND = -3,
    NIXL_ERR_NOT_FOUND = -4,
    NIXL_ERR_MISMATCH = -5,
    NIXL_ERR_NOT_ALLOWED = -6,
    NIXL_ERR_REPOST_ACTIVE = -7,
    NIXL_ERR_UNKNOWN = -8,
    NIXL_ERR_NOT_SUPPORTED = -9,
    NIXL_ERR_REMOTE_DISCONNECT = -10,
    NIXL_ERR_CANCELED = -11,
    NIXL_ERR_NO_TELEMETRY = -12
};

enum class nixl_thread_sync_t {
    NIXL_THREAD_SYNC_NONE,
    NIXL_THREAD_SYNC_STRICT,
    NIXL_THREAD_SYNC_RW,
    NIXL_THREAD_SYNC_DEFAULT = NIXL_THREAD_SYNC_NONE,
};

enum class nixl_cost_t {
    ANALYTICAL_BACKEND = 0,
};

// ---- aliases ---------------------------------------------------------------------

using nixl_backend_t = std::string;
using nixl_telemetry_plugin_t = std::string;
using nixl_blob_t = std::string;
using nixl_mem_list_t = std::vector<nixl_mem_t>;
using nixl_b_params_t = std::unordered_map<std::string, std::string>;
using nixl_notifs_t = std::unordered_map<std::string, std::vector<nixl_blob_t>>;
using nixl_query_resp_t = std::optional<nixl_b_params_t>;
using nixlMemViewH = void *;
using chrono_point_t = std::chrono::steady_clock::time_point;
using chrono_period_us_t = std::chrono::microseconds;

inline constexpr uint16_t default_comm_port = 8888;

#define NIXL_INIT_AGENT ""
// Agent name of a placeholder entry in a remote memory-view list
// (src/api/cpp/nixl_types.h:305, src/infra/nixl_descriptors.cpp:30).
extern const std::string nixl_null_agent;
// Label under which the reference's metadata side channel stores an agent's metadata
// (src/api/cpp/nixl_types.h:139, value from src/core/nixl_md_manager.cpp:37); kept for callers
// that name it.  The reference also declares default_partial_metadata_label (:145) but defines
// it nowhere, so it is not repeated here.
extern const std::string default_metadata_label;

namespace nixlEnumStrings {

inline std::string
memTypeStr(const nixl_mem_t &mem) {
    static const char *const names[] = {"DRAM_SEG", "VRAM_SEG", "BLK_SEG", "OBJ_SEG", "FILE_SEG"};
    return (mem >= DRAM_SEG && mem <= FILE_SEG) ? names[mem] : "BAD_SEG";
}

inline std::string
xferOpStr(const nixl_xfer_op_t &op) {
    return op == NIXL_READ ? "READ" : (op == NIXL_WRITE ? "WRITE" : "BAD_OP");
}

inline std::string
statusStr(const nixl_status_t &status) {
    switch (status) {
    case NIXL_IN_PROG: return "NIXL_IN_PROG";
    case NIXL_SUCCESS: return "NIXL_SUCCESS";
    case NIXL_ERR_NOT_POSTED: return "NIXL_ERR_NOT_POSTED";
    case NIXL_ERR_INVALID_PARAM: return "NIXL_ERR_INVALID_PARAM";
    case NIXL_ERR_BACKEND: return "NIXL_ERR_BACKEND";
    case NIXL_ERR_NOT_FOUND: return "NIXL_ERR_NOT_FOUND";
    case NIXL_ERR_MISMATCH: return "NIXL_ERR_MISMATCH";
    case NIXL_ERR_NOT_ALLOWED: return "NIXL_ERR_NOT_ALLOWED";
    case NIXL_ERR_REPOST_ACTIVE: return "NIXL_ERR_REPOST_ACTIVE";
    case NIXL_ERR_UNKNOWN: return "NIXL_ERR_UNKNOWN";
    case NIXL_ERR_NOT_SUPPORTED: return "NIXL_ERR_NOT_SUPPORTED";
    case NIXL_ERR_REMOTE_DISCONNECT: return "NIXL_ERR_REMOTE_DISCONNECT";
    case NIXL_ERR_CANCELED: return "NIXL_ERR_CANCELED";
    case NIXL_ERR_NO_TELEMETRY: return "NIXL_ERR_NO_TELEMETRY";
    }
    return "BAD_STATUS";
}

} // namespace nixlEnumStrings

// ---- optional arguments and telemetry --------------------------------------------

struct nixlAgentOptionalArgs {
    std::vector<nixlBackendH *> backends;
    std::optional<nixl_blob_t> notif;
    nixl_blob_t notifMsg;
    bool hasNotif = false;
    bool skipDescMerge = false;
    bool includeConnInfo = false;
    std::string ipAddr;
    int port = default_comm_port;
    std::string metadataLabel;
    nixl_blob_t customParam;
};
using nixl_opt_args_t = nixlAgentOptionalArgs;

struct nixlXferTelemetry {
    chrono_point_t startTime;
    chrono_period_us_t postDuration;
    chrono_period_us_t xferDuration;
    size_t totalBytes;
    size_t descCount;
};
using nixl_xfer_telem_t = nixlXferTelemetry;

struct nixlAgentConfig {
    static constexpr bool kDefaultUseProgThread = false;
    static constexpr bool kDefaultUseListenThread = false;
    static constexpr uint16_t kDefaultListenPort = default_comm_port;
    static constexpr nixl_thread_sync_t kDefaultSyncMode =
        nixl_thread_sync_t::NIXL_THREAD_SYNC_DEFAULT;
    static constexpr bool kDefaultCaptureTelemetry = false;
    static constexpr uint64_t kDefaultPthrDelayUs = 0;
    static constexpr uint64_t kDefaultLthrDelayUs = 100000;
    static constexpr std::chrono::microseconds kDefaultEtcdWatchTimeout =
        std::chrono::microseconds(5000000);

    bool useProgThread = kDefaultUseProgThread;
    bool useListenThread = kDefaultUseListenThread;
    uint16_t listenPort = kDefaultListenPort;
    nixl_thread_sync_t syncMode = kDefaultSyncMode;
    bool captureTelemetry = kDefaultCaptureTelemetry;
    uint64_t pthrDelay = kDefaultPthrDelayUs;
    uint64_t lthrDelay = kDefaultLthrDelayUs;
    std::chrono::microseconds etcdWatchTimeout = kDefaultEtcdWatchTimeout;

    nixlAgentConfig() = default;

    explicit nixlAgentConfig(const bool use_prog_thread,
                             const bool use_listen_thread = kDefaultUseListenThread,
                             uint16_t port = kDefaultListenPort,
                             nixl_thread_sync_t sync_mode = kDefaultSyncMode,
                             unsigned int /*num_workers*/ = 1,
                             uint64_t pthr_delay_us = kDefaultPthrDelayUs,
                             uint64_t lthr_delay_us = kDefaultLthrDelayUs,
                             bool capture_telemetry = kDefaultCaptureTelemetry,
                             std::chrono::microseconds etcd_watch_timeout =
                                 kDefaultEtcdWatchTimeout) noexcept
        : useProgThread(use_prog_thread),
          useListenThread(use_listen_thread),
          listenPort(port),
          syncMode(sync_mode),
          captureTelemetry(capture_telemetry),
          pthrDelay(pthr_delay_us),
          lthrDelay(lthr_delay_us),
          etcdWatchTimeout(etcd_watch_timeout) {}
};

// ---- descriptors -----------------------------------------------------------------

// One contiguous span: (address | offset, byte length, device | block | file id).
// Plain data, no virtual members; ordering is devId, then addr, then len.
class nixlBasicDesc {
public:
    uintptr_t addr;
    size_t len;
    uint64_t devId;

    nixlBasicDesc() {}

    nixlBasicDesc(const uintptr_t &addr_, const size_t &len_, const uint64_t &dev_id)
        : addr(addr_),
          len(len_),
          devId(dev_id) {}

    // From the raw 24-byte image; any other size yields the all-zero descriptor.
    nixlBasicDesc(const nixl_blob_t &blob) {
        if (blob.size() == sizeof(nixlBasicDesc)) {
            std::memcpy(static_cast<void *>(this), blob.data(), sizeof(nixlBasicDesc));
        } else {
            addr = 0;
            len = 0;
            devId = 0;
        }
    }

    nixlBasicDesc(const nixlBasicDesc &) = default;
    nixlBasicDesc &
    operator=(const nixlBasicDesc &) = default;
    ~nixlBasicDesc() = default;

    bool
    operator<(const nixlBasicDesc &o) const noexcept {
        if (devId != o.devId) return devId < o.devId;
        if (addr != o.addr) return addr < o.addr;
        return len < o.len;
    }

    friend bool
    operator==(const nixlBasicDesc &a, const nixlBasicDesc &b) {
        return a.addr == b.addr && a.len == b.len && a.devId == b.devId;
    }

    friend bool
    operator!=(const nixlBasicDesc &a, const nixlBasicDesc &b) {
        return !(a == b);
    }

    bool
    covers(const nixlBasicDesc &q) const noexcept {
        return devId == q.devId && addr <= q.addr && (addr + len) >= (q.addr + q.len);
    }

    bool
    overlaps(const nixlBasicDesc &q) const {
        if (devId != q.devId) return false;
        return !((addr + len <= q.addr) || (q.addr + q.len <= addr));
    }

    nixl_blob_t
    serialize() const {
        return std::string(reinterpret_cast<const char *>(this), sizeof(nixlBasicDesc));
    }

    void
    print(const std::string &suffix) const {
        std::cerr << "Desc (" << addr << ", " << len << ") from devID " << devId << suffix
                  << std::endl;
    }
};

// A span plus an opaque blob (registration hints such as a file path).
class nixlBlobDesc : public nixlBasicDesc {
public:
    nixl_blob_t metaInfo;

    using nixlBasicDesc::nixlBasicDesc;

    nixlBlobDesc(const uintptr_t &addr_,
                 const size_t &len_,
                 const uint64_t &dev_id,
                 const nixl_blob_t &meta_info)
        : nixlBasicDesc(addr_, len_, dev_id),
          metaInfo(meta_info) {}

    nixlBlobDesc(const nixlBasicDesc &desc, const nixl_blob_t &meta_info)
        : nixlBasicDesc(desc),
          metaInfo(meta_info) {}

    nixlBlobDesc(const nixl_blob_t &blob) {
        if (blob.size() >= sizeof(nixlBasicDesc)) {
            std::memcpy(static_cast<nixlBasicDesc *>(this), blob.data(), sizeof(nixlBasicDesc));
            metaInfo = blob.substr(sizeof(nixlBasicDesc));
        } else {
            addr = 0;
            len = 0;
            devId = 0;
        }
    }

    friend bool
    operator==(const nixlBlobDesc &a, const nixlBlobDesc &b) {
        return static_cast<const nixlBasicDesc &>(a) == static_cast<const nixlBasicDesc &>(b) &&
            a.metaInfo == b.metaInfo;
    }

    nixl_blob_t
    serialize() const {
        return nixlBasicDesc::serialize() + metaInfo;
    }

    void
    print(const std::string &suffix) const {
        nixlBasicDesc::print(", Metadata: " + metaInfo + suffix);
    }
};

// A span on a named remote agent (memory-view preparation).
struct nixlRemoteDesc : public nixlBasicDesc {
    std::string remoteAgent;

    using nixlBasicDesc::nixlBasicDesc;

    nixlRemoteDesc(const uintptr_t addr_,
                   const size_t len_,
                   const uint64_t dev_id,
                   const std::string &remote_agent)
        : nixlBasicDesc{addr_, len_, dev_id},
          remoteAgent{remote_agent} {}

    nixlRemoteDesc(const nixlBasicDesc &desc, const std::string &remote_agent)
        : nixlBasicDesc{desc},
          remoteAgent{remote_agent} {}

    explicit nixlRemoteDesc(const nixl_blob_t &blob) {
        if (blob.size() < sizeof(nixlBasicDesc)) {
            addr = 0;
            len = 0;
            devId = 0;
            return;
        }
        std::memcpy(static_cast<nixlBasicDesc *>(this), blob.data(), sizeof(nixlBasicDesc));
        remoteAgent = blob.substr(sizeof(nixlBasicDesc));
    }

    nixl_blob_t
    serialize() const {
        return nixlBasicDesc::serialize() + remoteAgent;
    }
};

inline bool
operator==(const nixlRemoteDesc &a, const nixlRemoteDesc &b) {
    return static_cast<const nixlBasicDesc &>(a) == static_cast<const nixlBasicDesc &>(b) &&
        a.remoteAgent == b.remoteAgent;
}

// A typed, ordered list of descriptors.  Object layout is {vptr, type, descs}; the
// virtual members, in declaration order, are the destructor, resize, addDesc, getIndex.
template<class T> class nixlDescList {
protected:
    nixl_mem_t type;
    std::vector<T> descs;

public:
    nixlDescList(const nixl_mem_t &type_, const int &init_size = 0)
        : type(type_),
          descs(static_cast<size_t>(init_size)) {}

    nixlDescList(const nixlDescList<T> &) = default;
    nixlDescList &
    operator=(const nixlDescList<T> &) = default;
    nixlDescList(nixlDescList<T> &&) = default;
    nixlDescList &
    operator=(nixlDescList<T> &&) = default;

    virtual ~nixlDescList() = default;

    inline nixl_mem_t
    getType() const {
        return type;
    }

    inline int
    descCount() const {
        return static_cast<int>(descs.size());
    }

    bool
    isEmpty() const noexcept {
        return descs.empty();
    }

    const T &
    operator[](size_t index) const {
        return descs[index];
    }

    T &
    operator[](size_t index) {
        return descs[index];
    }

    inline typename std::vector<T>::const_iterator
    begin() const {
        return descs.begin();
    }

    inline typename std::vector<T>::const_iterator
    end() const {
        return descs.end();
    }

    inline typename std::vector<T>::iterator
    begin() {
        return descs.begin();
    }

    inline typename std::vector<T>::iterator
    end() {
        return descs.end();
    }

    template<class Y>
    friend bool
    operator==(const nixlDescList<Y> &lhs, const nixlDescList<Y> &rhs);

    virtual void
    resize(const size_t &count) {
        descs.resize(count);
    }

    inline void
    reserve(size_t count) {
        descs.reserve(count);
    }

    inline void
    clear() {
        descs.clear();
    }

    virtual void
    addDesc(const T &desc) {
        descs.push_back(desc);
    }

    template<class... Args>
    T &
    emplace(Args &&...args) {
        return descs.emplace_back(std::forward<Args>(args)...);
    }

    void
    remDesc(const int &index) {
        if (index < 0 || static_cast<size_t>(index) >= descs.size())
            throw std::out_of_range("nixlDescList::remDesc: index out of range");
        descs.erase(descs.begin() + index);
    }

    nixlDescList<nixlBasicDesc>
    trim() const {
        nixlDescList<nixlBasicDesc> out(type);
        out.reserve(descs.size());
        for (const auto &d : descs)
            out.addDesc(static_cast<const nixlBasicDesc &>(d));
        return out;
    }

    virtual int
    getIndex(const nixlBasicDesc &query) const {
        for (size_t i = 0; i < descs.size(); ++i)
            if (static_cast<const nixlBasicDesc &>(descs[i]) == query) return static_cast<int>(i);
        return NIXL_ERR_NOT_FOUND;
    }

    void
    print() const {
        std::cerr << to_string() << std::endl;
    }

    std::string
    to_string(bool compact = false) const {
        std::ostringstream os;
        os << "DescList mem type " << nixlEnumStrings::memTypeStr(type) << " count "
           << descs.size();
        if (!compact)
            for (const auto &d : descs) {
                const nixlBasicDesc &b = d;
                os << "\n  (" << b.addr << ", " << b.len << ", dev " << b.devId << ")";
            }
        return os.str();
    }
};

template<class Y>
bool
operator==(const nixlDescList<Y> &lhs, const nixlDescList<Y> &rhs) {
    if (lhs.getType() != rhs.getType() || lhs.descCount() != rhs.descCount()) return false;
    for (size_t i = 0; i < static_cast<size_t>(lhs.descCount()); ++i)
        if (!(lhs[i] == rhs[i])) return false;
    return true;
}

using nixl_xfer_dlist_t = nixlDescList<nixlBasicDesc>;
using nixl_reg_dlist_t = nixlDescList<nixlBlobDesc>;
using nixl_remote_dlist_t = nixlDescList<nixlRemoteDesc>;
using nixl_local_dlist_t = nixlDescList<nixlBasicDesc>;

#endif // NIXL_AMD_NB_API_H
