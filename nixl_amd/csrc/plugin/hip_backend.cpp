#include "hip_backend.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <unordered_map>

#include "backend/backend_plugin.h"
#include "common/nixl_log.h"
#include "nixl_amd_device.h"

namespace {

int
paramInt(const nixl_b_params_t *params, const char *key, int fallback) {
    if (!params) return fallback;
    const auto it = params->find(key);
    if (it == params->end()) return fallback;
    char *end = nullptr;
    const long v = std::strtol(it->second.c_str(), &end, 10);
    if (end == it->second.c_str() || *end != '\0')
        throw std::runtime_error(std::string("HIP backend: parameter '") + key +
                                 "' is not an integer: " + it->second);
    return static_cast<int>(v);
}

bool
hipOk(hipError_t e, const char *what) {
    if (e == hipSuccess) return true;
    NIXL_ERROR << "HIP backend: " << what << " failed: " << hipGetErrorString(e);
    return false;
}

// Makes `device` current for the calling thread while the object lives and restores the
// thread's previous device afterwards, so that a call into the backend never leaves the
// application on another GPU than it was on.
class DeviceScope {
public:
    explicit DeviceScope(int device) {
        int current = -1;
        if (hipGetDevice(&current) != hipSuccess) current = -1;
        if (current == device) return;
        status_ = hipSetDevice(device);
        if (status_ == hipSuccess && current >= 0) previous_ = current;
    }

    ~DeviceScope() {
        if (previous_ >= 0) (void)hipSetDevice(previous_);
    }

    DeviceScope(const DeviceScope &) = delete;
    DeviceScope &
    operator=(const DeviceScope &) = delete;

    bool
    ok() const {
        if (status_ != hipSuccess) NIXL_ERROR << "HIP backend: hipSetDevice failed: " << hipGetErrorString(status_);
        return status_ == hipSuccess;
    }

private:
    int previous_ = -1;
    hipError_t status_ = hipSuccess;
};

// Engines of this process by agent name: how a notification reaches another agent's queue.
std::mutex g_registryMutex;
std::unordered_map<std::string, const nixlHipEngine *> g_registry;

// What a peer needs to address a region (getPublicData / loadRemoteMD).  A peer of another
// process also needs the IPC handle of the allocation the region lies in.
struct PublicRegion {
    uint64_t magic;
    uint64_t addr;
    uint64_t len;
    int64_t pid;
    int32_t device;
    int32_t mem;
    uint64_t alloc_base;
    uint64_t alloc_size;
    uint32_t has_ipc;
    uint32_t reserved;
    hipIpcMemHandle_t ipc;
};
constexpr uint64_t kRegionMagic = 0x324e474552504948ull; // "HIPREGN2"
constexpr const char *kConnPrefix = "HIP2:pid=";
constexpr const char *kConnMailbox = ";mbox=";
// Allocations of 2 GiB and more are not shared between processes: opening such a mapping has
// been seen not to return.
constexpr size_t kMaxIpcAllocation = (size_t{2} << 30) - 1;

using nixl_amd_hip::kMailboxSlotBytes;
std::atomic<unsigned> g_mailboxCounter{0};

} // namespace

nixlHipEngine::Mailbox *
nixlHipEngine::mapMailbox(const std::string &name, bool create) {
    return nixl_amd_hip::mapMailbox(name, create);
}

void
nixlHipEngine::unmapMailbox(Mailbox *m) {
    nixl_amd_hip::unmapMailbox(m);
}

nixlHipReqH::~nixlHipReqH() {
    const DeviceScope on_device(device);
    if (plan) (void)nixl_amd_copy_plan_destroy(plan);
}

// NIXL_SUCCESS when nothing of the request is running any more, NIXL_IN_PROG while its posted
// copy runs, NIXL_ERR_BACKEND if it failed.  The plan itself keeps the event behind its last
// launch, so a post costs one event record, not two.
nixl_status_t
nixlHipReqH::state(bool wait) const {
    if (!posted) return NIXL_SUCCESS;
    const int rc = nixl_amd_copy_plan_status(plan, wait ? 1 : 0);
    if (rc == NIXL_AMD_OK) return NIXL_SUCCESS;
    if (rc == NIXL_AMD_ERR_BUSY) return NIXL_IN_PROG;
    NIXL_ERROR << "HIP backend: transfer failed: " << nixl_amd_last_error();
    return NIXL_ERR_BACKEND;
}

nixlHipEngine::nixlHipEngine(const nixlBackendInitParams *init_params)
    : nixlBackendEngine(init_params) {
    const nixl_b_params_t *p = init_params->customParams;
    tuning_.units_per_lane = paramInt(p, "units_per_lane", 0);
    tuning_.nontemporal = paramInt(p, "nontemporal", 0);
    tuning_.sort_scatter = paramInt(p, "sort_scatter", 0);
    tuning_.max_workgroups = paramInt(p, "max_workgroups", 0);
    tuning_.waves_per_workgroup = paramInt(p, "waves_per_workgroup", 0);
    tuning_.xcd_swizzle = paramInt(p, "xcd_swizzle", 0);
    indexedPrep_ = paramInt(p, "indexed_prep", 1) != 0;
    prepThreads_ = paramInt(p, "prep_threads", 1);
    if (prepThreads_ < 1 || prepThreads_ > 16) throw std::runtime_error("HIP backend: prep_threads must be in [1, 16]");
    streamsPerDevice_ = paramInt(p, "num_streams", 1);
    if (streamsPerDevice_ < 1 || streamsPerDevice_ > 16)
        throw std::runtime_error("HIP backend: num_streams must be in [1, 16]");
    if (p) {
        // "stream" carries a hipStream_t of the application, as an integer.  Transfers are
        // then enqueued there, ordered with the application's own work on that stream, and
        // the application may bracket them with its own events.
        const auto it = p->find("stream");
        if (it != p->end() && !it->second.empty()) {
            char *end = nullptr;
            const unsigned long long v = std::strtoull(it->second.c_str(), &end, 0);
            if (end == it->second.c_str() || *end != '\0')
                throw std::runtime_error("HIP backend: parameter 'stream' is not an integer: " + it->second);
            externalStream_ = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(v));
            useExternalStream_ = true;
        }
    }

    const int n = nixl_amd_device_count();
    if (n <= 0) {
        NIXL_ERROR << "HIP backend: no HIP device visible (" << nixl_amd_last_error() << ")";
        initErr = true;
        return;
    }
    numDevices_ = n;
    streams_.assign(static_cast<size_t>(n) * streamsPerDevice_, nullptr);
    {
        std::lock_guard<std::mutex> lock(g_registryMutex);
        g_registry[localAgent] = this;
    }
    // Where agents of other processes leave their notifications.  Without it (no /dev/shm)
    // the engine still serves this process.
    mailboxName_ = "/nixl_amd_hip_" + std::to_string(static_cast<long long>(getpid())) + "_" +
        std::to_string(g_mailboxCounter.fetch_add(1));
    mailbox_ = mapMailbox(mailboxName_, true);
    if (!mailbox_ && errno == EEXIST) {
        // The name holds this process's id: an object of that name is what a process that died
        // with the same id left behind.
        shm_unlink(mailboxName_.c_str());
        mailbox_ = mapMailbox(mailboxName_, true);
    }
    if (!mailbox_) {
        NIXL_WARN << "HIP backend: no shared-memory mailbox (" << std::strerror(errno) << "); agents of other processes cannot notify '"
                  << localAgent << "'";
        mailboxName_.clear();
    }
    if (init_params->enableProgTh) {
        progressOn_ = true;
        progressDelayUs_ = init_params->pthrDelay;
        progress_ = std::thread(&nixlHipEngine::progressLoop, this);
    }
}

nixlHipEngine::~nixlHipEngine() {
    if (progress_.joinable()) {
        {
            std::lock_guard<std::mutex> lock(pendingMutex_);
            stopProgress_ = true;
        }
        pendingCv_.notify_all();
        progress_.join();
    }
    {
        std::lock_guard<std::mutex> lock(g_registryMutex);
        const auto it = g_registry.find(localAgent);
        if (it != g_registry.end() && it->second == this) g_registry.erase(it);
    }
    reapRetired(true);
    if (mailbox_) {
        unmapMailbox(mailbox_);
        shm_unlink(mailboxName_.c_str());
    }
    for (auto &[name, peer] : peers_)
        unmapMailbox(peer.mailbox);
    for (auto &[key, map] : ipcMaps_) {
        const DeviceScope on_device(map.device);
        (void)hipIpcCloseMemHandle(map.base);
    }
    for (const auto &[table, device] : memViews_) {
        const DeviceScope on_device(device);
        (void)hipFree(table);
    }
    for (size_t i = 0; i < streams_.size(); ++i) {
        if (!streams_[i]) continue;
        const DeviceScope on_device(static_cast<int>(i / streamsPerDevice_));
        (void)hipStreamSynchronize(streams_[i]);
        (void)hipStreamDestroy(streams_[i]);
    }
}

hipStream_t
nixlHipEngine::pickStream(int device) const {
    if (useExternalStream_) return externalStream_;
    const unsigned slot = nextStream_.fetch_add(1, std::memory_order_relaxed) % streamsPerDevice_;
    const size_t idx = static_cast<size_t>(device) * streamsPerDevice_ + slot;
    std::lock_guard<std::mutex> lock(streamsMutex_);
    if (!streams_[idx]) {
        // Default priority on purpose; non-blocking so that the legacy default stream
        // of the host application does not serialise against transfers.
        if (!hipOk(hipStreamCreateWithFlags(&streams_[idx], hipStreamNonBlocking), "hipStreamCreateWithFlags"))
            streams_[idx] = nullptr;
    }
    return streams_[idx];
}

nixl_amd_hip::WorkerPool *
nixlHipEngine::prepPool() const {
    std::call_once(prepPoolOnce_, [this] {
        try {
            prepPool_ = std::make_unique<WorkerPool>(static_cast<unsigned>(prepThreads_ - 1));
        } catch (const std::exception &e) {
            NIXL_WARN << "HIP backend: no helper threads for prepXfer (" << e.what() << ")";
        }
    });
    return prepPool_.get();
}

void
nixlHipEngine::reapRetired(bool wait) const {
    std::lock_guard<std::mutex> lock(retiredMutex_);
    size_t keep = 0;
    for (nixlHipReqH *r : retired_) {
        const nixl_status_t state = r->state(wait);
        if (state != NIXL_IN_PROG) {
            deliverPending(r, state == NIXL_SUCCESS);
            delete r;
        } else
            retired_[keep++] = r;
    }
    retired_.resize(keep);
}

nixl_status_t
nixlHipEngine::registerMem(const nixlBlobDesc &mem, const nixl_mem_t &nixl_mem, nixlBackendMD *&out) {
    out = nullptr;
    if (nixl_mem != VRAM_SEG && nixl_mem != DRAM_SEG) return NIXL_ERR_NOT_SUPPORTED;
    if (mem.len == 0 || mem.addr == 0) return NIXL_ERR_INVALID_PARAM;

    hipPointerAttribute_t attr{};
    const void *ptr = reinterpret_cast<const void *>(mem.addr);
    if (hipPointerGetAttributes(&attr, ptr) != hipSuccess) {
        (void)hipGetLastError(); // clear the sticky error left by the failed query
        NIXL_ERROR << "HIP backend: address " << mem.addr << " is not known to the HIP runtime";
        return NIXL_ERR_INVALID_PARAM;
    }

    int device = 0;
    if (nixl_mem == VRAM_SEG) {
        if (attr.type != hipMemoryTypeDevice) {
            NIXL_ERROR << "HIP backend: VRAM_SEG registration of non-device memory";
            return NIXL_ERR_INVALID_PARAM;
        }
        if (static_cast<uint64_t>(attr.device) != mem.devId) {
            NIXL_ERROR << "HIP backend: region lives on device " << attr.device << ", descriptor says "
                       << mem.devId;
            return NIXL_ERR_MISMATCH;
        }
        device = attr.device;
    } else {
        // Host memory is usable only if the runtime allocated it pinned (device-mapped);
        // pageable or merely registered host memory is refused rather than staged.
        if (attr.type != hipMemoryTypeHost) {
            NIXL_ERROR << "HIP backend: DRAM_SEG registration requires hipHostMalloc memory";
            return NIXL_ERR_NOT_SUPPORTED;
        }
        if (hipGetDevice(&device) != hipSuccess) return NIXL_ERR_BACKEND;
    }
    if (device < 0 || device >= numDevices_) return NIXL_ERR_INVALID_PARAM;

    void *base = nullptr;
    size_t size = 0;
    bool have_range = false;
    if (hipMemGetAddressRange(reinterpret_cast<hipDeviceptr_t *>(&base), &size,
                              reinterpret_cast<hipDeviceptr_t>(const_cast<void *>(ptr))) == hipSuccess) {
        const uintptr_t b = reinterpret_cast<uintptr_t>(base);
        if (mem.addr < b || mem.len > size || (mem.addr - b) > (size - mem.len)) {
            NIXL_ERROR << "HIP backend: region [" << mem.addr << ", +" << mem.len
                       << ") exceeds its allocation";
            return NIXL_ERR_INVALID_PARAM;
        }
        have_range = true;
    } else {
        (void)hipGetLastError();
        // Device memory whose allocation the runtime cannot name is not registered: nothing
        // would bound the region, and a descriptor beyond the allocation is a GPU fault.
        if (nixl_mem == VRAM_SEG) {
            NIXL_ERROR << "HIP backend: the allocation behind address " << mem.addr << " cannot be queried";
            return NIXL_ERR_INVALID_PARAM;
        }
    }

    auto *md = new nixlHipMD(mem.addr, mem.len, device, nixl_mem);
    if (nixl_mem == VRAM_SEG && have_range && size <= kMaxIpcAllocation) {
        // What an agent of another process needs to map this allocation.  A failure only means
        // that the region stays private to this process.
        const DeviceScope on_device(device);
        if (on_device.ok() && hipIpcGetMemHandle(&md->ipc, base) == hipSuccess) {
            md->hasIpc = true;
            md->allocBase = reinterpret_cast<uintptr_t>(base);
            md->allocSize = size;
        } else {
            (void)hipGetLastError();
        }
    }
    out = md;
    return NIXL_SUCCESS;
}

nixl_status_t
nixlHipEngine::deregisterMem(nixlBackendMD *meta) {
    delete static_cast<nixlHipMD *>(meta);
    return NIXL_SUCCESS;
}

// The general lowering's pass: every descriptor pair checked against its registrations and
// written out as {src, dst, len} with the direction applied.
nixl_status_t
nixlHipEngine::lowerGeneral(bool write,
                            const nixl_meta_dlist_t &local,
                            const nixl_meta_dlist_t &remote,
                            nixl_amd_copy_desc_t *lowered,
                            int &device,
                            size_t &bytes) const {
    const int n = local.descCount();
    const nixlHipMD *prev_lmd = nullptr, *prev_rmd = nullptr;
    for (int i = 0; i < n; ++i) {
        const nixlMetaDesc &l = local[i];
        const nixlMetaDesc &r = remote[i];
        if (l.len != r.len) {
            NIXL_ERROR << "HIP backend: length mismatch at descriptor " << i;
            return NIXL_ERR_INVALID_PARAM;
        }
        const auto *lmd = static_cast<const nixlHipMD *>(l.metadataP);
        const auto *rmd = static_cast<const nixlHipMD *>(r.metadataP);
        if (!lmd || !rmd || !lmd->contains(l.addr, l.len) || !rmd->contains(r.addr, r.len)) {
            NIXL_ERROR << "HIP backend: descriptor " << i << " is outside its registered region";
            return NIXL_ERR_INVALID_PARAM;
        }
        // The kernel runs on the device that owns the VRAM side(s); two VRAM regions on
        // different devices would need peer mappings, which this backend does not set up.
        // Checked once per pair of regions: consecutive descriptors mostly share theirs.
        const bool same_regions = (lmd == prev_lmd && rmd == prev_rmd);
        prev_lmd = lmd;
        prev_rmd = rmd;
        if (!same_regions) for (const nixlHipMD *md : {lmd, rmd}) {
            if (md->mem != VRAM_SEG) continue;
            if (device < 0) device = md->device;
            if (md->device != device) {
                NIXL_ERROR << "HIP backend: descriptors span devices " << device << " and " << md->device;
                return NIXL_ERR_NOT_SUPPORTED;
            }
        }
        const uintptr_t la = lmd->here(l.addr), ra = rmd->here(r.addr); // a peer's region may be mapped elsewhere here
        lowered[i].src = write ? la : ra;
        lowered[i].dst = write ? ra : la;
        lowered[i].len = l.len;
        bytes += l.len;
    }
    if (device < 0) device = static_cast<const nixlHipMD *>(local[0].metadataP)->device;
    return NIXL_SUCCESS;
}

// The block pass of prepXfer over descriptor pairs [begin, end): pair i becomes record i.
// While the two registrations do not change from one pair to the next (a pool and a staging
// buffer: never) their bounds stay in registers and the checks are accumulated without
// branches and looked at once per stretch.  A pair of several blocks (neighbours the agent
// merged) writes its first block and is noted in `merged`; a pair that is no whole number of
// blocks ends the pass (`blocks` false).  The pass also gathers what the plan wants to know
// of the records (nixl_amd_copy_record_facts_t), so that nothing reads them a second time.
struct nixlHipEngine::blockSlice {
    nixl_status_t status = NIXL_SUCCESS;
    bool blocks = true;
    int device = -1; // of the VRAM regions seen
    size_t bytes = 0;
    nixl_amd_copy_record_facts_t facts{};
    std::vector<std::pair<size_t, size_t>> merged; // {pair, blocks}
};

void
nixlHipEngine::lowerBlockSlice(bool write,
                               const nixlMetaDesc *L,
                               const nixlMetaDesc *R,
                               size_t begin,
                               size_t end,
                               size_t len0,
                               nixl_amd_copy_record_t *records,
                               blockSlice &out) const {
    uint64_t address_bits = 0;
    size_t total = 0;
    for (size_t i = begin; i < end;) {
        const auto *lmd = static_cast<const nixlHipMD *>(L[i].metadataP);
        const auto *rmd = static_cast<const nixlHipMD *>(R[i].metadataP);
        if (!lmd || !rmd) {
            NIXL_ERROR << "HIP backend: descriptor " << i << " carries no registration";
            out.status = NIXL_ERR_INVALID_PARAM;
            return;
        }
        // The kernel runs on the device that owns the VRAM side(s); two VRAM regions on
        // different devices would need peer mappings, which this backend does not set up.
        for (const nixlHipMD *md : {lmd, rmd}) {
            if (md->mem != VRAM_SEG) continue;
            if (out.device < 0) out.device = md->device;
            if (md->device != out.device) {
                NIXL_ERROR << "HIP backend: descriptors span devices " << out.device << " and " << md->device;
                out.status = NIXL_ERR_NOT_SUPPORTED;
                return;
            }
        }
        const nixlBackendMD *const lkey = L[i].metadataP, *const rkey = R[i].metadataP;
        const uintptr_t lbase = lmd->addr, rbase = rmd->addr;
        const size_t lspan = lmd->len, rspan = rmd->len;
        // a peer's region may be mapped elsewhere here; the direction decides which side is read
        const uintptr_t to_src = static_cast<uintptr_t>(write ? lmd->delta : rmd->delta);
        const uintptr_t to_dst = static_cast<uintptr_t>(write ? rmd->delta : lmd->delta);
        const size_t stretch_begin = i;
        size_t bad = 0;
        for (; i < end; ++i) {
            const nixlMetaDesc &l = L[i], &r = R[i];
            if (l.metadataP != lkey || r.metadataP != rkey) break; // other registrations: hoist again
            const size_t len = l.len;
            // inside its region on both sides (an address below the region wraps to a huge offset)
            bad |= static_cast<size_t>(len != r.len) | static_cast<size_t>(len > lspan) | static_cast<size_t>(len > rspan) |
                static_cast<size_t>(l.addr - lbase > lspan - len) | static_cast<size_t>(r.addr - rbase > rspan - len);
            const uintptr_t src = (write ? l.addr : r.addr) + to_src, dst = (write ? r.addr : l.addr) + to_dst;
            records[i] = nixl_amd_copy_record_t{src, dst};
            address_bits |= src | dst;
            total += len;
            if (len != len0) [[unlikely]] {
                const size_t k = len / len0;
                if (k == 0 || k * len0 != len) {
                    out.blocks = false;
                    return;
                }
                out.merged.emplace_back(i, k);
            }
        }
        if (bad) {
            // which one: walk the stretch again, this time with the words
            out.status = NIXL_ERR_INVALID_PARAM;
            for (size_t j = stretch_begin; j < i; ++j) {
                if (L[j].len != R[j].len) {
                    NIXL_ERROR << "HIP backend: length mismatch at descriptor " << j;
                    return;
                }
                if (!lmd->contains(L[j].addr, L[j].len) || !rmd->contains(R[j].addr, R[j].len)) {
                    NIXL_ERROR << "HIP backend: descriptor " << j << " is outside its registered region";
                    return;
                }
            }
            return;
        }
    }
    out.bytes = total;
    out.facts.address_bits = address_bits;
    // How the destinations and the sources advance decides the plan's cache policy and record
    // order by majority, so a sample answers it: the first 64 steps of every 1024 records
    // (carrying three values from pair to pair through the loop above cost it half its time
    // again).  A pair of several blocks shows up as one irregular step.
    constexpr size_t kWindow = 1024, kLook = 64;
    uint64_t regular = 0, follows = 0, steps = 0;
    for (size_t w = begin; w + 2 < end; w += kWindow) {
        const size_t last = std::min(end, w + kLook + 2);
        for (size_t i = w + 2; i < last; ++i) {
            const uintptr_t step = records[i].dst - records[i - 1].dst, before = records[i - 1].dst - records[i - 2].dst;
            regular += static_cast<uint64_t>(step == len0) | static_cast<uint64_t>(step == before);
            follows += static_cast<uint64_t>(records[i].src - records[i - 1].src == len0);
        }
        steps += last - (w + 2);
    }
    out.facts.regular_dst_steps = regular;
    out.facts.following_src_steps = follows;
    out.facts.steps = steps;
}

// Runs the block pass over the whole request: alone for short lists, with the helper threads
// for long ones (sixteen slices that the threads take as they come).  The records of pairs of
// several blocks beyond their first go behind the others: the order of records decides
// nothing about the bytes that arrive.
nixlHipEngine::blockPass
nixlHipEngine::lowerBlocks(bool write,
                           const nixl_meta_dlist_t &local,
                           const nixl_meta_dlist_t &remote,
                           nixl_amd_copy_record_t *records,
                           size_t room,
                           size_t &n_records,
                           int &device,
                           size_t &bytes,
                           nixl_amd_copy_record_facts_t &facts) const {
    const size_t n = static_cast<size_t>(local.descCount());
    const nixlMetaDesc *const L = &local[0], *const R = &remote[0];
    const size_t len0 = L[0].len;
    constexpr size_t kParallelFrom = 16384; // pairs; below that the pass is shorter than waking a helper
    constexpr unsigned kSlices = 16;
    std::vector<blockSlice> slices(1);
    bool shared = false;
    if (n >= kParallelFrom && prepThreads_ > 1) {
        WorkerPool *pool = prepPool();
        if (pool) {
            slices.assign(kSlices, blockSlice{});
            shared = pool->run(kSlices, [&](unsigned s) {
                lowerBlockSlice(write, L, R, n * s / kSlices, n * (s + 1) / kSlices, len0, records, slices[s]);
            });
            if (!shared) slices.assign(1, blockSlice{}); // the pool serves another thread's request
        }
    }
    if (!shared) lowerBlockSlice(write, L, R, 0, n, len0, records, slices[0]);

    device = -1;
    bytes = 0;
    facts = nixl_amd_copy_record_facts_t{};
    size_t made = n;
    for (const blockSlice &s : slices) {
        if (s.status != NIXL_SUCCESS) return {s.status, false};
        if (!s.blocks) return {NIXL_SUCCESS, false};
        if (s.device >= 0) {
            if (device < 0) device = s.device;
            if (s.device != device) {
                NIXL_ERROR << "HIP backend: descriptors span devices " << device << " and " << s.device;
                return {NIXL_ERR_NOT_SUPPORTED, false};
            }
        }
        bytes += s.bytes;
        facts.address_bits |= s.facts.address_bits;
        facts.regular_dst_steps += s.facts.regular_dst_steps;
        facts.following_src_steps += s.facts.following_src_steps;
        facts.steps += s.facts.steps;
        for (const auto &[pair, blocks] : s.merged) {
            if (blocks - 1 > room - made) return {NIXL_SUCCESS, false};
            for (size_t j = 1; j < blocks; ++j)
                records[made++] = nixl_amd_copy_record_t{records[pair].src + j * len0, records[pair].dst + j * len0};
        }
    }
    if (device < 0) device = static_cast<const nixlHipMD *>(L[0].metadataP)->device;
    n_records = made;
    return {NIXL_SUCCESS, true};
}

nixl_status_t
nixlHipEngine::prepXfer(const nixl_xfer_op_t &operation,
                        const nixl_meta_dlist_t &local,
                        const nixl_meta_dlist_t &remote,
                        const std::string &remote_agent,
                        nixlBackendReqH *&handle,
                        const nixl_opt_b_args_t *opt_args) const {
    handle = nullptr;
    reapRetired(false);

    if (!knowsAgent(remote_agent)) {
        NIXL_ERROR << "HIP backend: agent '" << remote_agent << "' is neither this agent ('" << localAgent
                   << "') nor a peer whose connection info was loaded";
        return NIXL_ERR_NOT_FOUND;
    }
    if (operation != NIXL_READ && operation != NIXL_WRITE) return NIXL_ERR_INVALID_PARAM;
    const int n = local.descCount();
    if (n == 0 || n != remote.descCount()) {
        NIXL_ERROR << "HIP backend: descriptor count mismatch (local " << n << ", remote "
                   << remote.descCount() << ")";
        return NIXL_ERR_INVALID_PARAM;
    }

    const auto t_start = std::chrono::steady_clock::now();
    auto req = std::make_unique<nixlHipReqH>();
    int device = -1;
    size_t bytes = 0;
    const bool write = (operation == NIXL_WRITE);
    const char *path = "general";
    auto t_pass = t_start;

    // Equal blocks (paged KV): ONE pass checks every descriptor pair against its registrations
    // and writes its {src, dst} record straight into the pinned buffer the plan is uploaded
    // from.  Anything else in the lists (mixed lengths, blocks too short or not on 128-byte
    // lines) sends the request to the general lowering below.
    if (nixl_amd_copy_block_len_fits(local[0].len, &tuning_)) {
        nixl_amd_copy_records_t *buffer = nullptr;
        nixl_amd_copy_record_t *records = nullptr;
        const size_t room = 2 * static_cast<size_t>(n); // merged neighbours become one record per block
        if (nixl_amd_copy_records_begin(room, &buffer, &records) != NIXL_AMD_OK) {
            NIXL_ERROR << "HIP backend: " << nixl_amd_last_error();
            return NIXL_ERR_BACKEND;
        }
        size_t n_records = 0;
        nixl_amd_copy_record_facts_t facts{};
        const blockPass pass = lowerBlocks(write, local, remote, records, room, n_records, device, bytes, facts);
        t_pass = std::chrono::steady_clock::now();
        if (pass.status != NIXL_SUCCESS) {
            (void)nixl_amd_copy_records_abandon(buffer);
            return pass.status;
        }
        if (!pass.blocks) {
            (void)nixl_amd_copy_records_abandon(buffer);
        } else {
            const int rc = nixl_amd_copy_plan_create_from_records(buffer, n_records, local[0].len, device, &tuning_, &facts, &req->plan);
            if (rc == NIXL_AMD_OK)
                path = "blocks";
            else if (rc != NIXL_AMD_ERR_INVALID) { // INVALID: not on 128-byte lines, say; the general lowering judges
                NIXL_ERROR << "HIP backend: " << nixl_amd_last_error();
                return NIXL_ERR_BACKEND;
            }
        }
    }
    const auto t_lowered = std::chrono::steady_clock::now();

    if (!req->plan) {
        const std::unique_ptr<nixl_amd_copy_desc_t[]> lowered(new nixl_amd_copy_desc_t[static_cast<size_t>(n)]); // not zero-filled
        device = -1;
        bytes = 0;
        const nixl_status_t st = lowerGeneral(write, local, remote, lowered.get(), device, bytes);
        if (st != NIXL_SUCCESS) return st;
        if (nixl_amd_copy_plan_create(lowered.get(), static_cast<size_t>(n), device, &tuning_, &req->plan) != NIXL_AMD_OK) {
            NIXL_ERROR << "HIP backend: " << nixl_amd_last_error();
            return NIXL_ERR_BACKEND;
        }
    }
    req->device = device;
    req->bytes = bytes;
    req->stream = pickStream(device);
    if (!req->stream && !useExternalStream_) return NIXL_ERR_BACKEND;

    const auto t_done = std::chrono::steady_clock::now();
    const auto us = [](auto from, auto to) { return std::chrono::duration<double, std::micro>(to - from).count(); };
    NIXL_DEBUG << "HIP backend: prepXfer of " << n << " descriptors (" << path << "): block pass " << us(t_start, t_pass)
               << " us, plan from records " << us(t_pass, t_lowered) << " us, rest (general lowering, event, stream) "
               << us(t_lowered, t_done) << " us";
    handle = req.release();
    return NIXL_SUCCESS;
}

nixl_status_t
nixlHipEngine::prepXferIndexed(const nixl_xfer_op_t &operation,
                               const nixlStrideDesc *local_runs,
                               size_t n_local_runs,
                               const int *local_indices,
                               const nixlStrideDesc *remote_runs,
                               size_t n_remote_runs,
                               const int *remote_indices,
                               size_t count,
                               const std::string &remote_agent,
                               nixlBackendReqH *&handle) const {
    handle = nullptr;
    if (!indexedPrep_) return NIXL_ERR_NOT_SUPPORTED; // switched off: every request comes through prepXfer
    reapRetired(false);
    if (!knowsAgent(remote_agent)) return NIXL_ERR_NOT_FOUND;
    if (operation != NIXL_READ && operation != NIXL_WRITE) return NIXL_ERR_INVALID_PARAM;
    if (!local_runs || !remote_runs || !local_indices || !remote_indices || count == 0) return NIXL_ERR_INVALID_PARAM;
    constexpr size_t kMaxRuns = 256; // what the kernels library takes a side
    if (n_local_runs == 0 || n_remote_runs == 0 || n_local_runs > kMaxRuns || n_remote_runs > kMaxRuns)
        return NIXL_ERR_NOT_SUPPORTED;

    // Every run inside its registered region, one block length and one device throughout;
    // addresses of another process's regions become the addresses they are mapped at here.
    const size_t len = local_runs[0].len;
    int device = -1;
    const nixlHipMD *first_md = nullptr;
    std::vector<nixl_amd_copy_run_t> tables[2];
    size_t flat[2] = {0, 0};
    for (int side = 0; side < 2; ++side) {
        const nixlStrideDesc *runs = side ? remote_runs : local_runs;
        const size_t n_runs = side ? n_remote_runs : n_local_runs;
        tables[side].reserve(n_runs);
        for (size_t r = 0; r < n_runs; ++r) {
            const nixlStrideDesc &run = runs[r];
            if (run.count == 0 || run.start_idx != flat[side]) return NIXL_ERR_NOT_SUPPORTED;
            if (run.len != len) return NIXL_ERR_NOT_SUPPORTED; // mixed lengths: the descriptor path judges them
            const auto *md = static_cast<const nixlHipMD *>(run.metadataP);
            // bytes from the run's first block to the end of its last, without wrapping around
            size_t span = 0;
            const bool fits = md && !__builtin_mul_overflow(run.count - 1, run.stride, &span) &&
                !__builtin_add_overflow(span, run.len, &span) && md->contains(run.addr, span);
            if (!fits) {
                NIXL_ERROR << "HIP backend: a prepared list reaches outside its registered region";
                return NIXL_ERR_INVALID_PARAM;
            }
            if (!first_md) first_md = md;
            if (md->mem == VRAM_SEG) {
                if (device < 0) device = md->device;
                if (md->device != device) return NIXL_ERR_NOT_SUPPORTED;
            }
            tables[side].push_back(nixl_amd_copy_run_t{md->here(run.addr), run.stride, flat[side], run.count});
            flat[side] += run.count;
        }
    }
    if (device < 0) device = first_md->device;
    // every index must name a block of its list: one pass over each vector
    int lmin = local_indices[0], lmax = lmin, rmin = remote_indices[0], rmax = rmin;
    for (size_t i = 1; i < count; ++i) {
        lmin = std::min(lmin, local_indices[i]);
        lmax = std::max(lmax, local_indices[i]);
        rmin = std::min(rmin, remote_indices[i]);
        rmax = std::max(rmax, remote_indices[i]);
    }
    if (lmin < 0 || static_cast<size_t>(lmax) >= flat[0] || rmin < 0 || static_cast<size_t>(rmax) >= flat[1]) {
        NIXL_ERROR << "HIP backend: index outside its prepared list";
        return NIXL_ERR_INVALID_PARAM;
    }

    const bool write = (operation == NIXL_WRITE);
    auto req = std::make_unique<nixlHipReqH>();
    req->device = device;
    req->bytes = count * len;
    const int src = write ? 0 : 1, dst = 1 - src;
    const int *index_of[2] = {local_indices, remote_indices};
    const int rc = nixl_amd_copy_plan_create_indexed_runs(tables[src].data(), tables[src].size(), index_of[src],
                                                          tables[dst].data(), tables[dst].size(), index_of[dst], count, len,
                                                          device, &tuning_, &req->plan);
    if (rc == NIXL_AMD_ERR_INVALID) return NIXL_ERR_NOT_SUPPORTED; // shape or alignment: the descriptor path handles it
    if (rc != NIXL_AMD_OK) {
        NIXL_ERROR << "HIP backend: " << nixl_amd_last_error();
        return NIXL_ERR_BACKEND;
    }
    req->stream = pickStream(device);
    if (!req->stream && !useExternalStream_) return NIXL_ERR_BACKEND;
    handle = req.release();
    return NIXL_SUCCESS;
}

nixl_status_t
nixlHipEngine::postXfer(const nixl_xfer_op_t &,
                        const nixl_meta_dlist_t &,
                        const nixl_meta_dlist_t &,
                        const std::string &remote_agent,
                        nixlBackendReqH *&handle,
                        const nixl_opt_b_args_t *opt_args) const {
    auto *req = static_cast<nixlHipReqH *>(handle);
    if (!req || !req->plan) return NIXL_ERR_INVALID_PARAM;
    const DeviceScope on_device(req->device);
    if (!on_device.ok()) return NIXL_ERR_BACKEND;
    if (req->posted) {
        const nixl_status_t earlier = req->state(false);
        if (earlier == NIXL_IN_PROG) return NIXL_ERR_REPOST_ACTIVE;
        // the notification of an earlier post that nobody polled to completion goes out first
        deliverPending(req, earlier == NIXL_SUCCESS);
    }

    if (nixl_amd_copy_plan_launch(req->plan, req->stream) != NIXL_AMD_OK) {
        NIXL_ERROR << "HIP backend: " << nixl_amd_last_error();
        return NIXL_ERR_BACKEND;
    }
    req->posted = true; // the launch recorded the plan's event behind its kernels
    if (opt_args && opt_args->hasNotif) {
        // only now: whoever sees the flag must find the event of THIS post behind it
        std::lock_guard<std::mutex> lock(pendingMutex_);
        req->notifPending = true;
        req->notifTarget = remote_agent;
        req->notifMsg = opt_args->notifMsg;
        if (progressOn_) {
            watched_.push_back(req);
            pendingCv_.notify_one();
        }
    }
    return NIXL_IN_PROG;
}

nixl_status_t
nixlHipEngine::checkXfer(nixlBackendReqH *handle) const {
    auto *req = static_cast<nixlHipReqH *>(handle);
    if (!req) return NIXL_ERR_INVALID_PARAM;
    flushBacklog();
    if (!req->posted) return NIXL_SUCCESS; // nothing outstanding
    const nixl_status_t state = req->state(false);
    // the peer learns of the transfer only after its bytes have landed
    if (state != NIXL_IN_PROG) deliverPending(req, state == NIXL_SUCCESS);
    return state;
}

nixl_status_t
nixlHipEngine::releaseReqH(nixlBackendReqH *handle) const {
    auto *req = static_cast<nixlHipReqH *>(handle);
    if (!req) return NIXL_SUCCESS;
    const nixl_status_t state = req->state(false);
    if (state == NIXL_IN_PROG) {
        // A launched kernel cannot be cancelled; keep its plan alive until it has
        // drained and free it from a later call, so that this call never blocks.
        std::lock_guard<std::mutex> lock(retiredMutex_);
        retired_.push_back(req);
        return NIXL_SUCCESS;
    }
    deliverPending(req, state == NIXL_SUCCESS);
    delete req;
    return NIXL_SUCCESS;
}

// ---- peers in this process, notifications ------------------------------------------------

bool
nixlHipEngine::knowsAgent(const std::string &name) const {
    if (name == localAgent) return true;
    std::lock_guard<std::mutex> lock(peersMutex_);
    return peers_.count(name) != 0;
}

// Takes the request off the progress thread's list and, if its copy completed, queues its
// message at the target.  The message of a copy that failed is dropped: the peer must not
// read bytes that never arrived.
void
nixlHipEngine::deliverPending(nixlHipReqH *req, bool completed) const {
    std::string target, msg;
    {
        std::lock_guard<std::mutex> lock(pendingMutex_);
        if (!req->notifPending) return;
        req->notifPending = false;
        target = req->notifTarget;
        msg = req->notifMsg;
        const auto it = std::find(watched_.begin(), watched_.end(), req);
        if (it != watched_.end()) watched_.erase(it);
    }
    if (!completed) {
        NIXL_ERROR << "HIP backend: transfer failed, notification for agent '" << target << "' dropped";
        return;
    }
    if (genNotif(target, msg) != NIXL_SUCCESS)
        NIXL_WARN << "HIP backend: notification for agent '" << target << "' could not be delivered";
}

// The progress thread: sleeps while no posted transfer carries a notification; otherwise
// polls the events of those that do and queues each message at its target once the copy has
// finished.  A request is only ever touched under pendingMutex_, and every path that deletes
// one takes it off the list first (deliverPending), under the same mutex.
void
nixlHipEngine::progressLoop() {
    const auto nap = std::chrono::microseconds(progressDelayUs_ ? progressDelayUs_ : 20);
    for (;;) {
        std::vector<std::pair<std::string, std::string>> ready;
        {
            std::unique_lock<std::mutex> lock(pendingMutex_);
            pendingCv_.wait(lock, [&] { return stopProgress_ || !watched_.empty() || backlog_.load(std::memory_order_acquire); });
            if (stopProgress_) return;
            for (size_t i = 0; i < watched_.size();) {
                nixlHipReqH *req = watched_[i];
                const nixl_status_t state = req->state(false);
                if (state == NIXL_IN_PROG) {
                    ++i;
                    continue;
                }
                req->notifPending = false;
                if (state == NIXL_SUCCESS)
                    ready.emplace_back(req->notifTarget, req->notifMsg);
                else
                    NIXL_ERROR << "HIP backend: transfer failed, notification for agent '" << req->notifTarget
                               << "' dropped";
                watched_[i] = watched_.back();
                watched_.pop_back();
            }
        }
        for (const auto &[target, msg] : ready)
            if (genNotif(target, msg) != NIXL_SUCCESS)
                NIXL_WARN << "HIP backend: notification for agent '" << target << "' could not be delivered";
        flushBacklog(); // messages that found a peer's ring full
        if (ready.empty()) std::this_thread::sleep_for(nap);
    }
}

nixl_status_t
nixlHipEngine::getConnInfo(std::string &str) const {
    str = kConnPrefix + std::to_string(static_cast<long long>(getpid())) + kConnMailbox + mailboxName_;
    return NIXL_SUCCESS;
}

nixl_status_t
nixlHipEngine::loadRemoteConnInfo(const std::string &remote_agent, const std::string &remote_conn_info) {
    const size_t n = std::strlen(kConnPrefix);
    if (remote_conn_info.compare(0, n, kConnPrefix) != 0) return NIXL_ERR_MISMATCH;
    char *end = nullptr;
    const long long pid = std::strtoll(remote_conn_info.c_str() + n, &end, 10);
    if (end == remote_conn_info.c_str() + n || std::strncmp(end, kConnMailbox, std::strlen(kConnMailbox)) != 0)
        return NIXL_ERR_MISMATCH;
    peerInfo peer;
    peer.pid = pid;
    peer.mailboxName = end + std::strlen(kConnMailbox);
    if (pid != static_cast<long long>(getpid())) {
        // An agent of another process is reached through its mailbox: without one it could
        // never be told that a transfer has landed.
        if (peer.mailboxName.empty() || peer.mailboxName[0] != '/') return NIXL_ERR_MISMATCH;
        peer.mailbox = mapMailbox(peer.mailboxName, false);
        peer.sender = nixl_amd_hip::MailboxSender(peer.mailbox);
        if (!peer.mailbox) {
            NIXL_ERROR << "HIP backend: mailbox '" << peer.mailboxName << "' of agent '" << remote_agent << "' (process " << pid
                       << ") cannot be opened";
            return NIXL_ERR_NOT_FOUND;
        }
    }
    std::lock_guard<std::mutex> lock(peersMutex_);
    const auto it = peers_.find(remote_agent);
    if (it != peers_.end()) {
        unmapMailbox(it->second.mailbox);
        it->second = peer;
    } else {
        peers_.emplace(remote_agent, peer);
    }
    return NIXL_SUCCESS;
}

nixl_status_t
nixlHipEngine::connect(const std::string &remote_agent) {
    return knowsAgent(remote_agent) ? NIXL_SUCCESS : NIXL_ERR_NOT_FOUND;
}

nixl_status_t
nixlHipEngine::disconnect(const std::string &remote_agent) {
    if (remote_agent == localAgent) return NIXL_SUCCESS;
    std::lock_guard<std::mutex> lock(peersMutex_);
    const auto it = peers_.find(remote_agent);
    if (it == peers_.end()) return NIXL_ERR_NOT_FOUND;
    unmapMailbox(it->second.mailbox);
    peers_.erase(it);
    return NIXL_SUCCESS;
}

nixl_status_t
nixlHipEngine::getPublicData(const nixlBackendMD *meta, std::string &str) const {
    const auto *md = static_cast<const nixlHipMD *>(meta);
    if (!md) return NIXL_ERR_INVALID_PARAM;
    PublicRegion region{};
    region.magic = kRegionMagic;
    region.addr = md->addr;
    region.len = md->len;
    region.pid = static_cast<int64_t>(getpid());
    region.device = md->device;
    region.mem = static_cast<int32_t>(md->mem);
    region.alloc_base = md->allocBase;
    region.alloc_size = md->allocSize;
    region.has_ipc = md->hasIpc ? 1u : 0u;
    region.ipc = md->ipc;
    str.assign(reinterpret_cast<const char *>(&region), sizeof(region));
    return NIXL_SUCCESS;
}

nixl_status_t
nixlHipEngine::loadRemoteMD(const nixlBlobDesc &input,
                            const nixl_mem_t &nixl_mem,
                            const std::string &remote_agent,
                            nixlBackendMD *&output) {
    output = nullptr;
    if (!knowsAgent(remote_agent)) return NIXL_ERR_NOT_FOUND;
    PublicRegion region{};
    if (input.metaInfo.size() != sizeof(region)) return NIXL_ERR_MISMATCH;
    std::memcpy(&region, input.metaInfo.data(), sizeof(region));
    if (region.magic != kRegionMagic) return NIXL_ERR_MISMATCH;
    if (region.addr != input.addr || region.len != input.len || region.mem != static_cast<int32_t>(nixl_mem) ||
        region.len == 0 || region.device < 0 || region.device >= numDevices_) {
        NIXL_ERROR << "HIP backend: published data of agent '" << remote_agent << "' does not match its descriptor";
        return NIXL_ERR_MISMATCH;
    }

    if (region.pid == static_cast<int64_t>(getpid())) {
        // A peer of this process: the region must be memory the runtime knows NOW, of the
        // stated kind, on the stated device, inside one allocation.  A blob that outlived its
        // registration (the peer freed the memory) would otherwise send kernels to unmapped
        // addresses.
        hipPointerAttribute_t attr{};
        const void *ptr = reinterpret_cast<const void *>(static_cast<uintptr_t>(region.addr));
        void *base = nullptr;
        size_t size = 0;
        const bool known = hipPointerGetAttributes(&attr, ptr) == hipSuccess &&
            attr.type == (nixl_mem == VRAM_SEG ? hipMemoryTypeDevice : hipMemoryTypeHost) &&
            (nixl_mem != VRAM_SEG || attr.device == region.device) &&
            hipMemGetAddressRange(reinterpret_cast<hipDeviceptr_t *>(&base), &size,
                                  reinterpret_cast<hipDeviceptr_t>(const_cast<void *>(ptr))) == hipSuccess &&
            region.len <= size && region.addr - reinterpret_cast<uintptr_t>(base) <= size - region.len;
        if (!known) {
            (void)hipGetLastError(); // a failed query leaves a sticky error behind
            NIXL_ERROR << "HIP backend: region [" << region.addr << ", +" << region.len << ") published by agent '" << remote_agent
                       << "' is not live memory of the stated kind";
            return NIXL_ERR_INVALID_PARAM;
        }
        output = new nixlHipMD(region.addr, region.len, region.device, nixl_mem, /*of_peer=*/true);
        return NIXL_SUCCESS;
    }

    // A peer of another process: map the allocation the region lies in (once per allocation).
    if (nixl_mem != VRAM_SEG || !region.has_ipc) {
        NIXL_ERROR << "HIP backend: agent '" << remote_agent << "' (process " << region.pid
                   << ") published a region that cannot be shared between processes (pinned host memory, or an allocation of 2 GiB or more)";
        return NIXL_ERR_NOT_SUPPORTED;
    }
    if (region.alloc_size == 0 || region.alloc_size > kMaxIpcAllocation || region.addr < region.alloc_base ||
        region.len > region.alloc_size || region.addr - region.alloc_base > region.alloc_size - region.len)
        return NIXL_ERR_MISMATCH;
    const std::string key = std::to_string(region.pid) + ":" + std::to_string(region.alloc_base);
    void *mapped = nullptr;
    {
        std::lock_guard<std::mutex> lock(ipcMutex_);
        auto it = ipcMaps_.find(key);
        if (it == ipcMaps_.end()) {
            const DeviceScope on_device(region.device);
            void *base = nullptr;
            if (!on_device.ok() || hipIpcOpenMemHandle(&base, region.ipc, hipIpcMemLazyEnablePeerAccess) != hipSuccess || !base) {
                (void)hipGetLastError();
                NIXL_ERROR << "HIP backend: the allocation of agent '" << remote_agent << "' (process " << region.pid
                           << ") cannot be opened; it may have been freed";
                return NIXL_ERR_INVALID_PARAM;
            }
            it = ipcMaps_.emplace(key, ipcMapping{base, region.device, 0}).first;
        }
        // What the peer says about its allocation is checked against what got mapped: the
        // region must lie inside the mapping as this process sees it.
        void *seen_base = nullptr;
        size_t seen_size = 0;
        const uint64_t offset = region.addr - region.alloc_base;
        if (hipMemGetAddressRange(reinterpret_cast<hipDeviceptr_t *>(&seen_base), &seen_size,
                                  reinterpret_cast<hipDeviceptr_t>(it->second.base)) != hipSuccess ||
            seen_base != it->second.base || region.len > seen_size || offset > seen_size - region.len) {
            (void)hipGetLastError();
            NIXL_ERROR << "HIP backend: region published by agent '" << remote_agent << "' (process " << region.pid
                       << ") does not fit the allocation it names (" << seen_size << " bytes as mapped here)";
            if (it->second.refs == 0) {
                const DeviceScope on_device(it->second.device);
                (void)hipIpcCloseMemHandle(it->second.base);
                ipcMaps_.erase(it);
            }
            return NIXL_ERR_INVALID_PARAM;
        }
        ++it->second.refs;
        mapped = it->second.base;
    }
    const intptr_t delta = static_cast<intptr_t>(reinterpret_cast<uintptr_t>(mapped)) - static_cast<intptr_t>(region.alloc_base);
    auto *md = new nixlHipMD(region.addr, region.len, region.device, nixl_mem, /*of_peer=*/true, delta);
    md->ipcKey = key;
    output = md;
    return NIXL_SUCCESS;
}

nixl_status_t
nixlHipEngine::unloadMD(nixlBackendMD *input) {
    // loadLocalMD hands out the registration itself, which deregisterMem frees
    const auto *md = static_cast<const nixlHipMD *>(input);
    if (!md || !md->ofPeer) return NIXL_SUCCESS;
    if (!md->ipcKey.empty()) {
        // Kernels of transfers still in flight may be using the mapping.
        reapRetired(true);
        std::lock_guard<std::mutex> lock(ipcMutex_);
        const auto it = ipcMaps_.find(md->ipcKey);
        if (it != ipcMaps_.end() && --it->second.refs == 0) {
            const DeviceScope on_device(it->second.device);
            (void)hipDeviceSynchronize();
            (void)hipIpcCloseMemHandle(it->second.base);
            ipcMaps_.erase(it);
        }
    }
    delete md;
    return NIXL_SUCCESS;
}

nixl_status_t
nixlHipEngine::genNotif(const std::string &remote_agent, const std::string &msg) const {
    {
        std::lock_guard<std::mutex> registry(g_registryMutex);
        const auto it = g_registry.find(remote_agent);
        if (it != g_registry.end()) {
            const nixlHipEngine *target = it->second;
            std::lock_guard<std::mutex> lock(target->notifMutex_);
            target->notifs_.emplace_back(localAgent, msg);
            return NIXL_SUCCESS;
        }
    }
    // not an engine of this process: a peer with a mailbox in shared memory
    std::lock_guard<std::mutex> lock(peersMutex_);
    const auto it = peers_.find(remote_agent);
    if (it == peers_.end() || !it->second.mailbox) return NIXL_ERR_NOT_FOUND;
    using Result = nixl_amd_hip::MailboxSender::Result;
    switch (it->second.sender.send(localAgent, msg)) {
    case Result::kSent:
        return NIXL_SUCCESS;
    case Result::kQueued: // the ring is full: the message waits here, in order, until the peer has drained some
        backlog_.store(true, std::memory_order_release);
        if (progressOn_) pendingCv_.notify_one(); // the progress thread keeps trying
        return NIXL_SUCCESS;
    case Result::kTooLong:
        NIXL_ERROR << "HIP backend: a notification to another process holds at most " << kMailboxSlotBytes
                   << " bytes (agent name included)";
        return NIXL_ERR_NOT_SUPPORTED;
    default:
        NIXL_ERROR << "HIP backend: agent '" << remote_agent << "' has not read its mailbox for "
                   << nixl_amd_hip::MailboxSender::kMaxBacklog << " notifications; it is taken to be gone";
        return NIXL_ERR_REMOTE_DISCONNECT;
    }
}

// Messages that found a peer's ring full go out as soon as the peer has made room.
void
nixlHipEngine::flushBacklog() const {
    if (!backlog_.load(std::memory_order_acquire)) return;
    std::lock_guard<std::mutex> lock(peersMutex_);
    bool left = false;
    for (auto &[name, peer] : peers_)
        if (peer.mailbox && !peer.sender.flush()) left = true;
    backlog_.store(left, std::memory_order_release);
}

nixl_status_t
nixlHipEngine::getNotifs(notif_list_t &notif_list) {
    // transfers released while in flight may have finished since
    reapRetired(false);
    flushBacklog();
    std::lock_guard<std::mutex> lock(notifMutex_);
    for (auto &n : notifs_)
        notif_list.push_back(std::move(n));
    notifs_.clear();
    if (mailbox_) {
        std::string sender, msg;
        while (mailbox_->pop(sender, msg))
            notif_list.emplace_back(std::move(sender), std::move(msg));
    }
    return NIXL_SUCCESS;
}

nixl_status_t
nixlHipEngine::queryMem(const nixl_reg_dlist_t &descs, std::vector<nixl_query_resp_t> &resp) const {
    resp.clear();
    resp.reserve(static_cast<size_t>(descs.descCount()));
    for (const nixlBlobDesc &d : descs) {
        hipPointerAttribute_t attr{};
        const void *ptr = reinterpret_cast<const void *>(d.addr);
        if (d.addr == 0 || hipPointerGetAttributes(&attr, ptr) != hipSuccess ||
            (attr.type != hipMemoryTypeDevice && attr.type != hipMemoryTypeHost)) {
            (void)hipGetLastError(); // a failed query leaves a sticky error behind
            resp.emplace_back(std::nullopt);
            continue;
        }
        nixl_b_params_t info;
        info["type"] = attr.type == hipMemoryTypeDevice ? "device" : "pinned host";
        info["device"] = std::to_string(attr.device);
        void *base = nullptr;
        size_t size = 0;
        if (hipMemGetAddressRange(reinterpret_cast<hipDeviceptr_t *>(&base), &size,
                                  reinterpret_cast<hipDeviceptr_t>(const_cast<void *>(ptr))) == hipSuccess) {
            const uintptr_t b = reinterpret_cast<uintptr_t>(base);
            info["allocation_bytes"] = std::to_string(size);
            info["fits"] = (d.addr >= b && d.len <= size && d.addr - b <= size - d.len) ? "1" : "0";
        } else {
            (void)hipGetLastError();
        }
        resp.emplace_back(std::move(info));
    }
    return NIXL_SUCCESS;
}

nixl_status_t
nixlHipEngine::estimateXferCost(const nixl_xfer_op_t &,
                                const nixl_meta_dlist_t &local,
                                const nixl_meta_dlist_t &,
                                const std::string &,
                                nixlBackendReqH *const &handle,
                                std::chrono::microseconds &duration,
                                std::chrono::microseconds &err_margin,
                                nixl_cost_t &method,
                                const nixl_opt_args_t *) const {
    size_t bytes = 0;
    if (const auto *req = static_cast<const nixlHipReqH *>(handle)) {
        bytes = req->bytes;
    } else {
        for (const auto &d : local)
            bytes += d.len;
    }
    // Read + write of every byte at a conservative 4 TB/s of HBM traffic, plus launch latency.
    const double us = 10.0 + (2.0 * static_cast<double>(bytes)) / 4.0e6;
    duration = std::chrono::microseconds(static_cast<long>(us));
    err_margin = std::chrono::microseconds(static_cast<long>(us * 0.5));
    method = nixl_cost_t::ANALYTICAL_BACKEND;
    return NIXL_SUCCESS;
}

// ---- memory views --------------------------------------------------------------------

nixl_status_t
nixlHipEngine::buildMemView(const std::vector<viewEntry> &entries, uint32_t kind, nixlMemViewH &mvh) const {
    mvh = nullptr;
    if (entries.empty()) return NIXL_ERR_INVALID_PARAM;

    std::vector<uint64_t> image(2 + 2 * entries.size());
    nixl_amd_mem_view_t head{};
    head.magic = NIXL_AMD_MEM_VIEW_MAGIC;
    head.kind = kind;
    head.count = entries.size();
    static_assert(sizeof(head) == 2 * sizeof(uint64_t) && sizeof(nixl_amd_mem_view_entry_t) == 2 * sizeof(uint64_t));
    std::memcpy(image.data(), &head, sizeof(head));

    int device = -1;
    for (size_t i = 0; i < entries.size(); ++i) {
        const viewEntry &e = entries[i];
        nixl_amd_mem_view_entry_t out{0, 0};
        if (e.md) {
            if (!e.md->contains(e.addr, e.len)) {
                NIXL_ERROR << "HIP backend: memory view entry " << i << " is outside its registered region";
                return NIXL_ERR_INVALID_PARAM;
            }
            // One table serves the kernels of one device; pinned host memory is reachable
            // from any of them.
            if (e.md->mem == VRAM_SEG) {
                if (device < 0) device = e.md->device;
                if (e.md->device != device) {
                    NIXL_ERROR << "HIP backend: memory view spans devices " << device << " and "
                               << e.md->device;
                    return NIXL_ERR_NOT_SUPPORTED;
                }
            }
            out.addr = e.md->here(e.addr);
            out.len = e.len;
        }
        std::memcpy(&image[2 + 2 * i], &out, sizeof(out));
    }
    if (device < 0 && hipGetDevice(&device) != hipSuccess) return NIXL_ERR_BACKEND;

    void *table = nullptr;
    const size_t bytes = image.size() * sizeof(uint64_t);
    const DeviceScope on_device(device);
    if (!on_device.ok() || !hipOk(hipMalloc(&table, bytes), "hipMalloc")) return NIXL_ERR_BACKEND;
    // Synchronous copy: the table is complete when the handle is handed out, whichever
    // stream the application launches its kernels on.
    if (!hipOk(hipMemcpy(table, image.data(), bytes, hipMemcpyHostToDevice), "hipMemcpy")) {
        (void)hipFree(table);
        return NIXL_ERR_BACKEND;
    }
    {
        std::lock_guard<std::mutex> lock(memViewsMutex_);
        memViews_.emplace(table, device);
    }
    mvh = table;
    return NIXL_SUCCESS;
}

nixl_status_t
nixlHipEngine::prepMemView(const nixl_meta_dlist_t &descs, nixlMemViewH &mvh, const nixl_opt_b_args_t *) const {
    std::vector<viewEntry> entries;
    entries.reserve(static_cast<size_t>(descs.descCount()));
    for (const nixlMetaDesc &d : descs) {
        const auto *md = static_cast<const nixlHipMD *>(d.metadataP);
        if (!md) return NIXL_ERR_INVALID_PARAM;
        entries.push_back({d.addr, d.len, md});
    }
    return buildMemView(entries, NIXL_AMD_MEM_VIEW_LOCAL, mvh);
}

nixl_status_t
nixlHipEngine::prepMemView(const nixl_remote_meta_dlist_t &descs,
                           nixlMemViewH &mvh,
                           const nixl_opt_b_args_t *) const {
    std::vector<viewEntry> entries;
    entries.reserve(static_cast<size_t>(descs.descCount()));
    for (const nixlRemoteMetaDesc &d : descs) {
        // A descriptor without registration data is a placeholder that keeps the indices
        // of the entries after it (the agent adds one for the null agent).
        entries.push_back({d.addr, d.len, static_cast<const nixlHipMD *>(d.metadataP)});
    }
    return buildMemView(entries, NIXL_AMD_MEM_VIEW_REMOTE, mvh);
}

void
nixlHipEngine::releaseMemView(nixlMemViewH mvh) const {
    int device = 0;
    {
        std::lock_guard<std::mutex> lock(memViewsMutex_);
        const auto it = memViews_.find(mvh);
        if (it == memViews_.end()) {
            NIXL_WARN << "HIP backend: unknown memory view handle " << mvh;
            return;
        }
        device = it->second;
        memViews_.erase(it);
    }
    // hipFree waits for the device, so a kernel still reading the table finishes first.
    const DeviceScope on_device(device);
    (void)hipFree(mvh);
}

// ---- plugin entry points -------------------------------------------------------------

using hip_plugin_t = nixlBackendPluginCreator<nixlHipEngine>;

extern "C" NIXL_PLUGIN_EXPORT nixlBackendPlugin *
nixl_plugin_init() {
    return hip_plugin_t::create(NIXL_PLUGIN_API_VERSION,
                                "HIP",
                                "0.1.0",
                                {{"units_per_lane", "0"},
                                 {"nontemporal", "0"},
                                 {"sort_scatter", "0"},
                                 {"max_workgroups", "0"},
                                 {"waves_per_workgroup", "0"},
                                 {"xcd_swizzle", "0"},
                                 {"num_streams", "1"},
                                 {"indexed_prep", "1"},
                                 {"prep_threads", "1"},
                                 {"stream", ""}},
                                {VRAM_SEG, DRAM_SEG});
}

extern "C" NIXL_PLUGIN_EXPORT void
nixl_plugin_fini() {}

// Optional entry of this plugin (not part of the reference's plugin interface): see
// nixlHipEngine::prepXferIndexed.  `engine` must be an engine this plugin created.
extern "C" NIXL_PLUGIN_EXPORT int
nixl_hip_prep_xfer_indexed(nixlBackendEngine *engine,
                           int operation,
                           const nixlStrideDesc *local_runs,
                           size_t n_local_runs,
                           const int *local_indices,
                           const nixlStrideDesc *remote_runs,
                           size_t n_remote_runs,
                           const int *remote_indices,
                           size_t count,
                           const char *remote_agent,
                           nixlBackendReqH **handle) {
    if (!engine || !local_runs || !remote_runs || !remote_agent || !handle) return NIXL_ERR_INVALID_PARAM;
    try {
        return static_cast<nixlHipEngine *>(engine)->prepXferIndexed(static_cast<nixl_xfer_op_t>(operation), local_runs,
                                                                     n_local_runs, local_indices, remote_runs, n_remote_runs,
                                                                     remote_indices, count, remote_agent, *handle);
    } catch (const std::exception &e) {
        NIXL_ERROR << "HIP backend: " << e.what();
        return NIXL_ERR_BACKEND;
    }
}
