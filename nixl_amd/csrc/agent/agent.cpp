// Single-process nixlAgent for the descriptor-transfer path.  Each public member follows
// the observable behaviour (argument checks, status codes, the sequence of south-bound
// calls a backend sees) of the reference member cited above it.
#include <dlfcn.h>

#include <algorithm>
#include <cstdlib>
#include <filesystem>
#include <mutex>

#include "agent_impl.h"
#include "serdes.h"
#include "common/nixl_log.h"

namespace fs = std::filesystem;

// =====================================================================================
// Plugin cache (reference: src/core/nixl_plugin_manager.cpp:94-122,334-359,385-399,463-529)
// =====================================================================================

nixlPluginCache &
nixlPluginCache::instance() {
    static nixlPluginCache cache;
    return cache;
}

std::vector<std::string>
nixlPluginCache::searchDirs() const {
    std::vector<std::string> dirs;
    if (const char *env = std::getenv("NIXL_PLUGIN_DIR")) {
        std::string s(env);
        size_t pos = 0;
        while (pos <= s.size()) {
            const size_t colon = s.find(':', pos);
            const std::string part = s.substr(pos, colon == std::string::npos ? std::string::npos : colon - pos);
            if (!part.empty()) dirs.push_back(part);
            if (colon == std::string::npos) break;
            pos = colon + 1;
        }
    }
    Dl_info info;
    if (dladdr(reinterpret_cast<void *>(&nixlPluginCache::instance), &info) && info.dli_fname)
        dirs.push_back((fs::path(info.dli_fname).parent_path() / "plugins").string());
    return dirs;
}

const nixlLoadedPlugin *
nixlPluginCache::load(const std::string &type) {
    std::lock_guard<std::mutex> guard(mutex_);
    const auto hit = loaded_.find(type);
    if (hit != loaded_.end()) return &hit->second;

    for (const std::string &dir : searchDirs()) {
        const fs::path path = fs::path(dir) / ("libplugin_" + type + ".so");
        std::error_code ec;
        if (!fs::exists(path, ec)) continue;
        // NODELETE: a plugin's static tables must outlive every engine it created.
        void *dl = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL | RTLD_NODELETE);
        if (!dl) {
            NIXL_WARN << "cannot load " << path.string() << ": " << dlerror();
            continue;
        }
        using init_fn = nixlBackendPlugin *(*)();
        auto init = reinterpret_cast<init_fn>(dlsym(dl, "nixl_plugin_init"));
        nixlBackendPlugin *table = init ? init() : nullptr;
        if (!table || table->api_version != NIXL_PLUGIN_API_VERSION) {
            NIXL_ERROR << path.string() << ": missing nixl_plugin_init, null table or API version mismatch";
            dlclose(dl);
            continue;
        }
        nixlLoadedPlugin &slot = loaded_[type];
        slot.dl = dl;
        slot.table = table;
        slot.path = path.string();
        return &slot;
    }
    return nullptr;
}

std::vector<std::string>
nixlPluginCache::discover() const {
    std::set<std::string> names;
    for (const std::string &dir : searchDirs()) {
        std::error_code ec;
        for (fs::directory_iterator it(dir, ec), end; !ec && it != end; it.increment(ec)) {
            const std::string f = it->path().filename().string();
            if (f.size() > 13 && f.rfind("libplugin_", 0) == 0 && f.substr(f.size() - 3) == ".so")
                names.insert(f.substr(10, f.size() - 13));
        }
    }
    return {names.begin(), names.end()};
}

// =====================================================================================
// Registered-memory sections
// =====================================================================================

void
nixlSecDescList::add(std::vector<nixlSectionDesc> batch) {
    if (batch.empty()) return;
    std::sort(batch.begin(), batch.end());
    std::vector<nixlSectionDesc> merged;
    merged.reserve(descs_.size() + batch.size());
    // Stable merge: existing entries stay ahead of equal new ones, duplicates are kept.
    std::merge(descs_.begin(), descs_.end(), batch.begin(), batch.end(), std::back_inserter(merged));
    descs_ = std::move(merged);
}

int
nixlSecDescList::indexOf(const nixlBasicDesc &query) const {
    const auto it = std::lower_bound(descs_.begin(), descs_.end(), query);
    if (it == descs_.end() || static_cast<const nixlBasicDesc &>(*it) != query) return -1;
    return static_cast<int>(it - descs_.begin());
}

int
nixlSecDescList::coveringIndex(const nixlBasicDesc &query) const {
    // First region not ordered before the query: a hit only if it starts exactly at the
    // query's address.  Otherwise the only candidate is the region just before it.
    const auto it = std::lower_bound(descs_.begin(), descs_.end(), query);
    if (it != descs_.end() && it->covers(query)) return static_cast<int>(it - descs_.begin());
    if (it != descs_.begin() && std::prev(it)->covers(query)) return static_cast<int>(it - descs_.begin()) - 1;
    return -1;
}

void
nixlSecDescList::removeAt(std::vector<size_t> indices) {
    std::sort(indices.begin(), indices.end());
    indices.erase(std::unique(indices.begin(), indices.end()), indices.end());
    size_t out = 0, next = 0;
    for (size_t i = 0; i < descs_.size(); ++i) {
        if (next < indices.size() && indices[next] == i) {
            ++next;
            continue;
        }
        if (out != i) descs_[out] = std::move(descs_[i]);
        ++out;
    }
    descs_.resize(out);
}

const std::set<nixlBackendEngine *> *
nixlMemSection::backendsFor(nixl_mem_t mem) const {
    if (mem < DRAM_SEG || mem > FILE_SEG) return nullptr;
    return &memToBackend[mem];
}

// reference: src/infra/nixl_memory_section.cpp:56-104
nixl_status_t
nixlMemSection::populate(const nixl_xfer_dlist_t &query, nixlBackendEngine *backend, nixl_meta_dlist_t &resp) const {
    if (query.getType() != resp.getType() || query.isEmpty()) return NIXL_ERR_INVALID_PARAM;
    const auto sec = sections.find({query.getType(), backend});
    if (sec == sections.end()) return NIXL_ERR_NOT_FOUND;
    const nixlSecDescList &base = sec->second;
    const int n_base = static_cast<int>(base.size());
    const int n = query.descCount();

    resp.clear();
    resp.reserve(n);
    int at = -1;
    for (int i = 0; i < n; ++i) {
        const nixlBasicDesc &q = query[i];
        if (i == 0 || q < query[i - 1]) {
            at = base.coveringIndex(q);
        } else {
            while (at < n_base && !base[at].covers(q))
                ++at;
            if (at == n_base) at = -1;
        }
        if (at < 0) {
            resp.clear();
            return NIXL_ERR_UNKNOWN;
        }
        resp.emplace(q.addr, q.len, q.devId, base[at].metadataP);
    }
    return NIXL_SUCCESS;
}

// reference: src/infra/nixl_memory_section.cpp:186-205
nixl_status_t
nixlMemSection::addElement(const nixlRemoteDesc &query,
                           nixlBackendEngine *backend,
                           nixl_remote_meta_dlist_t &resp) const {
    const auto sec = sections.find({resp.getType(), backend});
    if (sec == sections.end()) return NIXL_ERR_NOT_FOUND;
    const int at = sec->second.coveringIndex(query);
    if (at < 0) return NIXL_ERR_UNKNOWN;
    resp.addDesc(nixlRemoteMetaDesc(query.addr, query.len, query.devId, sec->second[at].metadataP));
    return NIXL_SUCCESS;
}

// reference: src/infra/nixl_memory_section.cpp:106-184
nixl_status_t
nixlMemSection::populate(const nixl_xfer_dlist_t &query,
                         nixlBackendEngine *backend,
                         nixl_stride_dlist_t &resp) const {
    if (query.getType() != resp.getType() || query.isEmpty()) return NIXL_ERR_INVALID_PARAM;
    const auto sec = sections.find({query.getType(), backend});
    if (sec == sections.end()) return NIXL_ERR_NOT_FOUND;
    const nixlSecDescList &base = sec->second;
    const int n_base = static_cast<int>(base.size());
    const int n = query.descCount();

    resp.clear();
    int at = base.coveringIndex(query[0]);
    if (at < 0) return NIXL_ERR_UNKNOWN;

    nixlStrideDesc run(query[0].addr, query[0].len, query[0].devId, base[at].metadataP, query[0].len, 1);
    uintptr_t prev = query[0].addr;
    for (int i = 1; i < n; ++i) {
        const nixlBasicDesc &q = query[i];
        if (!base[at].covers(q)) {
            if (q < query[i - 1]) {
                at = base.coveringIndex(q);
            } else {
                while (at < n_base && !base[at].covers(q))
                    ++at;
                if (at == n_base) at = -1;
            }
            if (at < 0) {
                resp.clear();
                return NIXL_ERR_UNKNOWN;
            }
        }
        nixlBackendMD *const md = base[at].metadataP;

        // A run continues while length, device and covering registration stay the same
        // and the address keeps advancing by the run's stride; the second element of a
        // run fixes that stride and must lie at a strictly higher address.
        bool extends = (q.len == run.len && q.devId == run.devId && md == run.metadataP);
        if (extends) {
            if (run.count == 1) {
                extends = q.addr > prev;
                if (extends) run.stride = q.addr - prev;
            } else {
                extends = (q.addr - prev) == run.stride;
            }
        }
        if (extends) {
            ++run.count;
        } else {
            resp.addDesc(run);
            run = nixlStrideDesc(q.addr, q.len, q.devId, md, q.len, 1);
            run.start_idx = static_cast<size_t>(i);
        }
        prev = q.addr;
    }
    resp.addDesc(run);
    return NIXL_SUCCESS;
}

// =====================================================================================
// Agent
// =====================================================================================

const std::string nixl_null_agent = "NULL_AGENT";
const std::string default_metadata_label = "metadata";

nixlAgentData::~nixlAgentData() {
    for (const auto &[view, engine] : mvhToEngine)
        engine->releaseMemView(view);
    // Peers' descriptors were loaded into the backends; hand them back
    // (reference: ~nixlRemoteSection, src/infra/nixl_memory_section.cpp:554-561).
    std::vector<std::string> peers;
    for (const auto &kv : remoteSections_)
        if (kv.first != name_) peers.push_back(kv.first);
    for (const std::string &peer : peers)
        dropRemote(peer);
    // Deregister whatever the application left registered, then destroy engines through
    // the plugin that made them (reference: src/infra/nixl_memory_section.cpp:416-423).
    for (auto &[key, list] : localSection_.sections)
        for (size_t i = 0; i < list.size(); ++i)
            key.second->deregisterMem(list[i].metadataP);
    for (auto it = engines_.rbegin(); it != engines_.rend(); ++it)
        if ((*it)->engine) (*it)->plugin->table->destroy_engine((*it)->engine);
}

nixlAgentData::engineSlot *
nixlAgentData::slotOf(const nixl_backend_t &type) const {
    for (const auto &s : engines_)
        if (s->engine->getType() == type) return s.get();
    return nullptr;
}

std::vector<nixlBackendEngine *>
nixlAgentData::backendsFor(const nixl_opt_args_t *extra, const nixlMemSection &section, nixl_mem_t mem) const {
    std::vector<nixlBackendEngine *> out;
    if (extra && !extra->backends.empty()) {
        for (const nixlBackendH *h : extra->backends)
            out.push_back(h->engine);
    } else if (const auto *avail = section.backendsFor(mem)) {
        out.assign(avail->begin(), avail->end());
    }
    return out;
}

nixlAgent::nixlAgent(const std::string &name, const nixlAgentConfig &cfg)
    : data(std::make_unique<nixlAgentData>(name, cfg)) {
    if (name.empty()) throw std::invalid_argument("Agent needs a name");
}

nixlAgent::~nixlAgent() = default;

// reference: src/core/nixl_agent.cpp:254-263
nixl_status_t
nixlAgent::getAvailPlugins(std::vector<nixl_backend_t> &plugins) {
    plugins = nixlPluginCache::instance().discover();
    return NIXL_SUCCESS;
}

// reference: src/core/nixl_agent.cpp:265-290
nixl_status_t
nixlAgent::getPluginParams(const nixl_backend_t &type, nixl_mem_list_t &mems, nixl_b_params_t &params) const {
    const nixlLoadedPlugin *p = nixlPluginCache::instance().load(type);
    if (!p) {
        NIXL_ERROR_FUNC << "plugin '" << type << "' could not be loaded";
        return NIXL_ERR_NOT_FOUND;
    }
    params = p->table->get_backend_options();
    mems = p->table->get_backend_mems();
    return NIXL_SUCCESS;
}

// reference: src/core/nixl_agent.cpp:292-315
nixl_status_t
nixlAgent::getBackendParams(const nixlBackendH *backend, nixl_mem_list_t &mems, nixl_b_params_t &params) const {
    if (!backend) return NIXL_ERR_INVALID_PARAM;
    std::shared_lock guard(data->lock);
    mems = backend->engine->getSupportedMems();
    params = backend->engine->getCustomParams();
    return NIXL_SUCCESS;
}

// reference: src/core/nixl_agent.cpp:317-426
nixl_status_t
nixlAgent::createBackend(const nixl_backend_t &type, const nixl_b_params_t &params, nixlBackendH *&backend) {
    backend = nullptr;
    std::unique_lock guard(data->lock);
    if (data->slotOf(type)) {
        NIXL_ERROR_FUNC << "backend already created for type '" << type << "'";
        return NIXL_ERR_INVALID_PARAM;
    }
    const nixlLoadedPlugin *plugin = nixlPluginCache::instance().load(type);
    if (!plugin) {
        NIXL_ERROR_FUNC << "unsupported backend '" << type << "'";
        return NIXL_ERR_NOT_FOUND;
    }

    auto slot = std::make_unique<nixlAgentData::engineSlot>();
    slot->params = params;
    slot->plugin = plugin;
    if (plugin->dl) // an optional entry some plugins export beside the two required ones
    {
        std::string symbol = "nixl_" + type + "_prep_xfer_indexed"; // e.g. nixl_hip_prep_xfer_indexed
        std::transform(symbol.begin(), symbol.end(), symbol.begin(), [](unsigned char c) { return std::tolower(c); });
        slot->prepIndexed = reinterpret_cast<nixlAgentData::prepIndexedFn>(dlsym(plugin->dl, symbol.c_str()));
    }

    nixlBackendInitParams init;
    init.localAgent = data->name_;
    init.type = type;
    init.customParams = &slot->params;
    init.enableProgTh = data->config_.useProgThread;
    init.pthrDelay = data->config_.pthrDelay;
    init.syncMode = data->config_.syncMode;
    init.enableTelemetry_ = data->config_.captureTelemetry;

    nixlBackendEngine *engine = plugin->table->create_engine(&init);
    if (!engine) {
        NIXL_ERROR_FUNC << "backend creation failed for '" << type << "'";
        return NIXL_ERR_BACKEND;
    }
    auto drop = [&](nixl_status_t st) {
        plugin->table->destroy_engine(engine);
        return st;
    };
    if (engine->getInitErr()) {
        NIXL_ERROR_FUNC << "backend initialization error for '" << type << "'";
        return drop(NIXL_ERR_BACKEND);
    }
    std::string conn;
    if (engine->supportsRemote()) {
        // A remote-capable backend must also carry notifications and connection info.
        if (!engine->supportsNotif()) return drop(NIXL_ERR_BACKEND);
        const nixl_status_t st = engine->getConnInfo(conn);
        if (st != NIXL_SUCCESS) return drop(st);
    }
    if (engine->supportsLocal()) {
        const nixl_status_t st = engine->connect(data->name_);
        if (st != NIXL_SUCCESS) {
            NIXL_ERROR_FUNC << "backend '" << type << "' failed intra-agent set-up with status " << st;
            return drop(st);
        }
    }
    if (engine->supportsRemote()) data->connMd_[type] = conn;
    if (engine->supportsNotif()) data->notifEngines.push_back(engine);
    for (nixl_mem_t m : engine->getSupportedMems())
        data->memToBackend[m].push_back(engine);

    slot->engine = engine;
    slot->handle = std::make_unique<nixlBackendH>(engine);
    backend = slot->handle.get();
    data->engines_.push_back(std::move(slot));
    return NIXL_SUCCESS;
}

namespace {

// Registers every region with one backend; all-or-nothing
// (reference: nixlLocalSection::addDescList, src/infra/nixl_memory_section.cpp:210-286).
nixl_status_t
registerWithBackend(nixlAgentData &d, const nixl_reg_dlist_t &descs, nixlBackendEngine *backend) {
    const nixl_mem_t mem = descs.getType();
    const bool local = backend->supportsLocal();
    std::vector<nixlSectionDesc> mine, self;
    nixl_status_t st = NIXL_SUCCESS;

    for (const nixlBlobDesc &region : descs) {
        nixlSectionDesc entry(region.addr, region.len, region.devId, nullptr);
        st = backend->registerMem(region, mem, entry.metadataP);
        if (st != NIXL_SUCCESS) break;
        nixlSectionDesc mirror = entry;
        if (local) {
            st = backend->loadLocalMD(entry.metadataP, mirror.metadataP);
            if (st != NIXL_SUCCESS) {
                backend->deregisterMem(entry.metadataP);
                break;
            }
        }
        if (backend->supportsRemote()) {
            // what a peer needs to address this region; travels in getLocalMD
            st = backend->getPublicData(entry.metadataP, entry.metaBlob);
            if (st != NIXL_SUCCESS) {
                if (local && mirror.metadataP != entry.metadataP) backend->unloadMD(mirror.metadataP);
                backend->deregisterMem(entry.metadataP);
                break;
            }
            mirror.metaBlob = entry.metaBlob;
        }
        mine.push_back(entry);
        if (local) self.push_back(mirror);
    }
    if (st != NIXL_SUCCESS) {
        for (size_t i = 0; i < mine.size(); ++i) {
            if (local && self[i].metadataP != mine[i].metadataP) backend->unloadMD(self[i].metadataP);
            backend->deregisterMem(mine[i].metadataP);
        }
        return st;
    }
    d.localSection_.sections[{mem, backend}].add(std::move(mine));
    d.localSection_.memToBackend[mem].insert(backend);
    if (local) {
        nixlMemSection &loop = d.remoteSections_[d.name_];
        loop.sections[{mem, backend}].add(std::move(self));
        loop.memToBackend[mem].insert(backend);
    }
    return NIXL_SUCCESS;
}

// reference: nixlLocalSection::remDescList, src/infra/nixl_memory_section.cpp:288-330
nixl_status_t
deregisterFromBackend(nixlAgentData &d, const nixl_reg_dlist_t &descs, nixlBackendEngine *backend) {
    const nixl_mem_t mem = descs.getType();
    const auto sec = d.localSection_.sections.find({mem, backend});
    if (sec == d.localSection_.sections.end()) return NIXL_ERR_NOT_FOUND;
    nixlSecDescList &mine = sec->second;

    // Nothing is deregistered unless every region is found.
    std::vector<size_t> idx;
    for (const nixlBlobDesc &region : descs) {
        const int i = mine.indexOf(region);
        if (i < 0) return NIXL_ERR_NOT_FOUND;
        idx.push_back(static_cast<size_t>(i));
    }

    if (backend->supportsLocal()) {
        const auto loop = d.remoteSections_.find(d.name_);
        if (loop != d.remoteSections_.end()) {
            const auto lsec = loop->second.sections.find({mem, backend});
            if (lsec != loop->second.sections.end()) {
                std::vector<size_t> lidx;
                for (const nixlBlobDesc &region : descs) {
                    const int i = lsec->second.indexOf(region);
                    if (i < 0) continue;
                    const int own = mine.indexOf(region);
                    if (own >= 0 && lsec->second[i].metadataP != mine[own].metadataP)
                        backend->unloadMD(lsec->second[i].metadataP);
                    lidx.push_back(static_cast<size_t>(i));
                }
                lsec->second.removeAt(std::move(lidx));
                if (lsec->second.empty()) {
                    loop->second.sections.erase(lsec);
                    loop->second.memToBackend[mem].erase(backend);
                }
            }
        }
    }
    for (size_t i : idx)
        backend->deregisterMem(mine[i].metadataP);
    mine.removeAt(std::move(idx));
    if (mine.empty()) {
        d.localSection_.sections.erase(sec);
        d.localSection_.memToBackend[mem].erase(backend);
    }
    return NIXL_SUCCESS;
}

void
carryNotif(const nixl_opt_args_t *extra, nixl_opt_b_args_t &opt) {
    if (!extra) return;
    if (extra->notif) {
        opt.notifMsg = *extra->notif;
        opt.hasNotif = true;
    } else if (extra->hasNotif) {
        opt.notifMsg = extra->notifMsg;
        opt.hasNotif = true;
    }
}

} // namespace

// reference: src/core/nixl_agent.cpp:441-506
nixl_status_t
nixlAgent::registerMem(const nixl_reg_dlist_t &descs, const nixl_opt_args_t *extra_params) {
    std::unique_lock guard(data->lock);
    std::vector<nixlBackendEngine *> targets;
    if (extra_params && !extra_params->backends.empty()) {
        for (nixlBackendH *h : extra_params->backends)
            targets.push_back(h->engine);
    } else {
        if (descs.getType() < DRAM_SEG || descs.getType() > FILE_SEG) return NIXL_ERR_INVALID_PARAM;
        targets = data->memToBackend[descs.getType()];
        if (targets.empty()) {
            NIXL_ERROR_FUNC << "no available backends for mem type '" << descs.getType() << "'";
            return NIXL_ERR_NOT_FOUND;
        }
    }
    // Best effort over the candidate backends: one success is enough.
    unsigned ok = 0;
    for (nixlBackendEngine *b : targets)
        if (registerWithBackend(*data, descs, b) == NIXL_SUCCESS) ++ok;
    if (ok) return NIXL_SUCCESS;
    NIXL_ERROR_FUNC << "registration failed for the specified or all potential backends";
    return NIXL_ERR_BACKEND;
}

// reference: src/core/nixl_agent.cpp:508-561
nixl_status_t
nixlAgent::deregisterMem(const nixl_reg_dlist_t &descs, const nixl_opt_args_t *extra_params) {
    std::unique_lock guard(data->lock);
    std::set<nixlBackendEngine *> targets;
    if (extra_params && !extra_params->backends.empty()) {
        for (nixlBackendH *h : extra_params->backends)
            targets.insert(h->engine);
    } else {
        const auto *avail = data->localSection_.backendsFor(descs.getType());
        if (!avail || avail->empty()) {
            NIXL_ERROR_FUNC << "no available backends for mem type '" << descs.getType() << "'";
            return NIXL_ERR_NOT_FOUND;
        }
        targets = *avail;
    }
    nixl_status_t bad = NIXL_SUCCESS;
    for (nixlBackendEngine *b : targets) {
        const nixl_status_t st = deregisterFromBackend(*data, descs, b);
        if (st != NIXL_SUCCESS) bad = st;
    }
    return bad;
}

// reference: src/core/nixl_agent.cpp:428-439
nixl_status_t
nixlAgent::queryMem(const nixl_reg_dlist_t &descs,
                    std::vector<nixl_query_resp_t> &resp,
                    const nixl_opt_args_t *extra_params) const {
    if (!extra_params || extra_params->backends.size() != 1) return NIXL_ERR_INVALID_PARAM;
    return extra_params->backends[0]->engine->queryMem(descs, resp);
}

// reference: src/core/nixl_agent.cpp:563-618 (only the agent itself is a known peer here)
nixl_status_t
nixlAgent::makeConnection(const std::string &remote_agent, const nixl_opt_args_t *extra_params) {
    std::unique_lock guard(data->lock);
    if (remote_agent == data->name_) {
        // the agent's own backends, as at creation
        nixl_status_t st = NIXL_ERR_BACKEND;
        for (const auto &s : data->engines_) {
            if (!s->engine->supportsLocal()) continue;
            st = s->engine->connect(remote_agent);
            if (st != NIXL_SUCCESS) return st;
        }
        return st;
    }
    const auto peer = data->remoteBackends_.find(remote_agent);
    if (peer == data->remoteBackends_.end() || peer->second.empty()) {
        NIXL_ERROR_FUNC << "metadata for remote agent '" << remote_agent << "' not found";
        return NIXL_ERR_NOT_FOUND;
    }
    std::set<nixl_backend_t> types;
    if (extra_params && !extra_params->backends.empty())
        for (const nixlBackendH *h : extra_params->backends)
            types.insert(h->getType());
    else
        for (const auto &kv : peer->second)
            types.insert(kv.first);
    int made = 0;
    for (const nixl_backend_t &type : types) {
        nixlAgentData::engineSlot *slot = data->slotOf(type);
        if (!slot) continue;
        const nixl_status_t st = slot->engine->connect(remote_agent);
        if (st != NIXL_SUCCESS) {
            NIXL_ERROR_FUNC << "connect('" << remote_agent << "') failed on backend '" << type << "' with status " << st;
            return st;
        }
        ++made;
    }
    if (made == 0) {
        NIXL_ERROR_FUNC << "no common backend to connect with '" << remote_agent << "'";
        return NIXL_ERR_BACKEND;
    }
    return NIXL_SUCCESS;
}

// reference: src/core/nixl_agent.cpp:620-687
nixl_status_t
nixlAgent::prepXferDlist(const std::string &agent_name,
                         const nixl_xfer_dlist_t &descs,
                         nixlDlistH *&dlist_hndl,
                         const nixl_opt_args_t *extra_params) const {
    dlist_hndl = nullptr;
    const bool init_side = (agent_name == NIXL_INIT_AGENT);
    std::shared_lock guard(data->lock);

    const nixlMemSection *section = &data->localSection_;
    if (!init_side) {
        const auto it = data->remoteSections_.find(agent_name);
        if (it == data->remoteSections_.end()) {
            NIXL_ERROR_FUNC << "metadata for remote agent '" << agent_name << "' not found";
            return NIXL_ERR_NOT_FOUND;
        }
        section = &it->second;
    }

    std::set<nixlBackendEngine *> candidates;
    if (extra_params && !extra_params->backends.empty()) {
        for (nixlBackendH *h : extra_params->backends)
            candidates.insert(h->engine);
    } else {
        const auto *avail = section->backendsFor(descs.getType());
        if (!avail || avail->empty()) {
            NIXL_ERROR_FUNC << "no available backends for mem type '" << descs.getType() << "'";
            return NIXL_ERR_NOT_FOUND;
        }
        candidates = *avail;
    }

    nixlDlistH::descs_t prepared;
    for (nixlBackendEngine *b : candidates) {
        nixl_stride_dlist_t runs(descs.getType());
        if (section->populate(descs, b, runs) == NIXL_SUCCESS) {
            NIXL_DEBUG << "backend " << b->getType() << ": prepared " << descs.descCount()
                       << " descriptors into " << runs.descCount() << " strides";
            prepared.try_emplace(b, std::make_unique<nixl_stride_dlist_t>(std::move(runs)));
        }
    }
    if (prepared.empty()) {
        NIXL_ERROR_FUNC << "failed to prepare the descriptors for any backend for agent '" << agent_name << "'";
        return NIXL_ERR_NOT_FOUND;
    }
    dlist_hndl = new nixlDlistH(agent_name, std::move(prepared));
    return NIXL_SUCCESS;
}

nixl_status_t
nixlAgent::prepXferDlist(const nixl_xfer_dlist_t &descs,
                         nixlDlistH *&dlist_hndl,
                         const nixl_opt_args_t *extra_params) const {
    return prepXferDlist(NIXL_INIT_AGENT, descs, dlist_hndl, extra_params);
}

// ---- pooled storage of request descriptor lists ------------------------------------------

nixlDescStoragePool &
nixlDescStoragePool::instance() {
    static nixlDescStoragePool *pool = new nixlDescStoragePool(); // never destroyed: requests may outlive static teardown
    return *pool;
}

void
nixlDescStoragePool::adopt(nixl_meta_dlist_t &list, size_t count) {
    storage_t taken;
    if (count >= kMinPooled) {
        std::lock_guard<std::mutex> guard(mutex_);
        // the smallest kept vector that is large enough
        size_t best = kept_.size();
        for (size_t i = 0; i < kept_.size(); ++i)
            if (kept_[i].capacity() >= count && (best == kept_.size() || kept_[i].capacity() < kept_[best].capacity())) best = i;
        if (best != kept_.size()) {
            taken.swap(kept_[best]);
            keptBytes_ -= taken.capacity() * sizeof(nixlMetaDesc);
            kept_.erase(kept_.begin() + static_cast<std::ptrdiff_t>(best)); // keeps the rest in order of age
        }
    }
    taken.resize(count); // shrinking costs nothing; growing a kept vector touches only its new tail
    storageOf(list).swap(taken);
}

void
nixlDescStoragePool::surrender(nixl_meta_dlist_t &list) {
    storage_t taken;
    storageOf(list).swap(taken);
    const size_t bytes = taken.capacity() * sizeof(nixlMetaDesc);
    if (taken.capacity() < kMinPooled || bytes > kMaxKeptBytes) return;
    std::vector<storage_t> dropped; // freed after the lock is gone
    std::lock_guard<std::mutex> guard(mutex_);
    // the storage just returned is the likeliest to be wanted again: the oldest make room for it
    while (!kept_.empty() && (kept_.size() >= kMaxKept || keptBytes_ + bytes > kMaxKeptBytes)) {
        keptBytes_ -= kept_.front().capacity() * sizeof(nixlMetaDesc);
        dropped.push_back(std::move(kept_.front()));
        kept_.erase(kept_.begin());
    }
    keptBytes_ += bytes;
    kept_.push_back(std::move(taken));
}

namespace {

// First position of `indices` that does not name an entry of a list of `flat` entries, or
// indices.size().  The scan has no early exit in its inner loop so that it vectorises; it is
// the only place the index vectors are checked.
size_t
firstIndexOutside(const std::vector<int> &indices, size_t flat) {
    constexpr size_t kBlock = 4096;
    const unsigned limit = flat > static_cast<size_t>(INT32_MAX) ? static_cast<unsigned>(INT32_MAX) + 1u : static_cast<unsigned>(flat);
    for (size_t b0 = 0; b0 < indices.size(); b0 += kBlock) {
        const size_t b1 = std::min(indices.size(), b0 + kBlock);
        unsigned bad = 0;
        for (size_t i = b0; i < b1; ++i)
            bad |= static_cast<unsigned>(static_cast<unsigned>(indices[i]) >= limit); // a negative index wraps to a large one
        if (bad)
            for (size_t i = b0; i < b1; ++i)
                if (static_cast<unsigned>(indices[i]) >= limit) return i;
    }
    return indices.size();
}

// Walks a prepared list by flat index.  Consecutive look-ups usually stay inside one run or
// step into the next one; any other index is looked for from a proportional first guess (run
// number = index x runs / blocks) by doubling steps and a bisection of the stretch they
// bracket.  A list that hardly compresses (runs of one block with a run of two here and there)
// made the list's own find() bisect 260 000 runs for every index: its first guess divides by
// the rounded-up mean run length.
class runCursor {
public:
    explicit runCursor(const nixl_stride_dlist_t &runs)
        : first_(runs.descCount() > 0 ? &runs[0] : nullptr),
          n_runs_(static_cast<size_t>(runs.descCount())),
          blocks_(runs.flatSize()) {}

    const nixlStrideDesc &
    at(size_t index) {
        if (run_) {
            if (index - run_->start_idx < run_->count) return *run_;
            const nixlStrideDesc *next = run_ + 1;
            if (next < first_ + n_runs_ && index - next->start_idx < next->count) return *(run_ = next);
        }
        return *(run_ = locate(index));
    }

private:
    // `index` is below blocks_ (the caller has checked the index vectors)
    const nixlStrideDesc *
    locate(size_t index) const {
        size_t at = static_cast<size_t>(static_cast<unsigned __int128>(index) * n_runs_ / blocks_);
        if (index - first_[at].start_idx < first_[at].count) return first_ + at;
        size_t lo, hi; // the run lies in [lo, hi]
        if (first_[at].start_idx > index) {
            size_t step = 1;
            hi = at - 1;
            while (step <= hi && first_[hi + 1 - step].start_idx > index)
                step <<= 1;
            lo = step <= hi ? hi + 1 - step : 0;
        } else {
            size_t step = 1;
            lo = at + 1;
            while (lo + step < n_runs_ && first_[lo + step].start_idx <= index)
                step <<= 1;
            hi = std::min(lo + step, n_runs_) - 1;
        }
        while (lo < hi) { // last run whose start_idx is at most index
            const size_t mid = (lo + hi + 1) >> 1;
            if (first_[mid].start_idx <= index)
                lo = mid;
            else
                hi = mid - 1;
        }
        return first_ + lo;
    }

    const nixlStrideDesc *const first_;
    const size_t n_runs_, blocks_;
    const nixlStrideDesc *run_ = nullptr;
};

// First backend that prepared both handles, in the caller's order of preference if one was given.
nixlBackendEngine *
commonBackend(const nixlDlistH &local_side, const nixlDlistH &remote_side, const nixl_opt_args_t *extra_params) {
    const auto both = [&](nixlBackendEngine *b) { return local_side.descs.count(b) && remote_side.descs.count(b); };
    if (extra_params && !extra_params->backends.empty()) {
        for (nixlBackendH *h : extra_params->backends)
            if (both(h->engine)) return h->engine;
        return nullptr;
    }
    for (const auto &kv : local_side.descs)
        if (both(kv.first)) return kv.first;
    return nullptr;
}

// Index pairs -> descriptor pairs (the result of src/core/nixl_agent.cpp:799-857).  With
// `merge`, a pair extends the descriptor pair before it when it advances by one on both
// sides inside the same run each and the two runs are dense with the same pitch: only then
// are the blocks adjacent in memory on both sides.  The lists get pooled storage of `count`
// entries and are filled through plain pointers (an emplace per entry cost six times the
// memory traffic's time at 65 536 pairs); they are cut to the merged count at the end.
nixl_status_t
expandIndexPairs(const nixl_stride_dlist_t &lruns,
                 const nixl_stride_dlist_t &rruns,
                 const std::vector<int> &local_indices,
                 const std::vector<int> &remote_indices,
                 bool merge,
                 nixl_meta_dlist_t &initiator,
                 nixl_meta_dlist_t &target,
                 size_t &total_bytes) {
    const size_t count = local_indices.size();
    if (const size_t at = firstIndexOutside(local_indices, lruns.flatSize()); at != count) {
        NIXL_ERROR << "makeXferReq: local index " << local_indices[at] << " (position " << at << ") is outside its list of "
                   << lruns.flatSize() << " entries";
        return NIXL_ERR_INVALID_PARAM;
    }
    if (const size_t at = firstIndexOutside(remote_indices, rruns.flatSize()); at != count) {
        NIXL_ERROR << "makeXferReq: remote index " << remote_indices[at] << " (position " << at << ") is outside its list of "
                   << rruns.flatSize() << " entries";
        return NIXL_ERR_INVALID_PARAM;
    }
    nixlDescStoragePool &pool = nixlDescStoragePool::instance();
    pool.adopt(initiator, count);
    pool.adopt(target, count);
    nixlMetaDesc *const lout = nixlDescStoragePool::data(initiator), *const rout = nixlDescStoragePool::data(target);
    const int *const lidx = local_indices.data(), *const ridx = remote_indices.data();
    runCursor lcur(lruns), rcur(rruns);
    size_t made = 0;
    total_bytes = 0;
    for (size_t i = 0; i < count;) {
        // a stretch of pairs that stays inside one run on each side
        const nixlStrideDesc &lrun = lcur.at(static_cast<size_t>(lidx[i])), &rrun = rcur.at(static_cast<size_t>(ridx[i]));
        if (lrun.len != rrun.len) {
            NIXL_ERROR << "makeXferReq: pair " << i << " joins a block of " << lrun.len << " bytes (local index " << lidx[i]
                       << ") with one of " << rrun.len << " bytes (remote index " << ridx[i] << ")";
            return NIXL_ERR_INVALID_PARAM;
        }
        const size_t len = lrun.len;
        const size_t lfirst = lrun.start_idx, lcount = lrun.count, rfirst = rrun.start_idx, rcount = rrun.count;
        const uintptr_t lbase = lrun.addr, rbase = rrun.addr;
        const size_t lstride = lrun.stride, rstride = rrun.stride;
        const uint64_t ldev = lrun.devId, rdev = rrun.devId;
        nixlBackendMD *const lmd = lrun.metadataP, *const rmd = rrun.metadataP;
        const bool adjacent = merge && lstride == len && rstride == len;
        // the stretch's first pair never extends a descriptor of another pair of runs
        size_t lprev = ~size_t{0} - 1, rprev = ~size_t{0} - 1;
        const size_t stretch_begin = i;
        for (; i < count; ++i) {
            const size_t lo = static_cast<size_t>(lidx[i]) - lfirst, ro = static_cast<size_t>(ridx[i]) - rfirst;
            if (lo >= lcount || ro >= rcount) break; // another run: look it up
            if (adjacent && lo == lprev + 1 && ro == rprev + 1) {
                lout[made - 1].len += len;
                rout[made - 1].len += len;
            } else {
                lout[made] = nixlMetaDesc(lbase + lo * lstride, len, ldev, lmd);
                rout[made] = nixlMetaDesc(rbase + ro * rstride, len, rdev, rmd);
                ++made;
            }
            lprev = lo;
            rprev = ro;
        }
        if (i == stretch_begin) return NIXL_ERR_UNKNOWN; // a run that does not hold the index it was found for
        total_bytes += (i - stretch_begin) * len;
    }
    nixlDescStoragePool::shrink(initiator, made);
    nixlDescStoragePool::shrink(target, made);
    return NIXL_SUCCESS;
}

} // namespace

// reference: src/core/nixl_agent.cpp:696-887
nixl_status_t
nixlAgent::makeXferReq(const nixl_xfer_op_t &operation,
                       const nixlDlistH *local_side,
                       const std::vector<int> &local_indices,
                       const nixlDlistH *remote_side,
                       const std::vector<int> &remote_indices,
                       nixlXferReqH *&req_hndl,
                       const nixl_opt_args_t *extra_params) const {
    req_hndl = nullptr;
    if (!local_side || !remote_side) {
        NIXL_ERROR_FUNC << "local or remote side handle is null";
        return NIXL_ERR_INVALID_PARAM;
    }
    if (!local_side->remoteAgent.empty() || remote_side->remoteAgent.empty()) {
        NIXL_ERROR_FUNC << "invalid sides (local must be local, remote must be remote)";
        return NIXL_ERR_INVALID_PARAM;
    }
    const size_t count = local_indices.size();
    if (count == 0 || count != remote_indices.size()) {
        NIXL_ERROR_FUNC << "different number of indices for local (" << count << "), remote ("
                        << remote_indices.size() << ")";
        return NIXL_ERR_INVALID_PARAM;
    }

    nixlBackendEngine *backend = commonBackend(*local_side, *remote_side, extra_params);
    if (!backend) {
        NIXL_ERROR_FUNC << "no backend has prepared both descriptor list handles";
        return NIXL_ERR_INVALID_PARAM;
    }

    nixl_opt_b_args_t opt;
    carryNotif(extra_params, opt);
    if (opt.hasNotif && !backend->supportsNotif()) {
        NIXL_ERROR_FUNC << "the selected backend '" << backend->getType() << "' does not support notifications";
        return NIXL_ERR_BACKEND;
    }

    std::shared_lock guard(data->lock);
    if (!data->remoteSections_.count(remote_side->remoteAgent)) return NIXL_ERR_NOT_FOUND;

    const nixl_stride_dlist_t &lruns = *local_side->descs.at(backend);
    const nixl_stride_dlist_t &rruns = *remote_side->descs.at(backend);
    auto req = std::make_unique<nixlXferReqH>(remote_side->remoteAgent, operation, lruns.getType(), rruns.getType());

    // Both lists a few runs each (a pool in one or several regions, a staging buffer) and a
    // backend that lowers index vectors itself: the descriptors are never written out here.
    // The request then carries no descriptor lists; its backend handle holds everything
    // postXfer needs.  Lists of many runs are cheaper to expand here than to search there.
    constexpr int kIndexedRuns = 256;
    if (lruns.descCount() >= 1 && rruns.descCount() >= 1 && lruns.descCount() <= kIndexedRuns &&
        rruns.descCount() <= kIndexedRuns) {
        const nixlAgentData::engineSlot *slot = data->slotOf(backend->getType());
        if (slot && slot->prepIndexed && slot->engine == backend) {
            const nixl_status_t st = static_cast<nixl_status_t>(
                slot->prepIndexed(backend, static_cast<int>(req->backendOp), &lruns[0], static_cast<size_t>(lruns.descCount()),
                                  local_indices.data(), &rruns[0], static_cast<size_t>(rruns.descCount()),
                                  remote_indices.data(), count, req->remoteAgent.c_str(), &req->backendHandle));
            if (st == NIXL_SUCCESS) {
                req->engine = backend;
                req->notifMsg = opt.notifMsg;
                req->hasNotif = opt.hasNotif;
                req->telemetry.totalBytes = count * lruns[0].len;
                req->telemetry.descCount = count;
                req_hndl = req.release();
                return NIXL_SUCCESS;
            }
            if (st != NIXL_ERR_NOT_SUPPORTED) {
                NIXL_ERROR_FUNC << "backend '" << backend->getType() << "' failed to prepare the indexed transfer request with status " << st;
                return st;
            }
        }
    }
    size_t total = 0;
    const auto t_expand = std::chrono::steady_clock::now();
    const nixl_status_t expanded = expandIndexPairs(lruns, rruns, local_indices, remote_indices,
                                                    !(extra_params && extra_params->skipDescMerge), req->initiatorDescs,
                                                    req->targetDescs, total);
    if (expanded != NIXL_SUCCESS) return expanded;
    NIXL_DEBUG << "makeXferReq: merged " << count << " indices into " << req->initiatorDescs.descCount() << " descriptors in "
               << std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t_expand).count() << " us";

    req->engine = backend;
    req->notifMsg = opt.notifMsg;
    req->hasNotif = opt.hasNotif;
    req->telemetry.totalBytes = total;
    req->telemetry.descCount = static_cast<size_t>(req->initiatorDescs.descCount());

    const nixl_status_t st = backend->prepXfer(req->backendOp, req->initiatorDescs, req->targetDescs,
                                               req->remoteAgent, req->backendHandle, &opt);
    if (st != NIXL_SUCCESS) {
        NIXL_ERROR_FUNC << "backend '" << backend->getType() << "' failed to prepare the transfer request with status " << st;
        return st;
    }
    req_hndl = req.release();
    return NIXL_SUCCESS;
}

// reference: src/core/nixl_agent.cpp:889-1032 (one descriptor per list entry, no merging)
nixl_status_t
nixlAgent::createXferReq(const nixl_xfer_op_t &operation,
                         const nixl_xfer_dlist_t &local_descs,
                         const nixl_xfer_dlist_t &remote_descs,
                         const std::string &remote_agent,
                         nixlXferReqH *&req_hndl,
                         const nixl_opt_args_t *extra_params) const {
    req_hndl = nullptr;
    if (local_descs.descCount() != remote_descs.descCount()) {
        NIXL_ERROR_FUNC << "different descriptor list sizes (local=" << local_descs.descCount()
                        << ", remote=" << remote_descs.descCount() << ")";
        return NIXL_ERR_INVALID_PARAM;
    }
    size_t total = 0;
    for (int i = 0; i < local_descs.descCount(); ++i) {
        if (local_descs[i].len != remote_descs[i].len) {
            NIXL_ERROR_FUNC << "length mismatch at index " << i;
            return NIXL_ERR_INVALID_PARAM;
        }
        total += local_descs[i].len;
    }

    std::shared_lock guard(data->lock);
    const auto rem = data->remoteSections_.find(remote_agent);
    if (rem == data->remoteSections_.end()) {
        NIXL_ERROR_FUNC << "metadata for remote agent '" << remote_agent << "' not found";
        return NIXL_ERR_NOT_FOUND;
    }

    std::vector<nixlBackendEngine *> candidates;
    if (extra_params && !extra_params->backends.empty()) {
        for (nixlBackendH *h : extra_params->backends)
            candidates.push_back(h->engine);
    } else {
        const auto *lset = data->localSection_.backendsFor(local_descs.getType());
        const auto *rset = rem->second.backendsFor(remote_descs.getType());
        if (!lset || !rset) return NIXL_ERR_NOT_FOUND;
        for (nixlBackendEngine *b : *lset)
            if (rset->count(b)) candidates.push_back(b);
        if (candidates.empty()) {
            NIXL_ERROR_FUNC << "no potential backend found to be able to do the transfer";
            return NIXL_ERR_NOT_FOUND;
        }
    }

    auto req = std::make_unique<nixlXferReqH>(remote_agent, operation, local_descs.getType(), remote_descs.getType());
    for (nixlBackendEngine *b : candidates) {
        const nixl_status_t s1 = data->localSection_.populate(local_descs, b, req->initiatorDescs);
        const nixl_status_t s2 = rem->second.populate(remote_descs, b, req->targetDescs);
        if (s1 == NIXL_SUCCESS && s2 == NIXL_SUCCESS) {
            req->engine = b;
            break;
        }
    }
    if (!req->engine) {
        NIXL_ERROR_FUNC << "no specified or potential backend had the required registrations";
        return NIXL_ERR_NOT_FOUND;
    }

    nixl_opt_b_args_t opt;
    carryNotif(extra_params, opt);
    if (extra_params && !extra_params->customParam.empty()) opt.customParam = extra_params->customParam;
    if (opt.hasNotif && !req->engine->supportsNotif()) {
        NIXL_ERROR_FUNC << "the selected backend '" << req->engine->getType() << "' does not support notifications";
        return NIXL_ERR_BACKEND;
    }
    req->notifMsg = opt.notifMsg;
    req->hasNotif = opt.hasNotif;
    req->telemetry.totalBytes = total;
    req->telemetry.descCount = static_cast<size_t>(req->initiatorDescs.descCount());

    const nixl_status_t st = req->engine->prepXfer(req->backendOp, req->initiatorDescs, req->targetDescs,
                                                   req->remoteAgent, req->backendHandle, &opt);
    if (st != NIXL_SUCCESS) {
        NIXL_ERROR_FUNC << "backend '" << req->engine->getType() << "' failed to prepare the transfer request with status " << st;
        return st;
    }
    req_hndl = req.release();
    return NIXL_SUCCESS;
}

// reference: src/core/nixl_agent.cpp:1034-1077
nixl_status_t
nixlAgent::estimateXferCost(const nixlXferReqH *req_hndl,
                            std::chrono::microseconds &duration,
                            std::chrono::microseconds &err_margin,
                            nixl_cost_t &method,
                            const nixl_opt_args_t *extra_params) const {
    if (!req_hndl || !req_hndl->engine) return NIXL_ERR_UNKNOWN;
    std::shared_lock guard(data->lock);
    return req_hndl->engine->estimateXferCost(req_hndl->backendOp, req_hndl->initiatorDescs, req_hndl->targetDescs,
                                              req_hndl->remoteAgent, req_hndl->backendHandle, duration, err_margin,
                                              method, extra_params);
}

// reference: src/core/nixl_agent.cpp:1079-1214
nixl_status_t
nixlAgent::postXferReq(nixlXferReqH *req_hndl, const nixl_opt_args_t *extra_params) const {
    if (!req_hndl) {
        NIXL_ERROR_FUNC << "transfer request handle is null";
        return NIXL_ERR_INVALID_PARAM;
    }
    req_hndl->telemetry.startTime = std::chrono::steady_clock::now();

    std::shared_lock guard(data->lock);
    if (!data->remoteSections_.count(req_hndl->remoteAgent)) return NIXL_ERR_NOT_FOUND;

    // A request that is still running cannot be posted again.
    if (req_hndl->status == NIXL_IN_PROG) {
        req_hndl->status = req_hndl->engine->checkXfer(req_hndl->backendHandle);
        if (req_hndl->status == NIXL_IN_PROG) {
            NIXL_ERROR_FUNC << "transfer request is still in progress and cannot be reposted";
            return NIXL_ERR_REPOST_ACTIVE;
        }
    }

    nixl_opt_b_args_t opt;
    if (req_hndl->hasNotif) {
        opt.notifMsg = req_hndl->notifMsg;
        opt.hasNotif = true;
    }
    if (extra_params) {
        nixl_opt_b_args_t fresh;
        carryNotif(extra_params, fresh);
        req_hndl->hasNotif = opt.hasNotif = fresh.hasNotif;
        if (fresh.hasNotif) req_hndl->notifMsg = opt.notifMsg = fresh.notifMsg;
    }
    if (opt.hasNotif && !req_hndl->engine->supportsNotif()) {
        NIXL_ERROR_FUNC << "the selected backend '" << req_hndl->engine->getType() << "' does not support notifications";
        return NIXL_ERR_BACKEND;
    }

    req_hndl->status = req_hndl->engine->postXfer(req_hndl->backendOp, req_hndl->initiatorDescs, req_hndl->targetDescs,
                                                  req_hndl->remoteAgent, req_hndl->backendHandle, &opt);
    req_hndl->postEnd = std::chrono::steady_clock::now();
    req_hndl->telemetry.postDuration =
        std::chrono::duration_cast<chrono_period_us_t>(req_hndl->postEnd - req_hndl->telemetry.startTime);
    if (req_hndl->status == NIXL_SUCCESS) req_hndl->telemetry.xferDuration = req_hndl->telemetry.postDuration;
    if (req_hndl->status < 0)
        NIXL_ERROR_FUNC << "backend '" << req_hndl->engine->getType() << "' failed to post the transfer request with status "
                        << req_hndl->status;
    return req_hndl->status;
}

// reference: src/core/nixl_agent.cpp:1216-1260
nixl_status_t
nixlAgent::getXferStatus(nixlXferReqH *req_hndl) const {
    if (!req_hndl) return NIXL_ERR_INVALID_PARAM;
    std::shared_lock guard(data->lock);
    // Only an in-flight request is re-checked; done or failed requests keep their status.
    if (req_hndl->status == NIXL_IN_PROG) {
        if (!data->remoteSections_.count(req_hndl->remoteAgent)) return NIXL_ERR_NOT_FOUND;
        req_hndl->status = req_hndl->engine->checkXfer(req_hndl->backendHandle);
        if (req_hndl->status == NIXL_SUCCESS)
            req_hndl->telemetry.xferDuration = std::chrono::duration_cast<chrono_period_us_t>(
                std::chrono::steady_clock::now() - req_hndl->telemetry.startTime);
        else if (req_hndl->status < 0)
            NIXL_ERROR_FUNC << "backend '" << req_hndl->engine->getType() << "' returned error status " << req_hndl->status;
    }
    return req_hndl->status;
}

// reference: src/core/nixl_agent.cpp:1262-1276
nixl_status_t
nixlAgent::getXferTelemetry(const nixlXferReqH *req_hndl, nixl_xfer_telem_t &telemetry) const {
    if (!data->config_.captureTelemetry) {
        NIXL_ERROR_FUNC << "cannot return values when telemetry is not enabled.";
        return NIXL_ERR_NO_TELEMETRY;
    }
    if (req_hndl->status != NIXL_SUCCESS) return req_hndl->status;
    telemetry = req_hndl->telemetry;
    return NIXL_SUCCESS;
}

// reference: src/core/nixl_agent.cpp:1278-1284
nixl_status_t
nixlAgent::queryXferBackend(const nixlXferReqH *req_hndl, nixlBackendH *&backend) const {
    std::shared_lock guard(data->lock);
    nixlAgentData::engineSlot *slot = data->slotOf(req_hndl->engine->getType());
    backend = slot ? slot->handle.get() : nullptr;
    return slot ? NIXL_SUCCESS : NIXL_ERR_NOT_FOUND;
}

// reference: src/core/nixl_agent.cpp:1286-1313
nixl_status_t
nixlAgent::releaseXferReq(nixlXferReqH *req_hndl) const {
    if (!req_hndl) return NIXL_ERR_INVALID_PARAM;
    std::shared_lock guard(data->lock);
    if (req_hndl->status == NIXL_IN_PROG) {
        req_hndl->status = req_hndl->engine->checkXfer(req_hndl->backendHandle);
        if (req_hndl->status == NIXL_IN_PROG) {
            // Ask the backend to abort; a backend that cannot must say so.
            req_hndl->status = req_hndl->engine->releaseReqH(req_hndl->backendHandle);
            if (req_hndl->status < 0) {
                NIXL_ERROR_FUNC << "backend '" << req_hndl->engine->getType() << "' could not release an active request";
                return NIXL_ERR_REPOST_ACTIVE;
            }
            req_hndl->backendHandle = nullptr;
        }
    }
    delete req_hndl;
    return NIXL_SUCCESS;
}

// reference: src/core/nixl_agent.cpp:1315-1320
nixl_status_t
nixlAgent::releasedDlistH(nixlDlistH *dlist_hndl) const {
    std::unique_lock guard(data->lock);
    delete dlist_hndl;
    return NIXL_SUCCESS;
}

// ---- outside the transfer path -----------------------------------------------------------

// reference: src/core/nixl_agent.cpp:1906-1976
nixl_status_t
nixlAgent::prepMemView(const nixl_remote_dlist_t &dlist,
                       nixlMemViewH &mvh,
                       const nixl_opt_args_t *extra_params) const {
    mvh = nullptr;
    const nixl_mem_t mem = dlist.getType();
    nixl_remote_meta_dlist_t resolved(mem);
    nixlBackendEngine *engine = nullptr;
    nixl_opt_b_args_t opt;
    if (extra_params) opt.customParam = extra_params->customParam;

    std::shared_lock guard(data->lock);
    for (const nixlRemoteDesc &desc : dlist) {
        if (desc.remoteAgent == nixl_null_agent) {
            resolved.addDesc(nixlRemoteMetaDesc(nixl_null_agent));
            continue;
        }
        const auto it = data->remoteSections_.find(desc.remoteAgent);
        if (it == data->remoteSections_.end()) {
            NIXL_ERROR_FUNC << "metadata for remote agent '" << desc.remoteAgent << "' not found";
            return NIXL_ERR_NOT_FOUND;
        }
        if (engine) {
            // The first resolvable descriptor fixed the engine; the rest must resolve there.
            const nixl_status_t st = it->second.addElement(desc, engine, resolved);
            if (st != NIXL_SUCCESS) return st;
            continue;
        }
        for (nixlBackendEngine *b : data->backendsFor(extra_params, it->second, mem)) {
            if (it->second.addElement(desc, b, resolved) == NIXL_SUCCESS) {
                engine = b;
                break;
            }
        }
        if (!engine) break;
    }
    if (!engine) {
        NIXL_ERROR_FUNC << "no backend can build this list of remote memory descriptors";
        return NIXL_ERR_NOT_FOUND;
    }

    const nixl_status_t st = engine->prepMemView(resolved, mvh, &opt);
    if (st == NIXL_SUCCESS) {
        std::lock_guard<std::mutex> views(data->mvhLock);
        data->mvhToEngine.emplace(mvh, engine);
    }
    return st;
}

// reference: src/core/nixl_agent.cpp:1978-2018
nixl_status_t
nixlAgent::prepMemView(const nixl_local_dlist_t &dlist,
                       nixlMemViewH &mvh,
                       const nixl_opt_args_t *extra_params) const {
    mvh = nullptr;
    const nixl_mem_t mem = dlist.getType();
    nixl_meta_dlist_t resolved(mem);
    nixlBackendEngine *engine = nullptr;
    nixl_opt_b_args_t opt;
    if (extra_params) opt.customParam = extra_params->customParam;

    std::shared_lock guard(data->lock);
    for (nixlBackendEngine *b : data->backendsFor(extra_params, data->localSection_, mem)) {
        if (data->localSection_.populate(dlist, b, resolved) == NIXL_SUCCESS) {
            engine = b;
            break;
        }
    }
    if (!engine) {
        NIXL_ERROR_FUNC << "no backend can build this list of local memory descriptors";
        return NIXL_ERR_NOT_FOUND;
    }

    const nixl_status_t st = engine->prepMemView(resolved, mvh, &opt);
    if (st == NIXL_SUCCESS) {
        std::lock_guard<std::mutex> views(data->mvhLock);
        data->mvhToEngine.emplace(mvh, engine);
    }
    return st;
}

// reference: src/core/nixl_agent.cpp:2020-2036
void
nixlAgent::releaseMemView(nixlMemViewH mvh) const {
    std::shared_lock guard(data->lock);
    nixlBackendEngine *engine = nullptr;
    {
        std::lock_guard<std::mutex> views(data->mvhLock);
        const auto it = data->mvhToEngine.find(mvh);
        if (it == data->mvhToEngine.end()) {
            NIXL_WARN << "invalid memory view handle: " << mvh;
            return;
        }
        engine = it->second;
        data->mvhToEngine.erase(it);
    }
    engine->releaseMemView(mvh);
}

// ---- notifications ------------------------------------------------------------------------

// reference: src/core/nixl_agent.cpp:1322-1380
nixl_status_t
nixlAgent::getNotifs(nixl_notifs_t &notif_map, const nixl_opt_args_t *extra_params) {
    std::unique_lock guard(data->lock);
    std::vector<nixlBackendEngine *> engines;
    if (extra_params && !extra_params->backends.empty()) {
        for (const nixlBackendH *h : extra_params->backends)
            if (h->engine->supportsNotif()) engines.push_back(h->engine);
    } else {
        engines = data->notifEngines;
    }
    if (engines.empty()) {
        NIXL_ERROR_FUNC << "no specified or potential backend supports notifications";
        return NIXL_ERR_BACKEND;
    }
    // Best effort: an error of one backend is reported, the others are still drained.
    nixl_status_t worst = NIXL_SUCCESS;
    for (nixlBackendEngine *e : engines) {
        notif_list_t fresh;
        const nixl_status_t st = e->getNotifs(fresh);
        if (st < 0) {
            NIXL_ERROR_FUNC << "backend '" << e->getType() << "' returned error status " << st
                            << " while getting notifications";
            worst = st;
        }
        for (auto &[from, msg] : fresh)
            notif_map[from].push_back(std::move(msg));
    }
    return worst;
}

// reference: src/core/nixl_agent.cpp:1382-1444
nixl_status_t
nixlAgent::genNotif(const std::string &remote_agent, const nixl_blob_t &msg, const nixl_opt_args_t *extra_params) const {
    std::shared_lock guard(data->lock);
    std::vector<nixlBackendEngine *> engines;
    if (extra_params && !extra_params->backends.empty()) {
        for (const nixlBackendH *h : extra_params->backends)
            if (h->engine->supportsNotif()) engines.push_back(h->engine);
    } else {
        engines = data->notifEngines;
    }
    if (engines.empty()) {
        NIXL_ERROR_FUNC << "no specified or potential backend supports notifications";
        return NIXL_ERR_BACKEND;
    }
    if (remote_agent == data->name_) {
        for (nixlBackendEngine *e : engines)
            if (e->supportsLocal()) return e->genNotif(remote_agent, msg);
        NIXL_ERROR_FUNC << "no specified or potential backend can send intra-agent notifications";
        return NIXL_ERR_NOT_FOUND;
    }
    const auto peer = data->remoteBackends_.find(remote_agent);
    if (peer != data->remoteBackends_.end())
        for (nixlBackendEngine *e : engines)
            if (peer->second.count(e->getType())) return e->genNotif(remote_agent, msg);
    NIXL_ERROR_FUNC << "no specified or potential backend could send the inter-agent notifications";
    return NIXL_ERR_NOT_FOUND;
}

// ---- metadata -----------------------------------------------------------------------------

namespace {

// A section list on the wire: "nixlSecElms" count, then per (memory type, backend) a "bknd"
// name and the descriptor list as a registration list whose blobs are the backends' public
// data (reference: serializeSections, src/infra/nixl_memory_section.cpp:333-363;
// nixlDescList<T>::serialize, src/infra/nixl_descriptors.cpp:236-282).
using section_pick_t = std::vector<std::pair<nixl_section_key_t, std::vector<const nixlSectionDesc *>>>;

nixl_status_t
writeSections(nixlSerDes &sd, const section_pick_t &picked) {
    const size_t count = picked.size();
    nixl_status_t st = sd.addBuf("nixlSecElms", &count, sizeof(count));
    for (const auto &[key, descs] : picked) {
        if (st != NIXL_SUCCESS) break;
        const nixl_mem_t mem = key.first;
        const size_t n = descs.size();
        st = sd.addStr("bknd", key.second->getType());
        if (st == NIXL_SUCCESS) st = sd.addStr("nixlDList", "nixlSDList");
        if (st == NIXL_SUCCESS) st = sd.addBuf("t", &mem, sizeof(mem));
        if (st == NIXL_SUCCESS) st = sd.addBuf("n", &n, sizeof(n));
        for (const nixlSectionDesc *d : descs) {
            if (st != NIXL_SUCCESS) break;
            st = sd.addStr("", static_cast<const nixlBasicDesc *>(d)->serialize() + d->metaBlob);
        }
    }
    return st;
}

// The inverse for one list (reference: nixlDescList<T>::nixlDescList(nixlSerDes *),
// src/infra/nixl_descriptors.cpp:141-190).  An empty result means a malformed list.
nixl_reg_dlist_t
readRegList(nixlSerDes &sd) {
    nixl_reg_dlist_t out(DRAM_SEG);
    if (sd.getStr("nixlDList") != "nixlSDList") return out;
    nixl_mem_t mem;
    size_t n = 0;
    if (sd.getBuf("t", &mem, sizeof(mem)) != NIXL_SUCCESS || mem < DRAM_SEG || mem > FILE_SEG) return out;
    if (sd.getBuf("n", &n, sizeof(n)) != NIXL_SUCCESS) return out;
    nixl_reg_dlist_t list(mem);
    for (size_t i = 0; i < n; ++i) {
        const std::string item = sd.getStr("");
        if (item.size() < sizeof(nixlBasicDesc)) return out;
        list.addDesc(nixlBlobDesc(item));
    }
    return list;
}

nixl_status_t
writeHeader(nixlSerDes &sd, const std::string &name, const std::vector<std::pair<nixl_backend_t, nixl_blob_t>> &conns) {
    const size_t count = conns.size();
    nixl_status_t st = sd.addStr("Agent", name);
    if (st == NIXL_SUCCESS) st = sd.addBuf("Conns", &count, sizeof(count));
    for (const auto &[type, info] : conns) {
        if (st == NIXL_SUCCESS) st = sd.addStr("t", type);
        if (st == NIXL_SUCCESS) st = sd.addStr("c", info);
    }
    if (st == NIXL_SUCCESS) st = sd.addStr("", "MemSection");
    return st;
}

} // namespace

// reference: src/core/nixl_agent.cpp:1446-1507
nixl_status_t
nixlAgent::getLocalMD(nixl_blob_t &str) const {
    std::shared_lock guard(data->lock);
    if (data->connMd_.empty()) {
        NIXL_ERROR_FUNC << "no backends support remote operations";
        return NIXL_ERR_INVALID_PARAM;
    }
    nixlSerDes sd;
    std::vector<std::pair<nixl_backend_t, nixl_blob_t>> conns(data->connMd_.begin(), data->connMd_.end());
    if (writeHeader(sd, data->name_, conns) != NIXL_SUCCESS) return NIXL_ERR_UNKNOWN;

    section_pick_t picked;
    for (const auto &[key, list] : data->localSection_.sections) {
        if (!key.second->supportsRemote()) continue;
        std::vector<const nixlSectionDesc *> descs;
        for (size_t i = 0; i < list.size(); ++i)
            descs.push_back(&list[i]);
        picked.emplace_back(key, std::move(descs));
    }
    const nixl_status_t st = writeSections(sd, picked);
    if (st != NIXL_SUCCESS) {
        NIXL_ERROR_FUNC << "serialization failed";
        return st;
    }
    str = sd.exportStr();
    return NIXL_SUCCESS;
}

// reference: src/core/nixl_agent.cpp:1509-1602, src/infra/nixl_memory_section.cpp:370-413
nixl_status_t
nixlAgent::getLocalPartialMD(const nixl_reg_dlist_t &descs, nixl_blob_t &str, const nixl_opt_args_t *extra_params) const {
    std::shared_lock guard(data->lock);
    std::vector<nixlBackendEngine *> wanted;
    if (extra_params && !extra_params->backends.empty()) {
        for (const nixlBackendH *h : extra_params->backends)
            wanted.push_back(h->engine);
    } else if (!descs.isEmpty()) {
        wanted = data->memToBackend[descs.getType()];
        if (wanted.empty()) {
            NIXL_ERROR_FUNC << "no available backends for mem type '" << descs.getType() << "'";
            return NIXL_ERR_NOT_FOUND;
        }
    } else {
        for (const auto &slot : data->engines_)
            wanted.push_back(slot->engine);
    }
    // Best effort: a backend without connection info does not support remote operation.
    std::vector<nixlBackendEngine *> selected;
    std::vector<std::pair<nixl_backend_t, nixl_blob_t>> conns;
    for (nixlBackendEngine *b : wanted) {
        const auto it = data->connMd_.find(b->getType());
        if (it == data->connMd_.end()) continue;
        selected.push_back(b);
        conns.emplace_back(it->first, it->second);
    }
    if (selected.empty() && descs.descCount() > 0) {
        NIXL_ERROR_FUNC << "no backends support the requested descriptors";
        return NIXL_ERR_BACKEND;
    }
    // Connection info travels only on request, or when no descriptors were named.
    if (!((extra_params && extra_params->includeConnInfo) || descs.descCount() == 0)) conns.clear();

    nixlSerDes sd;
    if (writeHeader(sd, data->name_, conns) != NIXL_SUCCESS) return NIXL_ERR_UNKNOWN;
    section_pick_t picked;
    if (!descs.isEmpty()) {
        for (nixlBackendEngine *b : selected) {
            const nixl_section_key_t key{descs.getType(), b};
            const auto sec = data->localSection_.sections.find(key);
            if (sec == data->localSection_.sections.end()) continue;
            std::vector<const nixlSectionDesc *> found;
            for (const nixlBlobDesc &d : descs) {
                const int i = sec->second.indexOf(d);
                if (i < 0) {
                    NIXL_ERROR_FUNC << "serialization failed";
                    return NIXL_ERR_NOT_FOUND;
                }
                found.push_back(&sec->second[static_cast<size_t>(i)]);
            }
            picked.emplace_back(key, std::move(found));
        }
    }
    const nixl_status_t st = writeSections(sd, picked);
    if (st != NIXL_SUCCESS) {
        NIXL_ERROR_FUNC << "serialization failed";
        return st;
    }
    str = sd.exportStr();
    return NIXL_SUCCESS;
}

nixl_status_t
nixlAgentData::dropRemote(const std::string &remote_name) {
    const auto sec = remoteSections_.find(remote_name);
    if (sec == remoteSections_.end()) return NIXL_ERR_NOT_FOUND;
    for (auto &[key, list] : sec->second.sections)
        for (size_t i = 0; i < list.size(); ++i)
            key.second->unloadMD(list[i].metadataP);
    remoteSections_.erase(sec);
    const auto peer = remoteBackends_.find(remote_name);
    if (peer != remoteBackends_.end()) {
        for (const auto &kv : peer->second)
            if (engineSlot *slot = slotOf(kv.first)) slot->engine->disconnect(remote_name);
        remoteBackends_.erase(peer);
    }
    return NIXL_SUCCESS;
}

// reference: src/core/nixl_agent.cpp:1604-1683 (blob), :1746-1785 (connection info),
// :1787-1799 and src/infra/nixl_memory_section.cpp:430-505 (sections)
nixl_status_t
nixlAgent::loadRemoteMD(const nixl_blob_t &remote_metadata, std::string &agent_name) {
    std::unique_lock guard(data->lock);
    nixlSerDes sd;
    if (sd.importStr(remote_metadata) != NIXL_SUCCESS) {
        NIXL_ERROR_FUNC << "failed to deserialize remote metadata";
        return NIXL_ERR_MISMATCH;
    }
    const std::string remote = sd.getStr("Agent");
    if (remote.empty()) {
        NIXL_ERROR_FUNC << "error in deserializing remote agent name";
        return NIXL_ERR_MISMATCH;
    }
    if (remote == data->name_) {
        NIXL_ERROR_FUNC << "remote agent name same as local agent, no need to load metadata";
        return NIXL_ERR_INVALID_PARAM;
    }
    size_t conn_cnt = 0;
    if (sd.getBuf("Conns", &conn_cnt, sizeof(conn_cnt)) != NIXL_SUCCESS) {
        NIXL_ERROR_FUNC << "error getting connection count";
        return NIXL_ERR_MISMATCH;
    }

    size_t usable = 0;
    for (size_t i = 0; i < conn_cnt; ++i) {
        const nixl_backend_t type = sd.getStr("t");
        const nixl_blob_t info = sd.getStr("c");
        if (type.empty() || info.empty()) {
            NIXL_ERROR_FUNC << "failed to deserialize remote metadata";
            return NIXL_ERR_MISMATCH;
        }
        nixlAgentData::engineSlot *slot = data->slotOf(type);
        if (!slot || !slot->engine->supportsRemote()) continue; // not a common backend
        auto &known = data->remoteBackends_[remote];
        const auto seen = known.find(type);
        if (seen != known.end()) {
            // the same connection info again is fine; a different one is not accepted
            if (seen->second != info) return NIXL_ERR_NOT_ALLOWED;
            ++usable;
            continue;
        }
        const nixl_status_t st = slot->engine->loadRemoteConnInfo(remote, info);
        if (st == NIXL_SUCCESS) {
            known.emplace(type, info);
            ++usable;
        } else {
            if (known.empty()) data->remoteBackends_.erase(remote);
            if (st != NIXL_ERR_NOT_SUPPORTED) {
                NIXL_ERROR_FUNC << "error loading connection info for backend '" << type << "' with status " << st;
                return st;
            }
        }
    }
    if (usable == 0 && conn_cnt > 0) {
        NIXL_ERROR_FUNC << "no common backend found";
        return NIXL_ERR_BACKEND;
    }
    if (sd.getStr("") != "MemSection") {
        NIXL_ERROR_FUNC << "failed to deserialize remote metadata";
        return NIXL_ERR_MISMATCH;
    }

    size_t sections = 0;
    nixl_status_t st = sd.getBuf("nixlSecElms", &sections, sizeof(sections));
    nixlMemSection &target = data->remoteSections_[remote];
    for (size_t i = 0; st == NIXL_SUCCESS && i < sections; ++i) {
        const nixl_backend_t type = sd.getStr("bknd");
        if (type.empty()) {
            st = NIXL_ERR_INVALID_PARAM;
            break;
        }
        const nixl_reg_dlist_t regions = readRegList(sd);
        if (regions.isEmpty()) {
            st = NIXL_ERR_NOT_FOUND;
            break;
        }
        nixlAgentData::engineSlot *slot = data->slotOf(type);
        if (!slot) continue; // a backend this agent does not have
        nixlBackendEngine *backend = slot->engine;
        if (!backend->supportsRemote()) {
            st = NIXL_ERR_UNKNOWN;
            break;
        }
        const nixl_mem_t mem = regions.getType();
        nixlSecDescList &list = target.sections[{mem, backend}];
        target.memToBackend[mem].insert(backend);
        std::vector<nixlSectionDesc> fresh;
        for (const nixlBlobDesc &region : regions) {
            const int at = list.indexOf(region);
            if (at >= 0) {
                // already known: the published data must not have changed
                if (list[static_cast<size_t>(at)].metaBlob != region.metaInfo) st = NIXL_ERR_NOT_ALLOWED;
                if (st != NIXL_SUCCESS) break;
                continue;
            }
            nixlSectionDesc entry(region.addr, region.len, region.devId, nullptr);
            st = backend->loadRemoteMD(region, mem, remote, entry.metadataP);
            if (st != NIXL_SUCCESS) break;
            entry.metaBlob = region.metaInfo;
            fresh.push_back(std::move(entry));
        }
        // what was loaded is kept in the list either way, so that a failure unloads it below
        list.add(std::move(fresh));
    }
    if (st != NIXL_SUCCESS) {
        NIXL_ERROR_FUNC << "error loading remote metadata for agent '" << remote << "' with status " << st;
        data->dropRemote(remote);
        return st;
    }
    agent_name = remote;
    return NIXL_SUCCESS;
}

// reference: src/core/nixl_agent.cpp:1801-1836
nixl_status_t
nixlAgent::invalidateRemoteMD(const std::string &remote_agent) {
    std::unique_lock guard(data->lock);
    if (remote_agent == data->name_) {
        NIXL_ERROR_FUNC << "agent '" << data->name_ << "' cannot invalidate itself";
        return NIXL_ERR_INVALID_PARAM;
    }
    return data->dropRemote(remote_agent);
}

// reference: src/core/nixl_agent.cpp:1862-1887
nixl_status_t
nixlAgent::checkRemoteMD(const std::string remote_name, const nixl_xfer_dlist_t &descs) const {
    std::shared_lock guard(data->lock);
    const auto sec = data->remoteSections_.find(remote_name);
    if (sec == data->remoteSections_.end()) return NIXL_ERR_NOT_FOUND;
    if (descs.isEmpty()) return NIXL_SUCCESS;
    const auto peer = data->remoteBackends_.find(remote_name);
    if (peer == data->remoteBackends_.end()) return NIXL_ERR_NOT_FOUND;
    nixl_meta_dlist_t scratch(descs.getType());
    for (const auto &kv : peer->second) {
        nixlAgentData::engineSlot *slot = data->slotOf(kv.first);
        if (slot && sec->second.populate(descs, slot->engine, scratch) == NIXL_SUCCESS) return NIXL_SUCCESS;
    }
    return NIXL_ERR_NOT_FOUND;
}

// ---- metadata side channels of the reference (listener thread, sockets, ETCD;
// src/core/nixl_agent.cpp:1838-1860, src/core/nixl_listener.cpp): not part of this build ----

nixl_status_t
nixlAgent::sendLocalMD(const nixl_opt_args_t *) const {
    return NIXL_ERR_NOT_SUPPORTED;
}

nixl_status_t
nixlAgent::sendLocalPartialMD(const nixl_reg_dlist_t &, const nixl_opt_args_t *) const {
    return NIXL_ERR_NOT_SUPPORTED;
}

nixl_status_t
nixlAgent::fetchRemoteMD(const std::string, const nixl_opt_args_t *) {
    return NIXL_ERR_NOT_SUPPORTED;
}

nixl_status_t
nixlAgent::invalidateLocalMD(const nixl_opt_args_t *) const {
    return NIXL_ERR_NOT_SUPPORTED;
}
