// extern "C" façade over nixlAgent (declared in include/nixl_amd_capi.h).
#include "nixl_amd_capi.h"

#include <cstdlib>
#include <cstring>
#include <exception>
#include <iterator>
#include <thread>

#include "agent_impl.h"

struct nixl_capi_agent_s {
    nixlAgent *inner;
};
struct nixl_capi_params_s {
    nixl_b_params_t params;
};
struct nixl_capi_backend_s {
    nixlBackendH *backend;
};
struct nixl_capi_opt_args_s {
    nixl_opt_args_t args;
};
struct nixl_capi_xfer_dlist_s {
    nixl_xfer_dlist_t *dlist;
};
struct nixl_capi_query_resp_list_s {
    std::vector<nixl_query_resp_t> responses;
};
struct nixl_capi_notif_map_s {
    nixl_notifs_t notifs;
};
struct nixl_capi_remote_dlist_s {
    nixl_remote_dlist_t *dlist;
};
struct nixl_capi_xfer_dlist_handle_s {
    nixlDlistH *handle;
};
struct nixl_capi_reg_dlist_s {
    nixl_reg_dlist_t *dlist;
};
struct nixl_capi_xfer_req_s {
    nixlXferReqH *req;
};
struct nixl_capi_string_list_s {
    std::vector<std::string> strings;
};
struct nixl_capi_mem_list_s {
    nixl_mem_list_t mems;
};
struct nixl_capi_param_iter_s {
    nixl_b_params_t::const_iterator it, end;
};

namespace {

thread_local int g_last_status = NIXL_SUCCESS;

// Same folding as the reference wrapper: success, in-progress, not-found and
// no-telemetry survive; every other error becomes "backend".
nixl_capi_status_t
fold(nixl_status_t st) {
    g_last_status = st;
    switch (st) {
    case NIXL_SUCCESS: return NIXL_CAPI_SUCCESS;
    case NIXL_IN_PROG: return NIXL_CAPI_IN_PROG;
    case NIXL_ERR_NOT_FOUND: return NIXL_CAPI_ERROR_NOT_FOUND;
    case NIXL_ERR_NO_TELEMETRY: return NIXL_CAPI_ERROR_NO_TELEMETRY;
    default: return NIXL_CAPI_ERROR_BACKEND;
    }
}

template<typename F>
nixl_capi_status_t
guarded(F &&f) {
    try {
        return f();
    }
    catch (const std::exception &e) {
        std::cerr << "nixl_capi: exception: " << e.what() << std::endl;
        return NIXL_CAPI_ERROR_EXCEPTION;
    }
    catch (...) {
        return NIXL_CAPI_ERROR_EXCEPTION;
    }
}

nixl_mem_t
memOf(nixl_capi_mem_type_t t) {
    return static_cast<nixl_mem_t>(t);
}

} // namespace

extern "C" {

int
nixl_capi_last_nixl_status(void) {
    return g_last_status;
}

nixl_capi_status_t
nixl_capi_create_agent(const char *name, nixl_capi_agent_t *agent) {
    if (!name || !agent) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        nixlAgentConfig cfg(true);
        *agent = new nixl_capi_agent_s{new nixlAgent(name, cfg)};
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_create_configured_agent(const char *name, const nixl_capi_agent_config_t *cfg, nixl_capi_agent_t *agent) {
    if (!name || !cfg || !agent) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        nixlAgentConfig c(cfg->enable_prog_thread,
                          cfg->enable_listen_thread,
                          static_cast<uint16_t>(cfg->listen_port),
                          static_cast<nixl_thread_sync_t>(cfg->thread_sync),
                          cfg->num_workers,
                          cfg->pthr_delay_us,
                          cfg->lthr_delay_us,
                          cfg->capture_telemetry);
        *agent = new nixl_capi_agent_s{new nixlAgent(name, c)};
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_destroy_agent(nixl_capi_agent_t agent) {
    if (!agent) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        delete agent->inner;
        delete agent;
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_create_params(nixl_capi_params_t *params) {
    if (!params) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *params = new nixl_capi_params_s{};
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_params_add(nixl_capi_params_t params, const char *key, const char *value) {
    if (!params || !key || !value) return NIXL_CAPI_ERROR_INVALID_PARAM;
    params->params[key] = value;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_destroy_params(nixl_capi_params_t params) {
    if (!params) return NIXL_CAPI_ERROR_INVALID_PARAM;
    delete params;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_create_backend(nixl_capi_agent_t agent, const char *plugin_name, nixl_capi_params_t params, nixl_capi_backend_t *backend) {
    if (!agent || !plugin_name || !backend) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        static const nixl_b_params_t none;
        nixlBackendH *h = nullptr;
        const nixl_status_t st = agent->inner->createBackend(plugin_name, params ? params->params : none, h);
        if (st != NIXL_SUCCESS) return fold(st);
        *backend = new nixl_capi_backend_s{h};
        return fold(st);
    });
}

nixl_capi_status_t
nixl_capi_destroy_backend(nixl_capi_backend_t backend) {
    if (!backend) return NIXL_CAPI_ERROR_INVALID_PARAM;
    delete backend; // the engine itself belongs to the agent
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_create_opt_args(nixl_capi_opt_args_t *args) {
    if (!args) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *args = new nixl_capi_opt_args_s{};
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_destroy_opt_args(nixl_capi_opt_args_t args) {
    if (!args) return NIXL_CAPI_ERROR_INVALID_PARAM;
    delete args;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_opt_args_add_backend(nixl_capi_opt_args_t args, nixl_capi_backend_t backend) {
    if (!args || !backend) return NIXL_CAPI_ERROR_INVALID_PARAM;
    args->args.backends.push_back(backend->backend);
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_opt_args_set_notif_msg(nixl_capi_opt_args_t args, const void *data, size_t len) {
    if (!args || (!data && len)) return NIXL_CAPI_ERROR_INVALID_PARAM;
    args->args.notifMsg.assign(static_cast<const char *>(data), len);
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_opt_args_set_has_notif(nixl_capi_opt_args_t args, bool has_notif) {
    if (!args) return NIXL_CAPI_ERROR_INVALID_PARAM;
    args->args.hasNotif = has_notif;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_opt_args_set_skip_desc_merge(nixl_capi_opt_args_t args, bool skip_merge) {
    if (!args) return NIXL_CAPI_ERROR_INVALID_PARAM;
    args->args.skipDescMerge = skip_merge;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_opt_args_set_include_conn_info(nixl_capi_opt_args_t args, bool include) {
    if (!args) return NIXL_CAPI_ERROR_INVALID_PARAM;
    args->args.includeConnInfo = include;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_create_xfer_dlist(nixl_capi_mem_type_t mem_type, nixl_capi_xfer_dlist_t *dlist) {
    if (!dlist || mem_type >= NIXL_CAPI_MEM_UNKNOWN) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *dlist = new nixl_capi_xfer_dlist_s{new nixl_xfer_dlist_t(memOf(mem_type))};
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_destroy_xfer_dlist(nixl_capi_xfer_dlist_t dlist) {
    if (!dlist) return NIXL_CAPI_ERROR_INVALID_PARAM;
    delete dlist->dlist;
    delete dlist;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_xfer_dlist_add_desc(nixl_capi_xfer_dlist_t dlist, uintptr_t addr, size_t len, uint64_t dev_id) {
    if (!dlist) return NIXL_CAPI_ERROR_INVALID_PARAM;
    dlist->dlist->addDesc(nixlBasicDesc(addr, len, dev_id));
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_xfer_dlist_add_descs(nixl_capi_xfer_dlist_t dlist,
                               const uint64_t *addrs,
                               const uint64_t *lens,
                               const uint64_t *dev_ids,
                               size_t n) {
    if (!dlist || (n && (!addrs || !lens))) return NIXL_CAPI_ERROR_INVALID_PARAM;
    dlist->dlist->reserve(static_cast<size_t>(dlist->dlist->descCount()) + n);
    for (size_t i = 0; i < n; ++i)
        dlist->dlist->emplace(static_cast<uintptr_t>(addrs[i]), static_cast<size_t>(lens[i]),
                              dev_ids ? dev_ids[i] : uint64_t{0});
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_xfer_dlist_desc_count(nixl_capi_xfer_dlist_t dlist, size_t *count) {
    if (!dlist || !count) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *count = static_cast<size_t>(dlist->dlist->descCount());
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_xfer_dlist_clear(nixl_capi_xfer_dlist_t dlist) {
    if (!dlist) return NIXL_CAPI_ERROR_INVALID_PARAM;
    dlist->dlist->clear();
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_create_reg_dlist(nixl_capi_mem_type_t mem_type, nixl_capi_reg_dlist_t *dlist) {
    if (!dlist || mem_type >= NIXL_CAPI_MEM_UNKNOWN) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *dlist = new nixl_capi_reg_dlist_s{new nixl_reg_dlist_t(memOf(mem_type))};
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_destroy_reg_dlist(nixl_capi_reg_dlist_t dlist) {
    if (!dlist) return NIXL_CAPI_ERROR_INVALID_PARAM;
    delete dlist->dlist;
    delete dlist;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_reg_dlist_add_desc(nixl_capi_reg_dlist_t dlist, uintptr_t addr, size_t len, uint64_t dev_id, const void *metadata, size_t metadata_len) {
    if (!dlist || (!metadata && metadata_len)) return NIXL_CAPI_ERROR_INVALID_PARAM;
    nixl_blob_t meta;
    if (metadata_len) meta.assign(static_cast<const char *>(metadata), metadata_len);
    dlist->dlist->addDesc(nixlBlobDesc(addr, len, dev_id, meta));
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_reg_dlist_desc_count(nixl_capi_reg_dlist_t dlist, size_t *count) {
    if (!dlist || !count) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *count = static_cast<size_t>(dlist->dlist->descCount());
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_register_mem(nixl_capi_agent_t agent, nixl_capi_reg_dlist_t dlist, nixl_capi_opt_args_t opt_args) {
    if (!agent || !dlist) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] { return fold(agent->inner->registerMem(*dlist->dlist, opt_args ? &opt_args->args : nullptr)); });
}

nixl_capi_status_t
nixl_capi_deregister_mem(nixl_capi_agent_t agent, nixl_capi_reg_dlist_t dlist, nixl_capi_opt_args_t opt_args) {
    if (!agent || !dlist) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] { return fold(agent->inner->deregisterMem(*dlist->dlist, opt_args ? &opt_args->args : nullptr)); });
}

nixl_capi_status_t
nixl_capi_prep_xfer_dlist(nixl_capi_agent_t agent, const char *agent_name, nixl_capi_xfer_dlist_t descs, nixl_capi_xfer_dlist_handle_t *dlist_hndl, nixl_capi_opt_args_t opt_args) {
    if (!agent || !agent_name || !descs || !dlist_hndl) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        nixlDlistH *h = nullptr;
        const nixl_status_t st = agent->inner->prepXferDlist(agent_name, *descs->dlist, h, opt_args ? &opt_args->args : nullptr);
        if (st != NIXL_SUCCESS) return fold(st);
        *dlist_hndl = new nixl_capi_xfer_dlist_handle_s{h};
        return fold(st);
    });
}

nixl_capi_status_t
nixl_capi_release_xfer_dlist_handle(nixl_capi_agent_t agent, nixl_capi_xfer_dlist_handle_t dlist_handle) {
    if (!agent || !dlist_handle) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        const nixl_status_t st = agent->inner->releasedDlistH(dlist_handle->handle);
        delete dlist_handle;
        return fold(st);
    });
}

nixl_capi_status_t
nixl_capi_xfer_dlist_handle_run_count(nixl_capi_xfer_dlist_handle_t h, size_t *runs) {
    if (!h || !h->handle || !runs || h->handle->descs.empty()) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *runs = static_cast<size_t>(h->handle->descs.begin()->second->descCount());
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_make_xfer_req(nixl_capi_agent_t agent,
                        nixl_capi_xfer_op_t operation,
                        nixl_capi_xfer_dlist_handle_t local_descs,
                        const int *local_indices,
                        size_t local_indices_count,
                        nixl_capi_xfer_dlist_handle_t remote_descs,
                        const int *remote_indices,
                        size_t remote_indices_count,
                        nixl_capi_xfer_req_t *req_hndl,
                        nixl_capi_opt_args_t opt_args) {
    if (!agent || !local_descs || !remote_descs || !req_hndl || (!local_indices && local_indices_count) ||
        (!remote_indices && remote_indices_count))
        return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        const std::vector<int> li(local_indices, local_indices + local_indices_count);
        const std::vector<int> ri(remote_indices, remote_indices + remote_indices_count);
        nixlXferReqH *req = nullptr;
        const nixl_status_t st = agent->inner->makeXferReq(static_cast<nixl_xfer_op_t>(operation), local_descs->handle, li,
                                                          remote_descs->handle, ri, req, opt_args ? &opt_args->args : nullptr);
        if (st != NIXL_SUCCESS) return fold(st);
        *req_hndl = new nixl_capi_xfer_req_s{req};
        return fold(st);
    });
}

nixl_capi_status_t
nixl_capi_create_xfer_req(nixl_capi_agent_t agent,
                          nixl_capi_xfer_op_t operation,
                          nixl_capi_xfer_dlist_t local_descs,
                          nixl_capi_xfer_dlist_t remote_descs,
                          const char *remote_agent,
                          nixl_capi_xfer_req_t *req_hndl,
                          nixl_capi_opt_args_t opt_args) {
    if (!agent || !local_descs || !remote_descs || !remote_agent || !req_hndl) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        nixlXferReqH *req = nullptr;
        const nixl_status_t st = agent->inner->createXferReq(static_cast<nixl_xfer_op_t>(operation), *local_descs->dlist,
                                                            *remote_descs->dlist, remote_agent, req,
                                                            opt_args ? &opt_args->args : nullptr);
        if (st != NIXL_SUCCESS) return fold(st);
        *req_hndl = new nixl_capi_xfer_req_s{req};
        return fold(st);
    });
}

nixl_capi_status_t
nixl_capi_post_xfer_req(nixl_capi_agent_t agent, nixl_capi_xfer_req_t req_hndl, nixl_capi_opt_args_t opt_args) {
    if (!agent || !req_hndl) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] { return fold(agent->inner->postXferReq(req_hndl->req, opt_args ? &opt_args->args : nullptr)); });
}

nixl_capi_status_t
nixl_capi_get_xfer_status(nixl_capi_agent_t agent, nixl_capi_xfer_req_t req_hndl) {
    if (!agent || !req_hndl) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] { return fold(agent->inner->getXferStatus(req_hndl->req)); });
}

nixl_capi_status_t
nixl_capi_post_and_wait(nixl_capi_agent_t agent, nixl_capi_xfer_req_t req_hndl) {
    if (!agent || !req_hndl) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        nixl_status_t st = agent->inner->postXferReq(req_hndl->req, nullptr);
        while (st == NIXL_IN_PROG) {
            std::this_thread::yield();
            st = agent->inner->getXferStatus(req_hndl->req);
        }
        return fold(st);
    });
}

nixl_capi_status_t
nixl_capi_get_xfer_telemetry(nixl_capi_agent_t agent, nixl_capi_xfer_req_t req_hndl, nixl_capi_xfer_telemetry_t telemetry) {
    if (!agent || !req_hndl || !telemetry) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        nixl_xfer_telem_t t{};
        const nixl_status_t st = agent->inner->getXferTelemetry(req_hndl->req, t);
        if (st != NIXL_SUCCESS) return fold(st);
        telemetry->start_time_us = static_cast<uint64_t>(
            std::chrono::duration_cast<std::chrono::microseconds>(t.startTime.time_since_epoch()).count());
        telemetry->post_duration_us = static_cast<uint64_t>(t.postDuration.count());
        telemetry->xfer_duration_us = static_cast<uint64_t>(t.xferDuration.count());
        telemetry->total_bytes = t.totalBytes;
        telemetry->desc_count = t.descCount;
        return fold(st);
    });
}

nixl_capi_status_t
nixl_capi_xfer_req_desc_count(nixl_capi_xfer_req_t req, size_t *count, size_t *bytes) {
    if (!req || !req->req) return NIXL_CAPI_ERROR_INVALID_PARAM;
    if (count) *count = req->req->telemetry.descCount;
    if (bytes) *bytes = req->req->telemetry.totalBytes;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_xfer_req_get_desc(nixl_capi_xfer_req_t req, size_t i, uint64_t *local_addr, uint64_t *remote_addr, uint64_t *len) {
    if (!req || !req->req || i >= static_cast<size_t>(req->req->initiatorDescs.descCount()))
        return NIXL_CAPI_ERROR_INVALID_PARAM;
    if (local_addr) *local_addr = req->req->initiatorDescs[i].addr;
    if (remote_addr) *remote_addr = req->req->targetDescs[i].addr;
    if (len) *len = req->req->initiatorDescs[i].len;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_release_xfer_req(nixl_capi_agent_t agent, nixl_capi_xfer_req_t req) {
    if (!agent || !req || !req->req) return NIXL_CAPI_ERROR_INVALID_PARAM; // released before: src/bindings/rust/wrapper.cpp:1590-1592
    return guarded([&] {
        const nixl_status_t st = agent->inner->releaseXferReq(req->req);
        if (st == NIXL_SUCCESS) req->req = nullptr;
        return fold(st);
    });
}

nixl_capi_status_t
nixl_capi_destroy_xfer_req(nixl_capi_xfer_req_t req) {
    if (!req) return NIXL_CAPI_ERROR_INVALID_PARAM;
    // The inner request, its device plan and its event belong to the agent until
    // nixl_capi_release_xfer_req has handed them back (src/bindings/rust/wrapper.cpp:1606-1609).
    if (req->req) return NIXL_CAPI_ERROR_INVALID_STATE;
    delete req;
    return NIXL_CAPI_SUCCESS;
}

// ---- plugin and backend queries ---------------------------------------------------------------

nixl_capi_status_t
nixl_capi_get_available_plugins(nixl_capi_agent_t agent, nixl_capi_string_list_t *plugins) {
    if (!agent || !plugins) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        std::vector<nixl_backend_t> names;
        const nixl_status_t st = agent->inner->getAvailPlugins(names);
        if (st != NIXL_SUCCESS) return fold(st);
        *plugins = new nixl_capi_string_list_s{std::move(names)};
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_destroy_string_list(nixl_capi_string_list_t list) {
    if (!list) return NIXL_CAPI_ERROR_INVALID_PARAM;
    delete list;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_string_list_size(nixl_capi_string_list_t list, size_t *size) {
    if (!list || !size) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *size = list->strings.size();
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_string_list_get(nixl_capi_string_list_t list, size_t index, const char **str) {
    if (!list || !str || index >= list->strings.size()) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *str = list->strings[index].c_str();
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_get_plugin_params(nixl_capi_agent_t agent, const char *plugin_name, nixl_capi_mem_list_t *mems,
                            nixl_capi_params_t *params) {
    if (!agent || !plugin_name || !mems || !params) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        nixl_mem_list_t m;
        nixl_b_params_t p;
        const nixl_status_t st = agent->inner->getPluginParams(plugin_name, m, p);
        if (st != NIXL_SUCCESS) return fold(st);
        *mems = new nixl_capi_mem_list_s{std::move(m)};
        *params = new nixl_capi_params_s{std::move(p)};
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_get_backend_params(nixl_capi_agent_t agent, nixl_capi_backend_t backend, nixl_capi_mem_list_t *mems,
                             nixl_capi_params_t *params) {
    if (!agent || !backend || !mems || !params) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        nixl_mem_list_t m;
        nixl_b_params_t p;
        const nixl_status_t st = agent->inner->getBackendParams(backend->backend, m, p);
        if (st != NIXL_SUCCESS) return fold(st);
        *mems = new nixl_capi_mem_list_s{std::move(m)};
        *params = new nixl_capi_params_s{std::move(p)};
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_destroy_mem_list(nixl_capi_mem_list_t list) {
    if (!list) return NIXL_CAPI_ERROR_INVALID_PARAM;
    delete list;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_mem_list_is_empty(nixl_capi_mem_list_t list, bool *is_empty) {
    if (!list || !is_empty) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *is_empty = list->mems.empty();
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_mem_list_size(nixl_capi_mem_list_t list, size_t *size) {
    if (!list || !size) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *size = list->mems.size();
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_mem_list_get(nixl_capi_mem_list_t list, size_t index, nixl_capi_mem_type_t *mem_type) {
    if (!list || !mem_type || index >= list->mems.size()) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *mem_type = static_cast<nixl_capi_mem_type_t>(list->mems[index]);
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_mem_type_to_string(nixl_capi_mem_type_t mem_type, const char **str) {
    if (!str) return NIXL_CAPI_ERROR_INVALID_PARAM;
    static const char *const names[] = {"DRAM_SEG", "VRAM_SEG", "BLK_SEG", "OBJ_SEG", "FILE_SEG"};
    if (mem_type < NIXL_CAPI_MEM_DRAM || mem_type > NIXL_CAPI_MEM_FILE) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *str = names[mem_type];
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_params_is_empty(nixl_capi_params_t params, bool *is_empty) {
    if (!params || !is_empty) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *is_empty = params->params.empty();
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_params_create_iterator(nixl_capi_params_t params, nixl_capi_param_iter_t *iter) {
    if (!params || !iter) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *iter = new nixl_capi_param_iter_s{params->params.cbegin(), params->params.cend()};
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_params_iterator_next(nixl_capi_param_iter_t iter, const char **key, const char **value, bool *has_next) {
    if (!iter || !key || !value || !has_next) return NIXL_CAPI_ERROR_INVALID_PARAM;
    if (iter->it == iter->end) {
        *has_next = false;
        return NIXL_CAPI_ERROR_INVALID_STATE;
    }
    *key = iter->it->first.c_str();
    *value = iter->it->second.c_str();
    ++iter->it;
    *has_next = iter->it != iter->end;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_params_destroy_iterator(nixl_capi_param_iter_t iter) {
    if (!iter) return NIXL_CAPI_ERROR_INVALID_PARAM;
    delete iter;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_estimate_xfer_cost(nixl_capi_agent_t agent, nixl_capi_xfer_req_t req_hndl, nixl_capi_opt_args_t opt_args,
                             int64_t *duration_us, int64_t *err_margin_us, nixl_capi_cost_t *method) {
    if (!agent || !req_hndl || !duration_us || !err_margin_us || !method) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        std::chrono::microseconds duration{0}, margin{0};
        nixl_cost_t how = nixl_cost_t::ANALYTICAL_BACKEND;
        const nixl_status_t st =
            agent->inner->estimateXferCost(req_hndl->req, duration, margin, how, opt_args ? &opt_args->args : nullptr);
        if (st != NIXL_SUCCESS) return fold(st);
        *duration_us = duration.count();
        *err_margin_us = margin.count();
        *method = static_cast<nixl_capi_cost_t>(how);
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_query_xfer_backend(nixl_capi_agent_t agent, nixl_capi_xfer_req_t req_hndl, nixl_capi_backend_t *backend) {
    if (!agent || !req_hndl || !backend) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        nixlBackendH *b = nullptr;
        const nixl_status_t st = agent->inner->queryXferBackend(req_hndl->req, b);
        if (st != NIXL_SUCCESS) return fold(st);
        *backend = new nixl_capi_backend_s{b};
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_backend_get_type(nixl_capi_backend_t backend, const char **type) {
    if (!backend || !backend->backend || !type) return NIXL_CAPI_ERROR_INVALID_PARAM;
    thread_local std::string name;
    name = backend->backend->getType();
    *type = name.c_str();
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_prep_mem_view_local(nixl_capi_agent_t agent, nixl_capi_xfer_dlist_t descs, nixl_capi_mem_view_t *mvh,
                              nixl_capi_opt_args_t opt_args) {
    if (!agent || !descs || !mvh) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        nixlMemViewH view = nullptr;
        const nixl_status_t st = agent->inner->prepMemView(*descs->dlist, view, opt_args ? &opt_args->args : nullptr);
        if (st != NIXL_SUCCESS) return fold(st);
        *mvh = static_cast<nixl_capi_mem_view_t>(view);
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_prep_mem_view_remote(nixl_capi_agent_t agent, nixl_capi_remote_dlist_t descs, nixl_capi_mem_view_t *mvh,
                               nixl_capi_opt_args_t opt_args) {
    if (!agent || !descs || !mvh) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        nixlMemViewH view = nullptr;
        const nixl_status_t st = agent->inner->prepMemView(*descs->dlist, view, opt_args ? &opt_args->args : nullptr);
        if (st != NIXL_SUCCESS) return fold(st);
        *mvh = static_cast<nixl_capi_mem_view_t>(view);
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_create_remote_dlist(nixl_capi_mem_type_t mem_type, nixl_capi_remote_dlist_t *dlist) {
    if (!dlist) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        *dlist = new nixl_capi_remote_dlist_s{new nixl_remote_dlist_t(memOf(mem_type))};
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_destroy_remote_dlist(nixl_capi_remote_dlist_t dlist) {
    if (!dlist) return NIXL_CAPI_ERROR_INVALID_PARAM;
    delete dlist->dlist;
    delete dlist;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_remote_dlist_add_desc(nixl_capi_remote_dlist_t dlist, uintptr_t addr, size_t len, uint64_t dev_id,
                                const char *remote_agent) {
    if (!dlist) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        dlist->dlist->addDesc(nixlRemoteDesc(addr, len, dev_id, remote_agent ? remote_agent : nixl_null_agent));
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_release_mem_view(nixl_capi_agent_t agent, nixl_capi_mem_view_t mvh) {
    if (!agent || !mvh) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        agent->inner->releaseMemView(static_cast<nixlMemViewH>(mvh));
        return NIXL_CAPI_SUCCESS;
    });
}

namespace {

nixl_capi_status_t
copyOut(const std::string &blob, void **data, size_t *len) {
    void *copy = std::malloc(blob.size() ? blob.size() : 1);
    if (!copy) return NIXL_CAPI_ERROR_BACKEND;
    std::memcpy(copy, blob.data(), blob.size());
    *data = copy;
    *len = blob.size();
    return NIXL_CAPI_SUCCESS;
}

} // namespace

nixl_capi_status_t
nixl_capi_get_local_md(nixl_capi_agent_t agent, void **data, size_t *len) {
    if (!agent || !data || !len) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        nixl_blob_t blob;
        const nixl_status_t st = agent->inner->getLocalMD(blob);
        if (st != NIXL_SUCCESS) return fold(st);
        return copyOut(blob, data, len);
    });
}

nixl_capi_status_t
nixl_capi_get_local_partial_md(nixl_capi_agent_t agent, nixl_capi_reg_dlist_t descs, void **data, size_t *len,
                               nixl_capi_opt_args_t opt_args) {
    if (!agent || !descs || !data || !len) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        nixl_blob_t blob;
        const nixl_status_t st = agent->inner->getLocalPartialMD(*descs->dlist, blob, opt_args ? &opt_args->args : nullptr);
        if (st != NIXL_SUCCESS) return fold(st);
        return copyOut(blob, data, len);
    });
}

nixl_capi_status_t
nixl_capi_load_remote_md(nixl_capi_agent_t agent, const void *data, size_t len, char **agent_name) {
    if (!agent || !data || !len || !agent_name) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        std::string name;
        const nixl_status_t st = agent->inner->loadRemoteMD(nixl_blob_t(static_cast<const char *>(data), len), name);
        if (st != NIXL_SUCCESS) return fold(st);
        *agent_name = ::strdup(name.c_str());
        return *agent_name ? NIXL_CAPI_SUCCESS : NIXL_CAPI_ERROR_BACKEND;
    });
}

nixl_capi_status_t
nixl_capi_invalidate_remote_md(nixl_capi_agent_t agent, const char *remote_agent) {
    if (!agent || !remote_agent) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] { return fold(agent->inner->invalidateRemoteMD(remote_agent)); });
}

nixl_capi_status_t
nixl_capi_check_remote_md(nixl_capi_agent_t agent, const char *remote_name, nixl_capi_xfer_dlist_t descs) {
    if (!agent || !remote_name) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        // no list: only ask whether the peer's metadata is present
        static const nixl_xfer_dlist_t none(DRAM_SEG);
        return fold(agent->inner->checkRemoteMD(remote_name, descs ? *descs->dlist : none));
    });
}

nixl_capi_status_t
nixl_capi_agent_make_connection(nixl_capi_agent_t agent, const char *remote_agent, nixl_capi_opt_args_t opt_args) {
    if (!agent || !remote_agent) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] { return fold(agent->inner->makeConnection(remote_agent, opt_args ? &opt_args->args : nullptr)); });
}

nixl_capi_status_t
nixl_capi_free_buffer(void *data) {
    std::free(data);
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_create_notif_map(nixl_capi_notif_map_t *notif_map) {
    if (!notif_map) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        *notif_map = new nixl_capi_notif_map_s;
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_destroy_notif_map(nixl_capi_notif_map_t notif_map) {
    if (!notif_map) return NIXL_CAPI_ERROR_INVALID_PARAM;
    delete notif_map;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_get_notifs(nixl_capi_agent_t agent, nixl_capi_notif_map_t notif_map, nixl_capi_opt_args_t opt_args) {
    if (!agent || !notif_map) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] { return fold(agent->inner->getNotifs(notif_map->notifs, opt_args ? &opt_args->args : nullptr)); });
}

nixl_capi_status_t
nixl_capi_gen_notif(nixl_capi_agent_t agent, const char *remote_agent, const void *data, size_t len,
                    nixl_capi_opt_args_t opt_args) {
    if (!agent || !remote_agent || (len && !data)) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        const nixl_blob_t msg(static_cast<const char *>(data), len);
        return fold(agent->inner->genNotif(remote_agent, msg, opt_args ? &opt_args->args : nullptr));
    });
}

nixl_capi_status_t
nixl_capi_notif_map_size(nixl_capi_notif_map_t map, size_t *size) {
    if (!map || !size) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *size = map->notifs.size();
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_notif_map_get_agent_at(nixl_capi_notif_map_t map, size_t index, const char **agent_name) {
    if (!map || !agent_name || index >= map->notifs.size()) return NIXL_CAPI_ERROR_INVALID_PARAM;
    auto it = map->notifs.begin();
    std::advance(it, index);
    *agent_name = it->first.c_str();
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_notif_map_get_notifs_size(nixl_capi_notif_map_t map, const char *agent_name, size_t *size) {
    if (!map || !agent_name || !size) return NIXL_CAPI_ERROR_INVALID_PARAM;
    const auto it = map->notifs.find(agent_name);
    if (it == map->notifs.end()) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *size = it->second.size();
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_notif_map_get_notif(nixl_capi_notif_map_t map, const char *agent_name, size_t index, const void **data,
                              size_t *len) {
    if (!map || !agent_name || !data || !len) return NIXL_CAPI_ERROR_INVALID_PARAM;
    const auto it = map->notifs.find(agent_name);
    if (it == map->notifs.end() || index >= it->second.size()) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *data = it->second[index].data();
    *len = it->second[index].size();
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_notif_map_clear(nixl_capi_notif_map_t map) {
    if (!map) return NIXL_CAPI_ERROR_INVALID_PARAM;
    map->notifs.clear();
    return NIXL_CAPI_SUCCESS;
}

// ---- the remaining helpers of the reference wrapper ------------------------------------------

nixl_capi_status_t
nixl_capi_opt_args_get_notif_msg(nixl_capi_opt_args_t args, void **data, size_t *len) {
    if (!args || !data || !len) return NIXL_CAPI_ERROR_INVALID_PARAM;
    const nixl_blob_t &msg = args->args.notif.has_value() ? args->args.notif.value() : args->args.notifMsg;
    *data = nullptr;
    *len = 0;
    if (msg.empty()) return NIXL_CAPI_SUCCESS;
    return copyOut(msg, data, len);
}

nixl_capi_status_t
nixl_capi_opt_args_get_has_notif(nixl_capi_opt_args_t args, bool *has_notif) {
    if (!args || !has_notif) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *has_notif = args->args.hasNotif || args->args.notif.has_value();
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_opt_args_get_skip_desc_merge(nixl_capi_opt_args_t args, bool *skip_merge) {
    if (!args || !skip_merge) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *skip_merge = args->args.skipDescMerge;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_opt_args_set_ip_addr(nixl_capi_opt_args_t args, const char *ip_addr) {
    if (!args || !ip_addr) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        args->args.ipAddr = ip_addr;
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_opt_args_set_port(nixl_capi_opt_args_t args, uint16_t port) {
    if (!args) return NIXL_CAPI_ERROR_INVALID_PARAM;
    args->args.port = port;
    return NIXL_CAPI_SUCCESS;
}

extern "C++" {
namespace {

template<typename L>
nixl_capi_status_t
listType(L *list, nixl_capi_mem_type_t *mem_type) {
    if (!list || !mem_type) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *mem_type = static_cast<nixl_capi_mem_type_t>(list->dlist->getType());
    return NIXL_CAPI_SUCCESS;
}

template<typename L>
nixl_capi_status_t
listEmpty(L *list, bool *is_empty) {
    if (!list || !is_empty) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *is_empty = list->dlist->isEmpty();
    return NIXL_CAPI_SUCCESS;
}

template<typename L, typename F>
nixl_capi_status_t
listDo(L *list, F &&f) {
    if (!list) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        f(*list->dlist);
        return NIXL_CAPI_SUCCESS;
    });
}

} // namespace
} // extern "C++"

nixl_capi_status_t
nixl_capi_xfer_dlist_get_type(nixl_capi_xfer_dlist_t dlist, nixl_capi_mem_type_t *mem_type) {
    return listType(dlist, mem_type);
}

nixl_capi_status_t
nixl_capi_xfer_dlist_len(nixl_capi_xfer_dlist_t dlist, size_t *len) {
    if (!dlist || !len) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *len = static_cast<size_t>(dlist->dlist->descCount());
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_xfer_dlist_is_empty(nixl_capi_xfer_dlist_t dlist, bool *is_empty) {
    return listEmpty(dlist, is_empty);
}

nixl_capi_status_t
nixl_capi_xfer_dlist_trim(nixl_capi_xfer_dlist_t dlist) {
    return listDo(dlist, [](nixl_xfer_dlist_t &l) { (void)l.trim(); });
}

nixl_capi_status_t
nixl_capi_xfer_dlist_rem_desc(nixl_capi_xfer_dlist_t dlist, int index) {
    return listDo(dlist, [&](nixl_xfer_dlist_t &l) { l.remDesc(index); });
}

nixl_capi_status_t
nixl_capi_xfer_dlist_resize(nixl_capi_xfer_dlist_t dlist, size_t new_size) {
    return listDo(dlist, [&](nixl_xfer_dlist_t &l) { l.resize(new_size); });
}

nixl_capi_status_t
nixl_capi_xfer_dlist_print(nixl_capi_xfer_dlist_t dlist) {
    return listDo(dlist, [](nixl_xfer_dlist_t &l) { l.print(); });
}

nixl_capi_status_t
nixl_capi_reg_dlist_get_type(nixl_capi_reg_dlist_t dlist, nixl_capi_mem_type_t *mem_type) {
    return listType(dlist, mem_type);
}

nixl_capi_status_t
nixl_capi_reg_dlist_is_empty(nixl_capi_reg_dlist_t dlist, bool *is_empty) {
    return listEmpty(dlist, is_empty);
}

nixl_capi_status_t
nixl_capi_reg_dlist_trim(nixl_capi_reg_dlist_t dlist) {
    return listDo(dlist, [](nixl_reg_dlist_t &l) { (void)l.trim(); });
}

nixl_capi_status_t
nixl_capi_reg_dlist_rem_desc(nixl_capi_reg_dlist_t dlist, int index) {
    return listDo(dlist, [&](nixl_reg_dlist_t &l) { l.remDesc(index); });
}

nixl_capi_status_t
nixl_capi_reg_dlist_clear(nixl_capi_reg_dlist_t dlist) {
    return listDo(dlist, [](nixl_reg_dlist_t &l) { l.clear(); });
}

nixl_capi_status_t
nixl_capi_reg_dlist_resize(nixl_capi_reg_dlist_t dlist, size_t new_size) {
    return listDo(dlist, [&](nixl_reg_dlist_t &l) { l.resize(new_size); });
}

nixl_capi_status_t
nixl_capi_reg_dlist_print(nixl_capi_reg_dlist_t dlist) {
    return listDo(dlist, [](nixl_reg_dlist_t &l) { l.print(); });
}

nixl_capi_status_t
nixl_capi_create_query_resp_list(nixl_capi_query_resp_list_t *list) {
    if (!list) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        *list = new nixl_capi_query_resp_list_s;
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_destroy_query_resp_list(nixl_capi_query_resp_list_t list) {
    if (!list) return NIXL_CAPI_ERROR_INVALID_PARAM;
    delete list;
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_query_resp_list_size(nixl_capi_query_resp_list_t list, size_t *size) {
    if (!list || !size) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *size = list->responses.size();
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_query_resp_list_has_value(nixl_capi_query_resp_list_t list, size_t index, bool *has_value) {
    if (!list || !has_value || index >= list->responses.size()) return NIXL_CAPI_ERROR_INVALID_PARAM;
    *has_value = list->responses[index].has_value();
    return NIXL_CAPI_SUCCESS;
}

nixl_capi_status_t
nixl_capi_query_resp_list_get_params(nixl_capi_query_resp_list_t list, size_t index, nixl_capi_params_t *params) {
    if (!list || !params || index >= list->responses.size() || !list->responses[index].has_value())
        return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] {
        *params = new nixl_capi_params_s{list->responses[index].value()};
        return NIXL_CAPI_SUCCESS;
    });
}

nixl_capi_status_t
nixl_capi_query_mem(nixl_capi_agent_t agent, nixl_capi_reg_dlist_t descs, nixl_capi_query_resp_list_t resp,
                    nixl_capi_opt_args_t opt_args) {
    if (!agent || !descs || !resp) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] { return fold(agent->inner->queryMem(*descs->dlist, resp->responses, opt_args ? &opt_args->args : nullptr)); });
}

nixl_capi_status_t
nixl_capi_send_local_md(nixl_capi_agent_t agent, nixl_capi_opt_args_t opt_args) {
    return agent ? fold(agent->inner->sendLocalMD(opt_args ? &opt_args->args : nullptr)) : NIXL_CAPI_ERROR_INVALID_PARAM;
}

nixl_capi_status_t
nixl_capi_send_local_partial_md(nixl_capi_agent_t agent, nixl_capi_reg_dlist_t descs, nixl_capi_opt_args_t opt_args) {
    if (!agent || !descs) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return fold(agent->inner->sendLocalPartialMD(*descs->dlist, opt_args ? &opt_args->args : nullptr));
}

nixl_capi_status_t
nixl_capi_fetch_remote_md(nixl_capi_agent_t agent, const char *remote_name, nixl_capi_opt_args_t opt_args) {
    if (!agent || !remote_name) return NIXL_CAPI_ERROR_INVALID_PARAM;
    return guarded([&] { return fold(agent->inner->fetchRemoteMD(remote_name, opt_args ? &opt_args->args : nullptr)); });
}

nixl_capi_status_t
nixl_capi_invalidate_local_md(nixl_capi_agent_t agent, nixl_capi_opt_args_t opt_args) {
    return agent ? fold(agent->inner->invalidateLocalMD(opt_args ? &opt_args->args : nullptr)) : NIXL_CAPI_ERROR_INVALID_PARAM;
}

bool
nixl_capi_is_stub(void) {
    return false;
}

} // extern "C"
