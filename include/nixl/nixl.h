// nixlAgent: the north-bound class an application drives (reference: src/api/cpp/nixl.h:34-564).
// This tree implements the single-agent, loopback subset that the descriptor-transfer path
// needs — backend creation, memory registration, prepared descriptor lists, request
// creation / post / poll / release — with the reference's signatures and status codes.
// Metadata exchange, notifications and memory views belong to the reference's control
// plane; those members exist so callers link, and return NIXL_ERR_NOT_SUPPORTED.
#ifndef NIXL_AMD_AGENT_API_H
#define NIXL_AMD_AGENT_API_H

#include <memory>
#include <string>
#include <vector>

#include "nixl_descriptors.h"
#include "nixl_params.h"
#include "nixl_types.h"

class nixlAgent {
private:
    std::unique_ptr<nixlAgentData> data;

public:
    nixlAgent(const std::string &name, const nixlAgentConfig &cfg);
    ~nixlAgent();

    nixlAgent(nixlAgent &&) noexcept = delete;
    nixlAgent &
    operator=(nixlAgent &&) noexcept = delete;

    // Plugins and backends (reference: src/core/nixl_agent.cpp:254-426).
    nixl_status_t
    getAvailPlugins(std::vector<nixl_backend_t> &plugins);
    nixl_status_t
    getPluginParams(const nixl_backend_t &type, nixl_mem_list_t &mems, nixl_b_params_t &params) const;
    nixl_status_t
    getBackendParams(const nixlBackendH *backend, nixl_mem_list_t &mems, nixl_b_params_t &params) const;
    nixl_status_t
    createBackend(const nixl_backend_t &type, const nixl_b_params_t &params, nixlBackendH *&backend);

    // Registration (reference: src/core/nixl_agent.cpp:441-561).
    nixl_status_t
    registerMem(const nixl_reg_dlist_t &descs, const nixl_opt_args_t *extra_params = nullptr);
    nixl_status_t
    deregisterMem(const nixl_reg_dlist_t &descs, const nixl_opt_args_t *extra_params = nullptr);
    nixl_status_t
    queryMem(const nixl_reg_dlist_t &descs,
             std::vector<nixl_query_resp_t> &resp,
             const nixl_opt_args_t *extra_params) const;
    nixl_status_t
    makeConnection(const std::string &remote_agent, const nixl_opt_args_t *extra_params = nullptr);

    // Transfers (reference: src/core/nixl_agent.cpp:620-1320).
    nixl_status_t
    prepXferDlist(const std::string &agent_name,
                  const nixl_xfer_dlist_t &descs,
                  nixlDlistH *&dlist_hndl,
                  const nixl_opt_args_t *extra_params = nullptr) const;
    nixl_status_t
    prepXferDlist(const nixl_xfer_dlist_t &descs,
                  nixlDlistH *&dlist_hndl,
                  const nixl_opt_args_t *extra_params = nullptr) const;
    nixl_status_t
    makeXferReq(const nixl_xfer_op_t &operation,
                const nixlDlistH *local_side,
                const std::vector<int> &local_indices,
                const nixlDlistH *remote_side,
                const std::vector<int> &remote_indices,
                nixlXferReqH *&req_hndl,
                const nixl_opt_args_t *extra_params = nullptr) const;
    nixl_status_t
    createXferReq(const nixl_xfer_op_t &operation,
                  const nixl_xfer_dlist_t &local_descs,
                  const nixl_xfer_dlist_t &remote_descs,
                  const std::string &remote_agent,
                  nixlXferReqH *&req_hndl,
                  const nixl_opt_args_t *extra_params = nullptr) const;
    nixl_status_t
    estimateXferCost(const nixlXferReqH *req_hndl,
                     std::chrono::microseconds &duration,
                     std::chrono::microseconds &err_margin,
                     nixl_cost_t &method,
                     const nixl_opt_args_t *extra_params = nullptr) const;
    nixl_status_t
    postXferReq(nixlXferReqH *req_hndl, const nixl_opt_args_t *extra_params = nullptr) const;
    nixl_status_t
    getXferStatus(nixlXferReqH *req_hndl) const;
    nixl_status_t
    getXferTelemetry(const nixlXferReqH *req_hndl, nixl_xfer_telem_t &telemetry) const;
    nixl_status_t
    queryXferBackend(const nixlXferReqH *req_hndl, nixlBackendH *&backend) const;
    nixl_status_t
    releaseXferReq(nixlXferReqH *req_hndl) const;
    nixl_status_t
    releasedDlistH(nixlDlistH *dlist_hndl) const;

    // Memory views for kernels that move data themselves.
    nixl_status_t
    prepMemView(const nixl_remote_dlist_t &dlist,
                nixlMemViewH &mvh,
                const nixl_opt_args_t *extra_params = nullptr) const;
    nixl_status_t
    prepMemView(const nixl_local_dlist_t &dlist,
                nixlMemViewH &mvh,
                const nixl_opt_args_t *extra_params = nullptr) const;
    void
    releaseMemView(nixlMemViewH mvh) const;
    nixl_status_t
    getNotifs(nixl_notifs_t &notif_map, const nixl_opt_args_t *extra_params = nullptr);
    nixl_status_t
    genNotif(const std::string &remote_agent,
             const nixl_blob_t &msg,
             const nixl_opt_args_t *extra_params = nullptr) const;
    // Metadata exchange by hand: the blob of one agent, in the reference's wire format,
    // is given to another agent by whatever means the application has.  The side channels
    // of the reference (sockets, ETCD: sendLocalMD, fetchRemoteMD, invalidateLocalMD) are not
    // offered.
    nixl_status_t
    getLocalMD(nixl_blob_t &str) const;
    nixl_status_t
    getLocalPartialMD(const nixl_reg_dlist_t &descs,
                      nixl_blob_t &str,
                      const nixl_opt_args_t *extra_params = nullptr) const;
    nixl_status_t
    loadRemoteMD(const nixl_blob_t &remote_metadata, std::string &agent_name);
    nixl_status_t
    invalidateRemoteMD(const std::string &remote_agent);
    nixl_status_t
    checkRemoteMD(const std::string remote_name, const nixl_xfer_dlist_t &descs) const;
    // The side channels themselves: declared so that callers link; NIXL_ERR_NOT_SUPPORTED.
    nixl_status_t
    sendLocalMD(const nixl_opt_args_t *extra_params = nullptr) const;
    nixl_status_t
    sendLocalPartialMD(const nixl_reg_dlist_t &descs, const nixl_opt_args_t *extra_params = nullptr) const;
    nixl_status_t
    fetchRemoteMD(const std::string remote_name, const nixl_opt_args_t *extra_params = nullptr);
    nixl_status_t
    invalidateLocalMD(const nixl_opt_args_t *extra_params = nullptr) const;
};

#endif // NIXL_AMD_AGENT_API_H
