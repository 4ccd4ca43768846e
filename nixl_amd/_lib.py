"""ctypes loaders for the in-tree native libraries.

The libraries are built by ``__graft_entry__.build()`` (``make -C nixl_amd/csrc``) into
``nixl_amd/lib``.  Nothing here builds, and nothing falls back to Python or to a CPU
implementation: a missing library raises ``NativeLibraryMissing``.
"""
import ctypes
import os
from ctypes import (POINTER, Structure, c_bool, c_char_p, c_float, c_int, c_int64, c_size_t, c_uint16,
                    c_uint, c_uint32, c_uint64, c_void_p)

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(PKG_DIR, "lib")
PLUGIN_DIR = os.path.join(LIB_DIR, "plugins")


class NativeLibraryMissing(RuntimeError):
    pass


def _load(name):
    path = os.path.join(LIB_DIR, name)
    if not os.path.exists(path):
        raise NativeLibraryMissing(
            f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or `make -C nixl_amd/csrc`) first")
    return ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)


# ---------------------------------------------------------------------------------------
# Kernel layer (include/nixl_amd_hip.h, include/nixl_amd_ep.h)
# ---------------------------------------------------------------------------------------

class CopyDesc(Structure):
    _fields_ = [("src", c_uint64), ("dst", c_uint64), ("len", c_uint64)]


class CopyTuning(Structure):
    _fields_ = [("units_per_lane", c_int), ("nontemporal", c_int), ("max_workgroups", c_int),
                ("waves_per_workgroup", c_int), ("xcd_swizzle", c_int), ("sort_scatter", c_int)]


class CopyRun(Structure):
    _fields_ = [("base", c_uint64), ("stride", c_uint64), ("first_index", c_uint64), ("count", c_uint64)]


class CopyRecord(Structure):
    _fields_ = [("src", c_uint64), ("dst", c_uint64)]


class CopyRecordFacts(Structure):
    _fields_ = [("address_bits", c_uint64), ("regular_dst_steps", c_uint64), ("following_src_steps", c_uint64),
                ("steps", c_uint64)]


class CopyPlanInfo(Structure):
    _fields_ = [("payload_bytes", c_uint64), ("vec_descs", c_uint64), ("generic_descs", c_uint64),
                ("plan_device_bytes", c_uint64), ("vec_chunks", c_uint32),
                ("uniform_chunks", c_uint32), ("mixed_chunks", c_uint32),
                ("generic_items", c_uint32), ("units_per_lane", c_uint32),
                ("uniform_workgroups", c_uint32), ("piece_items", c_uint32)]


_kernels = None


def kernels():
    """libnixl_amd_kernels.so with argument types declared."""
    global _kernels
    if _kernels is not None:
        return _kernels
    lib = _load("libnixl_amd_kernels.so")
    lib.nixl_amd_last_error.restype = c_char_p
    lib.nixl_amd_device_count.restype = c_int
    lib.nixl_amd_copy_plan_create.argtypes = [POINTER(CopyDesc), c_size_t, c_int,
                                              POINTER(CopyTuning), POINTER(c_void_p)]
    lib.nixl_amd_copy_plan_create_indexed.argtypes = [c_uint64, c_uint64, c_void_p, c_uint64, c_uint64, c_void_p, c_size_t,
                                                      c_uint64, c_int, POINTER(CopyTuning), POINTER(c_void_p)]
    lib.nixl_amd_copy_plan_create_indexed.restype = c_int
    lib.nixl_amd_copy_plan_create_indexed_runs.argtypes = [POINTER(CopyRun), c_size_t, c_void_p, POINTER(CopyRun), c_size_t,
                                                           c_void_p, c_size_t, c_uint64, c_int, POINTER(CopyTuning),
                                                           POINTER(c_void_p)]
    lib.nixl_amd_copy_plan_create_indexed_runs.restype = c_int
    lib.nixl_amd_copy_records_begin.argtypes = [c_size_t, POINTER(c_void_p), POINTER(POINTER(CopyRecord))]
    lib.nixl_amd_copy_plan_create_from_records.argtypes = [c_void_p, c_size_t, c_uint64, c_int, POINTER(CopyTuning),
                                                           POINTER(CopyRecordFacts), POINTER(c_void_p)]
    lib.nixl_amd_copy_records_abandon.argtypes = [c_void_p]
    lib.nixl_amd_copy_block_len_fits.argtypes = [c_uint64, POINTER(CopyTuning)]
    for fn in ("nixl_amd_copy_records_begin", "nixl_amd_copy_plan_create_from_records", "nixl_amd_copy_records_abandon",
               "nixl_amd_copy_block_len_fits"):
        getattr(lib, fn).restype = c_int
    lib.nixl_amd_copy_plan_launch.argtypes = [c_void_p, c_void_p]
    lib.nixl_amd_copy_plan_destroy.argtypes = [c_void_p]
    lib.nixl_amd_copy_plan_status.argtypes = [c_void_p, c_int]
    lib.nixl_amd_copy_plan_status.restype = c_int
    lib.nixl_amd_copy_plan_query.argtypes = [c_void_p, POINTER(CopyPlanInfo)]
    lib.nixl_amd_copy_plan_time.argtypes = [c_void_p, c_void_p, c_int, POINTER(c_float)]
    for fn in ("nixl_amd_copy_plan_create", "nixl_amd_copy_plan_launch",
               "nixl_amd_copy_plan_destroy", "nixl_amd_copy_plan_query",
               "nixl_amd_copy_plan_time"):
        getattr(lib, fn).restype = c_int
    _kernels = lib
    return lib


def kernels_error():
    return kernels().nixl_amd_last_error().decode()


_EP_SIGS = {
    "nixl_amd_ep_ll_dispatch": [c_void_p] * 10 + [c_int] * 9 + [c_void_p, c_void_p, c_size_t, c_void_p],
    "nixl_amd_ep_ll_route_dispatch": [c_void_p] * 12 + [c_int] * 9 + [c_void_p, c_void_p, c_size_t, c_void_p],
    "nixl_amd_ep_ll_dispatch_status": [c_void_p, c_void_p, POINTER(c_int)],
    "nixl_amd_ep_ll_dispatch_phased": [c_void_p] * 11 + [c_int] * 9 + [c_void_p, c_void_p, c_size_t, c_int, c_uint64, c_int,
                                                                      c_void_p],
    "nixl_amd_ep_ll_combine_elastic": [c_void_p] * 11 + [c_int] * 7 + [c_uint64, c_void_p],
    "nixl_amd_ep_ll_dispatch_static": [c_void_p] * 10 + [c_int] * 9 + [c_void_p, c_void_p],
    "nixl_amd_ep_ll_combine": [c_void_p] * 9 + [c_int] * 7 + [c_void_p],
    "nixl_amd_ep_get_dispatch_layout": [c_void_p] * 4 + [c_int] * 4 + [c_void_p],
    "nixl_amd_ep_ht_notify_dispatch": [c_void_p] * 8 + [c_int] * 5 + [c_void_p],
    "nixl_amd_ep_ht_dispatch": [c_void_p] * 11 + [c_int] * 5 + [c_void_p],
    "nixl_amd_ep_ht_dispatch_scaled": [c_void_p] * 13 + [c_int] * 4 + [c_int64] * 3 + [c_int] * 3 + [c_void_p],
    "nixl_amd_ep_ht_combine": [c_void_p] * 10 + [c_int] * 4 + [c_void_p],
    "nixl_amd_ep_router_topk": [c_void_p] * 3 + [c_int] * 3 + [c_void_p],
    "nixl_amd_ep_f32_to_e4m3": [c_void_p, c_void_p, c_size_t, c_void_p],
    "nixl_amd_ep_ll_set_tuning": [c_int, c_int],
}

_ep = None


def ep_kernels():
    """The expert-parallel entry points of libnixl_amd_kernels.so (include/nixl_amd_ep.h)."""
    global _ep
    if _ep is not None:
        return _ep
    lib = kernels()
    for name, args in _EP_SIGS.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = c_int
    lib.nixl_amd_ep_ll_workspace_bytes.argtypes = [c_int] * 5
    lib.nixl_amd_ep_ll_workspace_bytes.restype = c_size_t
    _ep = lib
    return lib


def kernel_symbols():
    return sorted(["nixl_amd_last_error", "nixl_amd_device_count", "nixl_amd_copy_plan_create", "nixl_amd_copy_plan_create_indexed",
                   "nixl_amd_copy_plan_create_indexed_runs", "nixl_amd_copy_records_begin",
                   "nixl_amd_copy_plan_create_from_records", "nixl_amd_copy_records_abandon", "nixl_amd_copy_block_len_fits",
                   "nixl_amd_copy_plan_launch", "nixl_amd_copy_plan_destroy", "nixl_amd_copy_plan_status",
                   "nixl_amd_copy_plan_query", "nixl_amd_copy_plan_time", "nixl_amd_ep_ll_workspace_bytes"] + list(_EP_SIGS))


# ---------------------------------------------------------------------------------------
# Agent C API (include/nixl_amd_capi.h)
# ---------------------------------------------------------------------------------------

class AgentConfig(Structure):
    _fields_ = [("enable_prog_thread", c_bool), ("enable_listen_thread", c_bool),
                ("listen_port", c_int), ("thread_sync", c_int), ("num_workers", c_uint),
                ("pthr_delay_us", c_uint64), ("lthr_delay_us", c_uint64),
                ("capture_telemetry", c_bool)]


class XferTelemetry(Structure):
    _fields_ = [("start_time_us", c_uint64), ("post_duration_us", c_uint64),
                ("xfer_duration_us", c_uint64), ("total_bytes", c_uint64),
                ("desc_count", c_uint64)]


_agent = None

_CAPI_SIGS = {
    "nixl_capi_create_agent": [c_char_p, POINTER(c_void_p)],
    "nixl_capi_create_configured_agent": [c_char_p, POINTER(AgentConfig), POINTER(c_void_p)],
    "nixl_capi_destroy_agent": [c_void_p],
    "nixl_capi_create_params": [POINTER(c_void_p)],
    "nixl_capi_params_add": [c_void_p, c_char_p, c_char_p],
    "nixl_capi_destroy_params": [c_void_p],
    "nixl_capi_create_backend": [c_void_p, c_char_p, c_void_p, POINTER(c_void_p)],
    "nixl_capi_destroy_backend": [c_void_p],
    "nixl_capi_create_opt_args": [POINTER(c_void_p)],
    "nixl_capi_destroy_opt_args": [c_void_p],
    "nixl_capi_opt_args_add_backend": [c_void_p, c_void_p],
    "nixl_capi_opt_args_set_notif_msg": [c_void_p, c_char_p, c_size_t],
    "nixl_capi_opt_args_set_has_notif": [c_void_p, c_bool],
    "nixl_capi_opt_args_set_skip_desc_merge": [c_void_p, c_bool],
    "nixl_capi_create_xfer_dlist": [c_int, POINTER(c_void_p)],
    "nixl_capi_destroy_xfer_dlist": [c_void_p],
    "nixl_capi_xfer_dlist_add_desc": [c_void_p, c_uint64, c_size_t, c_uint64],
    "nixl_capi_xfer_dlist_add_descs": [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t],
    "nixl_capi_xfer_dlist_desc_count": [c_void_p, POINTER(c_size_t)],
    "nixl_capi_xfer_dlist_clear": [c_void_p],
    "nixl_capi_create_reg_dlist": [c_int, POINTER(c_void_p)],
    "nixl_capi_destroy_reg_dlist": [c_void_p],
    "nixl_capi_reg_dlist_add_desc": [c_void_p, c_uint64, c_size_t, c_uint64, c_char_p, c_size_t],
    "nixl_capi_reg_dlist_desc_count": [c_void_p, POINTER(c_size_t)],
    "nixl_capi_register_mem": [c_void_p, c_void_p, c_void_p],
    "nixl_capi_deregister_mem": [c_void_p, c_void_p, c_void_p],
    "nixl_capi_prep_xfer_dlist": [c_void_p, c_char_p, c_void_p, POINTER(c_void_p), c_void_p],
    "nixl_capi_release_xfer_dlist_handle": [c_void_p, c_void_p],
    "nixl_capi_xfer_dlist_handle_run_count": [c_void_p, POINTER(c_size_t)],
    "nixl_capi_make_xfer_req": [c_void_p, c_int, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p,
                                c_size_t, POINTER(c_void_p), c_void_p],
    "nixl_capi_create_xfer_req": [c_void_p, c_int, c_void_p, c_void_p, c_char_p,
                                  POINTER(c_void_p), c_void_p],
    "nixl_capi_post_xfer_req": [c_void_p, c_void_p, c_void_p],
    "nixl_capi_get_xfer_status": [c_void_p, c_void_p],
    "nixl_capi_post_and_wait": [c_void_p, c_void_p],
    "nixl_capi_get_xfer_telemetry": [c_void_p, c_void_p, POINTER(XferTelemetry)],
    "nixl_capi_xfer_req_desc_count": [c_void_p, POINTER(c_size_t), POINTER(c_size_t)],
    "nixl_capi_xfer_req_get_desc": [c_void_p, c_size_t, POINTER(c_uint64), POINTER(c_uint64),
                                    POINTER(c_uint64)],
    "nixl_capi_get_available_plugins": [c_void_p, POINTER(c_void_p)],
    "nixl_capi_destroy_string_list": [c_void_p],
    "nixl_capi_string_list_size": [c_void_p, POINTER(c_size_t)],
    "nixl_capi_string_list_get": [c_void_p, c_size_t, POINTER(c_char_p)],
    "nixl_capi_get_plugin_params": [c_void_p, c_char_p, POINTER(c_void_p), POINTER(c_void_p)],
    "nixl_capi_get_backend_params": [c_void_p, c_void_p, POINTER(c_void_p), POINTER(c_void_p)],
    "nixl_capi_destroy_mem_list": [c_void_p],
    "nixl_capi_mem_list_is_empty": [c_void_p, POINTER(c_bool)],
    "nixl_capi_mem_list_size": [c_void_p, POINTER(c_size_t)],
    "nixl_capi_mem_list_get": [c_void_p, c_size_t, POINTER(c_int)],
    "nixl_capi_mem_type_to_string": [c_int, POINTER(c_char_p)],
    "nixl_capi_params_is_empty": [c_void_p, POINTER(c_bool)],
    "nixl_capi_params_create_iterator": [c_void_p, POINTER(c_void_p)],
    "nixl_capi_params_iterator_next": [c_void_p, POINTER(c_char_p), POINTER(c_char_p), POINTER(c_bool)],
    "nixl_capi_params_destroy_iterator": [c_void_p],
    "nixl_capi_estimate_xfer_cost": [c_void_p, c_void_p, c_void_p, POINTER(c_int64), POINTER(c_int64), POINTER(c_int)],
    "nixl_capi_query_xfer_backend": [c_void_p, c_void_p, POINTER(c_void_p)],
    "nixl_capi_backend_get_type": [c_void_p, POINTER(c_char_p)],
    "nixl_capi_prep_mem_view_local": [c_void_p, c_void_p, POINTER(c_void_p), c_void_p],
    "nixl_capi_prep_mem_view_remote": [c_void_p, c_void_p, POINTER(c_void_p), c_void_p],
    "nixl_capi_create_remote_dlist": [c_int, POINTER(c_void_p)],
    "nixl_capi_destroy_remote_dlist": [c_void_p],
    "nixl_capi_remote_dlist_add_desc": [c_void_p, c_size_t, c_size_t, c_uint64, c_char_p],
    "nixl_capi_release_mem_view": [c_void_p, c_void_p],
    "nixl_capi_opt_args_set_include_conn_info": [c_void_p, c_bool],
    "nixl_capi_get_local_md": [c_void_p, POINTER(c_void_p), POINTER(c_size_t)],
    "nixl_capi_get_local_partial_md": [c_void_p, c_void_p, POINTER(c_void_p), POINTER(c_size_t), c_void_p],
    "nixl_capi_load_remote_md": [c_void_p, c_char_p, c_size_t, POINTER(c_void_p)],
    "nixl_capi_invalidate_remote_md": [c_void_p, c_char_p],
    "nixl_capi_check_remote_md": [c_void_p, c_char_p, c_void_p],
    "nixl_capi_agent_make_connection": [c_void_p, c_char_p, c_void_p],
    "nixl_capi_free_buffer": [c_void_p],
    "nixl_capi_create_notif_map": [POINTER(c_void_p)],
    "nixl_capi_destroy_notif_map": [c_void_p],
    "nixl_capi_get_notifs": [c_void_p, c_void_p, c_void_p],
    "nixl_capi_gen_notif": [c_void_p, c_char_p, c_char_p, c_size_t, c_void_p],
    "nixl_capi_notif_map_size": [c_void_p, POINTER(c_size_t)],
    "nixl_capi_notif_map_get_agent_at": [c_void_p, c_size_t, POINTER(c_char_p)],
    "nixl_capi_notif_map_get_notifs_size": [c_void_p, c_char_p, POINTER(c_size_t)],
    "nixl_capi_notif_map_get_notif": [c_void_p, c_char_p, c_size_t, POINTER(c_void_p), POINTER(c_size_t)],
    "nixl_capi_notif_map_clear": [c_void_p],
    "nixl_capi_opt_args_get_notif_msg": [c_void_p, POINTER(c_void_p), POINTER(c_size_t)],
    "nixl_capi_opt_args_get_has_notif": [c_void_p, POINTER(c_bool)],
    "nixl_capi_opt_args_get_skip_desc_merge": [c_void_p, POINTER(c_bool)],
    "nixl_capi_opt_args_set_ip_addr": [c_void_p, c_char_p],
    "nixl_capi_opt_args_set_port": [c_void_p, c_uint16],
    "nixl_capi_xfer_dlist_get_type": [c_void_p, POINTER(c_int)],
    "nixl_capi_xfer_dlist_len": [c_void_p, POINTER(c_size_t)],
    "nixl_capi_xfer_dlist_is_empty": [c_void_p, POINTER(c_bool)],
    "nixl_capi_xfer_dlist_trim": [c_void_p],
    "nixl_capi_xfer_dlist_rem_desc": [c_void_p, c_int],
    "nixl_capi_xfer_dlist_resize": [c_void_p, c_size_t],
    "nixl_capi_xfer_dlist_print": [c_void_p],
    "nixl_capi_reg_dlist_get_type": [c_void_p, POINTER(c_int)],
    "nixl_capi_reg_dlist_is_empty": [c_void_p, POINTER(c_bool)],
    "nixl_capi_reg_dlist_trim": [c_void_p],
    "nixl_capi_reg_dlist_rem_desc": [c_void_p, c_int],
    "nixl_capi_reg_dlist_clear": [c_void_p],
    "nixl_capi_reg_dlist_resize": [c_void_p, c_size_t],
    "nixl_capi_reg_dlist_print": [c_void_p],
    "nixl_capi_create_query_resp_list": [POINTER(c_void_p)],
    "nixl_capi_destroy_query_resp_list": [c_void_p],
    "nixl_capi_query_resp_list_size": [c_void_p, POINTER(c_size_t)],
    "nixl_capi_query_resp_list_has_value": [c_void_p, c_size_t, POINTER(c_bool)],
    "nixl_capi_query_resp_list_get_params": [c_void_p, c_size_t, POINTER(c_void_p)],
    "nixl_capi_query_mem": [c_void_p, c_void_p, c_void_p, c_void_p],
    "nixl_capi_send_local_md": [c_void_p, c_void_p],
    "nixl_capi_send_local_partial_md": [c_void_p, c_void_p, c_void_p],
    "nixl_capi_fetch_remote_md": [c_void_p, c_char_p, c_void_p],
    "nixl_capi_invalidate_local_md": [c_void_p, c_void_p],
    "nixl_capi_is_stub": [],
    "nixl_capi_release_xfer_req": [c_void_p, c_void_p],
    "nixl_capi_destroy_xfer_req": [c_void_p],
}


def agent_lib():
    """libnixl_amd_agent.so with argument types declared."""
    global _agent
    if _agent is not None:
        return _agent
    lib = _load("libnixl_amd_agent.so")
    for name, args in _CAPI_SIGS.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = c_int
    lib.nixl_capi_last_nixl_status.restype = c_int
    _agent = lib
    return lib


def capi_symbols():
    return sorted(list(_CAPI_SIGS) + ["nixl_capi_last_nixl_status"])
