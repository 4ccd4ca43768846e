"""Python view of the agent, shaped after the reference's ``nixl_agent``
(src/api/python/_api.py:189-1221): same method names, argument meaning and "DONE" /
"PROC" / "ERR" transfer states, over the C ABI in include/nixl_amd_capi.h.

Descriptor lists are numpy ``uint64`` arrays of shape (N, 3) holding (addr, len, devId),
lists of such triples, or lists of torch tensors (reference: get_xfer_descs,
_api.py:999-1092).  Only the single-agent loopback subset exists; there is no metadata
exchange or notification path.
"""
import ctypes
import logging
import os

import numpy as np

from . import _lib

logger = logging.getLogger("nixl_amd")

NIXL_INIT_AGENT = ""

# nixl_status_t, src/api/cpp/nixl_types.h:53-68
NIXL_IN_PROG = 1
NIXL_SUCCESS = 0
NIXL_ERR_NOT_POSTED = -1
NIXL_ERR_INVALID_PARAM = -2
NIXL_ERR_BACKEND = -3
NIXL_ERR_NOT_FOUND = -4
NIXL_ERR_MISMATCH = -5
NIXL_ERR_NOT_ALLOWED = -6
NIXL_ERR_REPOST_ACTIVE = -7
NIXL_ERR_UNKNOWN = -8
NIXL_ERR_NOT_SUPPORTED = -9
NIXL_ERR_REMOTE_DISCONNECT = -10
NIXL_ERR_CANCELED = -11
NIXL_ERR_NO_TELEMETRY = -12

_STATUS_NAMES = {v: k for k, v in list(globals().items()) if k.startswith("NIXL_") and isinstance(v, int)}

_MEM = {"DRAM": 0, "VRAM": 1, "BLOCK": 2, "BLK": 2, "OBJ": 3, "FILE": 4,
        "cpu": 0, "cuda": 1}


class NixlError(RuntimeError):
    """A nixl_status_t error (reference bindings raise one exception class per code)."""

    def __init__(self, where, capi_status, nixl_status):
        self.capi_status = capi_status
        self.status = nixl_status
        super().__init__(f"{where}: {_STATUS_NAMES.get(nixl_status, nixl_status)} (capi {capi_status})")


def _check(where, rc, ok=(0,)):
    if rc not in ok:
        st = _lib.agent_lib().nixl_capi_last_nixl_status() if rc not in (-1, -3, -4) else NIXL_ERR_INVALID_PARAM
        raise NixlError(where, rc, st)
    return rc


def _tensors_of(descs):
    """The tensors in `descs` if it is a tensor or a list of tensors, else None."""
    if hasattr(descs, "data_ptr"):
        return [descs]
    if not isinstance(descs, np.ndarray) and len(descs) and all(hasattr(d, "data_ptr") for d in descs):
        return list(descs)
    return None


def _as_triples(descs):
    """Normalise a descriptor list to a C-contiguous (N, 3) uint64 array."""
    if hasattr(descs, "data_ptr"):
        descs = [descs]
    if isinstance(descs, np.ndarray):
        arr = descs
    else:
        rows = []
        for d in descs:
            if hasattr(d, "data_ptr"):
                dev = d.device.index if d.device.type == "cuda" and d.device.index is not None else 0
                rows.append((d.data_ptr(), d.numel() * d.element_size(), dev))
            else:
                rows.append(tuple(d)[:3])
        arr = np.array(rows, dtype=np.uint64).reshape(-1, 3)
    if arr.ndim != 2 or arr.shape[1] != 3:
        raise ValueError("descriptor array must have shape (N, 3): addr, len, devId")
    return np.ascontiguousarray(arr, dtype=np.uint64)


def _guess_mem(descs, mem_type):
    if mem_type is not None:
        return _MEM[mem_type]
    tensors = _tensors_of(descs)
    if tensors:
        return _MEM[tensors[0].device.type]
    raise ValueError("mem_type is required for raw address lists")


class nixl_agent_config:
    """Reference: nixl_agent_config, src/api/python/_api.py:148-186."""

    def __init__(self, enable_prog_thread=True, enable_listen_thread=False, listen_port=0,
                 capture_telemetry=False, num_threads=0, backends=("HIP",)):
        self.enable_pthread = enable_prog_thread
        self.enable_listen = enable_listen_thread
        self.port = listen_port
        self.capture_telemetry = capture_telemetry
        self.num_threads = num_threads
        self.backends = list(backends)


class nixl_xfer_dlist:
    """Owned nixl_xfer_dlist_t (what get_xfer_descs returns in the reference)."""

    def __init__(self, triples, mem):
        self._lib = _lib.agent_lib()
        self.mem = mem
        self.triples = triples
        h = ctypes.c_void_p()
        _check("create_xfer_dlist", self._lib.nixl_capi_create_xfer_dlist(mem, ctypes.byref(h)))
        self._h = h
        n = triples.shape[0]
        if n:
            addrs = np.ascontiguousarray(triples[:, 0])
            lens = np.ascontiguousarray(triples[:, 1])
            devs = np.ascontiguousarray(triples[:, 2])
            _check("xfer_dlist_add_descs",
                   self._lib.nixl_capi_xfer_dlist_add_descs(h, addrs.ctypes.data, lens.ctypes.data,
                                                            devs.ctypes.data, n))

    def descCount(self):
        return int(self.triples.shape[0])

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.nixl_capi_destroy_xfer_dlist(self._h)
            self._h = None


class nixl_reg_dlist:
    def __init__(self, triples, mem):
        self._lib = _lib.agent_lib()
        self.mem = mem
        self.triples = triples
        h = ctypes.c_void_p()
        _check("create_reg_dlist", self._lib.nixl_capi_create_reg_dlist(mem, ctypes.byref(h)))
        self._h = h
        for a, l, d in triples:
            _check("reg_dlist_add_desc", self._lib.nixl_capi_reg_dlist_add_desc(h, int(a), int(l), int(d), None, 0))

    def descCount(self):
        return int(self.triples.shape[0])

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.nixl_capi_destroy_reg_dlist(self._h)
            self._h = None


class nixl_remote_dlist:
    """Owned nixl_remote_dlist_t: (addr, len, devId, agent name) entries; an agent name of
    None is the placeholder that keeps later indices (reference: nixlRemoteDList,
    src/bindings/python/nixl_bindings.cpp; wrapper.h:404-433)."""

    def __init__(self, entries, mem):
        self._lib = _lib.agent_lib()
        self.mem = mem
        self.entries = list(entries)
        h = ctypes.c_void_p()
        _check("create_remote_dlist", self._lib.nixl_capi_create_remote_dlist(mem, ctypes.byref(h)))
        self._h = h
        for a, l, d, name in self.entries:
            _check("remote_dlist_add_desc",
                   self._lib.nixl_capi_remote_dlist_add_desc(h, int(a), int(l), int(d),
                                                             None if name is None else name.encode()))

    def descCount(self):
        return len(self.entries)

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.nixl_capi_destroy_remote_dlist(self._h)
            self._h = None


class nixl_prepped_dlist_handle:
    """Reference: _api.py:49-86."""

    def __init__(self, agent, value):
        self._agent = agent
        self._handle = value

    def release(self):
        if self._handle:
            self._agent.release_dlist_handle(self)

    def run_count(self):
        n = ctypes.c_size_t()
        _check("run_count", _lib.agent_lib().nixl_capi_xfer_dlist_handle_run_count(self._handle, ctypes.byref(n)))
        return n.value


class nixl_xfer_handle:
    """Reference: _api.py:89-127."""

    def __init__(self, agent, value):
        self._agent = agent
        self._handle = value

    def release(self):
        if self._handle:
            self._agent.release_xfer_handle(self)

    def desc_count(self):
        n, b = ctypes.c_size_t(), ctypes.c_size_t()
        _check("desc_count", _lib.agent_lib().nixl_capi_xfer_req_desc_count(self._handle, ctypes.byref(n), ctypes.byref(b)))
        return n.value, b.value

    def get_desc(self, i):
        la, ra, ln = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_uint64()
        _check("get_desc", _lib.agent_lib().nixl_capi_xfer_req_get_desc(self._handle, i, ctypes.byref(la), ctypes.byref(ra), ctypes.byref(ln)))
        return la.value, ra.value, ln.value


class nixl_agent:
    """Reference: nixl_agent, src/api/python/_api.py:189-296."""

    def __init__(self, agent_name, nixl_conf=None, instantiate_all=False, plugin_dirs=()):
        """Reference: _api.py:200-282.  Without a configuration the defaults of
        nixl_agent_config apply (the HIP backend here, where the reference names UCX);
        instantiate_all creates a backend for every plugin found instead; plugin_dirs (not in
        the reference) adds directories to the plugin search path."""
        if not agent_name:
            raise ValueError("agent name must not be empty")  # as the reference bindings do
        self._lib = _lib.agent_lib()
        self.name = agent_name
        if nixl_conf and instantiate_all:
            instantiate_all = False
            logger.warning("Ignoring instantiate_all based on the provided config in agent creation.")
        conf = nixl_conf or nixl_agent_config()
        dirs = [_lib.PLUGIN_DIR] + list(plugin_dirs)
        prev = os.environ.get("NIXL_PLUGIN_DIR")
        if prev:
            dirs.append(prev)
        os.environ["NIXL_PLUGIN_DIR"] = ":".join(dict.fromkeys(dirs))
        cfg = _lib.AgentConfig(conf.enable_pthread, conf.enable_listen, conf.port, 0, 1, 0, 100000,
                               conf.capture_telemetry)
        h = ctypes.c_void_p()
        _check("create_agent", self._lib.nixl_capi_create_configured_agent(agent_name.encode(), ctypes.byref(cfg), ctypes.byref(h)))
        self._h = h
        self.backends = {}
        self.notifs = {}  # what update_notifs / check_remote_xfer_done have not handed out yet
        self.nixl_ops = {"WRITE": 1, "READ": 0}
        self.plugin_list = self.get_plugin_list()
        if not self.plugin_list:
            self.close()
            raise RuntimeError("No plugins available for NIXL, cannot start transfers!")
        for b in (self.plugin_list if instantiate_all else conf.backends):
            if b not in self.plugin_list:
                logger.warning("Skipping backend registration %s due to the missing plugin.", b)
                continue
            self.create_backend(b)

    def close(self):
        if getattr(self, "_h", None):
            for b in self.backends.values():
                self._lib.nixl_capi_destroy_backend(b)
            self.backends = {}
            self._lib.nixl_capi_destroy_agent(self._h)
            self._h = None

    def __del__(self):
        self.close()

    # -- backends ---------------------------------------------------------------------
    def create_backend(self, backend, initParams=None):
        params = ctypes.c_void_p()
        _check("create_params", self._lib.nixl_capi_create_params(ctypes.byref(params)))
        try:
            for k, v in (initParams or {}).items():
                _check("params_add", self._lib.nixl_capi_params_add(params, str(k).encode(), str(v).encode()))
            h = ctypes.c_void_p()
            _check(f"create_backend({backend})",
                   self._lib.nixl_capi_create_backend(self._h, backend.encode(), params, ctypes.byref(h)))
            self.backends[backend] = h
        finally:
            self._lib.nixl_capi_destroy_params(params)

    # -- plugin and backend queries (reference: _api.py:308-389) ----------------------------
    _MEM_NAMES = {0: "DRAM", 1: "VRAM", 2: "BLK", 3: "OBJ", 4: "FILE"}

    def get_plugin_list(self):
        lst = ctypes.c_void_p()
        _check("get_plugin_list", self._lib.nixl_capi_get_available_plugins(self._h, ctypes.byref(lst)))
        try:
            n = ctypes.c_size_t()
            self._lib.nixl_capi_string_list_size(lst, ctypes.byref(n))
            out = []
            for i in range(n.value):
                s = ctypes.c_char_p()
                self._lib.nixl_capi_string_list_get(lst, i, ctypes.byref(s))
                out.append(s.value.decode())
            return out
        finally:
            self._lib.nixl_capi_destroy_string_list(lst)

    def _mems_and_params(self, rc, mems, params):
        """Unpack and free the (memory list, parameters) pair of a query; an unknown name
        gives two empty results, as in the reference (test_nixl_api.py:145-154)."""
        if rc != 0:
            return [], {}
        try:
            n = ctypes.c_size_t()
            self._lib.nixl_capi_mem_list_size(mems, ctypes.byref(n))
            mem_names = []
            for i in range(n.value):
                m = ctypes.c_int()
                self._lib.nixl_capi_mem_list_get(mems, i, ctypes.byref(m))
                mem_names.append(self._MEM_NAMES.get(m.value, "UNKNOWN"))
            return mem_names, self._params_to_dict(params)
        finally:
            self._lib.nixl_capi_destroy_mem_list(mems)
            self._lib.nixl_capi_destroy_params(params)

    def _params_to_dict(self, params):
        out = {}
        empty = ctypes.c_bool()
        self._lib.nixl_capi_params_is_empty(params, ctypes.byref(empty))
        if not empty.value:
            it = ctypes.c_void_p()
            self._lib.nixl_capi_params_create_iterator(params, ctypes.byref(it))
            more = ctypes.c_bool(True)
            while more.value:
                k, v = ctypes.c_char_p(), ctypes.c_char_p()
                if self._lib.nixl_capi_params_iterator_next(it, ctypes.byref(k), ctypes.byref(v), ctypes.byref(more)) != 0:
                    break
                out[k.value.decode()] = v.value.decode()
            self._lib.nixl_capi_params_destroy_iterator(it)
        return out

    def _plugin_query(self, name):
        mems, params = ctypes.c_void_p(), ctypes.c_void_p()
        rc = self._lib.nixl_capi_get_plugin_params(self._h, name.encode(), ctypes.byref(mems), ctypes.byref(params))
        return self._mems_and_params(rc, mems, params)

    def _backend_query(self, name):
        if name not in self.backends:
            return [], {}
        mems, params = ctypes.c_void_p(), ctypes.c_void_p()
        rc = self._lib.nixl_capi_get_backend_params(self._h, self.backends[name], ctypes.byref(mems), ctypes.byref(params))
        return self._mems_and_params(rc, mems, params)

    def get_plugin_mem_types(self, backend):
        return self._plugin_query(backend)[0]

    def get_plugin_params(self, backend):
        return self._plugin_query(backend)[1]

    def get_backend_mem_types(self, backend):
        return self._backend_query(backend)[0]

    def get_backend_params(self, backend):
        return self._backend_query(backend)[1]

    def estimate_xfer_cost(self, req_handle):
        """Reference: _api.py:534-551.  (duration_us, err_margin_us, method)."""
        d, e, m = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int()
        _check("estimate_xfer_cost", self._lib.nixl_capi_estimate_xfer_cost(self._h, req_handle._handle, None, ctypes.byref(d),
                                                                             ctypes.byref(e), ctypes.byref(m)))
        return d.value, e.value, m.value

    def query_xfer_backend(self, handle):
        """Reference: _api.py:694-707: the name of the backend a request was bound to."""
        b = ctypes.c_void_p()
        _check("query_xfer_backend", self._lib.nixl_capi_query_xfer_backend(self._h, handle._handle, ctypes.byref(b)))
        try:
            name = ctypes.c_char_p()
            _check("backend_get_type", self._lib.nixl_capi_backend_get_type(b, ctypes.byref(name)))
            return name.value.decode()
        finally:
            self._lib.nixl_capi_destroy_backend(b)

    def query_memory(self, reg_list, backend, mem_type=None):
        """Reference: _api.py:448-485: per region, what the backend knows about it (a dict) or
        None.  The HIP backend reports the kind of memory, its device, the size of the
        allocation around the address and whether the region fits in it."""
        reg = self.get_reg_descs(reg_list, mem_type)
        if backend not in self.backends:
            raise ValueError(f"Backend '{backend}' not found. Available backends: {list(self.backends)}")
        resp = ctypes.c_void_p()
        _check("create_query_resp_list", self._lib.nixl_capi_create_query_resp_list(ctypes.byref(resp)))
        o = self._opt_args([backend])
        try:
            _check("query_memory", self._lib.nixl_capi_query_mem(self._h, reg._h, resp, o))
            n = ctypes.c_size_t()
            self._lib.nixl_capi_query_resp_list_size(resp, ctypes.byref(n))
            out = []
            for i in range(n.value):
                has = ctypes.c_bool()
                self._lib.nixl_capi_query_resp_list_has_value(resp, i, ctypes.byref(has))
                if not has.value:
                    out.append(None)
                    continue
                params = ctypes.c_void_p()
                _check("query_resp_list_get_params", self._lib.nixl_capi_query_resp_list_get_params(resp, i, ctypes.byref(params)))
                try:
                    out.append(self._params_to_dict(params))
                finally:
                    self._lib.nixl_capi_destroy_params(params)
            return out
        finally:
            self._free_opt(o)
            self._lib.nixl_capi_destroy_query_resp_list(resp)

    # -- metadata and notifications between agents ------------------------------------------
    def _take_buffer(self, data, size):
        try:
            return ctypes.string_at(data, size.value)
        finally:
            self._lib.nixl_capi_free_buffer(data)

    def get_agent_metadata(self):
        """Reference: _api.py:856-862.  The agent's metadata blob, in the reference's wire
        format; hand it to another agent's add_remote_agent by any means."""
        data, size = ctypes.c_void_p(), ctypes.c_size_t()
        _check("get_agent_metadata", self._lib.nixl_capi_get_local_md(self._h, ctypes.byref(data), ctypes.byref(size)))
        return self._take_buffer(data, size)

    def get_partial_agent_metadata(self, descs, inc_conn_info=False, backends=()):
        """Reference: _api.py:864-884.  Metadata of the listed registrations only (an empty
        list: connection info only)."""
        o = self._opt_args(backends, include_conn_info=inc_conn_info)
        data, size = ctypes.c_void_p(), ctypes.c_size_t()
        try:
            _check("get_partial_agent_metadata",
                   self._lib.nixl_capi_get_local_partial_md(self._h, descs._h, ctypes.byref(data), ctypes.byref(size), o))
        finally:
            self._free_opt(o)
        return self._take_buffer(data, size)

    def add_remote_agent(self, metadata):
        """Reference: _api.py:886-897.  Returns the peer's name."""
        name = ctypes.c_void_p()
        _check("add_remote_agent", self._lib.nixl_capi_load_remote_md(self._h, bytes(metadata), len(metadata), ctypes.byref(name)))
        try:
            return ctypes.string_at(name).decode()
        finally:
            self._lib.nixl_capi_free_buffer(name)

    def remove_remote_agent(self, agent):
        """Reference: _api.py:899-907."""
        _check("remove_remote_agent", self._lib.nixl_capi_invalidate_remote_md(self._h, agent.encode()))

    def check_remote_metadata(self, agent, descs=None):
        """Reference: _api.py:976-992."""
        return self._lib.nixl_capi_check_remote_md(self._h, agent.encode(), descs._h if descs is not None else None) == 0

    def make_connection(self, remote_agent, backends=()):
        """Reference: _api.py:471-481."""
        o = self._opt_args(backends)
        try:
            _check("make_connection", self._lib.nixl_capi_agent_make_connection(self._h, remote_agent.encode(), o))
        finally:
            self._free_opt(o)

    def _drain_notifs(self, into, backends=()):
        m = ctypes.c_void_p()
        _check("create_notif_map", self._lib.nixl_capi_create_notif_map(ctypes.byref(m)))
        o = self._opt_args(backends)
        try:
            _check("get_notifs", self._lib.nixl_capi_get_notifs(self._h, m, o))
            n = ctypes.c_size_t()
            self._lib.nixl_capi_notif_map_size(m, ctypes.byref(n))
            for i in range(n.value):
                name = ctypes.c_char_p()
                self._lib.nixl_capi_notif_map_get_agent_at(m, i, ctypes.byref(name))
                count = ctypes.c_size_t()
                self._lib.nixl_capi_notif_map_get_notifs_size(m, name.value, ctypes.byref(count))
                msgs = into.setdefault(name.value.decode(), [])
                for j in range(count.value):
                    data, size = ctypes.c_void_p(), ctypes.c_size_t()
                    self._lib.nixl_capi_notif_map_get_notif(m, name.value, j, ctypes.byref(data), ctypes.byref(size))
                    msgs.append(ctypes.string_at(data, size.value))
        finally:
            self._free_opt(o)
            self._lib.nixl_capi_destroy_notif_map(m)
        return into

    def get_new_notifs(self, backends=()):
        """Reference: _api.py:770-783: {agent name: [messages]} that arrived since the last call."""
        return self._drain_notifs({}, backends)

    def update_notifs(self, backends=()):
        """Reference: _api.py:785-799: like get_new_notifs, accumulated in self.notifs."""
        return self._drain_notifs(self.notifs, backends)

    def check_remote_xfer_done(self, remote_agent_name, lookup_tag, backends=(), tag_is_prefix=True):
        """Reference: _api.py:801-838: looks for one message of `remote_agent_name` that starts
        with (or contains) the tag, and removes just that one."""
        self._drain_notifs(self.notifs, backends)
        for msg in self.notifs.get(remote_agent_name, []):
            if (tag_is_prefix and msg.startswith(lookup_tag)) or (not tag_is_prefix and lookup_tag in msg):
                self.notifs[remote_agent_name].remove(msg)
                return True
        return False

    def send_notif(self, remote_agent_name, notif_msg, backend=None):
        """Reference: _api.py:840-854."""
        msg = notif_msg.encode() if isinstance(notif_msg, str) else bytes(notif_msg)
        o = self._opt_args([backend] if backend else ())
        try:
            _check("send_notif", self._lib.nixl_capi_gen_notif(self._h, remote_agent_name.encode(), msg, len(msg), o))
        finally:
            self._free_opt(o)

    # -- metadata side channels of the reference (sockets, ETCD): not offered ------------------
    def _no_side_channel(self, what):
        raise NixlError(f"{what}: no metadata side channel here; pass get_agent_metadata() to add_remote_agent() by hand",
                        -1, NIXL_ERR_NOT_SUPPORTED)

    def send_local_metadata(self, ip_addr="", port=0):
        """Reference: _api.py:909-920."""
        self._no_side_channel("send_local_metadata")

    def send_partial_agent_metadata(self, descs, inc_conn_info=False, backends=(), ip_addr="", port=0, label=""):
        """Reference: _api.py:922-951."""
        self._no_side_channel("send_partial_agent_metadata")

    def fetch_remote_metadata(self, remote_agent, ip_addr="", port=0, label=""):
        """Reference: _api.py:953-966."""
        self._no_side_channel("fetch_remote_metadata")

    def invalidate_local_metadata(self, ip_addr="", port=0):
        """Reference: _api.py:968-977."""
        self._no_side_channel("invalidate_local_metadata")

    # -- descriptor lists as bytes -------------------------------------------------------------
    _DESCS_MAGIC = b"NXDL1"

    def get_serialized_descs(self, descs):
        """Reference: _api.py:1201-1210 (which pickles the list).  Here a flat record that is
        safe to read back from an untrusted peer: magic, kind, memory type, count, then
        (addr, len, devId) triples; a registration list is serialised without its blobs."""
        if isinstance(descs, nixl_xfer_dlist):
            kind = 1
        elif isinstance(descs, nixl_reg_dlist):
            kind = 2
        else:
            raise TypeError("get_serialized_descs takes a nixl_xfer_dlist or a nixl_reg_dlist")
        tri = np.ascontiguousarray(descs.triples, dtype=np.uint64).reshape(-1, 3)
        return self._DESCS_MAGIC + bytes([kind, descs.mem]) + np.uint64(tri.shape[0]).tobytes() + tri.tobytes()

    def deserialize_descs(self, serialized_descs):
        """Reference: _api.py:1212-1221."""
        b = bytes(serialized_descs)
        m = len(self._DESCS_MAGIC)
        if len(b) < m + 10 or b[:m] != self._DESCS_MAGIC or b[m] not in (1, 2) or b[m + 1] not in _MEM.values():
            raise ValueError("not a serialized descriptor list")
        n = int(np.frombuffer(b, np.uint64, 1, m + 2)[0])
        if len(b) != m + 10 + 24 * n:
            raise ValueError("serialized descriptor list has the wrong length")
        tri = np.frombuffer(b, np.uint64, 3 * n, m + 10).reshape(n, 3).copy()
        return (nixl_xfer_dlist if b[m] == 1 else nixl_reg_dlist)(tri, b[m + 1])

    def prep_mem_view(self, dlist, *, backends=None):
        """Reference: _api.py:728-759.  A local (nixl_xfer_dlist) or remote
        (nixl_remote_dlist) list becomes a table that device code indexes; returns the handle
        as an integer (with the HIP backend: the table's device address)."""
        if isinstance(dlist, nixl_remote_dlist):
            call, what = self._lib.nixl_capi_prep_mem_view_remote, "prep_mem_view(remote)"
        elif isinstance(dlist, nixl_xfer_dlist):
            call, what = self._lib.nixl_capi_prep_mem_view_local, "prep_mem_view(local)"
        else:
            raise TypeError("prep_mem_view takes a nixl_xfer_dlist or a nixl_remote_dlist")
        o = self._opt_args(backends or ())
        mvh = ctypes.c_void_p()
        try:
            _check(what, call(self._h, dlist._h, ctypes.byref(mvh), o))
        finally:
            self._free_opt(o)
        return int(mvh.value)

    def release_mem_view(self, mvh):
        """Reference: _api.py:761-768."""
        _check("release_mem_view", self._lib.nixl_capi_release_mem_view(self._h, ctypes.c_void_p(int(mvh))))

    def _opt_args(self, backends=(), skip_desc_merge=False, notif_msg=b"", include_conn_info=False):
        if not backends and not skip_desc_merge and not notif_msg and not include_conn_info:
            return None
        o = ctypes.c_void_p()
        _check("create_opt_args", self._lib.nixl_capi_create_opt_args(ctypes.byref(o)))
        for b in backends:
            self._lib.nixl_capi_opt_args_add_backend(o, self.backends[b])
        if skip_desc_merge:
            self._lib.nixl_capi_opt_args_set_skip_desc_merge(o, True)
        if include_conn_info:
            self._lib.nixl_capi_opt_args_set_include_conn_info(o, True)
        if notif_msg:
            self._lib.nixl_capi_opt_args_set_notif_msg(o, notif_msg, len(notif_msg))
            self._lib.nixl_capi_opt_args_set_has_notif(o, True)
        return o

    def _free_opt(self, o):
        if o:
            self._lib.nixl_capi_destroy_opt_args(o)

    # -- descriptors ------------------------------------------------------------------
    def get_xfer_descs(self, descs, mem_type=None):
        """Reference: _api.py:999-1115.  Accepts a list of (addr, len, devId) tuples or an
        (N, 3) array with a memory type, a tensor, or a list of tensors; a tensor that is not
        contiguous cannot be described by one range and yields None."""
        if isinstance(descs, nixl_xfer_dlist):
            return descs
        tensors = _tensors_of(descs)
        if tensors and not all(t.is_contiguous() for t in tensors):
            return None
        return nixl_xfer_dlist(_as_triples(descs), _guess_mem(descs, mem_type))

    def get_remote_descs(self, descs, mem_type=None):
        """Reference: _api.py:1082-1113: a list of (addr, len, devId, agent name) tuples with a
        mandatory memory type, or a remote list passed along; anything else yields None."""
        if isinstance(descs, nixl_remote_dlist):
            return descs
        if not descs or not isinstance(descs[0], tuple) or mem_type is None or len(descs[0]) != 4:
            return None
        return nixl_remote_dlist(descs, _MEM[mem_type])

    def get_reg_descs(self, descs, mem_type=None):
        """Reference: _api.py:1117-1230; same inputs as get_xfer_descs."""
        if isinstance(descs, nixl_reg_dlist):
            return descs
        tensors = _tensors_of(descs)
        if tensors and not all(t.is_contiguous() for t in tensors):
            return None
        return nixl_reg_dlist(_as_triples(descs), _guess_mem(descs, mem_type))

    # -- registration -----------------------------------------------------------------
    def register_memory(self, reg_list, mem_type=None, backends=()):
        reg = self.get_reg_descs(reg_list, mem_type)
        o = self._opt_args(backends)
        try:
            _check("register_memory", self._lib.nixl_capi_register_mem(self._h, reg._h, o))
        finally:
            self._free_opt(o)
        return reg

    def deregister_memory(self, dereg_list, backends=()):
        o = self._opt_args(backends)
        try:
            _check("deregister_memory", self._lib.nixl_capi_deregister_mem(self._h, dereg_list._h, o))
        finally:
            self._free_opt(o)

    # -- transfers --------------------------------------------------------------------
    def prep_xfer_dlist(self, agent_name, xfer_list, mem_type=None, backends=()):
        descs = self.get_xfer_descs(xfer_list, mem_type)
        if agent_name == "NIXL_INIT_AGENT":
            agent_name = NIXL_INIT_AGENT
        o = self._opt_args(backends)
        h = ctypes.c_void_p()
        try:
            _check("prep_xfer_dlist",
                   self._lib.nixl_capi_prep_xfer_dlist(self._h, agent_name.encode(), descs._h, ctypes.byref(h), o))
        finally:
            self._free_opt(o)
        return nixl_prepped_dlist_handle(self, h)

    def make_prepped_xfer(self, operation, local_xfer_side, local_indices, remote_xfer_side,
                          remote_indices, notif_msg=b"", backends=(), skip_desc_merge=False):
        li = np.ascontiguousarray(local_indices, dtype=np.int32)
        ri = np.ascontiguousarray(remote_indices, dtype=np.int32)
        o = self._opt_args(backends, skip_desc_merge, notif_msg)
        h = ctypes.c_void_p()
        try:
            _check("make_prepped_xfer",
                   self._lib.nixl_capi_make_xfer_req(self._h, self.nixl_ops[operation], local_xfer_side._handle,
                                                     li.ctypes.data, li.size, remote_xfer_side._handle,
                                                     ri.ctypes.data, ri.size, ctypes.byref(h), o))
        finally:
            self._free_opt(o)
        return nixl_xfer_handle(self, h)

    def initialize_xfer(self, operation, local_descs, remote_descs, remote_agent, notif_msg=b"", backends=()):
        o = self._opt_args(backends, False, notif_msg)
        h = ctypes.c_void_p()
        try:
            _check("initialize_xfer",
                   self._lib.nixl_capi_create_xfer_req(self._h, self.nixl_ops[operation], local_descs._h,
                                                       remote_descs._h, remote_agent.encode(), ctypes.byref(h), o))
        finally:
            self._free_opt(o)
        return nixl_xfer_handle(self, h)

    @staticmethod
    def _state(rc):
        return "DONE" if rc == 0 else ("PROC" if rc == 1 else "ERR")

    def transfer(self, handle, notif_msg=b""):
        o = self._opt_args((), False, notif_msg)
        try:
            return self._state(self._lib.nixl_capi_post_xfer_req(self._h, handle._handle, o))
        finally:
            self._free_opt(o)

    def check_xfer_state(self, handle):
        return self._state(self._lib.nixl_capi_get_xfer_status(self._h, handle._handle))

    def transfer_and_wait(self, handle):
        """Post and poll to completion inside native code (no reference counterpart)."""
        return self._state(self._lib.nixl_capi_post_and_wait(self._h, handle._handle))

    def last_status(self):
        return self._lib.nixl_capi_last_nixl_status()

    def get_xfer_telemetry(self, handle):
        t = _lib.XferTelemetry()
        _check("get_xfer_telemetry", self._lib.nixl_capi_get_xfer_telemetry(self._h, handle._handle, ctypes.byref(t)))
        return t

    def release_xfer_handle(self, handle):
        _check("release_xfer_handle", self._lib.nixl_capi_release_xfer_req(self._h, handle._handle))
        self._lib.nixl_capi_destroy_xfer_req(handle._handle)
        handle._handle = None

    def release_dlist_handle(self, handle):
        _check("release_dlist_handle", self._lib.nixl_capi_release_xfer_dlist_handle(self._h, handle._handle))
        handle._handle = None
