"""Metadata exchange and notifications between agents of one process, on the CPU.

The agent code under test is the product's (libnixl_amd_agent.so); the backend is the memcpy
oracle plugin with peer_agents=1, which treats other agents of the process as remote peers
the same way the HIP backend does.  What is pinned here:

  * the metadata blob, byte for byte, against the reference's wire format restated by hand
    from src/utils/serdes/serdes.cpp:36-46,85-93 (item = tag | 8-byte length | payload | '|'),
    src/core/nixl_agent.cpp:1446-1500 (Agent, Conns, t/c pairs, "MemSection"),
    src/infra/nixl_memory_section.cpp:333-363 (nixlSecElms, bknd) and
    src/infra/nixl_descriptors.cpp:236-282 (nixlDList / t / n / one item per descriptor =
    24-byte nixlBasicDesc + the backend's public data);
  * the two-agent cases of the reference's test/python/test_nixl_api.py (:56-70 connected
    agents, :163-175 metadata pass returns the peer's name, :178-186 an empty tag consumes any
    message, :385-412 WRITE with a notification that check_remote_xfer_done finds) and of
    examples/python/partial_md_example.py (partial metadata, then the rest).
"""
import os
import struct

import numpy as np
import pytest

from nixl_amd import agent as ag
from nixl_amd.agent import nixl_agent, nixl_agent_config


def _agent(name, plugin_dir, peers=True):
    a = nixl_agent(name, nixl_agent_config(backends=()), plugin_dirs=[plugin_dir])
    a.create_backend("MEMCPY", {"peer_agents": "1"} if peers else {})
    return a


@pytest.fixture()
def two_agents(oracle_plugin_dir):
    a, b = _agent("alpha", oracle_plugin_dir), _agent("beta", oracle_plugin_dir)
    yield a, b
    a.close()
    b.close()


def _item(tag, payload):
    return tag + struct.pack("<Q", len(payload)) + payload + b"|"


def _reg(agent, buf):
    return agent.register_memory(np.array([[buf.ctypes.data, buf.nbytes, 0]], dtype=np.uint64), "DRAM")


def _descs(agent, buf, offs, lens):
    rows = [(buf.ctypes.data + o, l, 0) for o, l in zip(offs, lens)]
    return agent.get_xfer_descs(np.array(rows, dtype=np.uint64), "DRAM")


def _wait(agent, handle):
    state = agent.transfer(handle)
    while state == "PROC":
        state = agent.check_xfer_state(handle)
    assert state == "DONE"


def test_metadata_blob_is_the_reference_wire_format(two_agents):
    a, _ = two_agents
    x = np.zeros(4096, np.uint8)
    y = np.zeros(512, np.uint8)
    first, second = sorted([x, y], key=lambda t: t.ctypes.data)
    _reg(a, x)
    _reg(a, y)
    blob = a.get_agent_metadata()

    def region(t):
        basic = struct.pack("<QQQ", t.ctypes.data, t.nbytes, 0)
        public = struct.pack("<QQ", t.ctypes.data, t.nbytes)  # what the memcpy backend publishes
        return _item(b"", basic + public)

    want = (b"nixlSerDes|" + _item(b"Agent", b"alpha") + _item(b"Conns", struct.pack("<Q", 1)) +
            _item(b"t", b"MEMCPY") + _item(b"c", b"MEMCPY1:pid=%d" % os.getpid()) + _item(b"", b"MemSection") +
            _item(b"nixlSecElms", struct.pack("<Q", 1)) + _item(b"bknd", b"MEMCPY") +
            _item(b"nixlDList", b"nixlSDList") + _item(b"t", struct.pack("<i", 0)) + _item(b"n", struct.pack("<Q", 2)) +
            region(first) + region(second))
    assert blob == want

    # connection info alone: no descriptors, no sections
    empty = ag.nixl_reg_dlist(np.zeros((0, 3), np.uint64), 0)
    only_conn = a.get_partial_agent_metadata(empty)
    assert only_conn == (b"nixlSerDes|" + _item(b"Agent", b"alpha") + _item(b"Conns", struct.pack("<Q", 1)) +
                         _item(b"t", b"MEMCPY") + _item(b"c", b"MEMCPY1:pid=%d" % os.getpid()) +
                         _item(b"", b"MemSection") + _item(b"nixlSecElms", struct.pack("<Q", 0)))
    # one region, without connection info unless asked for
    one = ag.nixl_reg_dlist(np.array([[y.ctypes.data, y.nbytes, 0]], dtype=np.uint64), 0)
    part = a.get_partial_agent_metadata(one)
    assert part == (b"nixlSerDes|" + _item(b"Agent", b"alpha") + _item(b"Conns", struct.pack("<Q", 0)) +
                    _item(b"", b"MemSection") + _item(b"nixlSecElms", struct.pack("<Q", 1)) + _item(b"bknd", b"MEMCPY") +
                    _item(b"nixlDList", b"nixlSDList") + _item(b"t", struct.pack("<i", 0)) +
                    _item(b"n", struct.pack("<Q", 1)) + region(y))
    with_conn = a.get_partial_agent_metadata(one, inc_conn_info=True)
    assert _item(b"Conns", struct.pack("<Q", 1)) in with_conn and with_conn.endswith(region(y))
    # a region that was never registered cannot be published
    stray = np.zeros(64, np.uint8)
    with pytest.raises(ag.NixlError) as e:
        a.get_partial_agent_metadata(ag.nixl_reg_dlist(np.array([[stray.ctypes.data, 64, 0]], dtype=np.uint64), 0))
    assert e.value.status == ag.NIXL_ERR_NOT_FOUND


def test_a_backend_without_remote_support_has_no_metadata(oracle_plugin_dir):
    a = _agent("solo", oracle_plugin_dir, peers=False)
    with pytest.raises(ag.NixlError) as e:
        a.get_agent_metadata()
    assert e.value.status == ag.NIXL_ERR_INVALID_PARAM  # src/core/nixl_agent.cpp:1455-1458
    with pytest.raises(ag.NixlError) as e:
        a.get_new_notifs()
    assert e.value.status == ag.NIXL_ERR_BACKEND  # no backend supports notifications, :1335-1338
    a.close()


def test_write_with_notification_then_read_between_two_agents(two_agents):
    a, b = two_agents
    rng = np.random.default_rng(11)
    src = rng.integers(0, 256, 1 << 16, dtype=np.uint8)
    dst = np.zeros(1 << 16, np.uint8)
    _reg(a, src)
    _reg(b, dst)
    assert not a.check_remote_metadata("beta")
    assert a.add_remote_agent(b.get_agent_metadata()) == "beta"
    assert a.check_remote_metadata("beta")
    assert a.check_remote_metadata("beta", _descs(a, dst, [128], [256]))
    assert not a.check_remote_metadata("beta", _descs(a, src, [128], [256]))  # a region beta never registered
    a.make_connection("beta")

    offs = [0, 8192, 20000, 65000]
    lens = [4096, 10000, 33, 536]
    h = a.initialize_xfer("WRITE", _descs(a, src, offs, lens), _descs(a, dst, offs, lens), "beta", b"kv block 7 written")
    assert b.get_new_notifs() == {}
    _wait(a, h)
    want = np.zeros_like(dst)
    for o, l in zip(offs, lens):
        want[o:o + l] = src[o:o + l]
    assert np.array_equal(dst, want)
    assert b.get_new_notifs() == {"alpha": [b"kv block 7 written"]}
    assert b.get_new_notifs() == {}  # handed out once
    assert a.get_new_notifs() == {}  # the initiator gets none

    # reposting repeats the notification; one given to transfer() replaces it (:1144-1156)
    _wait(a, h)
    assert a.transfer(h, b"second form") in ("DONE", "PROC")
    while a.check_xfer_state(h) == "PROC":
        pass
    assert b.update_notifs() == {"alpha": [b"kv block 7 written", b"second form"]}
    assert b.check_remote_xfer_done("alpha", b"second")  # prefix
    assert not b.check_remote_xfer_done("alpha", b"block")  # not a prefix
    assert b.check_remote_xfer_done("alpha", b"block", tag_is_prefix=False)
    assert b.notifs == {"alpha": []}
    a.release_xfer_handle(h)

    # READ pulls beta's bytes into alpha's buffer
    dst[:] = rng.integers(0, 256, dst.size, dtype=np.uint8)
    h = a.initialize_xfer("READ", _descs(a, src, [100], [5000]), _descs(a, dst, [30000], [5000]), "beta")
    _wait(a, h)
    assert np.array_equal(src[100:5100], dst[30000:35000])
    assert b.get_new_notifs() == {}
    a.release_xfer_handle(h)

    # prepared lists against the peer
    local = a.prep_xfer_dlist("NIXL_INIT_AGENT", _descs(a, src, [0, 4096, 8192], [4096] * 3))
    remote = a.prep_xfer_dlist("beta", _descs(a, dst, [0, 4096, 8192], [4096] * 3))
    h = a.make_prepped_xfer("WRITE", local, [2, 0], remote, [0, 1], b"prepped")
    _wait(a, h)
    assert np.array_equal(dst[0:4096], src[8192:12288]) and np.array_equal(dst[4096:8192], src[0:4096])
    assert b.check_remote_xfer_done("alpha", b"")  # an empty tag consumes any message
    a.release_xfer_handle(h)


def test_standalone_notifications(two_agents):
    a, b = two_agents
    a.add_remote_agent(b.get_agent_metadata())
    b.add_remote_agent(a.get_agent_metadata())
    a.send_notif("beta", b"whatever")
    a.send_notif("beta", "text works too")
    b.send_notif("alpha", b"\x00\x01binary\xff")
    a.send_notif("alpha", b"to myself")
    assert b.get_new_notifs() == {"alpha": [b"whatever", b"text works too"]}
    assert a.get_new_notifs(backends=["MEMCPY"]) == {"beta": [b"\x00\x01binary\xff"], "alpha": [b"to myself"]}
    with pytest.raises(ag.NixlError) as e:
        a.send_notif("gamma", b"nobody there")
    assert e.value.status == ag.NIXL_ERR_NOT_FOUND


def test_removing_and_refusing_peers(two_agents, oracle_plugin_dir):
    a, b = two_agents
    x, y = np.zeros(4096, np.uint8), np.zeros(4096, np.uint8)
    _reg(a, x)
    _reg(b, y)
    md_b = b.get_agent_metadata()
    # an agent does not load its own metadata (src/core/nixl_agent.cpp:1627-1631)
    with pytest.raises(ag.NixlError) as e:
        b.add_remote_agent(md_b)
    assert e.value.status == ag.NIXL_ERR_INVALID_PARAM
    for bad in (b"garbage", md_b[:40], md_b[:-9], md_b.replace(b"MemSection", b"MemSectioX")):
        with pytest.raises(ag.NixlError) as e:
            a.add_remote_agent(bad)
        assert e.value.status in (ag.NIXL_ERR_MISMATCH, ag.NIXL_ERR_NOT_FOUND, ag.NIXL_ERR_INVALID_PARAM), bad
        assert not a.check_remote_metadata("beta")
    assert a.add_remote_agent(md_b) == "beta"
    assert a.add_remote_agent(md_b) == "beta"  # the same metadata again is accepted
    l, r = _descs(a, x, [0], [64]), _descs(a, y, [0], [64])
    h = a.initialize_xfer("WRITE", l, r, "beta")
    a.remove_remote_agent("beta")
    assert not a.check_remote_metadata("beta")
    assert a.transfer(h) == "ERR" and a.last_status() == ag.NIXL_ERR_NOT_FOUND
    a.release_xfer_handle(h)
    with pytest.raises(ag.NixlError) as e:
        a.initialize_xfer("WRITE", l, r, "beta")
    assert e.value.status == ag.NIXL_ERR_NOT_FOUND
    with pytest.raises(ag.NixlError) as e:
        a.remove_remote_agent("beta")
    assert e.value.status == ag.NIXL_ERR_NOT_FOUND
    with pytest.raises(ag.NixlError) as e:
        a.remove_remote_agent("alpha")  # not itself, :1806-1809
    assert e.value.status == ag.NIXL_ERR_INVALID_PARAM
    with pytest.raises(ag.NixlError):
        a.make_connection("beta")
    # a peer without a common backend: its metadata names a backend this agent lacks
    alien = md_b.replace(b"MEMCPY", b"MEMCPX")
    with pytest.raises(ag.NixlError) as e:
        a.add_remote_agent(alien)
    assert e.value.status == ag.NIXL_ERR_BACKEND  # "no common backend found", :1660-1663
    # metadata from another process is no use to a backend that shares an address space
    other = md_b.replace(b"pid=%d" % os.getpid(), b"pid=%d" % (os.getpid() + 1))
    with pytest.raises(ag.NixlError) as e:
        a.add_remote_agent(other)
    assert e.value.status == ag.NIXL_ERR_BACKEND


def test_partial_metadata_then_the_rest(two_agents):
    """examples/python/partial_md_example.py: the target publishes one region, the initiator can
    reach only that one; after the second region is published too, both."""
    a, b = two_agents
    src = np.arange(8192, dtype=np.uint8)
    r1, r2 = np.zeros(4096, np.uint8), np.zeros(4096, np.uint8)
    _reg(a, src)
    reg1, reg2 = _reg(b, r1), _reg(b, r2)
    assert a.add_remote_agent(b.get_partial_agent_metadata(reg1, inc_conn_info=True)) == "beta"
    assert a.check_remote_metadata("beta", _descs(a, r1, [0], [4096]))
    assert not a.check_remote_metadata("beta", _descs(a, r2, [0], [4096]))
    h = a.initialize_xfer("WRITE", _descs(a, src, [0], [4096]), _descs(a, r1, [0], [4096]), "beta")
    _wait(a, h)
    a.release_xfer_handle(h)
    assert np.array_equal(r1, src[:4096])
    with pytest.raises(ag.NixlError):
        a.initialize_xfer("WRITE", _descs(a, src, [4096], [4096]), _descs(a, r2, [0], [4096]), "beta")
    assert a.add_remote_agent(b.get_partial_agent_metadata(reg2)) == "beta"
    h = a.initialize_xfer("WRITE", _descs(a, src, [4096], [4096]), _descs(a, r2, [0], [4096]), "beta")
    _wait(a, h)
    a.release_xfer_handle(h)
    assert np.array_equal(r2, src[4096:])


def test_two_peers_through_the_cpp_api(oracle_plugin_dir):
    """The same exchange through nixlAgent from C++ (tests/cpp/agent_two_peers_check.cpp, the
    flow of the reference's examples/cpp/nixl_example.cpp), three generations of agents."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "cpp", "_build", "agent_two_peers_check")
    if not os.path.exists(exe):
        pytest.fail(f"{exe} missing: run __graft_entry__.build() first")
    proc = subprocess.run([exe, oracle_plugin_dir], capture_output=True, text=True, timeout=60)
    assert proc.returncode == 0 and proc.stdout.strip().endswith("OK"), proc.stdout + proc.stderr


def test_memory_view_lists_resolve_through_the_agent(two_agents):
    """prepMemView on the CPU: the agent resolves a local list against its own registrations
    and a remote list against the loaded metadata of each named peer, keeps placeholders, and
    refuses what it cannot resolve (src/core/nixl_agent.cpp:1906-2036; the reference's unit
    test PrepMemViewRemoteDRAM, test/gtest/unit/agent/agent.cpp:436-448).  The memcpy backend
    builds the table in host memory in the HIP backend's layout, which is read back here."""
    import ctypes
    a, b = two_agents
    mine, theirs = np.zeros(8192, np.uint8), np.zeros(4096, np.uint8)
    _reg(a, mine)
    _reg(b, theirs)

    def table(mvh, n):
        return list((ctypes.c_uint64 * (2 + 2 * n)).from_address(mvh))

    magic = 0x5649584C
    lv = a.prep_mem_view(_descs(a, mine, [0, 4096], [4096, 100]))
    assert table(lv, 2) == [magic, 2, mine.ctypes.data, 4096, mine.ctypes.data + 4096, 100]
    # the peer is unknown until its metadata is loaded
    remote = a.get_remote_descs([(theirs.ctypes.data + 16, 64, 0, "beta"), (0, 0, 0, None),
                                 (mine.ctypes.data, 8192, 0, "alpha")], "DRAM")
    with pytest.raises(ag.NixlError) as e:
        a.prep_mem_view(remote)
    assert e.value.status == ag.NIXL_ERR_NOT_FOUND
    a.add_remote_agent(b.get_agent_metadata())
    rv = a.prep_mem_view(remote)
    assert table(rv, 3) == [magic | (1 << 32), 3, theirs.ctypes.data + 16, 64, 0, 0, mine.ctypes.data, 8192]
    a.release_mem_view(rv)
    a.release_mem_view(lv)
    a.release_mem_view(lv)  # a handle the agent no longer knows is ignored (logged)
    for bad in ([(theirs.ctypes.data, 4097, 0, "beta")],          # longer than the registration
                [(mine.ctypes.data, 64, 0, "beta")],               # alpha's memory under beta's name
                [(0, 0, 0, None)]):                                # placeholders alone name no backend
        with pytest.raises(ag.NixlError) as e:
            a.prep_mem_view(a.get_remote_descs(bad, "DRAM"))
        assert e.value.status == ag.NIXL_ERR_NOT_FOUND
    with pytest.raises(ag.NixlError):
        a.prep_mem_view(_descs(a, theirs, [0], [64]))  # beta's memory is not a local registration
    # views left unreleased are freed with the agent
    a.prep_mem_view(_descs(a, mine, [0], [64]))


def test_agents_used_from_several_threads(oracle_plugin_dir):
    """tests/cpp/agent_threads_check.cpp: transfers with notifications, memory views,
    registration and metadata calls from six threads at once; every notification arrives once."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "cpp", "_build", "agent_threads_check")
    if not os.path.exists(exe):
        pytest.fail(f"{exe} missing: run __graft_entry__.build() first")
    proc = subprocess.run([exe, oracle_plugin_dir], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0 and proc.stdout.strip().endswith("OK"), proc.stdout + proc.stderr


def test_notification_ring_of_the_hip_backend_on_the_cpu():
    """tests/cpp/mailbox_check.cpp: the shared-memory ring that carries notifications between
    processes (nixl_amd/csrc/plugin/mailbox.h), fed by four threads and a child process at
    once: every message arrives once, in each producer's order, bytes intact; full ring,
    oversize message, taken name and foreign object are refused."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "cpp", "_build", "mailbox_check")
    if not os.path.exists(exe):
        pytest.fail(f"{exe} missing: run __graft_entry__.build() first")
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0 and proc.stdout.strip().endswith("OK"), proc.stdout + proc.stderr


def test_helper_threads_of_the_hip_backend_on_the_cpu():
    """tests/cpp/worker_pool_check.cpp: the helper threads that share prepXfer's pass over a long
    request (nixl_amd/csrc/plugin/worker_pool.h): every slice of every job runs exactly once,
    a second caller is turned away while the pool is busy, competing callers lose nothing, and
    the pool shuts down with its helpers polling or asleep."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "cpp", "_build", "worker_pool_check")
    if not os.path.exists(exe):
        pytest.fail(f"{exe} missing: run __graft_entry__.build() first")
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0 and proc.stdout.strip().endswith("OK"), proc.stdout + proc.stderr


def test_list_and_option_helpers_of_the_c_wrapper(two_agents):
    """The descriptor-list, option and stub helpers of the reference's C wrapper
    (src/bindings/rust/wrapper.h:193-201,297-326,457) behave as their names say; the metadata
    side channels that need sockets or ETCD answer with an error instead of being absent."""
    import ctypes
    from nixl_amd import _lib
    lib = _lib.agent_lib()
    a, _ = two_agents
    buf = np.zeros(4096, np.uint8)
    x = a.get_xfer_descs(np.array([[buf.ctypes.data, 64, 0], [buf.ctypes.data + 64, 64, 0]], dtype=np.uint64), "DRAM")
    n, empty, mem = ctypes.c_size_t(), ctypes.c_bool(), ctypes.c_int()
    assert lib.nixl_capi_xfer_dlist_len(x._h, ctypes.byref(n)) == 0 and n.value == 2
    assert lib.nixl_capi_xfer_dlist_get_type(x._h, ctypes.byref(mem)) == 0 and mem.value == 0
    assert lib.nixl_capi_xfer_dlist_rem_desc(x._h, 0) == 0
    assert lib.nixl_capi_xfer_dlist_rem_desc(x._h, 5) != 0  # out of range: an error, not a crash
    assert lib.nixl_capi_xfer_dlist_len(x._h, ctypes.byref(n)) == 0 and n.value == 1
    assert lib.nixl_capi_xfer_dlist_resize(x._h, 3) == 0 and lib.nixl_capi_xfer_dlist_trim(x._h) == 0
    assert lib.nixl_capi_xfer_dlist_len(x._h, ctypes.byref(n)) == 0 and n.value == 3
    assert lib.nixl_capi_xfer_dlist_is_empty(x._h, ctypes.byref(empty)) == 0 and not empty.value
    r = ag.nixl_reg_dlist(np.array([[buf.ctypes.data, 4096, 0]], dtype=np.uint64), 0)
    assert lib.nixl_capi_reg_dlist_get_type(r._h, ctypes.byref(mem)) == 0 and mem.value == 0
    assert lib.nixl_capi_reg_dlist_clear(r._h) == 0
    assert lib.nixl_capi_reg_dlist_is_empty(r._h, ctypes.byref(empty)) == 0 and empty.value
    o = ctypes.c_void_p()
    assert lib.nixl_capi_create_opt_args(ctypes.byref(o)) == 0
    flag, data, size = ctypes.c_bool(True), ctypes.c_void_p(), ctypes.c_size_t()
    assert lib.nixl_capi_opt_args_get_has_notif(o, ctypes.byref(flag)) == 0 and not flag.value
    assert lib.nixl_capi_opt_args_get_notif_msg(o, ctypes.byref(data), ctypes.byref(size)) == 0 and not data.value
    assert lib.nixl_capi_opt_args_set_notif_msg(o, b"m\x00sg", 4) == 0 and lib.nixl_capi_opt_args_set_has_notif(o, True) == 0
    assert lib.nixl_capi_opt_args_get_notif_msg(o, ctypes.byref(data), ctypes.byref(size)) == 0
    assert ctypes.string_at(data, size.value) == b"m\x00sg"
    lib.nixl_capi_free_buffer(data)
    assert lib.nixl_capi_opt_args_get_has_notif(o, ctypes.byref(flag)) == 0 and flag.value
    assert lib.nixl_capi_opt_args_set_skip_desc_merge(o, True) == 0
    assert lib.nixl_capi_opt_args_get_skip_desc_merge(o, ctypes.byref(flag)) == 0 and flag.value
    assert lib.nixl_capi_opt_args_set_ip_addr(o, b"127.0.0.1") == 0 and lib.nixl_capi_opt_args_set_port(o, 5555) == 0
    for call in (lambda: lib.nixl_capi_send_local_md(a._h, o), lambda: lib.nixl_capi_fetch_remote_md(a._h, b"beta", o),
                 lambda: lib.nixl_capi_invalidate_local_md(a._h, o), lambda: lib.nixl_capi_send_local_partial_md(a._h, r._h, o)):
        assert call() != 0 and a.last_status() == ag.NIXL_ERR_NOT_SUPPORTED
    lib.nixl_capi_destroy_opt_args(o)
    assert lib.nixl_capi_is_stub() == 0


def test_request_handles_are_destroyed_only_after_release(two_agents):
    """src/bindings/rust/wrapper.cpp:1586-1612: destroying a request wrapper that still owns
    its request is an INVALID_STATE error (nothing is freed), releasing it twice an
    INVALID_PARAM error."""
    from nixl_amd import _lib
    lib = _lib.agent_lib()
    a, _ = two_agents
    src, dst = np.arange(4096, dtype=np.uint8) % 251, np.zeros(4096, np.uint8)
    _reg(a, src)
    _reg(a, dst)
    req = a.initialize_xfer("WRITE", _descs(a, src, [0], [4096]), _descs(a, dst, [0], [4096]), "alpha")
    _wait(a, req)
    assert np.array_equal(src, dst)
    assert lib.nixl_capi_destroy_xfer_req(req._handle) == -3  # NIXL_CAPI_ERROR_INVALID_STATE: still owned
    _wait(a, req)  # and still usable
    assert lib.nixl_capi_release_xfer_req(a._h, req._handle) == 0
    assert lib.nixl_capi_release_xfer_req(a._h, req._handle) == -1  # NIXL_CAPI_ERROR_INVALID_PARAM: released before
    assert lib.nixl_capi_destroy_xfer_req(req._handle) == 0
    req._handle = None  # nothing left for the Python wrapper to release


def test_descriptor_lists_as_bytes_and_absent_side_channels(two_agents):
    """get_serialized_descs / deserialize_descs (reference _api.py:1201-1221; the reference
    pickles, this build writes a flat record) and the socket / ETCD metadata calls, which say
    that they are not offered."""
    a, b = two_agents
    buf = np.zeros(8192, np.uint8)
    _reg(b, buf)
    _reg(a, buf)
    x = _descs(a, buf, [0, 4096], [100, 200])
    wire = a.get_serialized_descs(x)
    y = b.deserialize_descs(wire)
    assert isinstance(y, ag.nixl_xfer_dlist) and y.mem == x.mem and np.array_equal(y.triples, x.triples)
    h = b.prep_xfer_dlist("NIXL_INIT_AGENT", y)  # usable as a list
    h.release()
    r = ag.nixl_reg_dlist(np.array([[buf.ctypes.data, 8192, 0]], dtype=np.uint64), 0)
    assert isinstance(a.deserialize_descs(a.get_serialized_descs(r)), ag.nixl_reg_dlist)
    for bad in (b"", wire[:-1], b"XXXXX" + wire[5:], wire + b"\x00", wire[:5] + bytes([9]) + wire[6:]):
        with pytest.raises(ValueError):
            a.deserialize_descs(bad)
    for call in (a.send_local_metadata, lambda: a.fetch_remote_metadata("beta"), a.invalidate_local_metadata,
                 lambda: a.send_partial_agent_metadata(r)):
        with pytest.raises(ag.NixlError) as e:
            call()
        assert e.value.status == ag.NIXL_ERR_NOT_SUPPORTED
