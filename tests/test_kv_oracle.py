"""CPU tests: the descriptor-transfer oracle against what the reference's own tests state,
and the C++ agent against the oracle (no GPU)."""
import numpy as np
import pytest

from oracle import kv_oracle as ko
from nixl_amd import NixlError, nixl_agent, nixl_agent_config
from nixl_amd import agent as ag


# ---- oracle pinned by reference-held expectations ----------------------------------------

def _regions_and_descs(n_regions, per_region, desc_len, base=1 << 20, gap=4096):
    regions, descs = [], []
    for r in range(n_regions):
        start = base + r * (per_region * desc_len + gap)
        regions.append((start, per_region * desc_len, 0))
        descs += [(start + i * desc_len, desc_len, 0) for i in range(per_region)]
    return regions, descs


def test_oracle_merge_counts_match_reference_example():
    # test/nixl/agent_example.cpp:45-153 (test_side_perf): 32 registered regions, each cut
    # into contiguous 8-byte descriptors.  All indices in order -> one descriptor per
    # region (:142-144); every other index -> n/2 descriptors, nothing merges (:147-152).
    # Scaled from 65536 to 2048 descriptors per region to keep the Python loops short.
    regions, descs = _regions_and_descs(32, 2048, 8)
    runs = ko.stride_runs(descs, regions)
    assert len(runs) == 32 and all(r["stride"] == 8 and r["count"] == 2048 for r in runs)
    n = len(descs)
    merged = ko.expand_and_merge(runs, runs, range(n), range(n))
    assert len(merged) == 32
    assert all(l == 2048 * 8 for _, _, l in merged)
    every_other = list(range(0, n, 2))
    assert len(ko.expand_and_merge(runs, runs, every_other, every_other)) == n // 2
    assert len(ko.expand_and_merge(runs, runs, range(n), range(n), skip_merge=True)) == n


def test_oracle_merge_is_byte_equivalent_to_unmerged():
    rng = np.random.default_rng(7)
    for trial in range(50):
        regions, descs = _regions_and_descs(int(rng.integers(1, 4)), int(rng.integers(1, 9)), 16)
        rregions, rdescs = _regions_and_descs(int(rng.integers(1, 4)), int(rng.integers(1, 9)), 16, base=1 << 24)
        lr, rr = ko.stride_runs(descs, regions), ko.stride_runs(rdescs, rregions)
        m = int(rng.integers(1, 12))
        # mix of ascending stretches and random picks
        li = [int(x) for x in rng.integers(0, len(descs), m)]
        ri = [int(x) for x in rng.integers(0, len(rdescs), m)]
        if trial % 2 == 0:
            k = min(len(descs), len(rdescs), m)
            li[:k] = range(k)
            ri[:k] = range(k)
        merged = ko.expand_and_merge(lr, rr, li, ri)
        flat = ko.expand_and_merge(lr, rr, li, ri, skip_merge=True)
        def cover(lst):
            out = []
            for la, ra, ln in lst:
                out += [(la + o, ra + o) for o in range(0, ln, 16)]
            return out
        assert cover(merged) == cover(flat)
        assert flat == [(descs[a][0], rdescs[b][0], 16) for a, b in zip(li, ri)]


def test_oracle_stride_runs_break_rules():
    regions = [(1000, 10000, 0)]
    # equal stride continues, change of stride / len / going backwards starts a new run
    descs = [(1000, 16, 0), (1064, 16, 0), (1128, 16, 0), (1160, 16, 0), (1100, 16, 0), (1300, 32, 0)]
    runs = ko.stride_runs(descs, regions)
    assert [(r["start_idx"], r["count"], r["stride"]) for r in runs] == \
        [(0, 3, 64), (3, 1, 16), (4, 1, 16), (5, 1, 32)]
    assert ko.stride_runs([(500, 16, 0)], regions) is None
    assert ko.stride_runs([(1000, 16, 1)], regions) is None


def test_oracle_copy_direction_and_canary():
    rng = np.random.default_rng(1)
    mem = rng.integers(0, 256, 4096, dtype=np.uint8)
    before = mem.copy()
    ko.copy_descs(mem, [0, 100], [2048, 3000], [64, 7])
    assert np.array_equal(mem[2048:2112], before[0:64]) and np.array_equal(mem[3000:3007], before[100:107])
    touched = np.zeros(4096, bool)
    touched[2048:2112] = True
    touched[3000:3007] = True
    assert np.array_equal(mem[~touched], before[~touched])


# ---- C++ agent against the oracle -----------------------------------------------------------

@pytest.fixture()
def cpu_agent(oracle_plugin_dir):
    a = nixl_agent("agent", nixl_agent_config(backends=()), plugin_dirs=[oracle_plugin_dir])
    a.create_backend("MEMCPY")
    yield a
    a.close()


def _np_descs(buf, offs, lens):
    offs = np.asarray(offs, dtype=np.uint64)
    lens = np.asarray(lens, dtype=np.uint64)
    return np.stack([np.uint64(buf.ctypes.data) + offs, lens, np.zeros_like(offs)], 1)


def test_agent_runs_and_merge_match_oracle(cpu_agent):
    rng = np.random.default_rng(3)
    a = cpu_agent
    bufs = [np.zeros(1 << 16, np.uint8) for _ in range(4)]
    for b in bufs:
        a.register_memory(_np_descs(b, [0], [b.nbytes]), "DRAM")
    regions = [(b.ctypes.data, b.nbytes, 0) for b in bufs]
    for trial in range(30):
        def side():
            n = int(rng.integers(1, 40))
            ln = int(rng.choice([16, 64, 256]))
            out = []
            while len(out) < n:
                b = bufs[int(rng.integers(0, 4))]
                k = int(rng.integers(1, 8))
                stride = ln * int(rng.choice([1, 1, 2]))
                start = int(rng.integers(0, (b.nbytes - k * stride) // 16)) * 16
                out += [(b.ctypes.data + start + j * stride, ln, 0) for j in range(k)]
            return out[:n], ln
        ld, ln = side()
        rd, _ = side()
        rd = [(x[0], ln, 0) for x in rd]
        rd = [d for d in rd if any(ko._covers(r, d) for r in regions)]
        ld = ld[:len(rd)]
        if not ld:
            continue
        hl = a.prep_xfer_dlist("", np.array(ld, dtype=np.uint64), "DRAM")
        hr = a.prep_xfer_dlist("agent", np.array(rd, dtype=np.uint64), "DRAM")
        lruns, rruns = ko.stride_runs(ld, regions), ko.stride_runs(rd, regions)
        assert hl.run_count() == len(lruns) and hr.run_count() == len(rruns)
        m = int(rng.integers(1, 30))
        li = rng.integers(0, len(ld), m)
        ri = rng.integers(0, len(rd), m)
        k = min(len(ld), len(rd), m)
        if trial % 2:
            li[:k] = np.arange(k)
            ri[:k] = np.arange(k)
        for skip in (False, True):
            req = a.make_prepped_xfer("WRITE", hl, li, hr, ri, skip_desc_merge=skip)
            want = ko.expand_and_merge(lruns, rruns, li, ri, skip_merge=skip)
            n, nbytes = req.desc_count()
            assert n == len(want) and nbytes == sum(w[2] for w in want)
            assert [req.get_desc(i) for i in range(n)] == want
            req.release()
        hl.release()
        hr.release()


def test_agent_index_lookup_in_long_irregular_lists(cpu_agent):
    """Prepared lists of a few thousand descriptors that hardly compress (runs of one block with
    longer runs strewn in, on one side none at all): index vectors that ascend, descend, jump at
    random and repeat must expand to what the oracle's expansion gives, merged and unmerged.
    (The run look-up steps to the next run, guesses proportionally and brackets by doubling.)"""
    rng = np.random.default_rng(11)
    a = cpu_agent
    ln = 64
    bufs = [np.zeros(1 << 20, np.uint8) for _ in range(2)]
    for b in bufs:
        a.register_memory(_np_descs(b, [0], [b.nbytes]), "DRAM")
    regions = [(b.ctypes.data, b.nbytes, 0) for b in bufs]

    def side(buf, n, run_lengths):
        out, slot = [], 0
        while len(out) < n:
            k = int(rng.choice(run_lengths))
            out += [(buf.ctypes.data + (slot + j) * ln, ln, 0) for j in range(k)]
            slot += k + int(rng.integers(1, 4))  # a gap ends the run
        return out[:n]

    n = 3000
    for run_lengths in ([1, 1, 1, 1, 1, 1, 2], [1, 1, 1, 7, 30], [1]):
        ld, rd = side(bufs[0], n, run_lengths), side(bufs[1], n, [1, 2, 3])
        hl = a.prep_xfer_dlist("", np.array(ld, dtype=np.uint64), "DRAM")
        hr = a.prep_xfer_dlist("agent", np.array(rd, dtype=np.uint64), "DRAM")
        lruns, rruns = ko.stride_runs(ld, regions), ko.stride_runs(rd, regions)
        assert hl.run_count() == len(lruns) and hr.run_count() == len(rruns)
        walks = [(np.arange(n), np.arange(n)), (np.arange(n)[::-1].copy(), np.arange(n)),
                 (rng.integers(0, n, 2000), rng.integers(0, n, 2000)),
                 (np.repeat(rng.integers(0, n, 40), 5), np.sort(rng.integers(0, n, 200))),
                 (np.array([0, n - 1, 0, n - 1, n // 2]), np.array([n - 1, 0, n - 1, 0, 1]))]
        for li, ri in walks:
            for skip in (False, True):
                req = a.make_prepped_xfer("WRITE", hl, li, hr, ri, skip_desc_merge=skip)
                want = ko.expand_and_merge(lruns, rruns, li, ri, skip_merge=skip)
                count, nbytes = req.desc_count()
                assert count == len(want) and nbytes == sum(w[2] for w in want)
                assert [req.get_desc(i) for i in range(count)] == want
                req.release()
        hl.release()
        hr.release()


def test_agent_reference_example_merge_counts(cpu_agent):
    # Same known answers as test_oracle_merge_counts_match_reference_example, now for the
    # C++ agent at the reference's full size (32 x 65536 descriptors of 8 bytes).
    a = cpu_agent
    per, n_reg = 65536, 32
    bufs = [np.zeros(per * 8, np.uint8) for _ in range(n_reg)]
    for b in bufs:
        a.register_memory(_np_descs(b, [0], [b.nbytes]), "DRAM")
    descs = np.concatenate([_np_descs(b, np.arange(per) * 8, np.full(per, 8)) for b in bufs])
    hl = a.prep_xfer_dlist("", descs, "DRAM")
    hr = a.prep_xfer_dlist("agent", descs, "DRAM")
    # buffers may happen to be adjacent in memory, but each registration is its own run
    assert hl.run_count() == n_reg
    idx = np.arange(per * n_reg)
    req = a.make_prepped_xfer("WRITE", hl, idx, hr, idx)
    assert req.desc_count() == (n_reg, per * n_reg * 8)
    req.release()
    req = a.make_prepped_xfer("WRITE", hl, idx[::2], hr, idx[::2])
    assert req.desc_count()[0] == per * n_reg // 2
    req.release()
    hl.release()
    hr.release()


def test_agent_argument_errors(cpu_agent):
    a = cpu_agent
    buf = np.zeros(4096, np.uint8)
    other = np.zeros(4096, np.uint8)
    a.register_memory(_np_descs(buf, [0], [4096]), "DRAM")
    d16 = _np_descs(buf, [0, 16, 32], [16, 16, 16])
    d32 = _np_descs(buf, [64, 128], [32, 32])
    hl = a.prep_xfer_dlist("", d16, "DRAM")
    hr = a.prep_xfer_dlist("agent", d16, "DRAM")
    hr32 = a.prep_xfer_dlist("agent", d32, "DRAM")
    # unregistered memory cannot be prepared (src/core/nixl_agent.cpp:676-684)
    with pytest.raises(NixlError) as e:
        a.prep_xfer_dlist("", _np_descs(other, [0], [16]), "DRAM")
    assert e.value.status == ag.NIXL_ERR_NOT_FOUND
    # unknown remote agent (:634-639)
    with pytest.raises(NixlError) as e:
        a.prep_xfer_dlist("nobody", d16, "DRAM")
    assert e.value.status == ag.NIXL_ERR_NOT_FOUND
    # sides swapped, index counts differ, index out of range, length mismatch (:715-834)
    for args in ((hr, [0], hl, [0]), (hl, [0, 1], hr, [0]), (hl, [3], hr, [0]), (hl, [0], hr, [-1]), (hl, [0], hr32, [0])):
        with pytest.raises(NixlError) as e:
            a.make_prepped_xfer("WRITE", *args)
        assert e.value.status == ag.NIXL_ERR_INVALID_PARAM
    # one bad entry deep inside long index vectors, on either side: the whole request is refused
    long_ok = np.tile(np.arange(3, dtype=np.int32), 4000)
    for pos, value in ((4096 + 17, 3), (11999, -2**31), (0, 2**31 - 1)):
        for side in (0, 1):
            li, ri = long_ok.copy(), long_ok.copy()
            (li if side == 0 else ri)[pos] = value
            with pytest.raises(NixlError) as e:
                a.make_prepped_xfer("WRITE", hl, li, hr, ri)
            assert e.value.status == ag.NIXL_ERR_INVALID_PARAM
    # notifications are refused for a backend without them (:771-775)
    with pytest.raises(NixlError) as e:
        a.make_prepped_xfer("WRITE", hl, [0], hr, [1], notif_msg=b"x")
    assert e.value.status == ag.NIXL_ERR_BACKEND
    # createXferReq: list sizes and lengths must agree (src/core/nixl_agent.cpp:905-920)
    with pytest.raises(NixlError):
        a.initialize_xfer("WRITE", a.get_xfer_descs(d16, "DRAM"), a.get_xfer_descs(d32, "DRAM"), "agent")
    # a second backend of the same type is refused (:323-327); unknown plugin -> NOT_FOUND (:355-358)
    with pytest.raises(NixlError) as e:
        a.create_backend("MEMCPY")
    assert e.value.status == ag.NIXL_ERR_INVALID_PARAM
    with pytest.raises(NixlError) as e:
        a.create_backend("NO_SUCH_BACKEND")
    assert e.value.status == ag.NIXL_ERR_NOT_FOUND
    # deregistering something never registered: NOT_FOUND, nothing else is touched
    with pytest.raises(NixlError) as e:
        a.deregister_memory(a.get_reg_descs(_np_descs(other, [0], [4096]), "DRAM"))
    assert e.value.status == ag.NIXL_ERR_NOT_FOUND


def test_config1_dram_loopback_bit_exact(cpu_agent):
    # BASELINE config 1: one agent, loopback, 4096 descriptors x 16 KiB, destination block
    # ids = seeded permutation, NIXL_WRITE; byte-exact plus canary outside the ranges.
    a = cpu_agent
    n, ln = 4096, 16384
    rng = np.random.default_rng(2024)
    src = rng.integers(0, 256, n * ln, dtype=np.uint8)
    dst = np.full(n * ln + 4096, 0xAA, np.uint8)
    perm = rng.permutation(n)
    a.register_memory(_np_descs(src, [0], [src.nbytes]), "DRAM")
    a.register_memory(_np_descs(dst, [0], [dst.nbytes]), "DRAM")
    offs = np.arange(n, dtype=np.uint64) * ln
    hl = a.prep_xfer_dlist("", _np_descs(src, offs, np.full(n, ln)), "DRAM")
    hr = a.prep_xfer_dlist("agent", _np_descs(dst, offs, np.full(n, ln)), "DRAM")
    req = a.make_prepped_xfer("WRITE", hl, np.arange(n), hr, perm)
    assert a.transfer(req) in ("DONE", "PROC")
    while a.check_xfer_state(req) == "PROC":
        pass
    assert a.check_xfer_state(req) == "DONE"
    want = np.full_like(dst, 0xAA)
    want[:n * ln].reshape(n, ln)[perm] = src.reshape(n, ln)
    assert np.array_equal(dst, want)
    # READ through the same prepared lists brings the permuted blocks back
    back = np.zeros_like(src)
    a.register_memory(_np_descs(back, [0], [back.nbytes]), "DRAM")
    hb = a.prep_xfer_dlist("", _np_descs(back, offs, np.full(n, ln)), "DRAM")
    req2 = a.make_prepped_xfer("READ", hb, np.arange(n), hr, perm)
    a.transfer(req2)
    assert a.check_xfer_state(req2) == "DONE" and np.array_equal(back, src)
    for h in (req, req2, hl, hr, hb):
        h.release()


def test_sorted_region_list_matches_reference_expectations():
    """tests/cpp/sec_desc_list_check.cpp: the agent's registration list against the orderings
    the reference's unit tests state for nixlSecDescList, and the covering search on top."""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "cpp", "_build", "sec_desc_list_check")
    if not os.path.exists(exe):
        pytest.fail(f"{exe} missing: run __graft_entry__.build() first")
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert proc.returncode == 0 and proc.stdout.strip() == "OK", proc.stdout + proc.stderr


def test_api_behaviour_of_the_reference_python_tests(cpu_agent, oracle_plugin_dir):
    """Cases of the reference's test/python/test_nixl_api.py that concern one agent:
    empty name (:90-93), unknown operation (:135-142), unknown plugin name gives empty
    answers (:145-154) and cannot be created (:157-160), non-contiguous tensors (:358-371)."""
    import torch
    a = cpu_agent
    with pytest.raises(ValueError):
        nixl_agent("")
    x = np.zeros(256, np.uint8)
    reg = a.register_memory(np.array([[x.ctypes.data, x.nbytes, 0]], dtype=np.uint64), "DRAM")
    l = a.get_xfer_descs(np.array([[x.ctypes.data, 64, 0]], dtype=np.uint64), "DRAM")
    r = a.get_xfer_descs(np.array([[x.ctypes.data + 128, 64, 0]], dtype=np.uint64), "DRAM")
    with pytest.raises(KeyError):
        a.initialize_xfer("WR", l, r, a.name)
    with pytest.raises(KeyError):
        a.make_prepped_xfer("RD", None, [], None, [])
    assert a.get_plugin_mem_types("UVX") == [] and a.get_plugin_params("UVX") == {}
    assert a.get_backend_mem_types("UVX") == [] and a.get_backend_params("UVX") == {}
    with pytest.raises(ag.NixlError) as err:
        a.create_backend("UVX")
    assert err.value.status == ag.NIXL_ERR_NOT_FOUND
    # what a real plugin answers
    assert "MEMCPY" in a.get_plugin_list()
    assert a.get_plugin_mem_types("MEMCPY") == ["DRAM"] and a.get_plugin_params("MEMCPY") == {"threads": "1", "peer_agents": "0"}
    assert a.get_backend_mem_types("MEMCPY") == ["DRAM"]
    req = a.initialize_xfer("WRITE", l, r, a.name)
    assert a.query_xfer_backend(req) == "MEMCPY"
    req.release()
    a.deregister_memory(reg)
    cont = torch.arange(8).reshape(2, 4)
    assert a.get_reg_descs(torch.transpose(cont, 0, 1)) is None and a.get_xfer_descs(torch.transpose(cont, 0, 1)) is None
    assert a.get_xfer_descs(cont, "DRAM").descCount() == 1  # a single tensor, not only a list


def test_python_agent_follows_the_reference_signatures(oracle_plugin_dir, caplog):
    """Every public method of the reference's nixl_agent (src/api/python/_api.py:189-1160) is
    here with the same leading arguments in the same order, and the constructor behaves as
    _api.py:200-264: a configured backend without a plugin is skipped with a warning,
    instantiate_all creates every backend found, instantiate_all next to a configuration is
    ignored."""
    import inspect
    import logging
    from nixl_amd.agent import nixl_agent, nixl_agent_config
    reference = {
        "get_plugin_list": [], "get_plugin_mem_types": ["backend"], "get_plugin_params": ["backend"],
        "get_backend_mem_types": ["backend"], "get_backend_params": ["backend"],
        "create_backend": ["backend", "initParams"], "register_memory": ["reg_list", "mem_type", "backends"],
        "deregister_memory": ["dereg_list", "backends"], "query_memory": ["reg_list", "backend", "mem_type"],
        "make_connection": ["remote_agent", "backends"],
        "prep_xfer_dlist": ["agent_name", "xfer_list", "mem_type", "backends"], "estimate_xfer_cost": ["req_handle"],
        "make_prepped_xfer": ["operation", "local_xfer_side", "local_indices", "remote_xfer_side", "remote_indices",
                              "notif_msg", "backends", "skip_desc_merge"],
        "initialize_xfer": ["operation", "local_descs", "remote_descs", "remote_agent", "notif_msg", "backends"],
        "transfer": ["handle", "notif_msg"], "check_xfer_state": ["handle"], "get_xfer_telemetry": ["handle"],
        "query_xfer_backend": ["handle"], "release_xfer_handle": ["handle"], "release_dlist_handle": ["handle"],
        "prep_mem_view": ["dlist"], "release_mem_view": ["mvh"], "get_new_notifs": ["backends"],
        "update_notifs": ["backends"],
        "check_remote_xfer_done": ["remote_agent_name", "lookup_tag", "backends", "tag_is_prefix"],
        "send_notif": ["remote_agent_name", "notif_msg", "backend"], "get_agent_metadata": [],
        "get_partial_agent_metadata": ["descs", "inc_conn_info", "backends"], "add_remote_agent": ["metadata"],
        "remove_remote_agent": ["agent"], "send_local_metadata": ["ip_addr", "port"],
        "send_partial_agent_metadata": ["descs", "inc_conn_info", "backends", "ip_addr", "port", "label"],
        "fetch_remote_metadata": ["remote_agent", "ip_addr", "port", "label"],
        "invalidate_local_metadata": ["ip_addr", "port"], "check_remote_metadata": ["agent", "descs"],
        "get_xfer_descs": ["descs", "mem_type"], "get_remote_descs": ["descs", "mem_type"],
        "get_reg_descs": ["descs", "mem_type"], "get_serialized_descs": ["descs"],
        "deserialize_descs": ["serialized_descs"],
    }
    for name, want in reference.items():
        fn = getattr(nixl_agent, name, None)
        assert callable(fn), name
        got = [p for p in inspect.signature(fn).parameters if p != "self"]
        assert got[:len(want)] == want, (name, got)
    ctor = [p for p in inspect.signature(nixl_agent.__init__).parameters if p != "self"]
    assert ctor[:3] == ["agent_name", "nixl_conf", "instantiate_all"]

    with caplog.at_level(logging.WARNING, logger="nixl_amd"):
        a = nixl_agent("ctor-a", nixl_agent_config(backends=("NOSUCH", "MEMCPY")), plugin_dirs=[oracle_plugin_dir])
    assert list(a.backends) == ["MEMCPY"]
    assert any("Skipping backend registration NOSUCH" in r.getMessage() for r in caplog.records)
    a.close()
    caplog.clear()
    with caplog.at_level(logging.WARNING, logger="nixl_amd"):
        b = nixl_agent("ctor-b", nixl_agent_config(backends=("MEMCPY",)), True, plugin_dirs=[oracle_plugin_dir])
    assert list(b.backends) == ["MEMCPY"]  # the configuration wins
    assert any("Ignoring instantiate_all" in r.getMessage() for r in caplog.records)
    b.close()
