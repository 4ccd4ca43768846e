"""GPU parity tests of the request path the benchmark's headline runs, at its size: requests
made from index vectors into prepared lists that hold a whole Llama-3-8B-shaped pool
(524 288 entries) and a staging buffer (65 536 entries), the call pattern of the reference's
test/python/prep_xfer_perf.py:35-67, both through the plugin's own lowering of index vectors
and through prepXfer with written-out descriptors (what an unchanged libnixl calls,
src/core/nixl_agent.cpp:799-880).  Also here: the records entry points of the kernel
library's C ABI, a plan destroyed while it runs, and the plugin on pinned host memory at
BASELINE config 1's shape."""
import ctypes

import numpy as np
import pytest

from oracle import kv_oracle as ko
from nixl_amd import _lib, nixl_agent, nixl_agent_config

pytestmark = pytest.mark.gpu

LK, POOL_BLOCKS, N_SEL = 64, 8192, 1024  # 32 layers x {K, V}; config 2's pool and request


def _wait(a, req):
    st = a.transfer(req)
    assert st in ("DONE", "PROC")
    while st == "PROC":
        st = a.check_xfer_state(req)
    assert st == "DONE"


def _triples(base, offsets, blk):
    offsets = np.asarray(offsets, dtype=np.uint64)
    return np.stack([np.uint64(base) + offsets, np.full(offsets.size, blk, np.uint64), np.zeros(offsets.size, np.uint64)], 1)


def _indices(block_ids, order):
    """Positions in a list that holds the pool in memory order ([layer][K|V][block]) of the
    sub-blocks of `block_ids`, listed layer by layer or block by block."""
    idx = np.arange(LK, dtype=np.int64)[:, None] * POOL_BLOCKS + np.asarray(block_ids, dtype=np.int64)[None, :]
    return np.ascontiguousarray((idx if order == "layer" else idx.T).reshape(-1), dtype=np.int32)


class _World:
    """The pools, the staging buffers and two agents over them: one whose plugin lowers index
    vectors itself, one with that entry switched off (every request through prepXfer)."""

    def __init__(self, cuda, blk):
        import torch
        self.torch, self.cuda, self.blk = torch, cuda, blk
        gen = torch.Generator(device=cuda)
        gen.manual_seed(4321)
        words = blk // 2
        self.src = torch.empty((LK, POOL_BLOCKS, words), dtype=torch.bfloat16, device=cuda)
        for i in range(LK):
            self.src[i] = torch.randn((POOL_BLOCKS, words), generator=gen, device=cuda).to(torch.bfloat16)
        self.dst = [torch.empty((LK, POOL_BLOCKS, words), dtype=torch.bfloat16, device=cuda) for _ in range(2)]
        self.stg = [torch.empty((N_SEL * LK, words), dtype=torch.bfloat16, device=cuda) for _ in range(2)]
        self.agents, self.lists = [], []
        pool_offsets = np.arange(LK * POOL_BLOCKS, dtype=np.uint64) * np.uint64(blk)
        stg_offsets = np.arange(LK * N_SEL, dtype=np.uint64) * np.uint64(blk)
        for which, indexed in enumerate(("1", "0")):
            name = f"kv{which}"
            a = nixl_agent(name, nixl_agent_config(backends=()))
            a.create_backend("HIP", {"indexed_prep": indexed})
            a.register_memory([self.src, self.dst[which], self.stg[which]])
            lists = {}
            for role, peer in (("local", ""), ("remote", name)):
                lists["src", role] = a.prep_xfer_dlist(peer, _triples(self.src.data_ptr(), pool_offsets, blk), "VRAM")
                lists["dst", role] = a.prep_xfer_dlist(peer, _triples(self.dst[which].data_ptr(), pool_offsets, blk), "VRAM")
                lists["stg", role] = a.prep_xfer_dlist(peer, _triples(self.stg[which].data_ptr(), stg_offsets, blk), "VRAM")
            assert all(h.run_count() == 1 for h in lists.values())
            self.agents.append(a)
            self.lists.append(lists)

    def close(self):
        for a, lists in zip(self.agents, self.lists):
            for h in lists.values():
                h.release()
            a.close()


@pytest.fixture(scope="module", params=[16384, 32768], ids=["16KiB", "32KiB"])
def world(request, cuda):
    w = _World(cuda, request.param)
    yield w
    w.close()
    import torch
    del w
    torch.cuda.empty_cache()


@pytest.mark.parametrize("op", ["WRITE", "READ"])
@pytest.mark.parametrize("ids", ["random", "ascending"])
@pytest.mark.parametrize("order", ["layer", "block"])
def test_headline_requests_indexed_and_through_descriptors(world, order, ids, op):
    """Gather 1024 blocks of the pool into staging, scatter staging into a second pool, as
    the benchmark does (65 536 blocks of 16 or 32 KiB a request): staging equals the torch
    gather of the source pool, the destination blocks equal the source blocks, every other
    destination block keeps its canary - for the request lowered on the device from its index
    vectors and for the same request written out as descriptors and passed through prepXfer,
    whose bytes must also equal each other."""
    torch, cuda, blk = world.torch, world.cuda, world.blk
    rng = np.random.default_rng({"layer": 1, "block": 2}[order] * 10 + {"random": 1, "ascending": 2}[ids])
    sel = rng.choice(POOL_BLOCKS, N_SEL, replace=False)
    if ids == "ascending":
        sel = np.sort(sel)
    dst_ids = rng.permutation(POOL_BLOCKS)[:N_SEL]
    src_idx, dst_idx = _indices(sel, order), _indices(dst_ids, order)
    stg_idx = np.arange(LK * N_SEL, dtype=np.int32)
    n_desc = LK * N_SEL
    for which, (a, lists) in enumerate(zip(world.agents, world.lists)):
        world.dst[which].fill_(-7.0)
        world.stg[which].fill_(3.0)
        torch.cuda.synchronize()
        if op == "WRITE":  # local -> remote
            gather = a.make_prepped_xfer("WRITE", lists["src", "local"], src_idx, lists["stg", "remote"], stg_idx)
            scatter = a.make_prepped_xfer("WRITE", lists["stg", "local"], stg_idx, lists["dst", "remote"], dst_idx)
        else:  # local <- remote
            gather = a.make_prepped_xfer("READ", lists["stg", "local"], stg_idx, lists["src", "remote"], src_idx)
            scatter = a.make_prepped_xfer("READ", lists["dst", "local"], dst_idx, lists["stg", "remote"], stg_idx)
        count, total = gather.desc_count()
        assert total == n_desc * blk
        # the device lowering keeps one entry per block; written-out descriptors may merge neighbours
        assert count == n_desc if which == 0 else count <= n_desc
        _wait(a, gather)
        _wait(a, scatter)
        gather.release()
        scatter.release()
    sel_t, dst_t = torch.from_numpy(sel).to(cuda), torch.from_numpy(dst_ids).to(cuda)
    moved = world.src[:, sel_t, :]  # [LK][n_sel][words]
    want_staging = (moved if order == "layer" else moved.permute(1, 0, 2)).reshape(n_desc, -1)
    untouched = torch.ones(POOL_BLOCKS, dtype=torch.bool, device=cuda)
    untouched[dst_t] = False
    for which in range(2):
        assert torch.equal(world.stg[which].view(torch.int16), want_staging.view(torch.int16)), which
        assert torch.equal(world.dst[which][:, dst_t, :].view(torch.int16), moved.view(torch.int16)), which
        assert bool((world.dst[which][:, untouched, :] == -7.0).all()), which
    assert torch.equal(world.dst[0].view(torch.int16), world.dst[1].view(torch.int16))


def test_descriptor_path_merges_neighbours_like_the_oracle(world):
    """Block ids 0..1023 listed layer by layer are neighbours in memory on both sides: through
    prepXfer the 65 536 index pairs arrive as 64 descriptors of 1024 blocks each (the merge of
    src/core/nixl_agent.cpp:838-851, pinned in oracle/kv_oracle.py), which the plugin turns back
    into one record per block; the bytes equal the device lowering's."""
    torch, cuda, blk = world.torch, world.cuda, world.blk
    sel = np.arange(N_SEL)
    src_idx = _indices(sel, "layer")
    stg_idx = np.arange(LK * N_SEL, dtype=np.int32)
    counts = []
    for which, (a, lists) in enumerate(zip(world.agents, world.lists)):
        world.stg[which].fill_(3.0)
        torch.cuda.synchronize()
        req = a.make_prepped_xfer("WRITE", lists["src", "local"], src_idx, lists["stg", "remote"], stg_idx)
        counts.append(req.desc_count()[0])
        _wait(a, req)
        req.release()
    assert counts == [LK * N_SEL, LK]
    want = world.src[:, :N_SEL, :].reshape(LK * N_SEL, -1)
    for which in range(2):
        assert torch.equal(world.stg[which].view(torch.int16), want.view(torch.int16))


# ---- the records entry points of the kernel library -----------------------------------------

def _records_plan(n, blk, src_addrs, dst_addrs, facts=None, expect=0):
    lib = _lib.kernels()
    handle, recs = ctypes.c_void_p(), ctypes.POINTER(_lib.CopyRecord)()
    assert lib.nixl_amd_copy_records_begin(2 * n, ctypes.byref(handle), ctypes.byref(recs)) == 0, _lib.kernels_error()
    view = np.ctypeslib.as_array(ctypes.cast(recs, ctypes.POINTER(ctypes.c_uint64)), shape=(2 * n, 2))
    view[:n, 0] = src_addrs
    view[:n, 1] = dst_addrs
    plan = ctypes.c_void_p()
    rc = lib.nixl_amd_copy_plan_create_from_records(handle, n, blk, 0, None, ctypes.byref(facts) if facts else None,
                                                    ctypes.byref(plan))
    assert rc == expect, (rc, _lib.kernels_error())
    return plan


@pytest.mark.parametrize("with_facts", [False, True])
def test_records_written_by_the_caller(cuda, with_facts):
    """nixl_amd_copy_records_begin / nixl_amd_copy_plan_create_from_records: 3000 blocks of
    8 KiB scattered out of consecutive memory (the plan sorts its records on the device),
    against the per-descriptor oracle; with the library reading the records' pattern itself
    and with the caller stating it."""
    import torch
    lib = _lib.kernels()
    n, blk = 3000, 8192
    rng = np.random.default_rng(11)
    host = rng.integers(0, 256, 3 * n * blk, dtype=np.uint8)
    mem = torch.from_numpy(host.copy()).to(cuda)
    src_off = np.arange(n, dtype=np.uint64) * np.uint64(blk)
    dst_off = np.uint64(n * blk) + rng.permutation(2 * n)[:n].astype(np.uint64) * np.uint64(blk)
    facts = None
    if with_facts:
        facts = _lib.CopyRecordFacts(int(np.bitwise_or.reduce(src_off | dst_off)) | mem.data_ptr(), 0, n - 1, n - 1)
    plan = _records_plan(n, blk, np.uint64(mem.data_ptr()) + src_off, np.uint64(mem.data_ptr()) + dst_off, facts)
    info = _lib.CopyPlanInfo()
    assert lib.nixl_amd_copy_plan_query(plan, ctypes.byref(info)) == 0
    assert info.payload_bytes == n * blk and info.uniform_chunks == n * blk // 1024
    torch.cuda.synchronize()
    assert lib.nixl_amd_copy_plan_launch(plan, None) == 0, _lib.kernels_error()
    torch.cuda.synchronize()
    assert lib.nixl_amd_copy_plan_destroy(plan) == 0
    assert np.array_equal(mem.cpu().numpy(), ko.copy_descs(host, src_off, dst_off, [blk] * n))


def test_records_that_do_not_qualify_are_refused(cuda):
    import torch
    lib = _lib.kernels()
    mem = torch.zeros(1 << 20, dtype=torch.uint8, device=cuda)
    base = np.uint64(mem.data_ptr())
    good_src, good_dst = base + np.arange(4, dtype=np.uint64) * np.uint64(8192), base + np.uint64(1 << 19) + np.arange(4, dtype=np.uint64) * np.uint64(8192)
    bad_src = good_src.copy()
    bad_src[2] += np.uint64(64)  # not on a 128-byte line
    _records_plan(4, 8192, bad_src, good_dst, expect=-1)
    _records_plan(4, 8192, bad_src, good_dst, facts=_lib.CopyRecordFacts(int(np.bitwise_or.reduce(bad_src)), 0, 0, 3), expect=-1)
    bad_src = good_src.copy()
    bad_src[1] = 0  # null
    _records_plan(4, 8192, bad_src, good_dst, expect=-1)
    _records_plan(4, 4096, good_src, good_dst, expect=-1)  # blocks too short for a record each
    _records_plan(4, 8192 + 16, good_src, good_dst, expect=-1)  # no whole number of chunks
    # more records than the buffer holds; a buffer given back unused
    handle, recs = ctypes.c_void_p(), ctypes.POINTER(_lib.CopyRecord)()
    assert lib.nixl_amd_copy_records_begin(4, ctypes.byref(handle), ctypes.byref(recs)) == 0
    plan = ctypes.c_void_p()
    assert lib.nixl_amd_copy_plan_create_from_records(handle, 5, 8192, 0, None, None, ctypes.byref(plan)) == -1
    assert lib.nixl_amd_copy_records_begin(4, ctypes.byref(handle), ctypes.byref(recs)) == 0
    assert lib.nixl_amd_copy_records_abandon(handle) == 0
    assert lib.nixl_amd_copy_block_len_fits(16384, None) == 1 and lib.nixl_amd_copy_block_len_fits(4096, None) == 0
    torch.cuda.synchronize()


def test_plan_destroyed_while_it_runs_is_refused(cuda):
    """nixl_amd_copy_plan_destroy while a launch is in flight answers NIXL_AMD_ERR_BUSY and
    leaves the plan whole: its arena would otherwise go back to the pool, and the next plan's
    upload would overwrite records the running kernel still reads.  A second plan made and
    launched meanwhile, and the first one's bytes, both come out right."""
    import torch
    lib = _lib.kernels()
    n, blk = 32768, 32768  # 1 GiB a launch
    rng = np.random.default_rng(3)
    src = torch.randint(0, 255, (n * blk,), dtype=torch.uint8, device=cuda)
    dst = torch.zeros(2 * n * blk, dtype=torch.uint8, device=cuda)
    perm = rng.permutation(n).astype(np.uint64)
    arr = np.stack([np.uint64(src.data_ptr()) + np.arange(n, dtype=np.uint64) * np.uint64(blk),
                    np.uint64(dst.data_ptr()) + perm * np.uint64(blk), np.full(n, blk, np.uint64)], 1)
    arr = np.ascontiguousarray(arr)
    first = ctypes.c_void_p()
    assert lib.nixl_amd_copy_plan_create(ctypes.cast(arr.ctypes.data, ctypes.POINTER(_lib.CopyDesc)), n, 0, None,
                                         ctypes.byref(first)) == 0, _lib.kernels_error()
    torch.cuda.synchronize()
    stream = torch.cuda.Stream(device=cuda)
    for _ in range(8):  # a few milliseconds of work
        assert lib.nixl_amd_copy_plan_launch(first, ctypes.c_void_p(stream.cuda_stream)) == 0, _lib.kernels_error()
    assert lib.nixl_amd_copy_plan_destroy(first) == -4, "destroy of a running plan must answer NIXL_AMD_ERR_BUSY"
    assert "not completed" in _lib.kernels_error()
    # a second plan of the same size class, made and launched while the first still runs
    arr2 = arr.copy()
    arr2[:, 1] += np.uint64(n * blk)
    second = ctypes.c_void_p()
    assert lib.nixl_amd_copy_plan_create(ctypes.cast(arr2.ctypes.data, ctypes.POINTER(_lib.CopyDesc)), n, 0, None,
                                         ctypes.byref(second)) == 0, _lib.kernels_error()
    assert lib.nixl_amd_copy_plan_launch(second, ctypes.c_void_p(stream.cuda_stream)) == 0, _lib.kernels_error()
    torch.cuda.synchronize()
    assert lib.nixl_amd_copy_plan_destroy(first) == 0 and lib.nixl_amd_copy_plan_destroy(second) == 0
    want = src.view(n, blk)
    perm_t = torch.from_numpy(perm.astype(np.int64)).to(cuda)
    assert torch.equal(dst[:n * blk].view(n, blk)[perm_t], want)
    assert torch.equal(dst[n * blk:].view(n, blk)[perm_t], want)


def test_config1_shape_on_pinned_host_memory(cuda):
    """BASELINE config 1's request (4096 descriptors of 16 KiB, 64 MiB, destination block ids a
    seeded permutation) through the HIP plugin with both sides in pinned host memory (DRAM_SEG):
    the copy kernel reads and writes host memory over the link; bytes against the
    per-descriptor oracle."""
    import torch
    n, blk = 4096, 16384
    rng = np.random.default_rng(1)
    host = rng.integers(0, 256, 2 * n * blk, dtype=np.uint8)
    pinned = torch.from_numpy(host.copy()).pin_memory()
    a = nixl_agent("c1", nixl_agent_config(backends=("HIP",)))
    try:
        base = np.uint64(pinned.data_ptr())
        a.register_memory(np.array([[pinned.data_ptr(), pinned.numel(), 0]], dtype=np.uint64), "DRAM")
        src_off = np.arange(n, dtype=np.uint64) * np.uint64(blk)
        dst_off = np.uint64(n * blk) + rng.permutation(n).astype(np.uint64) * np.uint64(blk)
        zeros, lens = np.zeros(n, np.uint64), np.full(n, blk, np.uint64)
        req = a.initialize_xfer("WRITE", a.get_xfer_descs(np.stack([base + src_off, lens, zeros], 1), "DRAM"),
                                a.get_xfer_descs(np.stack([base + dst_off, lens, zeros], 1), "DRAM"), "c1")
        _wait(a, req)
        torch.cuda.synchronize()
        assert np.array_equal(pinned.numpy(), ko.copy_descs(host, src_off, dst_off, [blk] * n))
        req.release()
    finally:
        a.close()
