"""GPU parity tests for the descriptor-transfer half: the copy kernels through their C ABI
and the HIP backend plugin through the agent, against the CPU oracle (per-descriptor
memcpy) and through size-independent properties at full configuration sizes."""
import ctypes

import numpy as np
import pytest

from oracle import kv_oracle as ko
from nixl_amd import _lib, nixl_agent, nixl_agent_config
from nixl_amd import agent as ag

pytestmark = pytest.mark.gpu


def _plan(descs, tuning=None):
    lib = _lib.kernels()
    arr = (_lib.CopyDesc * len(descs))(*[_lib.CopyDesc(int(s), int(d), int(n)) for s, d, n in descs])
    plan = ctypes.c_void_p()
    t = ctypes.byref(_lib.CopyTuning(*tuning)) if tuning else None
    rc = lib.nixl_amd_copy_plan_create(arr, len(descs), 0, t, ctypes.byref(plan))
    assert rc == 0, _lib.kernels_error()
    return plan


def _run_plan(torch, plan):
    lib = _lib.kernels()
    torch.cuda.synchronize()
    assert lib.nixl_amd_copy_plan_launch(plan, None) == 0, _lib.kernels_error()
    torch.cuda.synchronize()


def _check_against_oracle(torch, cuda, mem_bytes, src_off, dst_off, lens, tuning=None, seed=0):
    rng = np.random.default_rng(seed)
    host = rng.integers(0, 256, mem_bytes, dtype=np.uint8)
    dev = torch.from_numpy(host.copy()).to(cuda)
    base = dev.data_ptr()
    plan = _plan([(base + s, base + d, n) for s, d, n in zip(src_off, dst_off, lens)], tuning)
    info = _lib.CopyPlanInfo()
    _lib.kernels().nixl_amd_copy_plan_query(plan, ctypes.byref(info))
    _run_plan(torch, plan)
    want = ko.copy_descs(host, src_off, dst_off, lens)
    got = dev.cpu().numpy()
    assert _lib.kernels().nixl_amd_copy_plan_destroy(plan) == 0
    assert np.array_equal(got, want), f"first mismatch at byte {int(np.argmax(got != want))}"
    return info


def _disjoint_layout(rng, lens, align, region):
    """Random non-overlapping offsets for the given lengths inside [0, region)."""
    order = rng.permutation(len(lens))
    sizes = np.array([((int(lens[i]) + align - 1) // align + 1) * align for i in order], dtype=np.int64)
    starts = np.concatenate([[0], np.cumsum(sizes)])
    assert starts[-1] <= region
    offs = np.empty(len(lens), dtype=np.int64)
    offs[order] = starts[:-1]
    return offs


@pytest.mark.parametrize("upl", [1, 2, 4, 8, 16])
@pytest.mark.parametrize("nt", [1, 2, 3, 4])
def test_aligned_descriptors_match_oracle(cuda, upl, nt):
    import torch
    rng = np.random.default_rng(upl * 10 + nt)
    # sizes straddling every chunk boundary case: sub-wave, exactly one chunk, several chunks
    lens = [16, 32, 512, 1008, 1024, 4096, 8192, 8208, 16384, 32768, 65536 + 48, 16 * upl * 64, 16 * upl * 64 - 16]
    lens += [int(x) * 16 for x in rng.integers(1, 600, 200)]
    half = 8 << 20
    so = _disjoint_layout(rng, lens, 16, half)
    do = _disjoint_layout(rng, lens, 16, half) + half
    info = _check_against_oracle(torch, cuda, 2 * half, so, do, lens, (upl, nt, 0, 0, 0), seed=upl)
    assert info.vec_descs == len(lens) and info.generic_descs == 0
    assert info.payload_bytes == sum(lens)


@pytest.mark.parametrize("sort_scatter", [0, 2])
@pytest.mark.parametrize("n", [1024, 3000, 5121])
def test_scatter_of_consecutive_memory_matches_oracle(cuda, n, sort_scatter):
    """Equal blocks out of consecutive memory into a random permutation of places: the plan
    takes the single-pass lowering and (sort_scatter=0) reorders its records on the device;
    with the reordering off (2) the same bytes must arrive.  A few neighbouring blocks are
    merged into longer descriptors, as the agent does."""
    import torch
    rng = np.random.default_rng(n)
    blk = 8192
    half = (n + 8) * blk
    perm = rng.permutation(n)
    src_off = [i * blk for i in range(n)]
    dst_off = [half + int(p) * blk for p in perm]
    lens = [blk] * n
    # merge what happens to be adjacent on both sides
    so, do, ln = [src_off[0]], [dst_off[0]], [blk]
    for i in range(1, n):
        if dst_off[i] == do[-1] + ln[-1] and src_off[i] == so[-1] + ln[-1]:
            ln[-1] += blk
        else:
            so.append(src_off[i]); do.append(dst_off[i]); ln.append(blk)
    info = _check_against_oracle(torch, cuda, 2 * half, so, do, ln, (0, 0, 0, 0, 0, sort_scatter), seed=n)
    assert info.uniform_chunks == n * (blk // 1024) and info.mixed_chunks == 0 and info.piece_items == 0


def test_ragged_small_descriptors_match_oracle(cuda):
    # BASELINE config 3 in miniature: sizes log-uniform in [512, 4096] rounded to 16.
    import torch
    rng = np.random.default_rng(33)
    n = 20000
    lens = (np.exp(rng.uniform(np.log(512), np.log(4096), n)).astype(np.int64) // 16) * 16
    half = 96 << 20
    so = _disjoint_layout(rng, lens, 16, half)
    do = _disjoint_layout(rng, lens, 16, half) + half
    _check_against_oracle(torch, cuda, 2 * half, so, do, lens, seed=5)


def test_many_tiny_descriptors_in_one_chunk(cuda):
    # 16-byte descriptors: more than 64 descriptors fall into one 8 KiB chunk, which takes
    # the bisection path of the kernel.
    import torch
    rng = np.random.default_rng(4)
    lens = [16] * 3000 + [48] * 100
    half = 1 << 20
    so = _disjoint_layout(rng, lens, 16, half)
    do = _disjoint_layout(rng, lens, 16, half) + half
    _check_against_oracle(torch, cuda, 2 * half, so, do, lens, seed=6)


def test_unaligned_brute_force(cuda):
    # every length 1..80 with every src/dst residue mod 16 in turn, plus long odd spans
    import torch
    src_off, dst_off, lens = [], [], []
    pos_s, pos_d = 0, 1 << 20
    k = 0
    for n in list(range(1, 81)) + [255, 1000, 4097, 16385, 40001]:
        for _ in range(4):
            sa, da = k % 16, (k // 16 + k) % 16
            k += 7
            src_off.append(pos_s + sa)
            dst_off.append(pos_d + da)
            lens.append(n)
            pos_s += ((n + 31) // 16 + 1) * 16
            pos_d += ((n + 31) // 16 + 1) * 16
    assert pos_s <= (1 << 20)
    info = _check_against_oracle(torch, cuda, 2 << 20, src_off, dst_off, lens, seed=8)
    assert info.generic_descs > 0


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_mixture_of_every_descriptor_class(cuda, seed):
    """One request that mixes everything the planner tells apart: lengths log-uniform from
    1 byte to 200 KiB; addresses byte-aligned, 16-byte aligned, line-aligned or 4 KiB-aligned at
    random and independently on the two sides; a sprinkling of zero lengths, exact chunk
    multiples and lengths one unit off them.  All classes must land in one plan and every
    byte must match the per-descriptor oracle, including the gaps between destinations."""
    import torch
    rng = np.random.default_rng(1000 + seed)
    n = 3000
    lens = np.exp(rng.uniform(0, np.log(200 << 10), n)).astype(np.int64)
    special = rng.integers(0, n, 300)
    lens[special[:60]] = 0
    lens[special[60:140]] = rng.choice([1024, 2048, 4096, 8192, 16384, 65536], 80)
    lens[special[140:220]] = rng.choice([1024, 4096, 8192, 16384], 80) + rng.choice([-16, 16, -1, 1], 80)
    lens[special[220:]] = (lens[special[220:]] // 16) * 16
    grain = rng.choice([1, 16, 128, 4096], n, p=[0.3, 0.3, 0.25, 0.15])
    lens = np.where(grain >= 16, (lens // 16) * 16, lens)  # aligned addresses mostly carry aligned lengths
    lens[rng.integers(0, n, 40)] += 3  # ... but not always
    half = int(lens.sum() + n * (4096 + 256) + (1 << 20))
    half = (half + 4095) // 4096 * 4096

    def place(grains):
        order = rng.permutation(n)
        offs = np.empty(n, dtype=np.int64)
        at = 0
        for i in order:
            g = int(grains[i])
            at = (at + g - 1) // g * g
            offs[i] = at
            at += int(lens[i]) + int(rng.integers(0, 200))
        assert at <= half
        return offs

    so = place(grain)
    do = place(rng.permutation(grain)) + half
    info = _check_against_oracle(torch, cuda, 2 * half, so, do, lens, seed=seed)
    assert info.payload_bytes == int(lens.sum())
    assert info.generic_descs > 0 and info.piece_items > 0 and info.vec_descs > 0


def test_runs_of_different_lengths_are_expanded_on_the_device(cuda):
    """Line-aligned descriptors of at least 8 KiB whose lengths differ: the chunks inside each
    descriptor share nothing, so every chunk has a record, and those records are written on the
    device from one record per run.  One descriptor of 24 MiB among two thousand of 8 to 64 KiB
    (whole chunks, and lengths that leave a tail for the next chunk), every byte against the
    oracle; the plan holds a record per chunk."""
    import torch
    rng = np.random.default_rng(77)
    lens = [int(x) * 1024 for x in rng.integers(8, 65, 1200)] + [int(x) * 16 for x in rng.integers(512, 4097, 800)]
    lens.insert(700, 24 << 20)
    half = int(sum(lens) + len(lens) * 256 + (1 << 20))
    half = (half + 4095) // 4096 * 4096
    so = _disjoint_layout(rng, lens, 128, half)
    do = _disjoint_layout(rng, lens, 128, half) + half
    info = _check_against_oracle(torch, cuda, 2 * half, so, do, lens, seed=5)
    assert info.vec_descs == len(lens) and info.piece_items == 0 and info.generic_descs == 0
    assert info.uniform_chunks > 24 * 1024 and info.mixed_chunks > 0
    assert info.plan_device_bytes >= info.uniform_chunks * 16


def test_zero_length_and_empty(cuda):
    import torch
    dev = torch.zeros(4096, dtype=torch.uint8, device=cuda)
    plan = _plan([(dev.data_ptr(), dev.data_ptr() + 2048, 0)])
    info = _lib.CopyPlanInfo()
    _lib.kernels().nixl_amd_copy_plan_query(plan, ctypes.byref(info))
    assert info.payload_bytes == 0 and info.vec_chunks == 0
    _run_plan(torch, plan)
    _lib.kernels().nixl_amd_copy_plan_destroy(plan)
    # null address / bad tuning are rejected on the host, before any launch
    lib = _lib.kernels()
    out = ctypes.c_void_p()
    bad = (_lib.CopyDesc * 1)(_lib.CopyDesc(0, dev.data_ptr(), 16))
    assert lib.nixl_amd_copy_plan_create(bad, 1, 0, None, ctypes.byref(out)) == -1
    ok = (_lib.CopyDesc * 1)(_lib.CopyDesc(dev.data_ptr(), dev.data_ptr() + 16, 16))
    assert lib.nixl_amd_copy_plan_create(ok, 1, 0, ctypes.byref(_lib.CopyTuning(5, 0, 0, 0, 0)), ctypes.byref(out)) == -1
    assert lib.nixl_amd_copy_plan_create(ok, 1, 99, None, ctypes.byref(out)) == -1


# ---- through the agent and the plugin --------------------------------------------------------

@pytest.fixture()
def hip_agent(cuda):
    a = nixl_agent("agent", nixl_agent_config(backends=("HIP",)))
    yield a
    a.close()


def _wait(a, req):
    st = a.transfer(req)
    assert st in ("DONE", "PROC")
    while st == "PROC":
        st = a.check_xfer_state(req)
    assert st == "DONE"


def _descs(t, offs, lens):
    offs = np.asarray(offs, dtype=np.uint64)
    return np.stack([np.uint64(t.data_ptr()) + offs, np.asarray(lens, dtype=np.uint64), np.zeros_like(offs)], 1)


def test_prepared_lists_three_requests(hip_agent, cuda):
    # Shape of test/nixl/agent_example.cpp:375-531 (sideXferTest): 32 x 1 KiB buffers per
    # side, both sides prepared once, three requests with different index vectors off the
    # same handles; every destination byte must be 0xbb (check_buf, :28-34).
    import torch
    a = hip_agent
    n, ln = 32, 1024
    src = torch.full((n * ln,), 0xBB, dtype=torch.uint8, device=cuda)
    dst = torch.zeros(n * ln, dtype=torch.uint8, device=cuda)
    a.register_memory([src, dst])
    offs = np.arange(n) * ln
    hl = a.prep_xfer_dlist("", _descs(src, offs, [ln] * n), "VRAM")
    hr = a.prep_xfer_dlist("agent", _descs(dst, offs, [ln] * n), "VRAM")
    torch.cuda.synchronize()
    lo, hi = np.arange(16), np.arange(16, 32)
    r1 = a.make_prepped_xfer("WRITE", hl, lo, hr, lo)
    _wait(a, r1)
    assert bool((dst[:16 * ln] == 0xBB).all()) and bool((dst[16 * ln:] == 0).all())
    src[16 * ln:] = 0
    torch.cuda.synchronize()
    r2 = a.make_prepped_xfer("READ", hl, hi, hr, lo)  # local[16..31] <- remote[0..15]
    _wait(a, r2)
    assert bool((src == 0xBB).all())
    r3 = a.make_prepped_xfer("WRITE", hl, hi, hr, hi)
    _wait(a, r3)
    assert bool((dst == 0xBB).all())
    for h in (r1, r2, r3, hl, hr):
        h.release()


@pytest.mark.parametrize("op", ["WRITE", "READ"])
def test_index_vectors_into_single_run_lists(hip_agent, cuda, op):
    """A dense pool and a strided one, each prepared as ONE list that compresses into one
    run: the request is then lowered on the device from the two index vectors (no descriptor
    is written out on the host).  3000 blocks in random order (more than one sorting window,
    not a multiple of it), both directions, against the per-descriptor oracle; the same
    indices through lists that do not qualify (two regions) must give the same bytes."""
    import torch
    a = hip_agent
    blk, n_pool, n = 8192, 4096, 3000
    rng = np.random.default_rng(5)
    host = rng.integers(0, 256, (3 * n_pool) * blk, dtype=np.uint8)
    mem = torch.from_numpy(host.copy()).to(cuda)
    a.register_memory([mem])
    base = mem.data_ptr()
    dense_offs = np.arange(n_pool) * blk  # blocks 0..n_pool-1, adjoining
    strided_offs = n_pool * blk + np.arange(n_pool) * 2 * blk  # every other block of the rest
    h_local = a.prep_xfer_dlist("", _descs(mem, dense_offs, [blk] * n_pool), "VRAM")
    h_remote = a.prep_xfer_dlist("agent", _descs(mem, strided_offs, [blk] * n_pool), "VRAM")
    assert h_local.run_count() == 1 and h_remote.run_count() == 1
    li = rng.permutation(n_pool)[:n].astype(np.int32)
    ri = rng.permutation(n_pool)[:n].astype(np.int32)
    req = a.make_prepped_xfer(op, h_local, li, h_remote, ri)
    assert req.desc_count() == (n, n * blk)
    _wait(a, req)
    l_off, r_off = dense_offs[li], strided_offs[ri]
    src, dst = (l_off, r_off) if op == "WRITE" else (r_off, l_off)
    want = ko.copy_descs(host, src, dst, [blk] * n)
    assert np.array_equal(mem.cpu().numpy(), want)
    # an index outside its list is refused before anything is launched
    bad = li.copy()
    bad[7] = n_pool
    with pytest.raises(Exception):
        a.make_prepped_xfer(op, h_local, bad, h_remote, ri)
    # the ordinary path (explicit descriptors) on fresh memory gives the same bytes
    mem.copy_(torch.from_numpy(host))
    torch.cuda.synchronize()
    req2 = a.initialize_xfer(op, a.get_xfer_descs(_descs(mem, l_off, [blk] * n), "VRAM"),
                             a.get_xfer_descs(_descs(mem, r_off, [blk] * n), "VRAM"), "agent")
    _wait(a, req2)
    assert np.array_equal(mem.cpu().numpy(), want)
    for h in (req, req2, h_local, h_remote):
        h.release()


def test_index_vectors_into_lists_of_several_runs(hip_agent, cuda):
    """A pool registered as four separate allocations (what a pool must be for peers in other
    processes, whose mappings stay under 2 GiB each) prepared as one list of several runs, and
    a list whose second half has another stride (two runs in one region): requests are still
    lowered on the device, now through the run tables.  Indices cross every run boundary;
    checked against a per-block restatement in both directions; an index past the list is
    refused."""
    import torch
    a = hip_agent
    blk, per = 4096, 700
    n_pool, half = 4 * per, 2 * per
    rng = np.random.default_rng(11)
    parts = [torch.from_numpy(rng.integers(0, 256, per * blk, dtype=np.uint8)).to(cuda) for _ in range(4)]
    other = torch.from_numpy(rng.integers(0, 256, 3 * n_pool * blk, dtype=np.uint8)).to(cuda)
    a.register_memory(parts + [other])
    pool_descs = np.concatenate([_descs(p, np.arange(per) * blk, [blk] * per) for p in parts])
    other_offs = np.concatenate([np.arange(half) * blk, half * blk + np.arange(n_pool - half) * 2 * blk])
    h_local = a.prep_xfer_dlist("", pool_descs, "VRAM")
    h_remote = a.prep_xfer_dlist("agent", _descs(other, other_offs, [blk] * n_pool), "VRAM")
    assert 2 <= h_local.run_count() <= 4 and h_remote.run_count() == 2
    # distinct blocks on both sides, so that the order of the copies does not matter
    li = rng.permutation(n_pool)[:2500].astype(np.int32)
    ri = rng.permutation(n_pool)[:2500].astype(np.int32)
    edge = np.array([per - 1, per, 2 * per, n_pool - 1], dtype=np.int32)  # both sides of run boundaries, the last block
    li = np.concatenate([edge, li[~np.isin(li, edge)]])[:2400]
    ri = np.concatenate([edge[::-1], ri[~np.isin(ri, edge)]])[:2400]

    for op in ("WRITE", "READ"):
        pool_was = [p.cpu().numpy() for p in parts]
        other_was = other.cpu().numpy()
        req = a.make_prepped_xfer(op, h_local, li, h_remote, ri)
        assert req.desc_count() == (len(li), len(li) * blk)
        _wait(a, req)
        for l, r in zip(li.tolist(), ri.tolist()):
            part, off, ro = l // per, (l % per) * blk, int(other_offs[r])
            if op == "WRITE":
                other_was[ro:ro + blk] = pool_was[part][off:off + blk]
            else:
                pool_was[part][off:off + blk] = other_was[ro:ro + blk]
        for p, w in zip(parts, pool_was):
            assert np.array_equal(p.cpu().numpy(), w)
        assert np.array_equal(other.cpu().numpy(), other_was)
        req.release()
    bad = ri.copy()
    bad[3] = n_pool
    with pytest.raises(Exception):
        a.make_prepped_xfer("WRITE", h_local, li, h_remote, bad)
    for h in (h_local, h_remote):
        h.release()


def test_run_tables_through_the_kernel_library(cuda):
    """nixl_amd_copy_plan_create_indexed_runs called directly: three source runs with
    different strides, two destination runs, 5000 random blocks (more than one bisection
    depth, several sorting windows), against the descriptor oracle; run tables that do not
    follow each other are refused."""
    import torch
    lib = _lib.kernels()
    blk = 2048
    rng = np.random.default_rng(12)
    src_counts, src_strides = [1000, 1, 3000], [blk, blk, 2 * blk]
    dst_counts, dst_strides = [2500, 2500], [blk, 3 * blk]
    n_src, n_dst = sum(src_counts), sum(dst_counts)

    def layout(counts, strides, at):
        offs, table, first = [], [], 0
        for c, st in zip(counts, strides):
            table.append((at, st, first, c))
            offs.extend(at + np.arange(c) * st)
            at += c * st + 4096  # a gap between runs
            first += c
        return np.array(offs, dtype=np.int64), table, at

    src_offs, src_table, end = layout(src_counts, src_strides, 0)
    dst_offs, dst_table, end = layout(dst_counts, dst_strides, end)
    host = rng.integers(0, 256, end, dtype=np.uint8)
    mem = torch.from_numpy(host.copy()).to(cuda)
    base = mem.data_ptr()
    assert base % 128 == 0
    n = 5000
    si = rng.integers(0, n_src, n).astype(np.int32)  # a source block may be read twice
    di = rng.permutation(n_dst)[:n].astype(np.int32)
    si[:3] = [999, 1000, 1001]

    def c_table(table):
        arr = (_lib.CopyRun * len(table))()
        for r, (at, st, first, c) in enumerate(table):
            arr[r] = _lib.CopyRun(base + at, st, first, c)
        return arr

    plan = ctypes.c_void_p()
    rc = lib.nixl_amd_copy_plan_create_indexed_runs(c_table(src_table), len(src_table), si.ctypes.data, c_table(dst_table),
                                                    len(dst_table), di.ctypes.data, n, blk, 0, None, ctypes.byref(plan))
    assert rc == 0, _lib.kernels_error()
    _run_plan(torch, plan)
    assert lib.nixl_amd_copy_plan_destroy(plan) == 0
    want = ko.copy_descs(host, src_offs[si], dst_offs[di], [blk] * n)
    assert np.array_equal(mem.cpu().numpy(), want)
    broken = list(dst_table)
    broken[1] = (broken[1][0], broken[1][1], broken[1][2] + 1, broken[1][3])
    rc = lib.nixl_amd_copy_plan_create_indexed_runs(c_table(src_table), len(src_table), si.ctypes.data, c_table(broken),
                                                    len(broken), di.ctypes.data, n, blk, 0, None, ctypes.byref(plan))
    assert rc != 0 and "follow" in _lib.kernels_error()


def test_indexed_plans_launched_and_dropped_at_once(cuda):
    """Plan creation from index vectors returns before the records exist on the device.  A
    launch issued at once (no synchronisation in between, on the default stream and on
    another one) must still see them; plans dropped unused, and many plans in a row, must
    neither leak nor confuse the pinned buffers their indices travel through."""
    import torch
    lib = _lib.kernels()
    blk, n_pool, n = 4096, 3000, 2048
    rng = np.random.default_rng(17)
    host = rng.integers(0, 256, 2 * n_pool * blk, dtype=np.uint8)
    mem = torch.from_numpy(host.copy()).to(cuda)
    base = mem.data_ptr()
    other = torch.cuda.Stream(device=cuda)
    want = host.copy()
    plans = []
    for round_ in range(12):
        si = rng.permutation(n_pool)[:n].astype(np.int32)
        di = rng.permutation(n_pool)[:n].astype(np.int32)
        plan = ctypes.c_void_p()
        rc = lib.nixl_amd_copy_plan_create_indexed(base, blk, si.ctypes.data, base + n_pool * blk, blk, di.ctypes.data, n, blk, 0,
                                                   None, ctypes.byref(plan))
        assert rc == 0, _lib.kernels_error()
        if round_ % 3 == 2:  # dropped without a launch
            assert lib.nixl_amd_copy_plan_destroy(plan) == 0
            continue
        stream = other if round_ % 2 else torch.cuda.default_stream(cuda)
        torch.cuda.synchronize()  # earlier rounds' copies are over; this plan's upload may still be on its way
        assert lib.nixl_amd_copy_plan_launch(plan, ctypes.c_void_p(stream.cuda_stream)) == 0, _lib.kernels_error()
        plans.append(plan)
        ko.copy_descs(want, si.astype(np.int64) * blk, (n_pool + di.astype(np.int64)) * blk, [blk] * n)
    torch.cuda.synchronize()
    assert np.array_equal(mem.cpu().numpy(), want)
    for plan in plans:
        assert lib.nixl_amd_copy_plan_destroy(plan) == 0


def test_many_requests_leave_memory_where_it_was(hip_agent, cuda):
    """A serving loop: thousands of requests made from fresh index vectors, posted, waited for
    and released.  Plan arenas, pinned upload buffers and events are recycled, so device memory
    and the process's resident set stay where they were after a warm-up."""
    import psutil
    import torch
    a = hip_agent
    blk, n_pool, n = 4096, 4096, 1500
    mem = torch.zeros(2 * n_pool * blk, dtype=torch.uint8, device=cuda)
    a.register_memory([mem])
    h_l = a.prep_xfer_dlist("", _descs(mem, np.arange(n_pool) * blk, [blk] * n_pool), "VRAM")
    h_r = a.prep_xfer_dlist("agent", _descs(mem, (n_pool + np.arange(n_pool)) * blk, [blk] * n_pool), "VRAM")
    rng = np.random.default_rng(23)
    proc = psutil.Process()

    def burst(count):
        for i in range(count):
            li = rng.permutation(n_pool)[:n].astype(np.int32)
            ri = rng.permutation(n_pool)[:n].astype(np.int32)
            if i % 3 == 0:  # every third through explicit descriptors
                req = a.initialize_xfer("WRITE", a.get_xfer_descs(_descs(mem, li.astype(np.int64) * blk, [blk] * n), "VRAM"),
                                        a.get_xfer_descs(_descs(mem, (n_pool + ri.astype(np.int64)) * blk, [blk] * n), "VRAM"),
                                        "agent")
            else:
                req = a.make_prepped_xfer("WRITE", h_l, li, h_r, ri)
            if i % 7 != 6:  # some are released without ever being posted
                _wait(a, req)
            req.release()

    burst(200)
    torch.cuda.synchronize()
    free0, rss0 = torch.cuda.mem_get_info()[0], proc.memory_info().rss
    burst(2500)
    torch.cuda.synchronize()
    free1, rss1 = torch.cuda.mem_get_info()[0], proc.memory_info().rss
    assert free0 - free1 < (64 << 20), f"device memory shrank by {(free0 - free1) >> 20} MiB"
    assert rss1 - rss0 < (96 << 20), f"resident set grew by {(rss1 - rss0) >> 20} MiB"
    for h in (h_l, h_r):
        h.release()


def test_write_zero_read_roundtrip_and_repost(hip_agent, cuda):
    # transfer_handler round trip (test/gtest/plugins/transfer_handler.h:182-209 with
    # memory_handler.h:42-58): WRITE, clear the source, READ back, expect the increasing
    # pattern 0x11+i.  Then the repost rule of test/unit/plugins/posix/nixl_posix_test.cpp:
    # 714-770: the same handles posted again after the source changed deliver the new bytes.
    import torch
    a = hip_agent
    n = 1 << 20
    pattern = (torch.arange(n, device=cuda) + 0x11).to(torch.uint8)
    src = pattern.clone()
    dst = torch.zeros(n, dtype=torch.uint8, device=cuda)
    reg = a.register_memory([src, dst])
    # split_buf: four 16-byte entries at the start, then the rest in one descriptor
    offs = [0, 16, 32, 48, 64]
    lens = [16, 16, 16, 16, n - 64]
    ld = a.get_xfer_descs(_descs(src, offs, lens), "VRAM")
    rd = a.get_xfer_descs(_descs(dst, offs, lens), "VRAM")
    torch.cuda.synchronize()
    w = a.initialize_xfer("WRITE", ld, rd, "agent")
    r = a.initialize_xfer("READ", ld, rd, "agent")
    assert w.desc_count() == (5, n)  # createXferReq does not merge
    _wait(a, w)
    assert torch.equal(dst, pattern)
    src.zero_()
    torch.cuda.synchronize()
    _wait(a, r)
    assert torch.equal(src, pattern)
    src.fill_(0x5A)
    torch.cuda.synchronize()
    _wait(a, w)  # repost of the same handle
    assert bool((dst == 0x5A).all())
    a.deregister_memory(reg)  # before releasing the requests, as the reference test does
    w.release()
    r.release()


def test_plugin_rejects_what_it_cannot_do(hip_agent, cuda):
    import torch
    a = hip_agent
    t = torch.zeros(4096, dtype=torch.uint8, device=cuda)
    # wrong device id in the registration descriptor
    with pytest.raises(ag.NixlError):
        a.register_memory(np.array([[t.data_ptr(), 4096, 3]], dtype=np.uint64), "VRAM")
    # an address HIP does not know
    host = np.zeros(4096, np.uint8)
    with pytest.raises(ag.NixlError):
        a.register_memory(np.array([[host.ctypes.data, 4096, 0]], dtype=np.uint64), "VRAM")
    a.register_memory([t])
    # an agent nobody introduced
    ld = a.get_xfer_descs(_descs(t, [0], [16]), "VRAM")
    rd = a.get_xfer_descs(_descs(t, [2048], [16]), "VRAM")
    with pytest.raises(ag.NixlError) as e:
        a.initialize_xfer("WRITE", ld, rd, "stranger")
    assert e.value.status == ag.NIXL_ERR_NOT_FOUND


def test_two_agents_in_one_process(cuda):
    """Two agents with a HIP backend each exchange metadata by hand (get_agent_metadata /
    add_remote_agent, the reference's wire format) and move VRAM between their regions: WRITE
    with a notification that the target sees once the bytes have landed, READ, prepared lists,
    a device memory view over the peer's region, removal of the peer (reference cases:
    test/python/test_nixl_api.py:56-70,163-186,385-412; examples/cpp/nixl_example.cpp)."""
    import torch
    a = nixl_agent("initiator", nixl_agent_config(backends=()))
    b = nixl_agent("target", nixl_agent_config(backends=()))
    a.create_backend("HIP")
    b.create_backend("HIP")
    n = 8 << 20
    g = torch.Generator(device="cpu").manual_seed(3)
    src = torch.randint(0, 256, (n,), dtype=torch.uint8, generator=g).to(cuda)
    dst = torch.zeros(n, dtype=torch.uint8, device=cuda)
    a.register_memory([src])
    b.register_memory([dst])
    torch.cuda.synchronize()
    md = b.get_agent_metadata()
    assert md.startswith(b"nixlSerDes|Agent") and b"HIP2:pid=" in md and b"bknd" in md
    assert a.add_remote_agent(md) == "target"
    assert b.add_remote_agent(a.get_agent_metadata()) == "initiator"
    a.make_connection("target")
    assert a.check_remote_metadata("target", a.get_xfer_descs(_descs(dst, [4096], [4096]), "VRAM"))
    assert not a.check_remote_metadata("target", a.get_xfer_descs(_descs(src, [4096], [4096]), "VRAM"))

    blk = 32768
    idx = np.random.default_rng(5).permutation(n // blk)
    offs_src = [int(i) * blk for i in range(n // blk)]
    offs_dst = [int(i) * blk for i in idx]
    lens = [blk] * (n // blk)
    h = a.initialize_xfer("WRITE", a.get_xfer_descs(_descs(src, offs_src, lens), "VRAM"),
                          a.get_xfer_descs(_descs(dst, offs_dst, lens), "VRAM"), "target", b"blocks 0..255")
    state = a.transfer(h)
    while state == "PROC":
        state = a.check_xfer_state(h)
    assert state == "DONE"
    # the message is queued when the initiator sees the transfer complete, so the bytes are there
    assert b.get_new_notifs() == {"initiator": [b"blocks 0..255"]}
    want = torch.empty_like(src).view(-1, blk)
    want[torch.from_numpy(idx).to(cuda)] = src.view(-1, blk)
    assert torch.equal(dst, want.view(-1))
    a.release_xfer_handle(h)

    # READ: the target's bytes come back into a scratch region of the initiator
    back = torch.zeros(1 << 20, dtype=torch.uint8, device=cuda)
    a.register_memory([back])
    torch.cuda.synchronize()
    h = a.initialize_xfer("READ", a.get_xfer_descs(_descs(back, [0], [1 << 20]), "VRAM"),
                          a.get_xfer_descs(_descs(dst, [3 << 20], [1 << 20]), "VRAM"), "target")
    assert a.transfer_and_wait(h) == "DONE"
    assert torch.equal(back, dst[3 << 20:4 << 20])
    assert b.get_new_notifs() == {}
    a.release_xfer_handle(h)

    # prepared lists on both sides, a subset of indices, and a released-in-flight notification
    local = a.prep_xfer_dlist("NIXL_INIT_AGENT", a.get_xfer_descs(_descs(src, offs_src[:64], lens[:64]), "VRAM"))
    remote = a.prep_xfer_dlist("target", a.get_xfer_descs(_descs(dst, offs_src[:64], lens[:64]), "VRAM"))
    h = a.make_prepped_xfer("WRITE", local, list(range(0, 64, 2)), remote, list(range(1, 64, 2)), b"released early")
    assert a.transfer(h) in ("PROC", "DONE")
    a.release_xfer_handle(h)  # may still be running: the backend keeps it, and its message, until it has finished
    torch.cuda.synchronize()
    # the message leaves when the initiator's backend next looks at its released requests
    assert a.get_new_notifs() == {}
    assert b.check_remote_xfer_done("initiator", b"released")
    for i in range(0, 64, 2):
        assert torch.equal(dst[(i + 1) * blk:(i + 2) * blk], src[i * blk:(i + 1) * blk])

    # standalone messages both ways, and to oneself
    a.send_notif("target", b"ping")
    b.send_notif("initiator", b"pong")
    a.send_notif("initiator", b"note to self")
    assert b.get_new_notifs() == {"initiator": [b"ping"]}
    assert a.get_new_notifs() == {"target": [b"pong"], "initiator": [b"note to self"]}

    # a memory view over the peer's region resolves through the loaded metadata
    view = a.prep_mem_view(a.get_remote_descs([(dst.data_ptr() + 256, 4096, 0, "target")], "VRAM"))
    assert view
    a.release_mem_view(view)

    a.remove_remote_agent("target")
    with pytest.raises(ag.NixlError) as e:
        a.initialize_xfer("WRITE", a.get_xfer_descs(_descs(src, [0], [64]), "VRAM"),
                          a.get_xfer_descs(_descs(dst, [0], [64]), "VRAM"), "target")
    assert e.value.status == ag.NIXL_ERR_NOT_FOUND
    with pytest.raises(ag.NixlError):
        a.send_notif("target", b"gone")
    a.close()
    b.close()


def test_release_while_in_flight_does_not_block_or_corrupt(hip_agent, cuda):
    import torch
    a = hip_agent
    n = 256 << 20
    src = torch.full((n,), 7, dtype=torch.uint8, device=cuda)
    dst = torch.zeros(n, dtype=torch.uint8, device=cuda)
    a.register_memory([src, dst])
    torch.cuda.synchronize()
    req = a.initialize_xfer("WRITE", a.get_xfer_descs(_descs(src, [0], [n]), "VRAM"),
                            a.get_xfer_descs(_descs(dst, [0], [n]), "VRAM"), "agent")
    a.transfer(req)
    req.release()  # may still be running: the backend must keep the plan alive
    torch.cuda.synchronize()
    assert bool((dst == 7).all())


def test_config2_llama3_kv_gather_scatter_full_size(hip_agent, cuda):
    # BASELINE config 2 at full size: pool [32 layers][K,V][8192 blocks][32 KiB] of bf16
    # N(0,1); gather 1024 random blocks into contiguous staging (65536 descriptors), then
    # scatter to a seeded permutation of destination block ids in a second pool.  Checked
    # through properties: staging equals the torch gather of the source pool, the
    # destination blocks equal the source blocks, untouched destination blocks keep their
    # canary, and a checksum of the moved bytes is preserved.
    import torch
    a = hip_agent
    layers, pool_blocks, blk = 32, 8192, 32768
    n_sel = 1024
    lk = layers * 2
    gen = torch.Generator(device=cuda)
    gen.manual_seed(1234)
    src_pool = torch.empty((lk, pool_blocks, blk // 2), dtype=torch.bfloat16, device=cuda)
    for i in range(lk):
        src_pool[i] = torch.randn((pool_blocks, blk // 2), generator=gen, device=cuda, dtype=torch.float32).to(torch.bfloat16)
    dst_pool = torch.full((lk, pool_blocks, blk // 2), -7.0, dtype=torch.bfloat16, device=cuda)
    staging = torch.zeros((n_sel, lk, blk // 2), dtype=torch.bfloat16, device=cuda)
    a.register_memory([src_pool, dst_pool, staging])

    rng = np.random.default_rng(99)
    sel = rng.choice(pool_blocks, n_sel, replace=False)
    dst_ids = rng.permutation(pool_blocks)[:n_sel]
    n_desc = n_sel * lk
    lens = np.full(n_desc, blk, dtype=np.uint64)
    zeros = np.zeros(n_desc, dtype=np.uint64)
    src_addrs = ko.kv_block_descs(src_pool.data_ptr(), layers, pool_blocks, blk, sel)
    dst_addrs = ko.kv_block_descs(dst_pool.data_ptr(), layers, pool_blocks, blk, dst_ids)
    stg_addrs = np.uint64(staging.data_ptr()) + np.arange(n_desc, dtype=np.uint64) * np.uint64(blk)
    h_src = a.prep_xfer_dlist("", np.stack([src_addrs, lens, zeros], 1), "VRAM")
    h_stg_r = a.prep_xfer_dlist("agent", np.stack([stg_addrs, lens, zeros], 1), "VRAM")
    h_stg_l = a.prep_xfer_dlist("", np.stack([stg_addrs, lens, zeros], 1), "VRAM")
    h_dst = a.prep_xfer_dlist("agent", np.stack([dst_addrs, lens, zeros], 1), "VRAM")
    idx = np.arange(n_desc)
    gather = a.make_prepped_xfer("WRITE", h_src, idx, h_stg_r, idx)
    scatter = a.make_prepped_xfer("WRITE", h_stg_l, idx, h_dst, idx)
    assert gather.desc_count() == (n_desc, n_desc * blk)
    torch.cuda.synchronize()
    _wait(a, gather)
    _wait(a, scatter)

    sel_t = torch.from_numpy(sel).to(cuda)
    dst_t = torch.from_numpy(dst_ids).to(cuda)
    want_staging = src_pool[:, sel_t, :].permute(1, 0, 2)
    assert torch.equal(staging.view(torch.int16), want_staging.contiguous().view(torch.int16))
    assert torch.equal(dst_pool[:, dst_t, :].view(torch.int16), src_pool[:, sel_t, :].view(torch.int16))
    untouched = torch.ones(pool_blocks, dtype=torch.bool, device=cuda)
    untouched[dst_t] = False
    assert bool((dst_pool[:, untouched, :] == -7.0).all())
    moved_sum = src_pool[:, sel_t, :].view(torch.int16).to(torch.int64).sum()
    assert int(dst_pool[:, dst_t, :].view(torch.int16).to(torch.int64).sum()) == int(moved_sum)
    for h in (gather, scatter, h_src, h_stg_r, h_stg_l, h_dst):
        h.release()


def test_config3_small_descriptor_stress_full_size(hip_agent, cuda):
    # BASELINE config 3: 262144 descriptors, sizes log-uniform in [512 B, 4 KiB] rounded to
    # 16 B, random 16 B-aligned offsets in two 4 GiB buffers, destinations non-overlapping.
    # Verified exactly against a torch gather/scatter of the same spans done with 16-byte
    # elements, and by a canary (0xC3) over every destination byte no descriptor covers.
    import torch
    a = hip_agent
    n = 262144
    buf_bytes = 4 << 30
    rng = np.random.default_rng(2025)
    lens = (np.exp(rng.uniform(np.log(512), np.log(4096), n)).astype(np.int64) // 16) * 16
    src = torch.randint(0, 256, (buf_bytes,), dtype=torch.uint8, device=cuda)
    dst = torch.full((buf_bytes,), 0xC3, dtype=torch.uint8, device=cuda)
    a.register_memory([src, dst])
    so = rng.integers(0, (buf_bytes - 4096) // 16, n) * 16
    # non-overlapping destinations: shuffled slots of 4 KiB + random slack inside a slot
    slots = rng.permutation(buf_bytes // 8192)[:n] * 8192
    do = slots + (rng.integers(0, (8192 - 4096) // 16, n) * 16)
    zeros = np.zeros(n, dtype=np.uint64)
    hl = a.prep_xfer_dlist("", np.stack([np.uint64(src.data_ptr()) + so.astype(np.uint64), lens.astype(np.uint64), zeros], 1), "VRAM")
    hr = a.prep_xfer_dlist("agent", np.stack([np.uint64(dst.data_ptr()) + do.astype(np.uint64), lens.astype(np.uint64), zeros], 1), "VRAM")
    req = a.make_prepped_xfer("WRITE", hl, np.arange(n), hr, np.arange(n))
    torch.cuda.synchronize()
    _wait(a, req)

    units = lens // 16
    starts = np.concatenate([[0], np.cumsum(units)])
    owner = np.repeat(np.arange(n), units)
    within = np.arange(starts[-1]) - starts[owner]
    s_unit = torch.from_numpy(so[owner] // 16 + within).to(cuda)
    d_unit = torch.from_numpy(do[owner] // 16 + within).to(cuda)
    src16 = src.view(torch.int64).view(-1, 2)
    expect = torch.full((buf_bytes,), 0xC3, dtype=torch.uint8, device=cuda)
    expect.view(torch.int64).view(-1, 2)[d_unit] = src16[s_unit]
    diff = int((dst.view(torch.int64) != expect.view(torch.int64)).sum())
    assert diff == 0, f"{diff} of {buf_bytes // 8} 8-byte words differ"
    for h in (req, hl, hr):
        h.release()


def test_descriptors_longer_than_4_gib(cuda):
    """Two descriptors whose lengths do not fit in 32 bits: one 16-byte aligned (streamed in
    1 KiB chunks, chunk offsets beyond 2^32) and one that starts and ends on odd bytes (cut
    into byte-range items).  Canary bytes around both destinations."""
    import torch
    big = (4 << 30) + (3 << 20)
    odd = (4 << 30) + 12345
    src = torch.empty((big + odd + 64 + 7) // 8 * 8, dtype=torch.uint8, device=cuda)
    src.view(torch.int64).random_()
    dst = torch.full((big + odd + 4096,), 0x5A, dtype=torch.uint8, device=cuda)
    d0, d1 = 1024, 1024 + big + 1031  # the second destination starts on an odd byte
    s0, s1 = 0, big + 7
    plan = _plan([(src.data_ptr() + s0, dst.data_ptr() + d0, big), (src.data_ptr() + s1, dst.data_ptr() + d1, odd)])
    _run_plan(torch, plan)
    assert _lib.kernels().nixl_amd_copy_plan_destroy(plan) == 0
    assert torch.equal(dst[d0:d0 + big], src[s0:s0 + big])
    assert torch.equal(dst[d1:d1 + odd], src[s1:s1 + odd])
    assert bool((dst[:d0] == 0x5A).all()) and bool((dst[d0 + big:d1] == 0x5A).all()) and bool((dst[d1 + odd:] == 0x5A).all())


def test_more_pieces_than_one_launch_takes(cuda):
    """2^21 + 4097 descriptors of 256 bytes whose destinations start 16 bytes into a line: one
    piece (one wavefront) each, more than the largest grid of one launch, so the plan goes out
    as two launches.  Every destination row must hold its source row and the 16 bytes in front
    of it must keep the canary."""
    import torch
    n, blk, pitch = (1 << 21) + 4097, 256, 272
    g = torch.Generator(device=cuda).manual_seed(7)
    src = torch.randint(0, 256, (n, blk), dtype=torch.uint8, device=cuda, generator=g)
    dst = torch.full((n, pitch), 0xC3, dtype=torch.uint8, device=cuda)
    perm = torch.randperm(n, device=cuda, generator=g)
    descs = np.empty((n, 3), dtype=np.uint64)
    descs[:, 0] = np.uint64(src.data_ptr()) + np.arange(n, dtype=np.uint64) * np.uint64(blk)
    descs[:, 1] = np.uint64(dst.data_ptr()) + perm.cpu().numpy().astype(np.uint64) * np.uint64(pitch) + np.uint64(16)
    descs[:, 2] = blk
    lib = _lib.kernels()
    plan = ctypes.c_void_p()
    rc = lib.nixl_amd_copy_plan_create(ctypes.cast(descs.ctypes.data, ctypes.POINTER(_lib.CopyDesc)), n, 0, None, ctypes.byref(plan))
    assert rc == 0, _lib.kernels_error()
    info = _lib.CopyPlanInfo()
    lib.nixl_amd_copy_plan_query(plan, ctypes.byref(info))
    assert info.piece_items == n
    _run_plan(torch, plan)
    assert lib.nixl_amd_copy_plan_destroy(plan) == 0
    assert torch.equal(dst[perm, 16:], src)
    assert bool((dst[:, :16] == 0xC3).all())


def test_golden_descriptor_list(cuda):
    """Committed vector (tests/golden/kv_descs.npz): mixed aligned / unaligned / empty
    descriptors, destination pre-filled with a canary byte."""
    import os
    import torch
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kv_descs.npz"), allow_pickle=False)
    src = torch.from_numpy(g["src"]).to(cuda)
    dst = torch.full((g["src"].size,), int(g["canary"]), dtype=torch.uint8, device=cuda)
    plan = _plan([(src.data_ptr() + int(s), dst.data_ptr() + int(d), int(n))
                  for s, d, n in zip(g["src_off"], g["dst_off"], g["lens"])])
    _run_plan(torch, plan)
    assert _lib.kernels().nixl_amd_copy_plan_destroy(plan) == 0
    assert np.array_equal(dst.cpu().numpy(), g["dst"])
    assert np.array_equal(src.cpu().numpy(), g["src"])


def test_piece_path_line_misaligned_and_split(cuda):
    """Descriptors that are 16-byte but not 128-byte aligned, from 256 B to 40 KiB: the
    piece kernel with its destination-line-aligned splits, every src/dst line offset."""
    import torch
    rng = np.random.default_rng(12)
    src_off, dst_off, lens = [], [], []
    pos_s, pos_d = 0, 8 << 20
    for i, n in enumerate([256, 272, 1008, 1024, 4080, 4096, 4112, 8176, 8192, 8208, 12304, 40960, 40976] * 8):
        sa, da = (i * 16) % 128, (i * 48 + 16) % 128
        src_off.append(pos_s + sa)
        dst_off.append(pos_d + da)
        lens.append(n)
        pos_s += ((n + 255) // 128 + 1) * 128
        pos_d += ((n + 255) // 128 + 1) * 128
    assert pos_s <= (8 << 20)
    info = _check_against_oracle(torch, cuda, 16 << 20, src_off, dst_off, lens, seed=13)
    assert info.piece_items > len(lens) and info.generic_descs == 0
    # a long line-aligned descriptor still streams in uniform chunks, a short one is one piece
    info = _check_against_oracle(torch, cuda, 1 << 20, [0, 65536], [131072, 262144], [32768, 2048], seed=14)
    assert info.uniform_chunks == 32 and info.piece_items == 1


def test_raw_south_bound_api_from_cpp(cuda):
    """The plugin driven from C++ through nixlBackendEngine alone (no agent): plugin table,
    registerMem / loadLocalMD, prepXfer / postXfer / checkXfer for WRITE and READ, handle
    reuse, refusals, releaseReqH.  The program is tests/cpp/sb_api_roundtrip.cpp."""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "cpp", "_build", "sb_api_roundtrip")
    if not os.path.exists(exe):
        pytest.fail(f"{exe} missing: run __graft_entry__.build() first")
    proc = subprocess.run([exe, os.path.join(_lib.PLUGIN_DIR, "libplugin_HIP.so")], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0 and proc.stdout.strip().endswith("OK"), proc.stdout + proc.stderr


def test_device_memory_view_calls_from_hip(cuda):
    """Memory views and the device-side put / counter add / get-pointer calls over them,
    driven from a HIP program through nixlAgent (tests/cpp/mem_view_device_api.hip; the
    scenarios of the reference's test/gtest/device_api/single_write_test.cu plus ragged
    spans against memcpy, ordering of a counter after puts, and refusals)."""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "cpp", "_build", "mem_view_device_api")
    if not os.path.exists(exe):
        pytest.fail(f"{exe} missing: run __graft_entry__.build() first")
    env = dict(os.environ, NIXL_PLUGIN_DIR=_lib.PLUGIN_DIR)
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=120, env=env)
    assert proc.returncode == 0 and proc.stdout.strip().endswith("OK"), proc.stdout + proc.stderr


def test_memory_view_tables_from_python(cuda):
    """prep_mem_view / release_mem_view of the Python API (reference _api.py:728-768): the
    handle is the device address of a table {magic, kind, count, (addr, len)...}; a remote
    list may carry a placeholder; lists that name unregistered memory or an unknown agent
    are refused."""
    import torch
    from nixl_amd.agent import NixlError

    class _DeviceWords:
        def __init__(self, ptr, n):
            self.__cuda_array_interface__ = {"shape": (n,), "typestr": "<i8", "data": (ptr, False), "version": 2}

    a = nixl_agent("viewer", nixl_agent_config(backends=()))
    a.create_backend("HIP")
    x = torch.zeros(1 << 16, dtype=torch.uint8, device=cuda)
    y = torch.zeros(1 << 14, dtype=torch.uint8, device=cuda)
    a.register_memory([x, y])
    local = a.get_xfer_descs([(x.data_ptr() + 256, 1024, 0), (y.data_ptr(), 1 << 14, 0)], "VRAM")
    remote = a.get_remote_descs([(y.data_ptr() + 64, 128, 0, "viewer"), (0, 0, 0, None),
                                 (x.data_ptr(), 1 << 16, 0, "viewer")], "VRAM")
    assert a.get_remote_descs([(1, 2, 3)], "VRAM") is None and a.get_remote_descs([(1, 2, 3, "v")]) is None
    lv = a.prep_mem_view(local)
    rv = a.prep_mem_view(remote, backends=["HIP"])
    assert lv and rv and lv != rv
    magic = 0x5649584C
    got = torch.as_tensor(_DeviceWords(lv, 2 + 2 * 2), device=cuda).cpu().tolist()
    assert got == [magic | (0 << 32), 2, x.data_ptr() + 256, 1024, y.data_ptr(), 1 << 14]
    got = torch.as_tensor(_DeviceWords(rv, 2 + 2 * 3), device=cuda).cpu().tolist()
    assert got == [magic | (1 << 32), 3, y.data_ptr() + 64, 128, 0, 0, x.data_ptr(), 1 << 16]
    a.release_mem_view(rv)
    a.release_mem_view(lv)

    z = torch.zeros(4096, dtype=torch.uint8, device=cuda)  # never registered
    with pytest.raises(NixlError):
        a.prep_mem_view(a.get_xfer_descs([(z.data_ptr(), 4096, 0)], "VRAM"))
    with pytest.raises(NixlError):
        a.prep_mem_view(a.get_xfer_descs([(y.data_ptr(), (1 << 14) + 1, 0)], "VRAM"))
    with pytest.raises(NixlError):
        a.prep_mem_view(a.get_remote_descs([(x.data_ptr(), 64, 0, "nobody")], "VRAM"))
    with pytest.raises(TypeError):
        a.prep_mem_view([(x.data_ptr(), 64, 0)])


@pytest.mark.parametrize("prog_thread", [True, False])
def test_notification_without_initiator_polling(cuda, prog_thread):
    """With the agent's progress thread (the Python default, reference _api.py:166) the HIP
    backend watches posted transfers that carry a notification and queues the message at the
    target once the copy has finished, whatever the initiator does; without the thread the
    message waits for the initiator's next look at the request."""
    import time
    import torch
    cfg = lambda: nixl_agent_config(enable_prog_thread=prog_thread, backends=())
    a, b = nixl_agent("pt-initiator", cfg()), nixl_agent("pt-target", cfg())
    a.create_backend("HIP")
    b.create_backend("HIP")
    n = 64 << 20
    src = torch.full((n,), 7, dtype=torch.uint8, device=cuda)
    dst = torch.zeros(n, dtype=torch.uint8, device=cuda)
    a.register_memory([src])
    b.register_memory([dst])
    torch.cuda.synchronize()
    a.add_remote_agent(b.get_agent_metadata())
    blk = 1 << 20
    offs = [i * blk for i in range(n // blk)]
    h = a.initialize_xfer("WRITE", a.get_xfer_descs(_descs(src, offs, [blk] * len(offs)), "VRAM"),
                          a.get_xfer_descs(_descs(dst, offs, [blk] * len(offs)), "VRAM"), "pt-target", b"no poll")
    assert a.transfer(h) in ("PROC", "DONE")
    if prog_thread:
        deadline = time.monotonic() + 10
        got = {}
        while not got and time.monotonic() < deadline:
            got = b.get_new_notifs()
        assert got == {"pt-initiator": [b"no poll"]}
        assert bool((dst == 7).all())  # the bytes were there when the message arrived
    else:
        torch.cuda.synchronize()
        time.sleep(0.05)
        assert b.get_new_notifs() == {}
    assert a.check_xfer_state(h) == "DONE"
    assert b.get_new_notifs() == ({} if prog_thread else {"pt-initiator": [b"no poll"]})
    # many requests in flight at once, each with its own message; all arrive exactly once
    hs = []
    for i in range(16):
        l = a.get_xfer_descs(_descs(src, [i * blk], [blk]), "VRAM")
        r = a.get_xfer_descs(_descs(dst, [i * blk], [blk]), "VRAM")
        hs.append(a.initialize_xfer("WRITE", l, r, "pt-target", b"req %d" % i))
    for x in hs:
        assert a.transfer(x) in ("PROC", "DONE")
    for x in hs:
        while a.check_xfer_state(x) == "PROC":
            pass
    seen = []
    deadline = time.monotonic() + 10
    while len(seen) < 16 and time.monotonic() < deadline:
        seen += b.get_new_notifs().get("pt-initiator", [])
    assert sorted(seen) == sorted(b"req %d" % i for i in range(16))
    for x in hs + [h]:
        a.release_xfer_handle(x)
    a.close()
    b.close()


def test_query_memory(hip_agent, cuda):
    """query_memory (reference _api.py:448-485): the HIP backend says what the runtime knows of
    each region, and nothing for an address it does not know."""
    import torch
    t = torch.zeros(1 << 20, dtype=torch.uint8, device=cuda)
    pinned = torch.zeros(4096, dtype=torch.uint8, pin_memory=True)
    host = np.zeros(4096, np.uint8)
    got = hip_agent.query_memory(np.array([[t.data_ptr() + 4096, 8192, 0], [t.data_ptr(), 1 << 30, 0],
                                           [host.ctypes.data, 4096, 0]], dtype=np.uint64), "HIP", "VRAM")
    assert got[0]["type"] == "device" and got[0]["device"] == "0" and got[0]["fits"] == "1"
    assert int(got[0]["allocation_bytes"]) >= 1 << 20
    assert got[1]["fits"] == "0" and got[2] is None
    got = hip_agent.query_memory(np.array([[pinned.data_ptr(), 4096, 0]], dtype=np.uint64), "HIP", "DRAM")
    assert got[0]["type"] == "pinned host"
    with pytest.raises(ValueError):
        hip_agent.query_memory([t], "UCX")


def test_requests_from_several_threads(cuda):
    """The reference calls prepXfer / postXfer / checkXfer / releaseReqH concurrently from
    several threads, one request each (benchmark/nixlbench/src/worker/nixl/nixl_worker.cpp:
    1847-1879).  Four threads, each creating, posting, polling and releasing its own requests
    on a backend with four streams; every thread's bytes must arrive."""
    import threading
    import torch
    a = nixl_agent("mt", nixl_agent_config(backends=()))
    a.create_backend("HIP", {"num_streams": "4"})
    n_threads, n_desc, blk, rounds = 4, 256, 8192, 20
    rng = np.random.default_rng(21)
    src = torch.from_numpy(rng.integers(0, 256, n_threads * n_desc * blk, dtype=np.uint8)).to(cuda)
    dst = torch.zeros_like(src)
    a.register_memory([src, dst])
    torch.cuda.synchronize()
    errors = []

    def worker(tid):
        try:
            base = tid * n_desc * blk
            perm = np.random.default_rng(tid).permutation(n_desc)
            s_off = base + np.arange(n_desc) * blk
            d_off = base + perm * blk
            lens = np.full(n_desc, blk)
            for _ in range(rounds):
                req = a.initialize_xfer("WRITE", a.get_xfer_descs(_descs(src, s_off, lens), "VRAM"),
                                        a.get_xfer_descs(_descs(dst, d_off, lens), "VRAM"), "mt")
                _wait(a, req)
                req.release()
        except Exception as e:  # noqa: BLE001 - reported to the main thread
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(n_threads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
    assert not errors, errors
    torch.cuda.synchronize()
    got, want = dst.cpu().numpy().reshape(n_threads, n_desc, blk), src.cpu().numpy().reshape(n_threads, n_desc, blk)
    for tid in range(n_threads):
        perm = np.random.default_rng(tid).permutation(n_desc)
        assert np.array_equal(got[tid][perm], want[tid])
    a.close()
