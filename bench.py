#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

Headline (``value``): paged-KV transfer throughput in decimal GB/s of payload, on the
Llama-3-8B-shaped configuration with the 16 KiB descriptors the metric names: pool
[32 layers][K,V][8192 blocks][16 KiB] of bf16 N(0,1) in HBM, 1024 blocks chosen without
replacement, gathered into a contiguous staging buffer (65 536 descriptors) and then
scattered to a seeded permutation of destination block ids in a second pool (65 536
descriptors).  One step = one gather request + one scatter request posted through the agent
API (postXferReq -> poll getXferStatus) to the HIP backend plugin.  The 32 KiB point (16
tokens per block) and the other descriptor order are reported beside it.
The throughput formula is the reference benchmark's: bytes moved / wall time
(benchmark/nixlbench/src/utils/utils.cpp:1357-1368).

The JSON line also carries the roofline of the dominant kernel (the uniform-chunk copy
kernel, HBM bound), the expert-parallel dispatch+combine times, and a CPU baseline: the
same agent call sequence with the per-descriptor memcpy backend on the host cores.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E peak, decimal GB/s

# HBM bytes per launch of the dominant kernel from hardware counters.  Counters cannot be read
# from inside this process.  The headline's figure is measured by measure_traffic_live below
# (child runs under the profiler); the other points, and the headline when the profiler cannot
# be run, take the figures of earlier rocprofv3 --pmc runs of this same file (read requests by
# size class in one run, WRITE_SIZE in another, checked against a plain 1 GiB element-wise
# kernel in the same run); the summaries under profiles/ name the commands.  Keyed by (blocks, pool blocks, descriptor
# bytes) - the two descriptor orders move the same bytes; a shape without a counter run
# reports null.
_KV_PROFILE = "profiles/copy_uniform_kernel_kv_llama3_16KiB_32KiB.txt (rocprofv3 --pmc runs of this file, not this run)"
MEASURED_TRAFFIC = {
    (1024, 8192, 16384): {"bytes": 2155883520, "source": _KV_PROFILE},
    (1024, 8192, 32768): {"bytes": 4303367616, "source": _KV_PROFILE},
    ("small", 262144): {"bytes": 938782368,
                        "source": "profiles/copy_piece_kernel_small_descriptor_stress_262144x512B-4KiB.txt (rocprofv3 --pmc runs of "
                                  "this file, not this run)"},
}


def counter_samples(csv_path, counters, kernel_tag="copy_uniform_kernel", yardstick_tag="CUDAFunctorOnSelf_add<int>"):
    """Reads a rocprofv3 counter_collection.csv (one row per dispatch and counter: Kernel_Name,
    Counter_Name, Counter_Value).  Returns ({counter: median over the kernel's dispatches},
    {counter: largest value over the yardstick's dispatches}, number of kernel dispatches), or
    None when either has no sample of some counter."""
    import csv
    import statistics
    kernel = {c: [] for c in counters}
    yard = {c: [] for c in counters}
    with open(csv_path, newline="") as f:
        for row in csv.DictReader(f):
            c, name = row.get("Counter_Name"), row.get("Kernel_Name", "")
            if c not in kernel:
                continue
            if kernel_tag in name:
                kernel[c].append(float(row["Counter_Value"]))
            elif yardstick_tag in name:
                yard[c].append(float(row["Counter_Value"]))
    if any(not kernel[c] or not yard[c] for c in counters):
        return None
    return ({c: statistics.median(kernel[c]) for c in counters}, {c: max(yard[c]) for c in counters},
            len(kernel[counters[0]]))


def counter_medians(csv_path, counters, tags, yardstick_tag="CUDAFunctorOnSelf_add<int>"):
    """The same file read for several kernels at once: ({tag: {counter: median over the
    dispatches of the kernels whose name contains tag}}, {counter: largest value over the
    yardstick's dispatches}).  A tag without samples is left out."""
    import csv
    import statistics
    seen = {t: {c: [] for c in counters} for t in tags}
    yard = {c: [] for c in counters}
    with open(csv_path, newline="") as f:
        for row in csv.DictReader(f):
            c, name = row.get("Counter_Name"), row.get("Kernel_Name", "")
            if c not in yard:
                continue
            if yardstick_tag in name:
                yard[c].append(float(row["Counter_Value"]))
            for t in tags:
                if t in name:
                    seen[t][c].append(float(row["Counter_Value"]))
    medians = {t: {c: statistics.median(v) for c, v in per.items()} for t, per in seen.items() if all(per.values())}
    return medians, {c: (max(v) if v else None) for c, v in yard.items()}


def _counter_run(child, counters, timeout=150):
    """One child run under `rocprofv3 --pmc <counters>`; returns the path of its counter file
    inside a temporary directory the caller removes, or {"error": why}."""
    import glob
    import shutil
    import signal
    import subprocess
    import tempfile
    prof = shutil.which("rocprofv3")
    if not prof:
        return None, {"error": "rocprofv3 not found"}
    if any("rocprof" in os.environ.get(k, "") for k in ("LD_PRELOAD", "ROCP_TOOL_LIBRARIES", "HSA_TOOLS_LIB")):
        return None, {"error": "this process already runs under a profiler"}
    out_dir = tempfile.mkdtemp(prefix="nixl_amd_pmc_", dir="/tmp")
    cmd = [prof, "--pmc", *counters, "--output-format", "csv", "-d", out_dir, "-o", "t", "--"] + child
    proc = subprocess.Popen(cmd, cwd="/tmp", env={**os.environ, "TMPDIR": "/tmp"}, stdout=subprocess.DEVNULL,
                            stderr=subprocess.DEVNULL, start_new_session=True)
    try:
        rc = proc.wait(timeout=timeout)
    except subprocess.TimeoutExpired:
        os.killpg(proc.pid, signal.SIGKILL)
        proc.wait()
        return out_dir, {"error": f"the counter run did not finish in {timeout} s"}
    if rc != 0:
        return out_dir, {"error": f"the counter run ended with status {rc}"}
    files = glob.glob(os.path.join(out_dir, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        return out_dir, {"error": "the counter run left no counter file"}
    return out_dir, files[0]


def measure_ep_traffic_live():
    """HBM bytes of each expert-parallel call from hardware counters, measured now: the four
    calls are run by a child process (nixl_amd/ep_bench.py run_traffic_child) under `rocprofv3
    --pmc`, once for the read requests by size class and once for WRITE_SIZE, with the same 1 GiB
    element-wise yardstick as the KV figure; a call's bytes are the sum over its kernels of the
    median per launch.  Returns {call: {"traffic", "traffic_source", "traffic_by_kernel"}} or
    {"error": why}."""
    import shutil
    from nixl_amd import ep_bench
    child = [sys.executable, os.path.abspath(__file__), "--ep-traffic-child"]
    read_classes = {"TCC_EA0_RDREQ_128B_sum": 128, "TCC_EA0_RDREQ_64B_sum": 64, "TCC_EA0_RDREQ_32B_sum": 32}
    tags = sorted({k for ks in ep_bench.CALL_KERNELS.values() for k in ks})
    got = {}
    for run, counters in (("read", list(read_classes)), ("write", ["WRITE_SIZE"])):
        out_dir, found = _counter_run(child, counters, timeout=200)
        try:
            if isinstance(found, dict):
                return {"error": f"{run}: {found['error']}"}
            got[run] = counter_medians(found, counters, tags)
        finally:
            if out_dir:
                shutil.rmtree(out_dir, ignore_errors=True)
    if not got["write"][1]["WRITE_SIZE"]:
        return {"error": "the write counter shows nothing for the yardstick"}
    write_scale = (1 << 20) / got["write"][1]["WRITE_SIZE"]
    out = {}
    for call, kernels in ep_bench.CALL_KERNELS.items():
        per_kernel = {}
        for k in kernels:
            if k not in got["read"][0] or k not in got["write"][0]:
                return {"error": f"no counter samples of {k}"}
            read = sum(got["read"][0][k][c] * size for c, size in read_classes.items())
            written = got["write"][0][k]["WRITE_SIZE"] * write_scale * 1024.0
            per_kernel[k] = int(round(read + written))
        out[call] = {"traffic": sum(per_kernel.values()), "traffic_by_kernel": per_kernel,
                     "traffic_source": "rocprofv3 --pmc over two child runs of this bench invocation (the four expert-parallel "
                                       "calls alone), median per launch summed over the call's kernels: reads = the L2's requests "
                                       "to memory by size class, writes = WRITE_SIZE scaled by a 1 GiB element-wise kernel"}
    return out


def measure_traffic_live(args, blk):
    """HBM bytes per launch of the headline kernel from hardware counters, measured now: the
    headline leg of this file is run twice more as a child process under `rocprofv3 --pmc`.
    Reads: the L2's requests to memory by size class (TCC_EA0_RDREQ_128B / _64B / _32B, one
    run), bytes = 128 a + 64 b + 32 c.  Writes: WRITE_SIZE (KiB per dispatch, second run).
    Each run also holds one plain element-wise kernel of known size (1 GiB read, 1 GiB
    written): the write counter is scaled by what it shows for that kernel, and the read
    classes must reproduce its 1 GiB (reported as `yardstick`).
    Returns {"bytes", "source", ...}, or {"error": why} when the profiler is not there or a run
    fails; the caller then falls back to the figures of profiles/."""
    import glob
    import shutil
    import signal
    import subprocess
    import tempfile
    prof = shutil.which("rocprofv3")
    if not prof:
        return {"error": "rocprofv3 not found"}
    if any("rocprof" in os.environ.get(k, "") for k in ("LD_PRELOAD", "ROCP_TOOL_LIBRARIES", "HSA_TOOLS_LIB")):
        return {"error": "this process already runs under a profiler"}
    child = [sys.executable, os.path.abspath(__file__), "--quick", "--no-ep", "--no-small", "--no-cpu-baseline",
             "--no-live-traffic", "--calibrate-copy", "--steps", "3", "--warmup", "1", "--fresh-requests", "1",
             "--block-bytes", str(blk), "--order", args.order, "--blocks", str(args.blocks),
             "--pool-blocks", str(args.pool_blocks)]
    for kv in args.backend_param:
        child += ["--backend-param", kv]
    read_classes = {"TCC_EA0_RDREQ_128B_sum": 128, "TCC_EA0_RDREQ_64B_sum": 64, "TCC_EA0_RDREQ_32B_sum": 32}
    got = {}
    for run, counters in (("read", list(read_classes)), ("write", ["WRITE_SIZE"])):
        out_dir = tempfile.mkdtemp(prefix="nixl_amd_pmc_", dir="/tmp")
        try:
            cmd = [prof, "--pmc", *counters, "--output-format", "csv", "-d", out_dir, "-o", "t", "--"] + child
            proc = subprocess.Popen(cmd, cwd="/tmp", env={**os.environ, "TMPDIR": "/tmp"}, stdout=subprocess.DEVNULL,
                                    stderr=subprocess.DEVNULL, start_new_session=True)
            try:
                rc = proc.wait(timeout=150)
            except subprocess.TimeoutExpired:
                os.killpg(proc.pid, signal.SIGKILL)
                proc.wait()
                return {"error": f"the {run} counter run did not finish in 150 s"}
            if rc != 0:
                return {"error": f"the {run} counter run ended with status {rc}"}
            files = glob.glob(os.path.join(out_dir, "**", "*counter_collection.csv"), recursive=True)
            if not files:
                return {"error": f"the {run} counter run left no counter file"}
            parsed = counter_samples(files[0], counters)
            if parsed is None:
                return {"error": f"the {run} counter run has no samples of the copy kernel or of the yardstick"}
            got[run] = parsed
        finally:
            shutil.rmtree(out_dir, ignore_errors=True)
    read = sum(got["read"][0][c] * size for c, size in read_classes.items())
    yard_read = sum(got["read"][1][c] * size for c, size in read_classes.items())
    if got["write"][1]["WRITE_SIZE"] <= 0:
        return {"error": "the write counter shows nothing for the yardstick"}
    write_scale = (1 << 20) / got["write"][1]["WRITE_SIZE"]  # the yardstick writes exactly 2^20 KiB
    written = got["write"][0]["WRITE_SIZE"] * write_scale * 1024.0
    return {"bytes": int(round(read + written)), "read_bytes": int(round(read)), "written_bytes": int(round(written)),
            "read_requests": {c[len("TCC_EA0_RDREQ_"):-len("_sum")]: int(got["read"][0][c]) for c in read_classes},
            "yardstick": {"read_bytes_counted_for_1GiB": int(round(yard_read)), "write_scale": round(write_scale, 4)},
            "launches_sampled": got["read"][2],
            "source": "rocprofv3 --pmc over two child runs of this bench invocation's headline leg, median over the copy "
                      "kernel's launches: reads = the L2's requests to memory by size class (TCC_EA0_RDREQ_128B/64B/32B), "
                      "writes = WRITE_SIZE scaled by a 1 GiB element-wise kernel in the same run"}


def _kv_layout():
    """Llama-3.1-8B with 16 tokens per block in bf16: 32 layers x {K, V}, 32 KiB per sub-block
    (nixl_amd/kvshape.py restates the reference's KV-size model)."""
    from nixl_amd import kvshape
    return kvshape.paged_kv_layout(kvshape.model("LLAMA3.1_8B"), 16, "bfloat16")


def _kv_descs(base, layers, pool_blocks, blk, block_ids, order):
    """One descriptor per (block, layer, K|V) in a pool laid out [layer][K|V][block][blk], listed
    layer by layer ("layer": the order in which per-layer registrations are walked) or block by
    block ("block": all 64 sub-blocks of one block id together)."""
    block_ids = np.asarray(block_ids, dtype=np.uint64)
    lk = np.arange(layers * 2, dtype=np.uint64)
    addr = (np.uint64(base) + lk[:, None] * np.uint64(pool_blocks * blk) + block_ids[None, :] * np.uint64(blk))
    return (addr if order == "layer" else addr.T).reshape(-1)


def _kv_indices(lk, pool_blocks, block_ids, order):
    """Positions, in a prepared list that holds the whole pool in memory order
    ([layer][K|V][block]), of the sub-blocks of `block_ids`, in the request's order."""
    idx = np.arange(lk, dtype=np.int64)[:, None] * pool_blocks + np.asarray(block_ids, dtype=np.int64)[None, :]
    return np.ascontiguousarray((idx if order == "layer" else idx.T).reshape(-1), dtype=np.int32)


def _triples(addrs, blk):
    n = addrs.size
    return np.stack([addrs, np.full(n, blk, np.uint64), np.zeros(n, np.uint64)], 1)


def run_kv(args, blk, order, steps, warmup, fresh_requests=4, sorted_ids=False, descriptor_path=False, pad_blocks=0):
    """Gather + scatter of config 2's shape with `blk`-byte descriptors.  The pools and the
    staging buffer are prepared ONCE as descriptor lists (prep_xfer_dlist); every request is
    made from index vectors into those lists (make_prepped_xfer), the call pattern of the
    reference's test/python/prep_xfer_perf.py:35-67.  Timed: (a) steady state, the same two
    requests re-posted; (b) requests whose block list is new every time, prepare included."""
    import torch
    from nixl_amd import nixl_agent, nixl_agent_config
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    kv = _kv_layout()
    layers, pool_blocks, n_sel = kv.layers, args.pool_blocks, args.blocks
    lk = layers * kv.sub_blocks_per_layer
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    # pad_blocks > 0: every (layer, K|V) slab of the two pools is that many blocks longer than the
    # blocks it is used for, so that the slabs do not lie a power of two apart
    slab_blocks = pool_blocks + pad_blocks
    src_pool = torch.empty((lk, slab_blocks, blk // 2), dtype=torch.bfloat16, device=dev)
    for i in range(lk):
        src_pool[i] = torch.randn((slab_blocks, blk // 2), generator=gen, device=dev).to(torch.bfloat16)
    dst_pool = torch.zeros((lk, slab_blocks, blk // 2), dtype=torch.bfloat16, device=dev)
    staging = torch.zeros((n_sel * lk, blk // 2), dtype=torch.bfloat16, device=dev)

    # Launches go to a stream of ours so that HIP events recorded on that same stream
    # bracket every kernel launch of the timed region.
    stream = torch.cuda.Stream(device=dev)
    agent = nixl_agent("bench", nixl_agent_config(backends=()))
    agent.create_backend("HIP", {"stream": str(stream.cuda_stream), **dict(kv.split("=", 1) for kv in args.backend_param)})
    agent.register_memory([src_pool, dst_pool, staging])

    n_desc, n_pool = n_sel * lk, lk * pool_blocks
    pool_offsets = ((np.arange(lk, dtype=np.uint64)[:, None] * np.uint64(slab_blocks)
                     + np.arange(pool_blocks, dtype=np.uint64)[None, :]) * np.uint64(blk)).reshape(-1)
    stg_addrs = np.uint64(staging.data_ptr()) + np.arange(n_desc, dtype=np.uint64) * np.uint64(blk)
    t0 = time.perf_counter()
    h_src = agent.prep_xfer_dlist("", _triples(np.uint64(src_pool.data_ptr()) + pool_offsets, blk), "VRAM")
    h_dst = agent.prep_xfer_dlist("bench", _triples(np.uint64(dst_pool.data_ptr()) + pool_offsets, blk), "VRAM")
    h_stg_r = agent.prep_xfer_dlist("bench", _triples(stg_addrs, blk), "VRAM")
    h_stg_l = agent.prep_xfer_dlist("", _triples(stg_addrs, blk), "VRAM")
    prep_dlist_ms = (time.perf_counter() - t0) * 1e3
    stg_idx = np.arange(n_desc, dtype=np.int32)

    def block_list(rng):
        """What a scheduler hands over: which blocks to send and where they go, as indices
        into the prepared lists."""
        sel = rng.choice(pool_blocks, n_sel, replace=False)
        if sorted_ids:  # a scheduler that hands its block list over in ascending order of the source blocks
            sel = np.sort(sel)
        dst_ids = rng.permutation(pool_blocks)[:n_sel]
        return sel, dst_ids, _kv_indices(lk, pool_blocks, sel, order), _kv_indices(lk, pool_blocks, dst_ids, order)

    handles = {"src": h_src, "dst": h_dst, "stg_r": h_stg_r, "stg_l": h_stg_l}

    def make(src_idx, dst_idx, ag=agent, h=handles):
        t = time.perf_counter()
        gather = ag.make_prepped_xfer("WRITE", h["src"], src_idx, h["stg_r"], stg_idx)
        scatter = ag.make_prepped_xfer("WRITE", h["stg_l"], stg_idx, h["dst"], dst_idx)
        return gather, scatter, (time.perf_counter() - t) * 1e3

    def check(sel, dst_ids):
        sel_t, dst_t = torch.from_numpy(sel).to(dev), torch.from_numpy(dst_ids).to(dev)
        if not torch.equal(dst_pool[:, dst_t, :].view(torch.int16), src_pool[:, sel_t, :].view(torch.int16)):
            raise RuntimeError("scattered blocks differ from the source blocks")

    def fresh_pairs(ag, h, rng):
        """Request pairs with a new block list every time, as a serving loop sees them, three
        ways.  (b) one after the other: make both requests, post and wait for the gather, post
        and wait for the scatter; the pair is released when it is done (its plan memory goes
        back to the engine's pool).  (b') each request posted as soon as it is made, so that
        the gather copies while the host makes the scatter (one stream keeps the order).
        (c) the host's share hidden altogether: the next pair is made and posted while the
        current one copies; a pair is waited for and released one iteration later."""
        def wait(req):
            state = ag.check_xfer_state(req)
            while state == "PROC":
                state = ag.check_xfer_state(req)
            if state != "DONE":
                raise RuntimeError(f"transfer ended in state {state}")

        def post(req):
            if ag.transfer(req) not in ("PROC", "DONE"):
                raise RuntimeError("post failed")

        n_pairs = max(fresh_requests, 1)
        make_ms, fresh_ms, as_made_ms = [], [], []
        for i in range(n_pairs + 2):
            sel, dst_ids, src_idx, dst_idx = block_list(rng)
            torch.cuda.synchronize()
            w0 = time.perf_counter()
            gather, scatter, m = make(src_idx, dst_idx, ag, h)
            for req in (gather, scatter):
                post(req)
                wait(req)
            w = (time.perf_counter() - w0) * 1e3
            check(sel, dst_ids)
            n_g, bytes_g = gather.desc_count()
            assert bytes_g == n_desc * blk and n_g <= n_desc  # neighbouring blocks may have been merged
            gather.release()
            scatter.release()
            if i >= 2:  # the first pairs also pay one-off allocations
                make_ms.append(m)
                fresh_ms.append(w)
        for i in range(n_pairs):
            sel, dst_ids, src_idx, dst_idx = block_list(rng)
            torch.cuda.synchronize()
            w0 = time.perf_counter()
            gather = ag.make_prepped_xfer("WRITE", h["src"], src_idx, h["stg_r"], stg_idx)
            post(gather)
            scatter = ag.make_prepped_xfer("WRITE", h["stg_l"], stg_idx, h["dst"], dst_idx)
            post(scatter)
            wait(gather)
            wait(scatter)
            as_made_ms.append((time.perf_counter() - w0) * 1e3)
            check(sel, dst_ids)
            gather.release()
            scatter.release()
        lists = [block_list(rng) for _ in range(n_pairs + 4)]
        torch.cuda.synchronize()
        w0 = time.perf_counter()
        in_flight = None
        for sel, dst_ids, src_idx, dst_idx in lists:
            gather, scatter, _ = make(src_idx, dst_idx, ag, h)
            post(gather)
            post(scatter)
            if in_flight is not None:
                for req in in_flight:
                    wait(req)
                    req.release()
            in_flight = (gather, scatter)
        for req in in_flight:
            wait(req)
        pipelined_ms = (time.perf_counter() - w0) * 1e3 / len(lists)
        check(*lists[-1][:2])
        for req in in_flight:
            req.release()

        def rate(ms):
            return round(2 * n_desc * blk / (ms * 1e-3) / 1e9, 1)

        return {"make_request_pair_ms": round(float(np.mean(make_ms)), 3),
                "value_including_prepare": rate(float(np.mean(fresh_ms))),
                "value_including_prepare_note": f"new block list per request pair: make_prepped_xfer x2, then post + wait "
                                                f"of each, mean of {len(fresh_ms)} pairs, wall clock",
                "value_including_prepare_posted_as_made": rate(float(np.mean(as_made_ms))),
                "value_including_prepare_posted_as_made_note": "the same, each request posted as soon as it is made: the gather "
                                                               "copies while the host makes the scatter",
                "value_including_prepare_pipelined": rate(pipelined_ms),
                "value_including_prepare_pipelined_note": f"the same, the next pair made and posted while the current one "
                                                          f"copies: wall clock over {len(lists)} pairs back to back"}

    rng = np.random.default_rng(99)
    fresh = {} if getattr(args, "headline_only", False) else fresh_pairs(agent, handles, rng)
    # The same loops with every request written out as descriptors and passed through prepXfer:
    # what an agent that knows nothing of this plugin's index entry does (the reference's
    # makeXferReq, src/core/nixl_agent.cpp:799-880).  A second agent over the same memory whose
    # backend has that entry switched off.
    through_prepxfer = None
    if descriptor_path:
        agent_d = nixl_agent("bench_d", nixl_agent_config(backends=()))
        agent_d.create_backend("HIP", {"stream": str(stream.cuda_stream), "indexed_prep": "0",
                                       **dict(kv.split("=", 1) for kv in args.backend_param)})
        agent_d.register_memory([src_pool, dst_pool, staging])
        handles_d = {"src": agent_d.prep_xfer_dlist("", _triples(np.uint64(src_pool.data_ptr()) + pool_offsets, blk), "VRAM"),
                     "dst": agent_d.prep_xfer_dlist("bench_d", _triples(np.uint64(dst_pool.data_ptr()) + pool_offsets, blk), "VRAM"),
                     "stg_r": agent_d.prep_xfer_dlist("bench_d", _triples(stg_addrs, blk), "VRAM"),
                     "stg_l": agent_d.prep_xfer_dlist("", _triples(stg_addrs, blk), "VRAM")}
        through_prepxfer = fresh_pairs(agent_d, handles_d, np.random.default_rng(98))
        through_prepxfer["entry"] = ("nixlBackendEngine::prepXfer with two lists of written-out descriptors a request "
                                    "(backend parameter indexed_prep=0): what an unchanged libnixl calls")
        for hd in handles_d.values():
            hd.release()
        agent_d.close()
    # the pairs of the steady-state measurement below, over different block sets
    pairs = []
    for i in range(max(fresh_requests, 1)):
        sel, dst_ids, src_idx, dst_idx = block_list(rng)
        gather, scatter, _ = make(src_idx, dst_idx)
        pairs.append((gather, scatter, sel, dst_ids))

    # (a) steady state: the prepared pairs re-posted in turn.  Which blocks a pair names moves
    # its time by several per cent (placement in DRAM), so the figure is the mean over the pairs.
    # A step posts its gather and, right behind it, its scatter (one stream keeps the order, and
    # the scatter reads what the gather wrote), then waits for the step BEFORE it: the GPU always
    # has the next request queued, as a transfer loop with a pipeline depth of two does
    # (the reference benchmark's --pipeline_depth, benchmark/nixlbench/src/utils/utils.cpp:48-250).
    # HIP events recorded on the same stream between the posts bracket every launch.
    def wait(req):
        state = agent.check_xfer_state(req)
        while state == "PROC":
            state = agent.check_xfer_state(req)
        if state != "DONE":
            raise RuntimeError(f"transfer ended in state {state}")

    post_us = []  # wall clock of the post call

    def run_steps(count, events=None):
        in_flight = None
        for k in range(count):
            pair = pairs[k % len(pairs)][:2]
            if in_flight is not None and in_flight[0] is pair[0]:  # a single pair: it must finish before it is posted again
                for req in in_flight:
                    wait(req)
                in_flight = None
            marks = []
            for req in pair:
                if events is not None:
                    marks.append(torch.cuda.Event(enable_timing=True))
                    marks[-1].record(stream)
                w0 = time.perf_counter()
                if agent.transfer(req) not in ("PROC", "DONE"):
                    raise RuntimeError("post failed")
                if events is not None:
                    post_us.append((time.perf_counter() - w0) * 1e6)
            if events is not None:
                marks.append(torch.cuda.Event(enable_timing=True))
                marks[-1].record(stream)
                events.append(marks)
            if in_flight is not None:
                for req in in_flight:
                    wait(req)
            in_flight = pair
        for req in in_flight:
            wait(req)

    torch.cuda.synchronize()
    run_steps(warmup)
    torch.cuda.synchronize()
    events = []
    t0 = time.perf_counter()
    run_steps(steps, events)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    check(*pairs[(steps - 1) % len(pairs)][2:])  # correctness of what was just timed (bit-exact)
    # post -> completion of one request at a time, wall clock, as nixlbench splits its report
    xfer_us = []
    for k in range(min(steps, 16)):
        for req in pairs[k % len(pairs)][:2]:
            w0 = time.perf_counter()
            agent.transfer(req)
            wait(req)
            xfer_us.append((time.perf_counter() - w0) * 1e6)

    payload_per_step = 2 * n_desc * blk  # gather + scatter
    kernel_ms = [m[i].elapsed_time(m[i + 1]) for m in events for i in (0, 1)]  # gather, scatter, gather, ...
    avg_launch_ms = float(np.mean(kernel_ms))
    algorithmic_bytes_per_launch = 2 * n_desc * blk  # every payload byte read once, written once
    achieved = algorithmic_bytes_per_launch / (avg_launch_ms * 1e-3) / 1e9
    traffic = MEASURED_TRAFFIC.get((n_sel, pool_blocks, blk))
    out = {
        "value": payload_per_step * steps / wall / 1e9,
        "ms_per_step": wall / steps * 1e3,
        "steps": steps,
        "warmup": warmup,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic["bytes"] if traffic else None,
                     "traffic_source": traffic["source"] if traffic else None,
                     "kernel": "copy_uniform_kernel<1,policy,1>",
                     "avg_launch_ms": round(avg_launch_ms, 4),
                     "min_launch_ms": round(float(np.min(kernel_ms)), 4),
                     "p99_launch_ms": round(float(np.percentile(kernel_ms, 99)), 4),
                     "gather_ms": round(float(np.mean(kernel_ms[0::2])), 4),
                     "scatter_ms": round(float(np.mean(kernel_ms[1::2])), 4),
                     "algorithmic_bytes_per_launch": algorithmic_bytes_per_launch},
        "kv": {"descriptors_per_request": n_desc, "descriptor_bytes": blk, "descriptor_order": order,
               "prepared_list_descriptors": {"pool": n_pool, "staging": n_desc},
               "prep_dlist_ms_once": round(prep_dlist_ms, 2),
               **fresh,
               "entry": "nixl_hip_prep_xfer_indexed (this plugin's own entry: index vectors lowered on the device)",
               **({"through_prepxfer": through_prepxfer} if through_prepxfer else {}),
               "block_sets_timed": len(pairs),
               "scatter_ms_by_block_set": [round(float(np.mean(kernel_ms[2 * k + 1::2 * len(pairs)])), 4) for k in range(len(pairs))],
               "post_us": {"avg": round(float(np.mean(post_us)), 1), "p99": round(float(np.percentile(post_us, 99)), 1)},
               "xfer_us": {"avg": round(float(np.mean(xfer_us)), 1), "p99": round(float(np.percentile(xfer_us, 99)), 1)}},
    }
    for g, sc, _, _ in pairs:
        g.release()
        sc.release()
    for h in (h_src, h_stg_r, h_stg_l, h_dst):
        h.release()
    agent.close()
    del src_pool, dst_pool, staging
    torch.cuda.empty_cache()
    return out


def run_concurrent_requests(args, blk, counts=(1, 2, 4), steps=10, warmup=3):
    """Several requests of config 2's shape in flight at once (the reference benchmark drives
    one request per thread, benchmark/nixlbench/src/worker/nixl/nixl_worker.cpp:1847-1879):
    n gathers posted together, each on a stream of its own (backend parameter num_streams=n),
    waited for, then the n scatters the same way; aggregate payload GB/s by wall clock beside
    the same loop with one request at a time.  Every request has its own staging buffer and its
    own block set; the scatters' destination blocks are disjoint, and the bytes are checked."""
    import torch
    from nixl_amd import nixl_agent, nixl_agent_config
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    kv = _kv_layout()
    pool_blocks, n_sel = args.pool_blocks, args.blocks
    lk = kv.layers * kv.sub_blocks_per_layer
    n_max = max(counts)
    gen = torch.Generator(device=dev)
    gen.manual_seed(77)
    src_pool = torch.empty((lk, pool_blocks, blk // 2), dtype=torch.bfloat16, device=dev)
    for i in range(lk):
        src_pool[i] = torch.randn((pool_blocks, blk // 2), generator=gen, device=dev).to(torch.bfloat16)
    dst_pool = torch.zeros((lk, pool_blocks, blk // 2), dtype=torch.bfloat16, device=dev)
    stagings = [torch.zeros((n_sel * lk, blk // 2), dtype=torch.bfloat16, device=dev) for _ in range(n_max)]
    n_desc, n_pool = n_sel * lk, lk * pool_blocks
    pool_offsets = np.arange(n_pool, dtype=np.uint64) * np.uint64(blk)
    stg_idx = np.arange(n_desc, dtype=np.int32)
    rng = np.random.default_rng(5)
    dst_perm = rng.permutation(pool_blocks)
    out = {}
    for n in counts:
        agent = nixl_agent("bench_c", nixl_agent_config(backends=()))
        agent.create_backend("HIP", {"num_streams": str(n), **dict(kv.split("=", 1) for kv in args.backend_param)})
        agent.register_memory([src_pool, dst_pool] + stagings[:n])
        h_src = agent.prep_xfer_dlist("", _triples(np.uint64(src_pool.data_ptr()) + pool_offsets, blk), "VRAM")
        h_dst = agent.prep_xfer_dlist("bench_c", _triples(np.uint64(dst_pool.data_ptr()) + pool_offsets, blk), "VRAM")
        handles, gathers, scatters, sets = [h_src, h_dst], [], [], []
        for i in range(n):
            stg_addrs = np.uint64(stagings[i].data_ptr()) + np.arange(n_desc, dtype=np.uint64) * np.uint64(blk)
            h_r = agent.prep_xfer_dlist("bench_c", _triples(stg_addrs, blk), "VRAM")
            h_l = agent.prep_xfer_dlist("", _triples(stg_addrs, blk), "VRAM")
            handles += [h_r, h_l]
            sel = rng.choice(pool_blocks, n_sel, replace=False)
            dst_ids = dst_perm[i * n_sel:(i + 1) * n_sel]  # disjoint between the requests
            sets.append((sel, dst_ids))
            gathers.append(agent.make_prepped_xfer("WRITE", h_src, _kv_indices(lk, pool_blocks, sel, args.order), h_r, stg_idx))
            scatters.append(agent.make_prepped_xfer("WRITE", h_l, stg_idx, h_dst, _kv_indices(lk, pool_blocks, dst_ids, args.order)))

        def phase(reqs):
            for req in reqs:
                if agent.transfer(req) not in ("PROC", "DONE"):
                    raise RuntimeError("post failed")
            for req in reqs:
                state = agent.check_xfer_state(req)
                while state == "PROC":
                    state = agent.check_xfer_state(req)
                if state != "DONE":
                    raise RuntimeError(f"transfer ended in state {state}")

        torch.cuda.synchronize()
        for _ in range(warmup):
            phase(gathers)
            phase(scatters)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            phase(gathers)
            phase(scatters)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        for sel, dst_ids in sets:
            sel_t, dst_t = torch.from_numpy(sel).to(dev), torch.from_numpy(dst_ids).to(dev)
            if not torch.equal(dst_pool[:, dst_t, :].view(torch.int16), src_pool[:, sel_t, :].view(torch.int16)):
                raise RuntimeError("scattered blocks differ from the source blocks")
        out[f"{n}_in_flight"] = {"aggregate_GBps": round(n * 2 * n_desc * blk * steps / wall / 1e9, 1),
                                 "ms_per_step": round(wall / steps * 1e3, 4), "streams": n}
        for req in gathers + scatters:
            req.release()
        for h in handles:
            h.release()
        agent.close()
    out["note"] = ("n gather requests posted together (a stream each) and waited for, then the n scatter requests: wall clock, "
                   f"payload of all requests; {steps} steps; descriptors of {blk} B; bytes verified")
    del src_pool, dst_pool, stagings
    torch.cuda.empty_cache()
    return out


def run_counter_sequence(args, blk, repeats=6):
    """A fixed sequence of launches for hardware-counter runs (rocprofv3 --pmc ... -- python3
    bench.py --counter-sequence), so that counters can be told apart per access pattern although
    the kernel is the same: copy_uniform_kernel `repeats` times each as (1) gather and (2)
    scatter of config 2 listed layer by layer, (3) gather and (4) scatter listed block by block,
    (5) one contiguous descriptor of the same payload; then the small-descriptor stress
    (copy_piece_kernel) and the expert-parallel dispatch and combine of both modes, whose
    kernels have names of their own.  Prints the order as one JSON line; times nothing."""
    import torch
    from nixl_amd import nixl_agent, nixl_agent_config
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    kv = _kv_layout()
    pool_blocks, n_sel = args.pool_blocks, args.blocks
    lk = kv.layers * kv.sub_blocks_per_layer
    n_desc, n_pool = n_sel * lk, lk * pool_blocks
    src_pool = torch.randint(0, 255, (lk, pool_blocks, blk), dtype=torch.uint8, device=dev)
    dst_pool = torch.zeros((lk, pool_blocks, blk), dtype=torch.uint8, device=dev)
    staging = torch.zeros((n_desc, blk), dtype=torch.uint8, device=dev)
    agent = nixl_agent("seq", nixl_agent_config(backends=()))
    agent.create_backend("HIP", dict(kv.split("=", 1) for kv in args.backend_param))
    agent.register_memory([src_pool, dst_pool, staging])
    pool_offsets = np.arange(n_pool, dtype=np.uint64) * np.uint64(blk)
    stg_addrs = np.uint64(staging.data_ptr()) + np.arange(n_desc, dtype=np.uint64) * np.uint64(blk)
    h_src = agent.prep_xfer_dlist("", _triples(np.uint64(src_pool.data_ptr()) + pool_offsets, blk), "VRAM")
    h_dst = agent.prep_xfer_dlist("seq", _triples(np.uint64(dst_pool.data_ptr()) + pool_offsets, blk), "VRAM")
    h_stg_r = agent.prep_xfer_dlist("seq", _triples(stg_addrs, blk), "VRAM")
    h_stg_l = agent.prep_xfer_dlist("", _triples(stg_addrs, blk), "VRAM")
    stg_idx = np.arange(n_desc, dtype=np.int32)
    rng = np.random.default_rng(99)
    sel = rng.choice(pool_blocks, n_sel, replace=False)
    dst_ids = rng.permutation(pool_blocks)[:n_sel]

    def run(req):
        state = agent.transfer(req)
        while state == "PROC":
            state = agent.check_xfer_state(req)
        if state != "DONE":
            raise RuntimeError(f"transfer ended in state {state}")

    order = []
    for listing in ("layer", "block"):
        gather = agent.make_prepped_xfer("WRITE", h_src, _kv_indices(lk, pool_blocks, sel, listing), h_stg_r, stg_idx)
        scatter = agent.make_prepped_xfer("WRITE", h_stg_l, stg_idx, h_dst, _kv_indices(lk, pool_blocks, dst_ids, listing))
        for name, req in ((f"gather, listed {listing} by {listing}", gather), (f"scatter, listed {listing} by {listing}", scatter)):
            for _ in range(repeats):
                run(req)
                order.append(name)
        gather.release()
        scatter.release()
    one = np.array([[src_pool.data_ptr(), n_desc * blk, 0]], dtype=np.uint64), np.array([[dst_pool.data_ptr(), n_desc * blk, 0]], dtype=np.uint64)
    req = agent.initialize_xfer("WRITE", agent.get_xfer_descs(one[0], "VRAM"), agent.get_xfer_descs(one[1], "VRAM"), "seq")
    for _ in range(repeats):
        run(req)
        order.append("one contiguous descriptor of the same payload")
    req.release()
    for h in (h_src, h_dst, h_stg_r, h_stg_l):
        h.release()
    agent.close()
    del src_pool, dst_pool, staging
    torch.cuda.empty_cache()
    run_small_descriptors(steps=repeats, warmup=1)
    from nixl_amd import ep_bench
    ep_bench.run_traffic_child(repeats=repeats, normal_mode=True)
    print(json.dumps({"copy_uniform_kernel_launches": order, "descriptor_bytes": blk, "repeats": repeats}))


def run_prep_breakdown_child(args, blk):
    """Child side of measure_prep_breakdown: requests of the headline's shape made through
    prepXfer (indexed_prep=0), each posted, waited for and released; prints the wall time of
    every make_prepped_xfer call.  The phase timings come out on stderr as the debug lines of
    the agent and of the plugin (NIXL_LOG_LEVEL=DEBUG, set by the parent)."""
    import torch
    from nixl_amd import nixl_agent, nixl_agent_config
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    kv = _kv_layout()
    pool_blocks, n_sel = args.pool_blocks, args.blocks
    lk = kv.layers * kv.sub_blocks_per_layer
    src_pool = torch.zeros((lk, pool_blocks, blk // 2), dtype=torch.bfloat16, device=dev)
    dst_pool = torch.zeros((lk, pool_blocks, blk // 2), dtype=torch.bfloat16, device=dev)
    staging = torch.zeros((n_sel * lk, blk // 2), dtype=torch.bfloat16, device=dev)
    agent = nixl_agent("bench_d", nixl_agent_config(backends=()))
    agent.create_backend("HIP", {"indexed_prep": "0", **dict(kv.split("=", 1) for kv in args.backend_param)})
    agent.register_memory([src_pool, dst_pool, staging])
    n_desc, n_pool = n_sel * lk, lk * pool_blocks
    pool_offsets = np.arange(n_pool, dtype=np.uint64) * np.uint64(blk)
    stg_addrs = np.uint64(staging.data_ptr()) + np.arange(n_desc, dtype=np.uint64) * np.uint64(blk)
    h_src = agent.prep_xfer_dlist("", _triples(np.uint64(src_pool.data_ptr()) + pool_offsets, blk), "VRAM")
    h_dst = agent.prep_xfer_dlist("bench_d", _triples(np.uint64(dst_pool.data_ptr()) + pool_offsets, blk), "VRAM")
    h_stg_r = agent.prep_xfer_dlist("bench_d", _triples(stg_addrs, blk), "VRAM")
    h_stg_l = agent.prep_xfer_dlist("", _triples(stg_addrs, blk), "VRAM")
    stg_idx = np.arange(n_desc, dtype=np.int32)
    rng = np.random.default_rng(7)
    wall_us = []
    for _ in range(10):
        sel = rng.choice(pool_blocks, n_sel, replace=False)
        dst_ids = rng.permutation(pool_blocks)[:n_sel]
        for local, li, remote, ri in ((h_src, _kv_indices(lk, pool_blocks, sel, args.order), h_stg_r, stg_idx),
                                      (h_stg_l, stg_idx, h_dst, _kv_indices(lk, pool_blocks, dst_ids, args.order))):
            t0 = time.perf_counter()
            req = agent.make_prepped_xfer("WRITE", local, li, remote, ri)
            wall_us.append((time.perf_counter() - t0) * 1e6)
            state = agent.transfer(req)
            while state == "PROC":
                state = agent.check_xfer_state(req)
            req.release()
    print(json.dumps({"make_prepped_xfer_wall_us": wall_us, "descriptors": n_desc}))
    for h in (h_src, h_dst, h_stg_r, h_stg_l):
        h.release()
    agent.close()


def parse_prep_debug_lines(text):
    """The phase timings in the debug output of the agent (makeXferReq) and of the plugin
    (prepXfer), one entry per request: lists of microseconds by phase."""
    import re
    phases = {"agent_expand_index_pairs": [], "plugin_block_pass": [], "plugin_plan_from_records": [], "plugin_rest": []}
    paths = []
    for line in text.splitlines():
        m = re.search(r"makeXferReq: merged \d+ indices into \d+ descriptors in ([0-9.e+-]+) us", line)
        if m:
            phases["agent_expand_index_pairs"].append(float(m.group(1)))
        m = re.search(r"prepXfer of \d+ descriptors \((\w+)\): block pass ([0-9.e+-]+) us, plan from records ([0-9.e+-]+) us, "
                      r"rest \([^)]*\) ([0-9.e+-]+) us", line)
        if m:
            paths.append(m.group(1))
            for key, value in zip(("plugin_block_pass", "plugin_plan_from_records", "plugin_rest"), m.groups()[1:]):
                phases[key].append(float(value))
    return phases, paths


def measure_prep_breakdown(args, blk):
    """Where the time of one request made through prepXfer goes, per phase, in microseconds
    (median over the requests of a child run of this file with the libraries' debug lines on):
    the agent's expansion of the index pairs into two descriptor lists, the plugin's pass over
    those lists (checks against the registrations + records written to the pinned upload
    buffer), the plan made from the records (arena, queued upload and sort, events), and what is
    left of the call's wall time (C wrapper, ctypes, copies of the index vectors)."""
    import subprocess
    child = [sys.executable, os.path.abspath(__file__), "--prep-breakdown-child", "--block-bytes", str(blk), "--order", args.order,
             "--blocks", str(args.blocks), "--pool-blocks", str(args.pool_blocks)]
    for kv in args.backend_param:
        child += ["--backend-param", kv]
    try:
        proc = subprocess.run(child, env={**os.environ, "NIXL_LOG_LEVEL": "DEBUG"}, capture_output=True, text=True, timeout=180)
    except subprocess.TimeoutExpired:
        return {"error": "the child run did not finish in 180 s"}
    if proc.returncode != 0:
        return {"error": f"the child run ended with status {proc.returncode}: {proc.stderr[-300:]}"}
    phases, paths = parse_prep_debug_lines(proc.stderr)
    try:
        report = json.loads(proc.stdout.strip().splitlines()[-1])
    except (ValueError, IndexError):
        return {"error": "the child run printed no timings"}
    wall = report["make_prepped_xfer_wall_us"][4:]  # the first requests also pay one-off allocations
    if not wall or any(len(v) < len(report["make_prepped_xfer_wall_us"]) for v in phases.values()):
        return {"error": "debug lines missing from the child run"}
    out = {k: round(float(np.median(v[4:])), 1) for k, v in phases.items()}
    out["make_prepped_xfer_wall"] = round(float(np.median(wall)), 1)
    out["wrapper_and_other"] = round(out["make_prepped_xfer_wall"] - sum(out[k] for k in phases), 1)
    out["plugin_prepxfer_total"] = round(out["plugin_block_pass"] + out["plugin_plan_from_records"] + out["plugin_rest"], 1)
    out["descriptors_per_request"] = report["descriptors"]
    out["plugin_path"] = sorted(set(paths))
    out["source"] = "median over the requests of a child run of this file with NIXL_LOG_LEVEL=DEBUG (phase timers of agent and plugin)"
    return out


def run_small_descriptors(steps=20, warmup=3, backend_params=None, in_destination_order=False):
    """Small-descriptor stress: 262 144 VRAM->VRAM descriptors with sizes log-uniform in
    [512 B, 4 KiB] rounded to 16 B, random 16-byte-aligned offsets in two 4 GiB buffers,
    destinations non-overlapping.  One request through the agent; HIP events on the launch
    stream around every post.  in_destination_order: the same descriptors listed by ascending
    destination address (what a caller that can order its list gets)."""
    import torch
    from nixl_amd import nixl_agent, nixl_agent_config
    dev = torch.device("cuda:0")
    n, buf_bytes = 262144, 4 << 30
    rng = np.random.default_rng(2025)
    lens = ((np.exp(rng.uniform(np.log(512), np.log(4096), n)).astype(np.int64) // 16) * 16).astype(np.uint64)
    src = torch.zeros(buf_bytes, dtype=torch.uint8, device=dev)
    dst = torch.zeros(buf_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.Stream(device=dev)
    agent = nixl_agent("small", nixl_agent_config(backends=()))
    agent.create_backend("HIP", {"stream": str(stream.cuda_stream), **(backend_params or {})})
    agent.register_memory([src, dst])
    so = (rng.integers(0, (buf_bytes - 4096) // 16, n) * 16).astype(np.uint64)
    do = (rng.permutation(buf_bytes // 8192)[:n] * 8192 + rng.integers(0, (8192 - 4096) // 16, n) * 16).astype(np.uint64)
    if in_destination_order:
        by_dst = np.argsort(do)
        so, do, lens = so[by_dst], do[by_dst], lens[by_dst]
    zeros = np.zeros(n, dtype=np.uint64)
    hl = agent.prep_xfer_dlist("", np.stack([np.uint64(src.data_ptr()) + so, lens, zeros], 1), "VRAM")
    hr = agent.prep_xfer_dlist("small", np.stack([np.uint64(dst.data_ptr()) + do, lens, zeros], 1), "VRAM")
    idx = np.arange(n)
    make_ms = []
    for _ in range(5):  # the first call also sizes the pooled storage
        t0 = time.perf_counter()
        req = agent.make_prepped_xfer("WRITE", hl, idx, hr, idx)
        make_ms.append((time.perf_counter() - t0) * 1e3)
        if len(make_ms) < 5:
            req.release()
    flush = torch.empty(512 << 20, dtype=torch.uint8, device=dev)  # twice the last-level cache
    torch.cuda.synchronize()
    times = []
    for i in range(warmup + steps):
        with torch.cuda.stream(stream):
            flush.fill_(i & 1)  # on the launch stream, so that it is over before the timed launch starts
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        state = agent.transfer(req)
        e1.record(stream)
        while state == "PROC":
            state = agent.check_xfer_state(req)
        if state != "DONE":
            raise RuntimeError(f"transfer ended in state {state}")
        e1.synchronize()
        if i >= warmup:
            times.append(e0.elapsed_time(e1) * 1e3)
    payload = int(lens.sum())
    us = float(np.mean(times))
    for h in (req, hl, hr):
        h.release()
    agent.close()
    del src, dst, flush
    torch.cuda.empty_cache()
    gbps = 2 * payload / (us * 1e-6) / 1e9
    traffic = MEASURED_TRAFFIC.get(("small", n))
    return {"descriptors": n, "payload_bytes": payload, "avg_launch_us": round(us, 1), "achieved_GBps": round(gbps, 1),
            "frac": round(gbps / HBM_PEAK_GBPS, 4), "ns_per_descriptor": round(us * 1e3 / n, 3),
            "make_request_ms": round(min(make_ms[1:]), 2),
            "traffic": traffic["bytes"] if traffic else None, "traffic_source": traffic["source"] if traffic else None,
            "cache_flush": "512 MB written on the launch stream before every timed launch",
            "kernel": "copy_piece_kernel<policy,4,1>"}


def run_ceilings(iters=20):
    """What this GPU gives a plain copy of 1 GiB, as context for the roofline fractions: the
    runtime's own device-to-device copy (torch's copy_, i.e. hipMemcpyAsync) and this
    backend's kernel on ONE contiguous 1 GiB descriptor.  HBM traffic (read + write) per
    second, HIP events on the launch stream, caches flushed before every launch."""
    import torch
    from nixl_amd import nixl_agent, nixl_agent_config
    dev = torch.device("cuda:0")
    n = 1 << 30
    src = torch.randint(0, 255, (n,), dtype=torch.uint8, device=dev)
    dst = torch.zeros(n, dtype=torch.uint8, device=dev)
    flush = torch.empty(512 << 20, dtype=torch.uint8, device=dev)
    stream = torch.cuda.Stream(device=dev)
    agent = nixl_agent("ceiling", nixl_agent_config(backends=()))
    agent.create_backend("HIP", {"stream": str(stream.cuda_stream)})
    agent.register_memory([src, dst])
    req = agent.initialize_xfer("WRITE", agent.get_xfer_descs(src), agent.get_xfer_descs(dst), "ceiling")

    def plugin():
        state = agent.transfer(req)
        while state == "PROC":
            state = agent.check_xfer_state(req)
        if state != "DONE":
            raise RuntimeError(f"transfer ended in state {state}")

    def runtime():
        with torch.cuda.stream(stream):
            dst.copy_(src)

    out = {}
    for name, fn in (("runtime_copy_1GiB", runtime), ("this_backend_one_1GiB_descriptor", plugin)):
        times = []
        for i in range(iters + 3):
            with torch.cuda.stream(stream):
                flush.fill_(i & 1)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            fn()
            e1.record(stream)
            e1.synchronize()
            if i >= 3:
                times.append(e0.elapsed_time(e1) * 1e-3)
        if not torch.equal(dst, src):
            raise RuntimeError(f"{name}: copy differs from its source")
        dst.zero_()
        gbps = 2 * n / float(np.mean(times)) / 1e9
        out[name] = {"traffic_GBps": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBPS, 4),
                     "avg_us": round(float(np.mean(times)) * 1e6, 1)}
    req.release()
    agent.close()
    del src, dst, flush
    torch.cuda.empty_cache()
    out["note"] = ("a plain copy of 1 GiB on this GPU, read + write per second: the runtime's device-to-device copy and this "
                   "backend's kernel on one contiguous descriptor; context for the fractions above, not a target")
    return out


def run_calibration_copy():
    """One launch of torch's element-wise add over 2^28 int32: reads exactly 1 GiB, writes 1 GiB."""
    import torch
    a = torch.ones(1 << 28, dtype=torch.int32, device="cuda:0")
    b = torch.empty_like(a)
    torch.cuda.synchronize()
    torch.add(a, 1, out=b)
    torch.cuda.synchronize()
    del a, b
    torch.cuda.empty_cache()


def run_ep_cpu_baseline(seconds=10.0, threads=1, full=False):
    """Scalar CPU restatement of the low-latency kernels (the oracle) on `threads` host
    threads.  full=True: BASELINE config 4 at its own size (32 virtual ranks x 128 tokens x
    7168, 256 experts, top-8, fp8), a few passes; otherwise a bounded sample of 1/8 of its
    tokens and experts for `seconds`."""
    from oracle import ep_oracle as eo
    R, T, H, K, E, M = (32, 128, 7168, 8, 256, 128) if full else (4, 128, 7168, 8, 32, 128)
    rng = np.random.default_rng(4)
    x = eo.f32_to_bf16(rng.standard_normal((R, T, H)).astype(np.float32))
    logits = rng.standard_normal((R * T, E)).astype(np.float32)
    topk, w = eo.router(logits, K)
    topk, w = topk.reshape(R, T, K), w.reshape(R, T, K)
    y = np.zeros((R, E // R, R * M, H), np.uint16)  # expert outputs; only the received rows are ever touched
    t0 = time.perf_counter()
    n = 0
    d_us, c_us = [], []
    while (n < 3) if full else (time.perf_counter() - t0 < seconds or n < 2):
        a = time.perf_counter()
        o = eo.ll_dispatch(x, topk, E, M, use_fp8=True, threads=threads, fill=None)
        b = time.perf_counter()
        eo.ll_combine(y, topk, w, o["src_info"], o["layout_range"], E, M, threads=threads)
        c = time.perf_counter()
        if n or not full:  # at full size the first pass also faults the output pages in
            d_us.append((b - a) * 1e6)
            c_us.append((c - b) * 1e6)
        n += 1
        del o
    return {"dispatch_us": round(float(np.mean(d_us)), 1), "combine_us": round(float(np.mean(c_us)), 1),
            "cores": threads, "kind": "port", "host_cpus": os.cpu_count(),
            "sample": f"{len(d_us)} passes, {R} virtual ranks x {T} tokens x {H}, {E} experts, top-{K}, fp8"
                      + (" (config 4 at full size)" if full else " (1/8 of config 4's tokens and experts)")}


def run_config1(seconds=6.0):
    """BASELINE config 1 as stated: DRAM->DRAM loopback through one agent, 4096 descriptors of
    16 KiB (64 MiB), payload uniform random bytes from a seed, destination block ids a seeded
    permutation of 0..4095, WRITE, verified bit for bit.  Backend: the per-descriptor memcpy
    plugin (the semantics of the reference's UCX loopback puts; libucp is not in this image).
    Stages split as the reference benchmark splits them
    (benchmark/nixlbench/src/worker/nixl/nixl_worker.cpp:1583-1644): prepare = createXferReq,
    post = postXferReq, transfer = post until completion."""
    from nixl_amd import nixl_agent, nixl_agent_config
    n, blk = 4096, 16384
    rng = np.random.default_rng(1)
    src = rng.integers(0, 256, n * blk, dtype=np.uint8)
    dst = np.zeros(n * blk, dtype=np.uint8)
    perm = rng.permutation(n).astype(np.uint64)
    agent = nixl_agent("c1", nixl_agent_config(backends=()), plugin_dirs=[os.path.join(ROOT, "oracle", "_build")])
    agent.create_backend("MEMCPY", {"threads": "1"})
    for a in (src, dst):
        agent.register_memory(np.array([[a.ctypes.data, a.nbytes, 0]], dtype=np.uint64), "DRAM")
    lens, zeros = np.full(n, blk, np.uint64), np.zeros(n, np.uint64)
    local = agent.get_xfer_descs(np.stack([np.uint64(src.ctypes.data) + np.arange(n, dtype=np.uint64) * np.uint64(blk), lens, zeros], 1), "DRAM")
    remote = agent.get_xfer_descs(np.stack([np.uint64(dst.ctypes.data) + perm * np.uint64(blk), lens, zeros], 1), "DRAM")
    prep, post, xfer = [], [], []
    t_end = time.perf_counter() + seconds
    while time.perf_counter() < t_end or len(xfer) < 3:
        t0 = time.perf_counter()
        req = agent.initialize_xfer("WRITE", local, remote, "c1")
        t1 = time.perf_counter()
        state = agent.transfer(req)
        t2 = time.perf_counter()
        while state == "PROC":
            state = agent.check_xfer_state(req)
        t3 = time.perf_counter()
        if state != "DONE":
            raise RuntimeError("config 1 transfer failed")
        req.release()
        prep.append((t1 - t0) * 1e6)
        post.append((t2 - t1) * 1e6)
        xfer.append((t3 - t1) * 1e6)
    if not np.array_equal(dst.reshape(n, blk)[perm.astype(np.int64)], src.reshape(n, blk)):
        raise RuntimeError("config 1: destination bytes differ")
    agent.close()
    stat = lambda v: {"avg": round(float(np.mean(v)), 1), "p99": round(float(np.percentile(v, 99)), 1)}
    return {"value": round(n * blk / (float(np.mean(xfer)) * 1e-6) / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{len(xfer)} iterations of {n} descriptors x {blk} B (64 MiB), DRAM->DRAM loopback, permuted "
                      "destinations, agent + per-descriptor memcpy backend, verified bit for bit",
            "prepare_us": stat(prep), "post_us": stat(post), "transfer_us": stat(xfer)}


def run_posix_analogue(seconds=4.0):
    """What the reference's POSIX backend does with a descriptor list, without the plugin: one
    pwrite per descriptor from DRAM into a file, then one pread per descriptor back
    (src/plugins/posix/posix_backend.cpp: local DRAM, remote FILE only).  The file lives in
    /dev/shm, so this is memory to memory through the kernel's file layer: a labelled
    substitute, not a KV-to-KV copy.  4096 descriptors x 16 KiB (BASELINE config 1)."""
    n, blk = 4096, 16384
    rng = np.random.default_rng(1)
    src = rng.integers(0, 256, n * blk, dtype=np.uint8)
    back = np.zeros_like(src)
    order = rng.permutation(n)
    path = f"/dev/shm/nixl_amd_bench_{os.getpid()}.bin"
    fd = os.open(path, os.O_RDWR | os.O_CREAT | os.O_TRUNC, 0o600)
    try:
        os.ftruncate(fd, n * blk)
        src_v, back_v = memoryview(src), memoryview(back)
        t0 = time.perf_counter()
        rounds = 0
        while time.perf_counter() - t0 < seconds or rounds == 0:
            for i, j in enumerate(order):
                os.pwrite(fd, src_v[i * blk:(i + 1) * blk], int(j) * blk)
            for i, j in enumerate(order):
                os.preadv(fd, [back_v[i * blk:(i + 1) * blk]], int(j) * blk)
            rounds += 1
        wall = time.perf_counter() - t0
        if not np.array_equal(src, back):
            raise RuntimeError("POSIX analogue: bytes read back differ")
    finally:
        os.close(fd)
        os.unlink(path)
    return {"value": round(2 * n * blk * rounds / wall / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{rounds} rounds of {n} x pwrite then {n} x pread of {blk} B, file in /dev/shm, {wall:.1f} s; "
                      "Python call overhead per descriptor included"}


def run_cpu_baseline(seconds=12.0, threads=1, blk=16384):
    """Reference-shaped CPU path: one agent, loopback, DRAM->DRAM, one memcpy per descriptor
    (the semantics of the reference's UCX loopback puts, src/plugins/ucx/ucx_backend.cpp:
    1216-1262).  Same KV shape as the GPU workload with the pool cut to 512 blocks and 64
    selected blocks (4096 descriptors of `blk` bytes per request)."""
    from nixl_amd import nixl_agent, nixl_agent_config
    plugin_dir = os.path.join(ROOT, "oracle", "_build")
    kv = _kv_layout()
    layers, pool_blocks, n_sel = kv.layers, 512, 64
    lk = layers * kv.sub_blocks_per_layer
    rng = np.random.default_rng(7)
    src_pool = rng.integers(0, 256, lk * pool_blocks * blk, dtype=np.uint8)
    dst_pool = np.zeros(lk * pool_blocks * blk, dtype=np.uint8)
    staging = np.zeros(n_sel * lk * blk, dtype=np.uint8)
    agent = nixl_agent("cpu", nixl_agent_config(backends=()), plugin_dirs=[plugin_dir])
    agent.create_backend("MEMCPY", {"threads": str(threads)})
    for a in (src_pool, dst_pool, staging):
        agent.register_memory(np.array([[a.ctypes.data, a.nbytes, 0]], dtype=np.uint64), "DRAM")
    sel = rng.choice(pool_blocks, n_sel, replace=False)
    dst_ids = rng.permutation(pool_blocks)[:n_sel]
    n_desc = n_sel * lk
    src_addrs = _kv_descs(src_pool.ctypes.data, layers, pool_blocks, blk, sel, "layer")
    dst_addrs = _kv_descs(dst_pool.ctypes.data, layers, pool_blocks, blk, dst_ids, "layer")
    stg_addrs = np.uint64(staging.ctypes.data) + np.arange(n_desc, dtype=np.uint64) * np.uint64(blk)
    h_src = agent.prep_xfer_dlist("", _triples(src_addrs, blk), "DRAM")
    h_stg_r = agent.prep_xfer_dlist("cpu", _triples(stg_addrs, blk), "DRAM")
    h_stg_l = agent.prep_xfer_dlist("", _triples(stg_addrs, blk), "DRAM")
    h_dst = agent.prep_xfer_dlist("cpu", _triples(dst_addrs, blk), "DRAM")
    idx = np.arange(n_desc)
    gather = agent.make_prepped_xfer("WRITE", h_src, idx, h_stg_r, idx)
    scatter = agent.make_prepped_xfer("WRITE", h_stg_l, idx, h_dst, idx)
    for req in (gather, scatter):
        agent.transfer(req)
    steps = 0
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for req in (gather, scatter):
            if agent.transfer(req) != "DONE":
                raise RuntimeError("CPU baseline transfer failed")
        steps += 1
    wall = time.perf_counter() - t0
    ok = np.array_equal(dst_pool.reshape(lk, pool_blocks, blk)[:, dst_ids], src_pool.reshape(lk, pool_blocks, blk)[:, sel])
    if not ok:
        raise RuntimeError("CPU baseline result is wrong")
    value = 2 * n_desc * blk * steps / wall / 1e9
    for h in (gather, scatter, h_src, h_stg_r, h_stg_l, h_dst):
        h.release()
    agent.close()
    return {"value": round(value, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{steps} steps of gather+scatter, {n_desc} descriptors x {blk} B per request, "
                      f"DRAM->DRAM loopback, agent + per-descriptor memcpy backend, {wall:.1f} s",
            "host_cpus": os.cpu_count()}


def _leg(fn, *a, **kw):
    """Runs one of the legs beside the headline; a leg that fails is reported in its place (and
    on stderr) instead of taking the line, and the legs that did run, with it."""
    try:
        return fn(*a, **kw)
    except Exception as e:  # noqa: BLE001 - whatever it was, the line still goes out
        import traceback
        traceback.print_exc()
        return {"error": f"{type(e).__name__}: {e}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--blocks", type=int, default=1024, help="KV blocks moved per request")
    ap.add_argument("--pool-blocks", type=int, default=8192)
    ap.add_argument("--block-bytes", type=int, default=0,
                    help="bytes per (layer, K|V) descriptor; 0: 16384, the size the metric names, with the 32 KiB point "
                         "(16 tokens per block) and the other descriptor order reported beside it")
    ap.add_argument("--backend-param", action="append", default=[], metavar="KEY=VALUE",
                    help="extra parameter for the HIP backend of the KV legs (units_per_lane, nontemporal, ...)")
    ap.add_argument("--fresh-requests", type=int, default=4,
                    help="request pairs with a new block list each, timed with their preparation")
    ap.add_argument("--quick", action="store_true", help="headline point only, no other sizes or orders")
    ap.add_argument("--headline-only", action="store_true",
                    help="nothing but the headline's steady-state loop (for a kernel trace whose rows are that loop's "
                         "launches alone); implies --quick --no-ep --no-small --no-cpu-baseline --no-live-traffic")
    ap.add_argument("--order", choices=("layer", "block"), default="layer",
                    help="descriptor list order: layer by layer, or block by block")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-ep", action="store_true")
    ap.add_argument("--no-small", action="store_true", help="skip the small-descriptor stress")
    ap.add_argument("--ep-iters", type=int, default=50, help="timed calls per expert-parallel kernel")
    ap.add_argument("--ep-warmup", type=int, default=20)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain element-wise kernel that reads 1 GiB and writes 1 GiB, as the "
                         "known-size yardstick for hardware counter runs")
    ap.add_argument("--prep-breakdown-child", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--ep-traffic-child", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--counter-sequence", action="store_true",
                    help="run a fixed sequence of launches for hardware-counter runs and print its order; nothing is timed")
    ap.add_argument("--no-live-traffic", action="store_true",
                    help="do not run the headline leg under rocprofv3 --pmc first; roofline.traffic then comes from "
                         "the counter runs summarised under profiles/")
    args = ap.parse_args()
    if args.headline_only:
        args.quick = args.no_ep = args.no_small = args.no_cpu_baseline = args.no_live_traffic = True
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (virtual ranks are regions of one "
                 "GPU's HBM); --gpus must be 1")

    import __graft_entry__ as entry
    entry._ensure_built()

    blk = args.block_bytes or 16384  # the metric is quoted "@16KB blocks"
    if args.prep_breakdown_child:
        run_prep_breakdown_child(args, blk)
        return
    if args.counter_sequence:
        run_counter_sequence(args, blk)
        return
    if args.ep_traffic_child:
        from nixl_amd import ep_bench
        run_calibration_copy()
        ep_bench.run_traffic_child()
        return
    if args.calibrate_copy:
        run_calibration_copy()
    kv = run_kv(args, blk, args.order, args.steps, args.warmup, fresh_requests=args.fresh_requests,
                descriptor_path=not args.quick)
    tokens_per_block = blk // (_kv_layout().bytes_per_sub_block // 16)
    line = {
        "metric": "KV xfer GB/s (% HBM peak) @16KB blocks; EP dispatch+combine µs @7168 top-8",
        "value": round(kv["value"], 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(kv["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": f"Llama-3-8B paged KV, VRAM->VRAM on one GPU: 32 layers x {{K,V}}, {tokens_per_block} tokens per "
                               f"block ({blk} B per layer/K-or-V block), pool {args.pool_blocks} blocks, {args.blocks} blocks "
                               f"gathered to staging then scattered, {kv['kv']['descriptors_per_request']} descriptors x "
                               f"{blk} B per request, listed {args.order} by {args.order}",
                   "payload_bytes_per_step": 2 * kv["kv"]["descriptors_per_request"] * blk,
                   "pct_hbm_peak_payload_x2": round(2 * kv["value"] / HBM_PEAK_GBPS * 100, 1)},
        "roofline": kv["roofline"],
        "kv": kv["kv"],
    }
    if not args.block_bytes and not args.quick:
        def other_points():
            # beside the headline: config 2 as BASELINE words it (16 tokens per block, 32 KiB), and
            # both sizes with the descriptors listed the other way round; each with its own roofline
            others = {}
            other_order = "block" if args.order == "layer" else "layer"
            for b, o in ((32768, args.order), (16384, other_order), (32768, other_order)):
                r = run_kv(args, b, o, max(args.steps // 2, 1), max(args.warmup // 2, 1), fresh_requests=2)
                others[f"{b // 1024}KiB_{o}_order"] = {
                    "value_GBps": round(r["value"], 1), "roofline": r["roofline"],
                    "make_request_pair_ms": r["kv"]["make_request_pair_ms"],
                    "value_including_prepare": r["kv"]["value_including_prepare"]}
            r = run_kv(args, 16384, "block", max(args.steps // 2, 1), max(args.warmup // 2, 1), fresh_requests=2, pad_blocks=1)
            others["16KiB_block_order_slabs_one_block_longer"] = {
                "value_GBps": round(r["value"], 1), "roofline": r["roofline"],
                "note": "the same requests over pools whose (layer, K|V) slabs are 8193 blocks long instead of 8192, so that "
                        "the 64 sub-blocks of a block id no longer lie a power of two (128 MiB) apart: what the layout, not "
                        "the engine, decides"}
            r = run_kv(args, blk, args.order, max(args.steps // 2, 1), max(args.warmup // 2, 1), fresh_requests=2, sorted_ids=True)
            others[f"{blk // 1024}KiB_{args.order}_order_source_blocks_ascending"] = {
                "value_GBps": round(r["value"], 1), "roofline": r["roofline"],
                "note": "the same random block sets and random destinations, the request listing its source blocks in "
                        "ascending order: the gather then reads the pool monotonically"}
            return others

        line["kv"]["other_points"] = _leg(other_points)
    if not args.quick:
        line["kv"]["concurrent_requests"] = _leg(run_concurrent_requests, args, blk)
    if not args.no_small:
        line["kv"]["small_descriptor_stress"] = _leg(run_small_descriptors)
        ordered = _leg(lambda: run_small_descriptors(steps=10, in_destination_order=True))
        if isinstance(ordered, dict) and "avg_launch_us" in ordered:
            ordered = {k: ordered[k] for k in ("avg_launch_us", "achieved_GBps", "frac", "ns_per_descriptor", "make_request_ms")}
            ordered["note"] = "the same descriptors listed by ascending destination address"
        line["kv"]["small_descriptor_stress_in_destination_order"] = ordered
    if not args.quick:
        line["kv"]["plain_copy_ceilings"] = _leg(run_ceilings)
    many = min(16, os.cpu_count() or 1)
    if not args.no_ep:
        from nixl_amd import ep_bench
        line["ep"] = _leg(ep_bench.run, args)
        if not args.no_cpu_baseline:
            line["ep"]["cpu_baseline"] = _leg(run_ep_cpu_baseline, seconds=6.0)
            if many > 1:
                line["ep"]["cpu_baseline"]["all_cores_full_size"] = _leg(run_ep_cpu_baseline, threads=many, full=True)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = _leg(run_cpu_baseline, blk=blk)
        # the same path with the descriptor list split over the box's CPU share, reported beside
        if many > 1:
            line["cpu_baseline"]["all_cores"] = _leg(run_cpu_baseline, seconds=5.0, threads=many, blk=blk)
        line["cpu_baseline"]["config1"] = _leg(run_config1)
        line["cpu_baseline"]["posix_path_analogue"] = _leg(run_posix_analogue)
        # the reference's own loopback needs libucp, which this image does not ship
        import ctypes.util
        line["cpu_baseline"]["libucp"] = ctypes.util.find_library("ucp") or "absent"
    # Last, when everything timed is over: the counter runs are processes of their own.  With
    # them ahead of the timed legs this process's wall-clock figures came out at half (its
    # kernel times unchanged); behind them they disturb nothing.
    if not args.quick:
        line["kv"]["through_prepxfer"]["prep_breakdown_us"] = _leg(measure_prep_breakdown, args, blk)
    if not args.no_live_traffic and not args.no_ep and "low_latency" in line.get("ep", {}):
        ep_live = _leg(measure_ep_traffic_live)
        for mode, call, key in (("low_latency", "dispatch", "ll_dispatch"), ("low_latency", "combine", "ll_combine"),
                                ("normal", "dispatch", "ht_dispatch"), ("normal", "combine", "ht_combine")):
            slot = line["ep"].get(mode, {}).get(call)
            if isinstance(slot, dict):
                slot.update(ep_live[key] if key in ep_live else {"traffic": None, "traffic_live_error": ep_live.get("error")})
    live = None if args.no_live_traffic else measure_traffic_live(args, blk)
    if live and "bytes" in live:
        line["roofline"]["traffic"] = live["bytes"]
        line["roofline"]["traffic_source"] = live["source"]
        line["roofline"]["traffic_detail"] = {k: live[k] for k in ("read_bytes", "written_bytes", "read_requests", "yardstick",
                                                                   "launches_sampled")}
    elif live:
        line["roofline"]["traffic_live_error"] = live["error"]
    print(json.dumps(line))


if __name__ == "__main__":
    main()
