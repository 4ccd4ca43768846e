#!/usr/bin/env python3
"""nixlbench-style sweep over the agent API, single instance.

Mirrors the reference benchmark's flags, loops and report
(benchmark/nixlbench/src/utils/utils.cpp:48-140 flags, :1295-1420 report;
benchmark/nixlbench/src/worker/nixl/nixl_worker.cpp:1707-1831 transfer loop) for the one
mode that needs no second process: one agent whose transfers target itself, the way the
reference runs storage backends (nixl_worker.cpp:1857).  For every block size from
--start_block_size to --max_block_size (doubling) and every batch size from
--start_batch_size to --max_batch_size (doubling): warm up, then run --num_iter transfers of
`batch` descriptors of `block` bytes with --pipeline_depth requests in flight, and print

    Block Size (B)  Batch Size  B/W (GB/Sec)  Avg Lat. (us)  Avg Prep (us)  P99 Prep (us)
    Avg Post (us)  P99 Post (us)  Avg Tx (us)  P99 Tx (us)

with B/W = block * batch * iterations / total wall time in decimal GB (utils.cpp:1357-1368).

    python -m nixl_amd.nixlbench --backend HIP --initiator_seg_type VRAM --target_seg_type VRAM \\
        --start_block_size 4096 --max_block_size 1048576 --start_batch_size 1 --max_batch_size 1024 \\
        --prepared_xfer --check_consistency
"""
import argparse
import sys
import time

import numpy as np

from .agent import NixlError, nixl_agent, nixl_agent_config

LARGE_BLOCK_SIZE = 1 << 20  # utils.h: iterations are divided by large_blk_iter_ftr above this


def parse(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--backend", default="HIP", help="backend plugin name (HIP, or any plugin found in --plugin_dir)")
    ap.add_argument("--plugin_dir", default="", help="extra directory searched for libplugin_<NAME>.so")
    ap.add_argument("--backend_params", default="", help="comma-separated key=value pairs passed to createBackend")
    ap.add_argument("--initiator_seg_type", default="VRAM", choices=["DRAM", "VRAM"])
    ap.add_argument("--target_seg_type", default="VRAM", choices=["DRAM", "VRAM"])
    ap.add_argument("--op_type", default="WRITE", choices=["READ", "WRITE"])
    ap.add_argument("--check_consistency", action="store_true")
    ap.add_argument("--total_buffer_size", type=int, default=8 << 30)
    ap.add_argument("--start_block_size", type=int, default=4 << 10)
    ap.add_argument("--max_block_size", type=int, default=64 << 20)
    ap.add_argument("--start_batch_size", type=int, default=1)
    ap.add_argument("--max_batch_size", type=int, default=1)
    ap.add_argument("--num_iter", type=int, default=1000)
    ap.add_argument("--warmup_iter", type=int, default=100)
    ap.add_argument("--large_blk_iter_ftr", type=int, default=16)
    ap.add_argument("--pipeline_depth", type=int, default=1)
    ap.add_argument("--num_threads", type=int, default=1,
                    help="threads that each drive their own requests over their own part of the buffers; num_iter must "
                         "be divisible by it (utils.cpp:94-98)")
    ap.add_argument("--recreate_xfer", action="store_true")
    ap.add_argument("--prepared_xfer", action="store_true")
    ap.add_argument("--randomize_location_mode", default="none", choices=["none", "blockaligned"])
    ap.add_argument("--device_id", type=int, default=0)
    ap.add_argument("--seed", type=int, default=1)
    a = ap.parse_args(argv)
    if a.start_block_size <= 0 or a.max_block_size < a.start_block_size:
        ap.error("block sizes must satisfy 0 < start_block_size <= max_block_size")
    if a.start_batch_size <= 0 or a.max_batch_size < a.start_batch_size:
        ap.error("batch sizes must satisfy 0 < start_batch_size <= max_batch_size")
    if a.pipeline_depth < 1 or a.num_iter < 1 or a.warmup_iter < 0:
        ap.error("pipeline_depth and num_iter must be positive, warmup_iter non-negative")
    if a.num_threads < 1 or a.num_iter < a.num_threads or a.num_iter % a.num_threads:
        ap.error("num_iter must be at least num_threads and divisible by it")
    if a.max_block_size * a.max_batch_size * 2 * a.num_threads > a.total_buffer_size:
        ap.error("max_block_size * max_batch_size needs two buffers a thread inside total_buffer_size")
    return a


class Segment:
    """One buffer of a memory type, with host-side fill / read-back for the consistency check."""

    def __init__(self, kind, nbytes, device_id, pinned=False):
        self.kind, self.nbytes = kind, nbytes
        self._pinned = None
        if kind == "DRAM" and pinned:  # page-locked host memory, which a GPU backend needs
            import torch
            self._pinned = torch.zeros(nbytes, dtype=torch.uint8, pin_memory=True)
            self.buf = self._pinned.numpy()
            self.addr = self._pinned.data_ptr()
        elif kind == "VRAM":
            import torch
            if not torch.cuda.is_available():
                raise SystemExit("nixlbench: VRAM segments need a GPU")
            self._torch = torch
            self.buf = torch.zeros(nbytes, dtype=torch.uint8, device=f"cuda:{device_id}")
            self.addr = self.buf.data_ptr()
        else:
            self.buf = np.zeros(nbytes, dtype=np.uint8)
            self.addr = self.buf.ctypes.data
        self.dev = device_id if kind == "VRAM" else 0

    def fill(self, host_bytes, at=0):
        if self.kind == "VRAM":
            self.buf[at:at + host_bytes.size].copy_(self._torch.from_numpy(host_bytes))
            self._torch.cuda.synchronize()
        else:
            self.buf[at:at + host_bytes.size] = host_bytes

    def read(self, n, at=0):
        if self.kind == "VRAM":
            self._torch.cuda.synchronize()
            return self.buf[at:at + n].cpu().numpy()
        return self.buf[at:at + n].copy()


class Stat:
    def __init__(self):
        self.v = []

    def add(self, x):
        self.v.append(x)

    def avg(self):
        return float(np.mean(self.v)) if self.v else 0.0

    def p99(self):
        return float(np.percentile(self.v, 99)) if self.v else 0.0


def _us():
    return time.perf_counter() * 1e6


def run_point(agent, a, local, remote, block, batch, out):
    """One (block size, batch size) point: warm-up, timed loop, optional byte check.  With
    --num_threads N the point runs in N threads at once, each over its own N-th of the two
    buffers with its own requests and num_iter / N iterations, as the reference's worker does
    (nixl_worker.cpp:1847-1879, 2004); the bandwidth is all threads' bytes over the wall time."""
    if a.num_threads > 1:
        return run_point_threads(agent, a, local, remote, block, batch, out)
    return run_point_one(agent, a, local, remote, block, batch, out)


def run_point_threads(agent, a, local, remote, block, batch, out):
    import copy
    import io
    import threading
    n = a.num_threads
    share = a.max_block_size * a.max_batch_size
    per = copy.copy(a)
    per.num_threads, per.num_iter, per.warmup_iter = 1, a.num_iter // n, max(a.warmup_iter // n, 0)
    results, errors = [None] * n, []
    gate = threading.Barrier(n + 1)

    def work(tid):
        try:
            results[tid] = run_point_one(agent, per, local, remote, block, batch, io.StringIO(), base=tid * share,
                                         seed_salt=tid, gate=gate)
        except BaseException as e:  # noqa: BLE001 - reported by the caller
            errors.append(e)
            try:
                gate.abort()
            except threading.BrokenBarrierError:
                pass

    threads = [threading.Thread(target=work, args=(t,)) for t in range(n)]
    for t in threads:
        t.start()
    try:
        gate.wait()  # everybody has warmed up: the timed loops start together
        t0 = _us()
        gate.wait()  # ... and have all ended
        total_us = _us() - t0
    except threading.BrokenBarrierError:
        total_us = 0.0
    for t in threads:
        t.join()
    if errors:
        raise errors[0]
    moved = sum(r["moved_bytes"] for r in results)
    bw = moved / 1e9 / (total_us / 1e6)
    iters = sum(r["iterations"] for r in results)
    lat = total_us / max(iters * results[0]["per_slot"], 1)
    ok = None if results[0]["consistent"] is None else all(r["consistent"] for r in results)

    def mean(key):
        return float(np.mean([r[key] for r in results]))

    out.write(f"{block:<20d}{batch:<15d}{bw:<15.6f}{lat:<15.1f}{mean('avg_prep_us'):<15.1f}{mean('p99_prep_us'):<15.1f}"
              f"{mean('avg_post_us'):<15.1f}{mean('p99_post_us'):<15.1f}{mean('avg_tx_us'):<15.1f}{mean('p99_tx_us'):<15.1f}"
              + ("" if ok is None else ("consistency: ok" if ok else "consistency: FAILED")) + "\n")
    out.flush()
    return {"block": block, "batch": batch, "gbps": bw, "avg_lat_us": lat, "avg_prep_us": mean("avg_prep_us"),
            "avg_post_us": mean("avg_post_us"), "avg_tx_us": mean("avg_tx_us"), "consistent": ok, "threads": n}


def run_point_one(agent, a, local, remote, block, batch, out, base=0, seed_salt=0, gate=None):
    """One thread's share of a point: its requests over [base, base + block * batch) of each buffer."""
    rng = np.random.default_rng(a.seed + block + batch + 7919 * seed_salt)
    slots_per_buf = batch
    l_off = np.uint64(base) + np.arange(slots_per_buf, dtype=np.uint64) * np.uint64(block)
    r_slots = rng.permutation(slots_per_buf) if a.randomize_location_mode == "blockaligned" else np.arange(slots_per_buf)
    r_off = np.uint64(base) + r_slots.astype(np.uint64) * np.uint64(block)
    depth = min(a.pipeline_depth, a.num_iter)
    if batch % depth:
        raise SystemExit(f"nixlbench: descriptor count ({batch}) is not divisible by pipeline depth ({depth})")
    per_slot = batch // depth

    def triples(base, offs, dev):
        return np.stack([np.uint64(base) + offs, np.full(offs.size, block, np.uint64), np.full(offs.size, dev, np.uint64)], 1)

    l_tr, r_tr = triples(local.addr, l_off, local.dev), triples(remote.addr, r_off, remote.dev)
    prep, post, tx = Stat(), Stat(), Stat()

    class Slot:
        pass

    slots = []
    for s in range(depth):
        sl = Slot()
        sl.l, sl.r = l_tr[s * per_slot:(s + 1) * per_slot], r_tr[s * per_slot:(s + 1) * per_slot]
        sl.req, sl.sides, sl.in_flight = None, (), False
        slots.append(sl)

    def prepare(sl, stats=True):
        t0 = _us()
        if a.prepared_xfer:
            lh = agent.prep_xfer_dlist("", sl.l, local.kind)
            rh = agent.prep_xfer_dlist(agent.name, sl.r, remote.kind)
            idx = np.arange(per_slot)
            sl.req = agent.make_prepped_xfer(a.op_type, lh, idx, rh, idx)
            sl.sides = (lh, rh)
        else:
            sl.req = agent.initialize_xfer(a.op_type, agent.get_xfer_descs(sl.l, local.kind),
                                           agent.get_xfer_descs(sl.r, remote.kind), agent.name)
        if stats:
            prep.add(_us() - t0)

    def recycle(sl):
        sl.req.release()
        for h in sl.sides:
            h.release()
        sl.req, sl.sides = None, ()

    def post_slot(sl, stats=True):
        t0 = _us()
        state = agent.transfer(sl.req)
        sl.post_ts = _us()
        if stats:
            post.add(sl.post_ts - t0)
        if state == "ERR":
            raise NixlError("postXferReq", 0, agent.last_status())
        sl.in_flight = state == "PROC"
        return state

    def loop(n_iter, stats):
        issued = completed = 0
        for sl in slots:
            if sl.req is None:
                prepare(sl, stats)
            if post_slot(sl, stats) == "DONE":
                completed += 1
                if stats:
                    tx.add(_us() - sl.post_ts)
            issued += 1
        while completed < n_iter:
            for sl in slots:
                if sl.in_flight:
                    state = agent.check_xfer_state(sl.req)
                    if state == "PROC":
                        continue
                    if state == "ERR":
                        raise NixlError("getXferStatus", 0, agent.last_status())
                    sl.in_flight = False
                    completed += 1
                    if stats:
                        tx.add(_us() - sl.post_ts)
                if issued >= n_iter or sl.in_flight:
                    continue
                if a.recreate_xfer:
                    recycle(sl)
                    prepare(sl, stats)
                if post_slot(sl, stats) == "DONE":
                    completed += 1
                    if stats:
                        tx.add(_us() - sl.post_ts)
                issued += 1
        for sl in slots:  # drain what the last round left in flight
            while sl.in_flight:
                sl.in_flight = agent.check_xfer_state(sl.req) == "PROC"

    n_iter = a.num_iter // a.large_blk_iter_ftr if block > LARGE_BLOCK_SIZE else a.num_iter
    n_iter = max(n_iter, depth)
    n_warm = a.warmup_iter // a.large_blk_iter_ftr if block > LARGE_BLOCK_SIZE else a.warmup_iter

    ok = None
    if a.check_consistency:
        nbytes = block * batch
        pattern = rng.integers(0, 256, nbytes, dtype=np.uint8)
        src, dst = (local, remote) if a.op_type == "WRITE" else (remote, local)
        s_off, d_off = (l_off, r_off) if a.op_type == "WRITE" else (r_off, l_off)
        image = np.zeros(nbytes, np.uint8)
        for i in range(batch):  # block i of the list sits at its own offset in each buffer
            at = int(s_off[i]) - base
            image[at:at + block] = pattern[i * block:(i + 1) * block]
        src.fill(image, base)
        dst.fill(np.zeros(nbytes, np.uint8), base)
    if n_warm:
        loop(max(n_warm, depth), False)
    if gate is not None:
        gate.wait()
    t0 = _us()
    loop(n_iter, True)
    total_us = _us() - t0
    if gate is not None:
        gate.wait()
    if a.check_consistency:
        got = dst.read(block * batch, base)
        ok = all(np.array_equal(got[int(d_off[i]) - base:int(d_off[i]) - base + block], pattern[i * block:(i + 1) * block])
                 for i in range(batch))
    for sl in slots:
        recycle(sl)
    # one iteration moves one slot's descriptors (per_slot blocks), as in the reference where
    # the list is split over the pipeline slots
    moved = block * per_slot * n_iter
    bw = moved / 1e9 / (total_us / 1e6)
    lat = total_us / (n_iter * per_slot)
    out.write(f"{block:<20d}{batch:<15d}{bw:<15.6f}{lat:<15.1f}{prep.avg():<15.1f}{prep.p99():<15.1f}"
              f"{post.avg():<15.1f}{post.p99():<15.1f}{tx.avg():<15.1f}{tx.p99():<15.1f}"
              + ("" if ok is None else ("consistency: ok" if ok else "consistency: FAILED")) + "\n")
    out.flush()
    return {"block": block, "batch": batch, "gbps": bw, "avg_lat_us": lat, "avg_prep_us": prep.avg(), "p99_prep_us": prep.p99(),
            "avg_post_us": post.avg(), "p99_post_us": post.p99(), "avg_tx_us": tx.avg(), "p99_tx_us": tx.p99(),
            "consistent": ok, "moved_bytes": moved, "iterations": n_iter, "per_slot": per_slot}


def main(argv=None, out=sys.stdout):
    a = parse(argv)
    if a.backend == "HIP" or "VRAM" in (a.initiator_seg_type, a.target_seg_type):
        # torch carries its own HIP runtime: it has to be the first one this process loads,
        # before the backend plugin brings in the system's
        import torch
        torch.cuda.is_available()
    agent = nixl_agent("initiator", nixl_agent_config(backends=()), plugin_dirs=[a.plugin_dir] if a.plugin_dir else ())
    params = dict(kv.split("=", 1) for kv in a.backend_params.split(",") if kv)
    agent.create_backend(a.backend, params)
    half = a.max_block_size * a.max_batch_size * a.num_threads
    pinned = a.backend == "HIP"
    local = Segment(a.initiator_seg_type, half, a.device_id, pinned)
    remote = Segment(a.target_seg_type, half, a.device_id, pinned)
    regs = [agent.register_memory(np.array([[s.addr, s.nbytes, s.dev]], dtype=np.uint64), s.kind) for s in (local, remote)]
    out.write(f"nixlbench (single instance): backend {a.backend}, {a.initiator_seg_type} -> {a.target_seg_type}, "
              f"{a.op_type}, {'prepared' if a.prepared_xfer else 'create'} transfers, pipeline depth {a.pipeline_depth}, "
              f"{a.num_threads} thread{'s' if a.num_threads > 1 else ''}\n")
    out.write(f"{'Block Size (B)':<20}{'Batch Size':<15}{'B/W (GB/Sec)':<15}{'Avg Lat. (us)':<15}{'Avg Prep (us)':<15}"
              f"{'P99 Prep (us)':<15}{'Avg Post (us)':<15}{'P99 Post (us)':<15}{'Avg Tx (us)':<15}{'P99 Tx (us)':<15}\n")
    out.write("-" * 155 + "\n")
    results, failed = [], False
    block = a.start_block_size
    while block <= a.max_block_size:
        batch = a.start_batch_size
        while batch <= a.max_batch_size:
            r = run_point(agent, a, local, remote, block, batch, out)
            failed |= r["consistent"] is False
            results.append(r)
            batch *= 2
        block *= 2
    for r in regs:
        agent.deregister_memory(r)
    agent.close()
    if failed:
        out.write("consistency check FAILED\n")
        return 1, results
    return 0, results


if __name__ == "__main__":
    sys.exit(main()[0])
