"""TEST INFRASTRUCTURE — CPU oracle for the descriptor-transfer half.

Plain numpy / Python-loop restatement of what the reference computes on this path.  Only
tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import
this module; nothing under ``nixl_amd/`` does.

Functions and the reference code each one follows:
  copy_descs        per-descriptor put/get loop, src/plugins/ucx/ucx_backend.cpp:1216-1244
                    (direction :1227-1229).  Closed form: memcpy per descriptor.
  covering_index    nixlSecDescList::getCoveringIndex, src/infra/nixl_descriptors.cpp:490-503
  stride_runs       nixlMemSection::populate (stride form), src/infra/nixl_memory_section.cpp:106-184
  expand_and_merge  index expansion + merge loop of nixlAgent::makeXferReq,
                    src/core/nixl_agent.cpp:799-857; run lookup src/api/cpp/backend/backend_aux.h:184-205

Pins (tests/test_kv_oracle.py): the merge counts the reference states for its own example
(test/nixl/agent_example.cpp:142-152: 32 regions x 65536 contiguous 8-byte descriptors, all
indices in order -> 32 descriptors; every other index -> n/2, nothing merges), brute force
against an unmerged expansion on random small inputs, and the canary/direction invariants
of copy_descs.
"""
import bisect

import numpy as np


def copy_descs(mem, src_off, dst_off, lens):
    """memcpy(mem[dst:dst+len], mem[src:src+len]) for each descriptor, in list order.

    ``mem`` is one uint8 array holding every region; offsets index into it.  For a
    NIXL_WRITE pass local offsets as src and remote offsets as dst; for NIXL_READ swap them.
    """
    for s, d, n in zip(src_off, dst_off, lens):
        s, d, n = int(s), int(d), int(n)
        if n:
            mem[d:d + n] = mem[s:s + n].copy()
    return mem


def _key(desc):
    addr, length, dev = desc
    return (dev, addr, length)


def _covers(region, q):
    ra, rl, rd = region
    qa, ql, qd = q
    return rd == qd and ra <= qa and ra + rl >= qa + ql


def covering_index(regions_sorted, q):
    """Index of a registered region covering q, or -1.  ``regions_sorted`` is a list of
    (addr, len, dev) sorted by (dev, addr, len)."""
    keys = [_key(r) for r in regions_sorted]
    i = bisect.bisect_left(keys, _key(q))
    if i < len(regions_sorted) and _covers(regions_sorted[i], q):
        return i
    if i > 0 and _covers(regions_sorted[i - 1], q):
        return i - 1
    return -1


def stride_runs(descs, regions):
    """Compress a descriptor list into stride runs.

    descs: sequence of (addr, len, dev).  regions: registered (addr, len, dev) triples.
    Returns a list of dicts {addr, len, dev, region, stride, count, start_idx}, or None if
    some descriptor is not covered by a registration.
    """
    regions_sorted = sorted(regions, key=_key)
    n_base = len(regions_sorted)
    at = covering_index(regions_sorted, descs[0])
    if at < 0:
        return None
    a0, l0, d0 = descs[0]
    run = dict(addr=a0, len=l0, dev=d0, region=at, stride=l0, count=1, start_idx=0)
    runs = []
    prev = a0
    for i in range(1, len(descs)):
        q = descs[i]
        if not _covers(regions_sorted[at], q):
            if _key(q) < _key(descs[i - 1]):
                at = covering_index(regions_sorted, q)
            else:
                while at < n_base and not _covers(regions_sorted[at], q):
                    at += 1
                if at == n_base:
                    at = -1
            if at < 0:
                return None
        qa, ql, qd = q
        extends = ql == run["len"] and qd == run["dev"] and at == run["region"]
        if extends:
            if run["count"] == 1:
                extends = qa > prev
                if extends:
                    run["stride"] = qa - prev
            else:
                extends = (qa - prev) == run["stride"]
        if extends:
            run["count"] += 1
        else:
            runs.append(run)
            run = dict(addr=qa, len=ql, dev=qd, region=at, stride=ql, count=1, start_idx=i)
        prev = qa
    runs.append(run)
    return runs


def _find_run(runs, flat_idx):
    starts = [r["start_idx"] for r in runs]
    return runs[bisect.bisect_right(starts, flat_idx) - 1]


def expand_and_merge(local_runs, remote_runs, local_idx, remote_idx, skip_merge=False):
    """Descriptors a backend receives for a prepared-list request.

    Returns a list of (local_addr, remote_addr, len).  Raises ValueError where the
    reference returns NIXL_ERR_INVALID_PARAM (index out of range, length mismatch).
    """
    count = len(local_idx)
    if count == 0 or count != len(remote_idx):
        raise ValueError("index count")
    lflat = local_runs[-1]["start_idx"] + local_runs[-1]["count"]
    rflat = remote_runs[-1]["start_idx"] + remote_runs[-1]["count"]
    out = []
    i = 0
    while i < count:
        li, ri = int(local_idx[i]), int(remote_idx[i])
        if not (0 <= li < lflat) or not (0 <= ri < rflat):
            raise ValueError("index out of range")
        lr, rr = _find_run(local_runs, li), _find_run(remote_runs, ri)
        if lr["len"] != rr["len"]:
            raise ValueError("length mismatch")
        step = 1
        if not skip_merge and lr["stride"] == lr["len"] and lr["stride"] == rr["stride"]:
            room = min(lr["start_idx"] + lr["count"] - li, rr["start_idx"] + rr["count"] - ri, count - i)
            while step < room and int(local_idx[i + step]) == li + step and int(remote_idx[i + step]) == ri + step:
                step += 1
        out.append((lr["addr"] + (li - lr["start_idx"]) * lr["stride"],
                    rr["addr"] + (ri - rr["start_idx"]) * rr["stride"],
                    lr["len"] * step))
        i += step
    return out


def kv_block_descs(base, n_layers, n_blocks_pool, block_bytes, block_ids):
    """Addresses of the per-layer K and V sub-blocks of the given block ids in a pool laid
    out as [layer][K|V][block][block_bytes] (one descriptor per (block, layer, K|V), block
    id outermost).  Shape source: Llama-3.1-8B, 32 layers x 8 KV heads x 128
    (benchmark/kvbench/examples/model_llama_3_1_8b.yaml:16-21)."""
    block_ids = np.asarray(block_ids, dtype=np.uint64)
    lk = np.arange(n_layers * 2, dtype=np.uint64)
    addr = (np.uint64(base) + lk[None, :] * np.uint64(n_blocks_pool * block_bytes)
            + block_ids[:, None] * np.uint64(block_bytes))
    return addr.reshape(-1)
