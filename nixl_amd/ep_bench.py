"""Timing of the expert-parallel kernels on the BASELINE shapes, used by bench.py.

Method follows the reference's EP benchmark helper (examples/device/ep/tests/utils.py:
116-143): device events around each call, a cache-flushing write of 512 MB before every
timed call (the reference flushes 256 MB for a 50 MB L2; MI355X has a 256 MB last-level
cache), warm-ups first, first sample dropped, average / min / max reported.  Byte counts
are the algorithmic ones: each input row read once, each output row written once
(reference formula for the low-latency mode: tests/elastic/elastic.py:424-432).
"""
import numpy as np
import torch

from .ep import Buffer

HBM_PEAK_GBPS = 8000.0

# HBM bytes per call from hardware counters cannot be read from inside the process: bench.py
# runs run_traffic_child below under the profiler and adds, per call, the medians of the
# kernels named here.
CALL_KERNELS = {
    "ll_dispatch": ("ll_bits_kernel<false", "ll_dispatch_kernel<true>", "ll_scales_kernel"),
    "ll_combine": ("ll_combine_kernel<false>",),
    "ht_dispatch": ("ht_scan_packed_kernel", "ht_prefix_kernel", "ht_dispatch_kernel", "ht_meta_kernel"),
    "ht_combine": ("ht_combine_kernel",),
}


def _timed(fn, flush, warmup, iters):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(iters + 1):
        flush.fill_(1)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1) * 1e3)
    times = np.array(times[1:])
    return {"avg_us": round(float(times.mean()), 2), "min_us": round(float(times.min()), 2),
            "max_us": round(float(times.max()), 2)}


def _rate(nbytes, us):
    gbps = nbytes / (us * 1e-6) / 1e9
    return {"bytes": int(nbytes), "GBps": round(gbps, 1), "frac_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4)}


def run_low_latency(dev, warmup=20, iters=50):
    """BASELINE config 4: 32 virtual ranks x 128 tokens x 7168, 256 experts, top-8, fp8."""
    R, T, H, K, E, M = 32, 128, 7168, 8, 256, 128
    El, N = E // R, R * M
    g = torch.Generator(device=dev).manual_seed(4)
    x = torch.randn((R, T, H), generator=g, device=dev).to(torch.bfloat16)
    logits = torch.randn((R, T, E), generator=g, device=dev)
    flush = torch.empty(512 << 20, dtype=torch.uint8, device=dev)
    buf = Buffer(R, device=dev)
    topk, w = buf.route(logits, K)
    state = {}

    def dispatch():
        state["out"] = buf.dispatch(x, topk, M, E, use_fp8=True)

    t_empty = _timed(lambda: None, flush, warmup, iters)  # what an event pair behind the flush shows with nothing in it
    t_router = _timed(lambda: buf.route(logits, K), flush, warmup, iters)
    t_dispatch = _timed(dispatch, flush, warmup, iters)
    (q, sc_t), cnt, handle, _, _ = state["out"]
    # expert step (not timed): dequantise, scale by (1 + 0.001 e), back to bf16
    sc = sc_t.contiguous()
    y = torch.zeros((R, El, N, H), dtype=torch.bfloat16, device=dev)
    valid = torch.arange(N, device=dev).view(1, 1, -1) < cnt.unsqueeze(-1)
    for d in range(R):
        deq = (q[d].float().view(El, N, H // 128, 128) * sc[d].unsqueeze(-1)).view(El, N, H)
        f = (1 + 0.001 * (d * El + torch.arange(El, device=dev, dtype=torch.float32))).view(El, 1, 1)
        y[d] = torch.where(valid[d].unsqueeze(-1), (deq.to(torch.bfloat16).float() * f).to(torch.bfloat16), y[d])
    del deq, sc
    t_combine = _timed(lambda: buf.combine(y, topk, w, handle), flush, warmup, iters)

    t_logfmt = _timed(lambda: buf.combine(y, topk, w, handle, use_logfmt=True), flush, warmup, iters)

    def both():  # one event pair around the two calls, as a layer would issue them
        dispatch()
        buf.combine(y, topk, w, handle)

    t_both = _timed(both, flush, warmup, iters)

    def route_dispatch():  # logits in: routing done by the kernel that prepares the dispatch
        state["routed"] = buf.route_dispatch(x, logits, K, M, use_fp8=True)

    t_route_dispatch = _timed(route_dispatch, flush, warmup, iters)

    def routed():  # logits -> top-k -> dispatch -> combine under one event pair
        route_dispatch()
        idx, wts, _, _, handle_r, _, _ = state["routed"]
        buf.combine(y, idx, wts, handle_r)

    t_routed = _timed(routed, flush, warmup, iters)

    tokens, pairs = R * T, int((topk >= 0).sum())
    meta = R * El * R * 8 + R * El * 4
    dispatch_bytes = tokens * H * 2 + tokens * K * 4 + pairs * (H + H // 128 * 4 + 4) + meta
    combine_bytes = pairs * H * 2 + tokens * K * 8 + tokens * H * 2
    both_us = t_dispatch["avg_us"] + t_combine["avg_us"]
    return {
        "workload": f"{R} virtual ranks x {T} tokens x hidden {H}, {E} experts, top-{K}, fp8 e4m3 dispatch, bf16 combine",
        "dispatch": {**t_dispatch, **_rate(dispatch_bytes, t_dispatch["avg_us"])},
        "combine": {**t_combine, **_rate(combine_bytes, t_combine["avg_us"])},
        "dispatch_plus_combine_us": round(both_us, 2),
        "dispatch_plus_combine": _rate(dispatch_bytes + combine_bytes, both_us),
        "dispatch_then_combine_one_event_pair": {**t_both, **_rate(dispatch_bytes + combine_bytes, t_both["avg_us"])},
        "route_dispatch": {**t_route_dispatch, **_rate(dispatch_bytes + tokens * E * 4, t_route_dispatch["avg_us"]),
                           "note": "dispatch from logits (top-k + softmax inside); adds 4.2 MB of logits and the written selection"},
        "route_dispatch_combine_one_event_pair": {
            **t_routed, **_rate(dispatch_bytes + combine_bytes + tokens * E * 4, t_routed["avg_us"]),
            "note": "router (logits -> top-k + softmax) included; its logits add 4.2 MB"},
        "combine_logfmt": {**t_logfmt, "note": "rows passed through the LogFMT-10 codec before accumulation"},
        "router": {**t_router, "bytes": tokens * E * 4},
        "empty_event_pair": {**t_empty, "note": "the same timing with no call between the two events: what every figure above "
                                                "contains besides its kernels; not subtracted anywhere"},
    }


def zipf_topk(rng, R, T, K, E, s=1.2):
    """K distinct experts per token from a Zipf(s) law over a seeded expert permutation
    (Gumbel top-k), softmax weights over the drawn scores."""
    perm = rng.permutation(E)
    p = 1.0 / np.arange(1, E + 1) ** s
    logp = np.log(p / p.sum())[np.argsort(perm)]
    keys = logp[None, None, :] + rng.gumbel(size=(R, T, E))
    topk = np.argsort(-keys, axis=2)[:, :, :K].astype(np.int32)
    sel = np.take_along_axis(keys, topk, 2)
    w = np.exp(sel - sel.max(2, keepdims=True))
    return topk, (w / w.sum(2, keepdims=True)).astype(np.float32)


def run_normal(dev, warmup=5, iters=20):
    """BASELINE config 5: 8 virtual ranks x 4096 tokens x 7168, 256 experts, top-8, Zipf."""
    R, T, H, K, E, C = 8, 4096, 7168, 8, 256, 10
    rng = np.random.default_rng(5)
    topk_h, w_h = zipf_topk(rng, R, T, K, E)
    g = torch.Generator(device=dev).manual_seed(5)
    x = torch.randn((R, T, H), generator=g, device=dev).to(torch.bfloat16)
    topk, w = torch.from_numpy(topk_h).to(dev), torch.from_numpy(w_h).to(dev)
    flush = torch.empty(512 << 20, dtype=torch.uint8, device=dev)
    buf = Buffer(R, low_latency_mode=False, device=dev)
    state = {}

    def layout():
        state["layout"] = buf.get_dispatch_layout(topk, E)

    def dispatch():
        per_rank, _, per_expert, in_rank, _ = state["layout"]
        state["out"] = buf.ht_dispatch(x, num_tokens_per_rank=per_rank, is_token_in_rank=in_rank,
                                       num_tokens_per_expert=per_expert, topk_idx=topk, topk_weights=w, num_channels=C)

    t_layout = _timed(layout, flush, warmup, iters)
    t_dispatch = _timed(dispatch, flush, warmup, iters)
    recv_x, recv_idx, recv_w, per_expert_list, handle, _ = state["out"]
    rows = recv_x.shape[0]
    t_cached = _timed(lambda: buf.ht_dispatch(x, handle=handle), flush, warmup, iters)
    coef = (recv_w * (recv_idx >= 0)).sum(1, keepdim=True)
    y = (recv_x.float() * coef).to(torch.bfloat16)
    t_combine = _timed(lambda: buf.ht_combine(y, handle, topk_weights=recv_w), flush, warmup, iters)
    # fp8 rows with their per-128-channel scales, the (x, x_scales) form; scales stored
    # transposed as the reference's test passes them (tests/test_ht.py:78-79)
    S = H // 128
    x8 = torch.randint(0, 256, (R, T, H), dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    sc = torch.rand((R, T, S), device=dev).transpose(1, 2).contiguous().transpose(1, 2)

    def dispatch_fp8():
        per_rank, _, per_expert, in_rank, _ = state["layout"]
        buf.ht_dispatch((x8, sc), num_tokens_per_rank=per_rank, is_token_in_rank=in_rank,
                        num_tokens_per_expert=per_expert, topk_idx=topk, topk_weights=w, num_channels=C)

    t_fp8 = _timed(dispatch_fp8, flush, warmup, iters)
    tokens = R * T
    fp8_bytes = (tokens + rows) * (H + S * 4) + tokens * K * 8 + rows * (K * 8 + 8) + tokens * K * 4 + tokens * R
    dispatch_bytes = tokens * H * 2 + rows * H * 2 + tokens * K * 8 + rows * (K * 8 + 8) + tokens * K * 4 + tokens * R
    combine_bytes = rows * H * 2 + rows * K * 4 + tokens * H * 2 + tokens * K * 4
    counts = np.array(per_expert_list).reshape(-1)
    return {
        "workload": f"{R} virtual ranks x {T} tokens x hidden {H}, {E} experts, top-{K}, Zipf(1.2) expert popularity, bf16",
        "rows_received": int(rows),
        "expert_load": {"max": int(counts.max()), "mean": round(float(counts.mean()), 1), "min": int(counts.min())},
        "layout": t_layout,
        "dispatch": {**t_dispatch, **_rate(dispatch_bytes, t_dispatch["avg_us"]),
                     "note": "count exchange + rows + per-row metadata; receive tensors sized for the worst case, so the "
                             "host's wait for the counts (pinned memory) overlaps the row kernel"},
        "dispatch_cached_handle": {**t_cached, **_rate(tokens * H * 2 + rows * H * 2, t_cached["avg_us"]),
                                   "note": "layout of an earlier dispatch reused: rows only, no count exchange"},
        "combine": {**t_combine, **_rate(combine_bytes, t_combine["avg_us"])},
        "dispatch_fp8_rows_with_scales": {**t_fp8, **_rate(fp8_bytes, t_fp8["avg_us"]),
                                          "note": "rows of 7168 fp8 bytes plus 56 fp32 scales per token"},
    }


def run_traffic_child(repeats=3, normal_mode=True):
    """The four timed calls of both configurations a few times over, nothing else: what bench.py
    runs under `rocprofv3 --pmc` to count each call's HBM bytes.  Only the forms named in
    CALL_KERNELS run (indices not logits, bf16 rows in normal mode, no LogFMT), so that every
    kernel name stands for one shape."""
    dev = torch.device("cuda:0")
    R, T, H, K, E, M = 32, 128, 7168, 8, 256, 128
    g = torch.Generator(device=dev).manual_seed(4)
    x = torch.randn((R, T, H), generator=g, device=dev).to(torch.bfloat16)
    logits = torch.randn((R, T, E), generator=g, device=dev)
    buf = Buffer(R, device=dev)
    topk, w = buf.route(logits, K)
    y = torch.zeros((R, E // R, R * M, H), dtype=torch.bfloat16, device=dev)
    for _ in range(repeats):
        _, _, handle, _, _ = buf.dispatch(x, topk, M, E, use_fp8=True)
        buf.combine(y, topk, w, handle)
    torch.cuda.synchronize()
    del x, y, buf
    if not normal_mode:
        return
    R, T, C = 8, 4096, 10
    rng = np.random.default_rng(5)
    topk_h, w_h = zipf_topk(rng, R, T, K, E)
    g = torch.Generator(device=dev).manual_seed(5)
    x = torch.randn((R, T, H), generator=g, device=dev).to(torch.bfloat16)
    topk, w = torch.from_numpy(topk_h).to(dev), torch.from_numpy(w_h).to(dev)
    buf = Buffer(R, low_latency_mode=False, device=dev)
    for _ in range(repeats):
        per_rank, _, per_expert, in_rank, _ = buf.get_dispatch_layout(topk, E)
        recv_x, recv_idx, recv_w, _, handle, _ = buf.ht_dispatch(x, num_tokens_per_rank=per_rank, is_token_in_rank=in_rank,
                                                                 num_tokens_per_expert=per_expert, topk_idx=topk, topk_weights=w,
                                                                 num_channels=C)
        buf.ht_combine(recv_x, handle, topk_weights=recv_w)
    torch.cuda.synchronize()


def run(args):
    dev = torch.device("cuda:0")
    warmup, iters = getattr(args, "ep_warmup", 20), getattr(args, "ep_iters", 50)
    out = {"low_latency": run_low_latency(dev, warmup, iters),
           "normal": run_normal(dev, max(warmup // 4, 1), max(iters // 2, 1))}
    return out
