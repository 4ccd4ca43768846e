#!/usr/bin/env python3
"""Writes the golden vectors in this directory.

The reference keeps no stored vectors for this path (its tests compute their expectations
at run time), so these come from library routines (torch CPU: bfloat16 / float8_e4m3fn
conversions, topk, softmax) and from plain Python loops that state the result contracts
directly:
  * low-latency dispatch: examples/device/ep/csrc/kernels/nixl_ep_ll.cu:134-182 (cast),
    :296-393 (packing), checked by the reference test examples/device/ep/tests/elastic/
    elastic.py:263-318;
  * low-latency combine: nixl_ep_ll.cu:875-1016;
  * normal mode: kernels/layout.cu:31-138, kernels/nixl_ep_ht.cu:295-314,1109-1243,1682-1737,
    checked by examples/device/ep/tests/test_ht.py:99-172,223-244,304-323;
  * descriptor copy: one memcpy per descriptor (src/plugins/ucx/ucx_backend.cpp:1216-1262).
Nothing here imports the oracle, the product or the reference.  Run:
    python tests/golden/make_fixtures.py
"""
import os
from fractions import Fraction

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def bf16_bits(t):
    return t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).copy()


def fma32(a, b, c):
    """fp32 fused multiply-add of arrays through fp64: the product of two fp32 values is
    exact in fp64; the sum is rounded to fp64 and then to fp32.  Returns None when one of
    the elements could be rounded differently by the two steps than by one (see `hazard`)."""
    a64, b64, c64 = np.float64(a) + np.zeros_like(c, np.float64), np.float64(b), np.float64(c)
    s = a64 * b64 + c64
    low = s.view(np.uint64) & np.uint64((1 << 29) - 1)
    for i in np.nonzero(low == np.uint64(1 << 28))[0]:
        if hazard(float(a64[i]), float(b64), float(c64[i]), float(s[i])):
            return None
    return s.astype(np.float32)


def hazard(a, b, c, s):
    """The fp64 sum s sits exactly on an fp32 rounding tie.  That is harmless when s is the
    exact value of a * b + c (the tie is then real); it is a double-rounding hazard when
    s was itself rounded."""
    return Fraction(a) * Fraction(b) + Fraction(c) != Fraction(s)


def e4m3_vectors():
    g = torch.Generator().manual_seed(11)
    vals = torch.cat([
        torch.randn(4096, generator=g) * 100,
        torch.randn(2048, generator=g),
        torch.randn(1024, generator=g) * 0.01,
        torch.tensor([0.0, -0.0, 448.0, -448.0, 449.0, 463.9, 464.0, 2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -10,
                      2.0 ** -6, 0.9999 * 2.0 ** -6, 17.0, 18.0, 19.0, 20.0, 22.0, 26.0, 240.0, 232.0, 248.0]),
    ]).float()
    vals = vals[vals.abs() <= 464.0]  # beyond 464 torch returns NaN where the kernels saturate
    codes = vals.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    # saturating edge by the format's definition: everything above 464 in magnitude -> +-448
    sat_in = np.array([465.0, 480.0, 1000.0, 3.0e38, np.inf, -465.0, -np.inf], np.float32)
    sat_out = np.array([0x7E, 0x7E, 0x7E, 0x7E, 0x7E, 0xFE, 0xFE], np.uint8)
    np.savez_compressed(os.path.join(HERE, "e4m3_encode.npz"), values=vals.numpy(), codes=codes, sat_values=sat_in,
             sat_codes=sat_out)


def router_vectors():
    g = torch.Generator().manual_seed(12)
    logits = torch.randn(64, 256, generator=g)
    logits[3, 10] = logits[3, 200] = logits[3].max() + 1  # a tie: the lower index must win
    v, i = torch.sort(logits, dim=1, descending=True, stable=True)
    idx = i[:, :8].to(torch.int32)
    w = torch.softmax(v[:, :8], dim=1)
    np.savez_compressed(os.path.join(HERE, "router.npz"), logits=logits.numpy(), topk_idx=idx.numpy(), topk_weights=w.numpy())


def cast_row(row):
    """row: fp32 tensor [H] holding bf16 values -> (codes uint8 [H], scale_inv fp32 [H/128])."""
    g = row.view(-1, 128)
    amax = torch.clamp(g.abs().amax(1), min=1e-4)
    scale = torch.div(torch.tensor(448.0), amax)
    inv = amax * torch.tensor(np.float32(1.0) / np.float32(448.0))
    q = (g * scale[:, None]).to(torch.float8_e4m3fn).view(torch.uint8).reshape(-1)
    return q.numpy(), inv.numpy()


def ll_world(seed=21, repeats=(), name="ll_world.npz"):
    """repeats: (rank, token, from k, to k) entries that make a token name one expert more than
    once; the reference gives such a token a row per selection (kernels/nixl_ep_ll.cu:186-190),
    next to each other here (tokens ascending, a token's selections together)."""
    R, T, H, K, E, M = 4, 5, 512, 3, 8, 6
    El, N = E // R, R * M
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    xf = torch.randn(R, T, H, generator=g).to(torch.bfloat16)
    xf[1, 0, :128] = 0  # an all-zero group: amax floor
    x = xf.float()
    topk = np.stack([np.stack([rng.permutation(E)[:K] for _ in range(T)]) for _ in range(R)]).astype(np.int32)
    topk[0, 1, 2] = -1
    topk[2, 4, 0] = -1
    for r_, t_, k_from, k_to in repeats:
        topk[r_, t_, k_to] = topk[r_, t_, k_from]
    num_tokens = np.array([5, 3, 5, 4], np.int32)
    w = rng.random((R, T, K)).astype(np.float32)

    recv_fp8 = np.zeros((R, El, N, H), np.uint8)
    recv_bf16 = np.zeros((R, El, N, H), np.uint16)
    scales = np.zeros((R, El, H // 128, N), np.float32)
    src_info = np.zeros((R, El, N), np.int32)
    layout_range = np.zeros((R, El, R), np.int64)
    recv_count = np.zeros((R, El), np.int32)
    row_of = -np.ones((R, T, K), np.int64)
    for d in range(R):
        for le in range(El):
            e = d * El + le
            n = 0
            for s in range(R):
                begin = n
                for t in range(int(num_tokens[s])):
                    ks = [k for k in range(K) if topk[s, t, k] == e]
                    if not ks:
                        continue
                    q, inv = cast_row(x[s, t])
                    for k in ks:  # a row per selection
                        recv_fp8[d, le, n] = q
                        recv_bf16[d, le, n] = bf16_bits(xf[s, t])
                        scales[d, le, :, n] = inv
                        src_info[d, le, n] = t
                        row_of[s, t, k] = (d * El + le) * N + n
                        n += 1
                layout_range[d, le, s] = (n - begin) | (begin << 32)
            recv_count[d, le] = n

    # expert outputs: random bf16 rows where valid; combine = fma chain in top-k order
    y = torch.randn(R, El, N, H, generator=g).to(torch.bfloat16)
    # an expert gives the rows of one token the same output (same input, same function)
    flat = y.view(R * El * N, H)
    for r_, t_, k_from, k_to in repeats:
        ks = [k for k in range(K) if topk[r_, t_, k] == topk[r_, t_, k_from]]
        for k in ks[1:]:
            flat[row_of[r_, t_, k]] = flat[row_of[r_, t_, ks[0]]]
    yb = bf16_bits(y).reshape(R * El * N, H)
    yf = y.float().numpy().reshape(R * El * N, H)
    combined = np.zeros((R, T, H), np.uint16)
    for r in range(R):
        for t in range(int(num_tokens[r])):
            acc = np.zeros(H, np.float32)
            for k in range(K):
                if topk[r, t, k] < 0:
                    continue
                row = yf[row_of[r, t, k]]
                acc = fma32(row, w[r, t, k], acc)
                if acc is None:
                    return None
            combined[r, t] = bf16_bits(torch.from_numpy(acc))
    valid = np.arange(N)[None, None, :] < recv_count[:, :, None]
    yb = np.where(valid.reshape(-1)[:, None], yb, 0).reshape(R, El, N, H).astype(np.uint16)
    np.savez_compressed(os.path.join(HERE, name), x=bf16_bits(xf), topk_idx=topk, topk_weights=w,
             num_tokens=num_tokens, num_experts=E, max_tok=M, recv_fp8=recv_fp8, recv_bf16=recv_bf16, scales=scales,
             src_info=src_info, layout_range=layout_range, recv_count=recv_count, expert_out=yb, combined=combined)
    return True


def ht_world():
    R, T, H, K, E, C = 3, 7, 128, 3, 6, 2
    El = E // R
    rng = np.random.default_rng(31)
    g = torch.Generator().manual_seed(31)
    xf = torch.randn(R, T, H, generator=g).to(torch.bfloat16)
    topk = np.stack([np.stack([rng.permutation(E)[:K] for _ in range(T)]) for _ in range(R)]).astype(np.int32)
    topk[1, 2, 1] = -1
    topk[0, 3, :] = [0, 1, -1]  # two selections on one rank: the token travels there once
    w = rng.random((R, T, K)).astype(np.float32)

    per_rank = np.zeros((R, R), np.int32)
    per_expert = np.zeros((R, E), np.int32)
    in_rank = np.zeros((R, T, R), np.uint8)
    for s in range(R):
        for t in range(T):
            for k in range(K):
                e = topk[s, t, k]
                if e >= 0:
                    per_expert[s, e] += 1
                    in_rank[s, t, e // El] = 1
        per_rank[s] = in_rank[s].sum(0)
    prefix = np.cumsum(per_rank.T, axis=1).astype(np.int32)  # [dst][src] inclusive
    expert_count = per_expert.sum(0).reshape(R, El).astype(np.int32)
    per_ch = -(-T // C)
    ch_prefix = np.zeros((R, R, C), np.int32)
    for s in range(R):
        for d in range(R):
            run = 0
            for c in range(C):
                run += int(in_rank[s, c * per_ch:min(T, (c + 1) * per_ch), d].sum())
                ch_prefix[s, d, c] = run
    total = int(prefix[:, -1].sum())
    offs = np.concatenate([[0], np.cumsum(prefix[:, -1])]).astype(np.int64)
    recv_x = np.zeros((total, H), np.uint16)
    recv_idx = np.zeros((total, K), np.int32)
    recv_w = np.zeros((total, K), np.float32)
    recv_meta = np.zeros((total, 2), np.int32)
    send_head = -np.ones((R, T, R), np.int32)
    xb = bf16_bits(xf)
    for d in range(R):
        row = int(offs[d])
        for s in range(R):
            pos = 0
            for t in range(T):
                if not in_rank[s, t, d]:
                    continue
                recv_x[row] = xb[s, t]
                for k in range(K):
                    e = topk[s, t, k]
                    local = e >= 0 and e // El == d
                    recv_idx[row, k] = e - d * El if local else -1
                    recv_w[row, k] = w[s, t, k] if local else 0.0
                recv_meta[row] = (s, t)
                send_head[s, t, d] = pos
                pos += 1
                row += 1
    # combine of y = recv_x (identity experts) with two biases
    b0 = torch.randn(R, T, H, generator=g).to(torch.bfloat16)
    b1 = torch.randn(R, T, H, generator=g).to(torch.bfloat16)
    combined = np.zeros((R, T, H), np.uint16)
    comb_w = np.zeros((R, T, K), np.float32)
    for s in range(R):
        for t in range(T):
            acc = b0[s, t].float().numpy() + b1[s, t].float().numpy()
            for d in range(R):
                if in_rank[s, t, d]:
                    row = int(offs[d]) + (int(prefix[d, s - 1]) if s else 0) + int(send_head[s, t, d])
                    acc = acc + xf[s, t].float().numpy()
                    comb_w[s, t] += recv_w[row]
            combined[s, t] = bf16_bits(torch.from_numpy(acc.astype(np.float32)))
    np.savez_compressed(os.path.join(HERE, "ht_world.npz"), x=xb, topk_idx=topk, topk_weights=w, num_experts=E,
             num_channels=C, per_rank=per_rank, per_expert=per_expert, in_rank=in_rank, prefix=prefix,
             expert_count=expert_count, channel_prefix=ch_prefix, row_offset=offs, recv_x=recv_x,
             recv_topk_idx=recv_idx, recv_topk_weights=recv_w, recv_src_meta=recv_meta, send_head=send_head,
             bias0=bf16_bits(b0), bias1=bf16_bits(b1), combined=combined, combined_topk_weights=comb_w)


def kv_vectors():
    rng = np.random.default_rng(41)
    size = 1 << 16
    src = rng.integers(0, 256, size, dtype=np.uint8)
    lens = np.array([16, 48, 1, 0, 255, 4096, 33, 1024, 7, 512], np.uint64)
    src_off = np.array([0, 32, 101, 0, 4097, 8192, 13001, 16384, 20003, 24000], np.uint64)
    dst_off = np.array([64, 128, 203, 0, 1001, 8192, 30003, 40000, 50001, 60000], np.uint64)
    dst = np.full(size, 0xA5, np.uint8)
    for s, d, n in zip(src_off, dst_off, lens):
        dst[int(d):int(d + n)] = src[int(s):int(s + n)]
    np.savez_compressed(os.path.join(HERE, "kv_descs.npz"), src=src, src_off=src_off, dst_off=dst_off, lens=lens, dst=dst,
             canary=np.uint8(0xA5))


if __name__ == "__main__":
    e4m3_vectors()
    router_vectors()
    seed = 21
    while ll_world(seed) is None:  # move to another seed if an fp64 sum sits on an fp32 tie
        seed += 1
    seed = 31
    while ll_world(seed, repeats=[(0, 2, 0, 1), (2, 1, 2, 0), (3, 0, 0, 1), (3, 0, 0, 2)], name="ll_world_repeats.npz") is None:
        seed += 1
    ht_world()
    kv_vectors()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)))
