"""CPU tests that pin the expert-parallel oracle (oracle/ep_oracle.c) before anything is
checked against it: library routines (torch CPU), the OCP FP8 specification, closed forms,
brute force on tiny shapes, and the invariants the reference's own tests assert."""
import numpy as np
import pytest
import torch

from oracle import ep_oracle as eo


def calc_diff(x, y):
    # examples/device/ep/tests/utils.py:63-67
    x, y = x.astype(np.float64) + 1, y.astype(np.float64) + 1
    return float(1 - 2 * (x * y).sum() / (x * x + y * y).sum())


def bf16_bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


# ---- scalar formats -------------------------------------------------------------------------

def test_bf16_decode_exhaustive_against_torch():
    codes = np.arange(65536, dtype=np.uint16)
    want = torch.from_numpy(codes.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    got = eo.bf16_to_f32(codes)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    one = np.array([eo.lib().oracle_bf16_to_f32(int(c)) for c in (0, 0x3F80, 0xC000, 0x7F80)], np.float32)
    assert list(one) == [0.0, 1.0, -2.0, np.inf]


def test_bf16_encode_against_torch():
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 200000).astype(np.float32),
        rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32),
        # exact ties between two bf16 neighbours, both parities, and the carry into the exponent
        (np.arange(0, 65536, dtype=np.uint32) << 16 | 0x8000).view(np.float32),
        (np.arange(0, 65536, dtype=np.uint32) << 16 | 0x7FFF).view(np.float32),
        (np.arange(0, 65536, dtype=np.uint32) << 16 | 0x8001).view(np.float32),
    ])
    finite = np.isfinite(vals)
    want = bf16_bits(torch.from_numpy(vals).to(torch.bfloat16))
    got = eo.f32_to_bf16(vals)
    assert np.array_equal(got[finite], want[finite])
    assert np.array_equal(got[np.isinf(vals)], want[np.isinf(vals)])
    nan = np.isnan(vals)
    assert np.all((got[nan] & 0x7F80) == 0x7F80) and np.all((got[nan] & 0x7F) != 0)


def test_e4m3_decode_by_specification():
    # OCP 8-bit floating point specification, E4M3: bias 7, subnormals m * 2^-9,
    # S.1111.111 is NaN, no infinities, largest finite 448.
    table = eo.e4m3_to_f32(np.arange(256, dtype=np.uint8))
    for code in range(256):
        s, e, m = code >> 7, (code >> 3) & 15, code & 7
        if e == 15 and m == 7:
            assert np.isnan(table[code])
            continue
        mag = m * 2.0 ** -9 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7)
        assert table[code] == (-mag if s else mag)
    assert table[0x7E] == 448.0 and table[0x08] == 2.0 ** -6 and table[0x01] == 2.0 ** -9
    want = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    ok = ~np.isnan(want)
    assert np.array_equal(table[ok], want[ok])


def test_e4m3_encode_exhaustive_against_torch_and_spec():
    codes = np.arange(65536, dtype=np.uint16)
    x = eo.bf16_to_f32(codes)
    x = x[np.isfinite(x)]
    rng = np.random.default_rng(1)
    amax = np.concatenate([[1e-4, 1.0, 3.0, 448.0, 0.37], np.abs(rng.standard_normal(11)) * 4 + 1e-3]).astype(np.float32)
    scales = (np.float32(448.0) / amax).astype(np.float32)
    for s in scales:
        v = (x * s).astype(np.float32)
        got = eo.f32_to_e4m3(v)
        in_range = np.abs(v) <= 464.0
        want = torch.from_numpy(v[in_range]).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        assert np.array_equal(got[in_range], want)
        # saturation edge: everything at or beyond 448 in magnitude is +-448
        big = np.abs(v) >= 448.0
        assert np.all((got[big] & 0x7F) == 0x7E)
        assert np.array_equal(got[big] >> 7, (v[big] < 0).astype(np.uint8))
    # ties: exactly halfway between neighbouring codes rounds to the even mantissa
    table = eo.e4m3_to_f32(np.arange(0x7F, dtype=np.uint8)).astype(np.float64)
    mids = ((table[:-1] + table[1:]) / 2).astype(np.float32)
    got = eo.f32_to_e4m3(mids)
    want = np.array([c if c % 2 == 0 else c + 1 for c in range(0x7E)], np.uint8)
    assert np.array_equal(got, want)
    special = eo.f32_to_e4m3(np.array([np.inf, -np.inf, np.nan, 0.0, -0.0, 1e-30, 2.0 ** -10, 3 * 2.0 ** -10], np.float32))
    assert list(special[:2]) == [0x7E, 0xFE] and (special[2] & 0x7F) == 0x7F
    assert list(special[3:]) == [0x00, 0x80, 0x00, 0x00, 0x02]


def test_fp8_scales_constants_and_division():
    # kernels/utils.cuh:430-456
    inv = np.float32(1) / np.float32(448.0)
    assert inv.view(np.uint32) == 0x3B124925
    rng = np.random.default_rng(2)
    for amax in np.concatenate([[1e-4, 1.0, 448.0], np.abs(rng.standard_normal(200)) * 3 + 1e-4]).astype(np.float32):
        s, si = eo.fp8_scales(amax)
        assert np.float32(s) == np.float32(448.0) / amax
        assert np.float32(si) == amax * inv
        s2, si2 = eo.fp8_scales(amax, round_scale=True)
        e = int(np.ceil(np.log2(np.float64(amax * inv))))
        assert si2 == 2.0 ** e and s2 == 2.0 ** -e


def test_cast_row_matches_torch_recipe_and_bounds():
    # per-128-channel cast against the reference test's torch recipe (tests/utils.py:70-77),
    # with its `448.0 / amax` written as a true fp32 division the way the kernel computes it
    # (kernels/utils.cuh:454; Python's scalar / tensor is reciprocal-then-multiply, one ulp
    # off for many amax).  The stored inverse scale is amax * (1/448.0f), not a division.
    rng = np.random.default_rng(3)
    for _ in range(20):
        row = torch.from_numpy(rng.standard_normal(512).astype(np.float32) * np.float32(rng.uniform(0.01, 30))).to(torch.bfloat16)
        q, sc = eo.cast_row_fp8(bf16_bits(row))
        xv = row.to(torch.float32).view(-1, 128)
        amax = xv.abs().amax(dim=1).clamp(1e-4)
        want_q = (xv * torch.div(torch.tensor(448.0), amax).unsqueeze(1)).to(torch.float8_e4m3fn).view(torch.uint8).numpy().reshape(-1)
        assert np.array_equal(q, want_q)
        assert np.array_equal(sc, (amax.numpy() * (np.float32(1) / np.float32(448.0))).astype(np.float32))
        deq = eo.e4m3_to_f32(q).reshape(-1, 128) * sc[:, None]
        assert np.all(np.abs(deq - xv.numpy()) <= amax.numpy()[:, None] * (2.0 ** -4) * 1.01)
    zero_q, zero_s = eo.cast_row_fp8(np.zeros(128, np.uint16))
    assert not zero_q.any() and zero_s[0] == np.float32(1e-4) * (np.float32(1) / np.float32(448.0))


# ---- low-latency dispatch ---------------------------------------------------------------------

def _world(rng, R, T, H, K, E, drop=0.1, scale=1.0):
    x = torch.from_numpy(rng.standard_normal((R, T, H)).astype(np.float32) * scale).to(torch.bfloat16)
    scores = rng.standard_normal((R, T, E))
    topk = np.argsort(-scores, axis=2)[:, :, :K].astype(np.int32)
    topk[rng.random((R, T, K)) < drop] = -1
    w = np.abs(rng.standard_normal((R, T, K))).astype(np.float32)
    return x, topk, w


def _brute_force_dispatch(xb, topk, E, M, use_fp8, round_scale=False, num_tokens=None, mask=None):
    """Independent restatement: enumerate (expert, src rank, token) in canonical order."""
    R, T, H = xb.shape
    El, N = E // R, R * M
    out = {}
    for d in range(R):
        for le in range(El):
            e = d * El + le
            rows, begin, ranges = [], 0, []
            for r in range(R):
                nt = T if num_tokens is None else num_tokens[r]
                blocked = mask is not None and (mask[r][d] or mask[d][r])
                toks = [] if blocked else [t for t in range(nt) if e in topk[r, t]]
                ranges.append((len(toks), begin))
                begin += len(toks)
                rows += [(r, t) for t in toks]
            out[(d, le)] = (rows, ranges)
    return out


@pytest.mark.parametrize("use_fp8,round_scale,use_ue8m0", [(False, False, False), (True, False, False), (True, True, False), (True, True, True)])
def test_ll_dispatch_brute_force_and_reference_invariants(use_fp8, round_scale, use_ue8m0):
    rng = np.random.default_rng(10 + use_fp8 + 2 * round_scale)
    R, T, H, K, E, M = 4, 12, 512, 3, 8, 16
    x, topk, _ = _world(rng, R, T, H, K, E)
    num_tokens = np.array([12, 7, 0, 12], np.int32)
    xb = bf16_bits(x).reshape(R, T, H)
    fill = 0x55
    o = eo.ll_dispatch(xb, topk, E, M, use_fp8, round_scale, use_ue8m0, num_tokens=num_tokens, fill=fill)
    El, N = E // R, R * M
    want = _brute_force_dispatch(xb, topk, E, M, use_fp8, round_scale, num_tokens)
    for d in range(R):
        for le in range(El):
            rows, ranges = want[(d, le)]
            e = d * El + le
            # invariants of tests/elastic/elastic.py:263-318
            assert o["recv_count"][d, le] == len(rows)
            assert o["recv_count"][d, le] == int((o["layout_range"][d, le] & 0xFFFFFFFF).sum())
            assert len(rows) == sum(int((topk[r, :num_tokens[r]] == e).sum()) for r in range(R))
            for r in range(R):
                n, b = ranges[r]
                assert int(o["layout_range"][d, le, r] & 0xFFFFFFFF) == n
                if n:
                    assert int(o["layout_range"][d, le, r] >> 32) == b
            for i, (r, t) in enumerate(rows):
                assert o["src_info"][d, le, i] == t
                if use_fp8:
                    q, sc = eo.cast_row_fp8(xb[r, t], round_scale)
                    assert np.array_equal(o["recv_x"][d, le, i], q)
                    if use_ue8m0:
                        words = o["scales"][d, le, :, i].view(np.uint8).reshape(-1)
                        assert np.array_equal(words, (sc.view(np.uint32) >> 23).astype(np.uint8))
                    else:
                        assert np.array_equal(o["scales"][d, le, :, i], sc)
                else:
                    assert np.array_equal(o["recv_x"][d, le, i], xb[r, t])
            # rows past recv_count are not written
            n = len(rows)
            assert np.all(o["recv_x"][d, le, n:].view(np.uint8) == fill)
            assert np.all(o["src_info"][d, le, n:].view(np.uint8) == fill)


def test_ll_dispatch_repeated_expert_takes_a_slot_per_selection():
    """A token whose top-k names one expert more than once: the reference's send phase takes a
    slot per (token, selection) with an atomicAdd (kernels/nixl_ep_ll.cu:186-190) and its
    receive phase packs whatever the count word says (:319-338), so the expert receives the
    token's row once per selection.  Enumerated here selection by selection, without the
    oracle's slot arithmetic: counts, ranges, sources and rows must agree, in the oracle's
    canonical order (tokens ascending, a token's selections together).  More selections from
    one rank to one expert than its slots hold is refused."""
    rng = np.random.default_rng(23)
    R, T, H, K, E, M = 3, 10, 256, 4, 6, 20
    x, topk, _ = _world(rng, R, T, H, K, E, drop=0.05)
    for r, t, k_from, k_to in [(0, 1, 0, 2), (0, 1, 0, 3), (1, 4, 1, 0), (2, 9, 3, 2), (2, 0, 0, 1)]:
        topk[r, t, k_to] = topk[r, t, k_from] if topk[r, t, k_from] >= 0 else 0
    topk[1, 7, :] = 5  # every selection of one token goes to the same expert
    xb = bf16_bits(x).reshape(R, T, H)
    fill = 0x55
    o = eo.ll_dispatch(xb, topk, E, M, False, fill=fill)
    El = E // R
    assert int(o["recv_count"].sum()) == int((topk >= 0).sum())
    for d in range(R):
        for le in range(El):
            e = d * El + le
            begin = 0
            for r in range(R):
                picks = [t for t in range(T) for k in range(K) if topk[r, t, k] == e]
                lr = int(o["layout_range"][d, le, r])
                assert (lr & 0xFFFFFFFF) == len(picks)
                if picks:
                    assert (lr >> 32) == begin
                assert o["src_info"][d, le, begin:begin + len(picks)].tolist() == picks
                for i, t in enumerate(picks):
                    assert np.array_equal(o["recv_x"][d, le, begin + i], xb[r, t])
                begin += len(picks)
            assert o["recv_count"][d, le] == begin
            assert np.all(o["recv_x"][d, le, begin:].view(np.uint8) == fill)
    # the expert of rank 1, token 7 holds that token four times in a row
    seg = int(o["layout_range"][5 // El, 5 % El, 1])
    rows = o["src_info"][5 // El, 5 % El, (seg >> 32):(seg >> 32) + (seg & 0xFFFFFFFF)].tolist()
    assert rows.count(7) == K
    crowded = topk.copy()
    crowded[0, :, :] = 2  # rank 0 sends T * K = 40 rows to expert 2, which holds M = 20 of its rows
    with pytest.raises(ValueError):
        eo.ll_dispatch(xb, crowded, E, M, False)


def test_ll_dispatch_reference_test_pattern():
    # Data pattern of tests/elastic/elastic.py:131-134: every channel = rank - 128 except the
    # last 128 channels, which hold the token index; bf16 dispatch must deliver it verbatim
    # and the per-source segments must carry their rank's value (:296-318).
    R, T, H, K, E, M = 4, 16, 256, 2, 8, 16
    rng = np.random.default_rng(5)
    x = torch.ones((R, T, H), dtype=torch.bfloat16) * (torch.arange(R).view(R, 1, 1) - 128).to(torch.bfloat16)
    x[:, :, -128:] = torch.arange(T).to(torch.bfloat16).view(1, T, 1)
    _, topk, _ = _world(rng, R, T, H, K, E, drop=0.05)
    o = eo.ll_dispatch(bf16_bits(x).reshape(R, T, H), topk, E, M, use_fp8=False)
    for d in range(R):
        for le in range(E // R):
            n = int(o["recv_count"][d, le])
            rx = eo.bf16_to_f32(o["recv_x"][d, le, :n])
            assert np.array_equal(rx[:, :-128].min(1), rx[:, :-128].max(1))
            assert np.array_equal(rx[:, -1], o["src_info"][d, le, :n].astype(np.float32))
            for r in range(R):
                cnt, b = int(o["layout_range"][d, le, r] & 0xFFFFFFFF), int(o["layout_range"][d, le, r] >> 32)
                assert np.all(rx[b:b + cnt, :-128] == r - 128)
                assert cnt == int((topk[r] == d * (E // R) + le).sum())


def test_ll_dispatch_mask_removes_rank_both_ways():
    # tests/elastic/elastic.py:359-383: a masked rank's tokens are absent from every count.
    rng = np.random.default_rng(6)
    R, T, H, K, E, M = 4, 8, 128, 2, 8, 8
    x, topk, _ = _world(rng, R, T, H, K, E, drop=0.0)
    dead = 2
    mask = np.zeros((R, R), np.int32)
    mask[:, dead] = 1
    mask[dead, :] = 1
    o = eo.ll_dispatch(bf16_bits(x).reshape(R, T, H), topk, E, M, use_fp8=False, mask=mask)
    alive = [r for r in range(R) if r != dead]
    for d in range(R):
        for le in range(E // R):
            e = d * (E // R) + le
            want = 0 if d == dead else sum(int((topk[r] == e).sum()) for r in alive)
            assert o["recv_count"][d, le] == want
            assert int(o["layout_range"][d, le, dead] & 0xFFFFFFFF) == 0


def test_ll_dispatch_argument_errors():
    x = np.zeros((2, 4, 128), np.uint16)
    topk = np.zeros((2, 4, 1), np.int32)
    with pytest.raises(ValueError):
        eo.ll_dispatch(x, topk, 4, 2)  # T > max tokens per rank
    with pytest.raises(ValueError):
        eo.ll_dispatch(x, topk, 4, 4, use_fp8=True)  # fp8 needs hidden % 512 == 0 (nixl_ep.cpp:1091)
    with pytest.raises(ValueError):
        eo.ll_dispatch(x, topk, 3, 4, use_fp8=False)  # experts must divide evenly over ranks


# ---- low-latency combine -----------------------------------------------------------------------

def test_ll_combine_closed_form_and_identity_experts():
    rng = np.random.default_rng(20)
    R, T, H, K, E, M = 4, 10, 512, 4, 16, 12
    x, topk, w = _world(rng, R, T, H, K, E, drop=0.15)
    xb = bf16_bits(x).reshape(R, T, H)
    o = eo.ll_dispatch(xb, topk, E, M, use_fp8=False)
    # identity experts: combined == x * sum of the valid weights (elastic.py:377-387)
    got = eo.ll_combine(o["recv_x"], topk, w, o["src_info"], o["layout_range"], E, M)
    xf = eo.bf16_to_f32(xb)
    wsum = (w * (topk >= 0)).sum(2)
    assert calc_diff(xf * wsum[:, :, None], eo.bf16_to_f32(got)) < 1e-5
    # closed form in float64 with per-expert outputs: within one bf16 ulp of the exact sum
    El, N = E // R, R * M
    y = o["recv_x"].copy()
    for d in range(R):
        for le in range(El):
            f = eo.bf16_to_f32(o["recv_x"][d, le]) * np.float32(1 + 0.001 * (d * El + le))
            y[d, le] = eo.f32_to_bf16(f)
    got_fma = eo.bf16_to_f32(eo.ll_combine(y, topk, w, o["src_info"], o["layout_range"], E, M, use_fma=True))
    got_mul = eo.bf16_to_f32(eo.ll_combine(y, topk, w, o["src_info"], o["layout_range"], E, M, use_fma=False))
    exact = np.zeros((R, T, H), np.float64)
    for r in range(R):
        for t in range(T):
            for k in range(K):
                e = topk[r, t, k]
                if e < 0:
                    continue
                d, le = divmod(int(e), El)
                n, b = int(o["layout_range"][d, le, r] & 0xFFFFFFFF), int(o["layout_range"][d, le, r] >> 32)
                i = b + list(o["src_info"][d, le, b:b + n]).index(t)
                exact[r, t] += eo.bf16_to_f32(y[d, le, i]).astype(np.float64) * np.float64(w[r, t, k])
    ulp = np.maximum(np.abs(exact), 2.0 ** -126) * 2.0 ** -7
    assert np.all(np.abs(got_fma - exact) <= ulp) and np.all(np.abs(got_mul - exact) <= ulp)
    # a single selection with weight 1 returns the expert row bit for bit
    topk1 = topk.copy()
    topk1[:, :, 1:] = -1
    topk1[:, :, 0] = np.abs(topk[:, :, 0])
    o1 = eo.ll_dispatch(xb, topk1, E, M, use_fp8=False)
    g1 = eo.ll_combine(o1["recv_x"], topk1, np.ones_like(w), o1["src_info"], o1["layout_range"], E, M)
    assert np.array_equal(g1, xb)


def test_ll_combine_accepts_any_valid_permutation():
    # The reference assigns slots with atomics, so a handle may list a segment's tokens in
    # any order; the reduction must follow src_info, not position.
    rng = np.random.default_rng(21)
    R, T, H, K, E, M = 2, 8, 128, 2, 4, 8
    x, topk, w = _world(rng, R, T, H, K, E, drop=0.0)
    xb = bf16_bits(x).reshape(R, T, H)
    o = eo.ll_dispatch(xb, topk, E, M, use_fp8=False)
    base = eo.ll_combine(o["recv_x"], topk, w, o["src_info"], o["layout_range"], E, M)
    rx, si = o["recv_x"].copy(), o["src_info"].copy()
    for d in range(R):
        for le in range(E // R):
            for r in range(R):
                n, b = int(o["layout_range"][d, le, r] & 0xFFFFFFFF), int(o["layout_range"][d, le, r] >> 32)
                p = rng.permutation(n)
                rx[d, le, b:b + n] = o["recv_x"][d, le, b:b + n][p]
                si[d, le, b:b + n] = o["src_info"][d, le, b:b + n][p]
    assert np.array_equal(eo.ll_combine(rx, topk, w, si, o["layout_range"], E, M), base)


# ---- normal mode ---------------------------------------------------------------------------------

def test_dispatch_layout_against_plain_torch():
    # tests/test_ht.py:99-152 recomputes the layout in plain torch
    rng = np.random.default_rng(30)
    T, K, R, E = 64, 4, 4, 16
    scores = rng.standard_normal((T, E))
    topk = np.argsort(-scores, axis=1)[:, :K].astype(np.int32)
    topk[rng.random((T, K)) < 0.1] = -1
    per_rank, per_expert, in_rank = eo.dispatch_layout(topk, R, E)
    tk = torch.from_numpy(topk)
    for e in range(E):
        assert per_expert[e] == int((tk == e).sum())
    rank_idx = torch.where(tk >= 0, tk // (E // R), tk)
    for r in range(R):
        hit = (rank_idx == r).any(dim=1)
        assert per_rank[r] == int(hit.sum())
        assert np.array_equal(in_rank[:, r].astype(bool), hit.numpy())


def _ht_world(rng, R, T, H, K, E):
    x, topk, w = _world(rng, R, T, H, K, E, drop=0.1)
    xb = bf16_bits(x).reshape(R, T, H)
    layouts = [eo.dispatch_layout(topk[r], R, E) for r in range(R)]
    in_rank = np.stack([l[2] for l in layouts])
    per_expert = np.stack([l[1] for l in layouts])
    return xb, topk, w, in_rank, per_expert


def test_ht_notify_dispatch_combine_properties():
    rng = np.random.default_rng(31)
    R, T, H, K, E, C = 4, 37, 256, 4, 16, 5
    xb, topk, w, in_rank, per_expert = _ht_world(rng, R, T, H, K, E)
    prefix, counts, chan = eo.ht_notify(in_rank, per_expert, C, expert_alignment=8)
    # receive prefix: inclusive over source ranks (nixl_ep_ht.cu:295-302)
    for d in range(R):
        assert np.array_equal(prefix[d], np.cumsum(in_rank[:, :, d].sum(1)))
        for le in range(E // R):
            n = int(per_expert[:, d * (E // R) + le].sum())
            assert counts[d, le] == -(-n // 8) * 8
    per_chan = -(-T // C)
    for r in range(R):
        for d in range(R):
            assert chan[r, d, -1] == in_rank[r, :, d].sum()
            for c in range(C):
                assert chan[r, d, c] == in_rank[r, :min(T, per_chan * (c + 1)), d].sum()
    o = eo.ht_dispatch(xb, topk, w, in_rank, prefix, E)
    El = E // R
    assert o["recv_x"].shape[0] == int(prefix[:, -1].sum())
    for d in range(R):
        base = int(o["row_offset"][d])
        # rows [prefix[i-1], prefix[i]) come from rank i, tokens ascending (test_ht.py:166-172)
        for r in range(R):
            lo = base + (0 if r == 0 else int(prefix[d, r - 1]))
            hi = base + int(prefix[d, r])
            assert np.all(o["recv_src_rank"][lo:hi] == r)
            toks = o["recv_src_token"][lo:hi]
            assert np.array_equal(toks, np.nonzero(in_rank[r, :, d])[0])
            assert np.array_equal(o["recv_x"][lo:hi], xb[r, toks])
            assert np.array_equal(o["send_head"][r, toks, d], np.arange(hi - lo))
        rows = slice(base, int(o["row_offset"][d + 1]))
        ridx = o["recv_topk_idx"][rows]
        assert np.all((ridx == -1) | ((ridx >= 0) & (ridx < El)))  # test_ht.py:236-244
        for le in range(El):
            assert int((ridx == le).sum()) == int(per_expert[:, d * El + le].sum())
        assert np.all(o["recv_topk_weights"][rows][ridx < 0] == 0)
    # combine: unweighted fp32 sum over holders; (combined - b0 - b1) / holders == x (test_ht.py:304-308)
    b0 = bf16_bits(torch.from_numpy(rng.standard_normal((R, T, H)).astype(np.float32)).to(torch.bfloat16)).reshape(R, T, H)
    comb, wsum = eo.ht_combine(o["recv_x"], o["recv_topk_weights"], in_rank, prefix, o["send_head"], o["row_offset"], bias0=b0)
    holders = in_rank.sum(2).astype(np.float64)
    exact = eo.bf16_to_f32(xb).astype(np.float64) * holders[:, :, None] + eo.bf16_to_f32(b0)
    ulp = np.maximum(np.abs(exact), 2.0 ** -126) * 2.0 ** -7
    assert np.all(np.abs(eo.bf16_to_f32(comb) - exact) <= ulp)
    want_w = np.where(topk >= 0, w, 0).astype(np.float32)
    assert np.allclose(wsum, want_w, rtol=0, atol=1e-9) or calc_diff(wsum, want_w) < 1e-9  # test_ht.py:309-323
    no_bias, _ = eo.ht_combine(o["recv_x"], o["recv_topk_weights"], in_rank, prefix, o["send_head"], o["row_offset"])
    one = holders == 1
    assert np.array_equal(no_bias[one], xb[one])


# ---- router ---------------------------------------------------------------------------------------

def test_router_against_torch_topk_softmax():
    rng = np.random.default_rng(40)
    logits = rng.standard_normal((200, 256)).astype(np.float32)
    logits[0, :] = 0.0  # all ties: lowest indices win
    logits[1, 5] = logits[1, 9] = 7.0
    idx, w = eo.router(logits, 8)
    tv, ti = torch.topk(torch.from_numpy(logits), 8, dim=1, largest=True, sorted=True)
    # torch does not promise an order among ties; compare values always, indices off ties
    assert np.array_equal(np.take_along_axis(logits, idx, 1), tv.numpy())
    assert np.array_equal(idx[2:], ti.numpy()[2:])
    assert list(idx[0]) == list(range(8)) and list(idx[1][:2]) == [5, 9]
    want = torch.softmax(tv, dim=1).numpy()
    assert np.allclose(w, want, rtol=2e-6, atol=0)
    assert np.allclose(w.sum(1), 1.0, atol=1e-6)


def test_low_latency_buffer_size_hint_follows_the_reference_layout():
    """EPLayout arithmetic (examples/device/ep/csrc/config.hpp:145-208) at the DeepSeek-V3
    shape: messages of 14 352 B and 14 560 B, send = recv = 256 * 128 * 14 560 B, 2 KiB of
    signalling, everything twice; the hint rounds up past the next multiple of 128."""
    from nixl_amd.ep import Buffer
    msg_d, msg_c = 16 + max(7168 * 2, 7168 + 56 * 4), 56 * 4 + 7168 * 2
    assert (msg_d, msg_c) == (14352, 14560)
    buf = 256 * 128 * msg_c
    total = 2 * buf + 2 * buf + 2 * 2048
    assert total == 1908412416
    assert Buffer.get_low_latency_buffer_size_hint(128, 7168, 32, 256) == total + 128
    assert Buffer.get_rdma_size_hint(128, 7168, 32, 256) == total + 128
    # a shape where the dispatch message is the larger one on the send side
    small = Buffer.get_low_latency_buffer_size_hint(64, 2048, 2, 1)
    d, c = 16 + 2048 * 2, 16 * 4 + 2048 * 2
    assert small == (2 * max(64 * d, 64 * c) + 2 * max(64 * d, 64 * c) + 2 * 128 + 128) // 128 * 128


def test_buffer_exposes_the_reference_method_names():
    """Every public method of the reference's Buffer (examples/device/ep/nixl_ep/buffer.py:
    43-886) exists here under the same name, so that code written against it finds them."""
    from nixl_amd.ep import Buffer
    names = ["destroy", "is_sm90_compiled", "set_num_sms", "capture", "get_low_latency_buffer_size_hint",
             "get_rdma_size_hint", "get_comm_stream", "get_local_buffer_tensor", "get_dispatch_config",
             "get_combine_config", "get_dispatch_layout", "low_latency_dispatch", "dispatch",
             "low_latency_combine", "combine", "ht_dispatch", "ht_combine", "update_mask_buffer",
             "query_mask_buffer", "clean_mask_buffer", "get_next_combine_buffer", "update_memory_buffers",
             "set_tcp_store_group", "connect_ranks", "disconnect_ranks", "barrier"]
    missing = [n for n in names if not callable(getattr(Buffer, n, None))]
    assert not missing, missing
    assert Buffer.is_sm90_compiled() is False
    # ... and takes its arguments in the reference's order (buffer.py:278-284, 329-341, 443-454,
    # 526-540, 663-672), so that positional calls mean the same; extensions come after them
    import inspect
    order = {
        "get_dispatch_layout": ["topk_idx", "num_experts", "previous_event", "async_finish", "allocate_on_comm_stream"],
        "low_latency_dispatch": ["x", "topk_idx", "num_max_dispatch_tokens_per_rank", "num_experts",
                                 "cumulative_local_expert_recv_stats", "dispatch_wait_recv_cost_stats", "use_fp8",
                                 "round_scale", "use_ue8m0", "async_finish", "return_recv_hook"],
        "low_latency_combine": ["x", "topk_idx", "topk_weights", "handle", "use_logfmt", "zero_copy", "async_finish",
                                "return_recv_hook", "out", "combine_wait_recv_cost_stats"],
        "ht_dispatch": ["x", "handle", "num_tokens_per_rank", "num_tokens_per_rdma_rank", "is_token_in_rank",
                        "num_tokens_per_expert", "topk_idx", "topk_weights", "expert_alignment", "config",
                        "previous_event", "async_finish", "allocate_on_comm_stream"],
        "ht_combine": ["x", "handle", "topk_weights", "bias", "config", "previous_event", "async_finish",
                       "allocate_on_comm_stream"],
    }
    for name, want in order.items():
        got = [p for p in inspect.signature(getattr(Buffer, name)).parameters if p != "self"]
        assert got[:len(want)] == want, (name, got)


def _logfmt_reference_f64(vals):
    """LogFMT-10 round trip of one 128-channel group in float64 from its definition
    (examples/device/ep/csrc/kernels/nixl_ep_ll.cu:459-616): returns (decoded, step) or
    (vals, None) when the group is not cast."""
    a = np.abs(vals.astype(np.float64))
    amax, amin = a.max(), a.min()
    with np.errstate(divide="ignore"):
        log_amax = np.log2(amax) if amax > 0 else -np.inf
        log_amin = max(np.log2(amin) if amin > 0 else -np.inf, log_amax - 32)
    if not (log_amax < 0 and log_amin < log_amax):
        return vals.astype(np.float64), None
    step = (log_amax - log_amin) / 510
    rounding = 2 - np.log2((1 + 2.0 ** step) * 0.5) / step
    with np.errstate(divide="ignore"):
        pos = np.maximum(np.where(a > 0, np.log2(np.where(a > 0, a, 1)), -np.inf) / step + rounding - log_amin / step, 0)
    code = np.floor(pos)
    dec = np.where(code == 0, 0.0, 2.0 ** ((code - 1) * step + log_amin))
    return np.where(np.signbit(vals), -dec, dec), step


def test_logfmt_roundtrip_against_float64_definition_and_properties():
    rng = np.random.default_rng(77)
    groups = [rng.standard_normal(128) * s for s in (0.5, 0.1, 0.01, 1e-3, 1e-6)]
    groups.append(rng.standard_normal(128) * 3.0)          # amax >= 1: not cast
    groups.append(np.full(128, 0.25))                       # constant: not cast
    z = rng.standard_normal(128) * 0.2
    z[::7] = 0.0
    z[5] = -0.0
    groups.append(z)                                        # zeros inside a cast group
    groups.append(np.concatenate([[0.9], np.full(127, 1e-30)]))  # range wider than 2^32: amin floored
    row = eo.f32_to_bf16(np.concatenate(groups).astype(np.float32))
    vals = eo.bf16_to_f32(row)
    got = eo.logfmt_roundtrip(row)
    for i in range(len(groups)):
        v, g = vals[i * 128:(i + 1) * 128], got[i * 128:(i + 1) * 128]
        want, step = _logfmt_reference_f64(v)
        if step is None:
            assert np.array_equal(g, v), i  # untouched
            continue
        assert np.array_equal(np.signbit(g), np.signbit(v)), i
        assert np.array_equal(g == 0, (want == 0)), i
        nz = want != 0
        # fp32 evaluation may land one code off the float64 one at a floor boundary
        ratio = np.abs(g[nz] / want[nz])
        assert np.all((ratio < 2.0 ** (1.01 * step)) & (ratio > 2.0 ** (-1.01 * step))), i
        assert np.mean(np.abs(np.log2(ratio)) < 1e-3) > 0.9, i  # almost all on the same code
        # the codec's own promise: what comes back is within half a step (in log2) of what went in,
        # except below the smallest representable level
        a = np.abs(v[nz].astype(np.float64))
        floor_level = 2.0 ** (np.log2(np.abs(v).max()) - 32) if i == len(groups) - 1 else 0
        big = a > floor_level * 2
        err = np.abs(np.log2(np.abs(g[nz][big]) / a[big]))
        assert np.all(err <= 0.51 * step + 1e-6), (i, err.max(), step)
    # monotone: a larger magnitude never decodes to a smaller one
    cast_group = eo.f32_to_bf16(np.sort(np.abs(rng.standard_normal(128)) * 0.3).astype(np.float32))
    dec = eo.logfmt_roundtrip(cast_group)
    assert np.all(np.diff(dec) >= 0)


def test_ll_combine_logfmt_is_the_sum_of_decoded_rows():
    R, T, H, K, E, M = 2, 5, 256, 2, 4, 8
    rng = np.random.default_rng(78)
    x = eo.f32_to_bf16((rng.standard_normal((R, T, H)) * 0.3).astype(np.float32))
    topk = np.stack([np.stack([rng.permutation(E)[:K] for _ in range(T)]) for _ in range(R)]).astype(np.int32)
    w = rng.random((R, T, K)).astype(np.float32)
    o = eo.ll_dispatch(x, topk, E, M, use_fp8=False)
    out = eo.ll_combine(o["recv_x"], topk, w, o["src_info"], o["layout_range"], E, M, use_logfmt=True)
    for r in range(R):
        for t in range(T):
            dec = eo.logfmt_roundtrip(x[r, t])  # every destination holds the token's own row
            acc = np.zeros(H, np.float32)
            for k in range(K):
                acc = (dec.astype(np.float64) * np.float64(w[r, t, k]) + acc).astype(np.float32)
            assert np.array_equal(out[r, t], eo.f32_to_bf16(acc)) or np.max(np.abs(eo.bf16_to_f32(out[r, t]) - acc)) < 1e-2


def test_normal_mode_config_shims():
    """Config / set_num_sms / get_*_config of the reference (buffer.py:54,116-126,221-275): only
    the SM count keeps a meaning here (channels = num_sms / 2, csrc/nixl_ep.cpp:630)."""
    from nixl_amd import ep
    assert ep.Buffer.num_sms == 20 and ep.Buffer.get_dispatch_config(8).num_sms == 20
    ep.Buffer.set_num_sms(24)
    try:
        assert ep.Buffer.get_combine_config(32).num_sms == 24
        with pytest.raises(ep.EPError):
            ep.Buffer.set_num_sms(7)
        assert ep.Config(24, 6, 256, 6, 128).chunk_sizes == (6, 256, 6, 128)
    finally:
        ep.Buffer.set_num_sms(20)
