"""GPU parity tests for the expert-parallel half: the HIP kernels through their C ABI
(include/nixl_amd_ep.h) and through the host-side Buffer, against the CPU oracle on seeded
inputs, on the reference tests' own data pattern, and through size-independent properties
at the full BASELINE sizes."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import ep_oracle as eo
from nixl_amd import _lib
from nixl_amd.ep import Buffer, EPError

pytestmark = pytest.mark.gpu


def bits16(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def calc_diff(x, y):
    # examples/device/ep/tests/utils.py:63-67
    x, y = x.double() + 1, y.double() + 1
    return float(1 - 2 * (x * y).sum() / (x * x + y * y).sum())


def make_world(seed, R, T, H, K, E, drop=0.1, scale=1.0):
    rng = np.random.default_rng(seed)
    x = torch.from_numpy(rng.standard_normal((R, T, H)).astype(np.float32) * scale).to(torch.bfloat16)
    scores = rng.standard_normal((R, T, E))
    topk = np.argsort(-scores, axis=2)[:, :, :K].astype(np.int32)
    topk[rng.random((R, T, K)) < drop] = -1
    w = np.abs(rng.standard_normal((R, T, K))).astype(np.float32)
    return x, topk, w


def raw_ll_dispatch(cuda, x, topk, E, M, use_fp8, round_scale=False, use_ue8m0=False, num_tokens=None, mask=None,
                    stats=None, fill=0x55):
    """Call the C ABI directly on buffers pre-filled with `fill`."""
    k = _lib.ep_kernels()
    R, T, H = x.shape
    K = topk.shape[2]
    El, N = E // R, R * M
    dev = lambda a, dt: None if a is None else torch.from_numpy(np.ascontiguousarray(a, dtype=dt)).to(cuda)
    xd = x.to(cuda)
    td = dev(topk, np.int32)
    ntd, md = dev(num_tokens, np.int32), dev(mask, np.int32)
    recv_x = torch.full((R, El, N, H * (1 if use_fp8 else 2)), fill, dtype=torch.uint8, device=cuda)
    scales = None
    if use_fp8:
        scales = torch.full((R, El, (H // 512 if use_ue8m0 else H // 128), N, 4), fill, dtype=torch.uint8, device=cuda)
    src_info = torch.full((R, El, N, 4), fill, dtype=torch.uint8, device=cuda)
    layout = torch.zeros((R, El, R), dtype=torch.int64, device=cuda)
    count = torch.zeros((R, El), dtype=torch.int32, device=cuda)
    ws = torch.empty(k.nixl_amd_ep_ll_workspace_bytes(R, E, T, K, H) + 16, dtype=torch.uint8, device=cuda)
    p = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())
    rc = k.nixl_amd_ep_ll_dispatch(p(recv_x), p(scales), p(src_info), p(layout), p(count), p(md), p(stats), p(xd), p(td),
                                   p(ntd), T, H, M, K, R, E, int(use_fp8), int(round_scale), int(use_ue8m0), None, p(ws),
                                   ws.numel(), None)
    torch.cuda.synchronize()
    return rc, dict(recv_x=recv_x.cpu().numpy(), scales=None if scales is None else scales.cpu().numpy(),
                    src_info=src_info.cpu().numpy(), layout_range=layout.cpu().numpy(), recv_count=count.cpu().numpy())


def assert_dispatch_equal(got, want, use_fp8, use_ue8m0=False, fill=0x55):
    assert np.array_equal(got["recv_count"], want["recv_count"])
    assert np.array_equal(got["layout_range"], want["layout_range"])
    R, El = want["recv_count"].shape
    wx = want["recv_x"].view(np.uint8).reshape(got["recv_x"].shape)
    wsi = want["src_info"].view(np.uint8).reshape(got["src_info"].shape)
    assert np.array_equal(got["recv_x"], wx)  # includes: rows past recv_count keep the fill byte
    assert np.array_equal(got["src_info"], wsi)
    if use_fp8:
        ws = want["scales"].view(np.uint8).reshape(got["scales"].shape)
        assert np.array_equal(got["scales"], ws)


# ---- encoder -------------------------------------------------------------------------------------

def test_fp8_encoder_exhaustive(cuda):
    codes = np.arange(65536, dtype=np.uint16)
    x = eo.bf16_to_f32(codes)
    rng = np.random.default_rng(1)
    amax = np.concatenate([[1e-4, 1.0, 3.0, 448.0, 0.37], np.abs(rng.standard_normal(27)) * 4 + 1e-3]).astype(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        v = (x[None, :] * (np.float32(448.0) / amax)[:, None]).astype(np.float32).reshape(-1)
    extra = np.array([np.inf, -np.inf, np.nan, -np.nan, 448.0, 463.9, 464.0, 1e30, 2.0 ** -10, 3 * 2.0 ** -10, 2.0 ** -9 * 7.5],
                     np.float32)
    rnd = rng.integers(0, 2 ** 32, 1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32)
    v = np.concatenate([v, extra, rnd])
    vin = torch.from_numpy(v).to(cuda)
    out = torch.empty(v.size, dtype=torch.uint8, device=cuda)
    rc = _lib.ep_kernels().nixl_amd_ep_f32_to_e4m3(ctypes.c_void_p(vin.data_ptr()), ctypes.c_void_p(out.data_ptr()), v.size, None)
    assert rc == 0, _lib.kernels_error()
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), eo.f32_to_e4m3(v))


# ---- low-latency dispatch ---------------------------------------------------------------------------

@pytest.mark.parametrize("use_fp8,round_scale,use_ue8m0", [(False, False, False), (True, False, False), (True, True, False), (True, True, True)])
@pytest.mark.parametrize("shape", [(4, 12, 512, 3, 8, 16), (2, 130, 1024, 8, 64, 130), (8, 5, 2560, 4, 16, 8)])
def test_ll_dispatch_matches_oracle(cuda, shape, use_fp8, round_scale, use_ue8m0):
    R, T, H, K, E, M = shape
    if use_fp8 and H % 512:
        pytest.skip("fp8 needs hidden % 512 == 0")
    x, topk, _ = make_world(hash(shape) % 1000 + use_fp8, R, T, H, K, E, scale=3.0)
    nt = np.full(R, T, np.int32)
    nt[1] = T // 2
    nt[-1] = 0
    rc, got = raw_ll_dispatch(cuda, x, topk, E, M, use_fp8, round_scale, use_ue8m0, num_tokens=nt)
    assert rc == 0, _lib.kernels_error()
    want = eo.ll_dispatch(bits16(x).reshape(R, T, H), topk, E, M, use_fp8, round_scale, use_ue8m0, num_tokens=nt, fill=0x55)
    assert_dispatch_equal(got, want, use_fp8, use_ue8m0)


@pytest.mark.parametrize("hidden", [2048, 2560, 3072, 3584, 4096, 5120, 6144, 7168, 8192])
def test_ll_every_hidden_size_of_the_reference(cuda, hidden):
    """The hidden sizes the reference's low-latency kernels are built for
    (kernels/launch.cuh:100-112): dispatch (fp8 where hidden % 512 == 0, as csrc/nixl_ep.cpp:1091
    demands, else bf16) and combine against the oracle, bit for bit."""
    R, T, K, E, M = 2, 19, 3, 8, 24
    El = E // R
    x, topk, w = make_world(hidden, R, T, hidden, K, E, scale=2.0)
    use_fp8 = hidden % 512 == 0
    rc, got = raw_ll_dispatch(cuda, x, topk, E, M, use_fp8)
    assert rc == 0, _lib.kernels_error()
    xb = bits16(x).reshape(R, T, hidden)
    assert_dispatch_equal(got, eo.ll_dispatch(xb, topk, E, M, use_fp8, fill=0x55), use_fp8)
    buf = Buffer(R, device=cuda)
    td, wd = torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
    rx, cnt, handle, _, _ = buf.dispatch(x.to(cuda), td, M, E, use_fp8=False)
    valid = (torch.arange(R * M, device=cuda).view(1, 1, -1) < cnt.unsqueeze(-1)).unsqueeze(-1)
    y = torch.where(valid, rx, torch.zeros_like(rx))
    out, _, _ = buf.combine(y, td, wd, handle)
    torch.cuda.synchronize()
    want = eo.ll_combine(bits16(y).reshape(R, El, R * M, hidden), topk, w, handle[0].cpu().numpy(), handle[1].cpu().numpy(), E, M)
    assert np.array_equal(bits16(out).reshape(R, T, hidden), want)
    # rows of more than 512 lanes are combined by two workgroups: the LogFMT codec's groups of
    # 16 lanes must stay whole (agreement with the libm restatement as in test_ll_combine_logfmt)
    out, _, _ = buf.combine(y, td, wd, handle, use_logfmt=True)
    torch.cuda.synchronize()
    want = eo.ll_combine(bits16(y).reshape(R, El, R * M, hidden), topk, w, handle[0].cpu().numpy(), handle[1].cpu().numpy(), E, M,
                         use_fma=True, use_logfmt=True)
    assert np.mean(bits16(out).reshape(R, T, hidden) == want) > 0.98


def test_ll_dispatch_extreme_values(cuda):
    # zeros (amax floor 1e-4), huge and tiny magnitudes, a constant row, negative zero
    R, T, H, K, E, M = 2, 8, 512, 2, 4, 8
    x, topk, _ = make_world(7, R, T, H, K, E, drop=0.0)
    x[0, 0] = 0
    x[0, 1] = 3.0e38
    x[0, 2] = 1.0e-38
    x[0, 3] = -0.0
    x[0, 4] = 1.0
    x[1, 0, ::2] = 1.0e-5
    x[1, 1] = torch.arange(H).to(torch.bfloat16) - 256
    rc, got = raw_ll_dispatch(cuda, x, topk, E, M, True)
    assert rc == 0
    assert_dispatch_equal(got, eo.ll_dispatch(bits16(x).reshape(R, T, H), topk, E, M, True, fill=0x55), True)


def test_ll_dispatch_mask_and_stats(cuda):
    R, T, H, K, E, M = 4, 16, 512, 4, 16, 16
    x, topk, _ = make_world(11, R, T, H, K, E, drop=0.0)
    mask = np.zeros((R, R), np.int32)
    mask[:, 2] = 1
    mask[2, :] = 1
    stats = torch.full((R, E // R), 5, dtype=torch.int32, device=cuda)
    rc, got = raw_ll_dispatch(cuda, x, topk, E, M, True, mask=mask, stats=stats)
    assert rc == 0
    want = eo.ll_dispatch(bits16(x).reshape(R, T, H), topk, E, M, True, mask=mask, fill=0x55)
    assert_dispatch_equal(got, want, True)
    assert np.array_equal(stats.cpu().numpy(), want["recv_count"] + 5)  # elastic.py:266-269
    assert got["recv_count"][2].sum() == 0


def test_ll_dispatch_rejects_bad_arguments(cuda):
    x, topk, _ = make_world(1, 2, 4, 512, 2, 4)
    assert raw_ll_dispatch(cuda, x, topk, 4, 2, True)[0] == -1  # T > max tokens per rank
    assert raw_ll_dispatch(cuda, x, topk, 3, 4, True)[0] == -1  # experts do not divide over ranks
    assert raw_ll_dispatch(cuda, x, topk, 4, 4, False, use_ue8m0=True)[0] == -1
    x2, topk2, _ = make_world(1, 2, 4, 384, 2, 4)
    assert raw_ll_dispatch(cuda, x2, topk2, 4, 4, True)[0] == -1  # fp8 needs hidden % 512 == 0
    buf = Buffer(2, device=cuda)
    with pytest.raises(EPError):
        buf.dispatch(x.to(cuda).float(), torch.from_numpy(topk).to(cuda), 4, 4)
    with pytest.raises(EPError):
        Buffer(2, low_latency_mode=False, device=cuda).dispatch(x.to(cuda), torch.from_numpy(topk).to(cuda), 4, 4)


# ---- low-latency combine -------------------------------------------------------------------------------

@pytest.mark.parametrize("shape", [(4, 12, 512, 3, 8, 16), (2, 130, 1024, 8, 64, 130), (8, 5, 2560, 4, 16, 8), (2, 9, 7168, 8, 16, 16)])
def test_ll_combine_matches_oracle(cuda, shape):
    R, T, H, K, E, M = shape
    x, topk, w = make_world(5 + R, R, T, H, K, E)
    nt = np.full(R, T, np.int32)
    nt[0] = max(T - 3, 0)
    buf = Buffer(R, device=cuda)
    td = torch.from_numpy(topk).to(cuda)
    wd = torch.from_numpy(w).to(cuda)
    ntd = torch.from_numpy(nt).to(cuda)
    rx, cnt, handle, _, _ = buf.dispatch(x.to(cuda), td, M, E, use_fp8=False, num_tokens_per_rank=ntd)
    # expert f_e(x) = x * (1 + 0.001 e) in bf16, only on the rows that exist
    El = E // R
    factor = (1 + 0.001 * torch.arange(E, device=cuda, dtype=torch.float32)).view(R, El, 1, 1)
    valid = (torch.arange(R * M, device=cuda).view(1, 1, -1) < cnt.unsqueeze(-1)).unsqueeze(-1)
    y = torch.where(valid, (rx.float() * factor).to(torch.bfloat16), torch.zeros_like(rx))
    comb = torch.full((R, T, H), 7.0, dtype=torch.bfloat16, device=cuda)
    out, _, _ = buf.combine(y, td, wd, handle, out=comb, num_tokens_per_rank=ntd)
    # the same through a plain tuple handle: rows are then found by searching src_info
    searched, _, _ = buf.combine(y, td, wd, tuple(handle), out=comb.clone(), num_tokens_per_rank=ntd)
    torch.cuda.synchronize()
    assert out is comb and handle.row_map is not None
    assert torch.equal(searched.view(torch.int16), comb.view(torch.int16))
    si, lr = handle[0].cpu().numpy(), handle[1].cpu().numpy()
    want = eo.ll_combine(bits16(y).reshape(R, El, R * M, H), topk, w, si, lr, E, M, num_tokens=nt, use_fma=True)
    got = bits16(comb).reshape(R, T, H)
    for r in range(R):
        assert np.array_equal(got[r, :nt[r]], want[r, :nt[r]])
        assert np.all(got[r, nt[r]:] == 0x40E0)  # rows of absent tokens keep the caller's 7.0
    # within one bf16 ulp of the unfused (multiply, then add) evaluation
    alt = eo.ll_combine(bits16(y).reshape(R, El, R * M, H), topk, w, si, lr, E, M, num_tokens=nt, use_fma=False)
    a, b = eo.bf16_to_f32(got), eo.bf16_to_f32(alt)
    for r in range(R):
        ulp = np.maximum(np.abs(b[r, :nt[r]]), 2.0 ** -126) * 2.0 ** -7
        assert np.all(np.abs(a[r, :nt[r]] - b[r, :nt[r]]) <= ulp)


def test_ll_combine_follows_src_info_not_position(cuda):
    R, T, H, K, E, M = 2, 70, 512, 2, 4, 70
    x, topk, w = make_world(21, R, T, H, K, E, drop=0.0)
    buf = Buffer(R, device=cuda)
    td, wd = torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
    rx, cnt, handle, _, _ = buf.dispatch(x.to(cuda), td, M, E, use_fp8=False)
    base, _, _ = buf.combine(rx.clone(), td, wd, handle)
    si, lr = handle[0].clone(), handle[1].cpu().numpy()
    rx2 = rx.clone()
    rng = np.random.default_rng(0)
    for d in range(R):
        for le in range(E // R):
            for r in range(R):
                n, b = int(lr[d, le, r] & 0xFFFFFFFF), int(lr[d, le, r] >> 32)
                p = torch.from_numpy(rng.permutation(n)).to(cuda)
                rx2[d, le, b:b + n] = rx[d, le, b:b + n][p]
                si[d, le, b:b + n] = handle[0][d, le, b:b + n][p]
    out, _, _ = buf.combine(rx2, td, wd, (si, handle[1], handle[2], handle[3]))
    assert torch.equal(out.view(torch.int16), base.view(torch.int16))


def test_ll_masked_rank_drops_out_of_dispatch_and_combine(cuda):
    # examples/device/ep/tests/elastic/elastic.py:359-383: after a rank is masked its tokens
    # vanish from every count and its experts no longer contribute to combine.
    R, T, H, K, E, M = 4, 16, 512, 4, 16, 16
    x, topk, w = make_world(31, R, T, H, K, E, drop=0.0)
    buf = Buffer(R, device=cuda)
    buf.update_mask_buffer(1, True)
    status = torch.zeros(R, dtype=torch.int32, device=cuda)
    buf.query_mask_buffer(status)
    assert status.tolist() == [0, 1, 0, 0]
    td, wd = torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
    rx, cnt, handle, _, _ = buf.dispatch(x.to(cuda), td, M, E, use_fp8=False)
    out, _, _ = buf.combine(torch.where(torch.isfinite(rx.float()), rx, torch.zeros_like(rx)), td, wd, handle)
    torch.cuda.synchronize()
    El = E // R
    alive = torch.tensor([0, 2, 3])
    for e in range(E):
        want = 0 if e // El == 1 else int((torch.from_numpy(topk)[alive] == e).sum())
        assert int(cnt[e // El, e % El]) == want
    keep = torch.from_numpy((topk // El != 1) & (topk >= 0))
    wsum = (torch.from_numpy(w) * keep).sum(2)
    for r in (0, 2, 3):
        assert calc_diff(x[r].float() * wsum[r].unsqueeze(1), out[r].float().cpu()) < 1e-5
    buf.clean_mask_buffer()
    buf.query_mask_buffer(status)
    assert status.sum().item() == 0


def test_reference_elastic_pattern_fp8_and_bf16(cuda):
    # The data of examples/device/ep/tests/elastic/elastic.py:131-134,153-175 and its checks
    # (:263-318, :377-387) with 4 virtual ranks, 32 experts, top-8 and 64 tokens.
    R, T, H, K, E, M = 4, 64, 2048, 8, 32, 64
    El = E // R
    g = torch.Generator().manual_seed(0)
    x = torch.ones((R, T, H), dtype=torch.bfloat16) * (torch.arange(R).view(R, 1, 1) - 128).to(torch.bfloat16)
    x[:, :, -128:] = torch.arange(T).to(torch.bfloat16).view(1, T, 1)
    scores = torch.randn((R, T, E), generator=g).abs() + 1
    topk = torch.topk(scores, K, dim=-1, largest=True, sorted=True)[1].to(torch.int32)
    for r in range(R):
        for _ in range(10):
            topk[r, int(torch.randint(0, T, (1,), generator=g)), int(torch.randint(0, K, (1,), generator=g))] = -1
    w = torch.randn((R, T, K), generator=g).abs()
    buf = Buffer(R, device=cuda)
    xd, td, wd = x.to(cuda), topk.to(cuda), w.to(cuda)
    for use_fp8 in (False, True):
        stats = torch.zeros((R, El), dtype=torch.int32, device=cuda)
        recv, cnt, handle, event, hook = buf.dispatch(xd, td, M, E, cumulative_local_expert_recv_stats=stats,
                                                      use_fp8=use_fp8, async_finish=True)
        event.current_stream_wait()
        torch.cuda.synchronize()
        if use_fp8:
            q, sc = recv[0], recv[1].contiguous()
            assert sc.shape == (R, El, R * M, H // 128)
            # cast back through bf16 like per_token_cast_back (tests/utils.py:80-89)
            deq = (q.float().view(R, El, R * M, H // 128, 128) * sc.unsqueeze(-1)).view(R, El, R * M, H)
            deq = deq.to(torch.bfloat16).float()
        else:
            deq = recv.float()
        for rank in range(R):
            for i in range(El):
                e = rank * El + i
                n = int(cnt[rank, i])
                assert int(stats[rank, i]) == n
                lr = handle[1][rank, i]
                assert n == int((lr & 0xFFFFFFFF).sum()) == int((topk == e).sum())
                if n == 0:
                    continue
                rx = deq[rank, i, :n]
                assert torch.equal(rx[:, :-128].amin(dim=-1), rx[:, :-128].amax(dim=-1))
                src = handle[0][rank, i, :n]
                assert float((rx[:, -128:] - src.view(-1, 1) % T).abs().sum()) == 0 or use_fp8
                if use_fp8:
                    assert calc_diff(rx[:, -1], src.float()) < 0.007
                for j in range(R):
                    b, c = int(lr[j] >> 32), int(lr[j] & 0xFFFFFFFF)
                    assert c == int((topk[j] == e).sum())
                    assert float((rx[b:b + c, :-128] - (j - 128)).abs().sum()) == 0
        # identity experts: combined == x * sum of valid weights
        y = deq.to(torch.bfloat16)
        y = torch.where(torch.isfinite(y.float()), y, torch.zeros_like(y))
        comb, _, _ = buf.combine(y, td, wd, handle)
        torch.cuda.synchronize()
        ref = xd.float() * (wd * (td >= 0)).sum(2, keepdim=True)
        assert calc_diff(ref, comb.float()) < (9e-4 if use_fp8 else 1e-5)


def test_config4_full_size_properties(cuda):
    # BASELINE config 4: 32 virtual ranks x 128 tokens x hidden 7168, 256 experts, top-8 by
    # the router from N(0,1) logits, fp8 dispatch, expert f_e = dequant(x) * (1 + 0.001 e) in
    # bf16, weighted combine.  Checked by: counts against a histogram, every delivered row
    # against the oracle's cast of its source token (sampled) and against a torch
    # re-quantisation (all rows, dequantised error bound), combine against the closed form
    # on sampled tokens (bit-exact) and against x * sum(w * f) globally.
    R, T, H, K, E, M = 32, 128, 7168, 8, 256, 128
    El, N = E // R, R * M
    g = torch.Generator(device=cuda).manual_seed(4)
    x = torch.randn((R, T, H), generator=g, device=cuda).to(torch.bfloat16)
    logits = torch.randn((R, T, E), generator=g, device=cuda)
    buf = Buffer(R, device=cuda)
    topk, w = buf.route(logits, K)
    (q, sc_t), cnt, handle, _, _ = buf.dispatch(x, topk, M, E, use_fp8=True)
    torch.cuda.synchronize()
    src_info, layout = handle[0], handle[1]
    hist = torch.bincount(topk.view(-1).long(), minlength=E).view(R, El)
    assert torch.equal(cnt.long(), hist)
    assert torch.equal((layout & 0xFFFFFFFF).sum(-1), hist)
    # segments: begin = exclusive prefix of counts over source ranks
    counts = layout & 0xFFFFFFFF
    begins = layout >> 32
    assert torch.equal(begins, torch.cumsum(counts, -1) - counts)
    per_src = torch.stack([torch.bincount(topk[r].view(-1).long(), minlength=E) for r in range(R)], 1).view(R, El, R)
    assert torch.equal(counts, per_src)
    sc = sc_t.contiguous()  # [R, El, N, G]
    rng = np.random.default_rng(0)
    xb = bits16(x).reshape(R, T, H)
    qh = q.view(torch.uint8)
    lr = layout.cpu().numpy()
    for _ in range(48):
        e = int(rng.integers(0, E))
        d, le = divmod(e, El)
        n = int(cnt[d, le])
        if n == 0:
            continue
        i = int(rng.integers(0, n))
        seg_begin = lr[d, le] >> 32
        r = int(np.searchsorted(seg_begin + (lr[d, le] & 0xFFFFFFFF), i, side="right"))
        t = int(src_info[d, le, i])
        assert e in topk[r, t].tolist()
        want_q, want_s = eo.cast_row_fp8(xb[r, t])
        assert np.array_equal(qh[d, le, i].cpu().numpy(), want_q)
        assert np.array_equal(sc[d, le, i].cpu().numpy(), want_s)
    # expert step and combine
    valid = (torch.arange(N, device=cuda).view(1, 1, -1) < cnt.unsqueeze(-1))
    y = torch.zeros((R, El, N, H), dtype=torch.bfloat16, device=cuda)
    for d in range(R):
        deq = (q[d].float().view(El, N, H // 128, 128) * sc[d].unsqueeze(-1)).view(El, N, H)
        f = (1 + 0.001 * (d * El + torch.arange(El, device=cuda, dtype=torch.float32))).view(El, 1, 1)
        y[d] = torch.where(valid[d].unsqueeze(-1), (deq.to(torch.bfloat16).float() * f).to(torch.bfloat16), y[d])
    comb, _, _ = buf.combine(y, topk, w, handle)
    torch.cuda.synchronize()
    fw = (w * (1 + 0.001 * topk.float())).sum(-1, keepdim=True)
    assert calc_diff(x.float() * fw, comb.float()) < 9e-4
    si_h = src_info.cpu().numpy()
    tk, wk = topk.cpu().numpy(), w.cpu().numpy()
    for _ in range(24):
        r, t = int(rng.integers(0, R)), int(rng.integers(0, T))
        rows = []
        for k in range(K):
            e = int(tk[r, t, k])
            d, le = divmod(e, El)
            b, n = int(lr[d, le, r] >> 32), int(lr[d, le, r] & 0xFFFFFFFF)
            i = b + int(np.nonzero(si_h[d, le, b:b + n] == t)[0][0])
            rows.append(bits16(y[d, le, i]))
        assert np.array_equal(bits16(comb[r, t]), eo.weighted_sum_rows(np.stack(rows), wk[r, t]))


# ---- normal mode -------------------------------------------------------------------------------------------

def zipf_topk(rng, R, T, K, E, s=1.2):
    """Skewed router for BASELINE config 5: K distinct experts per token drawn from a Zipf(s)
    law over a seeded permutation of the experts (Gumbel top-k = sampling without
    replacement), softmax weights of the drawn scores."""
    perm = rng.permutation(E)
    p = 1.0 / np.arange(1, E + 1) ** s
    logp = np.log(p / p.sum())[np.argsort(perm)]
    keys = logp[None, None, :] + rng.gumbel(size=(R, T, E))
    topk = np.argsort(-keys, axis=2)[:, :, :K].astype(np.int32)
    sel = np.take_along_axis(keys, topk, 2)
    w = np.exp(sel - sel.max(2, keepdims=True))
    return topk, (w / w.sum(2, keepdims=True)).astype(np.float32)


# 16 ranks take the per-pair scan kernel, up to 8 the packed one (2500 tokens: three chunks);
# hidden 2304: combine splits a row over three workgroups, the last one partly idle
@pytest.mark.parametrize("shape", [(4, 37, 256, 4, 16, 5, 8), (8, 300, 1024, 8, 64, 10, 1), (2, 1500, 512, 2, 4, 3, 4),
                                   (16, 50, 256, 4, 32, 3, 1), (8, 2500, 128, 3, 16, 7, 2), (5, 1030, 128, 2, 10, 4, 1),
                                   (3, 40, 2304, 4, 12, 3, 1)])
def test_ht_pipeline_matches_oracle(cuda, shape):
    R, T, H, K, E, C, align = shape
    x, topk, w = make_world(3 * R, R, T, H, K, E)
    buf = Buffer(R, low_latency_mode=False, device=cuda)
    xd, td, wd = x.to(cuda), torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
    per_rank, _, per_expert, in_rank, _ = buf.get_dispatch_layout(td, E)
    torch.cuda.synchronize()
    lay = [eo.dispatch_layout(topk[r], R, E) for r in range(R)]
    assert np.array_equal(per_rank.cpu().numpy(), np.stack([l[0] for l in lay]))
    assert np.array_equal(per_expert.cpu().numpy(), np.stack([l[1] for l in lay]))
    o_in_rank = np.stack([l[2] for l in lay])
    assert np.array_equal(in_rank.cpu().numpy().astype(np.uint8), o_in_rank)
    recv_x, recv_idx, recv_w, per_expert_list, handle, _ = buf.ht_dispatch(
        xd, num_tokens_per_rank=per_rank, is_token_in_rank=in_rank, num_tokens_per_expert=per_expert, topk_idx=td,
        topk_weights=wd, expert_alignment=align, num_channels=C)
    torch.cuda.synchronize()
    o_prefix, o_counts, o_chan = eo.ht_notify(o_in_rank, np.stack([l[1] for l in lay]), C, align)
    _, prefix, chan, meta, send_head, row_offset = handle
    assert np.array_equal(prefix.cpu().numpy(), o_prefix)
    assert np.array_equal(chan.cpu().numpy(), o_chan)
    assert per_expert_list == o_counts.tolist()
    o = eo.ht_dispatch(bits16(x).reshape(R, T, H), topk, w, o_in_rank, o_prefix, E)
    assert np.array_equal(row_offset.cpu().numpy(), o["row_offset"])
    assert np.array_equal(send_head.cpu().numpy(), o["send_head"])
    assert np.array_equal(bits16(recv_x).reshape(-1, H), o["recv_x"])
    assert np.array_equal(recv_idx.cpu().numpy(), o["recv_topk_idx"])
    assert np.array_equal(recv_w.cpu().numpy(), o["recv_topk_weights"])
    assert np.array_equal(meta.cpu().numpy(), np.stack([o["recv_src_rank"], o["recv_src_token"]], 1))
    # cached mode: the handle of the first dispatch moves another tensor without a count exchange
    x2 = (xd.float() * 0.5 + 1).to(torch.bfloat16)
    again, none_idx, none_w, none_list, none_handle, _ = buf.ht_dispatch(x2, handle=handle)
    torch.cuda.synchronize()
    assert none_idx is None and none_w is None and none_list is None and none_handle is None
    o2 = eo.ht_dispatch(bits16(x2).reshape(R, T, H), topk, w, o_in_rank, o_prefix, E)
    assert np.array_equal(bits16(again).reshape(-1, H), o2["recv_x"])
    b0 = torch.from_numpy(np.random.default_rng(1).standard_normal((R, T, H)).astype(np.float32)).to(torch.bfloat16)
    b1 = torch.from_numpy(np.random.default_rng(2).standard_normal((R, T, H)).astype(np.float32)).to(torch.bfloat16)
    for bias in (None, b0.to(cuda), (b0.to(cuda), b1.to(cuda))):
        comb, comb_w, _ = buf.ht_combine(recv_x, handle, topk_weights=recv_w, bias=bias)
        torch.cuda.synchronize()
        ob0 = None if bias is None else bits16(b0).reshape(R, T, H)
        ob1 = bits16(b1).reshape(R, T, H) if isinstance(bias, tuple) else None
        want, want_w = eo.ht_combine(o["recv_x"], o["recv_topk_weights"], o_in_rank, o_prefix, o["send_head"],
                                     o["row_offset"], ob0, ob1)
        assert np.array_equal(bits16(comb).reshape(R, T, H), want)
        assert np.array_equal(comb_w.cpu().numpy(), want_w)


@pytest.mark.parametrize("scale_dtype", [np.float32, np.int32])
def test_ht_dispatch_fp8_rows_with_scales(cuda, scale_dtype):
    """The (x, x_scales) form of normal-mode dispatch.  The reference's test passes fp8 rows
    with scales whose storage is transposed (tests/test_ht.py:78-79) and expects each received
    row's scales to be its source token's (:215-231: per_token_cast_back of the pair, then check_data).  Rows are
    checked as bytes against the oracle's row move, scales against a gather by the oracle's
    source rank and token, for the first dispatch, without top-k, and with a cached handle."""
    R, T, H, K, E, C = 4, 333, 512, 4, 16, 4
    S = H // 128
    _, topk, w = make_world(5, R, T, H, K, E)
    rng = np.random.default_rng(9)
    x8 = rng.integers(0, 256, (R, T, H), dtype=np.uint8)
    sc = (rng.standard_normal((R, T, S)) * 100).astype(scale_dtype)
    x8d = torch.from_numpy(x8).to(cuda).view(torch.float8_e4m3fn)
    sc_d = torch.from_numpy(sc).to(cuda).transpose(1, 2).contiguous().transpose(1, 2)
    assert sc_d.stride() == (T * S, 1, T)
    td, wd = torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
    buf = Buffer(R, low_latency_mode=False, device=cuda)
    per_rank, _, per_expert, in_rank, _ = buf.get_dispatch_layout(td, E)
    (recv_x, recv_sc), recv_idx, recv_w, _, handle, _ = buf.ht_dispatch(
        (x8d, sc_d), num_tokens_per_rank=per_rank, is_token_in_rank=in_rank, num_tokens_per_expert=per_expert,
        topk_idx=td, topk_weights=wd, num_channels=C)
    torch.cuda.synchronize()
    lay = [eo.dispatch_layout(topk[r], R, E) for r in range(R)]
    o_in_rank = np.stack([l[2] for l in lay])
    o_prefix, _, _ = eo.ht_notify(o_in_rank, np.stack([l[1] for l in lay]), C, 1)
    o = eo.ht_dispatch(x8.view(np.uint16), topk, w, o_in_rank, o_prefix, E)
    want_sc = sc[o["recv_src_rank"], o["recv_src_token"]]
    assert recv_x.dtype == torch.float8_e4m3fn and tuple(recv_x.shape) == (o["recv_x"].shape[0], H)
    assert np.array_equal(recv_x.view(torch.uint8).cpu().numpy(), o["recv_x"].view(np.uint8))
    assert recv_sc.is_contiguous() and np.array_equal(recv_sc.cpu().numpy(), want_sc)
    assert np.array_equal(recv_idx.cpu().numpy(), o["recv_topk_idx"])
    assert np.array_equal(recv_w.cpu().numpy(), o["recv_topk_weights"])
    # without top-k (tests/test_ht.py:176-199 runs both): rows, scales and the handle only
    (nx, nsc), n_idx, n_w, _, n_handle, _ = buf.ht_dispatch(
        (x8d, sc_d), num_tokens_per_rank=per_rank, is_token_in_rank=in_rank, num_tokens_per_expert=per_expert,
        num_channels=C)
    torch.cuda.synchronize()
    assert n_idx is None and n_w is None and torch.equal(n_handle[3], handle[3])
    assert torch.equal(nx.view(torch.uint8), recv_x.view(torch.uint8)) and torch.equal(nsc, recv_sc)
    # cached handle, other data, scales stored row-major this time
    x8b = rng.integers(0, 256, (R, T, H), dtype=np.uint8)
    scb = (rng.standard_normal((R, T, S)) * 100).astype(scale_dtype)
    (cx, csc), c_idx, _, _, _, _ = buf.ht_dispatch(
        (torch.from_numpy(x8b).to(cuda).view(torch.float8_e4m3fn), torch.from_numpy(scb).to(cuda)), handle=handle)
    torch.cuda.synchronize()
    o2 = eo.ht_dispatch(x8b.view(np.uint16), topk, w, o_in_rank, o_prefix, E)
    assert c_idx is None
    assert np.array_equal(cx.view(torch.uint8).cpu().numpy(), o2["recv_x"].view(np.uint8))
    assert np.array_equal(csc.cpu().numpy(), scb[o2["recv_src_rank"], o2["recv_src_token"]])
    # argument checks of csrc/nixl_ep.cpp:660,686,703-707
    with pytest.raises(EPError):
        buf.ht_dispatch((x8d, sc_d[:, :-1]), handle=handle)
    with pytest.raises(EPError):
        buf.ht_dispatch(x8d, handle=handle)  # fp8 rows need their scales
    with pytest.raises(EPError):
        buf.ht_dispatch((x8d, sc_d), num_tokens_per_rank=per_rank, is_token_in_rank=in_rank,
                        num_tokens_per_expert=per_expert, topk_idx=td, num_channels=C)


def test_ht_calls_honour_previous_event_and_async_finish(cuda):
    """previous_event / async_finish as the reference defines them (csrc/nixl_ep.cpp:558-571,
    596-611; its test passes buffer.capture() and waits on the returned event,
    tests/test_ht.py:204-214): the work waits for the event it is given, and with
    async_finish the returned event covers it.  The input is produced on a side stream behind
    a long fill, so a dispatch that ignored the event would read it too early."""
    R, T, H, K, E, C = 4, 257, 512, 4, 16, 4
    x, topk, w = make_world(13, R, T, H, K, E)
    td, wd = torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
    buf = Buffer(R, low_latency_mode=False, device=cuda)
    want_x = x.to(cuda)
    xd = torch.zeros_like(want_x)
    ballast = torch.empty(1 << 30, dtype=torch.uint8, device=cuda)
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device=cuda)
    with torch.cuda.stream(side):
        for _ in range(8):
            ballast.fill_(1)  # a few milliseconds of work ahead of the copy
        xd.copy_(want_x)
        produced = Buffer.capture()  # an EventOverlap on the side stream
    per_rank, _, per_expert, in_rank, ev0 = buf.get_dispatch_layout(td, E, previous_event=produced, async_finish=True)
    assert ev0.event is not None
    recv_x, recv_idx, recv_w, _, handle, ev1 = buf.ht_dispatch(
        xd, num_tokens_per_rank=per_rank, is_token_in_rank=in_rank, num_tokens_per_expert=per_expert, topk_idx=td,
        topk_weights=wd, previous_event=produced, async_finish=True, num_channels=C)
    assert ev1.event is not None
    # a consumer on another stream orders itself behind the dispatch through the returned event
    with torch.cuda.stream(side):
        ev1.current_stream_wait()
        seen = recv_x.clone()
        after = Buffer.capture()
    comb, _, ev2 = buf.ht_combine(seen, handle, topk_weights=recv_w, previous_event=after, async_finish=True)
    ev2.event.synchronize()
    torch.cuda.synchronize()
    lay = [eo.dispatch_layout(topk[r], R, E) for r in range(R)]
    o_in_rank = np.stack([l[2] for l in lay])
    o_prefix, _, _ = eo.ht_notify(o_in_rank, np.stack([l[1] for l in lay]), C, 1)
    o = eo.ht_dispatch(bits16(x).reshape(R, T, H), topk, w, o_in_rank, o_prefix, E)
    assert np.array_equal(bits16(seen).reshape(-1, H), o["recv_x"])
    want, _ = eo.ht_combine(o["recv_x"], o["recv_topk_weights"], o_in_rank, o_prefix, o["send_head"], o["row_offset"],
                            None, None)
    assert np.array_equal(bits16(comb).reshape(R, T, H), want)
    # csrc/nixl_ep.cpp:562,718,938
    with pytest.raises(EPError):
        buf.get_dispatch_layout(td, E, allocate_on_comm_stream=True)
    with pytest.raises(EPError):
        buf.ht_combine(seen, handle, allocate_on_comm_stream=True, async_finish=True)
    sync_out = buf.ht_combine(seen, handle)
    assert sync_out[2].event is None


def test_ht_dispatch_sized_ahead_equals_sized_exactly(cuda):
    """Normal-mode dispatch either sizes its receive tensors for the worst case and launches
    before the counts reach the host, or (past a byte limit) waits for the counts as the
    reference does (csrc/nixl_ep.cpp:762-800).  Both give the same tensors."""
    R, T, H, K, E, C = 4, 211, 512, 3, 16, 4
    x, topk, w = make_world(77, R, T, H, K, E)
    xd, td, wd = x.to(cuda), torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
    outs = []
    for limit in (16 << 30, 0):
        buf = Buffer(R, low_latency_mode=False, device=cuda)
        buf.ht_recv_worst_case_limit = limit
        per_rank, _, per_expert, in_rank, _ = buf.get_dispatch_layout(td, E)
        outs.append(buf.ht_dispatch(xd, num_tokens_per_rank=per_rank, is_token_in_rank=in_rank,
                                    num_tokens_per_expert=per_expert, topk_idx=td, topk_weights=wd, num_channels=C))
    torch.cuda.synchronize()
    (ax, ai, aw, al, ah, _), (bx, bi, bw, bl, bh, _) = outs
    assert ax.shape == bx.shape and ax.shape[0] == int(ah[5][-1]) and ax.is_contiguous()
    assert torch.equal(ax.view(torch.int16), bx.view(torch.int16)) and torch.equal(ai, bi) and torch.equal(aw, bw)
    assert al == bl and torch.equal(ah[3], bh[3]) and torch.equal(ah[5], bh[5])


def test_config5_full_size_properties(cuda):
    # BASELINE config 5: 8 virtual ranks x 4096 tokens x 7168, 256 experts, top-8, Zipf(1.2)
    # expert popularity; bf16 dispatch with counts and prefix layout; combine of per-rank
    # partial sums y_d[t] = bf16(sum over local selected experts of w * f_e(x)).
    R, T, H, K, E, C = 8, 4096, 7168, 8, 256, 10
    El = E // R
    rng = np.random.default_rng(5)
    topk, w = zipf_topk(rng, R, T, K, E)
    g = torch.Generator(device=cuda).manual_seed(5)
    x = torch.randn((R, T, H), generator=g, device=cuda).to(torch.bfloat16)
    td, wd = torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
    buf = Buffer(R, low_latency_mode=False, device=cuda)
    per_rank, _, per_expert, in_rank, _ = buf.get_dispatch_layout(td, E)
    # tests/test_ht.py:99-152
    assert torch.equal(per_expert.long(), torch.stack([torch.bincount(td[r].view(-1).long(), minlength=E) for r in range(R)]))
    rank_of = td // El
    want_in = torch.zeros((R, T, R), dtype=torch.bool, device=cuda).scatter_(2, rank_of.long(), True)
    assert torch.equal(in_rank, want_in)
    assert torch.equal(per_rank.long(), want_in.sum(1))
    recv_x, recv_idx, recv_w, per_expert_list, handle, _ = buf.ht_dispatch(
        x, num_tokens_per_rank=per_rank, is_token_in_rank=in_rank, num_tokens_per_expert=per_expert, topk_idx=td,
        topk_weights=wd, num_channels=C)
    torch.cuda.synchronize()
    _, prefix, chan, meta, send_head, row_offset = handle
    assert torch.equal(prefix.long(), torch.cumsum(want_in.sum(1).t(), 1))  # [dst][src], test_ht.py:166-172
    assert recv_x.shape[0] == int(want_in.sum())
    assert per_expert_list == per_expert.sum(0).view(R, El).tolist()  # test_ht.py:223-229
    # every received row is its source row; rows are ordered by (source rank, token)
    src_r, src_t = meta[:, 0].long(), meta[:, 1].long()
    assert torch.equal(recv_x.view(torch.int16), x[src_r, src_t].view(torch.int16))
    for d in range(R):
        lo, hi = int(row_offset[d]), int(row_offset[d + 1])
        key = src_r[lo:hi] * T + src_t[lo:hi]
        assert bool((key[1:] > key[:-1]).all())
        ridx = recv_idx[lo:hi]
        assert bool(((ridx == -1) | ((ridx >= 0) & (ridx < El))).all())  # test_ht.py:236-244
        assert torch.equal(torch.bincount(ridx[ridx >= 0].long(), minlength=El), per_expert.sum(0)[d * El:(d + 1) * El].long())
        assert bool((recv_w[lo:hi][ridx < 0] == 0).all())
    # expert step on each destination: partial weighted sum over its local experts
    f = 1 + 0.001 * (torch.arange(R, device=cuda).repeat_interleave(torch.diff(row_offset)).view(-1, 1) * El + recv_idx.clamp(min=0)).float()
    coef = (recv_w * f * (recv_idx >= 0)).sum(1, keepdim=True)
    y = (recv_x.float() * coef).to(torch.bfloat16)
    comb, comb_w, _ = buf.ht_combine(y, handle, topk_weights=recv_w)
    torch.cuda.synchronize()
    assert torch.allclose(comb_w, wd, rtol=0, atol=1e-7)  # test_ht.py:309-323
    ref = x.float() * (wd * (1 + 0.001 * td.float())).sum(-1, keepdim=True)
    assert calc_diff(ref, comb.float()) < 5e-5
    # exact check of the reduction on sampled tokens: ascending destination order, fp32 adds
    yb = y.view(torch.int16)
    for _ in range(16):
        r, t = int(rng.integers(0, R)), int(rng.integers(0, T))
        acc = np.zeros(H, np.float32)
        for d in range(R):
            if not bool(in_rank[r, t, d]):
                continue
            row = int(row_offset[d]) + (0 if r == 0 else int(prefix[d, r - 1])) + int(send_head[r, t, d])
            acc = acc + eo.bf16_to_f32(yb[row].cpu().numpy().view(np.uint16))
        assert np.array_equal(bits16(comb[r, t]), eo.f32_to_bf16(acc))


# ---- router ---------------------------------------------------------------------------------------------------

def test_router_matches_oracle(cuda):
    rng = np.random.default_rng(40)
    for T, E, K in ((200, 256, 8), (33, 7, 3), (5, 1024, 16), (64, 64, 1)):
        logits = rng.standard_normal((T, E)).astype(np.float32)
        logits[0, :] = 0.0
        if E > 9:
            logits[1, 5] = logits[1, 9] = 7.0
        buf = Buffer(2, device=cuda)
        idx, w = buf.route(torch.from_numpy(logits).to(cuda), K)
        torch.cuda.synchronize()
        oi, ow = eo.router(logits, K)
        assert np.array_equal(idx.cpu().numpy(), oi)
        # weights: exp() of the device and of libm may differ in the last place
        assert np.allclose(w.cpu().numpy(), ow, rtol=2e-6, atol=0)
    with pytest.raises(EPError):
        buf.route(torch.zeros((4, 2000), device=cuda), 2)


@pytest.mark.parametrize("shape", [(4, 70, 512, 3, 16, 80), (2, 130, 1024, 8, 256, 130), (8, 5, 512, 4, 1024, 8)])
@pytest.mark.parametrize("use_fp8", [True, False])
def test_route_dispatch_equals_route_then_dispatch(cuda, shape, use_fp8):
    """Routing folded into the dispatch call: the selection is the oracle router's, and every
    dispatch output equals the oracle's dispatch of that selection."""
    R, T, H, K, E, M = shape
    rng = np.random.default_rng(R * 100 + T)
    x = torch.from_numpy(rng.standard_normal((R, T, H)).astype(np.float32)).to(torch.bfloat16)
    logits = rng.standard_normal((R, T, E)).astype(np.float32)
    logits[0, 0, :] = 0.0  # all equal: ties go to the lower expert index
    nt = np.full(R, T, np.int32)
    nt[-1] = T // 2
    buf = Buffer(R, device=cuda)
    stats = torch.zeros((R, E // R), dtype=torch.int32, device=cuda)
    idx, w, recv, cnt, handle, _, _ = buf.route_dispatch(
        x.to(cuda), torch.from_numpy(logits).to(cuda), K, M, cumulative_local_expert_recv_stats=stats, use_fp8=use_fp8,
        num_tokens_per_rank=torch.from_numpy(nt).to(cuda))
    torch.cuda.synchronize()
    oi, ow = eo.router(logits.reshape(R * T, E), K)
    assert np.array_equal(idx.cpu().numpy().reshape(R * T, K), oi)
    assert np.allclose(w.cpu().numpy().reshape(R * T, K), ow, rtol=2e-6, atol=0)
    want = eo.ll_dispatch(bits16(x).reshape(R, T, H), oi.reshape(R, T, K), E, M, use_fp8, num_tokens=nt, fill=0)
    assert np.array_equal(cnt.cpu().numpy(), want["recv_count"])
    assert np.array_equal(stats.cpu().numpy(), want["recv_count"])
    assert np.array_equal(handle[1].cpu().numpy(), want["layout_range"])
    El, N = E // R, R * M
    rx = (recv[0] if use_fp8 else recv).view(torch.uint8).cpu().numpy().reshape(R, El, N, -1)
    wx = want["recv_x"].view(np.uint8).reshape(R, El, N, -1)
    si, wsi = handle[0].cpu().numpy(), want["src_info"].reshape(R, El, N)
    sc = recv[1].transpose(2, 3).contiguous().cpu().numpy() if use_fp8 else None  # back to [R][El][G][N]
    for r in range(R):
        for e in range(El):
            n = int(want["recv_count"][r, e])
            assert np.array_equal(rx[r, e, :n], wx[r, e, :n])
            assert np.array_equal(si[r, e, :n], wsi[r, e, :n])
            if use_fp8:
                assert np.array_equal(sc[r, e, :, :n].view(np.uint32), want["scales"].reshape(R, El, H // 128, N)[r, e, :, :n].view(np.uint32))


def test_ll_dispatch_reports_a_repeated_expert(cuda):
    """The K entries of a token must differ; a repeat is reported through the status word
    (and raised by Buffer.dispatch(check_duplicates=True)), a clean selection reports 0."""
    R, T, H, K, E, M = 2, 70, 512, 4, 8, 70
    x, topk, _ = make_world(3, R, T, H, K, E, drop=0.0)
    buf = Buffer(R, device=cuda)
    xd = x.to(cuda)
    buf.dispatch(xd, torch.from_numpy(topk).to(cuda), M, E, check_duplicates=True)
    bad = topk.copy()
    bad[1, 66, 3] = bad[1, 66, 0]
    with pytest.raises(EPError):
        buf.dispatch(xd, torch.from_numpy(bad).to(cuda), M, E, check_duplicates=True)
    bad[1, 66, 3] = -1  # "no selection" twice is not a repeat
    bad[1, 66, 2] = -1
    buf.dispatch(xd, torch.from_numpy(bad).to(cuda), M, E, check_duplicates=True)


def _with_repeats(rng, topk, per_rank, triple=True):
    """Makes `per_rank` tokens of every rank name one of their experts twice (and one token
    three times), in place; returns the number of selections that became repeats."""
    R, T, K = topk.shape
    made = 0
    for r in range(R):
        for n, t in enumerate(rng.choice(T, per_rank, replace=False)):
            ks = rng.choice(K, 3 if (triple and n == 0 and K >= 3) else 2, replace=False)
            if topk[r, t, ks[0]] < 0:
                topk[r, t, ks[0]] = 0
            for k in ks[1:]:
                topk[r, t, k] = topk[r, t, ks[0]]
                made += 1
    return made


@pytest.mark.parametrize("use_fp8", [True, False])
@pytest.mark.parametrize("shape", [(2, 40, 512, 4, 8, 48), (4, 150, 1024, 8, 32, 160), (3, 64, 512, 3, 6, 80)])
def test_ll_repeated_expert_gets_a_row_per_selection(cuda, shape, use_fp8):
    """A token that names an expert twice (or three times): the reference gives every selection
    a slot of its own (kernels/nixl_ep_ll.cu:186-190, an atomicAdd per selection), so the expert
    receives the token's row once per selection and recv_count, layout_range and src_info count
    them all.  Every dispatch output equals the oracle's, whose slots follow (token, selection)
    order; ranks with fewer tokens, a masked pair of ranks and several groups of 64 tokens per
    rank included.  The status word still says that a repeat was seen."""
    R, T, H, K, E, M = shape
    x, topk, _ = make_world(50 + R, R, T, H, K, E, drop=0.05)
    rng = np.random.default_rng(R * 7 + T)
    _with_repeats(rng, topk, min(T // 3, 9))
    nt = np.full(R, T, np.int32)
    nt[-1] = T - T // 4
    mask = np.zeros((R, R), np.int32)
    mask[0, R - 1] = 1
    stats = torch.zeros((R, E // R), dtype=torch.int32, device=cuda)
    rc, got = raw_ll_dispatch(cuda, x, topk, E, M, use_fp8, num_tokens=nt, mask=mask, stats=stats)
    assert rc == 0, _lib.kernels_error()
    want = eo.ll_dispatch(bits16(x), topk, E, M, use_fp8, num_tokens=nt, mask=mask, fill=0x55)
    El = E // R
    rows = sum(1 for r in range(R) for t in range(nt[r]) for e in topk[r, t]
               if e >= 0 and not (mask[r, e // El] or mask[e // El, r]))
    assert int(want["recv_count"].sum()) == rows  # a row per selection, repeats included
    assert_dispatch_equal(got, want, use_fp8)
    assert np.array_equal(stats.cpu().numpy(), want["recv_count"])


def test_ll_repeated_expert_combines_as_in_the_reference(cuda):
    """A token that names an expert twice: the reference gives the token two rows at that expert
    (kernels/nixl_ep_ll.cu:186-190), both hold the same data, and its combine reads, for each of
    the two selections, the row that was written back last into the token's slot for that
    expert (kernels/nixl_ep_ll.cu:959-1012): w1 * y + w2 * y.  Dispatch gives the two rows here
    too, combine reads each selection's own row, and the result equals the oracle's pipeline
    bit for bit, with the row map of the dispatch and with the rows found through src_info."""
    R, T, H, K, E, M = 2, 40, 512, 4, 8, 48
    x, topk, w = make_world(31, R, T, H, K, E, drop=0.0)
    rng = np.random.default_rng(7)
    _with_repeats(rng, topk, 6, triple=False)
    El = E // R
    buf = Buffer(R, device=cuda)
    td, wd = torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
    rx, cnt, handle, _, _ = buf.dispatch(x.to(cuda), td, M, E, use_fp8=False)
    factor = (1 + 0.001 * torch.arange(E, device=cuda, dtype=torch.float32)).view(R, El, 1, 1)
    valid = (torch.arange(R * M, device=cuda).view(1, 1, -1) < cnt.unsqueeze(-1)).unsqueeze(-1)
    y = torch.where(valid, (rx.float() * factor).to(torch.bfloat16), torch.zeros_like(rx))
    got, _, _ = buf.combine(y, td, wd, handle)
    searched, _, _ = buf.combine(y, td, wd, tuple(handle))  # rows found through src_info instead of the row map
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), searched.view(torch.int16))

    ref = eo.ll_dispatch(bits16(x), topk, E, M, use_fp8=False)  # every (token, selection) a slot of its own
    assert int(ref["recv_count"].sum()) == R * T * K and int(cnt.sum().item()) == R * T * K
    assert np.array_equal(cnt.cpu().numpy(), ref["recv_count"])
    ref_x = torch.from_numpy(ref["recv_x"].view(np.int16)).view(torch.bfloat16)
    ref_valid = (np.arange(R * M).reshape(1, 1, -1) < ref["recv_count"][..., None])[..., None]
    ref_y = (ref_x.float() * factor.cpu()).to(torch.bfloat16)
    ref_y = torch.where(torch.from_numpy(ref_valid), ref_y, torch.zeros_like(ref_y))
    want = eo.ll_combine(bits16(ref_y).reshape(R, El, R * M, H), topk, w, ref["src_info"], ref["layout_range"], E, M, use_fma=True)
    assert np.array_equal(bits16(got).reshape(R, T, H), want)


def test_ll_dispatch_without_tokens(cuda):
    R, H, K, E, M = 4, 512, 2, 8, 4
    x = torch.zeros((R, 0, H), dtype=torch.bfloat16)
    topk = np.zeros((R, 0, K), np.int32)
    rc, got = raw_ll_dispatch(cuda, x, topk, E, M, True)
    assert rc == 0, _lib.kernels_error()
    assert not got["recv_count"].any() and not got["layout_range"].any()
    assert (got["recv_x"] == 0x55).all()


# ---- the receive side's bounded wait: time-out -> mask (kernels/nixl_ep_ll.cu:316-340, 846-866) -----

def raw_ll_dispatch_phased(cuda, x, topk, E, M, use_fp8, mask, phases=(3,), timeout_us=0, withhold=-1, wait=None, fill=0x55,
                           header=None):
    """nixl_amd_ep_ll_dispatch_phased through the C ABI on buffers pre-filled with `fill`; one
    call per entry of `phases`, on the same buffers and workspace.  `header`: the workspace
    starts zeroed with these int32 words at its front instead of as allocated."""
    k = _lib.ep_kernels()
    R, T, H = x.shape
    K = topk.shape[2]
    El, N = E // R, R * M
    xd, td = x.to(cuda), torch.from_numpy(np.ascontiguousarray(topk, dtype=np.int32)).to(cuda)
    recv_x = torch.full((R, El, N, H * (1 if use_fp8 else 2)), fill, dtype=torch.uint8, device=cuda)
    scales = torch.full((R, El, H // 128, N, 4), fill, dtype=torch.uint8, device=cuda) if use_fp8 else None
    src_info = torch.full((R, El, N, 4), fill, dtype=torch.uint8, device=cuda)
    layout = torch.zeros((R, El, R), dtype=torch.int64, device=cuda)
    count = torch.zeros((R, El), dtype=torch.int32, device=cuda)
    ws = torch.empty(k.nixl_amd_ep_ll_workspace_bytes(R, E, T, K, H), dtype=torch.uint8, device=cuda)
    if header is not None:
        ws.zero_()
        ws[:4 * len(header)].view(torch.int32).copy_(torch.tensor(header, dtype=torch.int32))
    p = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())
    rcs = []
    for ph in phases:
        rcs.append(k.nixl_amd_ep_ll_dispatch_phased(p(recv_x), p(scales), p(src_info), p(layout), p(count), p(mask), None, p(wait),
                                                    p(xd), p(td), None, T, H, M, K, R, E, int(use_fp8), 0, 0, None, p(ws),
                                                    ws.numel(), ph, timeout_us, withhold, None))
    torch.cuda.synchronize()
    status = ctypes.c_int(-1)
    assert k.nixl_amd_ep_ll_dispatch_status(p(ws), None, ctypes.byref(status)) == 0
    return rcs, status.value, dict(recv_x=recv_x.cpu().numpy(), scales=None if scales is None else scales.cpu().numpy(),
                                   src_info=src_info.cpu().numpy(), layout_range=layout.cpu().numpy(),
                                   recv_count=count.cpu().numpy())


@pytest.mark.parametrize("use_fp8", [False, True])
def test_ll_dispatch_time_out_masks_the_late_rank(cuda, use_fp8):
    """A rank whose selections never arrive (its send phase is told to leave out the word the
    receivers wait for) costs the receive side its time-out, is entered in every receiver's
    mask and counts as having sent nothing: the outputs are those of a world in which that
    rank has no tokens, the others' waits are short, and the next dispatch treats it as
    masked.  T = 80: two groups of selections per rank, the second partly filled."""
    R, T, H, K, E, M = 4, 80, 512, 4, 16, 80
    x, topk, _ = make_world(21, R, T, H, K, E, drop=0.05)
    xb = bits16(x).reshape(R, T, H)
    mask = torch.zeros((R, R), dtype=torch.int32, device=cuda)
    wait = torch.zeros(R, dtype=torch.int64, device=cuda)
    timeout_us = 300
    rcs, status, got = raw_ll_dispatch_phased(cuda, x, topk, E, M, use_fp8, mask, timeout_us=timeout_us, withhold=2, wait=wait)
    assert rcs == [0], _lib.kernels_error()
    nt = np.array([T, T, 0, T], np.int32)
    assert_dispatch_equal(got, eo.ll_dispatch(xb, topk, E, M, use_fp8, num_tokens=nt, fill=0x55), use_fp8)
    assert status == 0
    want_mask = np.zeros((R, R), np.int32)
    want_mask[:, 2] = 1
    assert np.array_equal(mask.cpu().numpy(), want_mask)
    ticks = wait.cpu().numpy()
    budget = timeout_us * 100  # the wall clock of these GPUs runs at 100 MHz
    assert ticks[2] > budget and all(0 <= ticks[r] < budget for r in (0, 1, 3))
    # the mask now does what a mask set by hand does
    rc, got = raw_ll_dispatch(cuda, x, topk, E, M, use_fp8, mask=mask.cpu().numpy())
    assert rc == 0
    assert_dispatch_equal(got, eo.ll_dispatch(xb, topk, E, M, use_fp8, mask=want_mask, fill=0x55), use_fp8)
    # nobody late: the plain result, nothing masked, nearly nothing waited
    mask.zero_()
    wait.zero_()
    rcs, status, got = raw_ll_dispatch_phased(cuda, x, topk, E, M, use_fp8, mask, timeout_us=timeout_us, wait=wait)
    assert rcs == [0] and status == 0
    assert_dispatch_equal(got, eo.ll_dispatch(xb, topk, E, M, use_fp8, fill=0x55), use_fp8)
    assert not mask.any() and int(wait.max()) < budget


def test_ll_dispatch_in_two_phases(cuda):
    """Send phase and receive phase issued apart give the bytes of the single call, with and
    without the arrival check; a repeated expert is still reported when arrivals are stamped;
    arguments that make no sense are refused before anything is launched."""
    R, T, H, K, E, M = 3, 70, 1024, 4, 12, 70
    x, topk, _ = make_world(22, R, T, H, K, E, drop=0.1)
    want = eo.ll_dispatch(bits16(x).reshape(R, T, H), topk, E, M, True, fill=0x55)
    mask = torch.zeros((R, R), dtype=torch.int32, device=cuda)
    for timeout_us in (0, 500):
        rcs, status, got = raw_ll_dispatch_phased(cuda, x, topk, E, M, True, mask, phases=(1, 2), timeout_us=timeout_us)
        assert rcs == [0, 0] and status == 0, _lib.kernels_error()
        assert_dispatch_equal(got, want, True)
    assert not mask.any()
    bad = topk.copy()
    bad[2, 69, 1] = bad[2, 69, 0] = 5
    _, status, _ = raw_ll_dispatch_phased(cuda, x, bad, E, M, True, mask, timeout_us=500)
    assert status == 1
    for kwargs in (dict(phases=(0,)), dict(phases=(4,)), dict(withhold=1), dict(withhold=R, timeout_us=10),
                   dict(withhold=1, timeout_us=2_000_000)):
        rcs, _, _ = raw_ll_dispatch_phased(cuda, x, topk, E, M, True, mask, **kwargs)
        assert rcs == [-1], kwargs
    rcs, _, _ = raw_ll_dispatch_phased(cuda, x, topk, E, M, True, None, timeout_us=10)  # a time-out needs a mask buffer
    assert rcs == [-1]
    rcs, _, _ = raw_ll_dispatch_phased(cuda, x, topk, E, M, True, mask, timeout_us=100_000_001)  # at most 100 s
    assert rcs == [-1] and "100 s" in _lib.kernels_error()
    # A receive phase on a workspace that no send phase has written (here: a stamp nobody
    # published, no flags) must not wait out its budget: every rank is masked at once and nothing
    # is placed.  The budget is a second; the call is back long before.
    import time
    late_mask = torch.zeros((R, R), dtype=torch.int32, device=cuda)
    t0 = time.perf_counter()
    rcs, _, got = raw_ll_dispatch_phased(cuda, x, topk, E, M, True, late_mask, phases=(2,), timeout_us=1_000_000,
                                         header=[0, 12345, 0, 0, 0])
    assert rcs == [0] and time.perf_counter() - t0 < 0.5
    assert bool(late_mask.all()) and not got["recv_count"].any()


def test_buffer_time_out_hooks_and_ready_flags(cuda):
    """The same through Buffer: a buffer with timeout_ms checks arrivals; the recv hook issues
    the receive phase; combine waits for the ready word of each rank and masks the one whose
    word never comes (its experts then drop out of the sums, as for a rank masked by hand,
    examples/device/ep/tests/elastic/elastic.py:359-383)."""
    R, T, H, K, E, M = 4, 16, 512, 4, 16, 16
    El = E // R
    x, topk, w = make_world(31, R, T, H, K, E, drop=0.0)
    xd, td, wd = x.to(cuda), torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
    buf = Buffer(R, device=cuda, timeout_ms=0.3)
    status = torch.zeros(R, dtype=torch.int32, device=cuda)
    # dispatch in two halves: nothing of the payload exists before the hook has run
    rx, cnt, handle, _, hook = buf.dispatch(xd, td, M, E, use_fp8=False, return_recv_hook=True)
    cnt.fill_(-7)
    torch.cuda.synchronize()
    assert int(cnt[0, 0]) == -7
    hook()
    torch.cuda.synchronize()
    plain = Buffer(R, device=cuda)
    rx0, cnt0, handle0, _, _ = plain.dispatch(xd, td, M, E, use_fp8=False)
    torch.cuda.synchronize()
    assert torch.equal(cnt, cnt0) and torch.equal(handle[1], handle0[1]) and torch.equal(handle.row_map, handle0.row_map)
    buf.query_mask_buffer(status)
    assert status.sum().item() == 0
    y = torch.where(torch.isfinite(rx.float()), rx, torch.zeros_like(rx))
    # combine with a hook: the reduction is the receive phase, nothing is written before it
    canvas = torch.full((R, T, H), 7.0, dtype=torch.bfloat16, device=cuda)
    out, _, hook = buf.combine(y, td, wd, handle, out=canvas, return_recv_hook=True)
    torch.cuda.synchronize()
    assert bool((canvas == 7.0).all())
    hook()
    whole, _, _ = plain.combine(y, td, wd, handle0)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), whole.view(torch.int16))
    # combine: rank 3's expert outputs are never reported ready
    ready = torch.tensor([1, 1, 1, 0], dtype=torch.int32, device=cuda)
    waited = torch.zeros(R, dtype=torch.int64, device=cuda)
    out, _, _ = buf.combine(y, td, wd, handle, rank_ready=ready, combine_wait_recv_cost_stats=waited)
    torch.cuda.synchronize()
    buf.query_mask_buffer(status)
    assert status.tolist() == [0, 0, 0, 1]
    assert int(waited[3]) > 300 * 100 and int(waited[:3].max()) < 300 * 100
    keep = torch.from_numpy((topk // El != 3) & (topk >= 0))
    wsum = (torch.from_numpy(w) * keep).sum(2)
    for r in (0, 1, 2):
        assert calc_diff(x[r].float() * wsum[r].unsqueeze(1), out[r].float().cpu()) < 1e-5
    mask = np.zeros((R, R), np.int32)
    mask[:, 3] = 1
    want = eo.ll_combine(bits16(y).reshape(R, El, R * M, H), topk, w, handle[0].cpu().numpy(), handle[1].cpu().numpy(), E, M,
                         mask=mask)
    assert np.array_equal(bits16(out).reshape(R, T, H)[:3], want[:3])
    # a withheld rank in dispatch, through the one-shot knob
    buf.clean_mask_buffer()
    buf.withhold_rank = 1
    _, cnt, _, _, _ = buf.dispatch(xd, td, M, E, use_fp8=False)
    torch.cuda.synchronize()
    buf.query_mask_buffer(status)
    assert status.tolist() == [0, 1, 0, 0] and buf.withhold_rank == -1
    alive = torch.tensor([0, 2, 3])
    for e in range(E):
        assert int(cnt[e // El, e % El]) == int((torch.from_numpy(topk)[alive] == e).sum())


# ---- committed golden vectors (tests/golden, independent of the oracle) ---------------------------

def _golden(name):
    import os
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name), allow_pickle=False)


def test_golden_encoder_and_router(cuda):
    g = _golden("e4m3_encode.npz")
    v = np.concatenate([g["values"], g["sat_values"]])
    vin = torch.from_numpy(v).to(cuda)
    out = torch.empty(v.size, dtype=torch.uint8, device=cuda)
    rc = _lib.ep_kernels().nixl_amd_ep_f32_to_e4m3(ctypes.c_void_p(vin.data_ptr()), ctypes.c_void_p(out.data_ptr()), v.size, None)
    assert rc == 0, _lib.kernels_error()
    assert np.array_equal(out.cpu().numpy(), np.concatenate([g["codes"], g["sat_codes"]]))
    r = _golden("router.npz")
    idx, w = Buffer(2, device=cuda).route(torch.from_numpy(r["logits"]).to(cuda), r["topk_idx"].shape[1])
    assert np.array_equal(idx.cpu().numpy(), r["topk_idx"])
    assert np.allclose(w.cpu().numpy(), r["topk_weights"], rtol=2e-6, atol=0)


@pytest.mark.parametrize("world", ["ll_world.npz", "ll_world_repeats.npz"])
def test_golden_low_latency_world(cuda, world):
    g = _golden(world)
    E, M = int(g["num_experts"]), int(g["max_tok"])
    R, T, H = g["x"].shape
    El, N = E // R, R * M
    x = torch.from_numpy(g["x"].view(np.int16)).view(torch.bfloat16)
    for use_fp8 in (True, False):
        rc, got = raw_ll_dispatch(cuda, x, g["topk_idx"], E, M, use_fp8, num_tokens=g["num_tokens"])
        assert rc == 0, _lib.kernels_error()
        assert np.array_equal(got["recv_count"], g["recv_count"])
        assert np.array_equal(got["layout_range"], g["layout_range"])
        rx = got["recv_x"].reshape(R, El, N, -1)
        want = g["recv_fp8"] if use_fp8 else g["recv_bf16"].view(np.uint8).reshape(R, El, N, -1)
        si = got["src_info"].view(np.int32).reshape(R, El, N)
        for d in range(R):
            for le in range(El):
                n = int(g["recv_count"][d, le])
                assert np.array_equal(rx[d, le, :n], want[d, le, :n])
                assert np.array_equal(si[d, le, :n], g["src_info"][d, le, :n])
                if use_fp8:
                    sc = got["scales"].view(np.uint32).reshape(R, El, H // 128, N)
                    assert np.array_equal(sc[d, le, :, :n], g["scales"][d, le, :, :n].view(np.uint32))
    # combine from the fixture's own handle (rows located through src_info / layout_range)
    buf = Buffer(R, device=cuda)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(cuda)
    y = dev(g["expert_out"].view(np.int16)).view(torch.bfloat16)
    handle = (dev(g["src_info"]), dev(g["layout_range"]), M, H)
    out, _, _ = buf.combine(y, dev(g["topk_idx"]), dev(g["topk_weights"]), handle, num_tokens_per_rank=dev(g["num_tokens"]))
    torch.cuda.synchronize()
    got = bits16(out).reshape(R, T, H)
    for r, n in enumerate(g["num_tokens"]):
        assert np.array_equal(got[r, :n], g["combined"][r, :n])


def test_golden_normal_mode_world(cuda):
    g = _golden("ht_world.npz")
    R, T, K = g["topk_idx"].shape
    E, C = int(g["num_experts"]), int(g["num_channels"])
    H = g["x"].shape[2]
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(cuda)
    bf = lambda a: dev(a.view(np.int16)).view(torch.bfloat16)
    buf = Buffer(R, low_latency_mode=False, device=cuda)
    td, wd = dev(g["topk_idx"]), dev(g["topk_weights"])
    per_rank, _, per_expert, in_rank, _ = buf.get_dispatch_layout(td, E)
    assert np.array_equal(per_rank.cpu().numpy(), g["per_rank"])
    assert np.array_equal(per_expert.cpu().numpy(), g["per_expert"])
    assert np.array_equal(in_rank.cpu().numpy().astype(np.uint8), g["in_rank"])
    recv_x, recv_idx, recv_w, per_expert_list, handle, _ = buf.ht_dispatch(
        bf(g["x"]), num_tokens_per_rank=per_rank, is_token_in_rank=in_rank, num_tokens_per_expert=per_expert,
        topk_idx=td, topk_weights=wd, num_channels=C)
    _, prefix, chan, meta, send_head, row_offset = handle
    assert np.array_equal(prefix.cpu().numpy(), g["prefix"])
    assert np.array_equal(chan.cpu().numpy(), g["channel_prefix"])
    assert per_expert_list == g["expert_count"].tolist()
    assert np.array_equal(row_offset.cpu().numpy(), g["row_offset"])
    assert np.array_equal(send_head.cpu().numpy(), g["send_head"])
    assert np.array_equal(bits16(recv_x).reshape(-1, H), g["recv_x"])
    assert np.array_equal(recv_idx.cpu().numpy(), g["recv_topk_idx"])
    assert np.array_equal(recv_w.cpu().numpy(), g["recv_topk_weights"])
    assert np.array_equal(meta.cpu().numpy(), g["recv_src_meta"])
    comb, comb_w, _ = buf.ht_combine(recv_x, handle, topk_weights=recv_w, bias=(bf(g["bias0"]), bf(g["bias1"])))
    assert np.array_equal(bits16(comb).reshape(R, T, H), g["combined"])
    assert np.array_equal(comb_w.cpu().numpy(), g["combined_topk_weights"])


@pytest.mark.parametrize("shape", [(64, 3, 512, 2, 128, 4), (2, 1, 8192, 16, 32, 1), (16, 64, 1024, 6, 48, 64), (1, 40, 512, 4, 8, 64),
                                   (3, 300, 512, 5, 12, 320), (80, 65, 512, 2, 160, 65)])
def test_ll_wide_and_narrow_worlds(cuda, shape):
    """Many ranks with few tokens, the largest hidden size and top-k, one rank alone:
    dispatch (fp8 and bf16) and combine against the oracle."""
    R, T, H, K, E, M = shape
    x, topk, w = make_world(R * 7 + K, R, T, H, K, E, drop=0.05, scale=2.0)
    for use_fp8 in (True, False):
        rc, got = raw_ll_dispatch(cuda, x, topk, E, M, use_fp8)
        assert rc == 0, _lib.kernels_error()
        assert_dispatch_equal(got, eo.ll_dispatch(bits16(x).reshape(R, T, H), topk, E, M, use_fp8, fill=0x55), use_fp8)
    buf = Buffer(R, device=cuda)
    td, wd = torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
    rx, cnt, handle, _, _ = buf.dispatch(x.to(cuda), td, M, E, use_fp8=False)
    valid = (torch.arange(R * M, device=cuda).view(1, 1, -1) < cnt.unsqueeze(-1)).unsqueeze(-1)
    y = torch.where(valid, rx, torch.zeros_like(rx))
    out, _, _ = buf.combine(y, td, wd, handle)
    torch.cuda.synchronize()
    want = eo.ll_combine(bits16(y).reshape(R, E // R, R * M, H), topk, w, handle[0].cpu().numpy(), handle[1].cpu().numpy(),
                         E, M, use_fma=True)
    assert np.array_equal(bits16(out).reshape(R, T, H), want)


def test_zero_copy_combine_and_connection_calls(cuda):
    """get_next_combine_buffer + combine(zero_copy=True) equals combine on a caller tensor;
    disconnect_ranks / connect_ranks drive the mask the way update_mask_buffer does."""
    R, T, H, K, E, M = 4, 10, 512, 3, 8, 16
    x, topk, w = make_world(77, R, T, H, K, E, drop=0.0)
    buf = Buffer(R, device=cuda)
    td, wd = torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
    rx, cnt, handle, _, _ = buf.dispatch(x.to(cuda), td, M, E, use_fp8=False)
    valid = (torch.arange(R * M, device=cuda).view(1, 1, -1) < cnt.unsqueeze(-1)).unsqueeze(-1)
    y = torch.where(valid, rx, torch.zeros_like(rx))
    want, _, _ = buf.combine(y, td, wd, handle)
    with pytest.raises(EPError):
        Buffer(R, device=cuda).combine(y, td, wd, handle, zero_copy=True)
    staging = buf.get_next_combine_buffer(handle)
    assert staging.shape == rx.shape and staging.dtype == torch.bfloat16
    staging.copy_(y)
    got, _, _ = buf.combine(torch.empty(0, device=cuda), td, wd, handle, zero_copy=True)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))

    buf.disconnect_ranks([2])
    status = torch.zeros(R, dtype=torch.int32, device=cuda)
    buf.query_mask_buffer(status)
    assert status.tolist() == [0, 0, 1, 0]
    _, cnt_masked, _, _, _ = buf.dispatch(x.to(cuda), td, M, E, use_fp8=False)
    assert int(cnt_masked[2].sum()) == 0
    buf.connect_ranks([2], activate=False)
    buf.query_mask_buffer(status)
    assert status.tolist() == [0, 0, 1, 0]
    buf.connect_ranks([2])
    _, cnt_again, _, _, _ = buf.dispatch(x.to(cuda), td, M, E, use_fp8=False)
    assert torch.equal(cnt_again, cnt)
    with pytest.raises(EPError):
        buf.connect_ranks([R])
    buf.barrier()
    buf.destroy()


def test_ll_calls_can_be_captured_in_a_graph(cuda):
    """Dispatch and combine allocate nothing and clear nothing with memset nodes (the caller
    brings outputs and workspace), so both can be recorded into one HIP graph.  Every replay,
    with eager work and synchronisation in between and outputs wiped, must equal the eager
    result."""
    R, T, H, K, E, M = 4, 32, 1024, 4, 16, 32
    El, N = E // R, R * M
    x, topk, w = make_world(91, R, T, H, K, E, drop=0.05)
    k = _lib.ep_kernels()
    xd, td, wd = x.to(cuda), torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
    recv_x = torch.zeros((R, El, N, H), dtype=torch.uint8, device=cuda)
    scales = torch.zeros((R, El, H // 128, N), dtype=torch.float32, device=cuda)
    src_info = torch.zeros((R, El, N), dtype=torch.int32, device=cuda)
    layout = torch.zeros((R, El, R), dtype=torch.int64, device=cuda)
    count = torch.zeros((R, El), dtype=torch.int32, device=cuda)
    row_map = torch.zeros((R, T, K), dtype=torch.int32, device=cuda)
    ws = torch.empty(k.nixl_amd_ep_ll_workspace_bytes(R, E, T, K, H), dtype=torch.uint8, device=cuda)
    y = torch.from_numpy(np.random.default_rng(5).standard_normal((R, El, N, H)).astype(np.float32)).to(torch.bfloat16).to(cuda)
    out = torch.zeros((R, T, H), dtype=torch.bfloat16, device=cuda)
    p = lambda t: ctypes.c_void_p(t.data_ptr())

    def both(stream):
        s = ctypes.c_void_p(stream)
        assert k.nixl_amd_ep_ll_dispatch(p(recv_x), p(scales), p(src_info), p(layout), p(count), None, None, p(xd), p(td), None,
                                         T, H, M, K, R, E, 1, 0, 0, p(row_map), p(ws), ws.numel(), s) == 0, _lib.kernels_error()
        assert k.nixl_amd_ep_ll_combine(p(out), p(y), p(td), p(wd), p(src_info), p(layout), None, None, p(row_map), T, H, M, K, R,
                                        E, 0, s) == 0, _lib.kernels_error()

    both(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    want = [t.clone() for t in (recv_x, scales, src_info, layout, count, row_map, out)]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=torch.cuda.Stream()):
        both(torch.cuda.current_stream().cuda_stream)
    for i in range(3):
        for t in (layout, count, row_map, out):
            t.zero_()
        (xd.float().sum() + i).item()  # eager work and a synchronisation between replays
        graph.replay()
        torch.cuda.synchronize()
        valid = torch.arange(N, device=cuda).view(1, 1, -1) < count.unsqueeze(-1)
        assert torch.equal(layout, want[3]) and torch.equal(count, want[4]) and torch.equal(row_map, want[5])
        assert torch.equal(out.view(torch.int16), want[6].view(torch.int16))
        assert torch.equal(recv_x[valid], want[0][valid]) and torch.equal(src_info[valid], want[2][valid])


def test_ll_combine_logfmt(cuda):
    """LogFMT-10 rows: against the CPU restatement (same formulas, libm instead of the GPU's
    log2 / exp2, so a magnitude may land on the neighbouring code: at most one step of
    2^(32/510) per term), and the reference test's own criterion for identity experts
    (calc_diff < 1e-5, examples/device/ep/tests/elastic/elastic.py:377-387) on its own kind of
    input (small random values, which are cast, mixed with values >= 1, which are not)."""
    R, T, H, K, E, M = 4, 24, 1024, 4, 16, 32
    El = E // R
    rng = np.random.default_rng(61)
    xs = rng.standard_normal((R, T, H)).astype(np.float32) * 0.5 * rng.random((R, T, 1)).astype(np.float32)
    xs[:, ::5, :256] *= 8.0  # some groups at or above 1: left as bf16
    xs[:, 1::7, 300:340] = 0.0
    x = torch.from_numpy(xs).to(torch.bfloat16)
    topk = np.stack([np.stack([rng.permutation(E)[:K] for _ in range(T)]) for _ in range(R)]).astype(np.int32)
    topk[rng.random((R, T, K)) < 0.1] = -1
    w = rng.random((R, T, K)).astype(np.float32)
    buf = Buffer(R, device=cuda)
    td, wd = torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
    rx, cnt, handle, _, _ = buf.dispatch(x.to(cuda), td, M, E, use_fp8=False)
    valid = (torch.arange(R * M, device=cuda).view(1, 1, -1) < cnt.unsqueeze(-1)).unsqueeze(-1)
    y = torch.where(valid, rx, torch.zeros_like(rx))
    out, _, _ = buf.combine(y, td, wd, handle, use_logfmt=True)
    plain, _, _ = buf.combine(y, td, wd, handle)
    torch.cuda.synchronize()
    again, _, _ = buf.combine(y, td, wd, handle, use_logfmt=True)
    assert torch.equal(out.view(torch.int16), again.view(torch.int16))  # deterministic on one GPU
    want = eo.ll_combine(bits16(y).reshape(R, El, R * M, H), topk, w, handle[0].cpu().numpy(), handle[1].cpu().numpy(), E, M,
                         use_logfmt=True)
    g, o = eo.bf16_to_f32(bits16(out).reshape(R, T, H)), eo.bf16_to_f32(want)
    assert np.mean(g == o) > 0.98
    scale = np.abs(xs).max(axis=2, keepdims=True) * np.abs(w).sum(axis=2, keepdims=True)
    assert np.all(np.abs(g - o) <= (2.0 ** (32 / 510) - 1) * scale + 1e-6)
    # lossy but close to the uncompressed sum, and not identical to it
    p = eo.bf16_to_f32(bits16(plain).reshape(R, T, H))
    assert not np.array_equal(g, p)
    assert calc_diff(torch.from_numpy(g), torch.from_numpy(p)) < 1e-5
    ideal = x.float().numpy() * np.where(topk >= 0, w, 0).sum(axis=2, keepdims=True)
    assert calc_diff(torch.from_numpy(g), torch.from_numpy(ideal)) < 1e-5


def test_ll_narrow_workgroups_give_the_same_bytes(cuda):
    """nixl_amd_ep_ll_set_tuning: with workgroups of 64 and 128 lanes a token's row is split
    over several workgroups in dispatch and combine; results must not change."""
    k = _lib.ep_kernels()
    R, T, H, K, E, M = 4, 9, 2048, 4, 8, 12
    x, topk, w = make_world(123, R, T, H, K, E, drop=0.1, scale=2.0)
    want = eo.ll_dispatch(bits16(x).reshape(R, T, H), topk, E, M, True, fill=0x55)
    try:
        assert k.nixl_amd_ep_ll_set_tuning(100, 0) < 0 and k.nixl_amd_ep_ll_set_tuning(0, 2048) < 0
        for lanes in (64, 128, 1024):
            assert k.nixl_amd_ep_ll_set_tuning(lanes, lanes) == 0
            rc, got = raw_ll_dispatch(cuda, x, topk, E, M, True)
            assert rc == 0, _lib.kernels_error()
            assert_dispatch_equal(got, want, True)
            buf = Buffer(R, device=cuda)
            td, wd = torch.from_numpy(topk).to(cuda), torch.from_numpy(w).to(cuda)
            rx, cnt, handle, _, _ = buf.dispatch(x.to(cuda), td, M, E, use_fp8=False)
            valid = (torch.arange(R * M, device=cuda).view(1, 1, -1) < cnt.unsqueeze(-1)).unsqueeze(-1)
            y = torch.where(valid, rx, torch.zeros_like(rx))
            for h in (handle, tuple(handle)):
                for logfmt in (False, True):
                    out, _, _ = buf.combine(y, td, wd, h, use_logfmt=logfmt)
                    torch.cuda.synchronize()
                    ref = eo.ll_combine(bits16(y).reshape(R, E // R, R * M, H), topk, w, handle[0].cpu().numpy(),
                                        handle[1].cpu().numpy(), E, M, use_fma=True, use_logfmt=logfmt)
                    if logfmt:
                        assert np.mean(bits16(out).reshape(R, T, H) == ref) > 0.98
                    else:
                        assert np.array_equal(bits16(out).reshape(R, T, H), ref)
    finally:
        assert k.nixl_amd_ep_ll_set_tuning(-1, -1) == 0  # back to the built-in choice
