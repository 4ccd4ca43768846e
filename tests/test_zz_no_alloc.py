"""The low-latency dispatch entry point that allocates nothing
(nixl_amd_ep_ll_dispatch_static, scratch in a fixed device array inside the library) against
nixl_amd_ep_ll_dispatch with a caller-supplied workspace: identical bytes in every output, on
two calls in a row of which the second is smaller, so that what the first call left in the
shared scratch is seen not to leak into the second."""
import ctypes

import numpy as np
import pytest
import torch

from nixl_amd import _lib

pytestmark = pytest.mark.gpu

STATIC_BYTES = 2 << 20  # NIXL_AMD_EP_LL_STATIC_SCRATCH_BYTES


def _world(seed, R, T, H, K, E):
    rng = np.random.default_rng(seed)
    x = torch.from_numpy(rng.standard_normal((R, T, H)).astype(np.float32) * 2.0).to(torch.bfloat16)
    topk = np.argsort(-rng.standard_normal((R, T, E)), axis=2)[:, :, :K].astype(np.int32)
    topk[rng.random((R, T, K)) < 0.1] = -1
    return x, topk


def _dispatch(cuda, x, topk, E, M, use_fp8, static, fill=0x55):
    k = _lib.ep_kernels()
    R, T, H = x.shape
    K = topk.shape[2]
    El, N = E // R, R * M
    xd = x.to(cuda)
    td = torch.from_numpy(topk).to(cuda)
    out = dict(
        recv_x=torch.full((R, El, N, H * (1 if use_fp8 else 2)), fill, dtype=torch.uint8, device=cuda),
        scales=torch.full((R, El, H // 128, N, 4), fill, dtype=torch.uint8, device=cuda) if use_fp8 else None,
        src_info=torch.full((R, El, N, 4), fill, dtype=torch.uint8, device=cuda),
        layout_range=torch.zeros((R, El, R), dtype=torch.int64, device=cuda),
        recv_count=torch.zeros((R, El), dtype=torch.int32, device=cuda),
        row_map=torch.full((R, T, K), -7, dtype=torch.int32, device=cuda))
    p = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())
    head = (p(out["recv_x"]), p(out["scales"]), p(out["src_info"]), p(out["layout_range"]), p(out["recv_count"]), None,
            None, p(xd), p(td), None, T, H, M, K, R, E, int(use_fp8), 0, 0, p(out["row_map"]))
    if static:
        # Free device memory as the driver counts it: torch's own counters only see torch's
        # allocator, and a hipMalloc inside the library would not move them.  One call first,
        # outside the comparison: the first use of the scratch array may load the code object.
        rc = k.nixl_amd_ep_ll_dispatch_static(*head, None)
        torch.cuda.synchronize()
        assert rc == 0, _lib.kernels_error()
        before = torch.cuda.mem_get_info(cuda)[0]
        rc = k.nixl_amd_ep_ll_dispatch_static(*head, None)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(cuda)[0] == before, "the entry point that allocates nothing changed free device memory"
    else:
        ws = torch.empty(k.nixl_amd_ep_ll_workspace_bytes(R, E, T, K, H) + 16, dtype=torch.uint8, device=cuda)
        rc = k.nixl_amd_ep_ll_dispatch(*head, p(ws), ws.numel(), None)
    torch.cuda.synchronize()
    assert rc == 0, _lib.kernels_error()
    return {n: None if t is None else t.cpu().numpy() for n, t in out.items()}


def _assert_same(a, b):
    for name in a:
        if a[name] is None:
            assert b[name] is None
        else:
            assert np.array_equal(a[name], b[name]), name


@pytest.mark.parametrize("use_fp8", [True, False])
def test_static_dispatch_matches_workspace_dispatch_twice(cuda, use_fp8):
    # first a larger call, then a smaller one that reuses the front of the same scratch
    big = (8, 64, 2048, 8, 64, 64)
    small = (4, 12, 512, 3, 8, 16)
    for seed, (R, T, H, K, E, M) in ((3, big), (4, small)):
        x, topk = _world(seed, R, T, H, K, E)
        want = _dispatch(cuda, x, topk, E, M, use_fp8, static=False)
        got = _dispatch(cuda, x, topk, E, M, use_fp8, static=True)
        assert want["recv_count"].sum() > 0
        _assert_same(got, want)


def test_static_dispatch_at_the_low_latency_configuration(cuda):
    """32 ranks x 128 tokens x 7168, 256 experts, top-8, fp8 (BASELINE config 4): 1.0 MiB of the
    2 MiB scratch array; every output equal to the workspace call's."""
    R, T, H, K, E, M = 32, 128, 7168, 8, 256, 128
    assert _lib.ep_kernels().nixl_amd_ep_ll_workspace_bytes(R, E, T, K, H) <= STATIC_BYTES
    x, topk = _world(5, R, T, H, K, E)
    want = _dispatch(cuda, x, topk, E, M, True, static=False)
    got = _dispatch(cuda, x, topk, E, M, True, static=True)
    assert want["recv_count"].sum() == (topk >= 0).sum()
    _assert_same(got, want)


def test_static_dispatch_refuses_what_does_not_fit(cuda):
    k = _lib.ep_kernels()
    R, T, H, K, E, M = 32, 1024, 7168, 8, 256, 1024
    assert k.nixl_amd_ep_ll_workspace_bytes(R, E, T, K, H) > STATIC_BYTES
    one = torch.zeros(16, dtype=torch.uint8, device=cuda)  # never touched: the call is refused on the host
    p = ctypes.c_void_p(one.data_ptr())
    rc = k.nixl_amd_ep_ll_dispatch_static(p, p, p, p, p, None, None, p, p, None, T, H, M, K, R, E, 1, 0, 0, None, None)
    assert rc == -5, rc  # NIXL_AMD_ERR_TOO_LARGE
    assert "scratch" in _lib.kernels_error()
    torch.cuda.synchronize()
