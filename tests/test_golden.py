"""The oracle against the committed golden vectors (tests/golden/*.npz, written by
tests/golden/make_fixtures.py from torch-CPU library routines and plain loops that never
touch the oracle).  The GPU tests compare the HIP path with the same files."""
import os

import numpy as np
import pytest

from oracle import ep_oracle as eo
from oracle import kv_oracle as ko

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def test_e4m3_encoder_golden():
    g = load("e4m3_encode.npz")
    assert np.array_equal(eo.f32_to_e4m3(g["values"]), g["codes"])
    assert np.array_equal(eo.f32_to_e4m3(g["sat_values"]), g["sat_codes"])


def test_router_golden():
    g = load("router.npz")
    idx, w = eo.router(g["logits"], g["topk_idx"].shape[1])
    assert np.array_equal(idx, g["topk_idx"])
    assert np.allclose(w, g["topk_weights"], rtol=2e-6, atol=0)


def check_ll_dispatch(got, g, use_fp8):
    """Rows at or beyond recv_count are unspecified; everything before must match."""
    assert np.array_equal(got["recv_count"], g["recv_count"])
    assert np.array_equal(got["layout_range"], g["layout_range"])
    R, El = g["recv_count"].shape
    want_x = g["recv_fp8"] if use_fp8 else g["recv_bf16"]
    for d in range(R):
        for le in range(El):
            n = int(g["recv_count"][d, le])
            assert np.array_equal(got["recv_x"][d, le, :n], want_x[d, le, :n])
            assert np.array_equal(got["src_info"][d, le, :n], g["src_info"][d, le, :n])
            if use_fp8:
                assert np.array_equal(got["scales"][d, le, :, :n].view(np.uint32), g["scales"][d, le, :, :n].view(np.uint32))


# ll_world_repeats.npz: some tokens name one expert two or three times and get a row per
# selection (kernels/nixl_ep_ll.cu:186-190)
@pytest.mark.parametrize("world", ["ll_world.npz", "ll_world_repeats.npz"])
def test_ll_dispatch_golden(world):
    g = load(world)
    E, M = int(g["num_experts"]), int(g["max_tok"])
    for use_fp8 in (True, False):
        got = eo.ll_dispatch(g["x"], g["topk_idx"], E, M, use_fp8=use_fp8, num_tokens=g["num_tokens"])
        check_ll_dispatch(got, g, use_fp8)


@pytest.mark.parametrize("world", ["ll_world.npz", "ll_world_repeats.npz"])
def test_ll_combine_golden(world):
    g = load(world)
    E, M = int(g["num_experts"]), int(g["max_tok"])
    out = eo.ll_combine(g["expert_out"], g["topk_idx"], g["topk_weights"], g["src_info"], g["layout_range"], E, M,
                        num_tokens=g["num_tokens"], use_fma=True)
    for r, n in enumerate(g["num_tokens"]):
        assert np.array_equal(out[r, :n], g["combined"][r, :n])


def test_ht_golden():
    g = load("ht_world.npz")
    R, T, K = g["topk_idx"].shape
    E, C = int(g["num_experts"]), int(g["num_channels"])
    lay = [eo.dispatch_layout(g["topk_idx"][r], R, E) for r in range(R)]
    assert np.array_equal(np.stack([l[0] for l in lay]), g["per_rank"])
    assert np.array_equal(np.stack([l[1] for l in lay]), g["per_expert"])
    assert np.array_equal(np.stack([l[2] for l in lay]), g["in_rank"])
    prefix, counts, chan = eo.ht_notify(g["in_rank"], g["per_expert"], C, 1)
    assert np.array_equal(prefix, g["prefix"])
    assert np.array_equal(counts, g["expert_count"])
    assert np.array_equal(chan, g["channel_prefix"])
    o = eo.ht_dispatch(g["x"], g["topk_idx"], g["topk_weights"], g["in_rank"], prefix, E)
    assert np.array_equal(o["row_offset"], g["row_offset"])
    assert np.array_equal(o["recv_x"], g["recv_x"])
    assert np.array_equal(o["recv_topk_idx"], g["recv_topk_idx"])
    assert np.array_equal(o["recv_topk_weights"], g["recv_topk_weights"])
    assert np.array_equal(np.stack([o["recv_src_rank"], o["recv_src_token"]], 1), g["recv_src_meta"])
    assert np.array_equal(o["send_head"], g["send_head"])
    comb, comb_w = eo.ht_combine(g["recv_x"], g["recv_topk_weights"], g["in_rank"], prefix, g["send_head"],
                                 g["row_offset"], g["bias0"], g["bias1"])
    assert np.array_equal(comb, g["combined"])
    assert np.array_equal(comb_w, g["combined_topk_weights"])


def test_kv_copy_golden():
    g = load("kv_descs.npz")
    size = g["src"].size
    mem = np.concatenate([g["src"], np.full(size, g["canary"], np.uint8)])
    ko.copy_descs(mem, g["src_off"], g["dst_off"] + np.uint64(size), g["lens"])
    assert np.array_equal(mem[size:], g["dst"])
    assert np.array_equal(mem[:size], g["src"])
