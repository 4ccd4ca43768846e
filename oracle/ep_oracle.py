"""TEST INFRASTRUCTURE — numpy front end of the scalar C oracle for the expert-parallel
kernels (oracle/ep_oracle.c, built into oracle/_build/liboracle.so).  Only tests, the smoke
check and the CPU-baseline leg of the benchmark import this."""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_P = ctypes.c_void_p
_I = ctypes.c_int


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "_build", "liboracle.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} missing: run __graft_entry__.build() or `make -C oracle`")
        L = ctypes.CDLL(path)
        L.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_bf16_to_f32.restype = ctypes.c_float
        L.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.oracle_f32_to_e4m3.argtypes = [ctypes.c_float]
        L.oracle_f32_to_e4m3.restype = ctypes.c_uint8
        L.oracle_e4m3_to_f32.argtypes = [ctypes.c_uint8]
        L.oracle_e4m3_to_f32.restype = ctypes.c_float
        L.oracle_fp8_scales.argtypes = [ctypes.c_float, _I, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float)]
        L.oracle_cast_row_fp8.argtypes = [_P, _I, _I, _P, _P]
        L.oracle_f32_to_e4m3_n.argtypes = [_P, _P, ctypes.c_size_t]
        L.oracle_f32_to_bf16_n.argtypes = [_P, _P, ctypes.c_size_t]
        L.oracle_ll_dispatch.argtypes = [_P, _P, _P, _P] + [_I] * 9 + [_P] * 5 + [_I]
        L.oracle_ll_dispatch.restype = _I
        L.oracle_ll_combine.argtypes = [_P] * 7 + [_I] * 7 + [_P, _I]
        L.oracle_ll_combine.restype = _I
        L.oracle_weighted_sum_rows.argtypes = [_P, _P, _I, _I, _I, _P]
        L.oracle_dispatch_layout.argtypes = [_P, _I, _I, _I, _I, _P, _P, _P]
        L.oracle_ht_notify.argtypes = [_P, _P, _I, _I, _I, _I, _I, _P, _P, _P]
        L.oracle_ht_dispatch.argtypes = [_P] * 5 + [_I] * 5 + [_P] * 7
        L.oracle_ht_combine.argtypes = [_P] * 8 + [_I] * 4 + [_P, _P]
        L.oracle_router.argtypes = [_P, _I, _I, _I, _P, _P]
        L.oracle_logfmt_roundtrip.argtypes = [_P, _I, _P]
        _LIB = L
    return _LIB


def _p(a):
    return None if a is None else a.ctypes.data


def _c(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


# ---- scalar formats ------------------------------------------------------------------------

def f32_to_bf16(a):
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().oracle_f32_to_bf16_n(_p(a), _p(out), a.size)
    return out


def bf16_to_f32(a):
    return (np.asarray(a, np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_e4m3(a):
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.uint8)
    lib().oracle_f32_to_e4m3_n(_p(a), _p(out), a.size)
    return out


def e4m3_to_f32(codes):
    table = np.array([lib().oracle_e4m3_to_f32(i) for i in range(256)], np.float32)
    return table[np.asarray(codes, np.uint8)]


def fp8_scales(amax, round_scale=False):
    s, si = ctypes.c_float(), ctypes.c_float()
    lib().oracle_fp8_scales(float(amax), int(round_scale), ctypes.byref(s), ctypes.byref(si))
    return s.value, si.value


def cast_row_fp8(row_bf16, round_scale=False):
    row = _c(row_bf16, np.uint16)
    q = np.empty(row.size, np.uint8)
    sc = np.empty(row.size // 128, np.float32)
    lib().oracle_cast_row_fp8(_p(row), row.size, int(round_scale), _p(q), _p(sc))
    return q, sc


# ---- low-latency mode ------------------------------------------------------------------------

def ll_dispatch(x, topk_idx, num_experts, max_tok, use_fp8=True, round_scale=False, use_ue8m0=False,
                num_tokens=None, mask=None, threads=1, fill=0):
    """x [R,T,H] uint16 (bf16 bits), topk_idx [R,T,K] int32.  Returns a dict of outputs;
    rows beyond recv_count keep the value `fill` (fill=None: they are not initialised at all)."""
    x = _c(x, np.uint16)
    topk_idx = _c(topk_idx, np.int32)
    R, T, H = x.shape
    K = topk_idx.shape[2]
    El, N = num_experts // R, R * max_tok
    def filled(shape, dtype):  # every byte = fill; fill=None leaves the memory as allocated (untouched pages)
        if fill is None:
            return np.empty(shape, dtype)
        return np.full(int(np.prod(shape)) * np.dtype(dtype).itemsize, fill, np.uint8).view(dtype).reshape(shape)

    recv_x = filled((R, El, N, H), np.uint8 if use_fp8 else np.uint16)
    scales = None
    if use_fp8:
        scales = filled((R, El, H // 512, N), np.int32) if use_ue8m0 else filled((R, El, H // 128, N), np.float32)
    src_info = filled((R, El, N), np.int32)
    layout_range = np.zeros((R, El, R), np.int64)
    recv_count = np.zeros((R, El), np.int32)
    nt, mk = _c(num_tokens, np.int32), _c(mask, np.int32)
    rc = lib().oracle_ll_dispatch(_p(x), _p(topk_idx), _p(nt), _p(mk), R, T, H, K, num_experts, max_tok,
                                  int(use_fp8), int(round_scale), int(use_ue8m0), _p(recv_x), _p(scales),
                                  _p(src_info), _p(layout_range), _p(recv_count), threads)
    if rc != 0:
        raise ValueError(f"oracle_ll_dispatch rejected the arguments ({rc})")
    return dict(recv_x=recv_x, scales=scales, src_info=src_info, layout_range=layout_range, recv_count=recv_count)


def logfmt_roundtrip(row):
    """row [H] bf16 bits -> fp32 [H]: what a LogFMT-10 encoded row decodes to."""
    row = _c(row, np.uint16)
    out = np.zeros(row.shape[-1], np.float32)
    lib().oracle_logfmt_roundtrip(_p(row), row.shape[-1], _p(out))
    return out


def ll_combine(expert_out, topk_idx, topk_weights, src_info, layout_range, num_experts, max_tok,
               num_tokens=None, mask=None, use_fma=True, threads=1, use_logfmt=False):
    expert_out = _c(expert_out, np.uint16)
    topk_idx = _c(topk_idx, np.int32)
    topk_weights = _c(topk_weights, np.float32)
    src_info = _c(src_info, np.int32)
    layout_range = _c(layout_range, np.int64)
    R, T, K = topk_idx.shape
    H = expert_out.shape[-1]
    out = np.zeros((R, T, H), np.uint16)
    nt, mk = _c(num_tokens, np.int32), _c(mask, np.int32)
    rc = lib().oracle_ll_combine(_p(expert_out), _p(topk_idx), _p(topk_weights), _p(src_info), _p(layout_range),
                                 _p(nt), _p(mk), R, T, H, K, num_experts, max_tok, int(use_fma) | (int(use_logfmt) << 1), _p(out), threads)
    if rc != 0:
        raise ValueError(f"oracle_ll_combine rejected the arguments ({rc})")
    return out


def weighted_sum_rows(rows, weights, use_fma=True):
    """rows [K,H] bf16 bits, weights [K] -> bf16 bits [H] of sum_k rows[k] * weights[k]."""
    rows = _c(rows, np.uint16)
    weights = _c(weights, np.float32)
    out = np.zeros(rows.shape[1], np.uint16)
    lib().oracle_weighted_sum_rows(_p(rows), _p(weights), rows.shape[0], rows.shape[1], int(use_fma), _p(out))
    return out


# ---- normal mode -------------------------------------------------------------------------------

def dispatch_layout(topk_idx, num_ranks, num_experts):
    topk_idx = _c(topk_idx, np.int32)
    T, K = topk_idx.shape
    per_rank = np.zeros(num_ranks, np.int32)
    per_expert = np.zeros(num_experts, np.int32)
    in_rank = np.zeros((T, num_ranks), np.uint8)
    lib().oracle_dispatch_layout(_p(topk_idx), T, K, num_ranks, num_experts, _p(per_rank), _p(per_expert), _p(in_rank))
    return per_rank, per_expert, in_rank


def ht_notify(is_token_in_rank, per_expert, num_channels, expert_alignment=1):
    in_rank = _c(is_token_in_rank, np.uint8)
    per_expert = _c(per_expert, np.int32)
    R, T, _ = in_rank.shape
    E = per_expert.shape[1]
    prefix = np.zeros((R, R), np.int32)
    counts = np.zeros((R, E // R), np.int32)
    chan = np.zeros((R, R, num_channels), np.int32)
    lib().oracle_ht_notify(_p(in_rank), _p(per_expert), R, T, E, num_channels, expert_alignment, _p(prefix),
                           _p(counts), _p(chan))
    return prefix, counts, chan


def ht_dispatch(x, topk_idx, topk_weights, is_token_in_rank, recv_rank_prefix, num_experts):
    x = _c(x, np.uint16)
    topk_idx = _c(topk_idx, np.int32)
    topk_weights = _c(topk_weights, np.float32)
    in_rank = _c(is_token_in_rank, np.uint8)
    prefix = _c(recv_rank_prefix, np.int32)
    R, T, H = x.shape
    K = topk_idx.shape[2]
    row_offset = np.concatenate([[0], np.cumsum(prefix[:, -1].astype(np.int64))]).astype(np.int64)
    total = int(row_offset[-1])
    out = dict(row_offset=row_offset,
               recv_x=np.zeros((total, H), np.uint16), recv_topk_idx=np.zeros((total, K), np.int32),
               recv_topk_weights=np.zeros((total, K), np.float32), recv_src_rank=np.zeros(total, np.int32),
               recv_src_token=np.zeros(total, np.int32), send_head=np.zeros((R, T, R), np.int32))
    lib().oracle_ht_dispatch(_p(x), _p(topk_idx), _p(topk_weights), _p(in_rank), _p(prefix), R, T, H, K, num_experts,
                             _p(row_offset), _p(out["recv_x"]), _p(out["recv_topk_idx"]),
                             _p(out["recv_topk_weights"]), _p(out["recv_src_rank"]), _p(out["recv_src_token"]),
                             _p(out["send_head"]))
    return out


def ht_combine(recv_x, recv_topk_weights, is_token_in_rank, recv_rank_prefix, send_head, row_offset,
               bias0=None, bias1=None):
    recv_x = _c(recv_x, np.uint16)
    w = _c(recv_topk_weights, np.float32)
    in_rank = _c(is_token_in_rank, np.uint8)
    prefix = _c(recv_rank_prefix, np.int32)
    send_head = _c(send_head, np.int32)
    row_offset = _c(row_offset, np.int64)
    R, T, _ = in_rank.shape
    H = recv_x.shape[1]
    K = w.shape[1] if w is not None else 0
    combined = np.zeros((R, T, H), np.uint16)
    wsum = np.zeros((R, T, max(K, 1)), np.float32)
    b0, b1 = _c(bias0, np.uint16), _c(bias1, np.uint16)
    lib().oracle_ht_combine(_p(recv_x), _p(w), _p(in_rank), _p(prefix), _p(send_head), _p(row_offset), _p(b0),
                            _p(b1), R, T, H, K, _p(combined), _p(wsum))
    return combined, wsum[:, :, :K]


def router(logits, k):
    logits = _c(logits, np.float32)
    T, E = logits.shape
    idx = np.zeros((T, k), np.int32)
    w = np.zeros((T, k), np.float32)
    lib().oracle_router(_p(logits), T, E, k, _p(idx), _p(w))
    return idx, w
