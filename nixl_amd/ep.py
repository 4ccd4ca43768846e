"""Host side of the expert-parallel path: a ``Buffer`` shaped after the reference's
``nixl_ep.Buffer`` (examples/device/ep/nixl_ep/buffer.py:43-886) for a world of virtual
ranks that all live in one GPU's HBM.

Where the reference runs one process per rank and every call handles that rank's tensors,
one ``Buffer`` here stands for the whole world and every tensor carries a leading rank
dimension: ``x`` is ``[R, T, H]`` where the reference takes ``[T, H]``, ``packed_recv_x`` is
``[R, El, N, H]`` where the reference returns ``[El, N, H]``, and so on; slice with ``[r]``
to get exactly what rank ``r`` of the reference would see.  Method names, argument order,
argument meaning and the tuple shapes of the return values are the reference's.  torch
only owns the memory and the stream; all work is done by the HIP kernels behind
include/nixl_amd_ep.h, and nothing here falls back to torch ops.
"""
import ctypes
import time

import numpy as np
import torch

from . import _lib

topk_idx_t = torch.int32  # reference default, csrc/kernels/configs.cuh:79-85


class EPError(RuntimeError):
    """Host-side argument or launch failure (the reference raises EPException,
    csrc/kernels/exception.cuh:34-60)."""


class EventOverlap:
    """Reference: nixl_ep/utils.py:30-70.  Work is enqueued on the current stream, so the
    event is simply recorded there."""

    def __init__(self, event=None, extra_tensors=None):
        self.event = event
        self.extra_tensors = extra_tensors

    def current_stream_wait(self):
        if self.event is not None:
            torch.cuda.current_stream().wait_event(self.event)


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(rc, what):
    if rc != 0:
        raise EPError(f"{what}: {_lib.kernels_error()} (status {rc})")


class Config:
    """The reference's normal-mode tuning record (nixl_ep_cpp.Config: SM count plus chunk sizes
    of its NVLink and RDMA staging queues).  There are no staging queues here; only num_sms
    keeps a meaning: num_sms / 2 is the number of channels the per-channel prefix matrix of
    the dispatch handle is cut into (csrc/nixl_ep.cpp:630)."""

    def __init__(self, num_sms=20, num_max_nvl_chunked_send_tokens=6, num_max_nvl_chunked_recv_tokens=256,
                 num_max_rdma_chunked_send_tokens=6, num_max_rdma_chunked_recv_tokens=256):
        # names and defaults of csrc/nixl_ep.cpp:1502-1506
        if num_sms <= 0 or num_sms % 2:
            raise EPError("the SM count must be positive and even")
        self.num_sms = int(num_sms)
        self.chunk_sizes = (num_max_nvl_chunked_send_tokens, num_max_nvl_chunked_recv_tokens,
                            num_max_rdma_chunked_send_tokens, num_max_rdma_chunked_recv_tokens)  # accepted, unused


class DispatchHandle(tuple):
    """The reference's dispatch handle (src_info, layout_range, num_max_dispatch_tokens_per_rank,
    hidden) (nixl_ep/buffer.py:415-420), plus the row map the dispatch kernel recorded, which
    lets combine skip its search.  A plain 4-tuple built by the caller works as well."""

    row_map = None


class Buffer:
    """All virtual ranks of one expert-parallel job on one GPU.

    Reference constructor: Buffer(rank, low_latency_mode, explicitly_destroy, ...)
    (nixl_ep/buffer.py:60-120); there is no rank argument here because the object holds
    every rank, and no RDMA buffer sizing because no staging buffers exist.
    """

    num_sms = 20  # reference default (buffer.py:54); see Config

    @staticmethod
    def set_num_sms(new_num_sms):
        """Reference: buffer.py:116-126."""
        if new_num_sms <= 0 or new_num_sms % 2:
            raise EPError("the SM count must be positive and even")
        Buffer.num_sms = int(new_num_sms)

    @staticmethod
    def get_dispatch_config(num_ranks):
        """Reference: buffer.py:221-247 (a table of queue chunk sizes per rank count, which
        have no counterpart here)."""
        return Config(Buffer.num_sms)

    @staticmethod
    def get_combine_config(num_ranks):
        """Reference: buffer.py:249-275."""
        return Config(Buffer.num_sms)

    def __init__(self, num_ranks, low_latency_mode=True, device="cuda:0", timeout_ms=None):
        """timeout_ms (reference: buffer.py:65,80-83; 30 s there): budget of the receive side's
        bounded waits in low-latency mode.  None (the default here) leaves the waits out: on
        one GPU every rank's data is in place before a receiver looks, so they only matter to
        callers that exercise the time-out -> mask path."""
        self.num_ranks = int(num_ranks)
        self.low_latency_mode = low_latency_mode
        self.device = torch.device(device)
        self.timeout_ms = timeout_ms
        # Fault injection for tests of that path: this rank's send phase leaves out the word
        # its receivers wait for, so that their wait runs out (one-shot knob, -1 = off).
        self.withhold_rank = -1
        self._k = _lib.ep_kernels()
        self.mask_buffer = torch.zeros((self.num_ranks, self.num_ranks), dtype=torch.int32, device=self.device)
        self._mask_active = False
        self._workspace = None
        # Normal-mode dispatch sizes its receive tensors for the worst case, and so avoids
        # waiting for the counts before it launches, while that takes no more than this.
        self.ht_recv_worst_case_limit = 16 << 30
        self.cpu_timeout_secs = 100  # NUM_CPU_TIMEOUT_SECS, csrc/kernels/configs.cuh

    # -- life cycle and sizing helpers kept for callers written against the reference ------
    def is_available(self):
        """Reference: csrc/nixl_ep.cpp Buffer::is_available: usable until destroy()."""
        return self.mask_buffer is not None

    def get_local_device_id(self):
        return self.device.index or 0

    # one GPU holds every rank: a single "RDMA rank" (node), reference csrc/nixl_ep.cpp:84-101
    def get_num_rdma_ranks(self):
        return 1

    def get_rdma_rank(self):
        return 0

    def get_root_rdma_rank(self, global_):
        return 0

    def destroy(self):
        """Reference: buffer.py:103-110.  Drops the device buffers this object owns."""
        self.mask_buffer = None
        self._workspace = None
        self._combine_buffer = None

    @staticmethod
    def capture():
        """Reference: buffer.py:129-136: an event on the current stream."""
        event = torch.cuda.Event()
        event.record()
        return EventOverlap(event)

    def get_comm_stream(self):
        """Reference: buffer.py:174-186.  The kernels run on the caller's current stream."""
        return torch.cuda.current_stream(self.device)

    @staticmethod
    def get_low_latency_buffer_size_hint(num_max_dispatch_tokens_per_rank, hidden, num_ranks, num_experts):
        """Bytes of RDMA staging per rank the reference would ask for (EPLayout,
        csrc/config.hpp:145-208): two send buffers, two receive buffers and two signalling
        buffers, rounded up past the next multiple of 128.  Nothing here allocates that
        memory (rows go straight to their final place); the figure is for callers that
        budget memory with the reference's own formula."""
        num_scales = hidden // 128
        if num_scales * 4 > hidden:
            raise EPError("hidden too small for per-128-channel scales")
        dispatch_msg = 16 + max(hidden * 2, hidden + num_scales * 4)
        combine_msg = num_scales * 4 + hidden * 2
        send = max(num_max_dispatch_tokens_per_rank * dispatch_msg,
                   num_experts * num_max_dispatch_tokens_per_rank * combine_msg)
        recv = max(num_experts * num_max_dispatch_tokens_per_rank * dispatch_msg,
                   num_experts * num_max_dispatch_tokens_per_rank * combine_msg)
        signalling = (num_experts * 8 + 127) // 128 * 128
        total = send * 2 + recv * 2 + signalling * 2
        return (total + 128) // 128 * 128

    @staticmethod
    def get_rdma_size_hint(num_max_dispatch_tokens_per_rank, hidden, num_ranks, num_experts):
        """Reference alias, buffer.py:163-172."""
        return Buffer.get_low_latency_buffer_size_hint(num_max_dispatch_tokens_per_rank, hidden, num_ranks, num_experts)

    @staticmethod
    def is_sm90_compiled():
        """Reference: buffer.py:112-114 (whether Hopper-only code paths were built)."""
        return False

    def get_local_buffer_tensor(self, dtype, size=None, offset=0, use_rdma_buffer=False):
        """Reference: buffer.py:188-209, a typed view of the rank's staging buffer.  There is
        no staging buffer here (rows are written straight to their final place), so there is
        nothing to view."""
        raise EPError("get_local_buffer_tensor: this Buffer has no staging buffer")

    def set_tcp_store_group(self, tcp_store_group):
        """Reference: buffer.py:789-797 (a store for metadata exchange between processes);
        all ranks share this process, so the store is only remembered."""
        self._tcp_store_group = tcp_store_group

    def get_next_combine_buffer(self, handle):
        """Reference: buffer.py:743-764.  A bf16 tensor shaped like the packed_recv_x of the
        dispatch that produced `handle`; experts may write their outputs into it and call
        combine(..., zero_copy=True), which then reads it instead of its `x` argument."""
        src_info, _layout_range, max_tok, hidden = handle
        R, El, N = src_info.shape
        shape = (R, El, N, hidden)
        if getattr(self, "_combine_buffer", None) is None or tuple(self._combine_buffer.shape) != shape:
            self._combine_buffer = torch.empty(shape, dtype=torch.bfloat16, device=self.device)
        return self._combine_buffer

    # Connection management of the reference (buffer.py:766-880) has nothing to do when all
    # ranks live in one process; the calls exist so that code written for it runs unchanged.
    def update_memory_buffers(self, num_ranks=None, num_experts_per_rank=None, num_rdma_bytes=0):
        if num_ranks is not None and int(num_ranks) != self.num_ranks:
            raise EPError("the number of ranks is fixed when the Buffer is created")

    def connect_ranks(self, remote_ranks, activate=True):
        for r in remote_ranks:
            if not 0 <= int(r) < self.num_ranks:
                raise EPError(f"rank {r} is outside this world of {self.num_ranks} ranks")
        for r in remote_ranks:  # activate=False keeps the new ranks masked (buffer.py:848)
            self.update_mask_buffer(int(r), not activate)

    def disconnect_ranks(self, remote_ranks):
        for r in remote_ranks:
            if not 0 <= int(r) < self.num_ranks:
                raise EPError(f"rank {r} is outside this world of {self.num_ranks} ranks")
            self.update_mask_buffer(int(r), True)

    def barrier(self):
        torch.cuda.current_stream(self.device).synchronize()

    # -- rank masks (reference: buffer.py:716-775, csrc/nixl_ep.cpp:463-549) ---------------
    def update_mask_buffer(self, rank, mask=True):
        """Mark `rank` failed (or healthy again) in every rank's view, which is the state the
        reference reaches after all survivors timed out on a dead rank."""
        v = 1 if mask else 0
        self.mask_buffer[:, rank] = v
        self.mask_buffer[rank, :] = v
        self._mask_active = bool(self.mask_buffer.any().item())

    def query_mask_buffer(self, mask_status):
        """mask_status[r] = 1 if rank r is regarded as failed by the lowest-numbered rank
        that is itself healthy (the reference returns the calling rank's own view)."""
        diag = torch.diagonal(self.mask_buffer)
        healthy = (diag == 0).nonzero()
        if healthy.numel() == 0:
            mask_status.fill_(1)
        else:
            mask_status.copy_(self.mask_buffer[int(healthy[0])].to(mask_status.dtype))

    def clean_mask_buffer(self):
        self.mask_buffer.zero_()
        self._mask_active = False

    def _mask_ptr(self):
        return _ptr(self.mask_buffer) if self._mask_active else None

    def _mapped_counts(self, n):
        """Pinned host words that the count kernel writes and the host polls, as a numpy view."""
        if getattr(self, "_mapped_tensor", None) is None or self._mapped_tensor.numel() != n:
            self._mapped_tensor = torch.empty(n, dtype=torch.int32, pin_memory=True)
            self._mapped_view = self._mapped_tensor.numpy()
        return self._mapped_view

    def _wait_counts(self, mapped, num_ranks):
        """Polls until the GPU has written every count (reference: csrc/nixl_ep.cpp:779-797,
        same time-out); returns the total number of rows."""
        deadline = time.monotonic() + self.cpu_timeout_secs
        while int(mapped.min()) < 0:
            if time.monotonic() > deadline:
                raise EPError("timeout (dispatch CPU): the receive counts never arrived")
        return int(mapped[:num_ranks].sum(dtype=np.int64))

    def _get_workspace(self, nbytes):
        if self._workspace is None or self._workspace.numel() < nbytes:
            self._workspace = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=self.device)
        return self._workspace

    # -- low-latency mode -------------------------------------------------------------------
    def low_latency_dispatch(self, x, topk_idx, num_max_dispatch_tokens_per_rank, num_experts=None,
                             cumulative_local_expert_recv_stats=None, dispatch_wait_recv_cost_stats=None,
                             use_fp8=True, round_scale=False, use_ue8m0=False, async_finish=False,
                             return_recv_hook=False, num_tokens_per_rank=None, check_duplicates=False):
        """Reference: buffer.py:329-437, csrc/nixl_ep.cpp:1030-1143.

        x [R, T, H] bf16, topk_idx [R, T, K] int32 (-1 = no selection).  Returns
        ((packed_recv_x, packed_recv_x_scales) or packed_recv_x, packed_recv_count, handle,
        event, hook) with handle = (src_info, layout_range, num_max_dispatch_tokens_per_rank,
        hidden).  `num_tokens_per_rank` ([R] int32 device tensor) is an extension for ragged
        worlds: rank r only owns the first num_tokens_per_rank[r] rows of x[r].
        With a `timeout_ms` on the buffer the receive side waits (bounded) for every source
        rank's selections and masks a rank that is late; dispatch_wait_recv_cost_stats ([R]
        int64, nixl_ep_ll.cu:349-350) then accumulates the wall-clock ticks waited per rank.
        return_recv_hook=True issues the send phase only; the hook issues the receive phase
        (`x` must stay as it is until then: the rows are read by the receive phase).
        A token that names an expert twice gets a row per selection, as in the reference
        (nixl_ep_ll.cu:186-190); `check_duplicates` waits for the kernels and raises if that
        happened (a top-k selection never does it), with return_recv_hook from inside the hook.
        """
        if topk_idx.dim() != 3 or not topk_idx.is_contiguous() or topk_idx.dtype != topk_idx_t:
            raise EPError("topk_idx must be a contiguous [R, T, K] int32 tensor")
        return self._ll_dispatch(x, topk_idx, None, topk_idx.shape[2], num_max_dispatch_tokens_per_rank, num_experts,
                                 cumulative_local_expert_recv_stats, use_fp8, round_scale, use_ue8m0, async_finish,
                                 return_recv_hook, num_tokens_per_rank, check_duplicates,
                                 dispatch_wait_recv_cost_stats)[2:]

    def route_dispatch(self, x, logits, num_topk, num_max_dispatch_tokens_per_rank,
                       cumulative_local_expert_recv_stats=None, use_fp8=True, round_scale=False, use_ue8m0=False,
                       async_finish=False, return_recv_hook=False, num_tokens_per_rank=None):
        """Routing and dispatch in one call (no reference counterpart: its callers bring
        their own top-k).  logits [R, T, E] float32.  Returns (topk_idx, topk_weights) followed
        by what low_latency_dispatch returns; the selection is that of route().  Issued whole:
        a `timeout_ms` on the buffer and return_recv_hook do not split or guard this call (its
        first kernel routes and publishes the selections in one go)."""
        if logits.dim() != 3 or not logits.is_contiguous() or logits.dtype != torch.float32:
            raise EPError("logits must be a contiguous [R, T, E] float32 tensor")
        return self._ll_dispatch(x, None, logits, num_topk, num_max_dispatch_tokens_per_rank, logits.shape[2],
                                 cumulative_local_expert_recv_stats, use_fp8, round_scale, use_ue8m0, async_finish,
                                 return_recv_hook, num_tokens_per_rank, False)

    def _ll_dispatch(self, x, topk_idx, logits, K, num_max_dispatch_tokens_per_rank, num_experts, stats, use_fp8,
                     round_scale, use_ue8m0, async_finish, return_recv_hook, num_tokens_per_rank, check_duplicates,
                     wait_stats=None):
        if not self.low_latency_mode:
            raise EPError("dispatch() requires low-latency mode (low_latency_mode=True)")
        if x.dim() != 3 or not x.is_contiguous() or x.dtype != torch.bfloat16:
            raise EPError("x must be a contiguous [R, T, H] bfloat16 tensor")
        R, T, H = x.shape
        sel = topk_idx if logits is None else logits
        if R != self.num_ranks or sel.shape[0] != R or sel.shape[1] != T:
            raise EPError("x and the selection must agree on ranks and tokens")
        if T > num_max_dispatch_tokens_per_rank:
            raise EPError("more tokens than num_max_dispatch_tokens_per_rank")
        if num_experts is None:
            raise EPError("num_experts is required")
        El, N = num_experts // R, R * num_max_dispatch_tokens_per_rank
        dev = x.device
        packed_recv_x = torch.empty((R, El, N, H), dtype=torch.float8_e4m3fn if use_fp8 else torch.bfloat16, device=dev)
        packed_recv_src_info = torch.empty((R, El, N), dtype=torch.int32, device=dev)
        packed_recv_layout_range = torch.empty((R, El, R), dtype=torch.int64, device=dev)
        packed_recv_count = torch.empty((R, El), dtype=torch.int32, device=dev)
        scales = None
        if use_fp8:
            if use_ue8m0:
                scales = torch.empty((R, El, H // 512, N), dtype=torch.int32, device=dev)
            else:
                scales = torch.empty((R, El, H // 128, N), dtype=torch.float32, device=dev)
        row_map = torch.empty((R, T, K), dtype=torch.int32, device=dev)
        ws_bytes = self._k.nixl_amd_ep_ll_workspace_bytes(R, num_experts, T, K, H)
        ws = self._get_workspace(ws_bytes)
        head = (_ptr(packed_recv_x), _ptr(scales), _ptr(packed_recv_src_info), _ptr(packed_recv_layout_range),
                _ptr(packed_recv_count), self._mask_ptr(), _ptr(stats), _ptr(x))
        tail = (_ptr(num_tokens_per_rank), T, H, num_max_dispatch_tokens_per_rank, K, R, num_experts, int(use_fp8),
                int(round_scale), int(use_ue8m0), _ptr(row_map), _ptr(ws), ws.numel(), _stream())
        topk_weights = None
        hook = None
        phased = logits is None and (self.timeout_ms is not None or return_recv_hook)
        if phased:
            if wait_stats is not None and (wait_stats.dtype != torch.int64 or wait_stats.numel() < R):
                raise EPError("dispatch_wait_recv_cost_stats must hold R int64 values")
            timeout_us = 0 if self.timeout_ms is None else max(int(self.timeout_ms * 1000), 1)
            withhold, self.withhold_rank = self.withhold_rank, -1
            if timeout_us:
                self._mask_active = True  # the kernels may enter a late rank
            mask = _ptr(self.mask_buffer) if timeout_us else self._mask_ptr()

            def issue(phases):
                return self._k.nixl_amd_ep_ll_dispatch_phased(
                    *head[:5], mask, _ptr(stats), _ptr(wait_stats), _ptr(x), _ptr(topk_idx), *tail[:-1], phases,
                    timeout_us, withhold, _stream())

            if return_recv_hook:
                rc = issue(1)
                keep = (x, topk_idx, ws, stats, wait_stats, num_tokens_per_rank)  # alive until the hook has run

                def hook(keep=keep, look=check_duplicates):
                    _check(issue(2), "low_latency_dispatch (receive phase)")
                    if look:  # the status word is written by the receive phase
                        self._raise_on_repeats(ws)

                check_duplicates = False  # not before the receive phase has run
            else:
                rc = issue(3)
        elif logits is None:
            rc = self._k.nixl_amd_ep_ll_dispatch(*head, _ptr(topk_idx), *tail)
        else:
            topk_idx = torch.empty((R, T, K), dtype=topk_idx_t, device=dev)
            topk_weights = torch.empty((R, T, K), dtype=torch.float32, device=dev)
            rc = self._k.nixl_amd_ep_ll_route_dispatch(*head, _ptr(logits), _ptr(topk_idx), _ptr(topk_weights), *tail)
        _check(rc, "low_latency_dispatch")
        if check_duplicates:
            self._raise_on_repeats(ws)
        event = None
        if async_finish:
            event = torch.cuda.Event()
            event.record()
        handle = DispatchHandle((packed_recv_src_info, packed_recv_layout_range, num_max_dispatch_tokens_per_rank, H))
        handle.row_map = row_map
        recv = (packed_recv_x, scales.transpose(2, 3)) if use_fp8 else packed_recv_x
        if return_recv_hook and hook is None:
            hook = lambda: None  # noqa: E731  (routing dispatch: issued whole)
        return topk_idx, topk_weights, recv, packed_recv_count, handle, EventOverlap(event), hook

    def _raise_on_repeats(self, ws):
        status = ctypes.c_int(0)
        _check(self._k.nixl_amd_ep_ll_dispatch_status(_ptr(ws), _stream(), ctypes.byref(status)), "dispatch status")
        if status.value:
            raise EPError("a token's top-k names the same expert twice")

    def dispatch(self, *args, **kwargs):
        return self.low_latency_dispatch(*args, **kwargs)

    def low_latency_combine(self, x, topk_idx, topk_weights, handle, use_logfmt=False, zero_copy=False,
                            async_finish=False, return_recv_hook=False, out=None,
                            combine_wait_recv_cost_stats=None, num_tokens_per_rank=None, rank_ready=None):
        """Reference: buffer.py:443-520, csrc/nixl_ep.cpp:1145-1246.

        x [R, El, N, H] bf16 expert outputs, topk_idx / topk_weights [R, T, K].  Returns
        (combined_x [R, T, H] bf16, event, hook).  rank_ready ([R] int32, an extension; needs a
        `timeout_ms` on the buffer): word j is set by the producer of `x` when rank j's rows are
        complete; combine waits for it (bounded) and masks a rank whose word stays zero, as the
        reference's receivers do with a rank whose flag never comes (nixl_ep_ll.cu:846-866);
        combine_wait_recv_cost_stats ([R] int64) accumulates the ticks waited."""
        if not self.low_latency_mode:
            raise EPError("combine() requires low-latency mode (low_latency_mode=True)")
        src_info, layout_range, max_tok, hidden = handle
        if zero_copy:
            x = getattr(self, "_combine_buffer", None)
            if x is None:
                raise EPError("zero_copy=True needs get_next_combine_buffer() first")
        if x.dim() != 4 or not x.is_contiguous() or x.dtype != torch.bfloat16 or x.shape[-1] != hidden:
            raise EPError("x must be a contiguous [R, El, N, H] bfloat16 tensor")
        if topk_weights.dtype != torch.float32 or not topk_weights.is_contiguous():
            raise EPError("topk_weights must be contiguous float32")
        R, T, K = topk_idx.shape
        num_experts = x.shape[1] * R
        combined = out if out is not None else torch.empty((R, T, hidden), dtype=torch.bfloat16, device=x.device)
        stats = combine_wait_recv_cost_stats
        if rank_ready is not None:
            if self.timeout_ms is None:
                raise EPError("rank_ready needs a buffer created with timeout_ms")
            if rank_ready.dtype != torch.int32 or rank_ready.numel() < R:
                raise EPError("rank_ready must hold R int32 values")
            if stats is not None and (stats.dtype != torch.int64 or stats.numel() < R):
                raise EPError("combine_wait_recv_cost_stats must hold R int64 values")
            self._mask_active = True
        row_map = getattr(handle, "row_map", None)

        def issue():
            if rank_ready is not None:
                return self._k.nixl_amd_ep_ll_combine_elastic(
                    _ptr(combined), _ptr(x), _ptr(topk_idx), _ptr(topk_weights), _ptr(src_info), _ptr(layout_range),
                    _ptr(self.mask_buffer), _ptr(rank_ready), _ptr(stats), _ptr(num_tokens_per_rank), _ptr(row_map), T,
                    hidden, max_tok, K, R, num_experts, int(use_logfmt), max(int(self.timeout_ms * 1000), 1), _stream())
            return self._k.nixl_amd_ep_ll_combine(
                _ptr(combined), _ptr(x), _ptr(topk_idx), _ptr(topk_weights), _ptr(src_info), _ptr(layout_range),
                self._mask_ptr(), _ptr(num_tokens_per_rank), _ptr(row_map), T, hidden, max_tok, K, R, num_experts,
                int(use_logfmt), _stream())

        # The send phase of the reference moves the expert outputs to their readers; here they
        # are read where they lie, so with a hook the whole reduction is the receive phase and
        # combined_x is valid once the hook has run (as in the reference).
        hook = None
        if return_recv_hook:
            hook = lambda: _check(issue(), "low_latency_combine (receive phase)")  # noqa: E731
        else:
            _check(issue(), "low_latency_combine")
        event = None
        if async_finish:
            event = torch.cuda.Event()
            event.record()
        return combined, EventOverlap(event), hook

    def combine(self, *args, **kwargs):
        return self.low_latency_combine(*args, **kwargs)

    # -- router (no reference counterpart; callers of the reference bring their own top-k) --
    def route(self, logits, num_topk):
        """logits [..., E] float32 -> (topk_idx int32 [..., K], topk_weights float32 [..., K])."""
        if logits.dtype != torch.float32 or not logits.is_contiguous():
            raise EPError("logits must be contiguous float32")
        E = logits.shape[-1]
        lead = logits.shape[:-1]
        n = logits.numel() // E
        idx = torch.empty((*lead, num_topk), dtype=torch.int32, device=logits.device)
        w = torch.empty((*lead, num_topk), dtype=torch.float32, device=logits.device)
        _check(self._k.nixl_amd_ep_router_topk(_ptr(logits), _ptr(idx), _ptr(w), n, E, num_topk, _stream()), "route")
        return idx, w

    # -- normal (high-throughput) mode ---------------------------------------------------------
    # The reference runs normal-mode work on a communication stream: it makes that stream wait
    # for `previous_event` (or for the caller's stream), and hands back an event instead of
    # joining the streams when `async_finish` is set (csrc/nixl_ep.cpp:558-571,596-611).  Here
    # the work runs on the caller's current stream, so only the two events remain.
    @staticmethod
    def _after(previous_event, async_finish, allocate_on_comm_stream):
        if allocate_on_comm_stream and not (previous_event is not None and async_finish):
            raise EPError("allocate_on_comm_stream needs previous_event and async_finish")  # csrc/nixl_ep.cpp:562
        event = getattr(previous_event, "event", None)
        if event is not None:
            torch.cuda.current_stream().wait_event(event)

    @staticmethod
    def _done(async_finish):
        if not async_finish:
            return EventOverlap(None)
        event = torch.cuda.Event()
        event.record()
        return EventOverlap(event)

    def get_dispatch_layout(self, topk_idx, num_experts, previous_event=None, async_finish=False,
                            allocate_on_comm_stream=False):
        """Reference: buffer.py:278-326, csrc/nixl_ep.cpp:551-613.  topk_idx [R, T, K].
        Returns (num_tokens_per_rank [R, R], num_tokens_per_rdma_rank=None,
        num_tokens_per_expert [R, E], is_token_in_rank [R, T, R] bool, event)."""
        R, T, K = topk_idx.shape
        dev = topk_idx.device
        self._after(previous_event, async_finish, allocate_on_comm_stream)
        per_rank = torch.empty((R, R), dtype=torch.int32, device=dev)
        per_expert = torch.empty((R, num_experts), dtype=torch.int32, device=dev)
        in_rank = torch.empty((R, T, R), dtype=torch.bool, device=dev)
        _check(self._k.nixl_amd_ep_get_dispatch_layout(_ptr(topk_idx), _ptr(per_rank), _ptr(per_expert), _ptr(in_rank),
                                                       T, K, R, num_experts, _stream()), "get_dispatch_layout")
        return per_rank, None, per_expert, in_rank, self._done(async_finish)

    def ht_dispatch(self, x, handle=None, num_tokens_per_rank=None, num_tokens_per_rdma_rank=None,
                    is_token_in_rank=None, num_tokens_per_expert=None, topk_idx=None, topk_weights=None,
                    expert_alignment=1, config=None, previous_event=None, async_finish=False,
                    allocate_on_comm_stream=False, num_channels=None):
        """Reference: buffer.py:526-660, csrc/nixl_ep.cpp:615-898.

        x [R, T, H] bfloat16, or a tuple (x, x_scales) of fp8 rows [R, T, H] and their
        per-token scales [R, T, S] (float32, or int32 for packed UE8M0; any strides, e.g. the
        transposed layout the reference's test passes); the layout tensors come from
        get_dispatch_layout and topk_idx / topk_weights are optional.  Returns (recv_x or
        (recv_x, recv_x_scales), recv_topk_idx, recv_topk_weights,
        num_recv_tokens_per_expert_list, handle, event).  recv_* hold every destination rank's
        rows back to back; destination d owns rows recv_row_offset[d] : recv_row_offset[d + 1]
        (handle field)."""
        if self.low_latency_mode:
            raise EPError("ht_dispatch() requires high-throughput mode (low_latency_mode=False)")
        x, x_scales = x if isinstance(x, tuple) else (x, None)
        if x.dim() != 3 or not x.is_contiguous():
            raise EPError("x must be a contiguous [R, T, H] tensor")
        if x_scales is None and x.dtype != torch.bfloat16:
            raise EPError("x must be bfloat16 unless it comes with scales, as (x, x_scales)")
        R, T, H = x.shape
        dev = x.device
        if (H * x.element_size()) % 16:
            raise EPError("a row of x must be a multiple of 16 bytes")  # csrc/nixl_ep.cpp:660
        S = 0
        if x_scales is not None:
            # csrc/nixl_ep.cpp:703-711
            if x_scales.dtype not in (torch.float32, torch.int32) or x_scales.dim() != 3 or tuple(x_scales.shape[:2]) != (R, T):
                raise EPError("x_scales must be a float32 or int32 tensor of shape [R, T, num_scales]")
            S = x_scales.shape[2]

        def rows_kernel(recv_x, recv_scales, recv_idx, recv_w, recv_meta, idx, w, in_rank, prefix, send_head, row_offset, K, E):
            strides = x_scales.stride() if x_scales is not None else (0, 0, 0)
            _check(self._k.nixl_amd_ep_ht_dispatch_scaled(
                _ptr(recv_x), _ptr(recv_scales), _ptr(recv_idx), _ptr(recv_w), _ptr(recv_meta), _ptr(x), _ptr(x_scales),
                _ptr(idx), _ptr(w), _ptr(in_rank), _ptr(prefix), _ptr(send_head), _ptr(row_offset), T, H,
                x.element_size(), S, strides[0], strides[1], strides[2], K, R, E, _stream()), "ht_dispatch")

        def with_scales(recv_x, recv_scales):
            return (recv_x, recv_scales) if x_scales is not None else recv_x

        self._after(previous_event, async_finish, allocate_on_comm_stream)

        if handle is not None:
            # Cached mode (buffer.py:560-597): the layout of an earlier dispatch is reused, so
            # there is no count exchange and no host synchronisation; only rows travel.
            in_rank, prefix, _chan, recv_src_meta, send_head, row_offset = handle
            if tuple(in_rank.shape) != (R, T, R):
                raise EPError("handle does not belong to a dispatch of this shape")
            n_rows = recv_src_meta.shape[0]
            recv_x = torch.empty((n_rows, H), dtype=x.dtype, device=dev)
            recv_scales = torch.empty((n_rows, S), dtype=x_scales.dtype, device=dev) if x_scales is not None else None
            rows_kernel(recv_x, recv_scales, None, None, None, None, None, in_rank, prefix, send_head, row_offset, 0, R)
            return with_scales(recv_x, recv_scales), None, None, None, None, self._done(async_finish)
        if num_tokens_per_rank is None or is_token_in_rank is None or num_tokens_per_expert is None:
            raise EPError("ht_dispatch needs either a handle or the tensors of get_dispatch_layout")
        if (topk_idx is None) != (topk_weights is None):
            raise EPError("topk_idx and topk_weights go together")  # csrc/nixl_ep.cpp:686
        if num_channels is None:  # as the reference derives it (csrc/nixl_ep.cpp:630)
            num_channels = (config or self.get_dispatch_config(R)).num_sms // 2
        K = topk_idx.shape[2] if topk_idx is not None else 0
        E = num_tokens_per_expert.shape[1]
        El = E // R
        prefix = torch.empty((R, R), dtype=torch.int32, device=dev)
        chan = torch.empty((R, R, num_channels), dtype=torch.int32, device=dev)
        send_head = torch.empty((R, T, R), dtype=torch.int32, device=dev)
        row_offset = torch.empty(R + 1, dtype=torch.int64, device=dev)
        # The counts the host needs go straight to pinned host memory, preset to -1 and polled
        # below, as in the reference (csrc/nixl_ep.cpp:762-800).
        mapped = self._mapped_counts(R + R * El)
        mapped.fill(-1)
        recv_counter_ptr = ctypes.c_void_p(self._mapped_tensor.data_ptr())
        expert_count_ptr = ctypes.c_void_p(self._mapped_tensor.data_ptr() + 4 * R)
        _check(self._k.nixl_amd_ep_ht_notify_dispatch(_ptr(is_token_in_rank), _ptr(num_tokens_per_expert), _ptr(prefix),
                                                      expert_count_ptr, _ptr(chan), _ptr(send_head), _ptr(row_offset),
                                                      recv_counter_ptr, T, R, E, num_channels, expert_alignment,
                                                      _stream()), "ht_notify_dispatch")
        # The reference waits here, because it sizes recv_x from the counts.  With 288 GB of
        # HBM the receive side can be sized for the worst case instead (every set entry of
        # is_token_in_rank is one row, so R*T*R rows bound the total): the row kernels are
        # queued right behind the count kernels, the GPU never idles through the host round
        # trip, and the host only waits for the counts to cut the views.
        capacity = R * T * R
        ahead = capacity * (H * x.element_size() + S * 4 + K * 8 + 8) <= self.ht_recv_worst_case_limit
        rows = capacity if ahead else self._wait_counts(mapped, R)
        recv_x = torch.empty((rows, H), dtype=x.dtype, device=dev)
        recv_scales = torch.empty((rows, S), dtype=x_scales.dtype, device=dev) if x_scales is not None else None
        recv_topk_idx = torch.empty((rows, K), dtype=torch.int32, device=dev) if K else None
        recv_topk_weights = torch.empty((rows, K), dtype=torch.float32, device=dev) if K else None
        recv_src_meta = torch.empty((rows, 2), dtype=torch.int32, device=dev)
        rows_kernel(recv_x, recv_scales, recv_topk_idx, recv_topk_weights, recv_src_meta, topk_idx, topk_weights,
                    is_token_in_rank, prefix, send_head, row_offset, K, E)
        if ahead:
            total = self._wait_counts(mapped, R)
            recv_x, recv_src_meta = recv_x[:total], recv_src_meta[:total]
            if recv_scales is not None:
                recv_scales = recv_scales[:total]
            if K:
                recv_topk_idx, recv_topk_weights = recv_topk_idx[:total], recv_topk_weights[:total]
        expert_count_list = mapped[R:].reshape(R, El).tolist()
        out_handle = (is_token_in_rank, prefix, chan, recv_src_meta, send_head, row_offset)
        return (with_scales(recv_x, recv_scales), recv_topk_idx, recv_topk_weights, expert_count_list, out_handle,
                self._done(async_finish))

    def ht_combine(self, x, handle, topk_weights=None, bias=None, config=None, previous_event=None,
                   async_finish=False, allocate_on_comm_stream=False):
        """Reference: buffer.py:663-714, csrc/nixl_ep.cpp:900-1028.  x [total, H] bf16 in the
        row order ht_dispatch produced.  Returns (combined_x [R, T, H], combined_topk_weights
        [R, T, K] or None, event)."""
        if self.low_latency_mode:
            raise EPError("ht_combine() requires high-throughput mode (low_latency_mode=False)")
        in_rank, prefix, _chan, _meta, send_head, row_offset = handle
        R, T, _ = in_rank.shape
        H = x.shape[1]
        dev = x.device
        bias_0, bias_1 = (bias if isinstance(bias, (tuple, list)) else (bias, None))
        K = topk_weights.shape[1] if topk_weights is not None else 0
        self._after(previous_event, async_finish, allocate_on_comm_stream)
        combined = torch.empty((R, T, H), dtype=torch.bfloat16, device=dev)
        combined_w = torch.empty((R, T, K), dtype=torch.float32, device=dev) if K else None
        _check(self._k.nixl_amd_ep_ht_combine(_ptr(combined), _ptr(combined_w), _ptr(x), _ptr(topk_weights),
                                              _ptr(bias_0), _ptr(bias_1), _ptr(in_rank), _ptr(prefix), _ptr(send_head),
                                              _ptr(row_offset), T, H, max(K, 1), R, _stream()), "ht_combine")
        return combined, combined_w, self._done(async_finish)
