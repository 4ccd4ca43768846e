/*
 * C ABI of the expert-parallel (EP) dispatch / combine kernels (libnixl_amd_kernels.so).
 *
 * These entry points stand where the reference's kernel launchers stand — plain functions
 * taking raw pointers, sizes and a stream (examples/device/ep/csrc/kernels/api.cuh:63-72,
 * 81-203,211-238) — with one change of shape: the reference launches one rank's kernel per
 * process and moves data between processes; here every rank of the job is a region of one
 * GPU's HBM, so each call processes ALL virtual ranks and every array carries a leading
 * rank dimension.  `rank`, the RDMA buffers, `next_clean`, `phases`, time-outs and the
 * device-side NIXL context of the reference signatures have no meaning on one GPU and are
 * gone.  Results are what the reference kernels deliver, in their canonical order (segments
 * by source rank ascending, tokens ascending), bit for bit.
 *
 * Notation: R ranks, E experts (E % R == 0), El = E / R, T tokens per rank as laid out,
 * K top-k, H hidden, M = num_max_dispatch_tokens_per_rank, N = R * M.
 * `stream` is a hipStream_t passed as void*.  All pointers are device pointers unless
 * stated otherwise.  Return value: 0 or a negative nixl_amd_status (nixl_amd_hip.h);
 * nixl_amd_last_error() has the text.  Arguments are validated on the host before any
 * launch; nothing falls back to a CPU path.
 */
#ifndef NIXL_AMD_EP_H
#define NIXL_AMD_EP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Launch-shape knob of the low-latency kernels (no reference counterpart): the largest
 * workgroup, in lanes, of the dispatch and combine kernels; a multiple of 64 in [64, 1024],
 * 0 to leave a value unchanged, or -1 to return to the built-in choice: dispatch takes a
 * workgroup per token, combine one per row, or two halves for a row of more than 512 lanes.
 * Process-wide; may be called from any thread: a dispatch or
 * combine call that runs at the same time uses the old or the new value. */
int
nixl_amd_ep_ll_set_tuning(int dispatch_lanes, int combine_lanes);

/* Bytes of scratch the low-latency dispatch needs (one 64-bit word of selection bits per
 * (expert, rank, 64 tokens), a flag per 64 tokens, per-token scales, a 256-byte header); the
 * scratch must be 16-byte aligned.  Reference: `workspace` of ep_kernels::dispatch, kernels/nixl_ep_ll.cu:423-426. */
size_t
nixl_amd_ep_ll_workspace_bytes(int num_ranks, int num_experts, int num_tokens, int num_topk, int hidden);

/*
 * Low-latency dispatch for all ranks.  Replaces ep_kernels::dispatch
 * (kernels/api.cuh:211-224; kernel kernels/nixl_ep_ll.cu:71-395; host
 * csrc/nixl_ep.cpp:1030-1143).
 *   x                      [R][T][H] bf16
 *   topk_idx               [R][T][K] int32, -1 = no selection.  A token that names an expert
 *                          more than once gets a row of that expert per selection, as in the
 *                          reference (kernels/nixl_ep_ll.cu:186-190: a slot per selection), in
 *                          (token, selection) order; such a call counts its rows from the
 *                          selection instead of from the selection bits (slower, and reported:
 *                          nixl_amd_ep_ll_dispatch_status then returns
 *                          NIXL_AMD_EP_STATUS_DUPLICATE_EXPERT).  An expert that would receive
 *                          more than N rows this way loses the rows beyond N
 *   num_tokens_per_rank    [R] int32 tokens present on each rank (<= T), or NULL = T
 *   mask_buffer            [R][R] int32 or NULL; tokens travel a -> b only if neither
 *                          mask[a][b] nor mask[b][a] is set (kernels/nixl_ep_ll.cu:197,266,319)
 *   packed_recv_x          [R][El][N][H]    fp8 e4m3 (use_fp8) or bf16
 *   packed_recv_x_scales   [R][El][H/128][N] float, or with use_ue8m0 [R][El][H/512][N]
 *                          int32 words of four exponent bytes; NULL unless use_fp8
 *   packed_recv_src_info   [R][El][N] int32
 *   packed_recv_layout_range [R][El][R] int64: count | begin << 32
 *   packed_recv_count      [R][El] int32
 *   cumulative_local_expert_recv_stats [R][El] int32 or NULL; incremented by the counts
 *   row_map                [R][T][K] int32 or NULL (no reference counterpart): receives, for
 *                          every selection, its row in the flattened [R*El*N] row space of
 *                          packed_recv_x, or -1.  Passing it on to the combine call saves
 *                          that call its search through src_info.
 * Rows at or beyond packed_recv_count are not written.
 */
int
nixl_amd_ep_ll_dispatch(void *packed_recv_x,
                        void *packed_recv_x_scales,
                        int *packed_recv_src_info,
                        int64_t *packed_recv_layout_range,
                        int *packed_recv_count,
                        const int *mask_buffer,
                        int *cumulative_local_expert_recv_stats,
                        const void *x,
                        const int32_t *topk_idx,
                        const int *num_tokens_per_rank,
                        int num_tokens,
                        int hidden,
                        int num_max_dispatch_tokens_per_rank,
                        int num_topk,
                        int num_ranks,
                        int num_experts,
                        int use_fp8,
                        int round_scale,
                        int use_ue8m0,
                        int *row_map,
                        void *workspace,
                        size_t workspace_bytes,
                        void *stream);

/*
 * Routing and low-latency dispatch in one call: nixl_amd_ep_ll_dispatch with the top-k
 * selection done first, by the kernel that prepares the dispatch (no launch of its own).
 * The reference's callers bring their own top-k (tests/elastic/elastic.py:153-158); this is
 * the north-star's "dispatch does top-k routing".
 *   logits        [R][T][E] float, in
 *   topk_idx      [R][T][K] int32, out: the K largest logits of each token, descending, ties
 *                 to the lower expert index (what nixl_amd_ep_router_topk returns)
 *   topk_weights  [R][T][K] float, out: softmax over those K logits
 * num_experts <= 1024.  Everything else as nixl_amd_ep_ll_dispatch.
 */
int
nixl_amd_ep_ll_route_dispatch(void *packed_recv_x,
                              void *packed_recv_x_scales,
                              int *packed_recv_src_info,
                              int64_t *packed_recv_layout_range,
                              int *packed_recv_count,
                              const int *mask_buffer,
                              int *cumulative_local_expert_recv_stats,
                              const void *x,
                              const float *logits,
                              int32_t *topk_idx,
                              float *topk_weights,
                              const int *num_tokens_per_rank,
                              int num_tokens,
                              int hidden,
                              int num_max_dispatch_tokens_per_rank,
                              int num_topk,
                              int num_ranks,
                              int num_experts,
                              int use_fp8,
                              int round_scale,
                              int use_ue8m0,
                              int *row_map,
                              void *workspace,
                              size_t workspace_bytes,
                              void *stream);

/* Status of the last dispatch that used `workspace`, read back after waiting for `stream`:
 * 0, or NIXL_AMD_EP_STATUS_DUPLICATE_EXPERT if some token's selection named an expert twice
 * (handled as the reference handles it, a row per selection; a caller whose selection is meant
 * to be a top-k learns here that it was not).  The word is written by the receive phase.  No
 * reference counterpart. */
#define NIXL_AMD_EP_STATUS_DUPLICATE_EXPERT 1
int
nixl_amd_ep_ll_dispatch_status(const void *workspace, void *stream, int *status);

/*
 * Low-latency dispatch in two phases, with the receive side's bounded wait.  Arguments and
 * results are those of nixl_amd_ep_ll_dispatch, plus:
 *   phases   1: send phase only (the selections are published; `x` is not read yet)
 *            2: receive phase only, for the send phase issued last on this workspace (same
 *               arguments): rows, scales and metadata are produced
 *            3: both.  This is the split behind return_recv_hook (csrc/nixl_ep.cpp:1125-1136).
 *   timeout_us > 0: before it places anything, the receive phase waits for each source rank's
 *            selections, at most that long per rank; a rank whose selections have not come is
 *            taken as having sent nothing and mask_buffer[dst][rank] is set for every dst, as
 *            the reference's receivers do (kernels/nixl_ep_ll.cu:316-340; the budget there is
 *            in clock cycles, csrc/nixl_ep.cpp:49-52).  Needs mask_buffer.  At most 100 s (the
 *            upper end of the reference's defaults).  A receive phase whose workspace holds no
 *            send phase's stamp (issued on its own, or on another workspace) waits for nothing:
 *            ranks whose selections are not there are masked at once.
 *   dispatch_wait_recv_cost_stats  [R] int64 or NULL: ticks of the GPU's constant-rate wall
 *            clock spent waiting for each source rank, accumulated (kernels/nixl_ep_ll.cu:349).
 *   withhold_rank  -1, or a rank whose send phase leaves out the word its receivers wait for:
 *            the way to make a time-out happen on one GPU, where every rank's selections are
 *            otherwise there before the receive phase starts.  The wait then lasts the whole
 *            time-out, which must be at most one second.
 * On a stream, the kernels of the send phase are complete before the receive phase looks, so
 * without a withheld rank the wait costs one small kernel and never spins.
 */
int
nixl_amd_ep_ll_dispatch_phased(void *packed_recv_x,
                               void *packed_recv_x_scales,
                               int *packed_recv_src_info,
                               int64_t *packed_recv_layout_range,
                               int *packed_recv_count,
                               int *mask_buffer,
                               int *cumulative_local_expert_recv_stats,
                               int64_t *dispatch_wait_recv_cost_stats,
                               const void *x,
                               const int32_t *topk_idx,
                               const int *num_tokens_per_rank,
                               int num_tokens,
                               int hidden,
                               int num_max_dispatch_tokens_per_rank,
                               int num_topk,
                               int num_ranks,
                               int num_experts,
                               int use_fp8,
                               int round_scale,
                               int use_ue8m0,
                               int *row_map,
                               void *workspace,
                               size_t workspace_bytes,
                               int phases,
                               uint64_t timeout_us,
                               int withhold_rank,
                               void *stream);

/*
 * Low-latency dispatch that allocates nothing.  No counterpart in the reference; it is for
 * callers that cannot allocate device memory: code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc.  Arguments and results are those of
 * nixl_amd_ep_ll_dispatch without `workspace`: the scratch is a fixed array of
 * NIXL_AMD_EP_LL_STATIC_SCRATCH_BYTES inside the library, one copy per GPU, held until the
 * process ends.  A shape whose nixl_amd_ep_ll_workspace_bytes exceeds that size is refused with
 * NIXL_AMD_ERR_TOO_LARGE before anything is launched.  All calls on one GPU share the array:
 * two calls may not overlap on one GPU (different streams, or threads), or they race.  The
 * call itself issues no hipMalloc, hipFree, memset or other allocating routine.
 */
#define NIXL_AMD_EP_LL_STATIC_SCRATCH_BYTES (2u << 20)
int
nixl_amd_ep_ll_dispatch_static(void *packed_recv_x,
                               void *packed_recv_x_scales,
                               int *packed_recv_src_info,
                               int64_t *packed_recv_layout_range,
                               int *packed_recv_count,
                               const int *mask_buffer,
                               int *cumulative_local_expert_recv_stats,
                               const void *x,
                               const int32_t *topk_idx,
                               const int *num_tokens_per_rank,
                               int num_tokens,
                               int hidden,
                               int num_max_dispatch_tokens_per_rank,
                               int num_topk,
                               int num_ranks,
                               int num_experts,
                               int use_fp8,
                               int round_scale,
                               int use_ue8m0,
                               int *row_map,
                               void *stream);

/*
 * Low-latency combine for all ranks.  Replaces ep_kernels::combine (kernels/api.cuh:226-238;
 * kernel kernels/nixl_ep_ll.cu:618-1017): combined_x[r][t] = bf16( sum over k, in top-k
 * order, of float(x[row(r,t,k)]) * topk_weights[r][t][k] ) with fused multiply-adds in
 * fp32, skipping idx < 0 and masked ranks.  row(r,t,k) is located through the dispatch
 * handle (src_info, layout_range), so any valid permutation inside a segment is accepted.
 *   x             [R][El][N][H] bf16 (expert outputs in packed_recv_x layout)
 *   combined_x    [R][T][H] bf16
 *   row_map       [R][T][K] int32 as written by the dispatch call that produced this
 *                 handle, or NULL to locate rows through src_info / layout_range
 * use_logfmt: every row goes through the reference's LogFMT-10 codec (encode as the sender
 * does, decode as the receiver does; kernels/nixl_ep_ll.cu:459-616) before it is accumulated.
 * The codec is lossy and built on log2 / exp2, whose last bits differ between GPUs and libm:
 * results are reproducible on one GPU and agree with the CPU restatement to a tolerance.
 */
int
nixl_amd_ep_ll_combine(void *combined_x,
                       const void *x,
                       const int32_t *topk_idx,
                       const float *topk_weights,
                       const int *src_info,
                       const int64_t *layout_range,
                       const int *mask_buffer,
                       const int *num_tokens_per_rank,
                       const int *row_map,
                       int num_tokens,
                       int hidden,
                       int num_max_dispatch_tokens_per_rank,
                       int num_topk,
                       int num_ranks,
                       int num_experts,
                       int use_logfmt,
                       void *stream);

/*
 * Low-latency combine behind a bounded wait for the ranks whose expert outputs it reads
 * (the receive side of kernels/nixl_ep_ll.cu:846-866).  rank_ready is [R] int32 in device or
 * pinned host memory: word j is set (nonzero) by whoever produces `x` once the rows of rank j's
 * experts are complete, e.g. by the last kernel of that rank's expert step on another stream.
 * A rank whose word is still zero after timeout_us (1 us .. 1 s) is entered in
 * mask_buffer[dst][j] for every dst and its experts drop out of the sums, here and in later
 * calls, exactly as for a rank masked by hand.  combine_wait_recv_cost_stats: [R] int64 or
 * NULL, wall-clock ticks waited per rank, accumulated.  The caller clears rank_ready.
 */
int
nixl_amd_ep_ll_combine_elastic(void *combined_x,
                               const void *x,
                               const int32_t *topk_idx,
                               const float *topk_weights,
                               const int *src_info,
                               const int64_t *layout_range,
                               int *mask_buffer,
                               const int *rank_ready,
                               int64_t *combine_wait_recv_cost_stats,
                               const int *num_tokens_per_rank,
                               const int *row_map,
                               int num_tokens,
                               int hidden,
                               int num_max_dispatch_tokens_per_rank,
                               int num_topk,
                               int num_ranks,
                               int num_experts,
                               int use_logfmt,
                               uint64_t timeout_us,
                               void *stream);

/*
 * Token counts per rank and per expert and the token-in-rank matrix, for all source ranks.
 * Replaces layout::get_dispatch_layout (kernels/api.cuh:63-72; kernels/layout.cu:31-153).
 *   topk_idx               [R][T][K] int32
 *   num_tokens_per_rank    [R src][R] int32
 *   num_tokens_per_expert  [R src][E] int32
 *   is_token_in_rank       [R src][T][R] bool (1 byte)
 */
int
nixl_amd_ep_get_dispatch_layout(const int32_t *topk_idx,
                                int *num_tokens_per_rank,
                                int *num_tokens_per_expert,
                                uint8_t *is_token_in_rank,
                                int num_tokens,
                                int num_topk,
                                int num_ranks,
                                int num_experts,
                                void *stream);

/*
 * Normal-mode count exchange.  Replaces the arithmetic of ht::notify_dispatch
 * (kernels/api.cuh:81-113; kernels/nixl_ep_ht.cu:257-314,324-374).
 *   recv_gbl_rank_prefix_sum [R dst][R src] int32, inclusive over source ranks
 *   recv_expert_count        [R dst][El] int32, rounded up to expert_alignment
 *   gbl_channel_prefix_matrix [R src][R dst][C] int32, inclusive over channels; channel c
 *                            covers tokens [c * ceil(T/C), (c+1) * ceil(T/C))
 *   send_head                [R src][T][R dst] int32: position of the token inside the
 *                            (src -> dst) segment, -1 if it does not go there
 *   recv_row_offset          [R + 1] int64 or NULL (no reference counterpart): exclusive prefix
 *                            of the per-destination row totals, the form ht_dispatch and
 *                            ht_combine take; its last entry is the row count of recv_x
 *   recv_counter             [R dst] int32 or NULL: rows each destination receives
 *
 * recv_counter and recv_expert_count are what the host needs to size the receive tensors; no
 * later kernel reads them.  As the reference's moe_recv_counter_mapped and
 * moe_recv_expert_counter_mapped (kernels/api.cuh:82,87; csrc/nixl_ep.cpp:762-800) they may
 * point to pinned host memory: the host presets them to -1 and polls until every entry is
 * non-negative, instead of copying them back.
 */
int
nixl_amd_ep_ht_notify_dispatch(const uint8_t *is_token_in_rank,
                               const int *num_tokens_per_expert,
                               int *recv_gbl_rank_prefix_sum,
                               int *recv_expert_count,
                               int *gbl_channel_prefix_matrix,
                               int *send_head,
                               int64_t *recv_row_offset,
                               int *recv_counter,
                               int num_tokens,
                               int num_ranks,
                               int num_experts,
                               int num_channels,
                               int expert_alignment,
                               void *stream);

/*
 * Normal-mode dispatch (bf16 rows).  Result contract of ht::dispatch
 * (kernels/api.cuh:115-160; kernels/nixl_ep_ht.cu:1109-1243): destination d's rows start at
 * recv_row_offset[d] in the concatenated outputs and are ordered by source rank, then by
 * source token index; top-k indices are rebased to d's local experts (-1 elsewhere) and
 * weights of non-local selections are zero.
 *   recv_row_offset  [R + 1] int64 device array (exclusive prefix of per-destination totals)
 *   recv_x           [total][H] bf16;  recv_topk_idx [total][K];  recv_topk_weights [total][K]
 *   recv_src_meta    [total][2] int32 = {source rank, source token}
 */
int
nixl_amd_ep_ht_dispatch(void *recv_x,
                        int32_t *recv_topk_idx,
                        float *recv_topk_weights,
                        int32_t *recv_src_meta,
                        const void *x,
                        const int32_t *topk_idx,
                        const float *topk_weights,
                        const uint8_t *is_token_in_rank,
                        const int *recv_gbl_rank_prefix_sum,
                        const int *send_head,
                        const int64_t *recv_row_offset,
                        int num_tokens,
                        int hidden,
                        int num_topk,
                        int num_ranks,
                        int num_experts,
                        void *stream);

/*
 * Normal-mode dispatch of rows of any element type, with optional per-token scales: the
 * (x, x_scales) form of ht::dispatch, which the reference uses for fp8 rows
 * (csrc/nixl_ep.cpp:701-711 argument checks, :840-857 launch; kernels/nixl_ep_ht.cu:729 reads
 * scale i of a token at token * scale_token_stride + i * scale_hidden_stride, :1198-1209
 * writes recv_x_scales densely as [total][num_scales]).
 *   x, recv_x          rows of `hidden` elements of `elem_bytes` (1, 2 or 4) bytes; a row is a
 *                      multiple of 16 bytes and at most 16 KiB
 *   x_scales           32-bit words (fp32, or packed UE8M0 as int32), addressed as
 *                      rank * scale_rank_stride + token * scale_token_stride +
 *                      i * scale_hidden_stride (strides in words, so that a transposed
 *                      tensor can be passed as it is); NULL with num_scales 0 for no scales
 *   recv_x_scales      [total][num_scales] words, row order as recv_x
 * Everything else as nixl_amd_ep_ht_dispatch, which is this call with elem_bytes 2 and no
 * scales.
 */
int
nixl_amd_ep_ht_dispatch_scaled(void *recv_x,
                               void *recv_x_scales,
                               int32_t *recv_topk_idx,
                               float *recv_topk_weights,
                               int32_t *recv_src_meta,
                               const void *x,
                               const void *x_scales,
                               const int32_t *topk_idx,
                               const float *topk_weights,
                               const uint8_t *is_token_in_rank,
                               const int *recv_gbl_rank_prefix_sum,
                               const int *send_head,
                               const int64_t *recv_row_offset,
                               int num_tokens,
                               int hidden,
                               int elem_bytes,
                               int num_scales,
                               int64_t scale_rank_stride,
                               int64_t scale_token_stride,
                               int64_t scale_hidden_stride,
                               int num_topk,
                               int num_ranks,
                               int num_experts,
                               void *stream);

/*
 * Normal-mode combine.  Replaces ht::combine with one reduction stage
 * (kernels/api.cuh:176-203; combine_token, kernels/nixl_ep_ht.cu:1682-1737):
 * combined_x[r][t] = bf16( float(bias_0) + float(bias_1) + sum over destination ranks that
 * hold the token, ascending, of float(x[row]) ); no weights are applied to x;
 * combined_topk_weights[r][t][k] = sum over those ranks of topk_weights[row][k].
 * bias_0, bias_1, topk_weights and combined_topk_weights may be NULL.
 */
int
nixl_amd_ep_ht_combine(void *combined_x,
                       float *combined_topk_weights,
                       const void *x,
                       const float *topk_weights,
                       const void *bias_0,
                       const void *bias_1,
                       const uint8_t *is_token_in_rank,
                       const int *recv_gbl_rank_prefix_sum,
                       const int *send_head,
                       const int64_t *recv_row_offset,
                       int num_tokens,
                       int hidden,
                       int num_topk,
                       int num_ranks,
                       void *stream);

/*
 * Router: for every token the K largest logits (descending, ties to the lower expert
 * index) and the softmax over those K logits in fp32.  No counterpart in the reference,
 * whose callers pass top-k indices in (examples/device/ep/tests/elastic/elastic.py:153-158).
 *   logits [num_tokens][E] float;  topk_idx [num_tokens][K] int32;  topk_weights float
 */
int
nixl_amd_ep_router_topk(const float *logits,
                        int32_t *topk_idx,
                        float *topk_weights,
                        int num_tokens,
                        int num_experts,
                        int num_topk,
                        void *stream);

/* Element-wise fp32 -> e4m3 codes with the kernels' own encoder (round-to-nearest-even,
 * saturating); exists so that the encoder can be checked exhaustively. */
int
nixl_amd_ep_f32_to_e4m3(const float *in, uint8_t *out, size_t n, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* NIXL_AMD_EP_H */
