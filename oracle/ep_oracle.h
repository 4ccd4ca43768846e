/*
 * TEST INFRASTRUCTURE — scalar CPU restatement of the reference's expert-parallel (EP)
 * kernels, for all virtual ranks of one "world" at once.  Only tests, the smoke check and
 * the CPU-baseline leg of the benchmark link or call this; the product never does.
 *
 * Array layouts (rank-major; R ranks, E experts, El = E / R local experts, T tokens per
 * rank as allocated, K top-k, H hidden, M = max dispatch tokens per rank, N = R * M):
 *   x                 [R][T][H]        bf16 bit patterns
 *   topk_idx          [R][T][K]        int32, -1 = no selection
 *   num_tokens        [R]              tokens actually present on each rank (<= T), or NULL = T
 *   mask              [R][R]           mask[a][b] != 0: rank a treats rank b as failed, or NULL
 *   packed_recv_x     [R][El][N][H]    fp8 e4m3 codes (1 B) or bf16 (2 B)
 *   packed_recv_scales[R][El][H/128][N] float  (column-major per expert: token index fastest)
 *                     or, UE8M0:  [R][El][H/512][N] int32, 4 exponent bytes per word
 *   src_info          [R][El][N]       int32 source token index
 *   layout_range      [R][El][R]       int64: low 32 bits = count, high 32 bits = begin
 *   recv_count        [R][El]          int32
 * Rows of packed_recv_x / scales / src_info at or beyond recv_count are left untouched.
 *
 * Parity unpinned: oracle_router (the reference has no router; pinned against torch CPU only)
 * and oracle_logfmt_roundtrip at bit level (the reference evaluates log2 / exp2 with
 * approximate GPU instructions; pinned against a float64 evaluation of the definition and the
 * codec's error bound).  Everything else is pinned by library routines, format definitions,
 * brute force and the reference tests' invariants (tests/test_ep_oracle.py, tests/test_golden.py).
 */
#ifndef NIXL_AMD_EP_ORACLE_H
#define NIXL_AMD_EP_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* scalar conversions */
float oracle_bf16_to_f32(uint16_t v);
uint16_t oracle_f32_to_bf16(float f);
uint8_t oracle_f32_to_e4m3(float f);
float oracle_e4m3_to_f32(uint8_t v);
void oracle_fp8_scales(float amax, int round_scale, float *scale, float *scale_inv);
/* one token row: H bf16 -> H fp8 codes + H/128 inverse scales */
void oracle_cast_row_fp8(const uint16_t *x, int hidden, int round_scale, uint8_t *q, float *scale_inv);
/* bulk helpers for exhaustive checks */
void oracle_f32_to_e4m3_n(const float *in, uint8_t *out, size_t n);
void oracle_f32_to_bf16_n(const float *in, uint16_t *out, size_t n);

/* low-latency mode */
int oracle_ll_dispatch(const uint16_t *x, const int32_t *topk_idx, const int32_t *num_tokens, const int32_t *mask,
                       int R, int T, int H, int K, int E, int M, int use_fp8, int round_scale, int use_ue8m0,
                       void *packed_recv_x, void *packed_recv_scales, int32_t *src_info, int64_t *layout_range,
                       int32_t *recv_count, int threads);
int oracle_ll_combine(const uint16_t *expert_out, const int32_t *topk_idx, const float *topk_weights,
                      const int32_t *src_info, const int64_t *layout_range, const int32_t *num_tokens,
                      const int32_t *mask, int R, int T, int H, int K, int E, int M, int flags,
                      uint16_t *combined, int threads); /* flags: 1 = fused multiply-add, 2 = LogFMT-10 rows */
/* LogFMT-10 encode + decode of one row (hidden % 128 == 0) into fp32 values */
void oracle_logfmt_roundtrip(const uint16_t *row, int hidden, float *out);

void oracle_weighted_sum_rows(const uint16_t *rows, const float *w, int K, int H, int use_fma, uint16_t *out);

/* normal (high-throughput) mode */
void oracle_dispatch_layout(const int32_t *topk_idx, int T, int K, int R, int E, int32_t *num_tokens_per_rank,
                            int32_t *num_tokens_per_expert, uint8_t *is_token_in_rank);
/* is_token_in_rank [R][T][R]; per_expert [R][E] (counts computed by each source rank).
 * Outputs: recv_rank_prefix [R dst][R src] inclusive; recv_expert_count [R][El] rounded up to
 * expert_alignment; channel_prefix [R src][R dst][C] inclusive over channels. */
void oracle_ht_notify(const uint8_t *is_token_in_rank, const int32_t *per_expert, int R, int T, int E, int C,
                      int expert_alignment, int32_t *recv_rank_prefix, int32_t *recv_expert_count,
                      int32_t *channel_prefix);
/* recv_* arrays are the per-destination outputs concatenated in destination-rank order;
 * row_offset[d] (R + 1 entries) is where destination d starts.  send_head [R][T][R] is the
 * position of token t of rank r inside the (r -> d) segment, or -1. */
void oracle_ht_dispatch(const uint16_t *x, const int32_t *topk_idx, const float *topk_weights,
                        const uint8_t *is_token_in_rank, const int32_t *recv_rank_prefix, int R, int T, int H, int K,
                        int E, const int64_t *row_offset, uint16_t *recv_x, int32_t *recv_topk_idx,
                        float *recv_topk_weights, int32_t *recv_src_rank, int32_t *recv_src_token,
                        int32_t *send_head);
void oracle_ht_combine(const uint16_t *recv_x, const float *recv_topk_weights, const uint8_t *is_token_in_rank,
                       const int32_t *recv_rank_prefix, const int32_t *send_head, const int64_t *row_offset,
                       const uint16_t *bias0, const uint16_t *bias1, int R, int T, int H, int K, uint16_t *combined,
                       float *combined_topk_weights);

/* router: top-k (descending, ties to the lower index) + softmax over the selected logits */
void oracle_router(const float *logits, int T, int E, int K, int32_t *topk_idx, float *topk_weights);

#ifdef __cplusplus
}
#endif
#endif
