/*
 * TEST INFRASTRUCTURE — scalar CPU restatement of the reference's expert-parallel kernels.
 * See ep_oracle.h for the array layouts.  Each function cites the reference code it
 * follows (paths relative to examples/device/ep/csrc/).  Compiled with -ffp-contract=off so
 * that every fused multiply-add below is an explicit fmaf().
 *
 * How each function is pinned (tests/test_ep_oracle.py):
 *   oracle_f32_to_bf16 / oracle_bf16_to_f32   exhaustive over all 65536 bf16 patterns and a
 *       random fp32 sample against torch CPU bfloat16 (library routine)
 *   oracle_f32_to_e4m3 / oracle_e4m3_to_f32   every bf16 value x a set of scales against torch
 *       CPU float8_e4m3fn where |v| <= 464 (above that torch returns NaN while the
 *       reference saturates, kernels/nixl_ep_ll.cu:175 __NV_SATFINITE); the saturating edge,
 *       NaN and the 256 decode values by the OCP FP8 specification
 *   oracle_fp8_scales   the constant 1/448.0f == 0x3B124925; IEEE division for `scale`
 *   oracle_ll_dispatch  the invariants the reference test checks (tests/elastic/elastic.py:
 *       263-318) + brute force against a direct Python restatement on tiny shapes
 *   oracle_ll_combine   closed form; identity experts give x * sum of weights
 *       (tests/elastic/elastic.py:377-387)
 *   oracle_dispatch_layout, oracle_ht_*   the plain-torch recomputation in tests/test_ht.py:
 *       99-152,166-172,223-244,304-323
 *   oracle_router       torch CPU topk / softmax (no reference counterpart: parity with the
 *       reference is unpinned for the router by construction)
 */
#include "ep_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

static inline uint32_t
f2u(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

static inline float
u2f(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* ---- scalar formats ---------------------------------------------------------------- */

float
oracle_bf16_to_f32(uint16_t v) {
    return u2f((uint32_t)v << 16);
}

/* round-to-nearest-even on the upper 16 bits; NaN stays NaN (quiet bit forced) */
uint16_t
oracle_f32_to_bf16(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* OCP FP8 E4M3 ("e4m3fn": bias 7, no infinity, NaN = S.1111.111, max finite 448),
 * round-to-nearest-even, saturating to +-448 (kernels/nixl_ep_ll.cu:175). */
uint8_t
oracle_f32_to_e4m3(float f) {
    const uint32_t u = f2u(f);
    const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    const uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint8_t)(sign | 0x7fu); /* NaN */
    if (a >= f2u(448.0f)) return (uint8_t)(sign | 0x7eu); /* saturate, infinity included */
    if (a < f2u(0.015625f)) {
        /* below the smallest normal 2^-6: multiples of 2^-9; 8 becomes the code of 2^-6 */
        const float q = nearbyintf(u2f(a) * 512.0f);
        return (uint8_t)(sign | (uint8_t)q);
    }
    const uint32_t r = a + 0x7ffffu + ((a >> 20) & 1u); /* RNE at bit 20 */
    const uint32_t e = (r >> 23) - 127u + 7u;
    const uint32_t m = (r >> 20) & 7u;
    return (uint8_t)(sign | (e << 3) | m);
}

float
oracle_e4m3_to_f32(uint8_t v) {
    const int sign = v >> 7, e = (v >> 3) & 15, m = v & 7;
    float mag;
    if (e == 15 && m == 7)
        mag = NAN;
    else if (e == 0)
        mag = ldexpf((float)m, -9);
    else
        mag = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return sign ? -mag : mag;
}

/* kernels/utils.cuh:430-456.  kFinfoAmaxInvE4M3 is the float nearest to 1/448. */
void
oracle_fp8_scales(float amax, int round_scale, float *scale, float *scale_inv) {
    const float amax_inv = 1 / 448.0f;
    if (round_scale) {
        const uint32_t b = f2u(amax * amax_inv);
        const int e = (int)((b >> 23) & 0xff) - 127 + ((b & 0x7fffffu) != 0);
        *scale = u2f((uint32_t)(-e + 127) << 23);
        *scale_inv = u2f((uint32_t)(e + 127) << 23);
    } else {
        *scale_inv = amax * amax_inv;
        *scale = 448.0f / amax;
    }
}

/* kernels/nixl_ep_ll.cu:147-182: amax starts at 1e-4, one scale per 128 channels,
 * q = e4m3(float(x) * scale). */
void
oracle_cast_row_fp8(const uint16_t *x, int hidden, int round_scale, uint8_t *q, float *scale_inv) {
    for (int g = 0; g < hidden / 128; ++g) {
        float amax = 1e-4f;
        for (int j = 0; j < 128; ++j)
            amax = fmaxf(amax, fabsf(oracle_bf16_to_f32(x[g * 128 + j])));
        float scale, inv;
        oracle_fp8_scales(amax, round_scale, &scale, &inv);
        scale_inv[g] = inv;
        for (int j = 0; j < 128; ++j)
            q[g * 128 + j] = oracle_f32_to_e4m3(oracle_bf16_to_f32(x[g * 128 + j]) * scale);
    }
}

void
oracle_f32_to_e4m3_n(const float *in, uint8_t *out, size_t n) {
    for (size_t i = 0; i < n; ++i)
        out[i] = oracle_f32_to_e4m3(in[i]);
}

void
oracle_f32_to_bf16_n(const float *in, uint16_t *out, size_t n) {
    for (size_t i = 0; i < n; ++i)
        out[i] = oracle_f32_to_bf16(in[i]);
}

/* ---- low-latency dispatch ------------------------------------------------------------ */

static inline int
masked(const int32_t *mask, int R, int a, int b) {
    return mask != NULL && mask[(size_t)a * R + b] != 0;
}

/*
 * kernels/nixl_ep_ll.cu:71-395 for every rank of the world.  The two phases are kept:
 *   send  (:134-283)  each rank casts its tokens into messages
 *                     [int4 header: source token index | payload | H/128 float scales]
 *                     and copies message (t, k) into slot `slot` of the receive area
 *                     recv_area[dst rank][local expert][src rank][slot]; the per
 *                     (expert, src rank) count is delivered as count + 1
 *   recv  (:296-393)  each rank packs, per local expert, the segments of all source ranks
 *                     contiguously and records (count, begin) in layout_range
 * The reference hands out slots and segment begins with atomicAdd, so any order inside a
 * segment and any order of segments is a valid result.  This restatement fixes the
 * canonical one: tokens ascending inside a segment, segments by source rank ascending.
 * A token that names an expert more than once takes a slot per selection (:186-190), so the
 * expert receives its row once per selection, next to each other in the canonical order.  More
 * than M selections from one rank to one expert would run past the reference's receive area:
 * refused here with -3.
 * A message travels from a to b only if neither mask[a][b] nor mask[b][a] is set
 * (send side :197,266; receive side :319-338 treats a masked or silent rank as zero tokens).
 */
int
oracle_ll_dispatch(const uint16_t *x, const int32_t *topk_idx, const int32_t *num_tokens, const int32_t *mask,
                   int R, int T, int H, int K, int E, int M, int use_fp8, int round_scale, int use_ue8m0,
                   void *packed_recv_x, void *packed_recv_scales, int32_t *src_info, int64_t *layout_range,
                   int32_t *recv_count, int threads) {
    if (R <= 0 || E % R != 0 || H % 128 != 0 || T > M) return -1;
    if (use_ue8m0 && !(use_fp8 && round_scale)) return -1;
    if (use_fp8 && H % 512 != 0) return -1;
    const int El = E / R, G = H / 128, N = R * M;
    const size_t elem = use_fp8 ? 1 : 2;
    const size_t msg_bytes = 16 + (use_fp8 ? (size_t)H + (size_t)G * 4 : (size_t)H * 2);
    /* receive area of every rank: [R dst][El][R src][M] messages, and the count words */
    const size_t area_msgs = (size_t)R * El * R * M;
    uint8_t *area = (uint8_t *)malloc(area_msgs * msg_bytes);
    int64_t *count_words = (int64_t *)calloc((size_t)R * El * R, sizeof(int64_t));
    if (!area || !count_words) {
        free(area);
        free(count_words);
        return -2;
    }
    (void)threads;
    int overflow = 0; /* a rank names one expert more often than its M slots there hold (only repeats can) */

    /* send phase */
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
    for (int r = 0; r < R; ++r) {
        const int nt = num_tokens ? num_tokens[r] : T;
        uint8_t *msg = (uint8_t *)malloc(msg_bytes);
        int *next_slot = (int *)calloc((size_t)E, sizeof(int));
        for (int t = 0; t < nt; ++t) {
            const uint16_t *row = x + ((size_t)r * T + t) * H;
            int32_t hdr[4] = {t, 0, 0, 0};
            memcpy(msg, hdr, 16);
            if (use_fp8)
                oracle_cast_row_fp8(row, H, round_scale, msg + 16, (float *)(msg + 16 + H));
            else
                memcpy(msg + 16, row, (size_t)H * 2);
            for (int k = 0; k < K; ++k) {
                const int e = topk_idx[((size_t)r * T + t) * K + k];
                if (e < 0) continue;
                const int d = e / El, le = e % El;
                const int slot = next_slot[e]++;
                if (slot >= M) { /* the reference would write past its receive area: refused here */
                    __atomic_store_n(&overflow, 1, __ATOMIC_RELAXED);
                    next_slot[e] = M;
                    continue;
                }
                if (masked(mask, R, r, d)) continue;
                memcpy(area + ((((size_t)d * El + le) * R + r) * M + slot) * msg_bytes, msg, msg_bytes);
            }
        }
        for (int e = 0; e < E; ++e) {
            const int d = e / El, le = e % El;
            if (!masked(mask, R, r, d)) count_words[((size_t)d * El + le) * R + r] = (int64_t)next_slot[e] + 1;
        }
        free(msg);
        free(next_slot);
    }

    /* receive phase */
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
    for (int d = 0; d < R; ++d) {
        for (int le = 0; le < El; ++le) {
            int begin = 0;
            for (int r = 0; r < R; ++r) {
                int64_t w = count_words[((size_t)d * El + le) * R + r];
                if (masked(mask, R, d, r) || w == 0) w = 1; /* masked or silent: zero tokens */
                const int n = (int)(w - 1);
                layout_range[((size_t)d * El + le) * R + r] = (int64_t)(uint32_t)n | ((int64_t)begin << 32);
                for (int i = 0; i < n; ++i) {
                    const uint8_t *m = area + ((((size_t)d * El + le) * R + r) * M + i) * msg_bytes;
                    const size_t row = ((size_t)d * El + le) * N + (size_t)(begin + i);
                    memcpy(&src_info[row], m, 4);
                    memcpy((uint8_t *)packed_recv_x + row * H * elem, m + 16, (size_t)H * elem);
                    if (use_fp8) {
                        const float *sc = (const float *)(m + 16 + H);
                        const size_t tok = (size_t)(begin + i);
                        for (int g = 0; g < G; ++g) {
                            if (!use_ue8m0) {
                                ((float *)packed_recv_scales)[(((size_t)d * El + le) * G + g) * N + tok] = sc[g];
                            } else {
                                /* one exponent byte per group, four groups per int32 word,
                                 * words laid out [H/512][N] (kernels/nixl_ep_ll.cu:372-391) */
                                uint8_t *base = (uint8_t *)packed_recv_scales + ((size_t)d * El + le) * (G / 4) * N * 4;
                                base[((size_t)(g / 4) * N + tok) * 4 + (g % 4)] = (uint8_t)(f2u(sc[g]) >> 23);
                            }
                        }
                    }
                }
                begin += n;
            }
            recv_count[(size_t)d * El + le] = begin;
        }
    }
    free(area);
    free(count_words);
    return overflow ? -3 : 0;
}

/*
 * LogFMT-10 as the combine sender applies it to one row and the receiver undoes it
 * (kernels/nixl_ep_ll.cu:459-528 encode, :530-562 amax/amin check, :564-616 decode): per 128
 * channels, with amax / amin the largest / smallest magnitude, the group is cast when
 * log2(amax) < 0 and log2(amin) (floored at log2(amax) - 32) < log2(amax); a magnitude x
 * becomes code = floor(max(log2(x) * step_inv + rounding - log_amin * step_inv, 0)) with
 * step = (log_amax - log_amin) / 510, and comes back as 0 for code 0, else
 * exp2((code - 1) * step + log_amin), with the sign restored.  Groups that are not cast pass
 * unchanged.  The reference evaluates log2 / exp2 with approximate hardware instructions
 * (lg2.approx, ex2.approx); libm stands in here, so results agree with any GPU only to the
 * accuracy of those instructions: PARITY UNPINNED at bit level, checked by tolerance.
 */
void
oracle_logfmt_roundtrip(const uint16_t *row, int hidden, float *out) {
    for (int g0 = 0; g0 < hidden; g0 += 128) {
        float amax = 0.0f, amin = INFINITY;
        for (int j = 0; j < 128; ++j) {
            const float a = fabsf(oracle_bf16_to_f32(row[g0 + j]));
            amax = fmaxf(amax, a);
            amin = fminf(amin, a);
        }
        const float log_amax = log2f(amax);
        const float log_amin = fmaxf(log2f(amin), log_amax - 32.0f);
        const int cast = log_amax < 0.0f && log_amin < log_amax;
        if (!cast) {
            for (int j = 0; j < 128; ++j)
                out[g0 + j] = oracle_bf16_to_f32(row[g0 + j]);
            continue;
        }
        const float step = (log_amax - log_amin) / 510.0f;
        const float step_inv = 1.0f / step;
        const float rounding = 2.0f - log2f((1.0f + exp2f(step)) * 0.5f) * step_inv;
        const float fused_rounding = rounding - log_amin * step_inv;
        for (int j = 0; j < 128; ++j) {
            const uint16_t bits = row[g0 + j];
            const float a = oracle_bf16_to_f32((uint16_t)(bits & 0x7fffu));
            const float pos = fmaxf(fmaf(log2f(a), step_inv, fused_rounding), 0.0f);
            const uint32_t code = (uint32_t)floorf(pos);
            const float dec = code == 0 ? 0.0f : exp2f(fmaf((float)(code - 1), step, log_amin));
            out[g0 + j] = (bits & 0x8000u) ? -dec : dec;
        }
    }
}

/*
 * kernels/nixl_ep_ll.cu:618-1017.  Send (:683-837): expert rank d copies row `i` of local
 * expert le, for i in the segment of source rank r, into r's slot (global expert * M +
 * src_info[i]).  Receive (:875-1016): token t accumulates, in top-k order,
 * float(row) * weight in fp32 (decode_and_accumulate bf16 branch :608-615; nvcc contracts
 * the multiply-add, so use_fma = 1 is the reference build) and rounds to bf16.
 * Selections with idx < 0 or on a masked rank are skipped (:930-932,972-974).
 */
int
oracle_ll_combine(const uint16_t *expert_out, const int32_t *topk_idx, const float *topk_weights,
                  const int32_t *src_info, const int64_t *layout_range, const int32_t *num_tokens,
                  const int32_t *mask, int R, int T, int H, int K, int E, int M, int flags,
                  uint16_t *combined, int threads) {
    if (R <= 0 || E % R != 0) return -1;
    const int use_fma = flags & 1, use_logfmt = (flags >> 1) & 1; /* the cast always accumulates fused */
    if (use_logfmt && H % 128 != 0) return -1;
    const int El = E / R, N = R * M;
    /* slot area of every rank: [R][E][M] -> row index into expert_out, or -1 */
    int64_t *slot_row = (int64_t *)malloc((size_t)R * E * M * sizeof(int64_t));
    if (!slot_row) return -2;
    for (size_t i = 0; i < (size_t)R * E * M; ++i)
        slot_row[i] = -1;
    for (int d = 0; d < R; ++d)
        for (int le = 0; le < El; ++le)
            for (int r = 0; r < R; ++r) {
                if (masked(mask, R, d, r)) continue;
                const int64_t lr = layout_range[((size_t)d * El + le) * R + r];
                const int n = (int)(lr & 0xffffffff), begin = (int)(lr >> 32);
                for (int i = begin; i < begin + n; ++i) {
                    const size_t row = ((size_t)d * El + le) * N + (size_t)i;
                    slot_row[((size_t)r * E + (size_t)(d * El + le)) * M + src_info[row]] = (int64_t)row;
                }
            }
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
    for (int r = 0; r < R; ++r) {
        const int nt = num_tokens ? num_tokens[r] : T;
        float *acc = (float *)malloc((size_t)H * sizeof(float));
        float *dec = (float *)malloc((size_t)H * sizeof(float));
        for (int t = 0; t < nt; ++t) {
            for (int h = 0; h < H; ++h)
                acc[h] = 0.0f;
            for (int k = 0; k < K; ++k) {
                const int e = topk_idx[((size_t)r * T + t) * K + k];
                if (e < 0 || masked(mask, R, r, e / El)) continue;
                const int64_t row = slot_row[((size_t)r * E + e) * M + t];
                if (row < 0) continue; /* never sent: the receiver times out and masks the rank */
                const float w = topk_weights[((size_t)r * T + t) * K + k];
                const uint16_t *src = expert_out + (size_t)row * H;
                if (use_logfmt) {
                    oracle_logfmt_roundtrip(src, H, dec);
                    for (int h = 0; h < H; ++h)
                        acc[h] = fmaf(dec[h], w, acc[h]);
                } else if (use_fma)
                    for (int h = 0; h < H; ++h)
                        acc[h] = fmaf(oracle_bf16_to_f32(src[h]), w, acc[h]);
                else
                    for (int h = 0; h < H; ++h)
                        acc[h] = acc[h] + oracle_bf16_to_f32(src[h]) * w;
            }
            uint16_t *out = combined + ((size_t)r * T + t) * H;
            for (int h = 0; h < H; ++h)
                out[h] = oracle_f32_to_bf16(acc[h]);
        }
        free(acc);
        free(dec);
    }
    free(slot_row);
    return 0;
}

/* The reduction of one token on explicit rows: out = bf16(sum_k float(rows[k]) * w[k]) in
 * top-k order, fused (use_fma) or as separate multiply and add.  Lets a test check single
 * tokens of a large run without building the whole world on the CPU. */
void
oracle_weighted_sum_rows(const uint16_t *rows, const float *w, int K, int H, int use_fma, uint16_t *out) {
    for (int h = 0; h < H; ++h) {
        float acc = 0.0f;
        for (int k = 0; k < K; ++k) {
            const float v = oracle_bf16_to_f32(rows[(size_t)k * H + h]);
            acc = use_fma ? fmaf(v, w[k], acc) : acc + v * w[k];
        }
        out[h] = oracle_f32_to_bf16(acc);
    }
}

/* ---- normal mode ----------------------------------------------------------------------- */

/* kernels/layout.cu:31-138: tokens per expert, tokens per rank (a token counts once per
 * rank however many of its experts live there), and the token-in-rank matrix. */
void
oracle_dispatch_layout(const int32_t *topk_idx, int T, int K, int R, int E, int32_t *num_tokens_per_rank,
                       int32_t *num_tokens_per_expert, uint8_t *is_token_in_rank) {
    const int El = E / R;
    memset(num_tokens_per_rank, 0, (size_t)R * sizeof(int32_t));
    memset(num_tokens_per_expert, 0, (size_t)E * sizeof(int32_t));
    memset(is_token_in_rank, 0, (size_t)T * R);
    for (int t = 0; t < T; ++t) {
        for (int k = 0; k < K; ++k) {
            const int e = topk_idx[(size_t)t * K + k];
            if (e < 0 || e >= E) continue;
            ++num_tokens_per_expert[e];
            is_token_in_rank[(size_t)t * R + e / El] = 1;
        }
        for (int r = 0; r < R; ++r)
            num_tokens_per_rank[r] += is_token_in_rank[(size_t)t * R + r];
    }
}

/* kernels/nixl_ep_ht.cu:257-314 (receive-side prefix over source ranks, per-expert counts
 * rounded up to expert_alignment) and :324-373 (per destination, inclusive prefix over
 * channels; a channel is a contiguous range of ceil(T / C) tokens, kernels/utils.cuh:395-400). */
void
oracle_ht_notify(const uint8_t *is_token_in_rank, const int32_t *per_expert, int R, int T, int E, int C,
                 int expert_alignment, int32_t *recv_rank_prefix, int32_t *recv_expert_count,
                 int32_t *channel_prefix) {
    const int El = E / R;
    const int per_channel = (T + C - 1) / C;
    for (int d = 0; d < R; ++d) {
        int sum = 0;
        for (int r = 0; r < R; ++r) {
            for (int t = 0; t < T; ++t)
                sum += is_token_in_rank[((size_t)r * T + t) * R + d];
            recv_rank_prefix[(size_t)d * R + r] = sum;
        }
        for (int le = 0; le < El; ++le) {
            int n = 0;
            for (int r = 0; r < R; ++r)
                n += per_expert[(size_t)r * E + d * El + le];
            recv_expert_count[(size_t)d * El + le] = (n + expert_alignment - 1) / expert_alignment * expert_alignment;
        }
    }
    for (int r = 0; r < R; ++r)
        for (int d = 0; d < R; ++d) {
            int sum = 0;
            for (int c = 0; c < C; ++c) {
                int lo = per_channel * c, hi = lo + per_channel;
                if (lo > T) lo = T;
                if (hi > T) hi = T;
                for (int t = lo; t < hi; ++t)
                    sum += is_token_in_rank[((size_t)r * T + t) * R + d];
                channel_prefix[((size_t)r * R + d) * C + c] = sum;
            }
        }
}

/* Result contract of kernels/nixl_ep_ht.cu:1109-1243: destination d receives its rows
 * ordered by source rank, then by source token index; top-k indices are rebased to the
 * destination's local experts (-1 elsewhere) and the weights of non-local selections are
 * zeroed (:1221-1233). */
void
oracle_ht_dispatch(const uint16_t *x, const int32_t *topk_idx, const float *topk_weights,
                   const uint8_t *is_token_in_rank, const int32_t *recv_rank_prefix, int R, int T, int H, int K,
                   int E, const int64_t *row_offset, uint16_t *recv_x, int32_t *recv_topk_idx,
                   float *recv_topk_weights, int32_t *recv_src_rank, int32_t *recv_src_token,
                   int32_t *send_head) {
    const int El = E / R;
    for (int r = 0; r < R; ++r)
        for (int d = 0; d < R; ++d) {
            int pos = 0;
            const int seg_begin = r == 0 ? 0 : recv_rank_prefix[(size_t)d * R + r - 1];
            for (int t = 0; t < T; ++t) {
                if (!is_token_in_rank[((size_t)r * T + t) * R + d]) {
                    send_head[((size_t)r * T + t) * R + d] = -1;
                    continue;
                }
                send_head[((size_t)r * T + t) * R + d] = pos;
                const size_t row = (size_t)row_offset[d] + (size_t)seg_begin + (size_t)pos;
                memcpy(recv_x + row * H, x + ((size_t)r * T + t) * H, (size_t)H * 2);
                for (int k = 0; k < K; ++k) {
                    int e = topk_idx[((size_t)r * T + t) * K + k];
                    const int local = (e >= d * El && e < (d + 1) * El);
                    recv_topk_idx[row * K + k] = local ? e - d * El : -1;
                    recv_topk_weights[row * K + k] = local ? topk_weights[((size_t)r * T + t) * K + k] : 0.0f;
                }
                recv_src_rank[row] = r;
                recv_src_token[row] = t;
                ++pos;
            }
        }
}

/* kernels/nixl_ep_ht.cu:1682-1737 (combine_token, single reduction stage): fp32 sum of the
 * two optional bias rows, then of the rows held by the ranks that received the token, in
 * ascending rank order, no weights applied to x; top-k weights are summed separately. */
void
oracle_ht_combine(const uint16_t *recv_x, const float *recv_topk_weights, const uint8_t *is_token_in_rank,
                  const int32_t *recv_rank_prefix, const int32_t *send_head, const int64_t *row_offset,
                  const uint16_t *bias0, const uint16_t *bias1, int R, int T, int H, int K, uint16_t *combined,
                  float *combined_topk_weights) {
    float *acc = (float *)malloc((size_t)H * sizeof(float));
    for (int r = 0; r < R; ++r)
        for (int t = 0; t < T; ++t) {
            const size_t tok = (size_t)r * T + t;
            for (int h = 0; h < H; ++h) {
                const float b0 = bias0 ? oracle_bf16_to_f32(bias0[tok * H + h]) : 0.0f;
                const float b1 = bias1 ? oracle_bf16_to_f32(bias1[tok * H + h]) : 0.0f;
                acc[h] = b0 + b1;
            }
            float wsum[64];
            for (int k = 0; k < K; ++k)
                wsum[k] = 0.0f;
            for (int d = 0; d < R; ++d) {
                if (!is_token_in_rank[tok * R + d]) continue;
                const int seg_begin = r == 0 ? 0 : recv_rank_prefix[(size_t)d * R + r - 1];
                const size_t row = (size_t)row_offset[d] + (size_t)seg_begin + (size_t)send_head[tok * R + d];
                for (int h = 0; h < H; ++h)
                    acc[h] += oracle_bf16_to_f32(recv_x[row * H + h]);
                if (recv_topk_weights)
                    for (int k = 0; k < K; ++k)
                        wsum[k] += recv_topk_weights[row * K + k];
            }
            for (int h = 0; h < H; ++h)
                combined[tok * H + h] = oracle_f32_to_bf16(acc[h]);
            if (combined_topk_weights)
                for (int k = 0; k < K; ++k)
                    combined_topk_weights[tok * K + k] = wsum[k];
        }
    free(acc);
}

/* ---- router ------------------------------------------------------------------------------ */

/* No reference counterpart (its callers pass topk_idx in, tests/elastic/elastic.py:153-158).
 * Selection: K largest logits, descending, ties to the lower expert index.  Weights:
 * softmax over the K selected logits in fp32, exp(l - max) / sum in selection order. */
void
oracle_router(const float *logits, int T, int E, int K, int32_t *topk_idx, float *topk_weights) {
    uint8_t *taken = (uint8_t *)malloc((size_t)E);
    for (int t = 0; t < T; ++t) {
        const float *l = logits + (size_t)t * E;
        memset(taken, 0, (size_t)E);
        float sel[64];
        for (int k = 0; k < K; ++k) {
            int best = -1;
            for (int e = 0; e < E; ++e)
                if (!taken[e] && (best < 0 || l[e] > l[best])) best = e;
            taken[best] = 1;
            topk_idx[(size_t)t * K + k] = best;
            sel[k] = l[best];
        }
        float sum = 0.0f;
        const float top = sel[0]; /* the maximum: selection is in descending order */
        for (int k = 0; k < K; ++k) {
            sel[k] = expf(sel[k] - top);
            sum += sel[k];
        }
        for (int k = 0; k < K; ++k)
            topk_weights[(size_t)t * K + k] = sel[k] / sum;
    }
    free(taken);
}
