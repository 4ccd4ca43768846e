// Low-latency expert-parallel dispatch and combine for all virtual ranks of one GPU, and
// the C ABI that launches them (declared in include/nixl_amd_ep.h).
//
// What the reference does per rank with three passes over the payload (cast into a send
// buffer, K message copies into per-(expert, source rank) receive slots, repack into the
// per-expert contiguous output; kernels/nixl_ep_ll.cu:134-393) is done here in launches
// that touch the payload once, because every "remote" slot is an address in the same HBM:
//   1. ll_bits_kernel      one workgroup per 64 consecutive tokens of a rank builds, in LDS,
//                          one 64-bit word per expert (bit j: token j of the group selected the
//                          expert) and writes it to bits[e][rank][group]: every word has one
//                          writer, so nothing is cleared beforehand and nothing is atomic in
//                          global memory.  With logits instead of top-k indices the same
//                          kernel does the routing first (a wave per token) and writes the
//                          indices and weights out as well.  This is the send phase.
//   1b. ll_arrival_kernel  only for calls with a time-out: the receive side's bounded wait for
//                          each source rank's bits; a late rank loses its bits and is masked.
//   2. ll_dispatch_kernel  one workgroup per token reads its bf16 row once and, while the row
//                          travels, counts for each of its K experts the bits in front of its
//                          own (tokens of lower ranks, then lower tokens of its rank): that is
//                          its row inside the expert.  It quantises the row in registers and
//                          writes it straight to its K final rows of packed_recv_x, plus
//                          src_info and one row of inverse scales per token.  Workgroup e
//                          also turns expert e's bits into layout_range, recv_count and the
//                          statistics.
//   3. ll_scales_kernel    fp8 only: moves the per-token scales into their column-major place
//                          per expert, 64 rows at a time through LDS.
// Step 1 moves 0.3 MB, step 3 the scales (twice 16 MB at 32 x 128 x 7168, top-8); step 2 moves the payload.
// The order this produces is the canonical one among those the reference's atomics allow:
// segments by source rank ascending, tokens ascending inside a segment.
//
// HBM traffic per token (H hidden, K selections, G = H/128): read 2H, write
// K * (H + 4G + 4) for fp8 or K * (2H + 4) for bf16.
//
// Combine is one launch: one workgroup per token locates its K rows through the dispatch
// handle, reads them once and accumulates in fp32 with fused multiply-adds in top-k order
// (kernels/nixl_ep_ll.cu:959-1012).  Traffic per token: read K * 2H, write 2H.
#include <algorithm>
#include <atomic>
#include <cstdint>
#include <mutex>

#include "common.h"
#include "ep_common.h"
#include "nixl_amd_ep.h"

namespace {

constexpr int kBitsThreads = 256; // index path: two (token, k) entries per thread at top-8
constexpr int kRouteThreads = 1024; // routing path: 16 waves, a token each
constexpr int kRouteTokens = 16;
constexpr int kGroupTokens = 64; // tokens per word of the selection bits
constexpr int kMaxTopk = 16; // reference limit, kernels/nixl_ep_ll.cu:412,421
constexpr int kRouterMaxPerLane = 16; // E <= 1024 when routing
// Words of the workspace header: [0] status of the last dispatch on this workspace, [1] arrival
// stamp of its last send phase, [2] id of the last call in which a token repeated an expert,
// [3] id of the last call, [4] kSentMagic ^ [1], which tells a receive phase that a send phase
// wrote [1] (and not whoever had the memory before).
constexpr size_t kWorkspaceHeader = 256;
constexpr int kSentMagic = 0x5e4d1a7c;
constexpr uint64_t kMaxTimeoutUs = 100ull * 1000 * 1000; // 100 s, the upper end of the reference's defaults

struct LlDims {
    int R, T, H, K, E, El, M, N;
};

__device__ __forceinline__ bool
pair_blocked(const int *mask, int R, int a, int b) {
    return mask != nullptr && (mask[a * R + b] != 0 || mask[b * R + a] != 0);
}

__device__ __forceinline__ int
wave_sum(int v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1)
        v += __shfl_xor(v, off);
    return v;
}

// ---- 1. selection bits (and routing) -------------------------------------------------------------

struct BitsArgs {
    unsigned long long *bits; // [E][R][Wr]
    int *group_status; // [R][Wr]: bit 0: a token of the group names an expert twice; bits 1..: arrival stamp
    int *header; // workspace header; [1] receives the arrival stamp of this call
    int32_t *topk_idx; // [R][T][K]; written when routing, read otherwise
    float *topk_weights; // [R][T][K], routing only
    const float *logits; // [R][T][E], routing only
    const int *num_tokens_per_rank;
    const int *mask;
    LlDims d;
    int Wr; // words (groups of 64 tokens) per rank
    int stamp; // arrival stamp of this call (0 when nobody checks arrivals)
    int call_id; // never 0; header[3] receives it, and header[2] too if some group holds a repeated expert
    int withhold_rank; // this rank's groups leave their stamp out (its counts "never arrive"), or -1
};

// Index path: grid = R * Wr workgroups, one per word (64 tokens).  Routing path: grid =
// R * Wr * 4 workgroups, one per quarter word (16 tokens, a wave each), so that the routing
// runs as wide as a token-per-wave router; a quarter is written as its own 16-bit word.
// Dynamic LDS: E words.
template<bool ROUTE, int PL>
__global__ void __launch_bounds__(ROUTE ? kRouteThreads : kBitsThreads)
ll_bits_kernel(BitsArgs a) {
    constexpr int kTokens = ROUTE ? kRouteTokens : kGroupTokens; // tokens of this workgroup
    extern __shared__ unsigned long long words[]; // [E]
    __shared__ int dup;
    __shared__ int sel_i[ROUTE ? kTokens : 1][kMaxTopk];
    const LlDims d = a.d;
    const int tid = threadIdx.x, n_threads = blockDim.x;
    const int per_rank = a.Wr * (kGroupTokens / kTokens); // workgroups per rank
    const int r = blockIdx.x / per_rank, t0 = (blockIdx.x % per_rank) * kTokens;
    const int nt = a.num_tokens_per_rank ? min(a.num_tokens_per_rank[r], d.T) : d.T;
    for (int e = tid; e < d.E; e += n_threads)
        words[e] = 0ull;
    if (tid == 0) dup = 0;

    if constexpr (ROUTE) {
        // K rounds of a wave-wide argmax per token; lane l holds experts l, l + 64, ...
        const int lane = tid & (kWaveSize - 1), j = tid / kWaveSize;
        if (t0 + j < d.T) {
            const float *row = a.logits + (static_cast<size_t>(r) * d.T + t0 + j) * d.E;
            float v[PL];
            unsigned taken = 0;
#pragma unroll
            for (int q = 0; q < PL; ++q) {
                const int e = q * kWaveSize + lane;
                v[q] = e < d.E ? row[e] : 0.f;
                if (e >= d.E) taken |= 1u << q;
            }
            float mine = 0.f, first = 0.f; // lane k keeps the k-th selected logit
            int mine_i = 0;
            for (int k = 0; k < d.K; ++k) {
                float top;
                int win;
                router_round<PL>(v, taken, lane, top, win);
                if (k == 0) first = top;
                if (lane == k) {
                    mine = top;
                    mine_i = win;
                }
            }
            // softmax over the K selected logits, summed in selection order by lane 0
            const float ex = lane < d.K ? expf(mine - first) : 0.f;
            float sum = 0.f;
            for (int k = 0; k < d.K; ++k)
                sum += __shfl(ex, k);
            if (lane < d.K) {
                const size_t at = (static_cast<size_t>(r) * d.T + t0 + j) * d.K + lane;
                a.topk_idx[at] = mine_i;
                a.topk_weights[at] = ex / sum;
                sel_i[j][lane] = mine_i;
            }
        }
    }
    __syncthreads();

    const int32_t *idx = a.topk_idx + (static_cast<size_t>(r) * d.T + t0) * d.K;
    for (int p = tid; p < kTokens * d.K; p += n_threads) {
        const int j = p / d.K;
        if (t0 + j >= nt) break;
        const int e = ROUTE ? sel_i[j][p % d.K] : idx[p];
        if (e < 0 || e >= d.E || pair_blocked(a.mask, d.R, r, e / d.El)) continue;
        const unsigned long long old = atomicOr(&words[e], 1ull << j);
        if ((old >> j) & 1ull) dup = 1; // the same expert twice in one token's selection
    }
    __syncthreads();
    const size_t W = static_cast<size_t>(d.R) * a.Wr;
    if constexpr (ROUTE) {
        auto *quarters = reinterpret_cast<unsigned short *>(a.bits);
        for (int e = tid; e < d.E; e += n_threads)
            quarters[e * W * (kGroupTokens / kTokens) + blockIdx.x] = static_cast<unsigned short>(words[e]);
    } else {
        for (int e = tid; e < d.E; e += n_threads)
            a.bits[e * W + blockIdx.x] = words[e];
        // The stamp goes out with the flag, after this group's words: what a receiver that
        // checks arrivals (ll_arrival_kernel) waits for.
        if (tid == 0 && r != a.withhold_rank) a.group_status[blockIdx.x] = dup | (a.stamp << 1);
        if (tid == 0 && blockIdx.x == 0) {
            a.header[1] = a.stamp;
            a.header[3] = a.call_id;
            a.header[4] = kSentMagic ^ a.stamp;
        }
        // One word tells the kernels behind this one whether ANY group holds a repeat: it carries
        // this call's id then, and an older call's id (or whatever the memory held) otherwise.
        if (tid == 0 && dup) a.header[2] = a.call_id;
    }
}

// ---- 1b. arrival check (the receive side's bounded wait) -----------------------------------------
//
// The reference's receivers spin on each source rank's count with a cycle budget; when it
// runs out they set mask_buffer[src] and take the rank as having sent nothing
// (kernels/nixl_ep_ll.cu:316-340).  Here the counts are the selection bits, and a group's bits
// have arrived when its flag word carries this call's stamp.  One workgroup, a lane per source
// rank: wait (at most `timeout` ticks of the constant-rate wall clock) until every group of the
// rank is stamped; a rank that is not loses its bits (so the kernels behind this one place and
// count nothing of it) and is masked for every destination.  Ranks whose stamps are there,
// which is every rank unless the send side was told to withhold one, cost one pass over their
// flags.
struct ArrivalArgs {
    unsigned long long *bits; // [E][R][Wr]
    int *group_status; // [R][Wr]
    const int *header; // [1]: the stamp to wait for
    int *mask; // [R][R]
    long long *wait_stats; // [R] ticks waited per source rank, accumulated; may be null
    long long timeout; // wall-clock ticks
    long long max_polls; // second bound of the wait, should the clock not advance
    int R, E, Wr;
};

constexpr int kArrivalThreads = 256;

__global__ void __launch_bounds__(kArrivalThreads)
ll_arrival_kernel(ArrivalArgs a) {
    extern __shared__ int late[]; // [R]
    const int stamp = a.header[1];
    // A header that no send phase wrote (a receive phase issued on its own, or on another
    // workspace) holds no stamp anybody will ever publish: nothing is waited for then, and every
    // rank whose flags do not happen to match is masked at once.
    const bool sent = a.header[4] == (kSentMagic ^ stamp);
    int any_late = 0;
    for (int r = threadIdx.x; r < a.R; r += kArrivalThreads) {
        const int *flags = a.group_status + r * a.Wr;
        // the usual case first: everything is there, one pass of independent loads and no clock
        bool here = true;
        for (int w = 0; w < a.Wr; ++w)
            here &= (__hip_atomic_load(flags + w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 1) == stamp;
        long long waited = 0;
        if (!here && sent) {
            const long long start = wall_clock64();
            long long polls = 0;
            do {
                here = true;
                for (int w = 0; w < a.Wr; ++w)
                    here &= (__hip_atomic_load(flags + w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 1) == stamp;
                waited = wall_clock64() - start;
            } while (!here && waited <= a.timeout && ++polls < a.max_polls);
        }
        late[r] = here ? 0 : 1;
        if (a.wait_stats && waited) a.wait_stats[r] += waited;
        if (!here) {
            any_late = 1;
            for (int dst = 0; dst < a.R; ++dst)
                a.mask[dst * a.R + r] = 1;
            for (int w = 0; w < a.Wr; ++w)
                a.group_status[r * a.Wr + w] = 0;
        }
    }
    if (!__syncthreads_or(any_late)) return;
    // bits of the late ranks: every thread takes words of every expert
    const int words = a.R * a.Wr;
    for (int i = threadIdx.x; i < a.E * words; i += kArrivalThreads)
        if (late[(i % words) / a.Wr]) a.bits[i] = 0ull;
}

// ---- 2. cast + scatter ----------------------------------------------------------------------------

struct DispatchArgs {
    uint8_t *recv_x;
    float *token_scales; // [R][T][H/128] inverse scales, one row per source token
    int *src_info;
    long long *layout_range;
    int *recv_count;
    int *stats;
    const uint16_t *x;
    const int32_t *topk_idx;
    const int *num_tokens_per_rank;
    const unsigned long long *bits; // [E][R][Wr]
    const int *group_status; // [n_flags]; bit 0: some token of the group names an expert twice
    const int *mask; // [R][R] or null: pairs of ranks whose selections were left out of the bits
    int n_flags; // R * Wr, or 0 when the selection was made here (a top-k never repeats an expert)
    int *status; // workspace header
    int *rows_out; // [R][T][K] final row e * N + slot, -1 if none; may be null
    LlDims d;
    int Wr;
    int round_scale;
    int parts; // workgroups per token; each covers blockDim.x of the token's H/16 lanes
};

// A call in which some token names an expert twice: one bit per (expert, token) cannot carry
// how often, so nothing is counted from the bits then; every count comes from the selection
// itself.  Selections of expert `e` among the (token, selection) pairs of rank `r` that come
// before (until_t, until_k) in token-major order, taking tokens first, first + step, ...
// (until_t >= T counts the whole rank).  Every such pair owns a row of the expert, as in the
// reference (kernels/nixl_ep_ll.cu:186-190: a slot per selection).  Slow on purpose: a top-k
// selection never repeats an expert, so this only runs for hand-made index tensors.
__device__ __forceinline__ int
selections_before(const DispatchArgs &a, int e, int r, int first, int step, int until_t, int until_k) {
    const LlDims d = a.d;
    if (pair_blocked(a.mask, d.R, r, e / d.El)) return 0; // such selections were left out of the bits as well
    const int nt = a.num_tokens_per_rank ? min(a.num_tokens_per_rank[r], d.T) : d.T;
    const int32_t *idx = a.topk_idx + static_cast<size_t>(r) * d.T * d.K;
    int n = 0;
    for (int t = first; t < nt && t <= until_t; t += step) {
        const int ks = t == until_t ? until_k : d.K;
        for (int k = 0; k < ks; ++k)
            n += idx[static_cast<size_t>(t) * d.K + k] == e;
    }
    return n;
}

// Whether some group of this call holds a repeated expert (see ll_bits_kernel): decided once per
// workgroup from two header words, so that calls without repeats, which is every call whose
// selection is a top-k, run the same instructions as if repeats did not exist.
__device__ __forceinline__ bool
call_has_repeats(const DispatchArgs &a) {
    return a.n_flags != 0 && a.status[2] == a.status[3];
}

// layout_range, recv_count and statistics of expert e from its bits (or, in a call with
// repeats, from the selection); one wave.
template<bool REPEATS>
__device__ __forceinline__ void
expert_meta(const DispatchArgs &a, int e, int lane) {
    const LlDims d = a.d;
    const unsigned long long *bw = a.bits + static_cast<size_t>(e) * d.R * a.Wr;
    int carry = 0;
    for (int r0 = 0; r0 < d.R; r0 += kWaveSize) {
        const int r = r0 + lane;
        int n_r = 0;
        if (r < d.R) {
            if constexpr (REPEATS)
                n_r = selections_before(a, e, r, 0, 1, d.T, 0);
            else
                for (int w = 0; w < a.Wr; ++w)
                    n_r += __popcll(bw[static_cast<size_t>(r) * a.Wr + w]);
        }
        int incl = n_r;
#pragma unroll
        for (int off = 1; off < kWaveSize; off <<= 1) {
            const int up = __shfl_up(incl, off);
            if (lane >= off) incl += up;
        }
        incl += carry;
        if (r < d.R)
            a.layout_range[static_cast<size_t>(e) * d.R + r] =
                static_cast<long long>(static_cast<unsigned>(n_r)) | (static_cast<long long>(incl - n_r) << 32);
        carry = __shfl(incl, kWaveSize - 1);
    }
    if (lane == 0) {
        a.recv_count[e] = carry;
        if (a.stats) a.stats[e] += carry;
    }
}

// 1 if any group of 64 tokens reported a repeated expert; one wave.
__device__ __forceinline__ void
reduce_status(const DispatchArgs &a, int lane) {
    int any = 0;
    for (int g = lane; g < a.n_flags; g += kWaveSize)
        any |= a.group_status[g] & 1;
    any = wave_sum(any);
    if (lane == 0) a.status[0] = any ? NIXL_AMD_EP_STATUS_DUPLICATE_EXPERT : 0;
}

// For a call without tokens: grid = ceil(E / 4) workgroups of 4 waves, a wave per expert.
__global__ void __launch_bounds__(256)
ll_meta_kernel(DispatchArgs a) {
    const int lane = threadIdx.x & (kWaveSize - 1);
    const int e = blockIdx.x * 4 + threadIdx.x / kWaveSize;
    if (e < a.d.E) expert_meta<false>(a, e, lane); // no tokens, no repeats
    if (e == 0) reduce_status(a, lane);
}

// grid = R*T*parts workgroups.  A token's row is H/16 "lanes" of 16 consecutive channels
// (32 bytes of bf16, 16 bytes of fp8), so a 128-channel scale group is 8 neighbouring
// lanes; a workgroup covers blockDim.x of them (a multiple of 64).
template<bool FP8>
__global__ void __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(8, 8)))
ll_dispatch_kernel(DispatchArgs a) {
    const LlDims d = a.d;
    const int tid = threadIdx.x;
    const int wlane = tid & (kWaveSize - 1), wave = tid / kWaveSize, n_waves = blockDim.x / kWaveSize;
    __shared__ int row_of_k[kMaxTopk]; // e * N + slot, or -1
    const int token = blockIdx.x / a.parts, part = blockIdx.x % a.parts;
    const int r = token / d.T, t = token % d.T;
    const int nt = a.num_tokens_per_rank ? min(a.num_tokens_per_rank[r], d.T) : d.T;

    // This token's selections, one per lane, ahead of the row so that they arrive first.
    const int sel = (wlane < d.K && t < nt) ? a.topk_idx[(static_cast<size_t>(r) * d.T + t) * d.K + wlane] : -1;
    // The row is requested next so that it travels while the rows are being located.
    const int lane = part * blockDim.x + tid; // lane of the token's row
    const bool active = lane < d.H / 16 && t < nt;
    uint4 raw0 = make_uint4(0, 0, 0, 0), raw1 = raw0;
    if (active) {
        const uint4 *src = reinterpret_cast<const uint4 *>(a.x + (static_cast<size_t>(r) * d.T + t) * d.H) + lane * 2;
        raw0 = ld16_nt(src);
        raw1 = ld16_nt(src + 1);
    }

    // Receive-side metadata: the workgroup of token i derives it for experts i, i + R*T, ...
    const bool repeats = call_has_repeats(a);
    if (part == 0 && wave == n_waves - 1)
        for (int e = token; e < d.E; e += d.R * d.T) {
            if (repeats)
                expert_meta<true>(a, e, wlane);
            else
                expert_meta<false>(a, e, wlane);
        }
    if (blockIdx.x == 0 && wave == 0) reduce_status(a, wlane);

    if (t >= nt) {
        if (part == 0 && tid < d.K && a.rows_out) a.rows_out[(static_cast<size_t>(r) * d.T + t) * d.K + tid] = -1;
        return;
    }

    // Row of selection k inside expert e: the bits of e in front of this token's own bit.
    // Half a wave per selection: its 32 lanes fetch the words in parallel.
    const int wi = r * a.Wr + (t >> 6); // this token's word
    for (int k = tid >> 5; k < d.K; k += blockDim.x >> 5) {
        const int q0 = tid & 31;
        const int e = __shfl(sel, k);
        int row = -1, cnt = 0;
        unsigned long long own = 0ull;
        if (e >= 0 && e < d.E) {
            const unsigned long long *bw = a.bits + static_cast<size_t>(e) * d.R * a.Wr;
            own = bw[wi];
            if (!repeats) {
                if (q0 == 0) cnt = __popcll(own & ((1ull << (t & 63)) - 1ull));
                for (int j = q0; j < wi; j += 32)
                    cnt += __popcll(bw[j]);
            } else {
                // This selection's place among the (rank, token, selection) triples that name the
                // expert, in that order: the order of the reference's per-selection slots when
                // ranks and tokens are taken in turn.  The 32 lanes share the tokens out.
                cnt = selections_before(a, e, r, q0, 32, t, k);
                for (int rr = 0; rr < r; ++rr)
                    cnt += selections_before(a, e, rr, q0, 32, d.T, 0);
            }
        }
        cnt += __shfl_xor(cnt, 16);
        cnt += __shfl_xor(cnt, 8);
        cnt += __shfl_xor(cnt, 4);
        cnt += __shfl_xor(cnt, 2);
        cnt += __shfl_xor(cnt, 1);
        // cnt < N unless repeats push an expert beyond the rows it owns: such a row is dropped
        if (((own >> (t & 63)) & 1ull) && cnt < d.N) row = e * d.N + cnt;
        if (q0 == 0) row_of_k[k] = row;
    }
    uint4 q = make_uint4(0, 0, 0, 0);
    if constexpr (FP8) {
        const uint32_t w[8] = {raw0.x, raw0.y, raw0.z, raw0.w, raw1.x, raw1.y, raw1.z, raw1.w};
        float v[16];
        float amax = 1e-4f; // floor of the maximum, kernels/nixl_ep_ll.cu:155
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            v[2 * j] = bf16_lo_to_f32(w[j]);
            v[2 * j + 1] = bf16_hi_to_f32(w[j]);
            amax = fmaxf(amax, fmaxf(fabsf(v[2 * j]), fabsf(v[2 * j + 1])));
        }
        // maximum over the 8 lanes of one 128-channel group
        amax = fmaxf(amax, __shfl_xor(amax, 1));
        amax = fmaxf(amax, __shfl_xor(amax, 2));
        amax = fmaxf(amax, __shfl_xor(amax, 4));
        float scale, scale_inv;
        fp8_scales(amax, a.round_scale != 0, scale, scale_inv);
        if (active && (lane & 7) == 0)
            a.token_scales[(static_cast<size_t>(r) * d.T + t) * (d.H / 128) + (lane >> 3)] = scale_inv;
        uint32_t out[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            out[j] = e4m3_pack4(v[4 * j] * scale, v[4 * j + 1] * scale, v[4 * j + 2] * scale, v[4 * j + 3] * scale);
        q = make_uint4(out[0], out[1], out[2], out[3]);
    }
    __syncthreads();
    // Publish the rows (combine reads them back as its row map).
    if (part == 0 && tid < d.K && a.rows_out) a.rows_out[(static_cast<size_t>(r) * d.T + t) * d.K + tid] = row_of_k[tid];

    for (int k = 0; k < d.K; ++k) {
        const int row = row_of_k[k];
        if (row < 0) continue;
        if (lane == 0) a.src_info[row] = t;
        if (!active) continue;
        if constexpr (FP8) {
            st16_stream(reinterpret_cast<uint4 *>(a.recv_x + static_cast<size_t>(row) * d.H) + lane, q);
        } else {
            uint4 *dst = reinterpret_cast<uint4 *>(a.recv_x + static_cast<size_t>(row) * d.H * 2) + lane * 2;
            st16_stream(dst, raw0);
            st16_stream(dst + 1, raw1);
        }
    }
}

// ---- 3. scales, column-major per expert ------------------------------------------------------------
//
// packed_recv_x_scales[e] is [G][N] with the row index fastest (csrc/nixl_ep.cpp:1093-1100,
// kernels/nixl_ep_ll.cu:372-391), so the scales of one received row are G isolated words:
// written from the dispatch kernel they cost more than a quarter of the payload.  Here a
// workgroup takes 64 consecutive rows of one expert, finds their source tokens (src_info
// has the token, the segment the row lies in has the rank), gathers the tokens' scale rows
// (contiguous, 16 bytes per lane) into LDS and writes them out along the row index, 16 bytes
// per lane.

struct ScalesArgs {
    void *recv_scales; // [E][G][N] float, or [E][G/4][N] words of four exponent bytes
    const float *token_scales; // [R][T][G]
    const int *src_info; // [E][N]
    const long long *layout_range; // [E][R]
    LlDims d;
    int use_ue8m0;
    int parts; // workgroups per expert; each takes every parts-th tile of 64 rows
};

constexpr int kScaleThreads = 256;
constexpr int kScaleTile = 64; // rows per tile
constexpr int kScaleParts = 4;

// dynamic LDS: seg_end[R] ints, then tile[64][C + 1] words (C = G, or G / 4 for exponent
// bytes), then source[64] ints.
__global__ void __launch_bounds__(kScaleThreads)
ll_scales_kernel(ScalesArgs a) {
    extern __shared__ int lds[];
    const LlDims d = a.d;
    const int G = d.H / 128;
    const int C = a.use_ue8m0 ? G / 4 : G; // 32-bit words per row in the output
    int *seg_end = lds; // [R]: end of each source rank's segment
    uint32_t *tile = reinterpret_cast<uint32_t *>(lds + d.R); // [64][C + 1]
    int *source = lds + d.R + kScaleTile * (C + 1); // [64]: r * T + t
    const int e = blockIdx.x / a.parts, part = blockIdx.x % a.parts, tid = threadIdx.x;
    const int *info = a.src_info + static_cast<size_t>(e) * d.N;

    // the first tile's source tokens are fetched before it is known how many rows exist (in bounds either way)
    int s0 = part * kScaleTile;
    int t_src = (tid < kScaleTile && s0 + tid < d.N) ? info[s0 + tid] : 0;
    for (int r = tid; r < d.R; r += kScaleThreads) {
        const long long lr = a.layout_range[static_cast<size_t>(e) * d.R + r];
        seg_end[r] = static_cast<int>(lr >> 32) + static_cast<int>(lr & 0xffffffffll);
    }
    __syncthreads();
    const int n = seg_end[d.R - 1]; // segments follow each other in rank order
    uint32_t *out = static_cast<uint32_t *>(a.recv_scales) + static_cast<size_t>(e) * C * d.N;

    for (; s0 < n; s0 += a.parts * kScaleTile) {
        const int rows = min(kScaleTile, n - s0);
        if (tid < rows) {
            if (s0 != part * kScaleTile) t_src = info[s0 + tid];
            int lo = 0, hi = d.R - 1; // first rank whose segment ends beyond this row
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                if (seg_end[mid] > s0 + tid)
                    hi = mid;
                else
                    lo = mid + 1;
            }
            source[tid] = lo * d.T + min(max(t_src, 0), d.T - 1);
        }
        __syncthreads();
        // gather: G / 4 lanes per row, 16 bytes each
        const int quads = G / 4;
        for (int i = tid; i < rows * quads; i += kScaleThreads) {
            const int row = i / quads, q4 = i % quads;
            const float4 v = *reinterpret_cast<const float4 *>(a.token_scales + static_cast<size_t>(source[row]) * G + q4 * 4);
            if (!a.use_ue8m0) {
                uint32_t *dst = tile + row * (C + 1) + q4 * 4;
                dst[0] = __float_as_uint(v.x);
                dst[1] = __float_as_uint(v.y);
                dst[2] = __float_as_uint(v.z);
                dst[3] = __float_as_uint(v.w);
            } else {
                // one exponent byte per group, four groups per 32-bit word
                tile[row * (C + 1) + q4] = ((__float_as_uint(v.x) >> 23) & 0xffu) | (((__float_as_uint(v.y) >> 23) & 0xffu) << 8) |
                    (((__float_as_uint(v.z) >> 23) & 0xffu) << 16) | (((__float_as_uint(v.w) >> 23) & 0xffu) << 24);
            }
        }
        __syncthreads();
        // scatter: 16 lanes per column of the tile, four consecutive rows per lane
        const bool wide = (d.N & 3) == 0;
        for (int i = tid; i < C * (kScaleTile / 4); i += kScaleThreads) {
            const int c = i / (kScaleTile / 4), r4 = (i % (kScaleTile / 4)) * 4;
            if (r4 >= rows) continue;
            uint32_t *dst = out + static_cast<size_t>(c) * d.N + s0 + r4;
            const uint32_t v0 = tile[r4 * (C + 1) + c];
            if (wide && r4 + 3 < rows) {
                *reinterpret_cast<uint4 *>(dst) =
                    make_uint4(v0, tile[(r4 + 1) * (C + 1) + c], tile[(r4 + 2) * (C + 1) + c], tile[(r4 + 3) * (C + 1) + c]);
            } else {
                dst[0] = v0;
                for (int k = 1; k < 4 && r4 + k < rows; ++k)
                    dst[k] = tile[(r4 + k) * (C + 1) + c];
            }
        }
        __syncthreads();
    }
}

// ---- combine --------------------------------------------------------------------------------

struct CombineArgs {
    uint16_t *combined;
    const uint16_t *x;
    const int32_t *topk_idx;
    const float *topk_weights;
    const int *src_info;
    const long long *layout_range;
    const int *mask;
    const int *num_tokens_per_rank;
    const int *row_map; // optional [R][T][K] from dispatch; replaces the search below
    LlDims d;
    int parts; // workgroups per token; each covers blockDim.x of the token's H/8 lanes
};

// LogFMT-10 as the reference's combine sender encodes a row and its receiver decodes it
// (kernels/nixl_ep_ll.cu:459-616), applied in registers: v holds a lane's 8 magnitudes of one
// row, 16 neighbouring lanes hold one 128-channel group.  A group is cast when
// log2(amax) < 0 and the floored log2(amin) is below it; a magnitude then becomes
// floor(max(log2(x) * step_inv + rounding - log_amin * step_inv, 0)) and comes back as
// exp2((code - 1) * step + log_amin), or 0 for code 0.  Signs are kept by the caller.
__device__ __forceinline__ void
logfmt_roundtrip(float (&v)[8]) {
    float amax = 0.f, amin = INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        amax = fmaxf(amax, v[j]);
        amin = fminf(amin, v[j]);
    }
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
        amax = fmaxf(amax, __shfl_xor(amax, off));
        amin = fminf(amin, __shfl_xor(amin, off));
    }
    const float log_amax = log2f(amax);
    const float log_amin = fmaxf(log2f(amin), log_amax - 32.0f);
    if (!(log_amax < 0.0f && log_amin < log_amax)) return; // uniform over the 16 lanes
    const float step = (log_amax - log_amin) / 510.0f;
    const float step_inv = 1.0f / step;
    const float rounding = 2.0f - log2f((1.0f + exp2f(step)) * 0.5f) * step_inv;
    const float fused_rounding = rounding - log_amin * step_inv;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float pos = fmaxf(fmaf(log2f(v[j]), step_inv, fused_rounding), 0.0f);
        const uint32_t code = static_cast<uint32_t>(floorf(pos));
        v[j] = code == 0 ? 0.0f : exp2f(fmaf(static_cast<float>(code - 1), step, log_amin));
    }
}

// grid = R*T*parts workgroups; a token's row is H/8 lanes of 8 consecutive channels (16
// bytes); a workgroup covers blockDim.x of them (a multiple of 64).
template<bool LOGFMT>
__global__ void __launch_bounds__(1024)
ll_combine_kernel(CombineArgs a) {
    const LlDims d = a.d;
    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1), wave = tid / kWaveSize, n_waves = blockDim.x / kWaveSize;
    const int token = blockIdx.x / a.parts, part = blockIdx.x % a.parts;
    const int r = token / d.T, t = token % d.T;
    const int nt = a.num_tokens_per_rank ? min(a.num_tokens_per_rank[r], d.T) : d.T;
    if (t >= nt) return;
    const int col = part * blockDim.x + tid; // lane of the token's row
    __shared__ long long row_of_k[kMaxTopk];
    __shared__ float weight_of_k[kMaxTopk];

    if (a.row_map) {
        // Rows recorded by dispatch: one load per selection instead of a search.
        if (tid < d.K) {
            const size_t sel = (static_cast<size_t>(r) * d.T + t) * d.K + tid;
            const int e = a.topk_idx[sel];
            long long row = a.row_map[sel];
            if (e < 0 || e >= d.E || pair_blocked(a.mask, d.R, r, e / d.El)) row = -1;
            if (row >= static_cast<long long>(d.E) * d.N) row = -1; // a foreign handle must not make the kernel fault
            row_of_k[tid] = row;
            weight_of_k[tid] = a.topk_weights[sel];
        }
    } else
    // Locate the K rows: wave w searches selections w, w + n_waves, ...
    for (int k = wave; k < d.K; k += n_waves) {
        const size_t sel = (static_cast<size_t>(r) * d.T + t) * d.K + k;
        const int e = a.topk_idx[sel];
        long long row = -1;
        if (e >= 0 && e < d.E && !pair_blocked(a.mask, d.R, r, e / d.El)) {
            const long long lr = a.layout_range[static_cast<size_t>(e) * d.R + r];
            int n = static_cast<int>(lr & 0xffffffffll), begin = static_cast<int>(lr >> 32);
            begin = min(max(begin, 0), d.N); // the handle comes from the caller: keep the search inside the expert
            n = min(max(n, 0), d.N - begin);
            const int *seg = a.src_info + static_cast<size_t>(e) * d.N + begin;
            for (int i0 = 0; i0 < n && row < 0; i0 += kWaveSize) {
                const int i = i0 + lane;
                const bool hit = i < n && seg[i] == t;
                const unsigned long long m = __ballot(hit);
                if (m) row = static_cast<long long>(e) * d.N + begin + i0 + (__ffsll(static_cast<long long>(m)) - 1);
            }
        }
        if (lane == 0) {
            row_of_k[k] = row;
            weight_of_k[k] = a.topk_weights[sel];
        }
    }
    __syncthreads();
    if (col >= d.H / 8) return;

    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < d.K; k0 += 8) {
        uint4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const long long row = (k0 + j < d.K) ? row_of_k[k0 + j] : -1;
            v[j] = make_uint4(0, 0, 0, 0);
            if (row >= 0)
                v[j] = ld16_nt(reinterpret_cast<const uint4 *>(a.x + static_cast<size_t>(row) * d.H) + col);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (k0 + j >= d.K || row_of_k[k0 + j] < 0) continue;
            const float w = weight_of_k[k0 + j];
            const uint32_t u[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
            if constexpr (LOGFMT) {
                float mag[8];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    mag[2 * c] = bf16_lo_to_f32(u[c] & 0x7fff7fffu);
                    mag[2 * c + 1] = bf16_hi_to_f32(u[c] & 0x7fff7fffu);
                }
                logfmt_roundtrip(mag);
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    acc[2 * c] = fmaf((u[c] & 0x8000u) ? -mag[2 * c] : mag[2 * c], w, acc[2 * c]);
                    acc[2 * c + 1] = fmaf((u[c] & 0x80000000u) ? -mag[2 * c + 1] : mag[2 * c + 1], w, acc[2 * c + 1]);
                }
            } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    acc[2 * c] = fmaf(bf16_lo_to_f32(u[c]), w, acc[2 * c]);
                    acc[2 * c + 1] = fmaf(bf16_hi_to_f32(u[c]), w, acc[2 * c + 1]);
                }
            }
        }
    }
    uint4 out;
    out.x = f32_to_bf16(acc[0]) | (f32_to_bf16(acc[1]) << 16);
    out.y = f32_to_bf16(acc[2]) | (f32_to_bf16(acc[3]) << 16);
    out.z = f32_to_bf16(acc[4]) | (f32_to_bf16(acc[5]) << 16);
    out.w = f32_to_bf16(acc[6]) | (f32_to_bf16(acc[7]) << 16);
    st16_nt(reinterpret_cast<uint4 *>(a.combined + (static_cast<size_t>(r) * d.T + t) * d.H) + col, out);
}

// The combine side of the bounded wait (kernels/nixl_ep_ll.cu:846-866): a receiver waits for
// the flag of each rank whose experts' rows it is about to read and masks a rank whose flag
// does not come.  Here a flag is a word the caller's expert step sets when the rank's rows
// are complete; one workgroup, a lane per rank.
struct ReadyArgs {
    const int *ready; // [R], nonzero: the rank's expert outputs are there
    int *mask; // [R][R]
    long long *wait_stats; // [R], may be null
    long long timeout; // wall-clock ticks
    long long max_polls; // second bound of the wait, should the clock not advance
    int R;
};

__global__ void __launch_bounds__(kArrivalThreads)
ll_ready_kernel(ReadyArgs a) {
    for (int r = threadIdx.x; r < a.R; r += kArrivalThreads) {
        const long long start = wall_clock64();
        long long waited = 0, polls = 0;
        bool here;
        do {
            here = __hip_atomic_load(a.ready + r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0;
            waited = wall_clock64() - start;
        } while (!here && waited <= a.timeout && ++polls < a.max_polls);
        if (a.wait_stats) a.wait_stats[r] += waited;
        if (!here)
            for (int dst = 0; dst < a.R; ++dst)
                a.mask[dst * a.R + r] = 1;
    }
}

// Four values per thread through the same routine as the dispatch kernel, so that a NaN's
// neighbours are covered too; the last thread pads with zeros.
__global__ void
f32_to_e4m3_kernel(const float *in, uint8_t *out, size_t n) {
    const size_t i = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
    if (i >= n) return;
    float v[4];
    for (int j = 0; j < 4; ++j)
        v[j] = i + j < n ? in[i + j] : 0.f;
    const uint32_t codes = e4m3_pack4(v[0], v[1], v[2], v[3]);
    for (int j = 0; j < 4 && i + j < n; ++j)
        out[i + j] = static_cast<uint8_t>(codes >> (8 * j));
}

int
check_dims(const char *who, int T, int H, int M, int K, int R, int E, LlDims &d) {
    auto bad = [&](const std::string &why) { return nixl_amd_fail(NIXL_AMD_ERR_INVALID, std::string(who) + ": " + why); };
    if (R <= 0 || E <= 0 || E % R != 0) return bad("num_experts must be a positive multiple of num_ranks");
    if (T < 0 || M <= 0 || T > M) return bad("num_tokens must be in [0, num_max_dispatch_tokens_per_rank]");
    if (K <= 0 || K > kMaxTopk) return bad("num_topk must be in [1, 16]");
    if (H <= 0 || H % 128 != 0 || H > 8192) return bad("hidden must be a multiple of 128, at most 8192");
    if (static_cast<long long>(R) * M > (1ll << 30)) return bad("num_ranks * max tokens too large");
    d = LlDims{R, T, H, K, E, E / R, M, R * M};
    return NIXL_AMD_OK;
}

int
round_up_wave(int n) {
    return (n + kWaveSize - 1) / kWaveSize * kWaveSize;
}

// Largest workgroup (in lanes) of the dispatch and combine kernels; a token whose row needs
// more lanes is split over several workgroups.
// Read by every call, set by nixl_amd_ep_ll_set_tuning from any thread: a call sees the old or the
// new value, never a torn one.  Combine, while nobody has set it (0): a row of more than 512
// lanes is split into two halves (hidden 7168: two workgroups of 448 lanes, 91.6 us against
// 94.4 for one of 896; 128 and 64 lanes: 93.6-94.4).
std::atomic<int> g_dispatch_lanes{1024};
std::atomic<int> g_combine_lanes{0};

} // namespace

// Scratch of the entry point that allocates nothing (nixl_amd_ep_ll_dispatch_static): the
// dispatch workspace lives in this array instead of in memory the caller brings.  Every GPU
// the library runs on holds its own copy, at its own address, until the process ends.  The
// array's name is only a host-side handle for hipGetSymbolAddress; host code passes kernels
// the per-device address kept in g_scratch_ptr and never the name itself.
constexpr size_t kStaticScratchBytes = NIXL_AMD_EP_LL_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

// Address of the current device's copy of `scratch`; resolved once per device.
int
static_scratch(void **out) {
    int dev = -1;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_dispatch_static: device id out of range");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return nixl_amd_fail(NIXL_AMD_ERR_HIP, "ll_dispatch_static: the scratch array has no device address");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return NIXL_AMD_OK;
}

} // namespace

extern "C" {

int
nixl_amd_ep_ll_set_tuning(int dispatch_lanes, int combine_lanes) {
    auto ok = [](int v) { return v == 0 || v == -1 || (v >= 64 && v <= 1024 && v % 64 == 0); };
    if (!ok(dispatch_lanes) || !ok(combine_lanes))
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_set_tuning: lanes must be 0, -1 or a multiple of 64 in [64, 1024]");
    // -1: back to what the library starts with
    if (dispatch_lanes) g_dispatch_lanes.store(dispatch_lanes == -1 ? 1024 : dispatch_lanes, std::memory_order_relaxed);
    if (combine_lanes) g_combine_lanes.store(combine_lanes == -1 ? 0 : combine_lanes, std::memory_order_relaxed);
    return NIXL_AMD_OK;
}

size_t
nixl_amd_ep_ll_workspace_bytes(int num_ranks, int num_experts, int num_tokens, int num_topk, int hidden) {
    if (num_ranks <= 0 || num_experts <= 0 || num_tokens < 0 || num_topk <= 0 || hidden < 0) return 0;
    const size_t groups = static_cast<size_t>(num_ranks) * ((num_tokens + kGroupTokens - 1) / kGroupTokens);
    const size_t flags = (groups * sizeof(int) + 255) / 256 * 256;
    const size_t bits = static_cast<size_t>(num_experts) * groups * sizeof(unsigned long long);
    const size_t scales = static_cast<size_t>(num_ranks) * num_tokens * (hidden / 128) * sizeof(float);
    return kWorkspaceHeader + flags + (bits + 255) / 256 * 256 + scales;
}

} // extern "C"

namespace {

struct LlDispatchCall {
    void *packed_recv_x;
    void *packed_recv_x_scales;
    int *packed_recv_src_info;
    int64_t *packed_recv_layout_range;
    int *packed_recv_count;
    const int *mask_buffer;
    int *stats;
    const void *x;
    int32_t *topk_idx; // input, or output when logits are given
    const float *logits; // null: indices come from the caller
    float *topk_weights; // output, with logits only
    const int *num_tokens_per_rank;
    int num_tokens, hidden, max_tokens, num_topk, num_ranks, num_experts;
    int use_fp8, round_scale, use_ue8m0;
    int *row_map;
    void *workspace;
    size_t workspace_bytes;
    void *stream;
    // phased / elastic calls only
    int phases = 3; // bit 0: send (selection bits and their arrival stamps), bit 1: receive (everything else)
    uint64_t timeout_us = 0; // > 0: the receive phase checks arrivals first
    int withhold_rank = -1;
    int64_t *wait_stats = nullptr;
    int *mask_rw = nullptr; // the mask buffer again, writable: late ranks are entered here
};

// Stamps of calls that check arrivals: 1 .. 2^30 - 1, never 0 (the stamp of calls that do not).
std::atomic<uint32_t> g_arrival_stamp{0};
// Every send phase gets an id of its own (never 0), see BitsArgs::call_id.
std::atomic<uint32_t> g_call_id{0};

template<bool ROUTE>
void
launch_bits(int per_lane, dim3 grid, size_t lds, hipStream_t s, const BitsArgs &a) {
    constexpr int threads = ROUTE ? kRouteThreads : kBitsThreads;
    if (!ROUTE || per_lane <= 1)
        hipLaunchKernelGGL((ll_bits_kernel<ROUTE, 1>), grid, dim3(threads), lds, s, a);
    else if (per_lane <= 2)
        hipLaunchKernelGGL((ll_bits_kernel<ROUTE, 2>), grid, dim3(threads), lds, s, a);
    else if (per_lane <= 4)
        hipLaunchKernelGGL((ll_bits_kernel<ROUTE, 4>), grid, dim3(threads), lds, s, a);
    else if (per_lane <= 8)
        hipLaunchKernelGGL((ll_bits_kernel<ROUTE, 8>), grid, dim3(threads), lds, s, a);
    else
        hipLaunchKernelGGL((ll_bits_kernel<ROUTE, 16>), grid, dim3(threads), lds, s, a);
}

int
ll_dispatch_impl(const char *who, const LlDispatchCall &c) {
    auto bad = [&](int code, const std::string &why) { return nixl_amd_fail(code, std::string(who) + ": " + why); };
    LlDims d;
    const int rc = check_dims(who, c.num_tokens, c.hidden, c.max_tokens, c.num_topk, c.num_ranks, c.num_experts, d);
    if (rc) return rc;
    if (!c.packed_recv_x || !c.packed_recv_src_info || !c.packed_recv_layout_range || !c.packed_recv_count || !c.workspace ||
        (d.T > 0 && (!c.x || !c.topk_idx || (c.logits && !c.topk_weights)))) // a call without tokens reads no input
        return bad(NIXL_AMD_ERR_INVALID, "null pointer argument");
    if (c.use_fp8 && c.hidden % 512 != 0) // same restriction as csrc/nixl_ep.cpp:1091
        return bad(NIXL_AMD_ERR_INVALID, "fp8 needs hidden % 512 == 0");
    if (c.use_fp8 && !c.packed_recv_x_scales) return bad(NIXL_AMD_ERR_INVALID, "scales pointer is null");
    if (c.use_ue8m0 && !(c.use_fp8 && c.round_scale)) // kernels/nixl_ep_ll.cu:428-430
        return bad(NIXL_AMD_ERR_INVALID, "UE8M0 scales need use_fp8 and round_scale");
    if (c.workspace_bytes < nixl_amd_ep_ll_workspace_bytes(d.R, d.E, d.T, d.K, d.H))
        return bad(NIXL_AMD_ERR_INVALID, "workspace too small");
    if (reinterpret_cast<uintptr_t>(c.workspace) % 16 != 0) return bad(NIXL_AMD_ERR_INVALID, "workspace must be 16-byte aligned");
    if (c.use_fp8 && reinterpret_cast<uintptr_t>(c.packed_recv_x_scales) % 16 != 0)
        return bad(NIXL_AMD_ERR_INVALID, "packed_recv_x_scales must be 16-byte aligned");
    if (static_cast<long long>(d.E) * d.N >= (1ll << 31))
        return bad(NIXL_AMD_ERR_TOO_LARGE, "num_experts * num_ranks * max tokens must be below 2^31");
    if (static_cast<size_t>(d.E) * sizeof(unsigned long long) > 48 * 1024) return bad(NIXL_AMD_ERR_TOO_LARGE, "more than 6144 experts");
    if (static_cast<size_t>(d.R) * sizeof(int) > 32 * 1024) return bad(NIXL_AMD_ERR_TOO_LARGE, "more than 8192 ranks");
    if (c.logits && (d.E > kRouterMaxPerLane * kWaveSize || d.K > d.E))
        return bad(NIXL_AMD_ERR_INVALID, "routing needs num_experts <= 1024 and num_topk <= num_experts");
    if (c.phases < 1 || c.phases > 3) return bad(NIXL_AMD_ERR_INVALID, "phases must be 1 (send), 2 (receive) or 3 (both)");
    if (c.withhold_rank < -1 || c.withhold_rank >= d.R) return bad(NIXL_AMD_ERR_INVALID, "withhold_rank is not a rank");
    if (c.timeout_us > 0 && !c.mask_rw) // the reference traps when a wait runs out without a mask buffer
        return bad(NIXL_AMD_ERR_INVALID, "a time-out needs a mask buffer to record late ranks in");
    if (c.withhold_rank >= 0 && (c.timeout_us == 0 || c.timeout_us > 1000000))
        return bad(NIXL_AMD_ERR_INVALID, "a withheld rank is waited for: the time-out must be between 1 us and 1 s");
    if (c.timeout_us > kMaxTimeoutUs) return bad(NIXL_AMD_ERR_INVALID, "the time-out may be at most 100 s");

    hipStream_t s = static_cast<hipStream_t>(c.stream);
    const int Wr = (d.T + kGroupTokens - 1) / kGroupTokens;
    const size_t groups = static_cast<size_t>(d.R) * Wr;
    auto *base = static_cast<uint8_t *>(c.workspace);
    int *status = reinterpret_cast<int *>(base);
    int *group_status = reinterpret_cast<int *>(base + kWorkspaceHeader);
    const size_t off_bits = kWorkspaceHeader + (groups * sizeof(int) + 255) / 256 * 256;
    auto *bits = reinterpret_cast<unsigned long long *>(base + off_bits);
    auto *token_scales =
        reinterpret_cast<float *>(base + off_bits + (static_cast<size_t>(d.E) * groups * sizeof(unsigned long long) + 255) / 256 * 256);

    if (groups > 0 && (c.phases & 1)) {
        BitsArgs b{};
        b.bits = bits;
        b.group_status = group_status;
        b.header = status;
        b.withhold_rank = c.withhold_rank;
        b.call_id = static_cast<int>(g_call_id.fetch_add(1, std::memory_order_relaxed) % 0x7fffffffu) + 1;
        if (c.timeout_us > 0) {
            const uint32_t n = g_arrival_stamp.fetch_add(1, std::memory_order_relaxed) % 0x3fffffffu;
            b.stamp = static_cast<int>(n + 1);
        }
        b.topk_idx = c.topk_idx;
        b.topk_weights = c.topk_weights;
        b.logits = c.logits;
        b.num_tokens_per_rank = c.num_tokens_per_rank;
        b.mask = c.mask_buffer;
        b.d = d;
        b.Wr = Wr;
        const size_t lds = static_cast<size_t>(d.E) * sizeof(unsigned long long);
        if (c.logits)
            launch_bits<true>((d.E + kWaveSize - 1) / kWaveSize, dim3(static_cast<unsigned>(groups) * (kGroupTokens / kRouteTokens)), lds,
                              s, b);
        else
            launch_bits<false>(1, dim3(static_cast<unsigned>(groups)), lds, s, b);
        HIP_TRY(hipGetLastError());
    }
    if (!(c.phases & 2)) return NIXL_AMD_OK;

    if (groups > 0 && c.timeout_us > 0) {
        int dev = 0, khz = 0;
        HIP_TRY(hipGetDevice(&dev));
        HIP_TRY(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev));
        if (khz <= 0) return bad(NIXL_AMD_ERR_HIP, "the device reports no wall clock rate");
        ArrivalArgs w{};
        w.bits = bits;
        w.group_status = group_status;
        w.header = status;
        w.mask = c.mask_rw;
        w.wait_stats = reinterpret_cast<long long *>(c.wait_stats);
        w.timeout = static_cast<long long>(c.timeout_us * static_cast<uint64_t>(khz) / 1000u);
        // a poll is a round trip to memory (hundreds of ns): 16 a microsecond only happen if the clock stands still
        w.max_polls = static_cast<long long>(c.timeout_us) * 16 + 1024;
        w.R = d.R;
        w.E = d.E;
        w.Wr = Wr;
        hipLaunchKernelGGL(ll_arrival_kernel, dim3(1), dim3(kArrivalThreads), static_cast<size_t>(d.R) * sizeof(int), s, w);
        HIP_TRY(hipGetLastError());
    }

    DispatchArgs a{};
    a.recv_x = static_cast<uint8_t *>(c.packed_recv_x);
    a.token_scales = token_scales;
    a.src_info = c.packed_recv_src_info;
    a.layout_range = reinterpret_cast<long long *>(c.packed_recv_layout_range);
    a.recv_count = c.packed_recv_count;
    a.stats = c.stats;
    a.x = static_cast<const uint16_t *>(c.x);
    a.topk_idx = c.topk_idx;
    a.num_tokens_per_rank = c.num_tokens_per_rank;
    a.bits = bits;
    a.group_status = group_status;
    a.mask = c.mask_buffer;
    a.n_flags = c.logits ? 0 : static_cast<int>(groups);
    a.status = status;
    a.rows_out = c.row_map;
    a.d = d;
    a.Wr = Wr;
    a.round_scale = c.round_scale;
    if (d.T == 0) {
        hipLaunchKernelGGL(ll_meta_kernel, dim3((d.E + 3) / 4), dim3(256), 0, s, a);
        HIP_TRY(hipGetLastError());
        return NIXL_AMD_OK;
    }
    const int wg = std::min(round_up_wave(d.H / 16), g_dispatch_lanes.load(std::memory_order_relaxed));
    a.parts = (d.H / 16 + wg - 1) / wg;
    const dim3 grid(static_cast<unsigned>(d.R) * d.T * a.parts);
    const dim3 block(wg);
    if (c.use_fp8)
        hipLaunchKernelGGL(ll_dispatch_kernel<true>, grid, block, 0, s, a);
    else
        hipLaunchKernelGGL(ll_dispatch_kernel<false>, grid, block, 0, s, a);
    HIP_TRY(hipGetLastError());

    if (c.use_fp8) {
        ScalesArgs sa{};
        sa.recv_scales = c.packed_recv_x_scales;
        sa.token_scales = token_scales;
        sa.src_info = c.packed_recv_src_info;
        sa.layout_range = reinterpret_cast<const long long *>(c.packed_recv_layout_range);
        sa.d = d;
        sa.use_ue8m0 = c.use_ue8m0;
        sa.parts = kScaleParts;
        const int C = c.use_ue8m0 ? d.H / 512 : d.H / 128;
        const size_t lds = (static_cast<size_t>(d.R) + static_cast<size_t>(kScaleTile) * (C + 1) + kScaleTile) * sizeof(int);
        hipLaunchKernelGGL(ll_scales_kernel, dim3(static_cast<unsigned>(d.E) * sa.parts), dim3(kScaleThreads), lds, s, sa);
        HIP_TRY(hipGetLastError());
    }
    return NIXL_AMD_OK;
}

} // namespace

extern "C" {

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
                        void *stream) {
    const LlDispatchCall c{packed_recv_x, packed_recv_x_scales, packed_recv_src_info, packed_recv_layout_range,
                           packed_recv_count, mask_buffer, cumulative_local_expert_recv_stats, x,
                           const_cast<int32_t *>(topk_idx), nullptr, nullptr, num_tokens_per_rank, num_tokens, hidden,
                           num_max_dispatch_tokens_per_rank, num_topk, num_ranks, num_experts, use_fp8, round_scale,
                           use_ue8m0, row_map, workspace, workspace_bytes, stream};
    return ll_dispatch_impl("ll_dispatch", c);
}

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
                              void *stream) {
    if (!logits) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_route_dispatch: logits is null");
    const LlDispatchCall c{packed_recv_x, packed_recv_x_scales, packed_recv_src_info, packed_recv_layout_range,
                           packed_recv_count, mask_buffer, cumulative_local_expert_recv_stats, x, topk_idx, logits,
                           topk_weights, num_tokens_per_rank, num_tokens, hidden, num_max_dispatch_tokens_per_rank,
                           num_topk, num_ranks, num_experts, use_fp8, round_scale, use_ue8m0, row_map, workspace,
                           workspace_bytes, stream};
    return ll_dispatch_impl("ll_route_dispatch", c);
}

int
nixl_amd_ep_ll_dispatch_status(const void *workspace, void *stream, int *status) {
    if (!workspace || !status) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_dispatch_status: null pointer argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    HIP_TRY(hipMemcpyAsync(status, workspace, sizeof(int), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    return NIXL_AMD_OK;
}

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
                               void *stream) {
    LlDispatchCall c{packed_recv_x, packed_recv_x_scales, packed_recv_src_info, packed_recv_layout_range,
                     packed_recv_count, mask_buffer, cumulative_local_expert_recv_stats, x,
                     const_cast<int32_t *>(topk_idx), nullptr, nullptr, num_tokens_per_rank, num_tokens, hidden,
                     num_max_dispatch_tokens_per_rank, num_topk, num_ranks, num_experts, use_fp8, round_scale,
                     use_ue8m0, row_map, workspace, workspace_bytes, stream};
    c.phases = phases;
    c.timeout_us = timeout_us;
    c.withhold_rank = withhold_rank;
    c.wait_stats = dispatch_wait_recv_cost_stats;
    c.mask_rw = mask_buffer;
    return ll_dispatch_impl("ll_dispatch_phased", c);
}

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
                               void *stream) {
    const size_t need = nixl_amd_ep_ll_workspace_bytes(num_ranks, num_experts, num_tokens, num_topk, hidden);
    if (need > kStaticScratchBytes)
        return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE,
                             "ll_dispatch_static: this shape needs " + std::to_string(need) +
                                 " bytes of scratch, the built-in array holds " + std::to_string(kStaticScratchBytes) +
                                 "; use nixl_amd_ep_ll_dispatch with a workspace of the caller's");
    void *ws = nullptr;
    const int rc = static_scratch(&ws);
    if (rc) return rc;
    // Every word of the workspace that a kernel reads is written earlier in the same call
    // (selection bits and group flags by the first kernel, the status word by the second), so
    // what the previous call left behind needs no clearing.
    return nixl_amd_ep_ll_dispatch(packed_recv_x, packed_recv_x_scales, packed_recv_src_info, packed_recv_layout_range,
                                   packed_recv_count, mask_buffer, cumulative_local_expert_recv_stats, x, topk_idx,
                                   num_tokens_per_rank, num_tokens, hidden, num_max_dispatch_tokens_per_rank, num_topk,
                                   num_ranks, num_experts, use_fp8, round_scale, use_ue8m0, row_map, ws, kStaticScratchBytes,
                                   stream);
}

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
                       void *stream) {
    LlDims d;
    const int rc = check_dims("ll_combine", num_tokens, hidden, num_max_dispatch_tokens_per_rank, num_topk, num_ranks,
                              num_experts, d);
    if (rc) return rc;
    if (!combined_x || !x || !topk_idx || !topk_weights || !src_info || !layout_range)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_combine: null pointer argument");
    if (d.T == 0) return NIXL_AMD_OK;
    CombineArgs a{};
    a.combined = static_cast<uint16_t *>(combined_x);
    a.x = static_cast<const uint16_t *>(x);
    a.topk_idx = topk_idx;
    a.topk_weights = topk_weights;
    a.src_info = src_info;
    a.layout_range = reinterpret_cast<const long long *>(layout_range);
    a.mask = mask_buffer;
    a.num_tokens_per_rank = num_tokens_per_rank;
    a.row_map = row_map;
    a.d = d;
    const int row_lanes = round_up_wave(d.H / 8);
    int wg = g_combine_lanes.load(std::memory_order_relaxed);
    // the LogFMT codec's arithmetic wants more workgroups still (hidden 7168: 99.6 us with 192 lanes, 105 with 448)
    if (wg == 0) wg = row_lanes <= 512 ? row_lanes : (use_logfmt ? 192 : round_up_wave((d.H / 8 + 1) / 2));
    wg = std::min(row_lanes, wg);
    a.parts = (d.H / 8 + wg - 1) / wg;
    const dim3 grid(static_cast<unsigned>(d.R) * d.T * a.parts);
    if (use_logfmt)
        hipLaunchKernelGGL(ll_combine_kernel<true>, grid, dim3(wg), 0, static_cast<hipStream_t>(stream), a);
    else
        hipLaunchKernelGGL(ll_combine_kernel<false>, grid, dim3(wg), 0, static_cast<hipStream_t>(stream), a);
    HIP_TRY(hipGetLastError());
    return NIXL_AMD_OK;
}

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
                               void *stream) {
    if (!mask_buffer || !rank_ready)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_combine_elastic: mask buffer and ready flags are required");
    if (timeout_us == 0 || timeout_us > 1000000)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_combine_elastic: the time-out must be between 1 us and 1 s");
    if (num_ranks <= 0 || num_ranks > 8192) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_combine_elastic: bad number of ranks");
    int dev = 0, khz = 0;
    HIP_TRY(hipGetDevice(&dev));
    HIP_TRY(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev));
    if (khz <= 0) return nixl_amd_fail(NIXL_AMD_ERR_HIP, "ll_combine_elastic: the device reports no wall clock rate");
    ReadyArgs w{};
    w.ready = rank_ready;
    w.mask = mask_buffer;
    w.wait_stats = reinterpret_cast<long long *>(combine_wait_recv_cost_stats);
    w.timeout = static_cast<long long>(timeout_us * static_cast<uint64_t>(khz) / 1000u);
    w.max_polls = static_cast<long long>(timeout_us) * 16 + 1024;
    w.R = num_ranks;
    hipLaunchKernelGGL(ll_ready_kernel, dim3(1), dim3(kArrivalThreads), 0, static_cast<hipStream_t>(stream), w);
    HIP_TRY(hipGetLastError());
    return nixl_amd_ep_ll_combine(combined_x, x, topk_idx, topk_weights, src_info, layout_range, mask_buffer, num_tokens_per_rank,
                                  row_map, num_tokens, hidden, num_max_dispatch_tokens_per_rank, num_topk, num_ranks, num_experts,
                                  use_logfmt, stream);
}

int
nixl_amd_ep_f32_to_e4m3(const float *in, uint8_t *out, size_t n, void *stream) {
    if ((!in || !out) && n) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "f32_to_e4m3: null pointer argument");
    if (n == 0) return NIXL_AMD_OK;
    if (n > (1ull << 38)) return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "f32_to_e4m3: too many elements");
    hipLaunchKernelGGL(f32_to_e4m3_kernel, dim3(static_cast<unsigned>((n + 1023) / 1024)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), in, out, n);
    HIP_TRY(hipGetLastError());
    return NIXL_AMD_OK;
}

} // extern "C"
