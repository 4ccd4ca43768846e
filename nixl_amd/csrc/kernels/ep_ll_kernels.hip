// Low-latency expert-parallel dispatch and combine for all virtual ranks of one GPU, and
// the C ABI that launches them (declared in include/nixl_amd_ep.h).
//
// What the reference does per rank with three passes over the payload (cast into a send
// buffer, K message copies into per-(expert, source rank) receive slots, repack into the
// per-expert contiguous output; kernels/nixl_ep_ll.cu:134-393) is done here in two
// launches that touch the payload once, because every "remote" slot is an address in the
// same HBM:
//   1. ll_layout_kernel    one workgroup per source rank builds, in LDS, one bitmask of
//                          tokens per expert and derives count[r][e] and the position of
//                          every (token, k) inside its (r, e) segment;
//   2. ll_dispatch_kernel  one workgroup per token reads its bf16 row once, quantises it in
//                          registers and writes it straight to its K final rows of
//                          packed_recv_x (row = e * N + sum of the lower source ranks'
//                          counts for e + position), plus src_info and the token's H/128
//                          scales (once, contiguous);
//   3. ll_scales_kernel    workgroups per expert scan the per-rank counts into layout_range,
//                          recv_count and the statistics, and copy each received row's
//                          scales into the column-major scales array with coalesced stores
//                          (writing them from step 2 would be one isolated 4-byte store per
//                          scale).
// Steps 1 and 3 move a few megabytes; step 2 moves the payload.
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
#include <cstdint>
#include <mutex>

#include "common.h"
#include "ep_common.h"
#include "nixl_amd_ep.h"

namespace {

constexpr int kLayoutThreads = 1024; // one (token, k) per thread at 128 tokens x top-8
constexpr int kScaleThreads = 256;
constexpr int kLayoutLdsBytes = 32768;
constexpr int kMaxTopk = 16; // reference limit, kernels/nixl_ep_ll.cu:412,421

struct LlDims {
    int R, T, H, K, E, El, M, N;
};

__device__ __forceinline__ bool
pair_blocked(const int *mask, int R, int a, int b) {
    return mask != nullptr && (mask[a * R + b] != 0 || mask[b * R + a] != 0);
}

// ---- 1. counts and positions ------------------------------------------------------------

// grid = R workgroups.  send_count [R][E]; pos [R][T][K] (position inside the (r, e)
// segment, -1 for no selection / out-of-range expert / blocked rank pair / absent token).
__global__ void __launch_bounds__(kLayoutThreads)
ll_layout_kernel(const int32_t *__restrict__ topk_idx,
                 const int *__restrict__ num_tokens_per_rank,
                 const int *__restrict__ mask,
                 int *__restrict__ send_count,
                 int *__restrict__ pos,
                 LlDims d,
                 int experts_per_pass) {
    extern __shared__ unsigned long long bits[]; // [experts_per_pass][W]
    const int r = blockIdx.x;
    const int tid = threadIdx.x;
    const int W = (d.T + 63) / 64;
    const int nt = num_tokens_per_rank ? min(num_tokens_per_rank[r], d.T) : d.T;
    const int32_t *idx = topk_idx + static_cast<size_t>(r) * d.T * d.K;
    int *my_pos = pos + static_cast<size_t>(r) * d.T * d.K;

    for (int p = nt * d.K + tid; p < d.T * d.K; p += kLayoutThreads)
        my_pos[p] = -1;

    for (int e0 = 0; e0 < d.E; e0 += experts_per_pass) {
        const int ne = min(experts_per_pass, d.E - e0);
        for (int i = tid; i < ne * W; i += kLayoutThreads)
            bits[i] = 0ull;
        __syncthreads();
        for (int p = tid; p < nt * d.K; p += kLayoutThreads) {
            const int e = idx[p];
            if (e >= e0 && e < e0 + ne) {
                const int t = p / d.K;
                atomicOr(&bits[(e - e0) * W + (t >> 6)], 1ull << (t & 63));
            }
        }
        __syncthreads();
        for (int i = tid; i < ne; i += kLayoutThreads) {
            int c = 0;
            for (int w = 0; w < W; ++w)
                c += __popcll(bits[i * W + w]);
            const int e = e0 + i;
            send_count[r * d.E + e] = pair_blocked(mask, d.R, r, e / d.El) ? 0 : c;
        }
        for (int p = tid; p < nt * d.K; p += kLayoutThreads) {
            const int e = idx[p];
            if (e0 == 0 && (e < 0 || e >= d.E)) my_pos[p] = -1;
            if (e >= e0 && e < e0 + ne) {
                const int t = p / d.K;
                const unsigned long long *row = bits + (e - e0) * W;
                int c = __popcll(row[t >> 6] & ((1ull << (t & 63)) - 1ull));
                for (int w = 0; w < (t >> 6); ++w)
                    c += __popcll(row[w]);
                my_pos[p] = pair_blocked(mask, d.R, r, e / d.El) ? -1 : c;
            }
        }
        __syncthreads();
    }
}

// ---- 2. cast + scatter ----------------------------------------------------------------------------

struct DispatchArgs {
    uint8_t *recv_x;
    int *src_info;
    float *token_scales; // [R][T][H/128] inverse scales, one row per source token
    const uint16_t *x;
    const int32_t *topk_idx;
    const int *num_tokens_per_rank;
    const int *send_count; // [R][E]
    const int *rows; // [R][T][K] position inside the (r, e) segment, -1 if none
    int *rows_out; // [R][T][K] final row e * N + begin + position, -1 if none
    LlDims d;
    int round_scale;
    int parts; // workgroups per token; each covers blockDim.x of the token's H/16 lanes
};

// grid = R*T*parts workgroups.  A token's row is H/16 "lanes" of 16 consecutive channels
// (32 bytes of bf16, 16 bytes of fp8), so a 128-channel scale group is 8 neighbouring
// lanes; a workgroup covers blockDim.x of them (a multiple of 64).
template<bool FP8>
__global__ void __launch_bounds__(1024)
ll_dispatch_kernel(DispatchArgs a) {
    const LlDims d = a.d;
    const int tid = threadIdx.x;
    __shared__ int row_of_k[kMaxTopk]; // e * N + slot, or -1
    const int token = blockIdx.x / a.parts, part = blockIdx.x % a.parts;
    const int r = token / d.T, t = token % d.T;
    const int nt = a.num_tokens_per_rank ? min(a.num_tokens_per_rank[r], d.T) : d.T;
    if (t >= nt) return;

    // The row is requested first so that it travels while the rows are being located.
    const int lane = part * blockDim.x + tid; // lane of the token's row
    const bool active = lane < d.H / 16;
    uint4 raw0 = make_uint4(0, 0, 0, 0), raw1 = raw0;
    if (active) {
        const uint4 *src = reinterpret_cast<const uint4 *>(a.x + (static_cast<size_t>(r) * d.T + t) * d.H) + lane * 2;
        raw0 = ld16_nt(src);
        raw1 = ld16_nt(src + 1);
    }


    // Final row of selection k: e * N + (tokens the lower source ranks send to e) + position.
    // Half a wave per selection: its 32 lanes fetch the lower ranks' counts in parallel.
    for (int k = tid >> 5; k < d.K; k += blockDim.x >> 5) {
        const int q0 = tid & 31;
        const size_t sel = (static_cast<size_t>(r) * d.T + t) * d.K + k;
        const int p = a.rows[sel];
        const int e = a.topk_idx[sel];
        int partial = 0;
        if (p >= 0)
            for (int q = q0; q < r; q += 32)
                partial += a.send_count[q * d.E + e];
        partial += __shfl_xor(partial, 16);
        partial += __shfl_xor(partial, 8);
        partial += __shfl_xor(partial, 4);
        partial += __shfl_xor(partial, 2);
        partial += __shfl_xor(partial, 1);
        if (q0 == 0) row_of_k[k] = p >= 0 ? e * d.N + partial + p : -1;
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
        for (int j = 0; j < 4; ++j) {
            out[j] = f32_to_e4m3(v[4 * j] * scale) | (f32_to_e4m3(v[4 * j + 1] * scale) << 8) |
                (f32_to_e4m3(v[4 * j + 2] * scale) << 16) | (f32_to_e4m3(v[4 * j + 3] * scale) << 24);
        }
        q = make_uint4(out[0], out[1], out[2], out[3]);
    }
    __syncthreads();
    // Publish the rows (combine reads them back as its row map).  They go to an array of
    // their own: the other workgroups of this token may still be reading the positions.
    if (part == 0 && tid < d.K) a.rows_out[(static_cast<size_t>(r) * d.T + t) * d.K + tid] = row_of_k[tid];

    for (int k = 0; k < d.K; ++k) {
        const int row = row_of_k[k];
        if (row < 0) continue;
        if (lane == 0) a.src_info[row] = t;
        if (!active) continue;
        if constexpr (FP8) {
            st16_nt(reinterpret_cast<uint4 *>(a.recv_x + static_cast<size_t>(row) * d.H) + lane, q);
        } else {
            uint4 *dst = reinterpret_cast<uint4 *>(a.recv_x + static_cast<size_t>(row) * d.H * 2) + lane * 2;
            st16_nt(dst, raw0);
            st16_nt(dst + 1, raw1);
        }
    }
}

// ---- 3. receive-side metadata and scales, column-major per expert ----------------------------------------------------------------

struct ScalesArgs {
    void *recv_scales; // null: metadata only
    const float *token_scales;
    const int *src_info;
    const int *send_count; // [R][E]
    long long *layout_range;
    int *recv_count;
    int *stats;
    LlDims d;
    int use_ue8m0;
    int parts; // workgroups per expert
};

// grid = E * kScaleParts workgroups.  Every workgroup of expert e scans the R per-rank
// counts into segment ends (part 0 also writes them out as layout_range, recv_count and the
// statistics); workgroup (e, part) then copies scale groups part, part + kScaleParts, ... of
// every received row of expert e.  A thread owns row `slot`
// (= tid, tid + 256, ...): it finds the row's source rank from the segment ends, then
// gathers that token's scales (contiguous per token) and writes them at stride N, so that
// for each scale group the threads of a wave write consecutive addresses (the column-major
// layout of csrc/nixl_ep.cpp:1093-1100, kernels/nixl_ep_ll.cu:372-391).
constexpr int kScaleParts = 4; // workgroups per expert; 8 and 14 measured slower
constexpr int kScaleBatch = 8;

__global__ void __launch_bounds__(kScaleThreads)
ll_scales_kernel(ScalesArgs a) {
    extern __shared__ int seg_end[]; // [R] end of each source rank's segment of expert e
    const LlDims d = a.d;
    const int parts = a.parts;
    const int e = blockIdx.x / parts, part = blockIdx.x % parts, tid = threadIdx.x;
    const int G = d.H / 128;
    if (!a.recv_scales && part != 0) return; // metadata only: one workgroup per expert is enough
    // the first row's source token is fetched before its validity is known (always in bounds)
    int t_next = a.src_info[static_cast<size_t>(e) * d.N + min(tid, d.N - 1)];
    for (int r = tid; r < d.R; r += kScaleThreads)
        seg_end[r] = a.send_count[r * d.E + e];
    __syncthreads();
    if (tid < kWaveSize) {
        // inclusive scan of the R counts by one wave, 64 ranks per step
        int carry = 0;
        for (int r0 = 0; r0 < d.R; r0 += kWaveSize) {
            const int r = r0 + tid;
            const int n_r = r < d.R ? seg_end[r] : 0;
            int incl = n_r;
#pragma unroll
            for (int off = 1; off < kWaveSize; off <<= 1) {
                const int up = __shfl_up(incl, off);
                if (tid >= off) incl += up;
            }
            incl += carry;
            if (r < d.R) {
                seg_end[r] = incl;
                if (part == 0)
                    a.layout_range[static_cast<size_t>(e) * d.R + r] =
                        static_cast<long long>(static_cast<unsigned>(n_r)) | (static_cast<long long>(incl - n_r) << 32);
            }
            carry = __shfl(incl, kWaveSize - 1);
        }
        if (part == 0 && tid == 0) {
            a.recv_count[e] = carry;
            if (a.stats) a.stats[e] += carry;
        }
    }
    __syncthreads();
    if (!a.recv_scales) return;
    const int n = seg_end[d.R - 1];
    for (int slot = tid; slot < n; slot += kScaleThreads) {
        const int t = min(max(t_next, 0), d.T - 1); // written by the dispatch kernel; clamped so that a stale buffer cannot fault
        if (slot + kScaleThreads < n) t_next = a.src_info[static_cast<size_t>(e) * d.N + slot + kScaleThreads];
        int lo = 0, hi = d.R - 1; // first rank whose segment ends beyond `slot`
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (seg_end[mid] > slot)
                hi = mid;
            else
                lo = mid + 1;
        }
        const float *__restrict__ src = a.token_scales + (static_cast<size_t>(lo) * d.T + t) * G;
        if (!a.use_ue8m0) {
            float *__restrict__ dst = static_cast<float *>(a.recv_scales) + static_cast<size_t>(e) * G * d.N + slot;
            for (int g0 = part; g0 < G; g0 += parts * kScaleBatch) {
                float v[kScaleBatch];
#pragma unroll
                for (int j = 0; j < kScaleBatch; ++j) {
                    const int g = g0 + j * parts;
                    v[j] = g < G ? src[g] : 0.f;
                }
#pragma unroll
                for (int j = 0; j < kScaleBatch; ++j) {
                    const int g = g0 + j * parts;
                    if (g < G) dst[static_cast<size_t>(g) * d.N] = v[j];
                }
            }
        } else {
            // one exponent byte per group, four groups per 32-bit word, words [H/512][N]
            uint32_t *__restrict__ dst =
                static_cast<uint32_t *>(a.recv_scales) + static_cast<size_t>(e) * (G / 4) * d.N + slot;
            for (int g4 = part; g4 < G / 4; g4 += parts) {
                uint32_t word = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    word |= ((__float_as_uint(src[g4 * 4 + j]) >> 23) & 0xffu) << (8 * j);
                dst[static_cast<size_t>(g4) * d.N] = word;
            }
        }
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

__global__ void
f32_to_e4m3_kernel(const float *in, uint8_t *out, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) out[i] = static_cast<uint8_t>(f32_to_e4m3(in[i]));
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
int g_dispatch_lanes = 1024;
int g_combine_lanes = 1024;

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
    auto ok = [](int v) { return v == 0 || (v >= 64 && v <= 1024 && v % 64 == 0); };
    if (!ok(dispatch_lanes) || !ok(combine_lanes))
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_set_tuning: lanes must be 0 or a multiple of 64 in [64, 1024]");
    if (dispatch_lanes) g_dispatch_lanes = dispatch_lanes;
    if (combine_lanes) g_combine_lanes = combine_lanes;
    return NIXL_AMD_OK;
}

size_t
nixl_amd_ep_ll_workspace_bytes(int num_ranks, int num_experts, int num_tokens, int num_topk, int hidden) {
    if (num_ranks <= 0 || num_experts <= 0 || num_tokens < 0 || num_topk <= 0 || hidden < 0) return 0;
    const size_t counts = static_cast<size_t>(num_ranks) * num_experts * sizeof(int);
    const size_t rows = static_cast<size_t>(num_ranks) * num_tokens * num_topk * sizeof(int);
    const size_t scales = static_cast<size_t>(num_ranks) * num_tokens * (hidden / 128) * sizeof(float);
    return counts + 2 * rows + scales; // positions and final rows are separate arrays
}

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
    LlDims d;
    const int rc = check_dims("ll_dispatch", num_tokens, hidden, num_max_dispatch_tokens_per_rank, num_topk, num_ranks,
                              num_experts, d);
    if (rc) return rc;
    if (!packed_recv_x || !packed_recv_src_info || !packed_recv_layout_range || !packed_recv_count || !x || !topk_idx ||
        !workspace)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_dispatch: null pointer argument");
    if (use_fp8 && hidden % 512 != 0) // same restriction as csrc/nixl_ep.cpp:1091
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_dispatch: fp8 needs hidden % 512 == 0");
    if (use_fp8 && !packed_recv_x_scales) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_dispatch: scales pointer is null");
    if (use_ue8m0 && !(use_fp8 && round_scale)) // kernels/nixl_ep_ll.cu:428-430
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_dispatch: UE8M0 scales need use_fp8 and round_scale");
    if (workspace_bytes < nixl_amd_ep_ll_workspace_bytes(num_ranks, num_experts, num_tokens, num_topk, hidden))
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_dispatch: workspace too small");
    if (reinterpret_cast<uintptr_t>(workspace) % 4 != 0)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_dispatch: workspace must be 4-byte aligned");
    if (static_cast<long long>(d.E) * d.N >= (1ll << 31))
        return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "ll_dispatch: num_experts * num_ranks * max tokens must be below 2^31");
    if (static_cast<size_t>(d.E) * sizeof(int) > 48 * 1024 || static_cast<size_t>(d.R) * sizeof(int) > 48 * 1024)
        return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "ll_dispatch: too many experts or ranks");

    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t n_sel = static_cast<size_t>(d.R) * d.T * d.K;
    int *send_count = static_cast<int *>(workspace);
    int *positions = send_count + static_cast<size_t>(d.R) * d.E;
    int *rows_ws = positions + n_sel;
    float *token_scales = reinterpret_cast<float *>(rows_ws + n_sel);
    int *rows = row_map ? row_map : rows_ws;

    const int W = (d.T + 63) / 64 > 0 ? (d.T + 63) / 64 : 1;
    int per_pass = kLayoutLdsBytes / (W * 8);
    if (per_pass < 1) return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "ll_dispatch: too many tokens per rank for the layout pass");
    if (per_pass > d.E) per_pass = d.E;
    hipLaunchKernelGGL(ll_layout_kernel, dim3(d.R), dim3(kLayoutThreads), static_cast<size_t>(per_pass) * W * 8, s, topk_idx,
                       num_tokens_per_rank, mask_buffer, send_count, positions, d, per_pass);
    HIP_TRY(hipGetLastError());

    if (d.T > 0) {
        DispatchArgs a{};
        a.recv_x = static_cast<uint8_t *>(packed_recv_x);
        a.src_info = packed_recv_src_info;
        a.token_scales = token_scales;
        a.x = static_cast<const uint16_t *>(x);
        a.topk_idx = topk_idx;
        a.num_tokens_per_rank = num_tokens_per_rank;
        a.send_count = send_count;
        a.rows = positions;
        a.rows_out = rows;
        a.d = d;
        a.round_scale = round_scale;
        const int wg = std::min(round_up_wave(d.H / 16), g_dispatch_lanes);
        a.parts = (d.H / 16 + wg - 1) / wg;
        const dim3 grid(static_cast<unsigned>(d.R) * d.T * a.parts);
        const dim3 block(wg);
        if (use_fp8)
            hipLaunchKernelGGL(ll_dispatch_kernel<true>, grid, block, 0, s, a);
        else
            hipLaunchKernelGGL(ll_dispatch_kernel<false>, grid, block, 0, s, a);
        HIP_TRY(hipGetLastError());
    }

    ScalesArgs sa{};
    sa.recv_scales = use_fp8 ? packed_recv_x_scales : nullptr;
    sa.token_scales = token_scales;
    sa.src_info = packed_recv_src_info;
    sa.send_count = send_count;
    sa.layout_range = reinterpret_cast<long long *>(packed_recv_layout_range);
    sa.recv_count = packed_recv_count;
    sa.stats = cumulative_local_expert_recv_stats;
    sa.d = d;
    sa.use_ue8m0 = use_ue8m0;
    sa.parts = kScaleParts;
    hipLaunchKernelGGL(ll_scales_kernel, dim3(d.E * sa.parts), dim3(kScaleThreads),
                       static_cast<size_t>(d.R) * sizeof(int), s, sa);
    HIP_TRY(hipGetLastError());
    return NIXL_AMD_OK;
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
    // (counts and positions by the layout kernel, rows and scales by the dispatch kernel), so
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
    const int wg = std::min(round_up_wave(d.H / 8), g_combine_lanes);
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
nixl_amd_ep_f32_to_e4m3(const float *in, uint8_t *out, size_t n, void *stream) {
    if ((!in || !out) && n) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "f32_to_e4m3: null pointer argument");
    if (n == 0) return NIXL_AMD_OK;
    if (n > (1ull << 38)) return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "f32_to_e4m3: too many elements");
    hipLaunchKernelGGL(f32_to_e4m3_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), in, out, n);
    HIP_TRY(hipGetLastError());
    return NIXL_AMD_OK;
}

} // extern "C"
