// Normal-mode ("high-throughput") expert-parallel kernels and the router, for all virtual
// ranks of one GPU, with their C ABI (declared in include/nixl_amd_ep.h).
//
// The reference streams token rows through RDMA and NVLink ring queues, forwarding them hop
// by hop (kernels/nixl_ep_ht.cu:472-1245).  None of that exists when every rank is a region
// of the same HBM; what remains is the result: destination rows ordered by source rank then
// source token, rebased top-k indices, and the unweighted fp32 reduction on the way back.
// Positions come from prefix sums instead of queue heads:
//   row(r, t, d) = recv_row_offset[d] + recv_rank_prefix[d][r - 1] + send_head[r][t][d].
//
// HBM traffic: dispatch reads every source row once (2H) and writes it once per destination
// rank that holds one of its experts; combine reads those rows once and writes 2H per token.
#include <algorithm>
#include <cstdint>

#include "common.h"
#include "ep_common.h"
#include "nixl_amd_ep.h"

namespace {

constexpr int kScanThreads = 1024;

// Exclusive prefix of `v` over the workgroup (blockDim.x == kScanThreads); `total` gets the sum.
template<typename V>
__device__ __forceinline__ V
block_exclusive_scan(V v, V *wave_sums, V &total) {
    const int lane = threadIdx.x & (kWaveSize - 1), wave = threadIdx.x / kWaveSize;
    V incl = v;
#pragma unroll
    for (int off = 1; off < kWaveSize; off <<= 1) {
        const V up = __shfl_up(incl, off);
        if (lane >= off) incl += up;
    }
    __syncthreads(); // wave_sums may still be read from a previous call
    if (lane == kWaveSize - 1) wave_sums[wave] = incl;
    __syncthreads();
    constexpr int kWaves = kScanThreads / kWaveSize;
    V before = 0, sum = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        const V s = wave_sums[w];
        if (w < wave) before += s;
        sum += s;
    }
    total = sum;
    return before + incl - v;
}

// ---- layout (kernels/layout.cu:31-138) ----------------------------------------------------
// grid = R source ranks x chunks of kLayoutTokens tokens, one token per thread; LDS: E + R
// counters per workgroup, added to the (zeroed) outputs at the end.  Integer sums: the
// result does not depend on the order of the additions.
constexpr int kLayoutTokens = 256;

__global__ void __launch_bounds__(256)
zero_ints_kernel(int *__restrict__ a, size_t na, int *__restrict__ b, size_t nb) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < na) a[i] = 0;
    if (i < nb) b[i] = 0;
}

__global__ void __launch_bounds__(kLayoutTokens)
layout_kernel(const int32_t *__restrict__ topk_idx,
              int *__restrict__ per_rank,
              int *__restrict__ per_expert,
              uint8_t *__restrict__ in_rank,
              int T,
              int K,
              int R,
              int E) {
    extern __shared__ int counters[]; // [E] experts, then [R] ranks
    const int chunks = (T + kLayoutTokens - 1) / kLayoutTokens;
    const int src = blockIdx.x / chunks, El = E / R;
    const int t = (blockIdx.x % chunks) * kLayoutTokens + threadIdx.x;
    for (int i = threadIdx.x; i < E + R; i += blockDim.x)
        counters[i] = 0;
    __syncthreads();
    // whether the R flag bytes of a token can be written as one aligned 8-byte word
    const bool word_flags = R == 8 && (reinterpret_cast<uintptr_t>(in_rank) & 7u) == 0;
    if (t < T) {
        const int32_t *sel = topk_idx + (static_cast<size_t>(src) * T + t) * K;
        uint8_t *flags = in_rank + (static_cast<size_t>(src) * T + t) * R;
        if (R <= 64) {
            // destination ranks of the token as a bit mask in a register
            unsigned long long mask = 0;
            for (int k = 0; k < K; ++k) {
                const int e = sel[k];
                if (e < 0 || e >= E) continue;
                atomicAdd(&counters[e], 1);
                mask |= 1ull << (e / El);
            }
            if (word_flags) {
                unsigned long long bytes = 0;
#pragma unroll
                for (int d = 0; d < 8; ++d)
                    bytes |= ((mask >> d) & 1ull) << (8 * d);
                *reinterpret_cast<unsigned long long *>(flags) = bytes;
            } else {
                for (int d = 0; d < R; ++d)
                    flags[d] = static_cast<uint8_t>((mask >> d) & 1ull);
            }
            while (mask) {
                const int d = __builtin_ctzll(mask);
                mask &= mask - 1;
                atomicAdd(&counters[E + d], 1);
            }
        } else {
            for (int d = 0; d < R; ++d)
                flags[d] = 0;
            for (int k = 0; k < K; ++k) {
                const int e = sel[k];
                if (e < 0 || e >= E) continue;
                atomicAdd(&counters[e], 1);
                flags[e / El] = 1;
            }
            for (int d = 0; d < R; ++d)
                if (flags[d]) atomicAdd(&counters[E + d], 1);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < E; i += blockDim.x)
        if (counters[i]) atomicAdd(&per_expert[static_cast<size_t>(src) * E + i], counters[i]);
    for (int i = threadIdx.x; i < R; i += blockDim.x)
        if (counters[E + i]) atomicAdd(&per_rank[static_cast<size_t>(src) * R + i], counters[E + i]);
}

// ---- notify, part 1: per (source, destination) pair, positions inside the segment and the
// per-channel prefix (kernels/nixl_ep_ht.cu:324-373).  grid = R * R workgroups. ----------------
__global__ void __launch_bounds__(kScanThreads)
ht_scan_kernel(const uint8_t *__restrict__ in_rank,
               int *__restrict__ send_head,
               int *__restrict__ channel_prefix,
               int T,
               int R,
               int C) {
    __shared__ int wave_sums[kScanThreads / kWaveSize];
    const int src = blockIdx.x / R, d = blockIdx.x % R;
    const int per_thread = (T + kScanThreads - 1) / kScanThreads;
    const int t0 = min(static_cast<int>(threadIdx.x) * per_thread, T), t1 = min(t0 + per_thread, T);
    const int per_channel = (T + C - 1) / C;
    int mine = 0;
    for (int t = t0; t < t1; ++t)
        mine += in_rank[(static_cast<size_t>(src) * T + t) * R + d] != 0;
    int total;
    int pos = block_exclusive_scan(mine, wave_sums, total);
    for (int t = t0; t < t1; ++t) {
        const bool hit = in_rank[(static_cast<size_t>(src) * T + t) * R + d] != 0;
        __builtin_nontemporal_store(hit ? pos : -1, &send_head[(static_cast<size_t>(src) * T + t) * R + d]);
        pos += hit;
        // `pos` is now the number of hits in tokens [0, t]; a channel's inclusive prefix
        // is that number at the channel's last token.
        if ((t + 1) % per_channel == 0 || t + 1 == T) {
            const int c = t / per_channel;
            channel_prefix[(static_cast<size_t>(src) * R + d) * C + c] = pos;
        }
    }
    // channels that start at or beyond T are empty: they repeat the grand total
    if (threadIdx.x == 0)
        for (int c = (T + per_channel - 1) / per_channel; c < C; ++c)
            channel_prefix[(static_cast<size_t>(src) * R + d) * C + c] = total;
}

// The same for up to 8 ranks and fewer than 65 536 tokens, which is every shipping
// configuration.  A workgroup owns one chunk of kScanThreads tokens of one source rank, one
// token per thread, and handles all destinations at once with four 16-bit counters to a
// 64-bit word: it first counts the hits of the chunks before its own (a reduction; chunks do
// not wait for each other), then scans its own.  A thread writes the R positions of its
// token as one run, a wave consecutive runs.  The positions are stored non-temporally: the
// row kernel that follows reads them from every XCD, and lines left dirty in the writer's L2
// made those reads slow (+45 us on 8 x 4096 tokens).  grid = R * ceil(T / kScanThreads).
constexpr int kPackedScanRanks = 8;
constexpr int kPackedScanMaxTokens = 65535;

struct PackedCounts {
    unsigned long long lo, hi; // destinations 0..3 and 4..7, 16 bits each
};

__device__ __forceinline__ int
packed_field(const PackedCounts &c, int d) {
    return static_cast<int>(((d < 4 ? c.lo : c.hi) >> (16 * (d & 3))) & 0xffffu);
}

__device__ __forceinline__ PackedCounts
packed_hits(const uint8_t *flags, int t, int R) {
    PackedCounts hit{0, 0};
    if (R == 8) {
        const unsigned long long f = *reinterpret_cast<const unsigned long long *>(flags + static_cast<size_t>(t) * 8);
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            hit.lo |= static_cast<unsigned long long>(((f >> (8 * d)) & 0xffu) != 0) << (16 * d);
            hit.hi |= static_cast<unsigned long long>(((f >> (8 * (d + 4))) & 0xffu) != 0) << (16 * d);
        }
    } else {
        for (int d = 0; d < R; ++d) {
            const unsigned long long bit = flags[static_cast<size_t>(t) * R + d] != 0;
            if (d < 4)
                hit.lo |= bit << (16 * d);
            else
                hit.hi |= bit << (16 * (d - 4));
        }
    }
    return hit;
}

__global__ void __launch_bounds__(kScanThreads)
ht_scan_packed_kernel(const uint8_t *__restrict__ in_rank,
                      int *__restrict__ send_head,
                      int *__restrict__ channel_prefix,
                      int T,
                      int R,
                      int C) {
    constexpr int kWaves = kScanThreads / kWaveSize;
    __shared__ PackedCounts wave_sums[kWaves], wave_before[kWaves];
    const int chunks = (T + kScanThreads - 1) / kScanThreads;
    const int src = blockIdx.x / chunks, base = (blockIdx.x % chunks) * kScanThreads;
    const int tid = threadIdx.x, lane = tid & (kWaveSize - 1), wave = tid / kWaveSize;
    const int per_channel = (T + C - 1) / C;
    const uint8_t *flags = in_rank + static_cast<size_t>(src) * T * R;
    const int t = base + tid;

    // own token first, so that its load overlaps the count of the earlier chunks
    PackedCounts hit{0, 0};
    if (t < T) hit = packed_hits(flags, t, R);
    PackedCounts earlier{0, 0};
    for (int u = tid; u < base; u += kScanThreads) {
        const PackedCounts h = packed_hits(flags, u, R);
        earlier.lo += h.lo;
        earlier.hi += h.hi;
    }
#pragma unroll
    for (int off = kWaveSize / 2; off > 0; off >>= 1) {
        earlier.lo += __shfl_xor(earlier.lo, off);
        earlier.hi += __shfl_xor(earlier.hi, off);
    }
    PackedCounts incl = hit; // inclusive scan inside the wave
#pragma unroll
    for (int off = 1; off < kWaveSize; off <<= 1) {
        const unsigned long long ulo = __shfl_up(incl.lo, off), uhi = __shfl_up(incl.hi, off);
        if (lane >= off) {
            incl.lo += ulo;
            incl.hi += uhi;
        }
    }
    if (lane == kWaveSize - 1) wave_sums[wave] = incl;
    if (lane == 0) wave_before[wave] = earlier;
    __syncthreads();
    // second level by the first wave: wave_sums[w] becomes the hits before wave w (earlier
    // chunks included), wave_before[0] the grand total up to the end of this chunk
    if (wave == 0) {
        PackedCounts s{0, 0}, e{0, 0};
        if (lane < kWaves) {
            s = wave_sums[lane];
            e = wave_before[lane];
        }
        PackedCounts run = s;
#pragma unroll
        for (int off = 1; off < kWaves; off <<= 1) {
            const unsigned long long ulo = __shfl_up(run.lo, off), uhi = __shfl_up(run.hi, off);
            if (lane >= off) {
                run.lo += ulo;
                run.hi += uhi;
            }
        }
#pragma unroll
        for (int off = kWaves / 2; off > 0; off >>= 1) {
            e.lo += __shfl_xor(e.lo, off);
            e.hi += __shfl_xor(e.hi, off);
        }
        if (lane < kWaves) wave_sums[lane] = PackedCounts{run.lo - s.lo + e.lo, run.hi - s.hi + e.hi};
        if (lane == kWaves - 1) wave_before[0] = PackedCounts{run.lo + e.lo, run.hi + e.hi};
    }
    __syncthreads();
    const PackedCounts before = wave_sums[wave], total = wave_before[0];
    incl.lo += before.lo; // hits in tokens [0, t]
    incl.hi += before.hi;
    if (t < T) {
        int out[kPackedScanRanks];
#pragma unroll
        for (int d = 0; d < kPackedScanRanks; ++d)
            out[d] = packed_field(hit, d) ? packed_field(incl, d) - 1 : -1;
        int *dst = send_head + (static_cast<size_t>(src) * T + t) * R;
        if (R == 8) {
            st16_nt(dst, make_uint4(out[0], out[1], out[2], out[3]));
            st16_nt(dst + 4, make_uint4(out[4], out[5], out[6], out[7]));
        } else {
#pragma unroll
            for (int d = 0; d < kPackedScanRanks; ++d)
                if (d < R) __builtin_nontemporal_store(out[d], dst + d);
        }
        if ((t + 1) % per_channel == 0 || t + 1 == T) {
            const int c = t / per_channel;
            for (int d = 0; d < R; ++d)
                channel_prefix[(static_cast<size_t>(src) * R + d) * C + c] = packed_field(incl, d);
        }
    }
    // channels that start at or beyond T are empty: they repeat the grand total, which the
    // workgroup of the last chunk knows
    if (tid == 0 && base + kScanThreads >= T)
        for (int c = (T + per_channel - 1) / per_channel; c < C; ++c)
            for (int d = 0; d < R; ++d)
                channel_prefix[(static_cast<size_t>(src) * R + d) * C + c] = packed_field(total, d);
}

// ---- notify, part 2: receive-side prefix over source ranks, aligned per-expert counts
// (kernels/nixl_ep_ht.cu:295-314) and where each destination's rows start in the
// concatenated outputs.  One workgroup. ------------------------------------------------------
__global__ void __launch_bounds__(kScanThreads)
ht_prefix_kernel(const int *__restrict__ channel_prefix,
                 const int *__restrict__ per_expert,
                 int *__restrict__ recv_rank_prefix,
                 int *__restrict__ recv_expert_count,
                 long long *__restrict__ row_offset,
                 int *__restrict__ recv_counter,
                 int R,
                 int E,
                 int C,
                 int alignment) {
    __shared__ int wave_sums[kScanThreads / kWaveSize];
    const int tid = threadIdx.x;
    // Loads go out eight at a time before anything depends on them: issued one by one, the
    // round trips of this single workgroup add up to most of the kernel's time.
    constexpr int kBatch = 8;
    for (int e = tid; e < E; e += kScanThreads) {
        int n = 0;
        for (int r0 = 0; r0 < R; r0 += kBatch) {
            int v[kBatch];
#pragma unroll
            for (int j = 0; j < kBatch; ++j)
                v[j] = r0 + j < R ? per_expert[static_cast<size_t>(r0 + j) * E + e] : 0;
#pragma unroll
            for (int j = 0; j < kBatch; ++j)
                n += v[j];
        }
        recv_expert_count[e] = (n + alignment - 1) / alignment * alignment;
    }
    // R <= kScanThreads: thread d owns destination d
    int total = 0;
    if (tid < R) {
        for (int r0 = 0; r0 < R; r0 += kBatch) {
            int v[kBatch];
#pragma unroll
            for (int j = 0; j < kBatch; ++j)
                v[j] = r0 + j < R ? channel_prefix[(static_cast<size_t>(r0 + j) * R + tid) * C + (C - 1)] : 0;
#pragma unroll
            for (int j = 0; j < kBatch; ++j)
                if (r0 + j < R) {
                    total += v[j];
                    recv_rank_prefix[tid * R + r0 + j] = total;
                }
        }
        if (recv_counter) recv_counter[tid] = total;
    }
    if (row_offset) {
        // exclusive prefix of the per-destination totals in 64 bits
        long long incl = total;
        const int lane = tid & (kWaveSize - 1), wave = tid / kWaveSize;
#pragma unroll
        for (int off = 1; off < kWaveSize; off <<= 1) {
            const long long up = __shfl_up(incl, off);
            if (lane >= off) incl += up;
        }
        // wave totals fit in 32 bits each only if R * T does; check_ht bounds R * T by 2^30
        if (lane == kWaveSize - 1) wave_sums[wave] = static_cast<int>(incl);
        __syncthreads();
        long long before = 0;
        for (int w = 0; w < wave; ++w)
            before += wave_sums[w];
        if (tid < R) row_offset[tid + 1] = before + incl;
        if (tid == 0) row_offset[0] = 0;
    }
}

struct HtDims {
    int R, T, H, K, E;
};

__device__ __forceinline__ long long
recv_row(const int *prefix, const int *send_head, const long long *row_offset, const HtDims &d, int r, int t, int dst) {
    const int seg = r == 0 ? 0 : prefix[dst * d.R + r - 1];
    return row_offset[dst] + seg + send_head[(static_cast<size_t>(r) * d.T + t) * d.R + dst];
}

constexpr int kMaxHtRanks = 1024;
constexpr int kHtBatch = 8; // row loads a lane keeps in flight in combine

// The rows of token (r, t) at the destination ranks that hold it, in ascending rank order,
// gathered into LDS by the first wave (64 destinations per step, compacted with a ballot).
// Every thread of the workgroup calls this; the return value is the number of rows.
__device__ __forceinline__ int
collect_rows(const uint8_t *in_rank,
             const int *prefix,
             const int *send_head,
             const long long *row_offset,
             const HtDims &d,
             int r,
             int t,
             long long *rows,
             int *dsts,
             int *n_rows) {
    if (threadIdx.x < kWaveSize) {
        const int lane = threadIdx.x;
        const size_t tok = static_cast<size_t>(r) * d.T + t;
        int n = 0;
        for (int d0 = 0; d0 < d.R; d0 += kWaveSize) {
            const int dst = d0 + lane;
            bool hit = dst < d.R && in_rank[tok * d.R + dst] != 0;
            long long row = hit ? recv_row(prefix, send_head, row_offset, d, r, t, dst) : 0;
            // the handle comes from the caller: a row outside the destination's range is dropped
            if (hit && (row < row_offset[dst] || row >= row_offset[dst + 1])) hit = false;
            const unsigned long long m = __ballot(hit);
            if (hit) {
                const int p = n + __popcll(m & ((1ull << lane) - 1ull));
                rows[p] = row;
                dsts[p] = dst;
            }
            n += __popcll(m);
        }
        if (lane == 0) *n_rows = n;
    }
    __syncthreads();
    return *n_rows;
}

// ---- dispatch (result of kernels/nixl_ep_ht.cu:1109-1243) -------------------------------------
// Rows: grid = R*T*parts; a row is H/8 lanes of 16 bytes and a workgroup covers blockDim.x
// of them.  Narrow workgroups (one wave) measured fastest for this write-dominated scatter.
// Dynamic LDS: R * 12 bytes (rows, then destination ranks).
constexpr int kHtDispatchLanes = 64;

__global__ void __launch_bounds__(1024)
ht_dispatch_kernel(uint16_t *__restrict__ recv_x,
                   const uint16_t *__restrict__ x,
                   const uint8_t *__restrict__ in_rank,
                   const int *__restrict__ prefix,
                   const int *__restrict__ send_head,
                   const long long *__restrict__ row_offset,
                   HtDims d,
                   int parts) {
    extern __shared__ long long rows[]; // [R] rows, then [R] int destination ranks
    int *dsts = reinterpret_cast<int *>(rows + d.R);
    __shared__ int n_rows;
    const int tid = threadIdx.x;
    const int token = blockIdx.x / parts, part = blockIdx.x % parts;
    const int r = token / d.T, t = token % d.T;
    const size_t tok = static_cast<size_t>(r) * d.T + t;
    const int col = part * blockDim.x + tid;
    const bool active = col < d.H / 8;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (active) v = ld16_nt(reinterpret_cast<const uint4 *>(x + tok * d.H) + col);
    const int n = collect_rows(in_rank, prefix, send_head, row_offset, d, r, t, rows, dsts, &n_rows);
    if (!active) return;
    for (int i = 0; i < n; ++i)
        st16_nt(reinterpret_cast<uint4 *>(recv_x + static_cast<size_t>(rows[i]) * d.H) + col, v);
}

// Per-row metadata: rebased top-k indices, weights of the local selections, source rank and
// token.  grid = R * R * ceil(T / 256): (source, destination) pairs major, one token per
// thread.  Consecutive tokens that go to the destination occupy consecutive rows,
// so a wave writes a contiguous stretch of each array; written from the row kernel above,
// the same bytes were isolated 32-byte stores and cost several times as long.
constexpr int kHtMetaThreads = 256;

// VEC: selections moved four at a time and the (rank, token) pair in one store; the host
// picks it when K is a multiple of 4 and every pointer is 16-byte aligned.
template <bool VEC>
__global__ void __launch_bounds__(kHtMetaThreads)
ht_meta_kernel(int32_t *__restrict__ recv_topk_idx,
               float *__restrict__ recv_topk_weights,
               int32_t *__restrict__ recv_src_meta,
               const int32_t *__restrict__ topk_idx,
               const float *__restrict__ topk_weights,
               const uint8_t *__restrict__ in_rank,
               const int *__restrict__ prefix,
               const int *__restrict__ send_head,
               const long long *__restrict__ row_offset,
               HtDims d) {
    const int blocks_per_pair = (d.T + kHtMetaThreads - 1) / kHtMetaThreads;
    const int pair = blockIdx.x / blocks_per_pair;
    const int r = pair / d.R, dst = pair % d.R;
    const int t = (blockIdx.x % blocks_per_pair) * kHtMetaThreads + threadIdx.x;
    if (t >= d.T) return;
    const size_t tok = static_cast<size_t>(r) * d.T + t;
    if (!in_rank[tok * d.R + dst]) return;
    const long long row = recv_row(prefix, send_head, row_offset, d, r, t, dst);
    if (row < row_offset[dst] || row >= row_offset[dst + 1]) return;
    const int El = d.E / d.R;
    if (VEC && recv_topk_idx) {
        // four selections a step: 16-byte loads and stores (tok*K and row*K are multiples of 4)
        const int lo = dst * El, hi = lo + El;
        for (int k = 0; k < d.K; k += 4) {
            const int4 sel = *reinterpret_cast<const int4 *>(topk_idx + tok * d.K + k);
            const bool l0 = sel.x >= lo && sel.x < hi, l1 = sel.y >= lo && sel.y < hi;
            const bool l2 = sel.z >= lo && sel.z < hi, l3 = sel.w >= lo && sel.w < hi;
            *reinterpret_cast<int4 *>(recv_topk_idx + row * d.K + k) =
                make_int4(l0 ? sel.x - lo : -1, l1 ? sel.y - lo : -1, l2 ? sel.z - lo : -1, l3 ? sel.w - lo : -1);
            if (recv_topk_weights) {
                float4 w = make_float4(0.f, 0.f, 0.f, 0.f);
                if (topk_weights) w = *reinterpret_cast<const float4 *>(topk_weights + tok * d.K + k);
                *reinterpret_cast<float4 *>(recv_topk_weights + row * d.K + k) =
                    make_float4(l0 ? w.x : 0.f, l1 ? w.y : 0.f, l2 ? w.z : 0.f, l3 ? w.w : 0.f);
            }
        }
    } else if (recv_topk_idx)
        for (int k = 0; k < d.K; ++k) {
            const int sel = topk_idx[tok * d.K + k];
            const bool local = sel >= dst * El && sel < (dst + 1) * El;
            recv_topk_idx[row * d.K + k] = local ? sel - dst * El : -1;
            if (recv_topk_weights) recv_topk_weights[row * d.K + k] = local && topk_weights ? topk_weights[tok * d.K + k] : 0.f;
        }
    if (recv_src_meta) {
        if (VEC) {
            *reinterpret_cast<int2 *>(recv_src_meta + row * 2) = make_int2(r, t);
        } else {
            recv_src_meta[row * 2] = r;
            recv_src_meta[row * 2 + 1] = t;
        }
    }
}

// Per-token scales that travel with the rows (kernels/nixl_ep_ht.cu:729 reads them at
// token * scale_token_stride + i * scale_hidden_stride, :1198-1209 writes them densely per
// received row).  grid = R * R * ceil(T / 64): the first wave resolves the rows of 64
// consecutive tokens of one (source, destination) pair into LDS; the workgroup then moves
// their scales through an LDS tile of 64 tokens x 64 scales.  The tile is filled along
// whichever index is contiguous in the source (tokens, for the transposed storage the
// reference's callers pass; scales otherwise) and drained along the scales, so that a wave
// reads and writes consecutive addresses either way (consecutive tokens that go to the
// destination occupy consecutive rows).  Scales are moved as 32-bit words whatever they
// hold (fp32 or packed UE8M0).
constexpr int kHtScaleTokens = 64;
constexpr int kHtScaleTile = 64;
constexpr int kHtScaleThreads = 256;

__global__ void __launch_bounds__(kHtScaleThreads)
ht_row_scales_kernel(uint32_t *__restrict__ recv_scales,
                     const uint32_t *__restrict__ scales,
                     const uint8_t *__restrict__ in_rank,
                     const int *__restrict__ prefix,
                     const int *__restrict__ send_head,
                     const long long *__restrict__ row_offset,
                     HtDims d,
                     int S,
                     long long rank_stride,
                     long long token_stride,
                     long long scale_stride,
                     int wide) {
    __shared__ long long rows[kHtScaleTokens];
    __shared__ uint32_t tile[kHtScaleTokens][kHtScaleTile + 1]; // odd pitch: no bank conflicts either way
    const int blocks_per_pair = (d.T + kHtScaleTokens - 1) / kHtScaleTokens;
    const int pair = blockIdx.x / blocks_per_pair;
    const int r = pair / d.R, dst = pair % d.R;
    const int t0 = (blockIdx.x % blocks_per_pair) * kHtScaleTokens;
    const int tid = threadIdx.x;
    if (tid < kHtScaleTokens) {
        const int t = t0 + tid;
        long long row = -1;
        if (t < d.T && in_rank[(static_cast<size_t>(r) * d.T + t) * d.R + dst]) {
            row = recv_row(prefix, send_head, row_offset, d, r, t, dst);
            if (row < row_offset[dst] || row >= row_offset[dst + 1]) row = -1;
        }
        rows[tid] = row;
    }
    __syncthreads();
    const uint32_t *__restrict__ src = scales + static_cast<long long>(r) * rank_stride;
    const bool tokens_contiguous = token_stride < scale_stride;
    for (int g0 = 0; g0 < S; g0 += kHtScaleTile) {
        const int gs = min(kHtScaleTile, S - g0);
        // every load of the tile is issued before the first value is used: one load, one
        // LDS write at a time, the round trips of the 16 steps add up
        constexpr int kSteps = kHtScaleTokens * kHtScaleTile / kHtScaleThreads;
        uint32_t v[kSteps];
        int at[kSteps];
#pragma unroll
        for (int k = 0; k < kSteps; ++k) {
            const int i = tid + k * kHtScaleThreads;
            const int j = tokens_contiguous ? i % kHtScaleTokens : i / gs;
            const int g = tokens_contiguous ? i / kHtScaleTokens : i - j * gs;
            at[k] = -1;
            v[k] = 0;
            if (i < kHtScaleTokens * gs && rows[j] >= 0) {
                at[k] = j * (kHtScaleTile + 1) + g;
                v[k] = src[static_cast<long long>(t0 + j) * token_stride + static_cast<long long>(g0 + g) * scale_stride];
            }
        }
#pragma unroll
        for (int k = 0; k < kSteps; ++k)
            if (at[k] >= 0) (&tile[0][0])[at[k]] = v[k];
        __syncthreads();
        if (wide) {
            // four scales a store: the isolated 4-byte stores of the narrow form run at a
            // fraction of the rate
            const int quads = gs / 4;
            for (int i = tid; i < kHtScaleTokens * quads; i += kHtScaleThreads) {
                const int j = i / quads, q = (i - j * quads) * 4;
                const long long row = rows[j];
                if (row >= 0)
                    *reinterpret_cast<uint4 *>(recv_scales + row * S + g0 + q) =
                        make_uint4(tile[j][q], tile[j][q + 1], tile[j][q + 2], tile[j][q + 3]);
            }
        } else {
            for (int i = tid; i < kHtScaleTokens * gs; i += kHtScaleThreads) {
                const int j = i / gs, g = i - j * gs;
                const long long row = rows[j];
                if (row >= 0) recv_scales[row * S + g0 + g] = tile[j][g];
            }
        }
        __syncthreads();
    }
}

// ---- combine (combine_token, kernels/nixl_ep_ht.cu:1682-1737) -----------------------------------
// grid = R*T*parts; a row is H/8 lanes of 16 bytes and a workgroup covers blockDim.x of them.
constexpr int kHtCombineLanes = 128;

__global__ void __launch_bounds__(1024)
ht_combine_kernel(uint16_t *__restrict__ combined,
                  float *__restrict__ combined_w,
                  const uint16_t *__restrict__ x,
                  const float *__restrict__ topk_weights,
                  const uint16_t *__restrict__ bias0,
                  const uint16_t *__restrict__ bias1,
                  const uint8_t *__restrict__ in_rank,
                  const int *__restrict__ prefix,
                  const int *__restrict__ send_head,
                  const long long *__restrict__ row_offset,
                  HtDims d,
                  int parts) {
    __shared__ long long rows[kMaxHtRanks];
    __shared__ int dsts[kMaxHtRanks];
    __shared__ int n_rows;
    const int tid = threadIdx.x;
    const int token = blockIdx.x / parts, part = blockIdx.x % parts;
    const int r = token / d.T, t = token % d.T;
    const size_t tok = static_cast<size_t>(r) * d.T + t;
    const int col = part * blockDim.x + tid;
    const bool active = col < d.H / 8;
    const bool weights = part == 0 && tid < d.K;
    uint4 b0 = make_uint4(0, 0, 0, 0), b1 = b0;
    if (active) {
        if (bias0) b0 = ld16_nt(reinterpret_cast<const uint4 *>(bias0 + tok * d.H) + col);
        if (bias1) b1 = ld16_nt(reinterpret_cast<const uint4 *>(bias1 + tok * d.H) + col);
    }
    const int n = collect_rows(in_rank, prefix, send_head, row_offset, d, r, t, rows, dsts, &n_rows);
    float acc[8];
    {
        const uint32_t u0[4] = {b0.x, b0.y, b0.z, b0.w}, u1[4] = {b1.x, b1.y, b1.z, b1.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            acc[2 * c] = bf16_lo_to_f32(u0[c]) + bf16_lo_to_f32(u1[c]);
            acc[2 * c + 1] = bf16_hi_to_f32(u0[c]) + bf16_hi_to_f32(u1[c]);
        }
    }
    float wsum = 0.f;
    for (int i0 = 0; i0 < n; i0 += kHtBatch) {
        // all loads of the batch first, then the additions in ascending rank order
        uint4 v[kHtBatch];
        float wv[kHtBatch];
#pragma unroll
        for (int j = 0; j < kHtBatch; ++j) {
            v[j] = make_uint4(0, 0, 0, 0);
            wv[j] = 0.f;
            if (i0 + j < n) {
                const long long row = rows[i0 + j];
                if (active) v[j] = ld16_nt(reinterpret_cast<const uint4 *>(x + static_cast<size_t>(row) * d.H) + col);
                if (topk_weights && weights) wv[j] = topk_weights[row * d.K + tid];
            }
        }
#pragma unroll
        for (int j = 0; j < kHtBatch; ++j) {
            if (i0 + j >= n) continue;
            const uint32_t u[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                acc[2 * c] += bf16_lo_to_f32(u[c]);
                acc[2 * c + 1] += bf16_hi_to_f32(u[c]);
            }
            wsum += wv[j];
        }
    }
    if (active) {
        uint4 out;
        out.x = f32_to_bf16(acc[0]) | (f32_to_bf16(acc[1]) << 16);
        out.y = f32_to_bf16(acc[2]) | (f32_to_bf16(acc[3]) << 16);
        out.z = f32_to_bf16(acc[4]) | (f32_to_bf16(acc[5]) << 16);
        out.w = f32_to_bf16(acc[6]) | (f32_to_bf16(acc[7]) << 16);
        st16_nt(reinterpret_cast<uint4 *>(combined + tok * d.H) + col, out);
    }
    if (combined_w && weights) combined_w[tok * d.K + tid] = wsum;
}

// ---- router -----------------------------------------------------------------------------------------
// One wave per token; lane l holds experts l, l + 64, ...  K rounds of a wave-wide argmax
// (larger value wins, equal values go to the lower expert index).  The two reductions of a
// round (maximum of the values, then lowest index among the lanes that hold it) run on
// the DPP data path: four steps inside the rows of 16 lanes, two row broadcasts, result in
// lane 63.  Cross-lane permutes through LDS took three times as long.
constexpr int kRouterMaxPerLane = 16; // E <= 1024

// PL = experts a lane holds (a power of two >= ceil(E / 64)): the argmax rounds only walk
// the slots that exist.
template<int PL>
__global__ void __launch_bounds__(256)
router_kernel(const float *__restrict__ logits, int32_t *__restrict__ topk_idx, float *__restrict__ topk_w, int n_tokens, int E, int K) {
    const int lane = threadIdx.x & (kWaveSize - 1);
    const int token = blockIdx.x * (blockDim.x / kWaveSize) + threadIdx.x / kWaveSize;
    if (token >= n_tokens) return; // whole waves leave together: the DPP steps below see full waves
    float v[PL];
    unsigned taken = 0;
#pragma unroll
    for (int j = 0; j < PL; ++j) {
        const int e = j * kWaveSize + lane;
        v[j] = e < E ? logits[static_cast<size_t>(token) * E + e] : 0.f;
        if (e >= E) taken |= 1u << j;
    }
    float mine = 0.f, first = 0.f; // lane k keeps the k-th selected logit
    int mine_i = 0;
    for (int k = 0; k < K; ++k) {
        float top;
        int win;
        router_round<PL>(v, taken, lane, top, win);
        if (k == 0) first = top;
        if (lane == k) {
            mine = top;
            mine_i = win;
        }
    }
    // softmax over the K selected logits; every lane adds them up in selection order
    const float ex = lane < K ? expf(mine - first) : 0.f;
    float sum = 0.f;
    for (int k = 0; k < K; ++k)
        sum += __shfl(ex, k);
    if (lane < K) {
        topk_idx[static_cast<size_t>(token) * K + lane] = mine_i;
        topk_w[static_cast<size_t>(token) * K + lane] = ex / sum;
    }
}

int
round_up_wave(int n) {
    return (n + kWaveSize - 1) / kWaveSize * kWaveSize;
}

int
check_ht(const char *who, int T, int H, int K, int R, int E) {
    auto bad = [&](const std::string &why) { return nixl_amd_fail(NIXL_AMD_ERR_INVALID, std::string(who) + ": " + why); };
    if (R <= 0 || R > 1024) return bad("num_ranks must be in [1, 1024]");
    if (E <= 0 || E % R != 0) return bad("num_experts must be a positive multiple of num_ranks");
    if (T <= 0) return bad("num_tokens must be positive");
    if (K < 0 || K > 16) return bad("num_topk must be at most 16");
    if (H % 8 != 0 || H < 0 || H > 8192) return bad("hidden must be a multiple of 8, at most 8192");
    if (static_cast<long long>(R) * T > (1ll << 30)) return bad("num_ranks * num_tokens too large");
    return NIXL_AMD_OK;
}

} // namespace

extern "C" {

int
nixl_amd_ep_get_dispatch_layout(const int32_t *topk_idx,
                                int *num_tokens_per_rank,
                                int *num_tokens_per_expert,
                                uint8_t *is_token_in_rank,
                                int num_tokens,
                                int num_topk,
                                int num_ranks,
                                int num_experts,
                                void *stream) {
    const int rc = check_ht("get_dispatch_layout", num_tokens, 0, num_topk, num_ranks, num_experts);
    if (rc) return rc;
    if (!topk_idx || !num_tokens_per_rank || !num_tokens_per_expert || !is_token_in_rank)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "get_dispatch_layout: null pointer argument");
    const size_t lds = static_cast<size_t>(num_experts + num_ranks) * sizeof(int);
    if (lds > 48 * 1024) return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "get_dispatch_layout: too many experts");
    hipStream_t s = static_cast<hipStream_t>(stream);
    // the counts are accumulated with atomics; cleared by a kernel, not a memset, so that a
    // caller may capture the call into a graph
    const size_t n_rank = static_cast<size_t>(num_ranks) * num_ranks, n_expert = static_cast<size_t>(num_ranks) * num_experts;
    hipLaunchKernelGGL(zero_ints_kernel, dim3(static_cast<unsigned>((std::max(n_rank, n_expert) + 255) / 256)), dim3(256), 0, s,
                       num_tokens_per_rank, n_rank, num_tokens_per_expert, n_expert);
    HIP_TRY(hipGetLastError());
    const long long chunks = (num_tokens + kLayoutTokens - 1) / kLayoutTokens;
    hipLaunchKernelGGL(layout_kernel, dim3(static_cast<unsigned>(num_ranks * chunks)), dim3(kLayoutTokens), lds, s, topk_idx,
                       num_tokens_per_rank, num_tokens_per_expert, is_token_in_rank, num_tokens, num_topk, num_ranks,
                       num_experts);
    HIP_TRY(hipGetLastError());
    return NIXL_AMD_OK;
}

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
                               void *stream) {
    const int rc = check_ht("ht_notify_dispatch", num_tokens, 0, 0, num_ranks, num_experts);
    if (rc) return rc;
    if (num_channels <= 0 || expert_alignment <= 0)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ht_notify_dispatch: num_channels and expert_alignment must be positive");
    if (!is_token_in_rank || !num_tokens_per_expert || !recv_gbl_rank_prefix_sum || !recv_expert_count ||
        !gbl_channel_prefix_matrix || !send_head)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ht_notify_dispatch: null pointer argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    // the packed kernel reads 8 flag bytes and writes 16-byte pieces at a time
    const bool aligned = reinterpret_cast<uintptr_t>(is_token_in_rank) % 8 == 0 && reinterpret_cast<uintptr_t>(send_head) % 16 == 0;
    if (num_ranks <= kPackedScanRanks && num_tokens <= kPackedScanMaxTokens && aligned)
        hipLaunchKernelGGL(ht_scan_packed_kernel,
                           dim3(static_cast<unsigned>(num_ranks) * ((num_tokens + kScanThreads - 1) / kScanThreads)),
                           dim3(kScanThreads), 0, s,
                           is_token_in_rank, send_head, gbl_channel_prefix_matrix, num_tokens, num_ranks, num_channels);
    else
        hipLaunchKernelGGL(ht_scan_kernel, dim3(static_cast<unsigned>(num_ranks) * num_ranks), dim3(kScanThreads), 0, s,
                           is_token_in_rank, send_head, gbl_channel_prefix_matrix, num_tokens, num_ranks, num_channels);
    HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(ht_prefix_kernel, dim3(1), dim3(kScanThreads), 0, s, gbl_channel_prefix_matrix,
                       num_tokens_per_expert, recv_gbl_rank_prefix_sum, recv_expert_count,
                       reinterpret_cast<long long *>(recv_row_offset), recv_counter, num_ranks, num_experts,
                       num_channels, expert_alignment);
    HIP_TRY(hipGetLastError());
    return NIXL_AMD_OK;
}

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
                               void *stream) {
    if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ht_dispatch: elem_bytes must be 1, 2 or 4");
    if (hidden <= 0) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ht_dispatch: hidden must be positive");
    if ((static_cast<long long>(hidden) * elem_bytes) % 16 != 0)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ht_dispatch: a row must be a multiple of 16 bytes");
    // the row kernels count a row in 2-byte elements, whatever it holds
    const long long row_halves = static_cast<long long>(hidden) * elem_bytes / 2;
    if (row_halves > 8192) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ht_dispatch: a row may hold at most 16 KiB");
    const int rc = check_ht("ht_dispatch", num_tokens, static_cast<int>(row_halves), num_topk, num_ranks, num_experts);
    if (rc) return rc;
    if (!recv_x || !x || !is_token_in_rank || !recv_gbl_rank_prefix_sum || !send_head || !recv_row_offset)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ht_dispatch: null pointer argument");
    if (recv_topk_idx && !topk_idx) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ht_dispatch: recv_topk_idx without topk_idx");
    if (num_scales < 0 || num_scales > 4096) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ht_dispatch: num_scales must be in [0, 4096]");
    if ((x_scales != nullptr) != (recv_x_scales != nullptr) || (x_scales && num_scales == 0))
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ht_dispatch: x_scales, recv_x_scales and num_scales go together");
    if (x_scales && (scale_rank_stride < 0 || scale_token_stride < 0 || scale_hidden_stride < 0))
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ht_dispatch: negative scale stride");
    const HtDims d{num_ranks, num_tokens, static_cast<int>(row_halves), num_topk, num_experts};
    const int lanes = round_up_wave(d.H / 8);
    const int parts = (lanes + kHtDispatchLanes - 1) / kHtDispatchLanes;
    if (static_cast<long long>(num_ranks) * num_tokens * parts >= (1ll << 31))
        return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "ht_dispatch: too many tokens");
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(ht_dispatch_kernel, dim3(static_cast<unsigned>(num_ranks) * num_tokens * parts), dim3(kHtDispatchLanes),
                       static_cast<size_t>(num_ranks) * 12, s, static_cast<uint16_t *>(recv_x),
                       static_cast<const uint16_t *>(x), is_token_in_rank, recv_gbl_rank_prefix_sum, send_head,
                       reinterpret_cast<const long long *>(recv_row_offset), d, parts);
    HIP_TRY(hipGetLastError());
    if (x_scales) {
        const long long blocks = static_cast<long long>(num_ranks) * num_ranks * ((num_tokens + kHtScaleTokens - 1) / kHtScaleTokens);
        if (blocks >= (1ll << 31)) return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "ht_dispatch: too many ranks and tokens");
        hipLaunchKernelGGL(ht_row_scales_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kHtScaleThreads), 0, s,
                           static_cast<uint32_t *>(recv_x_scales), static_cast<const uint32_t *>(x_scales), is_token_in_rank,
                           recv_gbl_rank_prefix_sum, send_head, reinterpret_cast<const long long *>(recv_row_offset), d,
                           num_scales, static_cast<long long>(scale_rank_stride), static_cast<long long>(scale_token_stride),
                           static_cast<long long>(scale_hidden_stride),
                           (num_scales % 4 == 0 && reinterpret_cast<uintptr_t>(recv_x_scales) % 16 == 0) ? 1 : 0);
        HIP_TRY(hipGetLastError());
    }
    if (recv_topk_idx || recv_src_meta) {
        const long long blocks = static_cast<long long>(num_ranks) * num_ranks * ((num_tokens + kHtMetaThreads - 1) / kHtMetaThreads);
        if (blocks >= (1ll << 31)) return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "ht_dispatch: too many ranks and tokens");
        const dim3 grid(static_cast<unsigned>(blocks));
        const uintptr_t bits = reinterpret_cast<uintptr_t>(recv_topk_idx) | reinterpret_cast<uintptr_t>(recv_topk_weights) |
                               reinterpret_cast<uintptr_t>(recv_src_meta) | reinterpret_cast<uintptr_t>(topk_idx) |
                               reinterpret_cast<uintptr_t>(topk_weights);
        const auto kernel = (num_topk % 4 == 0 && bits % 16 == 0) ? ht_meta_kernel<true> : ht_meta_kernel<false>;
        hipLaunchKernelGGL(kernel, grid, dim3(kHtMetaThreads), 0, s, recv_topk_idx, recv_topk_weights, recv_src_meta,
                           topk_idx, topk_weights, is_token_in_rank, recv_gbl_rank_prefix_sum, send_head,
                           reinterpret_cast<const long long *>(recv_row_offset), d);
    }
    HIP_TRY(hipGetLastError());
    return NIXL_AMD_OK;
}

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
                        void *stream) {
    return nixl_amd_ep_ht_dispatch_scaled(recv_x, nullptr, recv_topk_idx, recv_topk_weights, recv_src_meta, x, nullptr, topk_idx,
                                          topk_weights, is_token_in_rank, recv_gbl_rank_prefix_sum, send_head, recv_row_offset,
                                          num_tokens, hidden, 2, 0, 0, 0, 0, num_topk, num_ranks, num_experts, stream);
}

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
                       void *stream) {
    const int rc = check_ht("ht_combine", num_tokens, hidden, num_topk, num_ranks, num_ranks);
    if (rc) return rc;
    if (hidden == 0) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ht_combine: hidden must be positive");
    if (!combined_x || !x || !is_token_in_rank || !recv_gbl_rank_prefix_sum || !send_head || !recv_row_offset)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ht_combine: null pointer argument");
    const HtDims d{num_ranks, num_tokens, hidden, num_topk, num_ranks};
    // Two-wave workgroups over 2 KiB pieces of a row: more workgroups resident, so that the
    // look-ups of some overlap the row loads of others (485 us against 510 for a workgroup per
    // row at 8 x 4096 x 7168; one wave: 575, four: 514).
    const int lanes = std::min(kHtCombineLanes, round_up_wave(hidden / 8));
    const int parts = (round_up_wave(hidden / 8) + lanes - 1) / lanes;
    if (static_cast<long long>(num_ranks) * num_tokens * parts >= (1ll << 31))
        return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "ht_combine: too many tokens");
    hipLaunchKernelGGL(ht_combine_kernel, dim3(static_cast<unsigned>(num_ranks) * num_tokens * parts), dim3(lanes),
                       0, static_cast<hipStream_t>(stream), static_cast<uint16_t *>(combined_x), combined_topk_weights,
                       static_cast<const uint16_t *>(x), topk_weights, static_cast<const uint16_t *>(bias_0),
                       static_cast<const uint16_t *>(bias_1), is_token_in_rank, recv_gbl_rank_prefix_sum, send_head,
                       reinterpret_cast<const long long *>(recv_row_offset), d, parts);
    HIP_TRY(hipGetLastError());
    return NIXL_AMD_OK;
}

int
nixl_amd_ep_router_topk(const float *logits,
                        int32_t *topk_idx,
                        float *topk_weights,
                        int num_tokens,
                        int num_experts,
                        int num_topk,
                        void *stream) {
    if (!logits || !topk_idx || !topk_weights) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "router_topk: null pointer argument");
    if (num_tokens < 0 || num_experts <= 0 || num_experts > kRouterMaxPerLane * kWaveSize)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "router_topk: num_experts must be in [1, 1024]");
    if (num_topk <= 0 || num_topk > 16 || num_topk > num_experts)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "router_topk: num_topk must be in [1, min(16, num_experts)]");
    if (num_tokens == 0) return NIXL_AMD_OK;
    const dim3 grid((num_tokens + 3) / 4), block(256);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int per_lane = (num_experts + kWaveSize - 1) / kWaveSize;
    if (per_lane <= 1)
        hipLaunchKernelGGL(router_kernel<1>, grid, block, 0, s, logits, topk_idx, topk_weights, num_tokens, num_experts, num_topk);
    else if (per_lane <= 2)
        hipLaunchKernelGGL(router_kernel<2>, grid, block, 0, s, logits, topk_idx, topk_weights, num_tokens, num_experts, num_topk);
    else if (per_lane <= 4)
        hipLaunchKernelGGL(router_kernel<4>, grid, block, 0, s, logits, topk_idx, topk_weights, num_tokens, num_experts, num_topk);
    else if (per_lane <= 8)
        hipLaunchKernelGGL(router_kernel<8>, grid, block, 0, s, logits, topk_idx, topk_weights, num_tokens, num_experts, num_topk);
    else
        hipLaunchKernelGGL(router_kernel<16>, grid, block, 0, s, logits, topk_idx, topk_weights, num_tokens, num_experts, num_topk);
    HIP_TRY(hipGetLastError());
    return NIXL_AMD_OK;
}

} // extern "C"
