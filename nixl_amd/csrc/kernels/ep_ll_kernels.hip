// Low-latency expert-parallel dispatch and combine for all virtual ranks of one GPU, and
// the C ABI that launches them (declared in include/nixl_amd_ep.h).
//
// What the reference does per rank with three passes over the payload (cast into a send
// buffer, K message copies into per-(expert, source rank) receive slots, repack into the
// per-expert contiguous output; kernels/nixl_ep_ll.cu:134-393) is done here in two
// launches, because every "remote" slot is an address in the same HBM:
//   1. ll_layout_kernel    one workgroup per source rank builds, in LDS, one bitmask of
//                          tokens per expert and derives count[r][e] and the position of
//                          every (token, k) inside its (r, e) segment;
//   2. ll_dispatch_kernel  one workgroup per token reads its bf16 row once, quantises it in
//                          registers and writes it straight to its K final rows of
//                          packed_recv_x (and the scales column-major, src_info); the row
//                          index is begin[e][r] + position with begin = sum of counts of
//                          lower source ranks.  Extra workgroups write layout_range,
//                          recv_count and the statistics.
// The order this produces is the canonical one among those the reference's atomics allow:
// segments by source rank ascending, tokens ascending inside a segment.
//
// HBM traffic per token (H hidden, K selections, G = H/128): read 2H, write
// K * (H + 4G + 4) for fp8 or K * (2H + 4) for bf16.
//
// Combine is one launch: one workgroup per token locates its K rows through the dispatch
// handle, reads them once and accumulates in fp32 with fused multiply-adds in top-k order
// (kernels/nixl_ep_ll.cu:959-1012).  Traffic per token: read K * 2H, write 2H.
#include <cstdint>

#include "common.h"
#include "ep_common.h"
#include "nixl_amd_ep.h"

namespace {

constexpr int kLayoutThreads = 256;
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

// ---- 2. cast + scatter ------------------------------------------------------------------

struct DispatchArgs {
    uint8_t *recv_x;
    void *recv_scales;
    int *src_info;
    long long *layout_range;
    int *recv_count;
    int *stats;
    const uint16_t *x;
    const int32_t *topk_idx;
    const int *num_tokens_per_rank;
    const int *send_count;
    const int *pos;
    LlDims d;
    int round_scale;
    int use_ue8m0;
};

// grid = R metadata workgroups followed by R*T token workgroups; block = H/16 lanes rounded
// up to whole waves.  Each lane owns 16 consecutive channels (32 bytes of bf16, 16 bytes of
// fp8), so a 128-channel scale group is 8 neighbouring lanes.
template<bool FP8>
__global__ void __launch_bounds__(1024)
ll_dispatch_kernel(DispatchArgs a) {
    const LlDims d = a.d;
    const int tid = threadIdx.x;
    __shared__ long long row_of_k[kMaxTopk]; // e * N + slot, or -1

    if (blockIdx.x < static_cast<unsigned>(d.R)) {
        // Metadata role for source rank r: (count, begin) of every expert's segment r.
        const int r = blockIdx.x;
        for (int e = tid; e < d.E; e += blockDim.x) {
            int begin = 0;
            for (int q = 0; q < r; ++q)
                begin += a.send_count[q * d.E + e];
            const int n = a.send_count[r * d.E + e];
            a.layout_range[static_cast<size_t>(e) * d.R + r] =
                static_cast<long long>(static_cast<unsigned>(n)) | (static_cast<long long>(begin) << 32);
            if (r == d.R - 1) {
                a.recv_count[e] = begin + n;
                if (a.stats) a.stats[e] += begin + n;
            }
        }
        return;
    }

    const int token = blockIdx.x - d.R;
    const int r = token / d.T, t = token % d.T;
    const int nt = a.num_tokens_per_rank ? min(a.num_tokens_per_rank[r], d.T) : d.T;
    if (t >= nt) return;

    if (tid < d.K) {
        const int p = a.pos[(static_cast<size_t>(r) * d.T + t) * d.K + tid];
        long long row = -1;
        if (p >= 0) {
            const int e = a.topk_idx[(static_cast<size_t>(r) * d.T + t) * d.K + tid];
            int begin = 0;
            for (int q = 0; q < r; ++q)
                begin += a.send_count[q * d.E + e];
            row = static_cast<long long>(e) * d.N + begin + p;
        }
        row_of_k[tid] = row;
    }

    const int lanes = d.H / 16;
    const bool active = tid < lanes;
    uint4 raw0 = make_uint4(0, 0, 0, 0), raw1 = raw0;
    if (active) {
        const uint4 *src = reinterpret_cast<const uint4 *>(a.x + (static_cast<size_t>(r) * d.T + t) * d.H) + tid * 2;
        raw0 = ld16_nt(src);
        raw1 = ld16_nt(src + 1);
    }

    uint4 q = make_uint4(0, 0, 0, 0);
    float scale_inv = 0.f;
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
        float scale;
        fp8_scales(amax, a.round_scale != 0, scale, scale_inv);
        uint32_t out[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            out[j] = f32_to_e4m3(v[4 * j] * scale) | (f32_to_e4m3(v[4 * j + 1] * scale) << 8) |
                (f32_to_e4m3(v[4 * j + 2] * scale) << 16) | (f32_to_e4m3(v[4 * j + 3] * scale) << 24);
        }
        q = make_uint4(out[0], out[1], out[2], out[3]);
    }
    __syncthreads();

    const int G = d.H / 128;
    for (int k = 0; k < d.K; ++k) {
        const long long row = row_of_k[k];
        if (row < 0) continue;
        if (tid == 0) a.src_info[row] = t;
        if (!active) continue;
        if constexpr (FP8) {
            uint4 *dst = reinterpret_cast<uint4 *>(a.recv_x + static_cast<size_t>(row) * d.H) + tid;
            st16_nt(dst, q);
            if ((tid & 7) == 0) {
                const int g = tid >> 3;
                const long long e = row / d.N, slot = row % d.N;
                if (!a.use_ue8m0) {
                    static_cast<float *>(a.recv_scales)[(static_cast<size_t>(e) * G + g) * d.N + slot] = scale_inv;
                } else {
                    uint8_t *base = static_cast<uint8_t *>(a.recv_scales) + static_cast<size_t>(e) * (G / 4) * d.N * 4;
                    base[(static_cast<size_t>(g / 4) * d.N + slot) * 4 + (g & 3)] =
                        static_cast<uint8_t>(__float_as_uint(scale_inv) >> 23);
                }
            }
        } else {
            uint4 *dst = reinterpret_cast<uint4 *>(a.recv_x + static_cast<size_t>(row) * d.H * 2) + tid * 2;
            st16_nt(dst, raw0);
            st16_nt(dst + 1, raw1);
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
    LlDims d;
};

// grid = R*T workgroups; block = H/8 lanes rounded up to whole waves; each lane owns 8
// consecutive channels (16 bytes per row).
__global__ void __launch_bounds__(1024)
ll_combine_kernel(CombineArgs a) {
    const LlDims d = a.d;
    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1), wave = tid / kWaveSize, n_waves = blockDim.x / kWaveSize;
    const int r = blockIdx.x / d.T, t = blockIdx.x % d.T;
    const int nt = a.num_tokens_per_rank ? min(a.num_tokens_per_rank[r], d.T) : d.T;
    if (t >= nt) return;
    __shared__ long long row_of_k[kMaxTopk];
    __shared__ float weight_of_k[kMaxTopk];

    // Locate the K rows: wave w searches selections w, w + n_waves, ...
    for (int k = wave; k < d.K; k += n_waves) {
        const size_t sel = (static_cast<size_t>(r) * d.T + t) * d.K + k;
        const int e = a.topk_idx[sel];
        long long row = -1;
        if (e >= 0 && e < d.E && !pair_blocked(a.mask, d.R, r, e / d.El)) {
            const long long lr = a.layout_range[static_cast<size_t>(e) * d.R + r];
            const int n = static_cast<int>(lr & 0xffffffffll), begin = static_cast<int>(lr >> 32);
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
    if (tid >= d.H / 8) return;

    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < d.K; k0 += 8) {
        uint4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const long long row = (k0 + j < d.K) ? row_of_k[k0 + j] : -1;
            v[j] = make_uint4(0, 0, 0, 0);
            if (row >= 0)
                v[j] = ld16_nt(reinterpret_cast<const uint4 *>(a.x + static_cast<size_t>(row) * d.H) + tid);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (k0 + j >= d.K || row_of_k[k0 + j] < 0) continue;
            const float w = weight_of_k[k0 + j];
            const uint32_t u[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                acc[2 * c] = fmaf(bf16_lo_to_f32(u[c]), w, acc[2 * c]);
                acc[2 * c + 1] = fmaf(bf16_hi_to_f32(u[c]), w, acc[2 * c + 1]);
            }
        }
    }
    uint4 out;
    out.x = f32_to_bf16(acc[0]) | (f32_to_bf16(acc[1]) << 16);
    out.y = f32_to_bf16(acc[2]) | (f32_to_bf16(acc[3]) << 16);
    out.z = f32_to_bf16(acc[4]) | (f32_to_bf16(acc[5]) << 16);
    out.w = f32_to_bf16(acc[6]) | (f32_to_bf16(acc[7]) << 16);
    st16_nt(reinterpret_cast<uint4 *>(a.combined + (static_cast<size_t>(r) * d.T + t) * d.H) + tid, out);
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

} // namespace

extern "C" {

size_t
nixl_amd_ep_ll_workspace_bytes(int num_ranks, int num_experts, int num_tokens, int num_topk) {
    if (num_ranks <= 0 || num_experts <= 0 || num_tokens < 0 || num_topk <= 0) return 0;
    return (static_cast<size_t>(num_ranks) * num_experts + static_cast<size_t>(num_ranks) * num_tokens * num_topk) * sizeof(int);
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
    if (workspace_bytes < nixl_amd_ep_ll_workspace_bytes(num_ranks, num_experts, num_tokens, num_topk))
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_dispatch: workspace too small");

    hipStream_t s = static_cast<hipStream_t>(stream);
    int *send_count = static_cast<int *>(workspace);
    int *pos = send_count + static_cast<size_t>(d.R) * d.E;

    const int W = (d.T + 63) / 64 > 0 ? (d.T + 63) / 64 : 1;
    int per_pass = kLayoutLdsBytes / (W * 8);
    if (per_pass < 1) return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "ll_dispatch: too many tokens per rank for the layout pass");
    if (per_pass > d.E) per_pass = d.E;
    hipLaunchKernelGGL(ll_layout_kernel, dim3(d.R), dim3(kLayoutThreads), static_cast<size_t>(per_pass) * W * 8, s, topk_idx,
                       num_tokens_per_rank, mask_buffer, send_count, pos, d, per_pass);
    HIP_TRY(hipGetLastError());

    DispatchArgs a{};
    a.recv_x = static_cast<uint8_t *>(packed_recv_x);
    a.recv_scales = packed_recv_x_scales;
    a.src_info = packed_recv_src_info;
    a.layout_range = reinterpret_cast<long long *>(packed_recv_layout_range);
    a.recv_count = packed_recv_count;
    a.stats = cumulative_local_expert_recv_stats;
    a.x = static_cast<const uint16_t *>(x);
    a.topk_idx = topk_idx;
    a.num_tokens_per_rank = num_tokens_per_rank;
    a.send_count = send_count;
    a.pos = pos;
    a.d = d;
    a.round_scale = round_scale;
    a.use_ue8m0 = use_ue8m0;
    const dim3 grid(static_cast<unsigned>(d.R) + static_cast<unsigned>(d.R) * d.T);
    const dim3 block(round_up_wave(d.H / 16));
    if (use_fp8)
        hipLaunchKernelGGL(ll_dispatch_kernel<true>, grid, block, 0, s, a);
    else
        hipLaunchKernelGGL(ll_dispatch_kernel<false>, grid, block, 0, s, a);
    HIP_TRY(hipGetLastError());
    return NIXL_AMD_OK;
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
    if (use_logfmt) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "ll_combine: the LogFMT payload codec is not implemented");
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
    a.d = d;
    hipLaunchKernelGGL(ll_combine_kernel, dim3(static_cast<unsigned>(d.R) * d.T), dim3(round_up_wave(d.H / 8)), 0,
                       static_cast<hipStream_t>(stream), a);
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
