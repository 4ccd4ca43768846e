// Gather/scatter copy kernels for descriptor lists and the C ABI that plans and launches
// them (declared in include/nixl_amd_hip.h).
//
// Data layout of a plan in HBM
//   16-byte-aligned descriptors of 256 B to 8 KiB, and longer ones whose source or
//   destination does not start on a 128-byte line, become pieces of at most 4 KiB: a
//   16-byte record {src, dst | (units - 1) << 56} and one wavefront each
//   (wavefront-per-descriptor for anything up to 4 KiB); pieces after the first start on a
//   destination line.
//   The other 16-byte-aligned descriptors (long and line-aligned, or tiny) are
//   concatenated, in request order, into one virtual stream measured in 16-byte units.  The stream is cut into chunks of
//   64*UPL units; one wavefront moves one chunk: lane l moves units k*64 + l of the chunk,
//   k < UPL, so every load/store instruction of a wave touches 1 KiB of consecutive bytes
//   unless a descriptor boundary falls inside it.  Chunks are classified on the host:
//     * a full chunk that lies inside one descriptor becomes a 16-byte record
//       {src address, dst address} in `uniform[]`; the uniform kernel reads its record
//       with one scalar load and issues UPL 128-bit loads and UPL 128-bit stores per lane
//       with wave-uniform base addresses — no search, no LDS, few registers;
//     * any other chunk (it crosses descriptor boundaries, or it is the short last chunk)
//       is listed by chunk index in `mixed[]`; the mixed kernel stages the descriptors the
//       chunk touches (span[m] = {first, last} for the m-th listed chunk; src[j], dst[j], prefix[j] = first unit of
//       descriptor j, prefix[n] = total) in a per-wave LDS slice and walks them.
//   Descriptors that are not 16-byte aligned in src, dst and len are cut into byte-range
//   work items handled by a third, byte-exact kernel.
//   Lists of equal-length, line-aligned descriptors of whole chunks (KV blocks) take none of
//   these steps: one pass writes their records, or, when the request is two index vectors
//   into two strided runs, a kernel writes them from the indices on the device.  Arenas and
//   the pinned buffers they are uploaded from are pooled.
//
// What is equal to the reference: the bytes.  For every descriptor, in list order,
// dst[0..len) = src[0..len), the result of the per-descriptor put/get loop at
// src/plugins/ucx/ucx_backend.cpp:1216-1244.  Descriptors of one request must not
// overlap each other's destination ranges (the reference's puts are unordered too).
#include <algorithm>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

#include "common.h"

namespace {

constexpr int kMixedWaves = 4; // waves per workgroup of the mixed and byte-path kernels
constexpr int kMixedThreads = kWaveSize * kMixedWaves;
constexpr uint32_t kGenericItemBytes = 16384; // byte-path work item size
constexpr int kMaxLdsDescs = 64; // descriptors a wave stages in LDS for one chunk
constexpr int kNumXcd = 8; // accelerator dies; workgroup i is dispatched to die i % 8

struct UniformRec {
    uint64_t src;
    uint64_t dst;
};

struct MixedArgs {
    const uint64_t *src; // [n]
    const uint64_t *dst; // [n]
    const uint64_t *prefix; // [n + 1], units
    const uint2 *span; // [n_mixed], {first desc, last desc} of the m-th mixed chunk
    const uint32_t *chunks; // [n_mixed] chunk indices
    uint64_t total_units;
    uint32_t n_mixed;
};

// A piece of a small descriptor: at most kPieceUnits (256) 16-byte units, one wavefront's work.
// 16 bytes a record: the unit count, less one, rides in the top byte of the destination
// address (device and pinned host addresses stay far below 2^56; the host checks it).
struct PieceRec {
    uint64_t src;
    uint64_t dst_units; // dst | (units - 1) << 56
};
constexpr int kPieceUnitsShift = 56;

struct GenericItem {
    uint64_t src;
    uint64_t dst;
    uint32_t len; // <= kGenericItemBytes
    uint32_t pad;
};

// 16-byte vector in the global address space, so that accesses compile to
// global_load/store_dwordx4 rather than flat instructions.
using v4u = __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned;
using gv4_ptr = __attribute__((address_space(1))) v4u *;
using gv4_cptr = const __attribute__((address_space(1))) v4u *;

// Cache policy of a plan's loads and stores (tuning field `nontemporal`), measured on MI355X
// with 16 KiB blocks (TB/s of traffic; sequential = consecutive descriptors adjoin):
//                                     seq->seq  random->seq  seq->random  random->random
//   1  nt loads,    nt stores           6.66       6.28         5.76          5.12
//   2  plain loads, plain stores        6.44       5.30         5.80          5.12
//   3  plain loads, sc1 nt stores       6.65       6.07         5.90          5.31
//   4  nt loads,    sc1 nt stores       6.71       6.35         5.80          5.15
// "sc1 nt" is a streaming store with device scope.  A plan whose destinations adjoin or
// advance by a constant step takes 4, any other plan 3.
constexpr int kPolNtNt = 1, kPolPlain = 2, kPolPlainSc1Nt = 3, kPolNtSc1Nt = 4;

template<int POL>
__device__ __forceinline__ v4u
load16(uint64_t addr) {
    gv4_cptr g = (gv4_cptr)(addr);
    if constexpr (POL == kPolNtNt || POL == kPolNtSc1Nt)
        return __builtin_nontemporal_load(g);
    else
        return *g;
}

template<int POL>
__device__ __forceinline__ void
store16(uint64_t addr, const v4u &v) {
    gv4_ptr g = (gv4_ptr)(addr);
    if constexpr (POL == kPolNtNt)
        __builtin_nontemporal_store(v, g);
    else if constexpr (POL == kPolPlain)
        *g = v;
    else
        asm volatile("global_store_dwordx4 %0, %1, off sc1 nt" : : "v"(g), "v"(v) : "memory");
}

// Workgroups are handed to the 8 dies round-robin.  With the swizzle on, die x works
// through one contiguous eighth of the record array instead of every eighth record.
__device__ __forceinline__ uint32_t
logical_workgroup(uint32_t n_wgs, bool swizzle) {
    const uint32_t b = blockIdx.x;
    if (!swizzle) return b;
    const uint32_t per = (n_wgs + kNumXcd - 1) / kNumXcd;
    return (b % kNumXcd) * per + b / kNumXcd; // may be >= n_wgs; caller checks
}

// One wavefront per full, single-descriptor chunk.  A record covers `chunks_per_rec`
// consecutive chunks of one descriptor (1 when the runs of such chunks differ in length;
// with equal-length descriptors, e.g. KV blocks, one record per descriptor), so that the
// record array stays small next to the payload.
template<int UPL, int POL, int WAVES>
__global__ void __launch_bounds__(kWaveSize *WAVES)
copy_uniform_kernel(const UniformRec *recs, uint32_t first_chunk, uint32_t n_chunks, uint32_t n_wgs, int swizzle, uint32_t chunks_per_rec) {
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const uint32_t wave = threadIdx.x / kWaveSize;
    const uint32_t wg = logical_workgroup(n_wgs, swizzle != 0);
    if (wg >= n_wgs || wg * WAVES + wave >= n_chunks) return;
    const uint32_t c = uniform(first_chunk + wg * WAVES + wave); // n_chunks, n_wgs: of this launch
    const uint32_t r = c / chunks_per_rec;
    const uint64_t off = static_cast<uint64_t>(c % chunks_per_rec) * (kWaveSize * UPL * 16u) + lane * 16u;
    // The record is the same for every lane and does not change while the kernel runs: read
    // through the constant address space it comes with ONE scalar load (left as an ordinary
    // global access the compiler makes it a 16-byte vector load by all 64 lanes, followed by
    // four lane-0 read-outs).
    const auto *words = reinterpret_cast<const __attribute__((address_space(4))) uint64_t *>(reinterpret_cast<uintptr_t>(recs + r));
    const uint64_t s = words[0] + off; // UniformRec::src
    const uint64_t d = words[1] + off; // UniformRec::dst
    v4u v[UPL];
#pragma unroll
    for (int k = 0; k < UPL; ++k)
        v[k] = load16<POL>(s + k * (kWaveSize * 16u));
#pragma unroll
    for (int k = 0; k < UPL; ++k)
        store16<POL>(d + k * (kWaveSize * 16u), v[k]);
}

// One wavefront per piece: the descriptor's own {src, dst, units} record, up to
// kPieceLoads 128-bit loads in flight per lane, then the stores.  No search and no LDS:
// the shape for descriptors of a few hundred bytes to a few KiB.

constexpr int kPieceLoads = 4;
constexpr uint32_t kPieceUnits = kWaveSize * kPieceLoads; // 4 KiB

// Workgroups are handed to the 8 dies round-robin; die x takes the x-th eighth of the records
// (grid = a multiple of 8 workgroups, `per_die` of them a die), so that a line of records is
// fetched into one die's cache instead of into several: with records dealt out round-robin the
// record lines were read 3.3 times over.
template<int POL, int LOADS, int WAVES>
__global__ void __launch_bounds__(kWaveSize *WAVES)
copy_piece_kernel(const PieceRec *__restrict__ recs, uint32_t n_recs, uint32_t per_die) { // recs, n_recs: of this launch
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const uint32_t wg = (blockIdx.x % kNumXcd) * per_die + blockIdx.x / kNumXcd;
    const uint32_t p = uniform(wg * WAVES + threadIdx.x / kWaveSize);
    if (p >= n_recs) return;
    const PieceRec packed = recs[p]; // same address in every lane of the wave: a scalar load
    struct {
        uint64_t src, dst;
    } rec{packed.src, packed.dst_units & ((1ull << kPieceUnitsShift) - 1ull)};
    const uint32_t units = static_cast<uint32_t>(packed.dst_units >> kPieceUnitsShift) + 1u; // >= 1
    // Lane 0 of every instruction sits on a 128-byte line of the destination: the piece's
    // units are shifted up by the destination's offset inside its line (the plan cuts pieces
    // so that shift + units <= kPieceUnits), and each store instruction then writes whole
    // lines except at the two ends of the piece.  A line written half by one instruction
    // and half by the next would go out as two partial writes.
    const uint32_t shift = static_cast<uint32_t>(rec.dst >> 4) & 7u;
    // Loads are unconditional (a lane outside the piece re-reads its first or last unit) so
    // that all of them are in flight together; only the stores are predicated.
    v4u v[LOADS];
#pragma unroll
    for (int k = 0; k < LOADS; ++k) {
        const uint32_t at = k * kWaveSize + lane;
        const uint32_t u = min(at < shift ? 0u : at - shift, units - 1);
        v[k] = load16<POL>(rec.src + u * 16ull);
    }
#pragma unroll
    for (int k = 0; k < LOADS; ++k) {
        const uint32_t at = k * kWaveSize + lane;
        if (at >= shift && at - shift < units) store16<POL>(rec.dst + (at - shift) * 16ull, v[k]);
    }
}

// One wavefront per chunk that crosses descriptor boundaries or is short.
template<int UPL, int POL>
__global__ void __launch_bounds__(kMixedThreads)
copy_mixed_kernel(MixedArgs a) {
    constexpr uint32_t kChunkUnits = kWaveSize * UPL;
    __shared__ uint64_t lds_prefix[kMixedWaves][kMaxLdsDescs + 1];
    __shared__ uint64_t lds_src[kMixedWaves][kMaxLdsDescs];
    __shared__ uint64_t lds_dst[kMixedWaves][kMaxLdsDescs];

    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const uint32_t wave = threadIdx.x / kWaveSize;
    const uint32_t n_waves = gridDim.x * kMixedWaves;

    for (uint32_t m = uniform(blockIdx.x * kMixedWaves + wave); m < a.n_mixed; m += n_waves) {
        const uint32_t c = uniform(a.chunks[m]);
        const uint2 sp = a.span[m];
        const uint32_t j0 = uniform(sp.x);
        const uint32_t j1 = uniform(sp.y);
        const uint64_t u0 = static_cast<uint64_t>(c) * kChunkUnits;
        const uint64_t remaining = a.total_units - u0; // > 0: the host lists only real chunks
        const uint32_t n_units = remaining < kChunkUnits ? static_cast<uint32_t>(remaining) : kChunkUnits;
        const uint32_t nd = j1 - j0 + 1;

        if (nd <= kMaxLdsDescs) {
            // Stage this chunk's descriptors in the wave's LDS slice, then each lane walks
            // forward through them as its unit index grows by 64 per step.  Only this
            // wave touches the slice, and a wave's LDS operations complete in order.
            __builtin_amdgcn_wave_barrier();
            if (lane < nd) {
                lds_prefix[wave][lane] = a.prefix[j0 + lane];
                lds_src[wave][lane] = a.src[j0 + lane];
                lds_dst[wave][lane] = a.dst[j0 + lane];
            }
            if (lane == 0) lds_prefix[wave][nd] = a.prefix[j0 + nd];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

            uint32_t jj = 0;
            uint64_t sa[UPL], da[UPL];
            v4u v[UPL];
#pragma unroll
            for (int k = 0; k < UPL; ++k) {
                const uint32_t i = k * kWaveSize + lane;
                sa[k] = 0;
                da[k] = 0;
                if (i < n_units) {
                    const uint64_t u = u0 + i;
                    while (jj + 1 < nd && lds_prefix[wave][jj + 1] <= u)
                        ++jj;
                    const uint64_t off = (u - lds_prefix[wave][jj]) * 16u;
                    sa[k] = lds_src[wave][jj] + off;
                    da[k] = lds_dst[wave][jj] + off;
                }
            }
#pragma unroll
            for (int k = 0; k < UPL; ++k)
                if (sa[k]) v[k] = load16<POL>(sa[k]);
#pragma unroll
            for (int k = 0; k < UPL; ++k)
                if (da[k]) store16<POL>(da[k], v[k]);
            __builtin_amdgcn_wave_barrier();
        } else {
            // More than 64 tiny descriptors in one chunk: bisect the global prefix array.
            for (uint32_t i = lane; i < n_units; i += kWaveSize) {
                const uint64_t u = u0 + i;
                uint32_t lo = j0, hi = j1;
                while (lo < hi) {
                    const uint32_t mid = lo + (hi - lo + 1) / 2;
                    if (a.prefix[mid] <= u)
                        lo = mid;
                    else
                        hi = mid - 1;
                }
                const uint64_t off = (u - a.prefix[lo]) * 16u;
                store16<POL>(a.dst[lo] + off, load16<POL>(a.src[lo] + off));
            }
        }
    }
}

struct __attribute__((packed, aligned(1))) unaligned16 {
    uint32_t w[4];
};

// One wavefront per byte-range work item; correct for any alignment and length.
__global__ void __launch_bounds__(kMixedThreads)
copy_generic_kernel(const GenericItem *items, uint32_t n_items) {
    const uint32_t lane = threadIdx.x & (kWaveSize - 1);
    const uint32_t wave = threadIdx.x / kWaveSize;
    const uint32_t n_waves = gridDim.x * kMixedWaves;
    for (uint32_t it = uniform(blockIdx.x * kMixedWaves + wave); it < n_items; it += n_waves) {
        const uint64_t src = uniform64(items[it].src);
        const uint64_t dst = uniform64(items[it].dst);
        const uint32_t len = uniform(items[it].len);
        const uint8_t *s = reinterpret_cast<const uint8_t *>(src);
        uint8_t *d = reinterpret_cast<uint8_t *>(dst);

        // Head: bytes until dst is 16-byte aligned (at most 15).
        uint32_t head = static_cast<uint32_t>((16u - (dst & 15u)) & 15u);
        if (head > len) head = len;
        if (lane < head) d[lane] = s[lane];
        const uint32_t body = (len - head) / 16u;
        const uint8_t *sb = s + head;
        uint4 *db = reinterpret_cast<uint4 *>(d + head);
        if (((src + head) & 15u) == 0) {
            const uint4 *sv = reinterpret_cast<const uint4 *>(sb);
            for (uint32_t i = lane; i < body; i += kWaveSize)
                db[i] = sv[i];
        } else {
            const unaligned16 *sv = reinterpret_cast<const unaligned16 *>(sb);
            for (uint32_t i = lane; i < body; i += kWaveSize) {
                const unaligned16 t = sv[i];
                db[i] = make_uint4(t.w[0], t.w[1], t.w[2], t.w[3]);
            }
        }
        const uint32_t done = head + body * 16u;
        const uint32_t tail = len - done; // < 16
        if (lane < tail) d[done + lane] = s[done + lane];
    }
}

// Reorders the records of a scattering plan (sources that follow each other, destinations
// that do not) so that inside every window of 1024 records the destinations ascend.  Which
// record a wavefront takes does not change the bytes that arrive; it changes the order in
// which DRAM sees the writes: 16 KiB blocks scattered over a pool went from 5.8 to 6.1 TB/s.
// One workgroup per window, bitonic network in LDS (the key is the destination address).
constexpr uint32_t kSortWindow = 1024;

__global__ void __launch_bounds__(kSortWindow / 2)
sort_records_kernel(UniformRec *recs, uint32_t n) {
    __shared__ uint64_t key[kSortWindow];
    __shared__ uint64_t val[kSortWindow];
    const uint32_t base = blockIdx.x * kSortWindow, tid = threadIdx.x;
    for (uint32_t i = tid; i < kSortWindow; i += kSortWindow / 2) {
        const bool in = base + i < n;
        key[i] = in ? recs[base + i].dst : ~0ull; // padding sorts to the end
        val[i] = in ? recs[base + i].src : 0ull;
    }
    __syncthreads();
    for (uint32_t size = 2; size <= kSortWindow; size <<= 1) {
        for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            const uint32_t lo = 2 * tid - (tid & (stride - 1)); // partner pairs (lo, lo + stride)
            const uint32_t hi = lo + stride;
            const bool up = (lo & size) == 0;
            const uint64_t a = key[lo], b = key[hi];
            if ((a > b) == up) {
                key[lo] = b;
                key[hi] = a;
                const uint64_t t = val[lo];
                val[lo] = val[hi];
                val[hi] = t;
            }
            __syncthreads();
        }
    }
    for (uint32_t i = tid; i < kSortWindow; i += kSortWindow / 2)
        if (base + i < n) recs[base + i] = UniformRec{val[i], key[i]};
}

// Records of an indexed plan: block i goes from src_base + src_index[i] * src_stride to
// dst_base + dst_index[i] * dst_stride.  The index vectors are the only per-request data
// that crosses the bus (8 bytes per block instead of 16, and no host loop over descriptors).
__global__ void __launch_bounds__(256)
index_records_kernel(UniformRec *recs, const int32_t *src_index, const int32_t *dst_index, uint32_t n, uint64_t src_base,
                     uint64_t src_stride, uint64_t dst_base, uint64_t dst_stride) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        recs[i] = UniformRec{src_base + static_cast<uint64_t>(src_index[i]) * src_stride,
                             dst_base + static_cast<uint64_t>(dst_index[i]) * dst_stride};
}

// The same for lists of several runs (a pool registered as several regions): index i of a
// list lies in the run r with first[r] <= i < first[r + 1], at base[r] + (i - first[r]) *
// stride[r].  The run tables (at most kMaxIndexRuns entries a side) are staged in LDS and
// searched by bisection.
constexpr uint32_t kMaxIndexRuns = 256;

__device__ __forceinline__ uint64_t
run_address(const uint64_t *first, const uint64_t *base, const uint64_t *stride, uint32_t n_runs, uint64_t index) {
    uint32_t lo = 0, hi = n_runs; // first[lo] <= index < first[hi] (first[n_runs] = infinity)
    while (hi - lo > 1) {
        const uint32_t mid = (lo + hi) / 2;
        if (first[mid] <= index) lo = mid;
        else hi = mid;
    }
    return base[lo] + (index - first[lo]) * stride[lo];
}

__global__ void __launch_bounds__(256)
index_records_runs_kernel(UniformRec *recs, const int32_t *src_index, const int32_t *dst_index, uint32_t n,
                          const nixl_amd_copy_run_t *src_runs, uint32_t n_src, const nixl_amd_copy_run_t *dst_runs,
                          uint32_t n_dst) {
    __shared__ uint64_t first[2][kMaxIndexRuns], base[2][kMaxIndexRuns], stride[2][kMaxIndexRuns];
    for (uint32_t r = threadIdx.x; r < n_src; r += blockDim.x) {
        first[0][r] = src_runs[r].first_index;
        base[0][r] = src_runs[r].base;
        stride[0][r] = src_runs[r].stride;
    }
    for (uint32_t r = threadIdx.x; r < n_dst; r += blockDim.x) {
        first[1][r] = dst_runs[r].first_index;
        base[1][r] = dst_runs[r].base;
        stride[1][r] = dst_runs[r].stride;
    }
    __syncthreads();
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        recs[i] = UniformRec{run_address(first[0], base[0], stride[0], n_src, static_cast<uint64_t>(src_index[i])),
                             run_address(first[1], base[1], stride[1], n_dst, static_cast<uint64_t>(dst_index[i]))};
}

// Records of a plan whose runs of uniform chunks differ in length: run r covers chunks
// first_chunk[r] .. first_chunk[r + 1] - 1 and chunk c of it lies c - first_chunk[r] chunks
// behind the run's start on both sides.  A thread per chunk finds its run by bisection (the
// table stays in the L2), so that one long run among short ones costs no more than any other;
// 16 bytes per run cross the bus instead of 16 per chunk.
__global__ void __launch_bounds__(256)
expand_runs_kernel(UniformRec *recs, const UniformRec *runs, const uint32_t *first_chunk, uint32_t n_runs, uint32_t n_chunks,
                   uint32_t chunk_bytes) {
    for (uint64_t c64 = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; c64 < n_chunks;
         c64 += static_cast<uint64_t>(gridDim.x) * blockDim.x) {
        const uint32_t c = static_cast<uint32_t>(c64);
        uint32_t lo = 0, hi = n_runs; // first_chunk[lo] <= c < first_chunk[hi]
        while (hi - lo > 1) {
            const uint32_t mid = lo + (hi - lo) / 2;
            if (first_chunk[mid] <= c) lo = mid;
            else hi = mid;
        }
        const uint64_t off = static_cast<uint64_t>(c - first_chunk[lo]) * chunk_bytes;
        recs[c] = UniformRec{runs[lo].src + off, runs[lo].dst + off};
    }
}

// Largest grid of one launch: HIP refuses grids of 2^32 or more threads, i.e. 2^22 workgroups of
// 16 waves; a plan with more work than that goes out as several launches.
constexpr uint32_t kMaxGrid = 1u << 21;

struct UniformLaunch {
    const UniformRec *recs;
    uint32_t first_chunk, n_chunks, n_wgs, chunks_per_rec;
    int swizzle;
    dim3 grid;
    hipStream_t stream;
};

template<int UPL, int POL>
void
launch_uniform(int waves, const UniformLaunch &u) {
#define NIXL_AMD_UNIFORM(WV)                                                                              \
    hipLaunchKernelGGL((copy_uniform_kernel<UPL, POL, WV>), u.grid, dim3(kWaveSize * WV), 0, u.stream, u.recs, \
                       u.first_chunk, u.n_chunks, u.n_wgs, u.swizzle, u.chunks_per_rec)
    switch (waves) {
    case 1: NIXL_AMD_UNIFORM(1); break;
    case 2: NIXL_AMD_UNIFORM(2); break;
    case 4: NIXL_AMD_UNIFORM(4); break;
    case 8: NIXL_AMD_UNIFORM(8); break;
    default: NIXL_AMD_UNIFORM(16); break;
    }
#undef NIXL_AMD_UNIFORM
}

template<int POL>
void
launch_uniform_upl(int upl, int waves, const UniformLaunch &u) {
    switch (upl) {
    case 1: launch_uniform<1, POL>(waves, u); break;
    case 2: launch_uniform<2, POL>(waves, u); break;
    case 4: launch_uniform<4, POL>(waves, u); break;
    case 8: launch_uniform<8, POL>(waves, u); break;
    default: launch_uniform<16, POL>(waves, u); break;
    }
}

template<int POL>
void
launch_mixed_upl(int upl, dim3 grid, hipStream_t s, const MixedArgs &a) {
    const dim3 block(kMixedThreads);
    switch (upl) {
    case 1: hipLaunchKernelGGL((copy_mixed_kernel<1, POL>), grid, block, 0, s, a); break;
    case 2: hipLaunchKernelGGL((copy_mixed_kernel<2, POL>), grid, block, 0, s, a); break;
    case 4: hipLaunchKernelGGL((copy_mixed_kernel<4, POL>), grid, block, 0, s, a); break;
    case 8: hipLaunchKernelGGL((copy_mixed_kernel<8, POL>), grid, block, 0, s, a); break;
    default: hipLaunchKernelGGL((copy_mixed_kernel<16, POL>), grid, block, 0, s, a); break;
    }
}

template<int POL>
void
launch_pieces(uint32_t w, uint32_t n_wgs, hipStream_t s, const PieceRec *recs, uint32_t n) {
    const dim3 block(kWaveSize * w);
    const uint32_t per_die = (n_wgs + kNumXcd - 1) / kNumXcd;
    const dim3 grid(per_die * kNumXcd); // surplus workgroups exit at once
    if (w == 1)
        hipLaunchKernelGGL((copy_piece_kernel<POL, kPieceLoads, 1>), grid, block, 0, s, recs, n, per_die);
    else if (w == 2)
        hipLaunchKernelGGL((copy_piece_kernel<POL, kPieceLoads, 2>), grid, block, 0, s, recs, n, per_die);
    else
        hipLaunchKernelGGL((copy_piece_kernel<POL, kPieceLoads, 4>), grid, block, 0, s, recs, n, per_die);
}

// Calls f.template operator()<POL>() for the plan's policy.
template<typename F>
void
with_policy(int policy, F &&f) {
    switch (policy) {
    case kPolNtNt: f.template operator()<kPolNtNt>(); break;
    case kPolPlain: f.template operator()<kPolPlain>(); break;
    case kPolPlainSc1Nt: f.template operator()<kPolPlainSc1Nt>(); break;
    default: f.template operator()<kPolNtSc1Nt>(); break;
    }
}

} // namespace

namespace {

// Plan arenas and the pinned buffers they are uploaded from are recycled: a request whose
// descriptor list changes every time (paged KV) would otherwise pay a hipMalloc and a
// pageable-memory copy per request.  Blocks come in power-of-two sizes; the cache keeps the
// most recently returned ones up to a count and a byte limit and frees the oldest beyond that.
class BlockCache {
public:
    explicit BlockCache(bool pinned) : pinned_(pinned) {}

    // A block of at least `bytes` on `device` (ignored for pinned memory); `cap` receives its size.
    hipError_t
    get(int device, size_t bytes, void **out, size_t *cap) {
        size_t size = 4096;
        while (size < bytes)
            size <<= 1;
        {
            std::lock_guard<std::mutex> lock(mutex_);
            for (size_t i = 0; i < free_.size(); ++i)
                if (free_[i].size == size && (pinned_ || free_[i].device == device)) {
                    *out = free_[i].ptr;
                    *cap = size;
                    held_ -= size;
                    free_.erase(free_.begin() + static_cast<long>(i));
                    return hipSuccess;
                }
        }
        *cap = size;
        return pinned_ ? hipHostMalloc(out, size, hipHostMallocDefault) : hipMalloc(out, size);
    }

    // The block just given back is the likeliest to be asked for again (the next request of the
    // same shape), so when the cache is full the oldest blocks make room for it.
    void
    put(int device, void *ptr, size_t size) {
        std::vector<Block> evicted;
        {
            std::lock_guard<std::mutex> lock(mutex_);
            if (size <= kMaxHeld) {
                while (!free_.empty() && (held_ + size > kMaxHeld || free_.size() >= kMaxBlocks)) {
                    evicted.push_back(free_.front());
                    held_ -= free_.front().size;
                    free_.erase(free_.begin());
                }
                free_.push_back(Block{ptr, size, device});
                held_ += size;
            } else {
                evicted.push_back(Block{ptr, size, device});
            }
        }
        for (const Block &b : evicted) {
            if (pinned_)
                (void)hipHostFree(b.ptr);
            else
                (void)hipFree(b.ptr);
        }
    }

private:
    struct Block {
        void *ptr;
        size_t size;
        int device;
    };
    static constexpr size_t kMaxHeld = 256u << 20;
    static constexpr size_t kMaxBlocks = 32;
    const bool pinned_;
    std::mutex mutex_;
    std::vector<Block> free_;
    size_t held_ = 0;
};

BlockCache &
arena_cache() {
    static BlockCache *c = new BlockCache(false); // never destroyed: device memory outlives static teardown order
    return *c;
}

// Plans are uploaded on a stream of their own that does not synchronise with the default
// stream, so that preparing one request does not wait for another that is still copying.
hipError_t
upload_stream(int device, hipStream_t *out) {
    constexpr int kMaxDevices = 64;
    static std::mutex mutex;
    static hipStream_t streams[kMaxDevices] = {};
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mutex);
    if (!streams[device]) {
        const hipError_t e = hipStreamCreateWithFlags(&streams[device], hipStreamNonBlocking);
        if (e != hipSuccess) return e;
    }
    *out = streams[device];
    return hipSuccess;
}

BlockCache &
upload_cache() {
    static BlockCache *c = new BlockCache(true);
    return *c;
}

} // namespace

struct nixl_amd_copy_plan {
    int device = 0;
    int upl = 1;
    int policy = kPolNtSc1Nt;
    int piece_policy = kPolNtNt; // pieces of a few hundred bytes to 4 KiB: 225 us for the 262 144-descriptor stress, against 239 (4) and 285 (3)
    int waves = 1;
    int swizzle = 0;
    uint32_t max_wgs = 0;
    // device arrays
    void *arena = nullptr;
    size_t arena_bytes = 0; // bytes in use
    size_t arena_cap = 0; // size of the block
    const UniformRec *uniform_recs = nullptr;
    uint32_t n_uniform = 0; // uniform chunks
    uint32_t chunks_per_rec = 1;
    uint32_t uniform_wgs = 0;
    MixedArgs mixed_args{};
    uint32_t mixed_wgs = 0;
    const PieceRec *piece_recs = nullptr;
    uint32_t n_pieces = 0;
    const GenericItem *generic_items = nullptr;
    uint32_t n_generic = 0;
    uint32_t generic_wgs = 0;
    nixl_amd_copy_plan_info_t info{};
    hipEvent_t ev0 = nullptr, ev1 = nullptr; // timing events, created on first use
    // A plan built from index vectors returns before its records exist: they are written by
    // kernels queued on the upload stream, `uploaded` is recorded behind them, and the first
    // launches wait for it on their own stream.
    hipEvent_t uploaded = nullptr;
    // Recorded behind the kernels of every launch (not on a capturing stream): destroying the
    // plan while it has not completed is refused, because the arena would go back to the pool
    // and the next plan's upload would overwrite records a running kernel still reads.
    hipEvent_t launched = nullptr;
    bool launched_valid = false;
};

// Pinned buffers whose contents are still travelling to the device: each goes back to the
// upload cache once the event recorded behind its copy has completed, which the next plan
// creation on the device looks for.
struct PendingUpload {
    hipEvent_t done;
    void *staging;
    size_t cap;
};
static std::mutex g_pending_mutex;
static std::map<int, std::vector<PendingUpload>> g_pending; // by device

static void
reap_uploads(int device) {
    std::lock_guard<std::mutex> lock(g_pending_mutex);
    auto &list = g_pending[device];
    for (size_t i = 0; i < list.size();) {
        const hipError_t e = hipEventQuery(list[i].done);
        if (e == hipErrorNotReady) {
            (void)hipGetLastError();
            ++i;
            continue;
        }
        (void)hipEventDestroy(list[i].done);
        upload_cache().put(device, list[i].staging, list[i].cap);
        list[i] = list.back();
        list.pop_back();
    }
}

// Hands `staging` over: recycled when everything queued on `up` so far has run.  Without an
// event to watch, the stream is waited for instead.
static void
recycle_after(int device, hipStream_t up, void *staging, size_t cap) {
    hipEvent_t done = nullptr;
    if (hipEventCreateWithFlags(&done, hipEventDisableTiming) == hipSuccess && hipEventRecord(done, up) == hipSuccess) {
        std::lock_guard<std::mutex> lock(g_pending_mutex);
        g_pending[device].push_back(PendingUpload{done, staging, cap});
        return;
    }
    (void)hipGetLastError();
    if (done) (void)hipEventDestroy(done);
    (void)hipStreamSynchronize(up);
    upload_cache().put(device, staging, cap);
}

// The plan's records are in place (or `wait` and they are not yet: block until they are).
// Returns hipErrorNotReady when they are still being written and `wait` is false.
static hipError_t
settle_upload(nixl_amd_copy_plan *plan, bool wait) {
    if (!plan->uploaded) return hipSuccess;
    hipError_t e = wait ? hipEventSynchronize(plan->uploaded) : hipEventQuery(plan->uploaded);
    if (e == hipErrorNotReady) {
        (void)hipGetLastError();
        return e;
    }
    (void)hipEventDestroy(plan->uploaded);
    plan->uploaded = nullptr;
    return e;
}

struct Tuning {
    int upl = 1, nt = 0, waves = 1, swizzle = 0, sort_scatter = 0;
    uint32_t max_wgs = 0;
};

// Defaults from a sweep on MI355X: the smallest chunk (one 128-bit load and store per lane,
// one wave per workgroup) gave the highest HBM rate; the cache policy follows the
// destination pattern.
static int
parse_tuning(const nixl_amd_copy_tuning_t *tuning, Tuning &t, const char *who) {
    if (tuning) {
        if (tuning->units_per_lane) t.upl = tuning->units_per_lane;
        if (tuning->nontemporal) t.nt = tuning->nontemporal;
        if (tuning->max_workgroups > 0) t.max_wgs = static_cast<uint32_t>(tuning->max_workgroups);
        if (tuning->waves_per_workgroup) t.waves = tuning->waves_per_workgroup;
        if (tuning->xcd_swizzle) t.swizzle = tuning->xcd_swizzle == 1 ? 1 : 0;
        t.sort_scatter = tuning->sort_scatter;
    }
    if (t.upl != 1 && t.upl != 2 && t.upl != 4 && t.upl != 8 && t.upl != 16)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, std::string(who) + ": units_per_lane must be 1, 2, 4, 8 or 16");
    if (t.nt < 0 || t.nt > 4) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, std::string(who) + ": nontemporal must be 0 to 4");
    if (t.waves != 1 && t.waves != 2 && t.waves != 4 && t.waves != 8 && t.waves != 16)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, std::string(who) + ": waves_per_workgroup must be 1, 2, 4, 8 or 16");
    return NIXL_AMD_OK;
}

// Whether equal blocks of `len` bytes can be a plan of one record per block: whole chunks,
// long enough that a record is small next to its payload.
static bool
block_len_fits(uint64_t len, const Tuning &t) {
    const uint64_t chunk_bytes = static_cast<uint64_t>(kWaveSize) * t.upl * 16u;
    return len >= 8192 && len % chunk_bytes == 0;
}

constexpr int kNotBlocks = 1; // build_block_plan: the records are not what a block plan takes (no error recorded)

// A plan of `n_recs` equal blocks of `len` bytes whose {src, dst} records the host has written
// to the start of the pinned buffer `staging`.  One vectorisable pass over the records checks
// them (every address on a 128-byte line, none null, no range that wraps) and reads the
// pattern of the destinations (cache policy) and of the sources (record order); the copy to the
// device, the optional sort and the event behind them are queued on the upload stream and not
// waited for.  `staging` is taken over in every case.  Returns kNotBlocks when the records do
// not qualify, so that the caller can lower the request the general way.
static int
build_block_plan(int device, const Tuning &t, void *staging, size_t staging_cap, size_t n_recs, uint64_t len, size_t n_descs,
                 const nixl_amd_copy_record_facts_t *facts, nixl_amd_copy_plan_t **out) {
    const uint64_t chunk_bytes = static_cast<uint64_t>(kWaveSize) * t.upl * 16u;
    const auto *recs = static_cast<const UniformRec *>(staging);
    bool fits = n_recs > 0 && block_len_fits(len, t) && n_recs < (1ull << 31) && n_recs * (len / chunk_bytes) < (1ull << 32);
    uint64_t regular = 0, src_follows = 0, steps = n_recs ? n_recs - 1 : 0;
    if (fits && facts) {
        // the caller looked at every record while it wrote them
        fits = (facts->address_bits & 127u) == 0;
        regular = facts->regular_dst_steps;
        src_follows = facts->following_src_steps;
        steps = facts->steps;
    } else if (fits) {
        uint64_t misfit = 0;
        for (size_t i = 0; i < n_recs; ++i) {
            const uint64_t a = recs[i].src, b = recs[i].dst;
            misfit |= ((a | b) & 127u) | static_cast<uint64_t>(a == 0) | static_cast<uint64_t>(b == 0) |
                static_cast<uint64_t>(a + len < a) | static_cast<uint64_t>(b + len < b);
        }
        fits = misfit == 0;
        // Destination steps that are regular (one block on, or the same step as the one before)
        // and source steps that go one block on; nothing is carried from one iteration to the
        // next, so that the loop vectorises.
        if (n_recs > 1) {
            regular += (recs[1].dst - recs[0].dst) == len;
            src_follows += (recs[1].src - recs[0].src) == len;
        }
        for (size_t i = 2; i < n_recs; ++i) {
            const uint64_t step = recs[i].dst - recs[i - 1].dst, before = recs[i - 1].dst - recs[i - 2].dst;
            regular += static_cast<uint32_t>(step == len) | static_cast<uint32_t>(step == before);
            src_follows += static_cast<uint32_t>((recs[i].src - recs[i - 1].src) == len);
        }
    }
    if (!fits) {
        upload_cache().put(device, staging, staging_cap);
        return kNotBlocks;
    }
    const size_t bytes = n_recs * sizeof(UniformRec);
    auto *plan = new nixl_amd_copy_plan();
    plan->device = device;
    plan->upl = t.upl;
    plan->waves = t.waves;
    plan->swizzle = t.swizzle;
    plan->max_wgs = t.max_wgs;
    // cache policy by destination pattern, as in the general lowering
    const bool scattered = !(steps == 0 || 2 * regular >= steps);
    // a scatter out of consecutive memory is put into ascending destination order, window by window
    const bool sort = scattered && t.sort_scatter != 2 && 2 * src_follows >= steps && n_recs >= kSortWindow;
    plan->policy = t.nt ? t.nt : ((!scattered || sort) ? kPolNtSc1Nt : kPolPlainSc1Nt);
    hipStream_t up = nullptr;
    hipError_t e = arena_cache().get(device, bytes, &plan->arena, &plan->arena_cap);
    if (e == hipSuccess) e = upload_stream(device, &up);
    if (e == hipSuccess) e = hipMemcpyAsync(plan->arena, staging, bytes, hipMemcpyHostToDevice, up);
    if (e == hipSuccess && sort) {
        hipLaunchKernelGGL(sort_records_kernel, dim3(static_cast<uint32_t>((n_recs + kSortWindow - 1) / kSortWindow)),
                           dim3(kSortWindow / 2), 0, up, static_cast<UniformRec *>(plan->arena), static_cast<uint32_t>(n_recs));
        e = hipGetLastError();
    }
    // No wait here: the event goes behind the copy, launches wait for it on their stream.
    if (e == hipSuccess) e = hipEventCreateWithFlags(&plan->uploaded, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventRecord(plan->uploaded, up);
    if (e != hipSuccess) {
        if (up) (void)hipStreamSynchronize(up); // whatever was queued reads the buffers given back below
        if (plan->uploaded) (void)hipEventDestroy(plan->uploaded);
        upload_cache().put(device, staging, staging_cap);
        if (plan->arena) arena_cache().put(device, plan->arena, plan->arena_cap);
        delete plan;
        return nixl_amd_fail(NIXL_AMD_ERR_HIP, std::string("plan upload: ") + hipGetErrorString(e));
    }
    recycle_after(device, up, staging, staging_cap);
    plan->arena_bytes = bytes;
    plan->uniform_recs = static_cast<const UniformRec *>(plan->arena);
    plan->chunks_per_rec = static_cast<uint32_t>(len / chunk_bytes);
    plan->n_uniform = static_cast<uint32_t>(n_recs * plan->chunks_per_rec);
    plan->uniform_wgs = (plan->n_uniform + static_cast<uint32_t>(t.waves) - 1) / static_cast<uint32_t>(t.waves);
    plan->info.payload_bytes = n_recs * len;
    plan->info.vec_descs = n_descs;
    plan->info.plan_device_bytes = bytes;
    plan->info.vec_chunks = plan->n_uniform;
    plan->info.uniform_chunks = plan->n_uniform;
    plan->info.units_per_lane = static_cast<uint32_t>(t.upl);
    plan->info.uniform_workgroups = plan->uniform_wgs;
    *out = plan;
    return NIXL_AMD_OK;
}

// A pinned upload buffer that its caller fills with block records (nixl_amd_copy_records_begin).
struct nixl_amd_copy_records {
    void *staging = nullptr;
    size_t staging_cap = 0;
    size_t max_records = 0;
};

extern "C" {

int
nixl_amd_copy_plan_create(const nixl_amd_copy_desc_t *descs,
                          size_t n,
                          int device,
                          const nixl_amd_copy_tuning_t *tuning,
                          nixl_amd_copy_plan_t **out) {
    if (!out) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_create: out is null");
    *out = nullptr;
    if (!descs && n) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_create: descs is null");
    if (n >= (1ull << 32)) return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "plan_create: more than 2^32-1 descriptors");

    Tuning t;
    if (const int rc = parse_tuning(tuning, t, "plan_create")) return rc;
    const int upl = t.upl, waves = t.waves, swizzle = t.swizzle;
    int nt = t.nt;
    const uint32_t max_wgs = t.max_wgs;

    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev <= 0)
        return nixl_amd_fail(NIXL_AMD_ERR_NO_DEVICE, "plan_create: no HIP device");
    if (device < 0 || device >= ndev) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_create: bad device index");
    const DeviceScope on_device(device);
    HIP_TRY(on_device.status());

    const uint64_t chunk_units = static_cast<uint64_t>(kWaveSize) * upl;

    // ---- fast path: equal-length, line-aligned descriptors of whole chunks (KV blocks) ----
    // One pass over the descriptors writes the {src, dst} records straight into the pinned
    // upload buffer; nothing else is built.
    if (n > 0 && block_len_fits(descs[0].len, t)) {
        // Descriptors whose length is a multiple of the first one's (neighbouring blocks that
        // the caller merged) become that many records; room for twice as many records as
        // descriptors, beyond that the general lowering takes over.
        const uint64_t len0 = descs[0].len;
        const size_t cap = 2 * n;
        void *staging = nullptr;
        size_t staging_cap = 0;
        reap_uploads(device);
        const hipError_t e = upload_cache().get(device, cap * sizeof(UniformRec), &staging, &staging_cap);
        if (e != hipSuccess)
            return nixl_amd_fail(NIXL_AMD_ERR_HIP, std::string("hipHostMalloc(plan upload buffer): ") + hipGetErrorString(e));
        auto *recs = static_cast<UniformRec *>(staging);
        bool misfit = false;
        size_t n_recs = 0;
        for (size_t i = 0; i < n; ++i) {
            const nixl_amd_copy_desc_t &d = descs[i];
            if (d.len == len0) {
                recs[n_recs++] = UniformRec{d.src, d.dst};
                continue;
            }
            const uint64_t k = d.len / len0;
            if (k == 0 || d.len != k * len0 || k > cap - n_recs || d.src + d.len < d.src || d.dst + d.len < d.dst) {
                misfit = true;
                break;
            }
            for (uint64_t j = 0; j < k; ++j)
                recs[n_recs++] = UniformRec{d.src + j * len0, d.dst + j * len0};
            if (n_recs + (n - 1 - i) > cap) { // the rest must still fit one record each
                misfit = true;
                break;
            }
        }
        if (misfit) {
            upload_cache().put(device, staging, staging_cap); // something else: the general lowering decides
        } else {
            const int rc = build_block_plan(device, t, staging, staging_cap, n_recs, len0, n, nullptr, out);
            if (rc != kNotBlocks) return rc;
        }
    }

    // ---- host-side lowering ------------------------------------------------------
    std::vector<uint64_t> vsrc, vdst, vprefix;
    std::vector<GenericItem> items;
    std::vector<PieceRec> pieces;
    // Descriptors of 256 B to 8 KiB, and longer ones whose source or destination does not
    // start on a 128-byte line, go to the piece kernel: measured faster there (fewer lines
    // split between wavefronts); line-aligned long descriptors stream best in 1 KiB chunks.
    constexpr uint64_t kPieceMinUnits = 16, kPieceMaxDescUnits = 512;
    vsrc.reserve(n);
    vdst.reserve(n);
    vprefix.reserve(n + 1);
    pieces.reserve(n);
    uint64_t units = 0, payload = 0, n_generic_descs = 0, n_piece_descs = 0;
    for (size_t i = 0; i < n; ++i) {
        const nixl_amd_copy_desc_t &d = descs[i];
        if (d.len == 0) continue;
        if (d.src == 0 || d.dst == 0)
            return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_create: null address in descriptor " + std::to_string(i));
        if (d.src + d.len < d.src || d.dst + d.len < d.dst)
            return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_create: address range wraps in descriptor " + std::to_string(i));
        payload += d.len;
        const bool aligned16 = ((d.src | d.dst | d.len) & 15u) == 0;
        const uint64_t du = d.len / 16u;
        if (aligned16 && du >= kPieceMinUnits && (du < kPieceMaxDescUnits || ((d.src | d.dst) & 127u) != 0)) {
            // Pieces of at most kPieceUnits units, one wavefront each.  The first piece is
            // cut so that every later one starts on a 128-byte line of the destination: no
            // line is then written by two wavefronts.
            if ((d.dst + d.len) >> kPieceUnitsShift)
                return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_create: destination address beyond 2^56");
            const uint64_t head = kPieceUnits - ((d.dst >> 4) & 7u);
            for (uint64_t first = 0; first < du;) {
                const uint64_t n_units = std::min<uint64_t>(first == 0 ? head : kPieceUnits, du - first);
                pieces.push_back(PieceRec{d.src + first * 16u, (d.dst + first * 16u) | ((n_units - 1) << kPieceUnitsShift)});
                first += n_units;
            }
            ++n_piece_descs;
        } else if (aligned16) {
            vsrc.push_back(d.src);
            vdst.push_back(d.dst);
            vprefix.push_back(units);
            units += d.len / 16u;
        } else {
            ++n_generic_descs;
            for (uint64_t off = 0; off < d.len; off += kGenericItemBytes) {
                GenericItem it{};
                it.src = d.src + off;
                it.dst = d.dst + off;
                it.len = static_cast<uint32_t>(std::min<uint64_t>(kGenericItemBytes, d.len - off));
                items.push_back(it);
            }
        }
    }
    vprefix.push_back(units);
    const size_t nv = vsrc.size();
    const uint64_t n_chunks64 = (units + chunk_units - 1) / chunk_units;
    if (n_chunks64 >= (1ull << 32) || items.size() >= (1ull << 32) || pieces.size() >= (1ull << 31))
        return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "plan_create: request too large for 32-bit chunk index");
    const uint32_t n_chunks = static_cast<uint32_t>(n_chunks64);

    // Walk the stream by descriptor: the chunks that lie wholly inside one descriptor form a
    // run of uniform chunks (one step for the whole run, however long); a chunk that holds a
    // descriptor boundary, or the short last chunk, is "mixed" and remembers the first and
    // last descriptor it touches.  If all runs have the same length L, one record per run is
    // kept and the kernel derives the rest; otherwise every uniform chunk gets its record.
    struct Run {
        uint64_t src, dst;
        uint32_t chunks;
    };
    std::vector<Run> runs;
    std::vector<uint32_t> mixed;
    std::vector<uint2> span; // per mixed chunk: first and last descriptor
    uint32_t n_uniform_chunks = 0, common_run = 0;
    bool runs_equal = true;
    // Equal-length descriptors that are whole numbers of chunks (KV blocks): every descriptor
    // is one run, nothing is mixed, and the walk below is not needed.
    const uint64_t chunk_bytes_all = chunk_units * 16u;
    bool all_whole = nv > 0;
    for (size_t j = 0; j < nv && all_whole; ++j)
        all_whole = (vprefix[j + 1] - vprefix[j]) * 16u == (vprefix[1] - vprefix[0]) * 16u;
    all_whole = all_whole && ((vprefix[1] - vprefix[0]) * 16u) % chunk_bytes_all == 0;
    if (all_whole) {
        common_run = static_cast<uint32_t>((vprefix[1] - vprefix[0]) * 16u / chunk_bytes_all);
        n_uniform_chunks = n_chunks;
    } else {
        size_t j = 0;
        for (uint32_t c = 0; c < n_chunks;) {
            const uint64_t first = static_cast<uint64_t>(c) * chunk_units;
            while (vprefix[j + 1] <= first)
                ++j;
            const uint64_t inside = (vprefix[j + 1] - first) / chunk_units; // whole chunks left in descriptor j
            if (inside > 0) {
                const uint32_t len = static_cast<uint32_t>(inside);
                const uint64_t off = (first - vprefix[j]) * 16u;
                runs.push_back(Run{vsrc[j] + off, vdst[j] + off, len});
                if (common_run == 0)
                    common_run = len;
                else if (common_run != len)
                    runs_equal = false;
                n_uniform_chunks += len;
                c += len;
                continue;
            }
            const uint64_t last = std::min(units, first + chunk_units) - 1;
            size_t jl = j;
            while (vprefix[jl + 1] <= last)
                ++jl;
            mixed.push_back(c);
            span.push_back(make_uint2(static_cast<uint32_t>(j), static_cast<uint32_t>(jl)));
            ++c;
        }
    }
    std::vector<UniformRec> uni;
    std::vector<uint32_t> first_chunk; // runs of different lengths: run r starts at uniform chunk first_chunk[r]
    uint32_t chunks_per_rec = 1;
    if (all_whole) {
        chunks_per_rec = common_run;
        uni.resize(nv);
        for (size_t j = 0; j < nv; ++j)
            uni[j] = UniformRec{vsrc[j], vdst[j]};
    } else if (runs_equal && common_run > 1) {
        chunks_per_rec = common_run;
        uni.reserve(runs.size());
        for (const Run &r : runs)
            uni.push_back(UniformRec{r.src, r.dst});
    } else if (!runs.empty()) {
        // a record per chunk, written on the device from a record per run
        uni.reserve(runs.size());
        first_chunk.reserve(runs.size() + 1);
        uint32_t at = 0;
        for (const Run &r : runs) {
            uni.push_back(UniformRec{r.src, r.dst});
            first_chunk.push_back(at);
            at += r.chunks;
        }
        first_chunk.push_back(at);
    }
    const bool expand = !first_chunk.empty();
    const size_t n_uniform_recs = expand ? n_uniform_chunks : uni.size();

    // ---- one device arena for all plan arrays --------------------------------------
    auto align256 = [](size_t x) { return (x + 255) & ~size_t(255); };
    const bool need_desc_arrays = !mixed.empty();
    // The arena starts with the records the copy kernel reads.  When they are expanded on the
    // device, that stretch is not uploaded: the upload starts behind it, and the records per run
    // and their first chunks travel at the arena's end.
    const size_t off_uni = 0;
    const size_t off_src = off_uni + align256(n_uniform_recs * sizeof(UniformRec));
    const size_t off_dst = off_src + (need_desc_arrays ? align256(nv * 8) : 0);
    const size_t off_prefix = off_dst + (need_desc_arrays ? align256(nv * 8) : 0);
    const size_t off_span = off_prefix + (need_desc_arrays ? align256((nv + 1) * 8) : 0);
    const size_t off_mixed = off_span + (need_desc_arrays ? align256(span.size() * sizeof(uint2)) : 0);
    const size_t off_pieces = off_mixed + align256(mixed.size() * sizeof(uint32_t));
    const size_t off_items = off_pieces + align256(pieces.size() * sizeof(PieceRec));
    const size_t off_runs = off_items + align256(items.size() * sizeof(GenericItem));
    const size_t off_first = off_runs + (expand ? align256(uni.size() * sizeof(UniformRec)) : 0);
    const size_t total = off_first + (expand ? align256(first_chunk.size() * sizeof(uint32_t)) : 0);
    const size_t upload_from = expand ? off_src : 0;

    auto *plan = new nixl_amd_copy_plan();
    plan->device = device;
    plan->upl = upl;
    if (nt == 0) {
        // Destinations that adjoin (a gather into staging, one long copy) or advance by a
        // constant step (the same block of every layer of a pool) take non-temporal loads;
        // destinations without such a pattern (a scatter over a pool) take plain loads.
        uint64_t pairs = 0, regular = 0, prev_dst = 0, prev_end = 0, prev_step = 0;
        for (size_t i = 0; i < n; ++i) {
            if (descs[i].len == 0) continue;
            if (prev_end) {
                const uint64_t step = descs[i].dst - prev_dst;
                ++pairs;
                regular += (descs[i].dst == prev_end || step == prev_step);
                prev_step = step;
            }
            prev_dst = descs[i].dst;
            prev_end = descs[i].dst + descs[i].len;
        }
        nt = (pairs == 0 || 2 * regular >= pairs) ? kPolNtSc1Nt : kPolPlainSc1Nt;
    }
    plan->policy = nt;
    if (tuning && tuning->nontemporal) plan->piece_policy = tuning->nontemporal;
    plan->waves = waves;
    plan->swizzle = swizzle;
    plan->max_wgs = max_wgs;

    if (total > 0) {
        void *staging = nullptr;
        size_t staging_cap = 0;
        reap_uploads(device);
        hipError_t e = upload_cache().get(device, std::max<size_t>(total - upload_from, 256), &staging, &staging_cap);
        if (e != hipSuccess) {
            delete plan;
            return nixl_amd_fail(NIXL_AMD_ERR_HIP, std::string("hipHostMalloc(plan upload buffer): ") + hipGetErrorString(e));
        }
        // the pinned buffer mirrors the arena from upload_from on
        const auto host = [&](size_t arena_offset) { return static_cast<uint8_t *>(staging) + (arena_offset - upload_from); };
        if (expand) {
            std::memcpy(host(off_runs), uni.data(), uni.size() * sizeof(UniformRec));
            std::memcpy(host(off_first), first_chunk.data(), first_chunk.size() * sizeof(uint32_t));
        } else if (!uni.empty())
            std::memcpy(host(off_uni), uni.data(), uni.size() * sizeof(UniformRec));
        if (need_desc_arrays) {
            std::memcpy(host(off_src), vsrc.data(), nv * 8);
            std::memcpy(host(off_dst), vdst.data(), nv * 8);
            std::memcpy(host(off_prefix), vprefix.data(), (nv + 1) * 8);
            std::memcpy(host(off_span), span.data(), span.size() * sizeof(uint2));
            std::memcpy(host(off_mixed), mixed.data(), mixed.size() * sizeof(uint32_t));
        }
        if (!pieces.empty()) std::memcpy(host(off_pieces), pieces.data(), pieces.size() * sizeof(PieceRec));
        if (!items.empty()) std::memcpy(host(off_items), items.data(), items.size() * sizeof(GenericItem));
        e = arena_cache().get(device, total, &plan->arena, &plan->arena_cap);
        if (e != hipSuccess) {
            upload_cache().put(device, staging, staging_cap);
            delete plan;
            return nixl_amd_fail(NIXL_AMD_ERR_HIP, std::string("hipMalloc(plan arena): ") + hipGetErrorString(e));
        }
        // No wait here either: the event goes behind the copy, launches wait for it on their
        // stream, and the pinned buffer is recycled once the copy has completed.
        hipStream_t up = nullptr;
        e = upload_stream(device, &up);
        auto *arena = static_cast<uint8_t *>(plan->arena);
        if (e == hipSuccess && total > upload_from)
            e = hipMemcpyAsync(arena + upload_from, staging, total - upload_from, hipMemcpyHostToDevice, up);
        if (e == hipSuccess && expand) {
            const uint32_t wgs = static_cast<uint32_t>(std::min<uint64_t>((static_cast<uint64_t>(n_uniform_chunks) + 255) / 256, 1u << 20));
            hipLaunchKernelGGL(expand_runs_kernel, dim3(wgs), dim3(256), 0, up, reinterpret_cast<UniformRec *>(arena + off_uni),
                               reinterpret_cast<const UniformRec *>(arena + off_runs),
                               reinterpret_cast<const uint32_t *>(arena + off_first), static_cast<uint32_t>(uni.size()),
                               n_uniform_chunks, static_cast<uint32_t>(chunk_units * 16u));
            e = hipGetLastError();
        }
        if (e == hipSuccess) e = hipEventCreateWithFlags(&plan->uploaded, hipEventDisableTiming);
        if (e == hipSuccess) e = hipEventRecord(plan->uploaded, up);
        if (e != hipSuccess) {
            if (up) (void)hipStreamSynchronize(up); // a queued copy still reads the buffer given back below
            if (plan->uploaded) (void)hipEventDestroy(plan->uploaded);
            upload_cache().put(device, staging, staging_cap);
            arena_cache().put(device, plan->arena, plan->arena_cap);
            delete plan;
            return nixl_amd_fail(NIXL_AMD_ERR_HIP, std::string("hipMemcpy(plan arena): ") + hipGetErrorString(e));
        }
        recycle_after(device, up, staging, staging_cap);
        plan->arena_bytes = total;
        auto *base = static_cast<uint8_t *>(plan->arena);
        plan->uniform_recs = reinterpret_cast<const UniformRec *>(base + off_uni);
        plan->mixed_args.src = reinterpret_cast<const uint64_t *>(base + off_src);
        plan->mixed_args.dst = reinterpret_cast<const uint64_t *>(base + off_dst);
        plan->mixed_args.prefix = reinterpret_cast<const uint64_t *>(base + off_prefix);
        plan->mixed_args.span = reinterpret_cast<const uint2 *>(base + off_span);
        plan->mixed_args.chunks = reinterpret_cast<const uint32_t *>(base + off_mixed);
        plan->piece_recs = reinterpret_cast<const PieceRec *>(base + off_pieces);
        plan->generic_items = reinterpret_cast<const GenericItem *>(base + off_items);
    }
    plan->n_pieces = static_cast<uint32_t>(pieces.size());
    plan->n_uniform = n_uniform_chunks;
    plan->chunks_per_rec = chunks_per_rec;
    plan->mixed_args.total_units = units;
    plan->mixed_args.n_mixed = static_cast<uint32_t>(mixed.size());
    plan->n_generic = static_cast<uint32_t>(items.size());

    auto wgs_for = [&](uint32_t n_waves, uint32_t waves_per_wg, bool cap) {
        uint32_t w = (n_waves + waves_per_wg - 1) / waves_per_wg;
        if (cap && plan->max_wgs && w > plan->max_wgs) w = plan->max_wgs;
        if (cap && w > kMaxGrid) w = kMaxGrid; // those kernels loop over their work items
        return w;
    };
    plan->uniform_wgs = wgs_for(plan->n_uniform, static_cast<uint32_t>(waves), false);
    plan->mixed_wgs = wgs_for(plan->mixed_args.n_mixed, kMixedWaves, true);
    plan->generic_wgs = wgs_for(plan->n_generic, kMixedWaves, true);

    plan->info.payload_bytes = payload;
    plan->info.vec_descs = nv + n_piece_descs;
    plan->info.generic_descs = n_generic_descs;
    plan->info.plan_device_bytes = plan->arena_bytes;
    plan->info.vec_chunks = n_chunks;
    plan->info.uniform_chunks = plan->n_uniform;
    plan->info.mixed_chunks = plan->mixed_args.n_mixed;
    plan->info.generic_items = plan->n_generic;
    plan->info.piece_items = plan->n_pieces;
    plan->info.units_per_lane = static_cast<uint32_t>(upl);
    plan->info.uniform_workgroups = plan->uniform_wgs;
    *out = plan;
    return NIXL_AMD_OK;
}

int
nixl_amd_copy_block_len_fits(uint64_t len, const nixl_amd_copy_tuning_t *tuning) {
    Tuning t;
    if (parse_tuning(tuning, t, "block_len_fits")) return 0;
    return block_len_fits(len, t) ? 1 : 0;
}

int
nixl_amd_copy_records_begin(size_t max_records, nixl_amd_copy_records_t **out, nixl_amd_copy_record_t **records) {
    static_assert(sizeof(nixl_amd_copy_record_t) == sizeof(UniformRec));
    if (!out || !records) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "records_begin: null argument");
    *out = nullptr;
    *records = nullptr;
    if (max_records == 0 || max_records >= (1ull << 31))
        return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "records_begin: between 1 and 2^31-1 records");
    auto *r = new nixl_amd_copy_records();
    r->max_records = max_records;
    const hipError_t e = upload_cache().get(0, max_records * sizeof(UniformRec), &r->staging, &r->staging_cap);
    if (e != hipSuccess) {
        delete r;
        return nixl_amd_fail(NIXL_AMD_ERR_HIP, std::string("hipHostMalloc(plan upload buffer): ") + hipGetErrorString(e));
    }
    *records = static_cast<nixl_amd_copy_record_t *>(r->staging);
    *out = r;
    return NIXL_AMD_OK;
}

int
nixl_amd_copy_records_abandon(nixl_amd_copy_records_t *records) {
    if (!records) return NIXL_AMD_OK;
    upload_cache().put(0, records->staging, records->staging_cap);
    delete records;
    return NIXL_AMD_OK;
}

int
nixl_amd_copy_plan_create_from_records(nixl_amd_copy_records_t *records,
                                       size_t n,
                                       uint64_t len,
                                       int device,
                                       const nixl_amd_copy_tuning_t *tuning,
                                       const nixl_amd_copy_record_facts_t *facts,
                                       nixl_amd_copy_plan_t **out) {
    if (!records) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_create_from_records: records is null");
    // the buffer is taken over whatever happens below
    void *staging = records->staging;
    const size_t staging_cap = records->staging_cap, max_records = records->max_records;
    delete records;
    const auto give_back = [&](int code, const char *why) {
        upload_cache().put(0, staging, staging_cap);
        return nixl_amd_fail(code, why);
    };
    if (!out) return give_back(NIXL_AMD_ERR_INVALID, "plan_create_from_records: out is null");
    *out = nullptr;
    if (n == 0 || n > max_records) return give_back(NIXL_AMD_ERR_INVALID, "plan_create_from_records: record count outside the buffer");
    Tuning t;
    if (const int rc = parse_tuning(tuning, t, "plan_create_from_records")) {
        upload_cache().put(0, staging, staging_cap);
        return rc;
    }
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev <= 0) return give_back(NIXL_AMD_ERR_NO_DEVICE, "plan_create_from_records: no HIP device");
    if (device < 0 || device >= ndev) return give_back(NIXL_AMD_ERR_INVALID, "plan_create_from_records: bad device index");
    const DeviceScope on_device(device);
    if (on_device.status() != hipSuccess) return give_back(NIXL_AMD_ERR_HIP, "plan_create_from_records: hipSetDevice failed");
    reap_uploads(device);
    const int rc = build_block_plan(device, t, staging, staging_cap, n, len, n, facts, out);
    if (rc == kNotBlocks)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID,
                             "plan_create_from_records: blocks must be whole chunks of at least 8 KiB, start on 128-byte lines and not wrap");
    return rc;
}

int
nixl_amd_copy_plan_create_indexed_runs(const nixl_amd_copy_run_t *src_runs,
                                       size_t n_src_runs,
                                       const int32_t *src_index,
                                       const nixl_amd_copy_run_t *dst_runs,
                                       size_t n_dst_runs,
                                       const int32_t *dst_index,
                                       size_t n,
                                  uint64_t len,
                                  int device,
                                  const nixl_amd_copy_tuning_t *tuning,
                                  nixl_amd_copy_plan_t **out) {
    if (!out) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_create_indexed: out is null");
    *out = nullptr;
    if (!src_index || !dst_index || n == 0) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_create_indexed: no indices");
    Tuning t;
    if (const int rc = parse_tuning(tuning, t, "plan_create_indexed")) return rc;
    const int upl = t.upl, nt = t.nt, waves = t.waves, swizzle = t.swizzle, sort_scatter = t.sort_scatter;
    const uint64_t chunk_bytes = static_cast<uint64_t>(kWaveSize) * upl * 16u;
    if (!src_runs || !dst_runs || n_src_runs == 0 || n_dst_runs == 0 || n_src_runs > kMaxIndexRuns || n_dst_runs > kMaxIndexRuns)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_create_indexed: between 1 and 256 runs a side");
    bool src_all_dense = true, dst_all_dense = true;
    for (int side = 0; side < 2; ++side) {
        const nixl_amd_copy_run_t *runs = side ? dst_runs : src_runs;
        const size_t n_runs = side ? n_dst_runs : n_src_runs;
        for (size_t r = 0; r < n_runs; ++r) {
            if (runs[r].base == 0 || ((runs[r].base | runs[r].stride) & 127u) != 0 || len == 0 || len % chunk_bytes != 0)
                return nixl_amd_fail(NIXL_AMD_ERR_INVALID,
                                     "plan_create_indexed: blocks must be whole chunks and start on 128-byte lines");
            if (runs[r].first_index != (r ? runs[r - 1].first_index + runs[r - 1].count : 0))
                return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_create_indexed: runs must follow each other from index 0");
            (side ? dst_all_dense : src_all_dense) &= runs[r].stride == len;
        }
    }
    if (n >= (1ull << 31) || n * (len / chunk_bytes) >= (1ull << 32))
        return nixl_amd_fail(NIXL_AMD_ERR_TOO_LARGE, "plan_create_indexed: request too large for 32-bit chunk index");
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev <= 0)
        return nixl_amd_fail(NIXL_AMD_ERR_NO_DEVICE, "plan_create_indexed: no HIP device");
    if (device < 0 || device >= ndev) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_create_indexed: bad device index");
    const DeviceScope on_device(device);
    HIP_TRY(on_device.status());

    // Destination pattern (cache policy, record order) and source pattern from the index
    // vectors, while they are copied into the pinned upload buffer.
    const size_t index_bytes = n * sizeof(int32_t);
    void *staging = nullptr;
    size_t staging_cap = 0;
    const bool tables = n_src_runs > 1 || n_dst_runs > 1;
    const size_t table_at = (2 * index_bytes + 15) & ~size_t(15); // the run tables follow the index vectors
    const size_t table_bytes = tables ? (n_src_runs + n_dst_runs) * sizeof(nixl_amd_copy_run_t) : 0;
    const size_t upload_bytes = tables ? table_at + table_bytes : 2 * index_bytes;
    reap_uploads(device);
    hipError_t e = upload_cache().get(device, upload_bytes, &staging, &staging_cap);
    if (e != hipSuccess)
        return nixl_amd_fail(NIXL_AMD_ERR_HIP, std::string("hipHostMalloc(plan upload buffer): ") + hipGetErrorString(e));
    auto *up_src = static_cast<int32_t *>(staging), *up_dst = up_src + n;
    std::memcpy(up_src, src_index, index_bytes);
    std::memcpy(up_dst, dst_index, index_bytes);
    // How many destination steps are regular (one block on in dense lists, or the same step as
    // the one before) and how many source steps go one block on: differences taken modulo 2^32
    // and without a value carried from one iteration to the next, so that the loop vectorises.
    uint32_t regular = 0, src_follows = 0; // n < 2^31
    const uint32_t dst_dense = dst_all_dense ? 1u : 0u, src_dense = src_all_dense ? 1u : 0u;
    const auto *sv = reinterpret_cast<const uint32_t *>(src_index);
    const auto *dv = reinterpret_cast<const uint32_t *>(dst_index);
    if (n > 1) {
        regular += ((dv[1] - dv[0]) == 1u) & dst_dense;
        src_follows += ((sv[1] - sv[0]) == 1u) & src_dense;
    }
    for (size_t i = 2; i < n; ++i) {
        const uint32_t step = dv[i] - dv[i - 1], before = dv[i - 1] - dv[i - 2];
        regular += (static_cast<uint32_t>(step == 1u) & dst_dense) | static_cast<uint32_t>(step == before);
        src_follows += static_cast<uint32_t>((sv[i] - sv[i - 1]) == 1u) & src_dense;
    }
    if (tables) {
        auto *up_runs = reinterpret_cast<nixl_amd_copy_run_t *>(static_cast<uint8_t *>(staging) + table_at);
        std::memcpy(up_runs, src_runs, n_src_runs * sizeof(nixl_amd_copy_run_t));
        std::memcpy(up_runs + n_src_runs, dst_runs, n_dst_runs * sizeof(nixl_amd_copy_run_t));
    }
    const bool scattered = !(n == 1 || 2 * static_cast<uint64_t>(regular) >= n - 1);
    const bool sort = scattered && sort_scatter != 2 && 2 * static_cast<uint64_t>(src_follows) >= n - 1 && n >= kSortWindow;

    auto *plan = new nixl_amd_copy_plan();
    plan->device = device;
    plan->upl = upl;
    plan->waves = waves;
    plan->swizzle = swizzle;
    plan->policy = nt ? nt : ((!scattered || sort) ? kPolNtSc1Nt : kPolPlainSc1Nt);
    // one arena: the records, then the two index vectors (and run tables) the records are built from
    const size_t rec_bytes = (n * sizeof(UniformRec) + 255) & ~size_t(255);
    hipStream_t up = nullptr;
    e = arena_cache().get(device, rec_bytes + upload_bytes, &plan->arena, &plan->arena_cap);
    if (e == hipSuccess) e = upload_stream(device, &up);
    auto *recs = static_cast<UniformRec *>(plan->arena);
    auto *dev_index = reinterpret_cast<int32_t *>(static_cast<uint8_t *>(plan->arena) + rec_bytes);
    if (e == hipSuccess) e = hipMemcpyAsync(dev_index, staging, upload_bytes, hipMemcpyHostToDevice, up);
    if (e == hipSuccess) {
        const dim3 grid(static_cast<uint32_t>((n + 255) / 256));
        if (tables) {
            const auto *dev_runs =
                reinterpret_cast<const nixl_amd_copy_run_t *>(reinterpret_cast<const uint8_t *>(dev_index) + table_at);
            hipLaunchKernelGGL(index_records_runs_kernel, grid, dim3(256), 0, up, recs, dev_index, dev_index + n,
                               static_cast<uint32_t>(n), dev_runs, static_cast<uint32_t>(n_src_runs), dev_runs + n_src_runs,
                               static_cast<uint32_t>(n_dst_runs));
        } else {
            hipLaunchKernelGGL(index_records_kernel, grid, dim3(256), 0, up, recs, dev_index, dev_index + n,
                               static_cast<uint32_t>(n), src_runs[0].base, src_runs[0].stride, dst_runs[0].base,
                               dst_runs[0].stride);
        }
        e = hipGetLastError();
    }
    if (e == hipSuccess && sort) {
        hipLaunchKernelGGL(sort_records_kernel, dim3(static_cast<uint32_t>((n + kSortWindow - 1) / kSortWindow)),
                           dim3(kSortWindow / 2), 0, up, recs, static_cast<uint32_t>(n));
        e = hipGetLastError();
    }
    // No wait here: the event goes behind the kernels, launches wait for it on their stream.
    if (e == hipSuccess) e = hipEventCreateWithFlags(&plan->uploaded, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventRecord(plan->uploaded, up);
    if (e != hipSuccess) {
        if (up) (void)hipStreamSynchronize(up); // whatever was queued reads the buffers given back below
        if (plan->uploaded) (void)hipEventDestroy(plan->uploaded);
        upload_cache().put(device, staging, staging_cap);
        if (plan->arena) arena_cache().put(device, plan->arena, plan->arena_cap);
        delete plan;
        return nixl_amd_fail(NIXL_AMD_ERR_HIP, std::string("plan upload: ") + hipGetErrorString(e));
    }
    recycle_after(device, up, staging, staging_cap);
    plan->arena_bytes = rec_bytes + upload_bytes;
    plan->uniform_recs = recs;
    plan->chunks_per_rec = static_cast<uint32_t>(len / chunk_bytes);
    plan->n_uniform = static_cast<uint32_t>(n * plan->chunks_per_rec);
    plan->uniform_wgs = (plan->n_uniform + static_cast<uint32_t>(waves) - 1) / static_cast<uint32_t>(waves);
    plan->info.payload_bytes = n * len;
    plan->info.vec_descs = n;
    plan->info.plan_device_bytes = plan->arena_bytes;
    plan->info.vec_chunks = plan->n_uniform;
    plan->info.uniform_chunks = plan->n_uniform;
    plan->info.units_per_lane = static_cast<uint32_t>(upl);
    plan->info.uniform_workgroups = plan->uniform_wgs;
    *out = plan;
    return NIXL_AMD_OK;
}

int
nixl_amd_copy_plan_create_indexed(uint64_t src_base,
                                  uint64_t src_stride,
                                  const int32_t *src_index,
                                  uint64_t dst_base,
                                  uint64_t dst_stride,
                                  const int32_t *dst_index,
                                  size_t n,
                                  uint64_t len,
                                  int device,
                                  const nixl_amd_copy_tuning_t *tuning,
                                  nixl_amd_copy_plan_t **out) {
    const nixl_amd_copy_run_t src{src_base, src_stride, 0, 0}, dst{dst_base, dst_stride, 0, 0};
    return nixl_amd_copy_plan_create_indexed_runs(&src, 1, src_index, &dst, 1, dst_index, n, len, device, tuning, out);
}

int
nixl_amd_copy_plan_launch(nixl_amd_copy_plan_t *plan, void *stream) {
    if (!plan) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_launch: plan is null");
    const DeviceScope on_device(plan->device);
    HIP_TRY(on_device.status());
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (plan->uploaded) {
        hipError_t e = settle_upload(plan, false);
        if (e == hipErrorNotReady) {
            // A stream under graph capture must not be made to depend on work outside the
            // graph: the host waits instead, and the graph holds the launch alone.
            hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
            if (s && hipStreamIsCapturing(s, &capture) != hipSuccess) (void)hipGetLastError();
            e = capture == hipStreamCaptureStatusNone ? hipStreamWaitEvent(s, plan->uploaded, 0) : hipErrorNotReady;
            if (e != hipSuccess) {
                (void)hipGetLastError();
                e = settle_upload(plan, true);
            }
        }
        HIP_TRY(e);
    }
    if (plan->uniform_wgs) {
        // One launch per kMaxGrid workgroups.  With the die swizzle each launch's grid is
        // rounded up to a multiple of 8 so that every die owns an equally long slice; surplus
        // workgroups exit at once.
        const uint32_t waves = static_cast<uint32_t>(plan->waves);
        for (uint64_t wg64 = 0; wg64 < plan->uniform_wgs; wg64 += kMaxGrid) {
            const uint32_t wg0 = static_cast<uint32_t>(wg64);
            UniformLaunch u{};
            u.recs = plan->uniform_recs;
            u.first_chunk = wg0 * waves;
            u.n_chunks = plan->n_uniform - u.first_chunk;
            u.n_wgs = std::min(kMaxGrid, plan->uniform_wgs - wg0);
            u.chunks_per_rec = plan->chunks_per_rec;
            u.swizzle = plan->swizzle;
            u.grid = dim3(plan->swizzle ? ((u.n_wgs + kNumXcd - 1) / kNumXcd) * kNumXcd : u.n_wgs);
            u.stream = s;
            with_policy(plan->policy, [&]<int POL>() { launch_uniform_upl<POL>(plan->upl, plan->waves, u); });
            HIP_TRY(hipGetLastError());
        }
    }
    if (plan->n_pieces) {
        const uint32_t w = static_cast<uint32_t>(plan->waves > 4 ? 4 : plan->waves);
        const uint32_t per_launch = kMaxGrid * w;
        for (uint32_t p0 = 0; p0 < plan->n_pieces; p0 += per_launch) {
            const uint32_t n = std::min(per_launch, plan->n_pieces - p0);
            with_policy(plan->piece_policy,
                        [&]<int POL>() { launch_pieces<POL>(w, (n + w - 1) / w, s, plan->piece_recs + p0, n); });
            HIP_TRY(hipGetLastError());
        }
    }
    if (plan->mixed_wgs) {
        with_policy(plan->policy, [&]<int POL>() { launch_mixed_upl<POL>(plan->upl, dim3(plan->mixed_wgs), s, plan->mixed_args); });
        HIP_TRY(hipGetLastError());
    }
    if (plan->generic_wgs) {
        hipLaunchKernelGGL(copy_generic_kernel, dim3(plan->generic_wgs), dim3(kMixedThreads), 0, s,
                           plan->generic_items, plan->n_generic);
        HIP_TRY(hipGetLastError());
    }
    // What nixl_amd_copy_plan_destroy looks at.  A stream under graph capture gets no event: the
    // graph's owner keeps the plan alive for as long as the graph may be replayed.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (s && hipStreamIsCapturing(s, &capture) != hipSuccess) (void)hipGetLastError();
    if (capture == hipStreamCaptureStatusNone) {
        if (!plan->launched) HIP_TRY(hipEventCreateWithFlags(&plan->launched, hipEventDisableTiming));
        HIP_TRY(hipEventRecord(plan->launched, s));
        plan->launched_valid = true;
    }
    return NIXL_AMD_OK;
}

int
nixl_amd_copy_plan_status(nixl_amd_copy_plan_t *plan, int wait) {
    if (!plan) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_status: plan is null");
    if (!plan->launched_valid) return NIXL_AMD_OK;
    const DeviceScope on_device(plan->device);
    const hipError_t state = wait ? hipEventSynchronize(plan->launched) : hipEventQuery(plan->launched);
    if (state == hipSuccess) return NIXL_AMD_OK;
    if (state == hipErrorNotReady) {
        (void)hipGetLastError();
        return NIXL_AMD_ERR_BUSY; // polled in a loop: no message is made for it
    }
    return nixl_amd_fail(NIXL_AMD_ERR_HIP, std::string("plan_status: ") + hipGetErrorString(state));
}

int
nixl_amd_copy_plan_destroy(nixl_amd_copy_plan_t *plan) {
    if (!plan) return NIXL_AMD_OK;
    const DeviceScope on_device(plan->device);
    if (plan->launched_valid) {
        // The arena goes back to a pool that the next plan's upload writes into: not while a
        // launch of this plan may still read it.  The plan stays as it is; destroy it later.
        const hipError_t state = hipEventQuery(plan->launched);
        if (state == hipErrorNotReady) {
            (void)hipGetLastError();
            return nixl_amd_fail(NIXL_AMD_ERR_BUSY, "plan_destroy: a launch of this plan has not completed");
        }
    }
    (void)settle_upload(plan, true); // the arena and the upload buffer go back only when nothing writes or reads them
    if (plan->launched) (void)hipEventDestroy(plan->launched);
    if (plan->ev0) (void)hipEventDestroy(plan->ev0);
    if (plan->ev1) (void)hipEventDestroy(plan->ev1);
    if (plan->arena) arena_cache().put(plan->device, plan->arena, plan->arena_cap);
    delete plan;
    return NIXL_AMD_OK;
}

int
nixl_amd_copy_plan_query(const nixl_amd_copy_plan_t *plan, nixl_amd_copy_plan_info_t *info) {
    if (!plan || !info) return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_query: null argument");
    *info = plan->info;
    return NIXL_AMD_OK;
}

int
nixl_amd_copy_plan_time(nixl_amd_copy_plan_t *plan, void *stream, int iters, float *ms_per_launch) {
    if (!plan || !ms_per_launch || iters <= 0)
        return nixl_amd_fail(NIXL_AMD_ERR_INVALID, "plan_time: bad argument");
    const DeviceScope on_device(plan->device);
    HIP_TRY(on_device.status());
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (!plan->ev0) HIP_TRY(hipEventCreate(&plan->ev0));
    if (!plan->ev1) HIP_TRY(hipEventCreate(&plan->ev1));
    HIP_TRY(hipEventRecord(plan->ev0, s));
    for (int i = 0; i < iters; ++i) {
        int rc = nixl_amd_copy_plan_launch(plan, stream);
        if (rc) return rc;
    }
    HIP_TRY(hipEventRecord(plan->ev1, s));
    HIP_TRY(hipEventSynchronize(plan->ev1));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, plan->ev0, plan->ev1));
    *ms_per_launch = ms / static_cast<float>(iters);
    return NIXL_AMD_OK;
}

} // extern "C"
