/*
 * C ABI of the descriptor-copy kernel layer (libnixl_amd_kernels.so).
 *
 * This is the lowest drop-in level of the HIP backend: a NIXL transfer request, once the
 * agent has resolved it to two equally long lists of (address, length) spans, becomes ONE
 * device-resident copy plan and ONE kernel launch per post.  The reference has no such
 * layer: its VRAM->VRAM path issues one UCX put/get per descriptor from a host loop
 * (src/plugins/ucx/ucx_backend.cpp:1216-1244 -> ucp_put_nbx / ucp_get_nbx,
 * src/plugins/ucx/ucx_utils.cpp:288,313) and then flushes the endpoint (:1246-1262).  The
 * result that must match is that loop's: for every descriptor i, in list order,
 * memcpy(dst_i, src_i, len_i).
 *
 * All handles are plain pointers; `stream` is a hipStream_t passed as void* (NULL = the
 * default stream).  Every function returns 0 on success or a negative nixl_amd_status
 * value; nixl_amd_last_error() gives the text of the last failure on the calling thread.
 * No function falls back to a host copy: without a usable HIP device they fail.
 */
#ifndef NIXL_AMD_HIP_H
#define NIXL_AMD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum nixl_amd_status {
    NIXL_AMD_OK = 0,
    NIXL_AMD_ERR_INVALID = -1, /* bad argument (null pointer, zero count, bad variant) */
    NIXL_AMD_ERR_HIP = -2, /* a HIP runtime call failed; see nixl_amd_last_error() */
    NIXL_AMD_ERR_NO_DEVICE = -3, /* no gfx950-class device visible */
    NIXL_AMD_ERR_BUSY = -4, /* plan destroyed while one of its launches has not completed */
    NIXL_AMD_ERR_TOO_LARGE = -5 /* request exceeds a documented fixed limit */
};

/* One span to copy: `len` bytes from device address `src` to device address `dst`.
 * This is one (local, remote) pair of nixlMetaDesc entries
 * (src/api/cpp/backend/backend_aux.h:92-105) with the direction already applied:
 * NIXL_WRITE copies local->remote, NIXL_READ remote->local
 * (src/plugins/ucx/ucx_backend.cpp:1227-1229). */
typedef struct nixl_amd_copy_desc {
    uint64_t src;
    uint64_t dst;
    uint64_t len;
} nixl_amd_copy_desc_t;

/* Launch-shape knobs.  Zero in any field selects the built-in default. */
typedef struct nixl_amd_copy_tuning {
    int units_per_lane; /* 16-byte units one lane moves per chunk: 1, 2, 4, 8 or 16 */
    int nontemporal; /* cache policy: 1 = non-temporal loads and stores, 2 = plain, 3 = plain loads and
                      * streaming device-scope stores, 4 = non-temporal loads and streaming
                      * device-scope stores; 0 = 4 if the destinations of consecutive
                      * descriptors adjoin or advance by a constant step, else 3 */
    int max_workgroups; /* grid cap of the mixed and byte-path kernels; waves loop beyond it */
    int waves_per_workgroup; /* uniform-chunk kernel: 1, 2, 4, 8 or 16 */
    int xcd_swizzle; /* 1 = each accelerator die walks a contiguous slice of the chunk list, 2 = off */
    int sort_scatter; /* a plan that scatters consecutive memory over irregular destinations has its records put
                       * into ascending destination order inside windows of 1024 (on the device): 1 = on, 2 = off */
} nixl_amd_copy_tuning_t;

typedef struct nixl_amd_copy_plan nixl_amd_copy_plan_t;

/* Text of the most recent error on this thread ("" if none). */
const char *
nixl_amd_last_error(void);

/* Number of HIP devices, or a negative status. */
int
nixl_amd_device_count(void);

/* Lower `n` host-side descriptors into a device-resident plan on `device`.
 * Replaces the per-request set-up of nixlUcxEngine::prepXfer
 * (src/plugins/ucx/ucx_backend.cpp:1061-1084), which defers all work to post time.
 * Zero-length descriptors are dropped.  Descriptors whose src, dst and len are all
 * multiples of 16 take the 128-bit streaming path; all others take a byte-exact path.
 * The descriptor array may be freed as soon as this returns. */
int
nixl_amd_copy_plan_create(const nixl_amd_copy_desc_t *descs,
                          size_t n,
                          int device,
                          const nixl_amd_copy_tuning_t *tuning,
                          nixl_amd_copy_plan_t **out);

/* A plan for `n` equal blocks given by index: block i is copied from
 * src_base + src_index[i] * src_stride to dst_base + dst_index[i] * dst_stride, `len` bytes.
 * This is what nixlAgent::makeXferReq asks for when both prepared lists are one dense or
 * strided run each (a paged KV pool and a staging buffer; src/core/nixl_agent.cpp:799-857
 * expands such indices into descriptors on the host, one by one): only the two index vectors
 * go to the device, where a kernel writes the records.  Bases and strides must be multiples
 * of 128 and `len` a whole number of chunks (1 KiB at the default tuning); the caller checks
 * the indices against the lists they index.  The index arrays may be freed on return.  The
 * call does not wait for the device: the records are written by kernels queued on a stream of
 * the library's, and nixl_amd_copy_plan_launch makes its stream wait for them. */
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
                                  nixl_amd_copy_plan_t **out);

/* One run of a prepared list: blocks first_index .. first_index + count - 1 of the list lie
 * at base, base + stride, ...  (the stride runs a prepared descriptor list compresses into,
 * src/api/cpp/backend/backend_aux.h:140-208). */
typedef struct nixl_amd_copy_run {
    uint64_t base;
    uint64_t stride;
    uint64_t first_index;
    uint64_t count;
} nixl_amd_copy_run_t;

/* The same for lists of several runs (a pool registered as several regions): index i of a
 * list names block i - first_index of the run that holds it.  Between 1 and 256 runs a side,
 * in index order from 0 without gaps (runs[r + 1].first_index == runs[r].first_index +
 * runs[r].count; the last run's count is not looked at); every base and stride a multiple
 * of 128.  The run tables travel to the device with the index vectors and are searched
 * there. */
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
                                       nixl_amd_copy_plan_t **out);

/* A plan of equal blocks from records the CALLER writes: what a backend's prepXfer does when
 * it checks the two nixl_meta_dlist_t of a request (src/api/cpp/backend/backend_engine.h:135-141)
 * in one pass and every descriptor pair is the same length.  nixl_amd_copy_records_begin hands
 * out room for `max_records` {src, dst} pairs in a pinned upload buffer of the library's
 * (recycled between requests); the caller fills records[0 .. n) and passes the handle to
 * nixl_amd_copy_plan_create_from_records, which checks the records (whole chunks of at least
 * 8 KiB, every address on a 128-byte line, none null, no range that wraps:
 * NIXL_AMD_ERR_INVALID otherwise), reads the destination and source patterns from them and
 * queues their copy to the device without waiting for it, or to nixl_amd_copy_records_abandon.
 * Either call consumes the handle, whatever it returns.  No reference counterpart: the
 * reference's backends keep the descriptor lists and walk them at post time
 * (src/plugins/ucx/ucx_backend.cpp:1216-1244). */
typedef struct nixl_amd_copy_record {
    uint64_t src;
    uint64_t dst;
} nixl_amd_copy_record_t;

typedef struct nixl_amd_copy_records nixl_amd_copy_records_t;

/* What a caller that looked at every record while writing it already knows, so that the
 * library does not read them all again: the OR of every src and dst address (its low seven
 * bits must be zero), of `steps` pairs of consecutive records (all of them, or a sample:
 * the counts only decide cache policy and record order by majority) how many advance the
 * destination regularly (by one block, or by the same amount as the pair before) and how many
 * advance the source by exactly one block.  Passing it also states that every record lies in
 * memory the device can address (not null, not wrapping): a backend knows that from its
 * registrations.  NULL makes the library find all of this out itself. */
typedef struct nixl_amd_copy_record_facts {
    uint64_t address_bits;
    uint64_t regular_dst_steps;
    uint64_t following_src_steps;
    uint64_t steps;
} nixl_amd_copy_record_facts_t;

int
nixl_amd_copy_records_begin(size_t max_records, nixl_amd_copy_records_t **out, nixl_amd_copy_record_t **records);

int
nixl_amd_copy_plan_create_from_records(nixl_amd_copy_records_t *records,
                                       size_t n,
                                       uint64_t len,
                                       int device,
                                       const nixl_amd_copy_tuning_t *tuning,
                                       const nixl_amd_copy_record_facts_t *facts,
                                       nixl_amd_copy_plan_t **out);

int
nixl_amd_copy_records_abandon(nixl_amd_copy_records_t *records);

/* 1 if equal blocks of `len` bytes can make such a plan under `tuning` (a whole number of
 * chunks, at least 8 KiB), else 0: lets a caller decide before it writes any record. */
int
nixl_amd_copy_block_len_fits(uint64_t len, const nixl_amd_copy_tuning_t *tuning);

/* Enqueue the whole plan on `stream`: the per-post work of
 * nixlUcxEngine::postXfer -> sendXferRange (src/plugins/ucx/ucx_backend.cpp:1183-1310).
 * Re-launching re-reads the current source bytes; nothing is cached at plan creation
 * (repost semantics of test/unit/plugins/posix/nixl_posix_test.cpp:714-770). */
int
nixl_amd_copy_plan_launch(nixl_amd_copy_plan_t *plan, void *stream);

/* Whether the plan's launches have completed: NIXL_AMD_OK when all have (or none was made),
 * NIXL_AMD_ERR_BUSY while one still runs (no error text is recorded for that answer: the call
 * is made to be polled), another negative status if a launch failed.  With `wait` non-zero the
 * call blocks until the answer is not BUSY.  This is what nixlBackendEngine::checkXfer
 * (src/api/cpp/backend/backend_engine.h:153) asks of a posted request.  Launches recorded
 * into a HIP graph are not tracked.  The answer follows the stream of the LAST launch: a
 * caller that launches one plan on several streams orders those streams itself.  Launch,
 * status and destroy of one plan are not to be called from several threads at once. */
int
nixl_amd_copy_plan_status(nixl_amd_copy_plan_t *plan, int wait);

/* Free the plan's device arrays.  While a launch of the plan has not completed the call
 * returns NIXL_AMD_ERR_BUSY and leaves the plan as it is (its arrays would go back to a pool
 * that the next plan's upload writes into): wait for the launch, then destroy again.  Launches
 * recorded into a HIP graph are not tracked: their owner keeps the plan for as long as the
 * graph may be replayed. */
int
nixl_amd_copy_plan_destroy(nixl_amd_copy_plan_t *plan);

/* Plan facts: total payload bytes, descriptors on the 128-bit paths, descriptors on the
 * byte path, device bytes held by the plan's own arrays, and how the 128-bit work was cut:
 * chunks of the packed stream lying inside one descriptor (uniform) versus chunks crossing
 * descriptor boundaries (mixed), and pieces (one wavefront each) of the descriptors that are
 * short or do not start on a 128-byte line. */
typedef struct nixl_amd_copy_plan_info {
    uint64_t payload_bytes;
    uint64_t vec_descs;
    uint64_t generic_descs;
    uint64_t plan_device_bytes;
    uint32_t vec_chunks;
    uint32_t uniform_chunks;
    uint32_t mixed_chunks;
    uint32_t generic_items;
    uint32_t units_per_lane;
    uint32_t uniform_workgroups;
    uint32_t piece_items;
} nixl_amd_copy_plan_info_t;

int
nixl_amd_copy_plan_query(const nixl_amd_copy_plan_t *plan, nixl_amd_copy_plan_info_t *info);

/* Convenience: launch the plan `iters` times back to back on `stream`, bracketed by HIP
 * events recorded on that same stream, wait, and return the mean milliseconds per launch.
 * Used by benchmarks to time the kernel itself. */
int
nixl_amd_copy_plan_time(nixl_amd_copy_plan_t *plan, void *stream, int iters, float *ms_per_launch);

#ifdef __cplusplus
}
#endif
#endif /* NIXL_AMD_HIP_H */
