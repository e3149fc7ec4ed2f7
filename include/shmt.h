/*
 * shmt.h — C ABI of libshmt.so: the GPU-cache hot path of ShmTensor
 * (static hashmap, cached feature fetch/set, cached neighbour sampling,
 * relabel, scan) as hand-written HIP for gfx950 (MI355X).
 *
 * Conventions
 *  - Every pointer is a raw address the GPU can dereference: device memory,
 *    or host memory that is pinned and device-mapped (see shmt_host_devptr).
 *    No torch types cross this boundary; callers allocate every buffer,
 *    including scratch (the library itself allocates no device memory; it
 *    keeps 256 bytes of pinned host memory for reading small results back), and
 *    pass element SIZES in bytes (4 or 8 for integer
 *    ids; any size for feature rows, which are copied bit for bit).
 *  - `stream` is a hipStream_t passed as void* (NULL = the null stream).
 *    All work is enqueued on it; no entry point synchronises unless it says so.
 *  - Return value: 0 on success, a negative SHMT_E* code on failure, with a
 *    human readable message available from shmt_last_error() (thread local).
 *    The library never calls exit()/abort() (the reference does on any CUDA
 *    error: include/common.h:15-27).
 *  - Zero-length inputs are valid and are no-ops (the reference launches a
 *    zero-size grid and exits: src/cache_feature_fetch.cu:77-83).
 *
 * Each entry point cites the reference interface (file:line under the
 * ShmTensor source tree) that it replaces.
 */
#ifndef SHMT_H_
#define SHMT_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SHMT_OK 0
#define SHMT_EINVAL (-1)  /* bad argument (null pointer, size, dtype width) */
#define SHMT_EHIP (-2)    /* a HIP runtime call failed                       */
#define SHMT_ENOTPINNED (-3) /* host pointer is not device-accessible        */
#define SHMT_ENOMEM (-4)  /* caller-provided buffer too small                */

#define SHMT_ABI_VERSION 2

/* Library identification / error channel (no counterpart in the reference,
 * whose errors are c10 exceptions or exit(): include/common.h:10-27). */
int shmt_abi_version(void);
const char *shmt_last_error(void);

/* ------------------------------------------------------------------ */
/* Host memory: PinMemory / UnpinMemory, src/cache_feature_fetch.cu:6-13
 * (cudaHostRegister(ptr, nbytes, cudaHostRegisterPortable) /
 * cudaHostUnregister), and the registration done by
 * include/shm_memory.h:19-21,35-37 and src/mmap_tensor.cc:42-45.          */

/* Page-lock and device-map an existing host range in place. */
int shmt_host_register(void *host_ptr, int64_t nbytes);
int shmt_host_unregister(void *host_ptr);
/* Translate a pointer a kernel is about to dereference. Device pointers
 * pass through unchanged; pinned host pointers (registered here, or
 * allocated pinned by the caller) yield their device-side alias, interior
 * pointers included; ordinary pageable host memory fails with
 * SHMT_ENOTPINNED instead of faulting inside a kernel.                     */
int shmt_host_devptr(const void *ptr, void **dev_ptr_out);

/* ------------------------------------------------------------------ */
/* Static hashmap: pycuco::CUCOHashmapWrapper, src/cuco_hashmap.cu:10-41,
 * include/cuco_hashmap.cuh:49-93 (cuco::static_map, linear probing, empty
 * key -1 / empty value -1), pybind class CUCOStaticHashmap
 * src/pybind.cc:60-64.                                                     */
typedef struct shmt_hashmap shmt_hashmap_t;

/* capacity() as the reference reports it: (int64)ceil(n / load_factor),
 * include/cuco_hashmap.cuh:62,75.                                          */
int64_t shmt_hashmap_capacity(int64_t n, double load_factor);
/* Bytes of device memory the table needs (what memory_usage() returns;
 * include/cuco_hashmap.cuh:25,76). key_bytes, val_bytes in {4, 8}.          */
int64_t shmt_hashmap_table_bytes(int64_t n, double load_factor, int key_bytes,
                                 int val_bytes);
/* Build (constructor, include/cuco_hashmap.cuh:57-77): fills `table_mem`
 * (device, >= shmt_hashmap_table_bytes, 128-byte aligned) with sentinels
 * and inserts keys[i] -> vals[i] for i < n. Keys equal to -1 are not
 * representable (sentinel). The table memory stays owned by the caller and
 * must outlive the handle. Asynchronous on `stream`.                       */
int shmt_hashmap_create(shmt_hashmap_t **out, const void *keys,
                        const void *vals, int64_t n, int key_bytes,
                        int val_bytes, double load_factor, void *table_mem,
                        int64_t table_bytes, void *stream);
/* Build with a layout chosen from the keys. Node ids are small dense
 * integers, so beside the general bucket table three flat forms exist:
 *   SHMT_MAP_DIRECT  keys lie in [lo, lo + span) and an int32 table
 *                    value[key - lo] is at most twice as large as the bucket
 *                    table would be: one 4-byte load per lookup;
 *   SHMT_MAP_RANGE   the keys are exactly lo .. lo + span - 1 and every value
 *                    is key + delta (the cache holds an id range, as in
 *                    re-numbered graphs): lookups are arithmetic, no table;
 *   SHMT_MAP_RANK    the pairs are given in ascending key order with values
 *                    v0, v0 + 1, ... (a cache whose rows are kept in id
 *                    order): a bitmap with running counts, 16 bytes per 96
 *                    ids of [lo, lo + span), value = rank of the key + delta;
 *                    one 16-byte load per lookup from a table that stays in
 *                    the caches (span / 6 bytes);
 * and the bucket table uses 8-byte slots whenever all keys and values fit 32
 * bits, whatever their dtype. Every form answers exactly like the general
 * table (same contract as the constructor above: include/cuco_hashmap.cuh:
 * 57-87). shmt_hashmap_plan looks at the keys and values (one sweep, plus a
 * repeat check for range candidates), SYNCHRONISES the stream once (twice
 * for a range candidate, whose repeat check is a second read-back) and fills
 * `layout`, including the table_bytes the caller has to provide;
 * shmt_hashmap_create_planned then builds that layout (asynchronous). The
 * layout must come from shmt_hashmap_plan on the same, unchanged keys and
 * values: the build trusts it (a rank layout is only re-checked for
 * n < 2^32, the width of its running counts).
 * `scratch` is device memory of shmt_hashmap_plan_scratch_bytes(n) bytes,
 * 16-byte aligned, free again when plan returns.                            */
#define SHMT_MAP_BUCKETS 0
#define SHMT_MAP_DIRECT 1
#define SHMT_MAP_RANGE 2
#define SHMT_MAP_RANK 3
typedef struct shmt_hashmap_layout {
  int kind;            /* SHMT_MAP_*                                        */
  int slot_bytes;      /* buckets: 16 or 8; direct: 4; range: 0; rank: 16   */
  int64_t lo, span;    /* flat forms: id range [lo, lo + span)              */
  int64_t delta;       /* range: value = key + delta; rank: rank + delta    */
  int64_t table_bytes; /* device memory the build needs (128-byte aligned)  */
} shmt_hashmap_layout;
int64_t shmt_hashmap_plan_scratch_bytes(int64_t n);
int shmt_hashmap_plan(const void *keys, const void *vals, int64_t n,
                      int key_bytes, int val_bytes, double load_factor,
                      void *scratch, int64_t scratch_bytes,
                      shmt_hashmap_layout *layout, void *stream);
int shmt_hashmap_create_planned(shmt_hashmap_t **out,
                                const shmt_hashmap_layout *layout,
                                const void *keys, const void *vals, int64_t n,
                                int key_bytes, int val_bytes,
                                double load_factor, void *table_mem,
                                int64_t table_bytes, void *stream);
/* SHMT_MAP_* of a built map, and the table bytes it actually uses.         */
int shmt_hashmap_kind(const shmt_hashmap_t *map);
int64_t shmt_hashmap_used_bytes(const shmt_hashmap_t *map);

/* Bulk lookup (query, src/cuco_hashmap.cu:24-34 + include/cuco_hashmap.cuh:
 * 81-87): requests of width req_bytes in {4,8} are first converted to the
 * key width (two's-complement narrowing / sign extension, as
 * requests.to(key_type_)), out[i] (width = val_bytes) = value or -1.        */
int shmt_hashmap_query(const shmt_hashmap_t *map, const void *requests,
                       int req_bytes, int64_t n, void *out, void *stream);
int shmt_hashmap_key_bytes(const shmt_hashmap_t *map);
int shmt_hashmap_val_bytes(const shmt_hashmap_t *map);
int64_t shmt_hashmap_size(const shmt_hashmap_t *map);
void shmt_hashmap_destroy(shmt_hashmap_t *map);

/* ------------------------------------------------------------------ */
/* Feature fetch: UVATensorFetch src/cache_feature_fetch.cu:47-87,
 * CacheTensorFetch :131-185, CacheTensorFetchWithMask :226-272.
 *   out[i,:] = slot_i >= 0 ? cache_data[slot_i,:] : miss_data[indices[i],:]
 * with slot_i = map.find(indices[i]) (map != NULL), mask[i] (mask != NULL)
 * or -1 (both NULL: the all-miss "uva" form; cache_data may be NULL).
 * Rows are `row_bytes` long and contiguous; indices are idx_bytes in {4,8}
 * wide; mask entries mask_bytes in {4,8} wide. `miss_data` is normally the
 * device alias of pinned host memory, but any device-addressable table
 * works. out has Q rows.                                                   */
int shmt_fetch(const void *miss_data, const void *cache_data,
               const void *indices, int idx_bytes, const shmt_hashmap_t *map,
               const void *mask, int mask_bytes, void *out, int64_t Q,
               int64_t row_bytes, void *stream);

/* shmt_fetch for a number of rows that only the GPU knows yet: moves the
 * first min(max_rows, *count) rows, where `count` is an int64 in device
 * memory written by earlier work of the stream (count_out of shmt_relabel*
 * / shmt_sample_hop, with unique_out as `indices`). `indices` (and `mask`)
 * hold at least that many entries, `out` has room for max_rows rows; rows
 * past the count are left untouched. If count_seen is not NULL (pinned host
 * memory) the kernel copies *count there as it starts, so the host learns
 * the count while the rows are still moving. With this the last relabel of
 * a mini-batch and the fetch of its input features run back to back without
 * a host wait between them; the reference reads the count on the host
 * (src/tensor_relabel.cu:173) before the caller can fetch
 * (src/cache_feature_fetch.cu:131-185).                                    */
int shmt_fetch_counted(const void *miss_data, const void *cache_data,
                       const void *indices, int idx_bytes,
                       const shmt_hashmap_t *map, const void *mask,
                       int mask_bytes, void *out, int64_t max_rows,
                       const int64_t *count, int64_t *count_seen,
                       int64_t row_bytes, void *stream);

/* A cached fetch in two launches, for callers that overlap fetches with
 * other GPU work (the next mini-batch's sampling). CacheTensorFetch
 * (src/cache_feature_fetch.cu:131-185) moves hits and misses in one kernel;
 * when the id-addressed table lives in pinned host memory the misses are
 * host-link reads, and a kernel that spans the whole GPU while it waits for
 * them keeps every other stream's kernels out and fills the link's queue.
 *   shmt_fetch_cached_part  moves the rows that hit (out[i,:] =
 *       cache_data[slot_i,:]) over the first min(max_rows, *count) entries
 *       (count may be NULL: exactly max_rows) and marks the rows that missed
 *       in miss_bits: bit (i & 31) of 32-bit word i / 32, room for
 *       ceil(max_rows / 32) words. Every word that covers an existing row is
 *       written, so the buffer needs no clearing.
 *   shmt_fetch_missed_part  moves out[i,:] = miss_data[indices[i],:] for the
 *       marked rows (same max_rows and count), on at most max_blocks
 *       workgroups (0: a default that saturates the host link and no more),
 *       and may run on another stream once the first call's work is done.
 * Together they give exactly what shmt_fetch[_counted] gives. Rows and
 * tables must allow 16-byte accesses (row_bytes and all base addresses
 * multiples of 16) and max_rows must be below 2^32; otherwise SHMT_EINVAL,
 * and the caller uses shmt_fetch.                                          */
int shmt_fetch_cached_part(const void *miss_data, const void *cache_data,
                           const void *indices, int idx_bytes,
                           const shmt_hashmap_t *map, const void *mask,
                           int mask_bytes, void *out, int64_t max_rows,
                           const int64_t *count, int64_t row_bytes,
                           uint32_t *miss_bits, void *stream);
int shmt_fetch_missed_part(const void *miss_data, const void *indices,
                           int idx_bytes, const uint32_t *miss_bits, void *out,
                           int64_t max_rows, const int64_t *count,
                           int64_t row_bytes, int max_blocks, void *stream);

/* Feature set: UVATensorSet src/cache_feature_set.cu:39-75, CacheTensorSet
 * :118-165, CacheTensorSetWithMask :209-248. Mirror of shmt_fetch:
 *   (slot_i >= 0 ? cache_data[slot_i,:] : miss_data[indices[i],:]) = update[i,:]
 * A hit does not write the miss-side row. Duplicate indices race, as in
 * the reference.                                                           */
int shmt_set(void *miss_data, void *cache_data, const void *indices,
             int idx_bytes, const shmt_hashmap_t *map, const void *mask,
             int mask_bytes, const void *update, int64_t Q, int64_t row_bytes,
             void *stream);

/* Write-through form of shmt_set. The reference has no such mode (its
 * CacheTensorSet leaves the host row stale on a hit,
 * src/cache_feature_set.cu:108-114): here a row that hits is written to
 * cache_data[slot_i,:] AND to miss_data[indices[i],:], a row that misses to
 * miss_data[indices[i],:] only, so the id-addressed table stays current and
 * the cache can be dropped or rebuilt without a write-back. Same arguments
 * and checks as shmt_set; with neither map nor mask it is shmt_set.          */
int shmt_set_through(void *miss_data, void *cache_data, const void *indices,
                     int idx_bytes, const shmt_hashmap_t *map, const void *mask,
                     int mask_bytes, const void *update, int64_t Q,
                     int64_t row_bytes, void *stream);

/* ------------------------------------------------------------------ */
/* Scan. shmt_exclusive_scan: cub_exclusiveSum, src/tensor_relabel.cu:11-26
 * and src/cache_graph_sampling.cu:30-45 — in-place exclusive prefix sum over
 * `len` integers of elem_bytes in {4,8} (wraparound arithmetic); callers pass
 * len = n + 1 so that the last output is the total.
 * shmt_inclusive_scan_i32: thrust_scan, src/thrust_scan.cu:9-18
 * (ptr[i] += ptr[i-1] in program order = in-place inclusive sum, int32).
 * `tmp` is device scratch of at least shmt_scan_tmp_bytes(len) bytes.       */
int64_t shmt_scan_tmp_bytes(int64_t len);
int shmt_exclusive_scan(void *data, int64_t len, int elem_bytes, void *tmp,
                        int64_t tmp_bytes, void *stream);
int shmt_inclusive_scan_i32(void *data, int64_t len, void *tmp,
                            int64_t tmp_bytes, void *stream);
/* The same two scans on a workspace that is KEPT clean. The scans above take
 * any memory for `tmp` and clear it first, one short launch per call (cub's
 * temporary storage, src/tensor_relabel.cu:15-25, likewise needs no
 * preparation). A workspace that is all zero when a scan starts is all zero
 * again when it ends (the last workgroup to finish clears what the scan
 * used), so a caller that clears its workspace once (shmt_scan_workspace_clear,
 * or any memset) and then hands it to nothing but these scans, one at a
 * time, saves that launch on every call. kept_tmp: at least
 * shmt_scan_tmp_bytes(len) bytes, 8-byte aligned.                           */
int shmt_scan_workspace_clear(void *tmp, int64_t tmp_bytes, void *stream);
int shmt_exclusive_scan_kept(void *data, int64_t len, int elem_bytes,
                             void *kept_tmp, int64_t tmp_bytes, void *stream);
int shmt_inclusive_scan_i32_kept(void *data, int64_t len, void *kept_tmp,
                                 int64_t tmp_bytes, void *stream);
/* Bounded waits. A tile of a device-wide scan waits for the sums of the
 * tiles before it; that wait is bounded, and a tile that gives up leaves its
 * part of the array as it was, publishes nothing and sets a bit in an error
 * word of the current GPU (no counterpart in the reference, whose kernels
 * have no such waits). shmt_async_error waits for the GPU's queued work,
 * stores the word in *code_out (0: no kernel gave up; bit 0: a scan's
 * look-back) and clears it; when it is not 0, shmt_last_error() says what
 * gave up.                                                                  */
int shmt_async_error(int *code_out);
/* Sets bits of that word from the host, as a kernel that gave up would: for
 * tests of the error path (no kernel has to starve for them).               */
int shmt_async_error_inject(int bits);
/* Optional: a 4-byte word in pinned host memory (its host address and the
 * address the current GPU reaches it at, shmt_host_devptr) that a kernel
 * giving up also sets to non-zero, so that a host loop which polls pinned
 * memory anyway learns of it without a device call; shmt_async_error clears
 * it together with the GPU's word. The word must outlive every later launch
 * on that GPU, or be withdrawn first (null, null). No counterpart in the
 * reference.                                                                */
int shmt_async_error_mirror(void *host_word, void *device_alias);
/* shmt_exclusive_scan without a workspace argument, and without any
 * allocation inside the call. It has no counterpart in the reference (whose
 * cub_exclusiveSum allocates its temporary storage on every call,
 * src/tensor_relabel.cu:15-25); it is for callers that cannot allocate:
 * code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc. The sums its tiles publish live in a 260 KiB array that is
 * part of the library's code object (one copy per GPU, held until the process
 * ends), so
 * len is limited to SHMT_SCAN_NOALLOC_MAX_LEN elements; longer inputs are
 * rejected with SHMT_EINVAL. Same results as shmt_exclusive_scan. The first
 * call on a device looks up the array's device address (a call with len = 0
 * does only that and can serve as set-up before a capture). All calls on one
 * GPU share the array: calls that overlap on one GPU (different streams
 * without ordering between them) race; calls on one stream, or ordered by
 * events, are safe (every call clears what it uses before it scans).       */
#define SHMT_SCAN_NOALLOC_MAX_LEN (268435456ll)
int shmt_exclusive_scan_noalloc(void *data, int64_t len, int elem_bytes,
                                void *stream);

/* ------------------------------------------------------------------ */
/* Relabel: TensorRelabel, src/tensor_relabel.cu:125-209 (RelabelHashmap
 * :68-123). Input: N integers (elem_bytes in {4,8}), the concatenation of the
 * caller's tensors. Output: unique_out[0..U) = distinct values in order of
 * first occurrence, labels_out[i] = position of total[i] in unique_out,
 * both of width elem_bytes; *count_out = U (int64). count_out must be
 * device-accessible; when it points into pinned host memory the caller reads
 * it after synchronising the stream. unique_out must hold N elements. The
 * value -1 is not representable (empty key, src/tensor_relabel.cu:119).
 * Inputs of 2^31 ids or more (elem_bytes must then be 8) are relabelled with
 * 64-bit positions throughout, by the passes of shmt_relabel_wide; the
 * reference stops at 2^31 (int numel, uint32_t table positions,
 * src/tensor_relabel.cu:75-76,122,136).                                    */
int64_t shmt_relabel_scratch_bytes(int64_t N);
int shmt_relabel(const void *total, int64_t N, int elem_bytes, void *scratch,
                 int64_t scratch_bytes, void *unique_out, void *labels_out,
                 int64_t *count_out, void *stream);
/* The 64-bit-position form on its own, for 8-byte ids and any N < 2^40
 * (shmt_relabel switches to it at N >= 2^31; below that it is the slower
 * choice: 16-byte slots, no per-workgroup de-duplication, 8-byte ranks).
 * scratch >= shmt_relabel_wide_scratch_bytes(N), 16-byte aligned.           */
int64_t shmt_relabel_wide_scratch_bytes(int64_t N);
int shmt_relabel_wide(const void *total, int64_t N, void *scratch,
                      int64_t scratch_bytes, void *unique_out,
                      void *labels_out, int64_t *count_out, void *stream);
/* How large inputs are relabelled (no counterpart in the reference, whose
 * four passes all probe one table in memory, src/tensor_relabel.cu:147-203).
 * From partition_min_ids ids on (and up to 7,340,032) the first-occurrence index of
 * every id is found by partitioning the ids by hash and giving every
 * partition a table in LDS, which reads and writes memory in streams instead
 * of touching one random line per id and pass; results are identical.
 * partition_min_ids <= 0 restores the defaults: 2,097,153 for a hop whose size
 * is only a loose bound of its ids (the chained hops of shmt_sample_hop_chained),
 * 1,048,576 for calls that know their size, 524,288 for hops that share their
 * launches with those of three or more other batches
 * (shmt_sample_hops_chained); a value given lowers all three to it.
 * lds_slots_log2 (0 = default, 14) and max_rounds_log2 (-1 = default, 10)
 * shrink a partition's table and the
 * number of rounds a partition may take before all pairs of its ids are
 * compared; they exist so that tests can drive those rare paths. Process-wide,
 * not synchronised with calls in flight on other threads.                    */
int shmt_relabel_tuning(int64_t partition_min_ids, int lds_slots_log2,
                        int max_rounds_log2);
/* Same, with the concatenation of the caller's tensors (torch::cat,
 * src/tensor_relabel.cu:131) done on the way in: nseg <= SHMT_RELABEL_MAX_SEGMENTS
 * segments seg_ptrs[s] of seg_lens[s] ids, seg_bytes[s] in {4,8} wide, are
 * widened to elem_bytes (the width torch::cat would promote to) and written
 * to total_out (N = sum of seg_lens elements), which then plays the role of
 * `total` above. The three arrays are host arrays read during the call.
 * When last_len_dev is not NULL the true length of the LAST segment is read by
 * the kernels from that device address (an integer last_len_bytes in {4,8}
 * wide, e.g. sub_indptr[S] written by shmt_sample_plan earlier on the same
 * stream) and seg_lens[nseg-1] is only its upper bound: launches, scratch,
 * total_out, unique_out and labels_out are sized for the bound, results cover
 * the true length. This lets a caller queue sampling and relabel of one hop
 * without learning nnz on the host in between.                             */
#define SHMT_RELABEL_MAX_SEGMENTS 8
int shmt_relabel_segments(const void *const *seg_ptrs, const int64_t *seg_lens,
                          const int *seg_bytes, int nseg, const void *last_len_dev,
                          int last_len_bytes, int elem_bytes, void *total_out,
                          void *scratch, int64_t scratch_bytes, void *unique_out,
                          void *labels_out, int64_t *count_out, void *stream);

/* ------------------------------------------------------------------ */
/* Neighbour sampling: CSRWiseSampling src/cache_graph_sampling.cu:179-220
 * (GetSubIndptr :47-89, kernels :91-177) and CSRWiseCacheSampling :382-426
 * (GetSubIndptrWithCache :222-289, kernels :291-380).
 *
 * Step 1, shmt_sample_plan: per seed s, adjacency = cached row
 * cache_indptr[slot..slot+1] when map finds seeds[s] (map may be NULL: no
 * cache), else indptr[v..v+1]; cnt = replace ? (deg > 0 ? k : 0)
 * : min(deg, k); sub_indptr[0..S] = exclusive scan of cnt with total at [S]
 * (width ptr_bytes, the indptr width). Also writes *nnz_out (int64,
 * device-accessible) = total and the per-seed plan (row start, degree,
 * source) into `plan` (>= shmt_sample_plan_bytes(S) bytes).
 * Step 2, shmt_sample_pick: fills sub_indices[sub_indptr[s] ..) for every
 * seed from the plan: whole adjacency in CSR order when deg <= k
 * (replace = 0), k independent uniform picks (replace = 1), or a uniformly
 * distributed k-subset (replace = 0, deg > k). Random choices are a pure
 * function of (rng_seed, rng_stream, node id, k, degree) via Philox4x32-10,
 * so they do not depend on batch composition or on whether the row was
 * cached. sub_indices has width idx_bytes (the indices width) and room for
 * the total (<= S * k).
 * The reference fixes its RNG seed to 7777
 * (src/cache_graph_sampling.cu:204,407).                                   */
int64_t shmt_sample_plan_bytes(int64_t S);
int shmt_sample_plan(const void *indptr, int ptr_bytes,
                     const void *cache_indptr, const shmt_hashmap_t *map,
                     const void *seeds, int seed_bytes, int64_t S, int64_t k,
                     int replace, void *sub_indptr, void *plan,
                     int64_t plan_bytes, int64_t *nnz_out, void *stream);
int shmt_sample_pick(const void *indices, const void *cache_indices,
                     int idx_bytes, const void *seeds, int seed_bytes,
                     int64_t S, int64_t k, int replace, const void *sub_indptr,
                     int ptr_bytes, const void *plan, void *sub_indices,
                     uint64_t rng_seed, uint32_t rng_stream, void *stream);

/* Both steps for callers that can give sub_indices room for the bound S * k
 * (the first *nnz_out entries are the result): plan and pick are then two
 * launches whatever the number of seeds, queued back to back, because the
 * pick kernel adds the tile offsets of the plan itself and publishes the
 * total; nothing needs *nnz_out before the pick is queued. Same results as
 * shmt_sample_plan + shmt_sample_pick (CSRWiseSampling / CSRWiseCacheSampling,
 * src/cache_graph_sampling.cu:179-220, :382-426, which read nnz on the host
 * between the two steps, :195, :403). Requires S >= 1, k >= 1.             */
int shmt_sample(const void *indptr, int ptr_bytes, const void *indices,
                int idx_bytes, const void *cache_indptr,
                const void *cache_indices, const shmt_hashmap_t *map,
                const void *seeds, int seed_bytes, int64_t S, int64_t k,
                int replace, uint64_t rng_seed, uint32_t rng_stream,
                void *sub_indptr, void *sub_indices, void *plan,
                int64_t plan_bytes, int64_t *nnz_out, void *stream);

/* One hop of mini-batch sampling as one launch sequence: the body of the
 * dataloader's loop, python/shmtensor/sampling.py:128-143, i.e.
 * CSRWise[Cache]Sampling (src/cache_graph_sampling.cu:179-220, :382-426)
 * followed by TensorRelabel({seeds, sub_indices}) (src/tensor_relabel.cu:125-209).
 * No single operator of the reference corresponds to it. Results are exactly
 * those of shmt_sample_plan + shmt_sample_pick + shmt_relabel_segments on
 * {seeds, sub_indices}; the kernels are arranged so that the host need not
 * learn nnz before the relabel is queued and so that no separate
 * concatenation, table-fill or offset pass is launched: the plan kernel also
 * writes the seeds to total_out[0..S), the pick kernel also writes every
 * sampled id to total_out[S + offset], adds the tile offsets and empties the
 * relabel table, and the relabel passes read the sampled count from
 * device memory (a word of the plan buffer).
 * Requires S >= 1, k >= 1 and S * (k + 1) < 2^31. Buffers: sub_indptr S + 1
 * entries (ptr_bytes); sub_indices S * k entries (idx_bytes; the first nnz are
 * the result); plan >= shmt_sample_plan_bytes(S); total_out, unique_out,
 * labels_out S + S * k entries of elem_bytes = max(seed_bytes, idx_bytes);
 * scratch >= shmt_relabel_scratch_bytes(S + S * k), 16-byte aligned.
 * *nnz_out and *count_out (int64, device-accessible) receive the number of
 * sampled ids and of distinct ids; labels_out[S .. S + nnz) are the labels of
 * the sampled ids, unique_out[0 .. count) the distinct ids, seeds first.    */
int shmt_sample_hop(const void *indptr, int ptr_bytes, const void *indices,
                    int idx_bytes, const void *cache_indptr,
                    const void *cache_indices, const shmt_hashmap_t *map,
                    const void *seeds, int seed_bytes, int64_t S, int64_t k,
                    int replace, uint64_t rng_seed, uint32_t rng_stream,
                    void *sub_indptr, void *sub_indices, void *plan,
                    int64_t plan_bytes, int elem_bytes, void *total_out,
                    void *scratch, int64_t scratch_bytes, void *unique_out,
                    void *labels_out, int64_t *nnz_out, int64_t *count_out,
                    void *stream);

/* shmt_sample_hop for a number of seeds that only the GPU knows yet, so that
 * the hops of a mini-batch (python/shmtensor/sampling.py:128-143: the unique
 * ids of one hop are the seeds of the next) queue back to back without the
 * host reading a size in between; the reference waits on the host inside
 * every sampling and relabel call (src/cache_graph_sampling.cu:195,403,
 * src/tensor_relabel.cu:173). `seeds` holds min(max_seeds, *seeds_len)
 * seeds, seeds_len being an int64 in device memory written by earlier work
 * of the stream (count_dev_out of the previous hop, whose unique_out is
 * then `seeds`); seeds_len == NULL means max_seeds seeds. Every buffer is
 * sized as shmt_sample_hop sizes it for S = max_seeds; the results are laid
 * out for the true number of seeds S': sub_indptr has S' + 1 entries,
 * total_out / labels_out hold the S' seeds followed by the sampled ids.
 * count_dev_out (device memory, may be NULL) receives the number of
 * distinct ids like count_out does. rng_seed_dev (device memory, may be
 * NULL) overrides rng_seed with a value read by the kernels, so that a
 * captured launch sequence can be replayed with another seed.              */
int shmt_sample_hop_chained(const void *indptr, int ptr_bytes,
                            const void *indices, int idx_bytes,
                            const void *cache_indptr,
                            const void *cache_indices,
                            const shmt_hashmap_t *map, const void *seeds,
                            int seed_bytes, int64_t max_seeds,
                            const int64_t *seeds_len, int64_t k, int replace,
                            uint64_t rng_seed, const uint64_t *rng_seed_dev,
                            uint32_t rng_stream, void *sub_indptr,
                            void *sub_indices, void *plan,
                            int64_t plan_bytes, int elem_bytes,
                            void *total_out, void *scratch,
                            int64_t scratch_bytes, void *unique_out,
                            void *labels_out, int64_t *nnz_out,
                            int64_t *count_out, int64_t *count_dev_out,
                            void *stream);

/* Several independent chained hops at once (the same hop of several
 * mini-batches): every job is one shmt_sample_hop_chained call, the fields
 * are its parameters. Jobs that run the same kernels (same cache mode,
 * fan-out class and size class) share their launches: one launch per kernel
 * for up to 8 jobs, the job being a grid dimension, instead of one per job;
 * other jobs are issued one after the other. Results are those of the
 * individual calls. With several mini-batches in flight the host's launch
 * rate, not the GPU, bounds the sampler; the reference issues every kernel of
 * every hop of every batch separately (python/shmtensor/sampling.py:128-143). */
typedef struct shmt_hop_job {
  const void *indptr;
  int ptr_bytes;
  const void *indices;
  int idx_bytes;
  const void *cache_indptr;
  const void *cache_indices;
  const shmt_hashmap_t *map;
  const void *seeds;
  int seed_bytes;
  int64_t max_seeds;
  const int64_t *seeds_len;
  int64_t k;
  int replace;
  uint64_t rng_seed;
  const uint64_t *rng_seed_dev;
  uint32_t rng_stream;
  void *sub_indptr;
  void *sub_indices;
  void *plan;
  int64_t plan_bytes;
  int elem_bytes;
  void *total_out;
  void *scratch;
  int64_t scratch_bytes;
  void *unique_out;
  void *labels_out;
  int64_t *nnz_out;
  int64_t *count_out;
  int64_t *count_dev_out;
  /* Coordinate form of the hop's block (create_block_from_coo,
   * python/shmtensor/sampling.py:21-27): when coo_dst is not NULL the pick kernel
   * also writes, for every sampled id, the position of the seed it was sampled
   * for (the destination node of that edge; the source is its label in
   * labels_out), coo_bytes in {4,8} wide, S * k entries of room. NULL: not
   * produced.                                                               */
  void *coo_dst;
  int coo_bytes;
} shmt_hop_job;
int shmt_sample_hops_chained(const shmt_hop_job *jobs, int n_jobs, void *stream);

/* Queues one wave that stays busy for about `microseconds` (0 .. 100,000)
 * and touches no memory. No counterpart in the reference. For callers that
 * spread work over several streams: streams share a small number of
 * hardware queues, two streams on one queue run one after the other, and
 * the runtime does not say which share; a short wait queued on one stream
 * and an event on another show it (the shim's side-stream choice).        */
int shmt_busy_wait(void *stream, int microseconds);

/* Replaying a mini-batch. The hops of a batch, queued with
 * shmt_sample_hop_chained on fixed buffers, never wait for the host, so the
 * whole sequence can be captured once as a HIP graph and replayed for every
 * further batch with one launch instead of one per kernel (the reference
 * issues each kernel of each hop from the host and waits in between,
 * python/shmtensor/sampling.py:128-143). shmt_capture_begin starts recording
 * what is queued on `stream` (not the null stream); shmt_capture_end stops and
 * returns an executable graph; shmt_graph_launch replays it on a stream;
 * shmt_graph_destroy frees it. shmt_stage_seeds is the eager step before a
 * replay: it copies the n seeds of the next batch into the captured
 * sequence's input buffer (`staged`, widened from seed_bytes to staged_bytes)
 * and stores n and the batch's RNG seed where the captured kernels read them
 * (seeds_len / rng_seed_dev of the first / every hop).                      */
int shmt_capture_begin(void *stream);
int shmt_capture_end(void *stream, void **graph_exec_out);
int shmt_graph_launch(void *graph_exec, void *stream);
void shmt_graph_destroy(void *graph_exec);
int shmt_stage_seeds(const void *seeds, int seed_bytes, int64_t n, void *staged,
                     int staged_bytes, int64_t *len_out, uint64_t rng_seed,
                     uint64_t *rng_seed_out, void *stream);

/* Row coordinate of every element of a CSR / CSC structure:
 * rows_out[e] = r for offsets[r] <= e < offsets[r + 1], e < nnz = offsets[S]
 * (given by the caller), out_bytes in {4,8} wide. Turns the (sub_indptr,
 * labels) pair of a sampled block into the (col, row) pair of
 * create_block_from_coo (python/shmtensor/sampling.py:21-27) for hops that
 * did not produce it on the way (shmt_hop_job.coo_dst).                     */
int shmt_csr_rows(const void *offsets, int ptr_bytes, int64_t S, int64_t nnz,
                  void *rows_out, int out_bytes, void *stream);

/* Cached sub-CSR: CreateCacheCSR, src/cache_graph_sampling.cu:455-492
 * (CSRIndicesCopyKernel :428-453). Step 1 writes
 * cache_indptr[0..C] = exclusive scan of deg(seeds[i]) (width ptr_bytes) and
 * *nnz_out; step 2 copies the adjacency lists, in seeds order, into
 * cache_indices (width idx_bytes).                                         */
int shmt_subcsr_plan(const void *indptr, int ptr_bytes, const void *seeds,
                     int seed_bytes, int64_t C, void *cache_indptr, void *tmp,
                     int64_t tmp_bytes, int64_t *nnz_out, void *stream);
int shmt_subcsr_copy(const void *indptr, const void *indices, int ptr_bytes,
                     int idx_bytes, const void *seeds, int seed_bytes,
                     int64_t C, const void *cache_indptr, int64_t nnz,
                     void *cache_indices, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SHMT_H_ */
