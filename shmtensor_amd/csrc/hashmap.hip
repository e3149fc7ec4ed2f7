// Static hashmap: build and bulk query.
// Replaces pycuco::CUCOHashmap (include/cuco_hashmap.cuh:49-93 in the
// ShmTensor tree): same contract (immutable id -> value map, -1 for absent),
// own bucketed layout and wavefront-cooperative probing (see hashmap_dev.h).
#include <math.h>
#include <stdlib.h>

#include <mutex>

#include "common.h"
#include "hashmap.h"
#include "hashmap_dev.h"
#include "launchers.h"

namespace shmt {

// Densest physical fill of the table. A lookup costs one dependent HBM round
// trip per bucket on its probe chain; with 8 slots per 128-byte line about 5 %
// of the lines are full at 50 % fill against 31 % at 80 %, so denser requests
// are built at 50 % (capacity() still reports ceil(n / load_factor)).
constexpr double kMaxPhysicalLoad = 0.5;

static int64_t slots_needed(int64_t n, double lf) {
  if (lf > kMaxPhysicalLoad) lf = kMaxPhysicalLoad;
  int64_t cap = shmt_hashmap_capacity(n, lf);
  // always leave an empty slot so that a probe for an absent key terminates
  if (cap < n + 1) cap = n + 1;
  return cap;
}

static int format_for(int key_bytes, int val_bytes) {
  return (key_bytes == 4 && val_bytes == 4) ? kSlot8 : kSlot16;
}

static int64_t buckets_for(int64_t n, double lf, int fmt) {
  int64_t slots_per_bucket = kBucketBytes / fmt;
  int64_t slots = slots_needed(n, lf);
  return (slots + slots_per_bucket - 1) / slots_per_bucket;
}

// ---- kernels ---------------------------------------------------------------

// Group insert of one (key, value) into the wide table. All 8 lanes of the
// probe group call with the same arguments.
__device__ __forceinline__ void group_insert16(uint64_t *table, uint32_t nbuckets,
                                               int64_t key, int64_t val) {
  const int sub = lane_id() & (kProbeGroup - 1);
  const int gbase = lane_id() & ~(kProbeGroup - 1);
  uint32_t b = reduce_range(hash_id(key), nbuckets);
  uint32_t probes = 0;
  while (probes < nbuckets) {
    uint64_t *slot = table + (static_cast<size_t>(b) * kProbeGroup + sub) * 2;
    // Fresh (L2-coherent) read of the slot key: another workgroup may have
    // claimed it since this CU last cached the line.
    int64_t k = static_cast<int64_t>(
        __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    if (group_ballot<kProbeGroup>(k == key)) return;  // duplicate key: first one wins
    uint64_t em = group_ballot<kProbeGroup>(k == -1);
    if (!em) {
      b = (b + 1 == nbuckets) ? 0 : b + 1;
      ++probes;
      continue;
    }
    const int target = __builtin_ctzll(em);
    int64_t old = 0;
    if (sub == target) {
      unsigned long long prev = atomicCAS(reinterpret_cast<unsigned long long *>(slot),
                                          ~0ull, static_cast<unsigned long long>(key));
      old = static_cast<int64_t>(prev);
      if (old == -1) slot[1] = static_cast<uint64_t>(val);
    }
    old = shfl64(old, gbase + target);
    if (old == -1 || old == key) return;
    // lost the race for that slot to a different key: look at the bucket again
  }
}

// Narrow table: each lane owns two 8-byte {key,value} words and claims one
// with a single 64-bit compare-and-swap.
__device__ __forceinline__ void group_insert8(uint64_t *table, uint32_t nbuckets,
                                              int32_t key, int32_t val) {
  const int sub = lane_id() & (kProbeGroup - 1);
  const int gbase = lane_id() & ~(kProbeGroup - 1);
  uint32_t b = reduce_range(hash_id(static_cast<int64_t>(key)), nbuckets);
  const uint64_t word = (static_cast<uint64_t>(static_cast<uint32_t>(val)) << 32) |
                        static_cast<uint32_t>(key);
  uint32_t probes = 0;
  while (probes < nbuckets) {
    uint64_t *slot = table + (static_cast<size_t>(b) * kProbeGroup + sub) * 2;
    uint64_t w0 = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint64_t w1 = __hip_atomic_load(slot + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    bool match = static_cast<int32_t>(static_cast<uint32_t>(w0)) == key ||
                 static_cast<int32_t>(static_cast<uint32_t>(w1)) == key;
    if (group_ballot<kProbeGroup>(match)) return;
    bool e0 = (w0 == ~0ull), e1 = (w1 == ~0ull);
    uint64_t em = group_ballot<kProbeGroup>(e0 || e1);
    if (!em) {
      b = (b + 1 == nbuckets) ? 0 : b + 1;
      ++probes;
      continue;
    }
    const int target = __builtin_ctzll(em);
    int64_t old = 0;
    if (sub == target) {
      unsigned long long prev = atomicCAS(
          reinterpret_cast<unsigned long long *>(slot + (e0 ? 0 : 1)), ~0ull,
          static_cast<unsigned long long>(word));
      old = static_cast<int64_t>(prev);
    }
    old = shfl64(old, gbase + target);
    if (old == -1 || static_cast<int32_t>(static_cast<uint32_t>(static_cast<uint64_t>(old))) == key)
      return;
  }
}

// One wave takes 64 consecutive (key, value) pairs with coalesced loads; in
// step j the probe group g inserts pair g*8+j, so 8 inserts proceed per wave
// at a time and every bucket read is a full-line transaction.
template <int FMT>
__global__ __launch_bounds__(256) void hashmap_insert_kernel(
    uint64_t *table, uint32_t nbuckets, const void *keys, const void *vals,
    int64_t n, int key_bytes, int val_bytes) {
  const int lane = lane_id();
  const int gbase = lane & ~(kProbeGroup - 1);
  const int64_t waves_per_block = blockDim.x / kWave;
  int64_t wave = static_cast<int64_t>(blockIdx.x) * waves_per_block + threadIdx.x / kWave;
  const int64_t nwaves = static_cast<int64_t>(gridDim.x) * waves_per_block;
  for (int64_t base = wave * kWave; base < n; base += nwaves * kWave) {
    int64_t i = base + lane;
    int64_t mykey = -1, myval = -1;
    if (i < n) {
      mykey = load_int(keys, i, key_bytes);
      myval = load_int(vals, i, val_bytes);
    }
#pragma unroll 1
    for (int j = 0; j < kProbeGroup; ++j) {
      int64_t k = shfl64(mykey, gbase + j);
      int64_t v = shfl64(myval, gbase + j);
      if (base + gbase + j < n) {
        if (FMT == kSlot16)
          group_insert16(table, nbuckets, k, v);
        else
          group_insert8(table, nbuckets, static_cast<int32_t>(k), static_cast<int32_t>(v));
      }
    }
  }
}

// ---- what do the keys look like? ---------------------------------------------
// One sweep over (keys, values): extrema of both, and whether value - key is
// the same for every pair. The host reads the result and picks the layout.
struct KeyStats {
  long long kmin, kmax, vmin, vmax;
  unsigned long long not_affine;  // != 0: value - key differs between pairs
  unsigned long long distinct;    // range candidates only: number of different keys
  unsigned long long not_ranked;  // != 0: keys do not ascend strictly, or value i is not value 0 + i
};

constexpr int kStatBlocks = 1024;          // workgroups of a sweep, each leaving one partial result
constexpr int64_t kStatPartialsOff = 256;  // scratch layout: header, partials, then one mark byte per id
constexpr int64_t kStatMarksOff = kStatPartialsOff + ((kStatBlocks * sizeof(KeyStats) + 255) & ~255ll);

__device__ __forceinline__ int64_t wave_min64(int64_t v) {
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int64_t o = shfl64(v, lane_id() ^ d);
    v = o < v ? o : v;
  }
  return v;
}
__device__ __forceinline__ int64_t wave_max64(int64_t v) {
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int64_t o = shfl64(v, lane_id() ^ d);
    v = o > v ? o : v;
  }
  return v;
}

// Combines the calling workgroup's per-thread values into one KeyStats, valid
// in thread 0 (no atomics: thousands of them on a handful of addresses would
// cost more than the sweep).
__device__ __forceinline__ KeyStats block_combine(KeyStats mine) {
  __shared__ KeyStats per_wave[256 / kWave];
  mine.kmin = wave_min64(mine.kmin);
  mine.kmax = wave_max64(mine.kmax);
  mine.vmin = wave_min64(mine.vmin);
  mine.vmax = wave_max64(mine.vmax);
  mine.not_affine = __builtin_amdgcn_ballot_w64(mine.not_affine != 0) != 0;
  mine.not_ranked = __builtin_amdgcn_ballot_w64(mine.not_ranked != 0) != 0;
  mine.distinct = wave_last(wave_inclusive_scan(static_cast<uint64_t>(mine.distinct)));
  if (lane_id() == 0) per_wave[threadIdx.x / kWave] = mine;
  __syncthreads();
  KeyStats all = per_wave[0];
  if (threadIdx.x == 0) {
    for (unsigned w = 1; w < blockDim.x / kWave; ++w) {
      const KeyStats o = per_wave[w];
      all.kmin = o.kmin < all.kmin ? o.kmin : all.kmin;
      all.kmax = o.kmax > all.kmax ? o.kmax : all.kmax;
      all.vmin = o.vmin < all.vmin ? o.vmin : all.vmin;
      all.vmax = o.vmax > all.vmax ? o.vmax : all.vmax;
      all.not_affine |= o.not_affine;
      all.not_ranked |= o.not_ranked;
      all.distinct += o.distinct;
    }
  }
  return all;
}

__device__ __forceinline__ KeyStats neutral_stats() {
  return KeyStats{INT64_MAX, INT64_MIN, INT64_MAX, INT64_MIN, 0, 0, 0};
}

__global__ __launch_bounds__(256) void key_stats_kernel(const void *keys, const void *vals, int64_t n,
                                                        int key_bytes, int val_bytes, KeyStats *partials) {
  const int64_t v0 = load_int(vals, 0, val_bytes);
  const int64_t delta0 = v0 - load_int(keys, 0, key_bytes);
  KeyStats mine = neutral_stats();
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int64_t k = load_int(keys, i, key_bytes), v = load_int(vals, i, val_bytes);
    mine.kmin = k < mine.kmin ? k : mine.kmin;
    mine.kmax = k > mine.kmax ? k : mine.kmax;
    mine.vmin = v < mine.vmin ? v : mine.vmin;
    mine.vmax = v > mine.vmax ? v : mine.vmax;
    mine.not_affine |= (v - k != delta0);
    // the neighbour's key is the load of the thread next door: served by the caches
    mine.not_ranked |= (v != v0 + i) || (i > 0 && load_int(keys, i - 1, key_bytes) >= k);
  }
  const KeyStats all = block_combine(mine);
  if (threadIdx.x == 0) partials[blockIdx.x] = all;
}

// One workgroup merges the partial results of a sweep and hands the outcome to
// the host through a slot of pinned host memory (a device-to-host copy into
// pageable memory would go through the runtime's staging path).
__global__ __launch_bounds__(256) void stats_merge_kernel(const KeyStats *partials, int nb, KeyStats *host_slot) {
  KeyStats mine = neutral_stats();
  for (int b = threadIdx.x; b < nb; b += blockDim.x) {
    const KeyStats o = partials[b];
    mine.kmin = o.kmin < mine.kmin ? o.kmin : mine.kmin;
    mine.kmax = o.kmax > mine.kmax ? o.kmax : mine.kmax;
    mine.vmin = o.vmin < mine.vmin ? o.vmin : mine.vmin;
    mine.vmax = o.vmax > mine.vmax ? o.vmax : mine.vmax;
    mine.not_affine |= o.not_affine;
    mine.not_ranked |= o.not_ranked;
    mine.distinct += o.distinct;
  }
  const KeyStats all = block_combine(mine);
  if (threadIdx.x == 0) *host_slot = all;
}

// One slot of pinned host memory per process, allocated on first use; map
// builds that run at the same time take turns at it.
static std::mutex g_stat_mutex;
static KeyStats *g_stat_slot = nullptr;      // pinned host memory
static KeyStats *g_stat_slot_dev = nullptr;  // its device alias

// Merge the partial results of a sweep, hand them to the host and wait for them.
static int read_stats(const KeyStats *partials, int nb, KeyStats *out, hipStream_t s) {
  std::lock_guard<std::mutex> lock(g_stat_mutex);
  if (g_stat_slot == nullptr) {
    void *p = nullptr, *d = nullptr;
    SHMT_HIP(hipHostMalloc(&p, 256, hipHostMallocMapped));
    SHMT_HIP(hipHostGetDevicePointer(&d, p, 0));
    g_stat_slot = static_cast<KeyStats *>(p);
    g_stat_slot_dev = static_cast<KeyStats *>(d);
  }
  hipLaunchKernelGGL(stats_merge_kernel, dim3(1), dim3(256), 0, s, partials, nb, g_stat_slot_dev);
  SHMT_LAUNCH_CHECK();
  SHMT_HIP(hipStreamSynchronize(s));
  *out = *g_stat_slot;
  return SHMT_OK;
}

// Range candidates (as many pairs as ids between the extrema): every key marks
// its byte (plain stores: racing writers all write the same value), then the
// marked bytes are counted; fewer marks than pairs means a key repeats, and
// then some id of the range is missing.
__global__ __launch_bounds__(256) void key_mark_kernel(const void *keys, int64_t n, int key_bytes,
                                                       int64_t lo, uint8_t *seen) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
    const uint64_t off = static_cast<uint64_t>(load_int(keys, i, key_bytes) - lo);
    if (off < static_cast<uint64_t>(n)) seen[off] = 1;  // always true for a genuine candidate
  }
}

__global__ __launch_bounds__(256) void key_count_marks_kernel(const uint32_t *seen_words, int64_t nwords,
                                                              KeyStats *partials) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  KeyStats mine = neutral_stats();
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nwords; i += stride)
    mine.distinct += __builtin_popcount(seen_words[i]);  // a marked byte is 0x01
  const KeyStats all = block_combine(mine);
  if (threadIdx.x == 0) partials[blockIdx.x] = all;
}

__global__ __launch_bounds__(256) void fill_zero_kernel(uint32_t *p, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = 0;
}

// Direct form: value[key - lo] for every pair (the table was filled with -1).
__global__ __launch_bounds__(256) void direct_build_kernel(int32_t *table, int64_t lo, int64_t span,
                                                           const void *keys, const void *vals, int64_t n,
                                                           int key_bytes, int val_bytes) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
    const uint64_t off = static_cast<uint64_t>(load_int(keys, i, key_bytes) - lo);
    if (off < static_cast<uint64_t>(span)) table[off] = static_cast<int32_t>(load_int(vals, i, val_bytes));
  }
}

// Rank form: one thread per 16-byte block = 96 consecutive ids. The keys
// ascend, so the thread finds the first key of its block by bisection (that
// index is the number of keys below the block) and walks the keys from there
// while they stay inside the block. Every block is written whole, the empty
// ones too: no clearing pass and no atomics.
__global__ __launch_bounds__(256) void rank_build_kernel(uint4 *table, int64_t nblocks, int64_t lo,
                                                         const void *keys, int64_t n, int key_bytes) {
  const int64_t b = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (b >= nblocks) return;
  const int64_t first_id = lo + b * kRankIdsPerBlock;
  int64_t below = 0, above = n;  // keys[below - 1] < first_id <= keys[above]
  while (below < above) {
    const int64_t mid = below + (above - below) / 2;
    if (load_int(keys, mid, key_bytes) < first_id)
      below = mid + 1;
    else
      above = mid;
  }
  uint32_t bits[3] = {0, 0, 0};
  for (int64_t j = below; j < n; ++j) {
    const uint64_t r = static_cast<uint64_t>(load_int(keys, j, key_bytes) - first_id);
    if (r >= static_cast<uint64_t>(kRankIdsPerBlock)) break;
    const uint32_t bit = 1u << (r & 31);
    bits[0] |= r < 32 ? bit : 0u;
    bits[1] |= (r >= 32 && r < 64) ? bit : 0u;
    bits[2] |= r >= 64 ? bit : 0u;
  }
  table[b] = make_uint4(static_cast<uint32_t>(below), bits[0], bits[1], bits[2]);
}

// Bulk query: a wave owns 64 consecutive requests. The eight bucket loads of
// a probe group (one per step) are all issued before the first is examined,
// which keeps 8 KiB of table reads in flight per wave; results are gathered
// back to the lane that loaded the request, so request reads and result
// writes are both fully coalesced.
template <int FMT>
__global__ __launch_bounds__(256) void hashmap_query_kernel(
    MapView m, const void *req, int req_bytes, void *out, int out_bytes, int64_t n) {
  const int lane = lane_id();
  const int64_t waves_per_block = blockDim.x / kWave;
  int64_t wave = static_cast<int64_t>(blockIdx.x) * waves_per_block + threadIdx.x / kWave;
  const int64_t nwaves = static_cast<int64_t>(gridDim.x) * waves_per_block;
  for (int64_t base = wave * kWave; base < n; base += nwaves * kWave) {
    const int64_t i = base + lane;
    int64_t mykey = -1;  // tail lanes look up the sentinel, which resolves to -1
    if (i < n) mykey = map_key(m, load_int(req, i, req_bytes));
    const int64_t myres = wave_find<FMT>(m, mykey);
    if (i < n) store_int(out, i, out_bytes, myres);
  }
}

}  // namespace shmt

using namespace shmt;

extern "C" {

int64_t shmt_hashmap_capacity(int64_t n, double load_factor) {
  if (n < 0 || !(load_factor > 0.0)) return -1;
  return static_cast<int64_t>(ceil(static_cast<double>(n) / load_factor));
}

int64_t shmt_hashmap_table_bytes(int64_t n, double load_factor, int key_bytes, int val_bytes) {
  if (n < 0 || !(load_factor > 0.0) || !(load_factor <= 1.0) || !width_ok(key_bytes) ||
      !width_ok(val_bytes)) {
    set_error("shmt_hashmap_table_bytes: bad arguments (n=%lld, load_factor=%g, key_bytes=%d, val_bytes=%d)",
              static_cast<long long>(n), load_factor, key_bytes, val_bytes);
    return -1;
  }
  return buckets_for(n, load_factor, format_for(key_bytes, val_bytes)) * kBucketBytes;
}

int64_t shmt_hashmap_plan_scratch_bytes(int64_t n) {
  if (n < 0) return -1;
  return kStatMarksOff + ((n + 3) / 4) * 4;
}

int shmt_hashmap_plan(const void *keys, const void *vals, int64_t n, int key_bytes, int val_bytes,
                      double load_factor, void *scratch, int64_t scratch_bytes,
                      shmt_hashmap_layout *layout, void *stream) {
  SHMT_REQUIRE(layout != nullptr, "shmt_hashmap_plan: layout is null");
  SHMT_REQUIRE(n >= 0, "shmt_hashmap_plan: n must be >= 0");
  SHMT_REQUIRE(width_ok(key_bytes) && width_ok(val_bytes),
               "shmt_hashmap_plan: ID can only be int32 or int64 (key_bytes=%d, val_bytes=%d)", key_bytes,
               val_bytes);
  SHMT_REQUIRE(load_factor > 0.0 && load_factor <= 1.0, "shmt_hashmap_plan: load_factor must be in (0, 1], got %g",
               load_factor);
  const int dtype_fmt = format_for(key_bytes, val_bytes);
  layout->kind = SHMT_MAP_BUCKETS;
  layout->slot_bytes = dtype_fmt;
  layout->lo = layout->span = layout->delta = 0;
  layout->table_bytes = buckets_for(n, load_factor, dtype_fmt) * kBucketBytes;
  if (n == 0) return SHMT_OK;
  SHMT_REQUIRE(keys != nullptr && vals != nullptr, "shmt_hashmap_plan: keys/vals are null");
  if (scratch == nullptr || scratch_bytes < shmt_hashmap_plan_scratch_bytes(n)) {
    set_error("shmt_hashmap_plan: scratch too small (%lld < %lld bytes)", static_cast<long long>(scratch_bytes),
              static_cast<long long>(shmt_hashmap_plan_scratch_bytes(n)));
    return SHMT_ENOMEM;
  }
  SHMT_REQUIRE((reinterpret_cast<uintptr_t>(scratch) & 15) == 0, "shmt_hashmap_plan: scratch must be 16-byte aligned");
  hipStream_t s = as_stream(stream);
  KeyStats *partials = reinterpret_cast<KeyStats *>(static_cast<char *>(scratch) + kStatPartialsOff);
  uint32_t *marks = reinterpret_cast<uint32_t *>(static_cast<char *>(scratch) + kStatMarksOff);  // one byte per id
  const unsigned nb = grid_for(n, 256 * 8, kStatBlocks);
  hipLaunchKernelGGL(key_stats_kernel, dim3(nb), dim3(256), 0, s, keys, vals, n, key_bytes, val_bytes, partials);
  SHMT_LAUNCH_CHECK();
  KeyStats st;
  int rc = read_stats(partials, static_cast<int>(nb), &st, s);
  if (rc) return rc;

  const bool keys32 = st.kmin >= INT32_MIN && st.kmax <= INT32_MAX;
  const bool vals32 = st.vmin >= INT32_MIN && st.vmax <= INT32_MAX;
  // narrow slots whenever every key and value fits 32 bits, whatever the dtypes say
  const int fmt = (keys32 && vals32) ? kSlot8 : kSlot16;
  layout->slot_bytes = fmt;
  layout->table_bytes = buckets_for(n, load_factor, fmt) * kBucketBytes;
  // flat forms need non-negative ids (-1 is the empty key) and a span that can be indexed
  if (st.kmin < 0 || st.kmax - st.kmin >= (1ll << 40)) return SHMT_OK;
  const int64_t span = st.kmax - st.kmin + 1;
  if (span == n && !st.not_affine) {
    // as many pairs as ids in the range and one offset for all: a range map unless a key repeats
    const int64_t words = (n + 3) / 4;
    hipLaunchKernelGGL(fill_zero_kernel, dim3(grid_for(words, 256 * 4)), dim3(256), 0, s, marks, words);
    hipLaunchKernelGGL(key_mark_kernel, dim3(grid_for(n, 256 * 8, 256 * 8)), dim3(256), 0, s, keys, n, key_bytes,
                       static_cast<int64_t>(st.kmin), reinterpret_cast<uint8_t *>(marks));
    const unsigned nbc = grid_for(words, 256 * 8, kStatBlocks);
    hipLaunchKernelGGL(key_count_marks_kernel, dim3(nbc), dim3(256), 0, s, marks, words, partials);
    SHMT_LAUNCH_CHECK();
    KeyStats counted;
    rc = read_stats(partials, static_cast<int>(nbc), &counted, s);
    if (rc) return rc;
    if (counted.distinct == static_cast<unsigned long long>(n)) {
      layout->kind = SHMT_MAP_RANGE;
      layout->slot_bytes = 0;
      layout->lo = st.kmin;
      layout->span = span;
      layout->delta = st.vmin - st.kmin;  // value - key is one constant, so the minima pair up
      layout->table_bytes = kBucketBytes;  // nothing is stored; callers still pass a valid pointer
      return SHMT_OK;
    }
  }
  // pairs in ascending key order with consecutive values: bitmap with running counts, 16 bytes per 96 ids,
  // while that stays within twice the bucket table's size (ids up to 190 times as many as keys)
  const int64_t rank_bytes = ((span + kRankIdsPerBlock - 1) / kRankIdsPerBlock * 16 + kBucketBytes - 1) /
                             kBucketBytes * kBucketBytes;
  if (!st.not_ranked && n < (1ll << 32) && rank_bytes <= 2 * layout->table_bytes) {
    layout->kind = SHMT_MAP_RANK;
    layout->slot_bytes = 16;
    layout->lo = st.kmin;
    layout->span = span;
    layout->delta = st.vmin;  // the first pair holds the smallest key and the smallest value
    layout->table_bytes = rank_bytes;
    return SHMT_OK;
  }
  // direct table while it stays within twice the bucket table's size (ids up to 8 times as many as
  // keys when both fit 32 bits): one load per lookup instead of a cooperative probe sequence
  if (vals32 && span * 4 <= 2 * layout->table_bytes) {
    layout->kind = SHMT_MAP_DIRECT;
    layout->slot_bytes = 4;
    layout->lo = st.kmin;
    layout->span = span;
    layout->table_bytes = (span * 4 + kBucketBytes - 1) / kBucketBytes * kBucketBytes;
  }
  return SHMT_OK;
}

static int build_buckets(shmt_hashmap_t **out, int fmt, const void *keys, const void *vals, int64_t n,
                         int key_bytes, int val_bytes, double load_factor, void *table_mem,
                         int64_t table_bytes, void *stream);

int shmt_hashmap_create_planned(shmt_hashmap_t **out, const shmt_hashmap_layout *layout, const void *keys,
                                const void *vals, int64_t n, int key_bytes, int val_bytes,
                                double load_factor, void *table_mem, int64_t table_bytes, void *stream) {
  SHMT_REQUIRE(out != nullptr && layout != nullptr, "shmt_hashmap_create_planned: null argument");
  *out = nullptr;
  SHMT_REQUIRE(n >= 0, "shmt_hashmap_create_planned: n must be >= 0");
  SHMT_REQUIRE(width_ok(key_bytes) && width_ok(val_bytes),
               "shmt_hashmap_create_planned: ID can only be int32 or int64 (key_bytes=%d, val_bytes=%d)",
               key_bytes, val_bytes);
  SHMT_REQUIRE(load_factor > 0.0 && load_factor <= 1.0,
               "shmt_hashmap_create_planned: load_factor must be in (0, 1], got %g", load_factor);
  if (layout->kind == SHMT_MAP_BUCKETS) {
    SHMT_REQUIRE(layout->slot_bytes == kSlot16 || layout->slot_bytes == kSlot8,
                 "shmt_hashmap_create_planned: bad slot size %d", layout->slot_bytes);
    return build_buckets(out, layout->slot_bytes, keys, vals, n, key_bytes, val_bytes, load_factor, table_mem,
                         table_bytes, stream);
  }
  SHMT_REQUIRE(layout->kind == SHMT_MAP_DIRECT || layout->kind == SHMT_MAP_RANGE || layout->kind == SHMT_MAP_RANK,
               "shmt_hashmap_create_planned: unknown layout kind %d", layout->kind);
  SHMT_REQUIRE(n > 0 && keys != nullptr && vals != nullptr && layout->lo >= 0 && layout->span > 0,
               "shmt_hashmap_create_planned: a flat layout needs keys and a non-negative id range");
  SHMT_REQUIRE(layout->kind != SHMT_MAP_RANK || n < (1ll << 32),
               "shmt_hashmap_create_planned: a rank layout holds fewer than 2^32 keys (32-bit running counts)");
  hipStream_t s = as_stream(stream);
  if (layout->kind == SHMT_MAP_DIRECT) {
    if (table_mem == nullptr || table_bytes < layout->table_bytes || layout->table_bytes < layout->span * 4) {
      set_error("shmt_hashmap_create_planned: table_mem too small (%lld < %lld bytes)",
                static_cast<long long>(table_bytes), static_cast<long long>(layout->table_bytes));
      return SHMT_ENOMEM;
    }
    SHMT_REQUIRE((reinterpret_cast<uintptr_t>(table_mem) & 127) == 0,
                 "shmt_hashmap_create_planned: table_mem must be 128-byte aligned");
    int rc = launch_fill_ones(table_mem, layout->table_bytes / 16, s);
    if (rc) return rc;
    hipLaunchKernelGGL(direct_build_kernel, dim3(grid_for(n, 256 * 4)), dim3(256), 0, s,
                       static_cast<int32_t *>(table_mem), layout->lo, layout->span, keys, vals, n, key_bytes,
                       val_bytes);
    SHMT_LAUNCH_CHECK();
  }
  if (layout->kind == SHMT_MAP_RANK) {
    const int64_t nblocks = (layout->span + kRankIdsPerBlock - 1) / kRankIdsPerBlock;
    if (table_mem == nullptr || table_bytes < layout->table_bytes || layout->table_bytes < nblocks * 16) {
      set_error("shmt_hashmap_create_planned: table_mem too small (%lld < %lld bytes)",
                static_cast<long long>(table_bytes), static_cast<long long>(layout->table_bytes));
      return SHMT_ENOMEM;
    }
    SHMT_REQUIRE((reinterpret_cast<uintptr_t>(table_mem) & 127) == 0,
                 "shmt_hashmap_create_planned: table_mem must be 128-byte aligned");
    hipLaunchKernelGGL(rank_build_kernel, dim3(grid_for(nblocks, 256)), dim3(256), 0, s,
                       static_cast<uint4 *>(table_mem), nblocks, layout->lo, keys, n, key_bytes);
    SHMT_LAUNCH_CHECK();
  }
  shmt_hashmap *h = static_cast<shmt_hashmap *>(calloc(1, sizeof(shmt_hashmap)));
  if (h == nullptr) {
    set_error("shmt_hashmap_create_planned: out of host memory");
    return SHMT_ENOMEM;
  }
  h->view = empty_map_view();
  h->view.buckets = static_cast<const uint4 *>(table_mem);
  h->view.key32 = (key_bytes == 4);
  h->view.kind = layout->kind == SHMT_MAP_DIRECT ? kKindDirect
                 : layout->kind == SHMT_MAP_RANK ? kKindRank : kKindRange;
  h->view.lo = layout->lo;
  h->view.span = layout->span;
  h->view.delta = layout->delta;
  h->kind = h->view.kind;
  h->fmt = kSlot8;  // kernels that branch on the kind at run time are launched in this form
  h->key_bytes = key_bytes;
  h->val_bytes = val_bytes;
  h->n = n;
  h->table_bytes = layout->kind == SHMT_MAP_RANGE ? 0 : layout->table_bytes;
  *out = h;
  return SHMT_OK;
}

int shmt_hashmap_create(shmt_hashmap_t **out, const void *keys, const void *vals, int64_t n,
                        int key_bytes, int val_bytes, double load_factor, void *table_mem,
                        int64_t table_bytes, void *stream) {
  SHMT_REQUIRE(width_ok(key_bytes) && width_ok(val_bytes),
               "shmt_hashmap_create: ID can only be int32 or int64 (key_bytes=%d, val_bytes=%d)",
               key_bytes, val_bytes);
  return build_buckets(out, format_for(key_bytes, val_bytes), keys, vals, n, key_bytes, val_bytes, load_factor,
                       table_mem, table_bytes, stream);
}

// Bucket table in slot format `fmt` (kSlot8 requires that every key and value fits 32 bits).
static int build_buckets(shmt_hashmap_t **out, const int fmt, const void *keys, const void *vals, int64_t n,
                         int key_bytes, int val_bytes, double load_factor, void *table_mem,
                         int64_t table_bytes, void *stream) {
  SHMT_REQUIRE(out != nullptr, "shmt_hashmap_create: out is null");
  *out = nullptr;
  SHMT_REQUIRE(n >= 0, "shmt_hashmap_create: n must be >= 0");
  SHMT_REQUIRE(width_ok(key_bytes) && width_ok(val_bytes),
               "shmt_hashmap_create: ID can only be int32 or int64 (key_bytes=%d, val_bytes=%d)",
               key_bytes, val_bytes);
  SHMT_REQUIRE(load_factor > 0.0 && load_factor <= 1.0,
               "shmt_hashmap_create: load_factor must be in (0, 1], got %g", load_factor);
  SHMT_REQUIRE(n == 0 || (keys != nullptr && vals != nullptr),
               "shmt_hashmap_create: keys/vals are null");
  const int64_t nb = buckets_for(n, load_factor, fmt);
  SHMT_REQUIRE(nb < (1ll << 31), "shmt_hashmap_create: table too large (%lld buckets)",
               static_cast<long long>(nb));
  if (table_mem == nullptr || table_bytes < nb * kBucketBytes) {
    set_error("shmt_hashmap_create: table_mem too small (%lld < %lld bytes)",
              static_cast<long long>(table_bytes), static_cast<long long>(nb * kBucketBytes));
    return SHMT_ENOMEM;
  }
  SHMT_REQUIRE((reinterpret_cast<uintptr_t>(table_mem) & 127) == 0,
               "shmt_hashmap_create: table_mem must be 128-byte aligned");

  hipStream_t s = as_stream(stream);
  int rc = launch_fill_ones(table_mem, nb * (kBucketBytes / 16), s);
  if (rc) return rc;
  if (n > 0) {
    unsigned grid = grid_for(n, 256);
    if (fmt == kSlot16)
      hipLaunchKernelGGL(hashmap_insert_kernel<kSlot16>, dim3(grid), dim3(256), 0, s,
                         static_cast<uint64_t *>(table_mem), static_cast<uint32_t>(nb), keys,
                         vals, n, key_bytes, val_bytes);
    else
      hipLaunchKernelGGL(hashmap_insert_kernel<kSlot8>, dim3(grid), dim3(256), 0, s,
                         static_cast<uint64_t *>(table_mem), static_cast<uint32_t>(nb), keys,
                         vals, n, key_bytes, val_bytes);
    SHMT_LAUNCH_CHECK();
  }

  shmt_hashmap *h = static_cast<shmt_hashmap *>(calloc(1, sizeof(shmt_hashmap)));
  if (h == nullptr) {
    set_error("shmt_hashmap_create: out of host memory");
    return SHMT_ENOMEM;
  }
  h->view = empty_map_view();
  h->view.buckets = static_cast<const uint4 *>(table_mem);
  h->view.nbuckets = static_cast<uint32_t>(nb);
  h->view.key32 = (key_bytes == 4);
  h->view.fits32 = (fmt == kSlot8 && key_bytes == 8);
  h->kind = kKindBuckets;
  h->fmt = fmt;
  h->key_bytes = key_bytes;
  h->val_bytes = val_bytes;
  h->n = n;
  h->table_bytes = nb * kBucketBytes;
  *out = h;
  return SHMT_OK;
}

int shmt_hashmap_query(const shmt_hashmap_t *map, const void *requests, int req_bytes,
                       int64_t n, void *out, void *stream) {
  SHMT_REQUIRE(map != nullptr, "shmt_hashmap_query: map is null");
  SHMT_REQUIRE(n >= 0, "shmt_hashmap_query: n must be >= 0");
  SHMT_REQUIRE(width_ok(req_bytes), "shmt_hashmap_query: ID can only be int32 or int64");
  if (n == 0) return SHMT_OK;
  SHMT_REQUIRE(requests != nullptr && out != nullptr, "shmt_hashmap_query: null buffer");
  unsigned grid = grid_for(n, 256);
  hipStream_t s = as_stream(stream);
  if (map->fmt == kSlot16)
    hipLaunchKernelGGL(hashmap_query_kernel<kSlot16>, dim3(grid), dim3(256), 0, s, map->view,
                       requests, req_bytes, out, map->val_bytes, n);
  else
    hipLaunchKernelGGL(hashmap_query_kernel<kSlot8>, dim3(grid), dim3(256), 0, s, map->view,
                       requests, req_bytes, out, map->val_bytes, n);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

int shmt_hashmap_kind(const shmt_hashmap_t *map) { return map ? map->kind : -1; }
int64_t shmt_hashmap_used_bytes(const shmt_hashmap_t *map) { return map ? map->table_bytes : 0; }
int shmt_hashmap_key_bytes(const shmt_hashmap_t *map) { return map ? map->key_bytes : 0; }
int shmt_hashmap_val_bytes(const shmt_hashmap_t *map) { return map ? map->val_bytes : 0; }
int64_t shmt_hashmap_size(const shmt_hashmap_t *map) { return map ? map->n : 0; }
void shmt_hashmap_destroy(shmt_hashmap_t *map) { free(map); }

}  // extern "C"
