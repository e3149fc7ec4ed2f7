// Relabel: distinct values in order of first occurrence + position of every
// input element in that list. Replaces TensorRelabel / RelabelHashmap
// (src/tensor_relabel.cu:68-209 in the ShmTensor tree).
//
// Passes over the N inputs (each a separate launch, no host round trip):
//   fill     table slots {key = -1, first = 0xFFFFFFFF}
//   insert   per-workgroup de-duplication in LDS, then one global insert per
//            distinct id of the tile (64-bit CAS on the key, atomicMin the index)
//   first    first[i] = smallest index holding the same key (kept in the
//            labels buffer); per-tile count of i with first[i] == i
//   partials exclusive scan of the per-tile counts (own launch only beyond 2 M ids)
//   unique   rank of every first occurrence; unique[rank] = key; per 64
//            elements a bitmap of the first occurrences among them and the
//            number of first occurrences before them (RlRanks)
//   labels   labels[i] = rank of element first[i], from that bitmap
// The table is touched only by `insert` and `first`; the last two passes read
// dense arrays. Slots are 16 bytes {int64 key, uint32 first, pad} at load
// factor <= 0.5 with a mixed hash (the reference hashes with the low bits of
// the id, src/tensor_relabel.cu:111-117); ids known to fit 32 bits use the
// same memory as packed 8-byte slots (see rl_packed_insert).
// Up to 8,192 ids all of this is one launch of one workgroup with its table
// in LDS (rl_small_kernel). Beyond 1 M ids (and up to 7.3 M) fill, insert and
// first are replaced by passes that partition the ids by hash and give every
// partition a table in LDS (rp_*_kernel, further down).
#include "common.h"
#include "launchers.h"
#include "scan_dev.h"

#include <atomic>
#include <type_traits>

namespace shmt {

constexpr int kRlBlock = 256;
constexpr int kRlItems = 2;
constexpr int kRlTile = kRlBlock * kRlItems;
constexpr int64_t kRlSelfPrefixTiles = 4096;  // up to 2 M ids the unique pass sums the tile counts itself

// Number of input ids: a host-known part plus, optionally, a part that only
// the device knows (the length of the last segment, e.g. the nnz a sampling
// kernel produced earlier on the same stream).
struct RlCount {
  int64_t fixed;
  const int64_t *fixed_dev;  // when set: the first part is this device-side figure, at most `fixed`
  const void *extra;  // device address of the extra length, or null
  int extra_bytes;    // its width, 4 or 8
  int64_t limit;      // what launches and buffers were sized for; the count is clamped to it
};

__device__ __forceinline__ int64_t rl_count(const RlCount &n) {
  if (!n.extra && !n.fixed_dev) return n.fixed;
  int64_t first = n.fixed;
  if (n.fixed_dev) {
    const int64_t f = *n.fixed_dev;
    first = f < 0 ? 0 : (f < n.fixed ? f : n.fixed);
  }
  int64_t extra = n.extra ? load_int(n.extra, 0, n.extra_bytes) : 0;
  if (extra < 0) extra = 0;
  const int64_t N = first + extra;
  return N < n.limit ? N : n.limit;
}

struct RlSlot {
  int64_t key;
  uint32_t first;
  uint32_t pad;
};
static_assert(sizeof(RlSlot) == 16, "slot must be 16 bytes");

// Table slots for the N ids the scratch buffer is sized for. When N is only an
// upper bound of the id count (fused hop) the whole table is still used:
// measured, the lower load shortens the probe chains of the insert pass by
// more than clearing the smaller table would save.
static int64_t rl_capacity(int64_t N) {
  int64_t cap = 2 * N;
  if (cap < 64) cap = 64;
  return (cap + 7) & ~7ll;
}

struct RlLayout {
  int64_t cap, table_off, rank_off, partial_off, flag_off, total;
};

static RlLayout rl_layout(int64_t N) {
  RlLayout l;
  l.cap = rl_capacity(N);
  l.table_off = 0;
  l.rank_off = l.cap * 16;
  int64_t rank_bytes = (N * 4 + 127) & ~127ll;
  l.partial_off = l.rank_off + rank_bytes;
  int64_t nb = (N + kRlTile - 1) / kRlTile;
  l.flag_off = l.partial_off + ((nb * 8 + 127) & ~127ll);
  l.total = l.flag_off + 128;
  return l;
}

// Claim a slot for `key` and lower its first index to `i`.
__device__ __forceinline__ void rl_global_insert(RlSlot *tbl, uint32_t cap, int64_t key, uint32_t i) {
  uint32_t pos = reduce_range(hash_id(key), cap);
  for (uint32_t probes = 0; probes < cap; ++probes) {
    // Look before the atomics: a stale cached view can only look emptier /
    // larger than the truth, in which case the atomic below settles it.
    const uint4 s = *reinterpret_cast<const uint4 *>(&tbl[pos]);
    const int64_t seen = static_cast<int64_t>((static_cast<uint64_t>(s.y) << 32) | s.x);
    if (seen == key) {
      if (s.z > i) atomicMin(&tbl[pos].first, i);
      return;
    }
    if (seen == -1) {
      unsigned long long prev =
          atomicCAS(reinterpret_cast<unsigned long long *>(&tbl[pos].key), ~0ull,
                    static_cast<unsigned long long>(key));
      if (prev == ~0ull || static_cast<int64_t>(prev) == key) {
        atomicMin(&tbl[pos].first, i);
        return;
      }
    }
    pos = (pos + 1 == cap) ? 0 : pos + 1;
  }
}

// ---- packed table for ids that fit 32 bits --------------------------------
// The same memory seen as 8-byte slots {key : 32 | first index : 32} (twice as
// many of them, so half the load). Key in the high half: one 64-bit atomicMin
// per probe both claims an empty slot (all ones is the maximum) and lowers the
// first index of a slot that already holds the key, where the 16-byte format
// needs a CAS and a separate atomicMin. A smaller entry of another key takes a
// slot over from a larger one; the thread that caused this carries the
// displaced entry on along the probe sequence. Slot values only ever decrease,
// occupied slots never become empty, and an entry moves only across occupied
// slots, so after the kernel every key sits exactly once in the occupied run
// that starts at its home slot, with the smallest index it was inserted with.
constexpr unsigned long long kRlEmpty8 = ~0ull;

// How insert / first address the table: 0 = 16-byte slots, 1 = packed,
// 2 = packed unless *wide_mark equals this call's nonce. The kernel that
// writes the ids earlier on the stream stores the nonce there when it sees an
// id outside [0, 2^32); the mark lives in uninitialised scratch and is never
// cleared: leftover bits can only pass for the nonce by a 2^-64 accident, and
// then the 16-byte format is used, which is correct for every id.
struct RlPath {
  int mode;
  const uint64_t *wide_mark;
  uint64_t nonce;
};

__device__ __forceinline__ bool rl_packed(const RlPath &p) {
  return p.mode == 1 || (p.mode == 2 && *p.wide_mark != p.nonce);
}

__device__ __forceinline__ uint32_t rl_cap8(uint32_t cap) {
  return cap <= 0x7FFFFFFFu ? 2 * cap : cap;
}

__device__ __forceinline__ uint32_t rl_home8(uint32_t key32, uint32_t cap8) {
  return reduce_range(hash_id(static_cast<int64_t>(key32)), cap8);
}

__device__ __forceinline__ void rl_packed_insert(unsigned long long *tbl, uint32_t cap8, uint32_t key32,
                                                 uint32_t i) {
  unsigned long long w = (static_cast<unsigned long long>(key32) << 32) | i;
  uint32_t pos = rl_home8(key32, cap8);
  for (uint32_t probes = 0; probes < cap8; ++probes) {
    // Look before the atomic: a stale cached view can only show a larger value
    // than the truth, in which case the atomic below settles it.
    const unsigned long long seen = tbl[pos];
    if ((seen >> 32) == (w >> 32) && seen <= w) return;  // key present with an index not larger
    if (seen > w) {
      const unsigned long long old = atomicMin(&tbl[pos], w);
      if (old == kRlEmpty8 || (old >> 32) == (w >> 32)) return;  // claimed, or merged with the same key
      if (old > w) w = old;  // took the slot from a larger key: carry that entry on
    }
    pos = (pos + 1 == cap8) ? 0 : pos + 1;
  }
}

constexpr int kRlInsertTile = kRlBlock;          // ids per workgroup pass: one per thread
constexpr int kRlLdsSlots = 2 * kRlInsertTile;   // per-workgroup staging table, load <= 0.5

// Insert pass. Ids of hub nodes repeat thousands of times in a sampled batch,
// and atomics on one address serialise in L2, so every workgroup first
// de-duplicates its 256 ids in an LDS table (key -> smallest index among
// them) and sends one global insert per distinct id, issued by the thread that
// holds the id's smallest index: at most one global probe chain per thread.
struct RlInsertArgs {
  RlSlot *tbl;
  uint32_t cap;
  const void *total;
  int eb;
  RlCount n;
  RlPath path;
};

// (bx, gx): this workgroup's index and the number of workgroups of its job:
// blockIdx.x / gridDim.x of a plain launch, the job's share of a merged one.
__device__ __forceinline__ void rl_insert_body(unsigned bx, unsigned gx, const RlInsertArgs &a) {
  RlSlot *const tbl = a.tbl;
  const uint32_t cap = a.cap;
  const void *const total = a.total;
  const int eb = a.eb;
  const int64_t N = rl_count(a.n);
  const bool packed = rl_packed(a.path);
  __shared__ unsigned long long lkey[kRlLdsSlots];
  __shared__ uint32_t lfirst[kRlLdsSlots];
  // ids that fit 32 bits (the packed table's case) are staged as 32-bit keys: a slot then lies in one LDS
  // bank and the compare-and-swap is a 32-bit one, which halves the staging table's bank conflicts
  uint32_t *const lkey32 = reinterpret_cast<uint32_t *>(lkey);
  const int64_t ntiles = (N + kRlInsertTile - 1) / kRlInsertTile;
  // The staging pays for ids that repeat within a tile. A workgroup that finds next to none in its first
  // tile (a batch without hub nodes: 99.4 % of the ids of the benchmark's largest hop are alone in their
  // tile) sends the ids of its later tiles straight to the table.
  bool staging = true;
  for (int64_t tile = bx; tile < ntiles; tile += gx) {
    if (!staging) {
      const int64_t i = tile * kRlInsertTile + threadIdx.x;
      if (i < N) {
        const int64_t key = load_int(total, i, eb);
        if (packed)
          rl_packed_insert(reinterpret_cast<unsigned long long *>(tbl), rl_cap8(cap),
                           static_cast<uint32_t>(key), static_cast<uint32_t>(i));
        else
          rl_global_insert(tbl, cap, key, static_cast<uint32_t>(i));
      }
      continue;
    }
    for (int t = threadIdx.x; t < kRlLdsSlots; t += kRlBlock) {
      if (packed) lkey32[t] = 0xFFFFFFFFu; else lkey[t] = ~0ull;
      lfirst[t] = 0xFFFFFFFFu;
    }
    __syncthreads();
    const int64_t i = tile * kRlInsertTile + threadIdx.x;
    int64_t key = 0;
    uint32_t pos = 0;
    bool staged = false;  // the id went through the staging table (always, except the one id that looks empty there)
    if (i < N) {
      key = load_int(total, i, eb);
      pos = hash_id(key) & (kRlLdsSlots - 1);
      staged = !(packed && static_cast<uint32_t>(key) == 0xFFFFFFFFu);
      // the staging table has twice as many slots as the tile has ids: a free slot always turns up
      for (int probes = 0; staged && probes < kRlLdsSlots; ++probes) {
        bool mine;
        if (packed) {
          const uint32_t prev = atomicCAS(&lkey32[pos], 0xFFFFFFFFu, static_cast<uint32_t>(key));
          mine = prev == 0xFFFFFFFFu || prev == static_cast<uint32_t>(key);
        } else {
          const unsigned long long prev = atomicCAS(&lkey[pos], ~0ull, static_cast<unsigned long long>(key));
          mine = prev == ~0ull || static_cast<int64_t>(prev) == key;
        }
        if (mine) {
          atomicMin(&lfirst[pos], static_cast<uint32_t>(i));
          break;
        }
        pos = (pos + 1) & (kRlLdsSlots - 1);
      }
    }
    // (also the barrier between staging and reading it back) ids of this tile that another thread inserts
    const int repeats = __syncthreads_count(i < N && staged && lfirst[pos] != static_cast<uint32_t>(i));
    if (tile == static_cast<int64_t>(bx)) staging = repeats * 32 > kRlInsertTile;  // more than 3 % repeats
    // the thread holding the smallest index of an id inserts it for the whole tile:
    // one global probe chain per thread at most
    if (i < N && (!staged || lfirst[pos] == static_cast<uint32_t>(i))) {
      if (packed)
        rl_packed_insert(reinterpret_cast<unsigned long long *>(tbl), rl_cap8(cap),
                         static_cast<uint32_t>(key), static_cast<uint32_t>(i));
      else
        rl_global_insert(tbl, cap, key, static_cast<uint32_t>(i));
    }
    __syncthreads();
  }
}

__global__ __launch_bounds__(kRlBlock) void rl_insert_kernel(RlInsertArgs a) {
  rl_insert_body(blockIdx.x, gridDim.x, a);
}

__global__ __launch_bounds__(kRlBlock) void rl_insert_jobs(Jobs<RlInsertArgs> j) {
  if (blockIdx.x < j.blocks[blockIdx.y]) rl_insert_body(blockIdx.x, j.blocks[blockIdx.y], j.a[blockIdx.y]);
}

// First-occurrence index of every element: one id per thread, a workgroup of
// kRlTile threads per tile (the tile whose count of first occurrences the
// unique pass ranks). One id per thread keeps every value in registers and
// every probe chain in its own lane; with several ids per thread the chains of
// a lane ran one after the other and a small input ran on a handful of
// workgroups.
template <bool PACKED>
__device__ __forceinline__ uint32_t rl_first_of(const RlSlot *tbl, uint32_t cap, int64_t key) {
  if (PACKED) {
    const unsigned long long *tbl8 = reinterpret_cast<const unsigned long long *>(tbl);
    const uint32_t cap8 = rl_cap8(cap);
    const uint32_t key32 = static_cast<uint32_t>(key);
    uint32_t p = rl_home8(key32, cap8);
    for (uint32_t probes = 0; probes < cap8; ++probes) {
      const unsigned long long s8 = tbl8[p];
      if (s8 == kRlEmpty8) break;
      if (static_cast<uint32_t>(s8 >> 32) == key32) return static_cast<uint32_t>(s8);
      p = (p + 1 == cap8) ? 0 : p + 1;
    }
  } else {
    uint32_t p = reduce_range(hash_id(key), cap);
    for (uint32_t probes = 0; probes < cap; ++probes) {
      const uint4 s = *reinterpret_cast<const uint4 *>(&tbl[p]);
      const int64_t k = static_cast<int64_t>((static_cast<uint64_t>(s.y) << 32) | s.x);
      if (k == key) return s.z;
      if (k == -1) break;
      p = (p + 1 == cap) ? 0 : p + 1;
    }
  }
  return 0xFFFFFFFFu;
}

struct RlFirstArgs {
  const RlSlot *tbl;
  uint32_t cap;
  const void *total;
  int eb;
  RlCount n;
  void *labels;
  uint64_t *partials;
  RlPath path;
};

__device__ __forceinline__ void rl_first_body(unsigned bx, const RlFirstArgs &a) {
  const int64_t N = rl_count(a.n);
  // launched for a bound of N: tiles past the ids have nothing to do, and nobody reads their count
  if (static_cast<int64_t>(bx) * kRlTile >= N) return;
  __shared__ uint64_t lds[kRlTile / kWave];
  const int64_t i = static_cast<int64_t>(bx) * kRlTile + threadIdx.x;
  uint64_t cnt = 0;
  if (i < N) {
    const int64_t key = load_int(a.total, i, a.eb);
    const uint32_t f = rl_packed(a.path) ? rl_first_of<true>(a.tbl, a.cap, key) : rl_first_of<false>(a.tbl, a.cap, key);
    store_int(a.labels, i, a.eb, static_cast<int64_t>(f));
    cnt = (f == static_cast<uint32_t>(i));
  }
  uint64_t tile_total;
  block_exclusive_scan<uint64_t, kRlTile>(cnt, lds, &tile_total);
  if (threadIdx.x == 0) a.partials[bx] = tile_total;
}

__global__ __launch_bounds__(kRlTile) void rl_first_kernel(RlFirstArgs a) { rl_first_body(blockIdx.x, a); }

__global__ __launch_bounds__(kRlTile) void rl_first_jobs(Jobs<RlFirstArgs> j) {
  if (blockIdx.x < j.blocks[blockIdx.y]) rl_first_body(blockIdx.x, j.a[blockIdx.y]);
}

// Ranks of the first occurrences, 16 bytes per 64 consecutive elements: bit b of `firsts` says that
// element 64 w + b is the first occurrence of its id, `before` is the number of first occurrences in
// front of element 64 w. The rank of a first occurrence f is before + popcount(firsts below bit f & 63):
// one 16-byte load from an array of N / 4 bytes, which stays in the L2s where an array of one rank per
// element (4 N bytes, read at random positions by the labels pass) did not.
struct RlRanks {
  uint64_t firsts;
  uint32_t before;
  uint32_t pad;
};
static_assert(sizeof(RlRanks) == 16, "one 16-byte load per lookup");
static_assert(kRlTile % kWave == 0 && kRlItems * kWave * (kRlBlock / kWave) == kRlTile, "a wave ranks whole 64-element words");

struct RlUniqueArgs {
  const void *total;
  int eb;
  RlCount n;
  const void *first;  // first-occurrence index of every element, fb bytes wide (the labels buffer, or an array of its own)
  int fb;
  const uint64_t *partials;
  void *unique_out;
  RlRanks *ranks;
  int64_t *count_out;
  int64_t *count_copy;
  int scanned;             // 0: partials are raw tile counts, 1: scanned, 2: raw, with the sums of whole groups in `coarse`
  const uint32_t *coarse;  // scanned == 2: coarse[g] = sum of the counts of tiles [g * group, (g + 1) * group)
  int group;
};

__device__ __forceinline__ void rl_unique_body(unsigned bx, const RlUniqueArgs &a) {
  const void *const total = a.total;
  const int eb = a.eb;
  const void *const labels = a.first;
  const uint64_t *const partials = a.partials;
  void *const unique_out = a.unique_out;
  const int64_t N = rl_count(a.n);
  // launched for a bound of N: only the tiles that hold ids work (tile 0 reports N = 0)
  if (bx > 0 && static_cast<int64_t>(bx) * kRlTile >= N) return;
  __shared__ uint32_t wave_firsts[kRlBlock / kWave];
  __shared__ uint64_t lds64[kRlBlock / kWave];
  // Tile prefix: either already scanned by a separate launch, or (few tiles)
  // summed here from the raw per-tile counts.
  uint64_t tile_prefix;
  if (a.scanned == 1) {
    tile_prefix = partials[bx];
  } else {
    uint64_t part = 0;
    int from = 0;
    if (a.scanned == 2) {
      const int groups = static_cast<int>(bx) / a.group;
      for (int t = threadIdx.x; t < groups; t += kRlBlock) part += a.coarse[t];
      from = groups * a.group;
    }
    for (int t = from + threadIdx.x; t < static_cast<int>(bx); t += kRlBlock) part += partials[t];
    uint64_t below;
    block_exclusive_scan<uint64_t, kRlBlock>(part, lds64, &below);
    tile_prefix = below;
  }
  // a wave takes kRlItems words of 64 consecutive elements: element = word start + lane
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  const int64_t wave_first = static_cast<int64_t>(bx) * kRlTile + static_cast<int64_t>(wave) * (kRlItems * kWave);
  bool win[kRlItems], ok[kRlItems];
  int64_t idx[kRlItems], lab[kRlItems], val[kRlItems];
#pragma unroll
  for (int j = 0; j < kRlItems; ++j) {
    idx[j] = wave_first + j * kWave + lane;
    ok[j] = idx[j] < N;
    lab[j] = -1;
    val[j] = 0;
  }
  load_ints<kRlItems>(labels, idx, ok, a.fb, lab);
  uint64_t firsts[kRlItems];
  uint32_t mine = 0;  // first occurrences of this wave
#pragma unroll
  for (int j = 0; j < kRlItems; ++j) {
    win[j] = ok[j] && lab[j] == idx[j];
    firsts[j] = __builtin_amdgcn_ballot_w64(win[j]);
    mine += static_cast<uint32_t>(__builtin_popcountll(firsts[j]));
  }
  load_ints<kRlItems>(total, idx, win, eb, val);
  if (lane == 0) wave_firsts[wave] = mine;
  __syncthreads();
  uint32_t before_wave = 0, tile_total = 0;
#pragma unroll
  for (int w = 0; w < kRlBlock / kWave; ++w) {
    const uint32_t c = wave_firsts[w];
    if (w < wave) before_wave += c;
    tile_total += c;
  }
  uint64_t word_rank = tile_prefix + before_wave;  // rank of the first first-occurrence of the word
  const uint64_t below_lane = (1ull << lane) - 1ull;
#pragma unroll
  for (int j = 0; j < kRlItems; ++j) {
    if (win[j])
      store_int(unique_out, static_cast<int64_t>(word_rank + __builtin_popcountll(firsts[j] & below_lane)), eb, val[j]);
    const int64_t word_start = wave_first + j * kWave;
    if (lane == 0 && word_start < N) a.ranks[word_start / kWave] = RlRanks{firsts[j], static_cast<uint32_t>(word_rank), 0u};
    word_rank += static_cast<uint64_t>(__builtin_popcountll(firsts[j]));
  }
  // the workgroup holding the last id reports the number of distinct ids
  const int64_t last_tile = N > 0 ? (N - 1) / kRlTile : 0;
  if (static_cast<int64_t>(bx) == last_tile && threadIdx.x == 0) {
    if (a.count_copy) *a.count_copy = static_cast<int64_t>(tile_prefix + tile_total);
    publish_size(a.count_out, static_cast<int64_t>(tile_prefix + tile_total));
  }
}

__global__ __launch_bounds__(kRlBlock) void rl_unique_kernel(RlUniqueArgs a) { rl_unique_body(blockIdx.x, a); }

__global__ __launch_bounds__(kRlBlock) void rl_unique_jobs(Jobs<RlUniqueArgs> j) {
  if (blockIdx.x < j.blocks[blockIdx.y]) rl_unique_body(blockIdx.x, j.a[blockIdx.y]);
}

struct RlLabelsArgs {
  void *labels;
  int eb;
  RlCount n;
  const RlRanks *ranks;
  const void *first;  // see RlUniqueArgs
  int fb;
};

__device__ __forceinline__ void rl_labels_body(unsigned bx, unsigned gx, const RlLabelsArgs &a) {
  const int64_t N = rl_count(a.n);
  int64_t i = static_cast<int64_t>(bx) * blockDim.x + threadIdx.x;
  const int64_t stride = static_cast<int64_t>(gx) * blockDim.x;
  for (; i < N; i += stride) {
    const int64_t f = load_int(a.first, i, a.fb);
    const uint4 r = *reinterpret_cast<const uint4 *>(&a.ranks[f >> 6]);
    const uint64_t firsts = (static_cast<uint64_t>(r.y) << 32) | r.x;
    const uint32_t rank = r.z + static_cast<uint32_t>(__builtin_popcountll(firsts & ((1ull << (f & 63)) - 1ull)));
    store_int(a.labels, i, a.eb, static_cast<int64_t>(rank));
  }
}

__global__ __launch_bounds__(256) void rl_labels_kernel(RlLabelsArgs a) {
  rl_labels_body(blockIdx.x, gridDim.x, a);
}

__global__ __launch_bounds__(256) void rl_labels_jobs(Jobs<RlLabelsArgs> j) {
  if (blockIdx.x < j.blocks[blockIdx.y]) rl_labels_body(blockIdx.x, j.blocks[blockIdx.y], j.a[blockIdx.y]);
}

struct RlSegments {
  const void *ptr[SHMT_RELABEL_MAX_SEGMENTS];
  int64_t start[SHMT_RELABEL_MAX_SEGMENTS + 1];  // start[s] = first index of segment s in total
  int bytes[SHMT_RELABEL_MAX_SEGMENTS];
  int n;
};

// First pass when the input arrives as segments: empties the table and writes
// the concatenated, widened ids in one sweep (both are streaming stores).
__global__ __launch_bounds__(256) void rl_fill_concat_kernel(uint4 *tbl16, int64_t cap, RlSegments segs,
                                                             void *total, int eb, RlCount n,
                                                             uint64_t *wide_mark, uint64_t nonce) {
  const int64_t N = rl_count(n);
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t span = cap > N ? cap : N;
  const uint4 ones = make_uint4(~0u, ~0u, ~0u, ~0u);
  for (; i < span; i += stride) {
    if (i < cap) tbl16[i] = ones;
    if (i < N) {
      int sgm = 0;
      while (sgm + 1 < segs.n && i >= segs.start[sgm + 1]) ++sgm;
      const int64_t id = load_int(segs.ptr[sgm], i - segs.start[sgm], segs.bytes[sgm]);
      store_int(total, i, eb, id);
      if (static_cast<uint64_t>(id) >> 32) *wide_mark = nonce;
    }
  }
}

// ---- small inputs: one workgroup, table in LDS -----------------------------
// Up to kRlSmallMax ids the five passes are one launch: the ids and an index
// table (slot = smallest index seen for the key that claimed it; keys are
// compared through the LDS copy of the ids, so any id width works) live in
// the workgroup's LDS, the grid-wide dependencies between the passes become
// workgroup barriers, and no global atomic is issued. The table memory is
// reused for the rank array once every first occurrence is known.
constexpr int kRlSmallMax = 8192;
constexpr int kRlSmallBlock = 1024;
constexpr int kRlSmallItems = kRlSmallMax / kRlSmallBlock;
constexpr int kRlSmallSlots = 2 * kRlSmallMax;
static_assert(kRlSmallItems == 8, "the rank scan packs eight 16-bit counters into two words");

struct RlSmallArgs {
  const void *total_in;  // the ids (SEGS = false)
  void *total_out;       // receives the concatenated ids (SEGS = true)
  int eb;
  RlCount n;
  void *unique_out;
  void *labels_out;
  int64_t *count_out;
  int64_t *count_copy;
};

template <bool SEGS>
__device__ __forceinline__ void rl_small_body(const RlSmallArgs &a, const RlSegments &segs) {
  const void *const total_in = a.total_in;
  void *const total_out = a.total_out;
  const int eb = a.eb;
  const RlCount n = a.n;
  void *const unique_out = a.unique_out;
  void *const labels_out = a.labels_out;
  int64_t *const count_out = a.count_out;
  int64_t *const count_copy = a.count_copy;
  __shared__ int64_t keys[kRlSmallMax];
  __shared__ uint32_t tbl[kRlSmallSlots];
  __shared__ uint64_t scan_lds[kRlSmallBlock / kWave];
  const int N = static_cast<int>(rl_count(n));
  const int t = threadIdx.x;
  for (int p = t; p < kRlSmallSlots; p += kRlSmallBlock) tbl[p] = 0xFFFFFFFFu;
  // element i = j * kRlSmallBlock + t: coalesced loads and stores for every j
  int64_t id[kRlSmallItems];
#pragma unroll
  for (int j = 0; j < kRlSmallItems; ++j) {
    const int i = j * kRlSmallBlock + t;
    id[j] = 0;
    if (i < N) {
      if (SEGS) {
        int sgm = 0;
        while (sgm + 1 < segs.n && i >= segs.start[sgm + 1]) ++sgm;
        id[j] = load_int(segs.ptr[sgm], i - segs.start[sgm], segs.bytes[sgm]);
        store_int(total_out, i, eb, id[j]);
      } else {
        id[j] = load_int(total_in, i, eb);
      }
      keys[i] = id[j];
    }
  }
  __syncthreads();
  // insert: claim the first free slot of the probe sequence with the element's index, or lower the
  // index of the slot that already stands for the same key. One workgroup on one compute unit is bound by
  // the latency of its dependent LDS accesses, so the first probes of a thread's eight elements are made side
  // by side (look, claim, compare, lower: four round trips for all eight instead of up to four each), and
  // only an element that meets another id at its home slot walks on alone. A key never leaves its slot:
  // where it sits is kept for the next phase.
  uint32_t slot[kRlSmallItems], cur[kRlSmallItems];
  bool open[kRlSmallItems];
#pragma unroll
  for (int j = 0; j < kRlSmallItems; ++j) {
    const uint32_t i = j * kRlSmallBlock + t;
    open[j] = static_cast<int>(i) < N;
    slot[j] = hash_id(id[j]) & (kRlSmallSlots - 1);
    cur[j] = open[j] ? tbl[slot[j]] : 0u;
  }
#pragma unroll
  for (int j = 0; j < kRlSmallItems; ++j) {
    const uint32_t i = j * kRlSmallBlock + t;
    if (open[j] && cur[j] == 0xFFFFFFFFu) {
      cur[j] = atomicCAS(&tbl[slot[j]], 0xFFFFFFFFu, i);
      if (cur[j] == 0xFFFFFFFFu) open[j] = false;  // claimed
    }
  }
  int64_t there[kRlSmallItems];
#pragma unroll
  for (int j = 0; j < kRlSmallItems; ++j) there[j] = open[j] ? keys[cur[j]] : 0;
#pragma unroll
  for (int j = 0; j < kRlSmallItems; ++j) {
    const uint32_t i = j * kRlSmallBlock + t;
    if (!open[j]) continue;
    if (there[j] == id[j]) {
      if (cur[j] > i) atomicMin(&tbl[slot[j]], i);
      continue;
    }
    uint32_t p = (slot[j] + 1) & (kRlSmallSlots - 1);
    for (int probes = 1; probes < kRlSmallSlots; ++probes) {
      uint32_t c = tbl[p];
      if (c == 0xFFFFFFFFu) {
        c = atomicCAS(&tbl[p], 0xFFFFFFFFu, i);
        if (c == 0xFFFFFFFFu) break;
      }
      if (keys[c] == id[j]) {
        if (c > i) atomicMin(&tbl[p], i);
        break;
      }
      p = (p + 1) & (kRlSmallSlots - 1);
    }
    slot[j] = p;
  }
  __syncthreads();
  // first occurrence of every element: what its key's slot holds now; count the elements that are their own
  // first occurrence, eight 16-bit counters (one per j) packed into two words
  uint32_t first[kRlSmallItems];
  uint64_t lo = 0, hi = 0;
#pragma unroll
  for (int j = 0; j < kRlSmallItems; ++j) {
    const uint32_t i = j * kRlSmallBlock + t;
    first[j] = static_cast<int>(i) < N ? tbl[slot[j]] : 0xFFFFFFFFu;
  }
#pragma unroll
  for (int j = 0; j < kRlSmallItems; ++j) {
    const uint32_t i = j * kRlSmallBlock + t;
    if (static_cast<int>(i) < N) {
      const uint64_t win = first[j] == i;
      if (j < 4) lo += win << (16 * j); else hi += win << (16 * (j - 4));
    }
  }
  // index order is j-major: rank = (winners of all smaller j) + (winners of this j in threads below)
  uint64_t tot_lo, tot_hi;
  const uint64_t ex_lo = block_exclusive_scan<uint64_t, kRlSmallBlock>(lo, scan_lds, &tot_lo);
  const uint64_t ex_hi = block_exclusive_scan<uint64_t, kRlSmallBlock>(hi, scan_lds, &tot_hi);
  // (the scans' barriers also mean every thread is done with the table: it becomes rank_of)
  uint32_t below = 0;
#pragma unroll
  for (int j = 0; j < kRlSmallItems; ++j) {
    const uint32_t i = j * kRlSmallBlock + t;
    const uint64_t ex = j < 4 ? ex_lo >> (16 * j) : ex_hi >> (16 * (j - 4));
    const uint64_t tot = j < 4 ? tot_lo >> (16 * j) : tot_hi >> (16 * (j - 4));
    if (static_cast<int>(i) < N && first[j] == i) {
      const uint32_t rank = below + static_cast<uint32_t>(ex & 0xFFFF);
      store_int(unique_out, rank, eb, id[j]);
      tbl[i] = rank;
    }
    below += static_cast<uint32_t>(tot & 0xFFFF);
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kRlSmallItems; ++j) {
    const int i = j * kRlSmallBlock + t;
    if (i < N) store_int(labels_out, i, eb, static_cast<int64_t>(tbl[first[j]]));
  }
  if (t == 0) {
    if (count_copy) *count_copy = static_cast<int64_t>(below);
    publish_size(count_out, static_cast<int64_t>(below));
  }
}

__global__ __launch_bounds__(kRlSmallBlock) void rl_small_segments_kernel(RlSmallArgs a, RlSegments segs) {
  rl_small_body<true>(a, segs);
}

__global__ __launch_bounds__(kRlSmallBlock) void rl_small_kernel(RlSmallArgs a) {
  rl_small_body<false>(a, RlSegments{});
}

__global__ __launch_bounds__(kRlSmallBlock) void rl_small_jobs(Jobs<RlSmallArgs> j) {
  rl_small_body<false>(j.a[blockIdx.y], RlSegments{});
}

__global__ void rl_zero_count_kernel(int64_t *count_out, int64_t *count_copy) {
  if (count_copy) *count_copy = 0;
  publish_size(count_out, 0);
}

// ---- large inputs: partition by hash, one workgroup per bin, table in LDS --------
// The insert and first-occurrence passes above touch a random line of a table
// that no cache holds once per id and pass, and the part moves such lines at
// 50 G per second whatever the kernel does (3.1 M ids: 74 + 54 us, plus 22 us to
// empty the table). From a million ids on (kRpExactMin; kRpDefaultMin for a
// hop sized by a loose bound, kRpMergedMin for hops that share their launches)
// the same two results -- the first-occurrence index of every element and the
// number of first occurrences per tile of kRlTile ids -- come from five passes
// that read and write memory in runs instead:
//   count    a workgroup per tile of kRpTile ids: histogram of the ids over P
//            bins (bin = top bits of the id's hash), one column of the P x W
//            matrix; ids that repeat within the tile are counted once
//   rows     exclusive prefix along every row of the matrix, bin totals
//   scatter  a workgroup per tile again: record {id, index} of every element
//            to its bin's run for this tile (bins are contiguous, runs in tile
//            order), through LDS so that a run is written by consecutive
//            lanes; per element the place of its record among the tile's
//   bins     a workgroup per bin: smallest index per id through a table in
//            LDS (the low bits of the hash address it), written per record
//   gather   a workgroup per tile: the results of its runs, read through LDS
//            the same way, handed to the elements: first[i], 4 bytes each
// Few, large bins: a tile's run for a bin should span whole lines (8,192 ids
// over 256 bins: 32 records; measured on 3.1 M ids, scatter / gather 24 / 14 us
// with 256 bins, 31 / 17 us with 1,024, and 42 / 29 us before the runs went
// through LDS).
// P = 256 up to 3.67 M ids, 512 up to 7.34 M (a bin's table is at most 7/8 full
// when every id of the input is distinct); larger inputs keep the table in memory.
// A bin's table has 4,096 to 16,384 slots (half for ids beyond 32 bits), two
// per id the bin can hold when all of the input's are distinct as far as
// that goes, in workgroups of 256 to 1,024 threads; the ids of a bin that do not fit (more
// than that many distinct ones, or ids crafted to collide) are worked through
// in 2, 4, ... rounds over classes of a second hash, and by comparing all
// pairs when 2^kRpMaxRoundsLog2 rounds do not do: slower, never wrong. Records are {id : 32 | index : 32} when the ids fit 32
// bits and 16 bytes otherwise; everything lives in the memory the table in
// memory would have had.
constexpr int kRpBlock = 1024;
constexpr int kRpSlotsLog2 = 14;     // 16,384 slots of 4 + 4 bytes = 128 KB of LDS
constexpr int kRpMinBinsLog2 = 8, kRpMaxBinsLog2 = 9;
constexpr int64_t kRpBinIds = 14336; // ids per bin from which on the number of bins grows: 7/8 of the largest table
constexpr int64_t kRpTile = 8192;    // ids per tile of the count / scatter / gather passes
constexpr int kRpMaxRoundsLog2 = 10;
constexpr int64_t kRpDefaultMin = kRlSelfPrefixTiles * kRlTile + 1;
// Hops that share their launches with those of other batches (launchers.h) are sized for a bound of their
// ids, and the five passes' fixed costs are paid once for all of them: from this bound and this many jobs on
// they take the partition passes as well.
constexpr int64_t kRpMergedMin = 512 * 1024;
// A call that knows its number of ids (not merely a loose bound of it) gains from about a million on.
constexpr int64_t kRpExactMin = 1024 * 1024;
constexpr int kRpMergedMinJobs = 4;
constexpr int kRpMinSlotsLog2 = 12;  // smallest table a bin pass is compiled for

struct RpTuning {
  int64_t min_ids, min_ids_merged;
  int slots_log2, max_rounds_log2;
};
static RpTuning g_rp_tuning{kRpDefaultMin, kRpMergedMin, kRpSlotsLog2, kRpMaxRoundsLog2};

struct RpPlan {
  bool ok;
  int log2P;
  int table_log2;  // which compiled table size the bin pass uses (the tuning may use less of it)
  uint32_t P, W;
  int64_t rec_off, first_off, firstp_off, local_off, hist_off, bintot_off, binstart_off, coarse_off, tile_off, end;
};

// Where the partition passes keep their arrays inside the table memory (16 * cap bytes) of a
// scratch buffer sized for N ids; ok = false when N is outside the range this path serves.
static RpPlan rp_plan(int64_t N, int merged_jobs = 0, bool loose = false) {
  RpPlan p{};
  const bool merged = merged_jobs >= kRpMergedMinJobs;
  if (merged_jobs > 0 && !merged) return p;
  const int64_t exact_min = g_rp_tuning.min_ids < kRpExactMin ? g_rp_tuning.min_ids : kRpExactMin;
  if (N < (merged ? g_rp_tuning.min_ids_merged : (loose ? g_rp_tuning.min_ids : exact_min)) || N <= kRlSmallMax) return p;
  int lg = kRpMinBinsLog2;
  while ((kRpBinIds << lg) < N) ++lg;
  if (lg > kRpMaxBinsLog2) return p;
  p.log2P = lg;
  p.P = 1u << lg;
  p.W = static_cast<uint32_t>((N + kRpTile - 1) / kRpTile);
  // two slots per id the bin may hold if every id of the input is distinct, as far as the largest table goes;
  // when N is a loose bound of the id count (a chained hop: typically three times what turns up) a quarter of
  // that, a bin that does get more taking two rounds
  p.table_log2 = kRpMinSlotsLog2;
  while (p.table_log2 < kRpSlotsLog2 && (static_cast<int64_t>(p.P) << p.table_log2) < (loose ? N / 2 : 2 * N)) ++p.table_log2;
  auto up = [](int64_t x) { return (x + 255) & ~255ll; };
  p.rec_off = 0;
  p.first_off = up(16 * N);
  p.firstp_off = p.first_off + up(4 * N);
  p.local_off = p.firstp_off + up(4 * N);
  p.hist_off = p.local_off + up(2 * N);
  p.bintot_off = p.hist_off + up(4ll * p.P * p.W);
  p.binstart_off = p.bintot_off + up(4ll * p.P);
  p.coarse_off = p.binstart_off + up(4ll * (p.P + 1));
  p.tile_off = p.coarse_off + up(4ll * p.W);
  p.end = p.tile_off + up(8ll * p.W * (p.P + 1));
  p.ok = p.end <= rl_capacity(N) * 16;
  return p;
}

struct RpArgs {
  const void *total;
  int eb;
  RlCount n;
  RlPath path;
  uint64_t *wide_mark;  // == path.wide_mark, writable: the count pass sets it itself
  int log2P;
  uint32_t W;
  void *rec;
  uint32_t *first;   // first-occurrence index of every element (what the unique and labels passes read)
  uint32_t *firstp;  // the same per record, in the records' order
  uint32_t *hist, *bintot, *binstart, *coarse;
  uint16_t *local;  // position of every element's record among its tile's records in bin order
  uint32_t *tile_runs;  // per tile: where its run of every bin starts in memory (P words), then among its records (P + 1 words)
  uint64_t *partials;
  int slots_log2, max_rounds_log2;
};

// A second hash of the id, independent of hash_id(): ids that collide there spread here.
__device__ __forceinline__ uint32_t rp_class(int64_t key) {
  return hash_id(static_cast<int64_t>(static_cast<uint64_t>(key) * 0x9E3779B97F4A7C15ull + 0xD6E8FEB86659FD93ull));
}

constexpr int kRpItems = static_cast<int>(kRpTile / kRpBlock);  // ids a thread keeps in flight
static_assert(kRpItems * kRpBlock == kRpTile && kRpTile % kRlTile == 0, "tiles are whole chunks of kRpTile ids");

// The ids of one chunk of kRpTile, element j * kRpBlock + t for thread t: all loads issued before any is used.
__device__ __forceinline__ void rp_load_chunk(const RpArgs &a, int64_t base, int64_t hi, int64_t (&idx)[kRpItems],
                                              bool (&ok)[kRpItems], int64_t (&key)[kRpItems]) {
#pragma unroll
  for (int j = 0; j < kRpItems; ++j) {
    idx[j] = base + j * kRpBlock + threadIdx.x;
    ok[j] = idx[j] < hi;
    key[j] = 0;
  }
  load_ints<kRpItems>(a.total, idx, ok, a.eb, key);
}

// Repeats within a tile. Ids of hub nodes come thousands of times in a sampled batch and would all land in
// one bin; within a tile only the occurrence with the smallest index becomes a record, and the others take
// over its position (and so its result) in the scatter pass. Found through a small direct-mapped table:
// slot = low bits of the hash, value = {index | low 32 bits of the id} of the element with the smallest index
// that maps there, so an id that comes often is the likely owner of its slot. An element is covered when
// the slot names an earlier element of the same id; an id that shares its slot with an earlier one of
// another id is simply not de-duplicated. The table's final content depends on the tile alone, so the
// count and the scatter pass decide alike.
constexpr int kRpDedupSlots = 2048;

__device__ __forceinline__ unsigned long long rp_dedup_word(int64_t key, int64_t idx) {
  return (static_cast<unsigned long long>(static_cast<uint32_t>(idx)) << 32) | static_cast<uint32_t>(key);
}

__device__ __forceinline__ void rp_dedup_clear(unsigned long long *dedup) {
  for (int t = threadIdx.x; t < kRpDedupSlots; t += kRpBlock) dedup[t] = ~0ull;
}

__device__ __forceinline__ bool rp_covered(const RpArgs &a, const unsigned long long *dedup, int64_t key,
                                           int64_t idx, uint32_t hash) {
  const unsigned long long v = dedup[hash & (kRpDedupSlots - 1)];
  if (static_cast<uint32_t>(v) != static_cast<uint32_t>(key) || static_cast<uint32_t>(v >> 32) == static_cast<uint32_t>(idx))
    return false;
  // same low half: 4-byte ids are then equal, 8-byte ids are compared in full
  return a.eb == 4 || static_cast<const int64_t *>(a.total)[static_cast<uint32_t>(v >> 32)] == key;
}

// SEGS: the ids are still in the caller's segments; the pass also writes their concatenation (`total`), so
// that no launch of its own reads and writes every id just for that.
template <bool SEGS>
__device__ __forceinline__ void rp_count_body(unsigned bx, const RpArgs &a, const RlSegments &segs) {
  extern __shared__ uint32_t hist[];  // P counters
  __shared__ unsigned long long dedup[kRpDedupSlots];
  const int64_t N = rl_count(a.n);
  const uint32_t P = 1u << a.log2P;
  const int64_t lo = static_cast<int64_t>(bx) * kRpTile;
  if (lo >= N) {
    // launched for a bound of N: a tile past the ids has an empty column
    for (uint32_t b = threadIdx.x; b < P; b += kRpBlock) a.hist[static_cast<size_t>(b) * a.W + bx] = 0;
    return;
  }
  for (uint32_t b = threadIdx.x; b < P; b += kRpBlock) hist[b] = 0;
  rp_dedup_clear(dedup);
  __syncthreads();
  const int64_t hi = lo + kRpTile < N ? lo + kRpTile : N;
  int64_t idx[kRpItems], key[kRpItems];
  bool ok[kRpItems];
  uint32_t hash[kRpItems];
  if (SEGS) {
    // as a rule a tile lies within one segment: one pointer and one width for all its loads
    int first_seg = 0, last_seg = 0;
    while (first_seg + 1 < segs.n && lo >= segs.start[first_seg + 1]) ++first_seg;
    while (last_seg + 1 < segs.n && hi - 1 >= segs.start[last_seg + 1]) ++last_seg;
#pragma unroll
    for (int j = 0; j < kRpItems; ++j) {
      idx[j] = lo + j * kRpBlock + threadIdx.x;
      ok[j] = idx[j] < hi;
      key[j] = 0;
    }
    if (first_seg == last_seg) {
      int64_t at[kRpItems];
#pragma unroll
      for (int j = 0; j < kRpItems; ++j) at[j] = idx[j] - segs.start[first_seg];
      load_ints<kRpItems>(segs.ptr[first_seg], at, ok, segs.bytes[first_seg], key);
    } else {
#pragma unroll
      for (int j = 0; j < kRpItems; ++j) {
        if (!ok[j]) continue;
        int sgm = first_seg;
        while (sgm < last_seg && idx[j] >= segs.start[sgm + 1]) ++sgm;
        key[j] = load_int(segs.ptr[sgm], idx[j] - segs.start[sgm], segs.bytes[sgm]);
      }
    }
#pragma unroll
    for (int j = 0; j < kRpItems; ++j)
      if (ok[j]) store_int(const_cast<void *>(a.total), idx[j], a.eb, key[j]);
    // the repeats test below reads ids of this tile back from `total`
    __syncthreads();
  } else {
    rp_load_chunk(a, lo, hi, idx, ok, key);
  }
  bool wide = false;
#pragma unroll
  for (int j = 0; j < kRpItems; ++j) {
    hash[j] = hash_id(key[j]);
    if (ok[j]) {
      wide |= (static_cast<uint64_t>(key[j]) >> 32) != 0;
      atomicMin(&dedup[hash[j] & (kRpDedupSlots - 1)], rp_dedup_word(key[j], idx[j]));
    }
  }
  if (wide && a.path.mode == 2) *a.wide_mark = a.path.nonce;
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kRpItems; ++j)
    if (ok[j] && !rp_covered(a, dedup, key[j], idx[j], hash[j])) atomicAdd(&hist[hash[j] >> (32 - a.log2P)], 1u);
  __syncthreads();
  for (uint32_t b = threadIdx.x; b < P; b += kRpBlock) a.hist[static_cast<size_t>(b) * a.W + bx] = hist[b];
}

__global__ __launch_bounds__(kRpBlock) void rp_count_kernel(RpArgs a) {
  rp_count_body<false>(blockIdx.x, a, RlSegments{});
}

__global__ __launch_bounds__(kRpBlock) void rp_count_segments_kernel(RpArgs a, RlSegments segs) {
  rp_count_body<true>(blockIdx.x, a, segs);
}

__global__ __launch_bounds__(kRpBlock) void rp_count_jobs(Jobs<RpArgs> j) {
  if (blockIdx.x < j.blocks[blockIdx.y]) rp_count_body<false>(blockIdx.x, j.a[blockIdx.y], RlSegments{});
}

// One wave per bin: the row's counts become the offsets of the tiles' runs inside the bin.
__device__ __forceinline__ void rp_rows_body(unsigned bx, const RpArgs &a) {
  const uint32_t b = bx * (256 / kWave) + threadIdx.x / kWave;
  if (b >= (1u << a.log2P)) return;
  uint32_t *const row = a.hist + static_cast<size_t>(b) * a.W;
  const uint32_t lane = lane_id();
  uint32_t carry = 0;
  for (uint32_t w0 = 0; w0 < a.W; w0 += kWave) {
    const uint32_t w = w0 + lane;
    const uint32_t v = w < a.W ? row[w] : 0u;
    const uint32_t inc = wave_inclusive_scan(v);
    if (w < a.W) row[w] = carry + inc - v;
    carry += wave_last(inc);
  }
  if (lane == 0) a.bintot[b] = carry;
}

__global__ __launch_bounds__(256) void rp_rows_kernel(RpArgs a) { rp_rows_body(blockIdx.x, a); }

__global__ __launch_bounds__(256) void rp_rows_jobs(Jobs<RpArgs> j) {
  if (blockIdx.x < j.blocks[blockIdx.y]) rp_rows_body(blockIdx.x, j.a[blockIdx.y]);
}

// The id a packed record stands for, as the count pass hashed it (4-byte ids are signed).
__device__ __forceinline__ int64_t rp_packed_key(unsigned long long rec, int eb) {
  const uint32_t k = static_cast<uint32_t>(rec >> 32);
  return eb == 4 ? static_cast<int64_t>(static_cast<int32_t>(k)) : static_cast<int64_t>(k);
}

// Scattered 8-byte stores cost one L2 transaction each and leave half-filled lines behind; the records of a
// tile are therefore put in bin order in LDS first (position = start of the bin among the tile's records +
// rank within the bin) and written out from there, consecutive lanes to consecutive addresses of a run.
// 16-byte records (ids beyond 32 bits) do not fit the LDS and are stored directly.
__device__ __forceinline__ void rp_scatter_body(unsigned bx, const RpArgs &a) {
  extern __shared__ uint32_t words[];  // run start in memory, record count, start among the tile's records: P (+ 1) each
  __shared__ unsigned long long stage[kRpTile];  // first the de-duplication table and the ranks of its owners
  __shared__ uint32_t scan_lds[kRpBlock / kWave];
  const int64_t N = rl_count(a.n);
  const uint32_t P = 1u << a.log2P;
  // launched for a bound of N: a tile past the ids has nothing to scatter (tile 0 also publishes the bin starts)
  if (bx > 0 && static_cast<int64_t>(bx) * kRpTile >= N) return;
  uint32_t *const run_at = words, *const cnt = words + P, *const lstart = words + 2 * P;
  unsigned long long *const dedup = stage;
  uint32_t *const rep_rank = reinterpret_cast<uint32_t *>(stage + kRpDedupSlots);
  static_assert(kRpDedupSlots * 12 <= kRpTile * 8, "table and ranks fit the staging memory");
  rp_dedup_clear(dedup);
  // where every bin starts: thread t sums `per` consecutive bin totals
  const uint32_t per = P > kRpBlock ? P / kRpBlock : 1u;
  const uint32_t b0 = threadIdx.x * per;
  uint32_t sum = 0;
  for (uint32_t j = 0; j < per; ++j)
    if (b0 + j < P) sum += a.bintot[b0 + j];
  uint32_t all;
  uint32_t run = block_exclusive_scan<uint32_t, kRpBlock>(sum, scan_lds, &all);
  for (uint32_t j = 0; j < per; ++j) {
    const uint32_t b = b0 + j;
    if (b < P) {
      run_at[b] = run + a.hist[static_cast<size_t>(b) * a.W + bx];
      cnt[b] = 0;
      if (bx == 0) a.binstart[b] = run;
      run += a.bintot[b];
    }
  }
  if (bx == 0 && threadIdx.x == 0) a.binstart[P] = all;
  __syncthreads();
  const bool packed = rl_packed(a.path);
  const int64_t lo = static_cast<int64_t>(bx) * kRpTile;
  const int64_t hi = lo + kRpTile < N ? lo + kRpTile : N;
  int64_t idx[kRpItems], key[kRpItems];
  bool ok[kRpItems];
  uint32_t hash[kRpItems], rank[kRpItems];
  rp_load_chunk(a, lo, hi, idx, ok, key);
#pragma unroll
  for (int j = 0; j < kRpItems; ++j) {
    hash[j] = hash_id(key[j]);
    if (ok[j]) atomicMin(&dedup[hash[j] & (kRpDedupSlots - 1)], rp_dedup_word(key[j], idx[j]));
  }
  __syncthreads();
  bool covered[kRpItems];
#pragma unroll
  for (int j = 0; j < kRpItems; ++j) {
    covered[j] = ok[j] && rp_covered(a, dedup, key[j], idx[j], hash[j]);
    rank[j] = 0;
    if (ok[j] && !covered[j]) {
      rank[j] = atomicAdd(&cnt[hash[j] >> (32 - a.log2P)], 1u);
      // the element a slot names tells the ones it covers (same id, so same bin) where its record goes
      if (dedup[hash[j] & (kRpDedupSlots - 1)] == rp_dedup_word(key[j], idx[j])) rep_rank[hash[j] & (kRpDedupSlots - 1)] = rank[j];
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kRpItems; ++j)
    if (covered[j]) rank[j] = rep_rank[hash[j] & (kRpDedupSlots - 1)];
  // start of every bin among the tile's records (the scan's barriers also end the use of the table)
  {
    uint32_t part = 0;
    for (uint32_t j = 0; j < per; ++j)
      if (b0 + j < P) part += cnt[b0 + j];
    uint32_t records;
    uint32_t at = block_exclusive_scan<uint32_t, kRpBlock>(part, scan_lds, &records);
    for (uint32_t j = 0; j < per; ++j) {
      const uint32_t b = b0 + j;
      if (b < P) {
        lstart[b] = at;
        at += cnt[b];
      }
    }
    if (threadIdx.x == 0) lstart[P] = records;
  }
  __syncthreads();
  uint32_t *const runs = a.tile_runs + static_cast<size_t>(bx) * (2 * P + 1);
  for (uint32_t t = threadIdx.x; t < 2 * P + 1; t += kRpBlock) runs[t] = t < P ? run_at[t] : lstart[t - P];
#pragma unroll
  for (int j = 0; j < kRpItems; ++j) {
    if (!ok[j]) continue;
    const uint32_t bin = hash[j] >> (32 - a.log2P);
    const uint32_t at = lstart[bin] + rank[j];
    a.local[idx[j]] = static_cast<uint16_t>(at);
    if (covered[j]) continue;
    if (packed)
      stage[at] = (static_cast<unsigned long long>(static_cast<uint32_t>(key[j])) << 32) | static_cast<uint32_t>(idx[j]);
    else
      static_cast<uint4 *>(a.rec)[run_at[bin] + rank[j]] =
          make_uint4(static_cast<uint32_t>(static_cast<uint64_t>(key[j])),
                     static_cast<uint32_t>(static_cast<uint64_t>(key[j]) >> 32), static_cast<uint32_t>(idx[j]), 0u);
  }
  if (!packed) return;
  __syncthreads();
  const uint32_t records = lstart[P];
  for (uint32_t q = threadIdx.x; q < records; q += kRpBlock) {
    const unsigned long long rec = stage[q];
    const uint32_t bin = hash_id(rp_packed_key(rec, a.eb)) >> (32 - a.log2P);
    static_cast<unsigned long long *>(a.rec)[run_at[bin] + (q - lstart[bin])] = rec;
  }
}

__global__ __launch_bounds__(kRpBlock) void rp_scatter_kernel(RpArgs a) { rp_scatter_body(blockIdx.x, a); }

__global__ __launch_bounds__(kRpBlock) void rp_scatter_jobs(Jobs<RpArgs> j) {
  if (blockIdx.x < j.blocks[blockIdx.y]) rp_scatter_body(blockIdx.x, j.a[blockIdx.y]);
}

// The table of a bin: per slot an id, claimed by a compare-and-swap, and the smallest index seen for it,
// lowered by an atomic minimum after a look (32-bit atomics, which the LDS executes several times faster than
// 64-bit ones: slots {id : 32 | index : 32} under one 64-bit atomic minimum per id measured 12 us per bin of
// 12,000 records for the inserts alone). Ids that fit 32 bits are kept as such, next to their index, so
// that one 8-byte read shows both (16,384 slots in 128 KB); others in full, in an array in front of the
// indices (8,192 slots in 96 KB). The id that looks like an empty slot (all ones) is kept in a word of its own.
template <bool PACKED>
struct RpTable {
  using Key = typename std::conditional<PACKED, uint32_t, unsigned long long>::type;
  static constexpr Key kEmpty = static_cast<Key>(~0ull);
  unsigned long long *mem;
  uint32_t *all_ones;  // smallest index of the id kEmpty
  uint32_t mask;       // slots - 1

  __device__ __forceinline__ Key *key_at(uint32_t p) const {
    if (PACKED) return reinterpret_cast<Key *>(reinterpret_cast<uint32_t *>(mem) + 2 * p);
    return reinterpret_cast<Key *>(mem) + p;
  }
  __device__ __forceinline__ uint32_t *index_at(uint32_t p) const {
    if (PACKED) return reinterpret_cast<uint32_t *>(mem) + 2 * p + 1;
    return reinterpret_cast<uint32_t *>(mem + mask + 1) + p;
  }
  __device__ __forceinline__ void look(uint32_t p, Key *key, uint32_t *index) const {
    if (PACKED) {
      const unsigned long long both = mem[p];
      *key = static_cast<Key>(static_cast<uint32_t>(both));
      *index = static_cast<uint32_t>(both >> 32);
    } else {
      *key = *key_at(p);
      *index = *index_at(p);
    }
  }

  __device__ __forceinline__ void clear() const {
    for (uint32_t t = threadIdx.x; t <= mask; t += blockDim.x) {
      mem[t] = ~0ull;
      if (!PACKED) *index_at(t) = 0xFFFFFFFFu;
    }
    if (threadIdx.x == 0) *all_ones = 0xFFFFFFFFu;
  }

  // An id sits within kMaxProbes slots of its home slot or not at all: a table so full that probe sequences
  // get longer (a bin of nearly as many distinct ids as it has slots) counts as one that does not fit, and
  // the bin takes two rounds at half the load instead of walking through thousands of slots per id.
  static constexpr uint32_t kMaxProbes = 256;

  // The probe sequence of an id: its home slot (low bits of the hash), then steps of an odd stride taken from
  // the hash's upper bits. LDS has no lines to stay within, so a stride costs nothing and keeps the sequences
  // of a nearly full table short (1 / (1 - load) probes where slot-by-slot probing needs the square of that).
  __device__ __forceinline__ uint32_t stride(uint32_t hash) const { return ((hash >> 15) | 1u) & mask; }

  // From the second slot of the sequence on (key != kEmpty); *slot: where the id sits (ids never move once
  // they have a slot).
  __device__ __forceinline__ bool insert_from(Key key, uint32_t i, uint32_t hash, uint32_t *slot) const {
    const uint32_t step = stride(hash);
    uint32_t p = (hash + step) & mask;
    const uint32_t limit = mask < kMaxProbes ? mask : kMaxProbes;
    for (uint32_t probes = 0; probes < limit; ++probes) {
      Key k;
      uint32_t cur;
      look(p, &k, &cur);
      if (k == kEmpty) k = atomicCAS(key_at(p), kEmpty, key);
      if (k == kEmpty || k == key) {
        if (cur > i) atomicMin(index_at(p), i);  // a look that is out of date can only show a larger index
        *slot = p;
        return true;
      }
      p = (p + step) & mask;
    }
    return false;
  }

  __device__ __forceinline__ uint32_t first_from(Key key, uint32_t hash) const {
    const uint32_t step = stride(hash);
    uint32_t p = (hash + step) & mask;
    const uint32_t limit = mask < kMaxProbes ? mask : kMaxProbes;
    for (uint32_t probes = 0; probes < limit; ++probes) {
      Key k;
      uint32_t cur;
      look(p, &k, &cur);
      if (k == key) return cur;
      p = (p + step) & mask;
    }
    return 0xFFFFFFFFu;  // cannot happen: every id was inserted
  }
};

template <bool PACKED>
struct RpRecord {
  int64_t key;
  uint32_t i;
  __device__ __forceinline__ void load(const void *rec, uint32_t at) {
    if (PACKED) {
      const unsigned long long r = static_cast<const unsigned long long *>(rec)[at];
      key = static_cast<int64_t>(r >> 32);
      i = static_cast<uint32_t>(r);
    } else {
      const uint4 r = static_cast<const uint4 *>(rec)[at];
      key = static_cast<int64_t>((static_cast<uint64_t>(r.y) << 32) | r.x);
      i = r.z;
    }
  }
};

constexpr int kRpBinItems = 8;  // records a thread has in flight while it walks over a bin
constexpr int kRpHeldPasses = 1;  // passes of kRpBinItems records per thread whose table slots stay in registers

// A bin whose ids do not fit its table is worked through in 2, 4, ... rounds over classes of its ids (bits
// of the second hash).
__device__ __forceinline__ bool rp_mine(int64_t key, uint32_t round_mask, uint32_t round) {
  return round_mask == 0 || (rp_class(key) & round_mask) == round;
}

// kRpBinItems records of a bin, element e0 + j * (threads of the workgroup) for j = 0 .., all loads in flight together.
template <bool PACKED>
__device__ __forceinline__ void rp_load_records(const RpArgs &a, uint32_t start, uint32_t cnt, uint32_t e0,
                                                uint32_t round_mask, uint32_t round,
                                                RpRecord<PACKED> (&rec)[kRpBinItems], uint32_t (&hash)[kRpBinItems],
                                                bool (&on)[kRpBinItems]) {
#pragma unroll
  for (int j = 0; j < kRpBinItems; ++j) {
    rec[j].key = 0;
    rec[j].i = 0;
    on[j] = e0 + j * blockDim.x < cnt;
    if (on[j]) rec[j].load(a.rec, start + e0 + j * blockDim.x);
  }
#pragma unroll
  for (int j = 0; j < kRpBinItems; ++j) {
    hash[j] = hash_id(rec[j].key);
    on[j] = on[j] && rp_mine(rec[j].key, round_mask, round);
  }
}

template <bool PACKED>
__device__ __forceinline__ void rp_bin_body(unsigned bx, const RpArgs &a, unsigned long long *mem,
                                            uint32_t *shared_words) {
  using Table = RpTable<PACKED>;
  using Key = typename Table::Key;
  const uint32_t start = a.binstart[bx];
  const uint32_t cnt = a.binstart[bx + 1] - start;
  if (cnt == 0) return;
  uint32_t *const overflow = &shared_words[0];
  const uint32_t slots = PACKED ? (1u << a.slots_log2) : (1u << (a.slots_log2 - 1));
  const Table tbl{mem, &shared_words[1], slots - 1};
  // Where the records of the first kRpHeldPasses passes over the bin went (a slot, or one of the two marks):
  // their results are then one LDS read each, without reading, hashing and probing a second time.
  constexpr uint32_t kNotMine = 0xFFFFFFFFu, kAllOnes = 0xFFFFFFFEu;
  uint32_t where[kRpHeldPasses][kRpBinItems];
  for (int lg = 0; lg <= a.max_rounds_log2; ++lg) {
    const uint32_t round_mask = (1u << lg) - 1u;
    bool done = true;
    for (uint32_t r = 0; r <= round_mask && done; ++r) {
      tbl.clear();
      if (threadIdx.x == 0) *overflow = 0;
      __syncthreads();
      bool fits = true;
      // one pass: kRpBinItems records per thread; `slot_out` is null beyond the passes whose slots are kept
      auto insert_pass = [&](uint32_t e0, uint32_t *slot_out) {
        RpRecord<PACKED> rec[kRpBinItems];
        uint32_t hash[kRpBinItems];
        bool on[kRpBinItems];
        rp_load_records<PACKED>(a, start, cnt, e0, round_mask, r, rec, hash, on);
        // the home slots of all records are looked at together, then claimed together, then their indices
        // lowered together; only a record that met another id goes on along its probe sequence
        Key k[kRpBinItems];
        uint32_t cur[kRpBinItems], slot[kRpBinItems];
#pragma unroll
        for (int j = 0; j < kRpBinItems; ++j) {
          const Key key = static_cast<Key>(rec[j].key);
          slot[j] = kNotMine;
          if (on[j] && key == Table::kEmpty) {
            atomicMin(tbl.all_ones, rec[j].i);
            on[j] = false;
            slot[j] = kAllOnes;
          }
          k[j] = 0;
          cur[j] = 0;
          if (on[j]) tbl.look(hash[j] & tbl.mask, &k[j], &cur[j]);
        }
#pragma unroll
        for (int j = 0; j < kRpBinItems; ++j)
          if (on[j] && k[j] == Table::kEmpty)
            k[j] = atomicCAS(tbl.key_at(hash[j] & tbl.mask), Table::kEmpty, static_cast<Key>(rec[j].key));
#pragma unroll
        for (int j = 0; j < kRpBinItems; ++j) {
          if (!on[j]) continue;
          if (k[j] == Table::kEmpty || k[j] == static_cast<Key>(rec[j].key)) {
            if (cur[j] > rec[j].i) atomicMin(tbl.index_at(hash[j] & tbl.mask), rec[j].i);
            slot[j] = hash[j] & tbl.mask;
          } else {
            fits &= tbl.insert_from(static_cast<Key>(rec[j].key), rec[j].i, hash[j], &slot[j]);
          }
        }
        if (slot_out) {
#pragma unroll
          for (int j = 0; j < kRpBinItems; ++j) slot_out[j] = slot[j];
        }
      };
      const uint32_t pass_records = kRpBinItems * blockDim.x;
#pragma unroll
      for (int pass = 0; pass < kRpHeldPasses; ++pass) {
#pragma unroll
        for (int j = 0; j < kRpBinItems; ++j) where[pass][j] = kNotMine;
        if (pass * pass_records < cnt) insert_pass(threadIdx.x + pass * pass_records, where[pass]);
      }
      for (uint32_t e0 = threadIdx.x + kRpHeldPasses * pass_records; e0 < cnt; e0 += pass_records) insert_pass(e0, nullptr);
      if (!fits) *overflow = 1;
      __syncthreads();
      done = *overflow == 0;
      if (done) {
#pragma unroll
        for (int pass = 0; pass < kRpHeldPasses; ++pass) {
#pragma unroll
          for (int j = 0; j < kRpBinItems; ++j) {
            const uint32_t w = where[pass][j];
            if (w != kNotMine)
              a.firstp[start + threadIdx.x + pass * pass_records + j * blockDim.x] =
                  w == kAllOnes ? *tbl.all_ones : *tbl.index_at(w);
          }
        }
        for (uint32_t e0 = threadIdx.x + kRpHeldPasses * pass_records; e0 < cnt; e0 += pass_records) {
          RpRecord<PACKED> rec[kRpBinItems];
          uint32_t hash[kRpBinItems];
          bool on[kRpBinItems];
          rp_load_records<PACKED>(a, start, cnt, e0, round_mask, r, rec, hash, on);
          Key k[kRpBinItems];
          uint32_t f[kRpBinItems];
#pragma unroll
          for (int j = 0; j < kRpBinItems; ++j) {
            k[j] = 0;
            f[j] = 0;
            if (on[j]) tbl.look(hash[j] & tbl.mask, &k[j], &f[j]);
          }
#pragma unroll
          for (int j = 0; j < kRpBinItems; ++j) {
            if (!on[j]) continue;
            const Key key = static_cast<Key>(rec[j].key);
            if (key == Table::kEmpty)
              f[j] = *tbl.all_ones;
            else if (k[j] != key)
              f[j] = tbl.first_from(key, hash[j]);
            a.firstp[start + e0 + j * blockDim.x] = f[j];
          }
        }
      }
      __syncthreads();
    }
    if (done) return;
  }
  // every pair: the ids of this bin defeat both hashes
  for (uint32_t e = threadIdx.x; e < cnt; e += blockDim.x) {
    RpRecord<PACKED> mine;
    mine.load(a.rec, start + e);
    uint32_t first = mine.i;
    for (uint32_t o = 0; o < cnt; ++o) {
      RpRecord<PACKED> other;
      other.load(a.rec, start + o);
      if (other.key == mine.key && other.i < first) first = other.i;
    }
    a.firstp[start + e] = first;
  }
}

// TABLE_LOG2: the table this instantiation has room for (a.slots_log2 <= TABLE_LOG2 of it are used). Small
// bins take small tables and small workgroups, so that several of them share a compute unit.
constexpr int rp_bins_threads(int table_log2) { return table_log2 >= 14 ? 1024 : (table_log2 == 13 ? 512 : 256); }

template <int TABLE_LOG2>
__device__ __forceinline__ void rp_bins_body(unsigned bx, const RpArgs &a) {
  __shared__ unsigned long long mem[1 << TABLE_LOG2];
  __shared__ uint32_t shared_words[2];
  if (rl_packed(a.path))
    rp_bin_body<true>(bx, a, mem, shared_words);
  else
    rp_bin_body<false>(bx, a, mem, shared_words);
}

template <int TABLE_LOG2>
__global__ __launch_bounds__(rp_bins_threads(TABLE_LOG2)) void rp_bins_kernel(RpArgs a) {
  rp_bins_body<TABLE_LOG2>(blockIdx.x, a);
}

template <int TABLE_LOG2>
__global__ __launch_bounds__(rp_bins_threads(TABLE_LOG2)) void rp_bins_jobs(Jobs<RpArgs> j) {
  if (blockIdx.x < j.blocks[blockIdx.y]) rp_bins_body<TABLE_LOG2>(blockIdx.x, j.a[blockIdx.y]);
}

// The results of the tile's records are read run by run, consecutive lanes from consecutive addresses, into
// LDS in the tile's bin order; every element then picks the one of its record there.
__device__ __forceinline__ void rp_gather_body(unsigned bx, const RpArgs &a) {
  extern __shared__ uint32_t words[];  // run start in memory (P), start among the tile's records (P + 1)
  __shared__ uint32_t result[kRpTile];
  __shared__ uint32_t firsts[kRpTile / kRlTile];
  const int64_t N = rl_count(a.n);
  const int64_t lo = static_cast<int64_t>(bx) * kRpTile;
  if (lo >= N) return;
  const int64_t hi = lo + kRpTile < N ? lo + kRpTile : N;
  const uint32_t P = 1u << a.log2P;
  const uint32_t *const runs = a.tile_runs + static_cast<size_t>(bx) * (2 * P + 1);
  for (uint32_t t = threadIdx.x; t < 2 * P + 1; t += kRpBlock) words[t] = runs[t];
  const int sub_tiles = static_cast<int>(kRpTile / kRlTile);
  for (int t = threadIdx.x; t < sub_tiles; t += kRpBlock) firsts[t] = 0;
  __syncthreads();
  const uint32_t *const run_at = words, *const lstart = words + P;
  const uint32_t records = lstart[P];
  for (uint32_t q = threadIdx.x; q < records; q += kRpBlock) {
    // the bin whose records include the q-th: the last one that starts at or before q
    uint32_t bin = 0;
    for (uint32_t step = P >> 1; step > 0; step >>= 1)
      if (lstart[bin + step] <= q) bin += step;
    result[q] = a.firstp[run_at[bin] + (q - lstart[bin])];
  }
  __syncthreads();
  uint16_t at[kRpItems];
#pragma unroll
  for (int j = 0; j < kRpItems; ++j) {
    const int64_t i = lo + j * kRpBlock + threadIdx.x;
    at[j] = i < hi ? a.local[i] : static_cast<uint16_t>(0);
  }
#pragma unroll
  for (int j = 0; j < kRpItems; ++j) {
    const int64_t i = lo + j * kRpBlock + threadIdx.x;
    const uint32_t f = i < hi ? result[at[j]] : 0xFFFFFFFFu;
    if (i < hi) a.first[i] = f;
    // a wave's 64 elements lie in one tile of kRlTile ids
    const uint64_t wins = __builtin_amdgcn_ballot_w64(i < hi && f == static_cast<uint32_t>(i));
    if (lane_id() == 0 && wins)
      atomicAdd(&firsts[(i - lo) / kRlTile], static_cast<uint32_t>(__builtin_popcountll(wins)));
  }
  __syncthreads();
  uint32_t all = 0;
  for (int t = threadIdx.x; t < sub_tiles; t += kRpBlock) {
    const int64_t tile = lo / kRlTile + t;
    if (tile * kRlTile < N) a.partials[tile] = firsts[t];
    all += firsts[t];
  }
  // (one wave covers all sub-tiles) the tile's own total, so that the unique pass needs no scan of the counts
  static_assert(kRpTile / kRlTile <= kWave, "the first wave sums a tile's counts");
  if (threadIdx.x < kWave) {
    all = wave_last(wave_inclusive_scan(all));
    if (threadIdx.x == 0) a.coarse[bx] = all;
  }
}

__global__ __launch_bounds__(kRpBlock) void rp_gather_kernel(RpArgs a) { rp_gather_body(blockIdx.x, a); }

__global__ __launch_bounds__(kRpBlock) void rp_gather_jobs(Jobs<RpArgs> j) {
  if (blockIdx.x < j.blocks[blockIdx.y]) rp_gather_body(blockIdx.x, j.a[blockIdx.y]);
}

// A value no earlier call has used (and that uninitialised memory is unlikely to hold).
uint64_t relabel_nonce() {
  static std::atomic<uint64_t> counter{0x9E3779B97F4A7C15ull};
  uint64_t z = counter.fetch_add(0x9E3779B97F4A7C15ull, std::memory_order_relaxed);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;  // splitmix64 finaliser
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}


// ---- 2^31 ids and more: 64-bit positions ------------------------------------------
// The passes above keep first-occurrence indices, ranks and table positions in
// 32 bits (the reference does the same: int numel / uint32_t positions,
// src/tensor_relabel.cu:75-76,122,136). Inputs of 2^31 ids or more take this
// path instead: the same four passes with 64-bit indices and ranks throughout
// ({int64 key, uint64 first index} slots, a 64-bit hash position, a rank array
// of 8 bytes per id), without the small-input, packed-slot and merged-launch
// forms, which such inputs have no use for. Ids are 8 bytes wide.
struct RlSlot64 {
  int64_t key;
  unsigned long long first;
};
static_assert(sizeof(RlSlot64) == 16, "slot must be 16 bytes");

constexpr int kRl64Tile = 512;  // ids per workgroup in the first-occurrence and unique passes

__device__ __forceinline__ uint64_t rl64_home(int64_t key, uint64_t cap) {
  uint64_t x = static_cast<uint64_t>(key);
  x ^= x >> 33;
  x *= 0xff51afd7ed558ccdull;
  x ^= x >> 33;
  x *= 0xc4ceb9fe1a85ec53ull;
  x ^= x >> 33;
  return __umul64hi(x, cap);  // floor(x * cap / 2^64) < cap
}

__global__ __launch_bounds__(256) void rl64_insert_kernel(RlSlot64 *tbl, uint64_t cap, const int64_t *total,
                                                          int64_t N) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < N; i += stride) {
    const int64_t key = total[i];
    uint64_t pos = rl64_home(key, cap);
    for (uint64_t probes = 0; probes < cap; ++probes) {
      // look before the atomics (see rl_global_insert)
      const int64_t seen = __hip_atomic_load(&tbl[pos].key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (seen == key) {
        if (__hip_atomic_load(&tbl[pos].first, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >
            static_cast<unsigned long long>(i))
          atomicMin(&tbl[pos].first, static_cast<unsigned long long>(i));
        break;
      }
      if (seen == -1) {
        const unsigned long long prev = atomicCAS(reinterpret_cast<unsigned long long *>(&tbl[pos].key), ~0ull,
                                                  static_cast<unsigned long long>(key));
        if (prev == ~0ull || static_cast<int64_t>(prev) == key) {
          atomicMin(&tbl[pos].first, static_cast<unsigned long long>(i));
          break;
        }
      }
      pos = (pos + 1 == cap) ? 0 : pos + 1;
    }
  }
}

// labels[i] = first index of total[i]; partials[tile] = number of first occurrences in the tile.
__global__ __launch_bounds__(kRl64Tile) void rl64_first_kernel(const RlSlot64 *tbl, uint64_t cap,
                                                               const int64_t *total, int64_t N, int64_t *labels,
                                                               uint64_t *partials) {
  __shared__ uint64_t lds[kRl64Tile / kWave];
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kRl64Tile + threadIdx.x;
  uint64_t cnt = 0;
  if (i < N) {
    const int64_t key = total[i];
    uint64_t pos = rl64_home(key, cap);
    unsigned long long f = ~0ull;
    for (uint64_t probes = 0; probes < cap; ++probes) {
      const RlSlot64 s = tbl[pos];
      if (s.key == key) {
        f = s.first;
        break;
      }
      if (s.key == -1) break;  // cannot happen: every key was inserted
      pos = (pos + 1 == cap) ? 0 : pos + 1;
    }
    labels[i] = static_cast<int64_t>(f);
    cnt = (f == static_cast<unsigned long long>(i));
  }
  uint64_t tile_total;
  block_exclusive_scan<uint64_t, kRl64Tile>(cnt, lds, &tile_total);
  if (threadIdx.x == 0) partials[blockIdx.x] = tile_total;
}

// partials: exclusive scan of the tile counts, partials[nb] = number of distinct ids.
__global__ __launch_bounds__(kRl64Tile) void rl64_unique_kernel(const int64_t *total, int64_t N,
                                                                const int64_t *labels, const uint64_t *partials,
                                                                int64_t nb, int64_t *unique_out,
                                                                unsigned long long *rank_of, int64_t *count_out) {
  __shared__ uint64_t lds[kRl64Tile / kWave];
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kRl64Tile + threadIdx.x;
  const bool win = i < N && labels[i] == i;
  uint64_t tile_total;
  const uint64_t ex = block_exclusive_scan<uint64_t, kRl64Tile>(win ? 1 : 0, lds, &tile_total);
  if (win) {
    const uint64_t rank = partials[blockIdx.x] + ex;
    unique_out[rank] = total[i];
    rank_of[i] = rank;
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) publish_size(count_out, static_cast<int64_t>(partials[nb]));
}

__global__ __launch_bounds__(256) void rl64_labels_kernel(int64_t *labels, int64_t N,
                                                          const unsigned long long *rank_of) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < N; i += stride)
    labels[i] = static_cast<int64_t>(rank_of[labels[i]]);
}

struct Rl64Layout {
  int64_t cap, table_off, rank_off, partial_off, scan_off, scan_bytes, total;
};

static Rl64Layout rl64_layout(int64_t N) {
  Rl64Layout l;
  l.cap = (2 * N + 7) & ~7ll;
  if (l.cap < 64) l.cap = 64;
  l.table_off = 0;
  l.rank_off = l.cap * 16;
  l.partial_off = l.rank_off + ((N * 8 + 255) & ~255ll);
  const int64_t nb = (N + kRl64Tile - 1) / kRl64Tile;
  l.scan_off = l.partial_off + (((nb + 1) * 8 + 255) & ~255ll);
  l.scan_bytes = shmt_scan_tmp_bytes(nb + 1);
  l.total = l.scan_off + ((l.scan_bytes + 255) & ~255ll) + 256;
  return l;
}

static int relabel_wide_impl(const void *total, int64_t N, void *scratch, int64_t scratch_bytes, void *unique_out,
                             void *labels_out, int64_t *count_out, hipStream_t s) {
  SHMT_REQUIRE(N >= 1, "shmt_relabel_wide: N must be >= 1");
  SHMT_REQUIRE(N < (1ll << 40), "shmt_relabel_wide: N must be < 2^40");
  SHMT_REQUIRE(total && unique_out && labels_out && count_out, "shmt_relabel_wide: null buffer");
  const Rl64Layout l = rl64_layout(N);
  if (scratch == nullptr || scratch_bytes < l.total) {
    set_error("shmt_relabel_wide: scratch too small (%lld < %lld bytes)", static_cast<long long>(scratch_bytes),
              static_cast<long long>(l.total));
    return SHMT_ENOMEM;
  }
  SHMT_REQUIRE((reinterpret_cast<uintptr_t>(scratch) & 15) == 0, "shmt_relabel_wide: scratch must be 16-byte aligned");
  char *base = static_cast<char *>(scratch);
  RlSlot64 *tbl = reinterpret_cast<RlSlot64 *>(base + l.table_off);
  unsigned long long *rank_of = reinterpret_cast<unsigned long long *>(base + l.rank_off);
  uint64_t *partials = reinterpret_cast<uint64_t *>(base + l.partial_off);
  const int64_t nb = (N + kRl64Tile - 1) / kRl64Tile;
  SHMT_REQUIRE(nb < (1ll << 31), "shmt_relabel_wide: input too large");
  int rc = launch_fill_ones(tbl, l.cap, s);
  if (rc) return rc;
  const int64_t *ids = static_cast<const int64_t *>(total);
  hipLaunchKernelGGL(rl64_insert_kernel, dim3(grid_for(N, 256, 4096)), dim3(256), 0, s, tbl,
                     static_cast<uint64_t>(l.cap), ids, N);
  SHMT_LAUNCH_CHECK();
  hipLaunchKernelGGL(rl64_first_kernel, dim3(static_cast<unsigned>(nb)), dim3(kRl64Tile), 0, s, tbl,
                     static_cast<uint64_t>(l.cap), ids, N, static_cast<int64_t *>(labels_out), partials);
  SHMT_LAUNCH_CHECK();
  // nb + 1 entries (the last one arbitrary: an exclusive scan ignores it) -> partials[nb] = number of distinct ids
  rc = shmt_exclusive_scan(partials, nb + 1, 8, base + l.scan_off, l.scan_bytes, s);
  if (rc) return rc;
  hipLaunchKernelGGL(rl64_unique_kernel, dim3(static_cast<unsigned>(nb)), dim3(kRl64Tile), 0, s, ids, N,
                     static_cast<const int64_t *>(labels_out), partials, nb, static_cast<int64_t *>(unique_out),
                     rank_of, count_out);
  SHMT_LAUNCH_CHECK();
  hipLaunchKernelGGL(rl64_labels_kernel, dim3(grid_for(N, 256, 8192)), dim3(256), 0, s,
                     static_cast<int64_t *>(labels_out), N, rank_of);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

}  // namespace shmt

using namespace shmt;

extern "C" {

int64_t shmt_relabel_scratch_bytes(int64_t N) {
  if (N < 0) return -1;
  return N < (1ll << 31) ? rl_layout(N).total : rl64_layout(N).total;
}

int64_t shmt_relabel_wide_scratch_bytes(int64_t N) {
  if (N < 0) return -1;
  return rl64_layout(N > 0 ? N : 1).total;
}

// N is the host-known number of ids, or an upper bound of it when `n.extra`
// names a device-side length: launches and scratch are sized for N, the
// kernels work on the true count.
static int relabel_impl(const void *total, const RlSegments *segs, int64_t N, RlCount n,
                        int elem_bytes, void *scratch, int64_t scratch_bytes, void *unique_out,
                        void *labels_out, int64_t *count_out, Launcher launcher, bool prepared = false,
                        uint64_t prepared_nonce = 0, int64_t *count_copy = nullptr,
                        int64_t prepared_slots = 0) {
  SHMT_REQUIRE(N >= 0, "shmt_relabel: N must be >= 0");
  if (N >= (1ll << 31)) {
    // 64-bit positions: a plain call only (segments are concatenated by the caller, hops stay below 2^31)
    SHMT_REQUIRE(!segs && !prepared && !launcher.defer && !n.fixed_dev && !n.extra,
                 "shmt_relabel: inputs of 2^31 ids or more are relabelled by shmt_relabel / shmt_relabel_wide only");
    SHMT_REQUIRE(elem_bytes == 8, "shmt_relabel: inputs of 2^31 ids or more must be 8 bytes wide");
    return relabel_wide_impl(total, N, scratch, scratch_bytes, unique_out, labels_out, count_out, launcher.stream);
  }
  SHMT_REQUIRE(width_ok(elem_bytes), "shmt_relabel: ID can only be int32 or int64");
  SHMT_REQUIRE(count_out != nullptr, "shmt_relabel: count_out is null");
  hipStream_t s = launcher.stream;
  StageList *const defer = launcher.defer;  // only the fused hop (prepared) records its launches
  if (N == 0) {
    if (defer) {
      defer->mergeable = false;
      return SHMT_OK;
    }
    hipLaunchKernelGGL(rl_zero_count_kernel, dim3(1), dim3(1), 0, s, count_out, count_copy);
    SHMT_LAUNCH_CHECK();
    return SHMT_OK;
  }
  SHMT_REQUIRE(total && unique_out && labels_out, "shmt_relabel: null buffer");
  const RlLayout l = rl_layout(N);
  if (scratch == nullptr || scratch_bytes < l.total) {
    set_error("shmt_relabel: scratch too small (%lld < %lld bytes)",
              static_cast<long long>(scratch_bytes), static_cast<long long>(l.total));
    return SHMT_ENOMEM;
  }
  SHMT_REQUIRE((reinterpret_cast<uintptr_t>(scratch) & 15) == 0,
               "shmt_relabel: scratch must be 16-byte aligned");
  char *base = static_cast<char *>(scratch);
  RlSlot *tbl = reinterpret_cast<RlSlot *>(base + l.table_off);
  RlRanks *ranks = reinterpret_cast<RlRanks *>(base + l.rank_off);  // N / 4 bytes of the N * 4 set aside
  uint64_t *partials = reinterpret_cast<uint64_t *>(base + l.partial_off);
  const int64_t nb = (N + kRlTile - 1) / kRlTile;
  // a caller that emptied the table itself says how much of it (relabel_table)
  const uint32_t cap = static_cast<uint32_t>(prepared && prepared_slots > 0 ? prepared_slots : l.cap);
  // 4-byte ids always fit the packed table; 8-byte ids use it when an earlier kernel vouches for them
  // (plain shmt_relabel has no kernel that sees the ids before the insert pass: 16-byte slots)
  uint64_t *wide_mark = reinterpret_cast<uint64_t *>(base + l.flag_off);
  const uint64_t nonce = prepared ? prepared_nonce : relabel_nonce();
  RlPath path{elem_bytes == 4 ? 1 : ((prepared || segs) ? 2 : 0), wide_mark, nonce};

  if (N <= kRlSmallMax) {
    const RlSmallArgs a{segs ? nullptr : total, segs ? const_cast<void *>(total) : nullptr, elem_bytes, n,
                        unique_out, labels_out, count_out, count_copy};
    if (defer) {
      if (segs) defer->mergeable = false; else stage_push(defer, kStageRlSmall, 1, kRlSmallBlock, a);
      return SHMT_OK;
    }
    if (segs)
      hipLaunchKernelGGL(rl_small_segments_kernel, dim3(1), dim3(kRlSmallBlock), 0, s, a, *segs);
    else
      hipLaunchKernelGGL(rl_small_kernel, dim3(1), dim3(kRlSmallBlock), 0, s, a);
    SHMT_LAUNCH_CHECK();
    return SHMT_OK;
  }

  int rc = SHMT_OK;
  const int scanned = nb > kRlSelfPrefixTiles;
  // a job among fewer merged ones than the partition passes pay for keeps the table (and stays mergeable)
  const RpPlan rp = rp_plan(N, defer ? (prepared ? defer->jobs : 1) : 0, n.fixed_dev != nullptr);
  if (!rp.ok && defer && rp_plan(N, 0, n.fixed_dev != nullptr).ok) {
    defer->mergeable = false;  // a hop of this size on its own takes the partition passes: one by one then
    return SHMT_OK;
  }
  if (rp.ok) {
    // 8-byte ids: the count pass looks at every id itself, so it can vouch for them like the kernels of a
    // fused hop do (and an earlier kernel that stored the mark already is just as good)
    if (path.mode == 0) path.mode = 2;
    const int slots_log2 = g_rp_tuning.slots_log2 < rp.table_log2 ? g_rp_tuning.slots_log2 : rp.table_log2;
    RpArgs a{total, elem_bytes, n, path, wide_mark, rp.log2P, rp.W, base + rp.rec_off,
             reinterpret_cast<uint32_t *>(base + rp.first_off), reinterpret_cast<uint32_t *>(base + rp.firstp_off),
             reinterpret_cast<uint32_t *>(base + rp.hist_off), reinterpret_cast<uint32_t *>(base + rp.bintot_off),
             reinterpret_cast<uint32_t *>(base + rp.binstart_off), reinterpret_cast<uint32_t *>(base + rp.coarse_off),
             reinterpret_cast<uint16_t *>(base + rp.local_off), reinterpret_cast<uint32_t *>(base + rp.tile_off),
             partials, slots_log2, g_rp_tuning.max_rounds_log2};
    const RlUniqueArgs unq{total, elem_bytes, n, a.first, 4, partials, unique_out, ranks, count_out, count_copy,
                           2, a.coarse, static_cast<int>(kRpTile / kRlTile)};
    const RlLabelsArgs lab{labels_out, elem_bytes, n, ranks, a.first, 4};
    if (defer) {
      stage_push(defer, kStageRpCount, rp.W, kRpBlock, a);
      stage_push(defer, kStageRpRows, (rp.P + 3) / 4, 256, a);
      stage_push(defer, kStageRpScatter, rp.W, kRpBlock, a);
      stage_push(defer, kStageRpBins + (kRpSlotsLog2 - rp.table_log2), rp.P, rp_bins_threads(rp.table_log2), a);
      stage_push(defer, kStageRpGather, rp.W, kRpBlock, a);
      stage_push(defer, kStageRlUnique, static_cast<unsigned>(nb), kRlBlock, unq);
      stage_push(defer, kStageRlLabels, grid_for(N, 256), 256, lab);
      return SHMT_OK;
    }
    if (segs && !prepared)  // the count pass concatenates on the way: there is no table to empty
      hipLaunchKernelGGL(rp_count_segments_kernel, dim3(rp.W), dim3(kRpBlock), rp.P * sizeof(uint32_t), s, a, *segs);
    else
      hipLaunchKernelGGL(rp_count_kernel, dim3(rp.W), dim3(kRpBlock), rp.P * sizeof(uint32_t), s, a);
    SHMT_LAUNCH_CHECK();
    hipLaunchKernelGGL(rp_rows_kernel, dim3((rp.P + 3) / 4), dim3(256), 0, s, a);
    SHMT_LAUNCH_CHECK();
    hipLaunchKernelGGL(rp_scatter_kernel, dim3(rp.W), dim3(kRpBlock), (3 * rp.P + 1) * sizeof(uint32_t), s, a);
    SHMT_LAUNCH_CHECK();
    if (rp.table_log2 >= 14)
      hipLaunchKernelGGL(rp_bins_kernel<14>, dim3(rp.P), dim3(rp_bins_threads(14)), 0, s, a);
    else if (rp.table_log2 == 13)
      hipLaunchKernelGGL(rp_bins_kernel<13>, dim3(rp.P), dim3(rp_bins_threads(13)), 0, s, a);
    else
      hipLaunchKernelGGL(rp_bins_kernel<12>, dim3(rp.P), dim3(rp_bins_threads(12)), 0, s, a);
    SHMT_LAUNCH_CHECK();
    hipLaunchKernelGGL(rp_gather_kernel, dim3(rp.W), dim3(kRpBlock), (2 * rp.P + 1) * sizeof(uint32_t), s, a);
    SHMT_LAUNCH_CHECK();
    hipLaunchKernelGGL(rl_unique_kernel, dim3(static_cast<unsigned>(nb)), dim3(kRlBlock), 0, s, unq);
    SHMT_LAUNCH_CHECK();
    hipLaunchKernelGGL(rl_labels_kernel, dim3(grid_for(N, 256)), dim3(256), 0, s, lab);
    SHMT_LAUNCH_CHECK();
    return SHMT_OK;
  }
  const RlInsertArgs ins{tbl, cap, total, elem_bytes, n, path};
  const RlFirstArgs fst{tbl, cap, total, elem_bytes, n, labels_out, partials, path};
  const RlUniqueArgs unq{total, elem_bytes, n, labels_out, elem_bytes, partials, unique_out, ranks, count_out,
                         count_copy, scanned, nullptr, 1};
  const RlLabelsArgs lab{labels_out, elem_bytes, n, ranks, labels_out, elem_bytes};
  // At most 1,024 workgroups insert, each walking its tiles in turn: random global atomics run at 20-26 G/s on
  // this part whatever the grid (a third of the rate of plain stores), and a workgroup's later tiles then find
  // the ids of hub nodes already in the table with a smaller index and skip their atomics, where 8,192
  // workgroups starting together all miss them (8 batches per launch: 64.5 -> 62.3 us per batch).
  const unsigned ins_blocks = grid_for(N, kRlInsertTile, 1024), lab_blocks = grid_for(N, 256);
  if (defer) {
    if (!prepared || scanned) {
      defer->mergeable = false;
      return SHMT_OK;
    }
    stage_push(defer, kStageRlInsert, ins_blocks, kRlBlock, ins);
    stage_push(defer, kStageRlFirst, static_cast<unsigned>(nb), kRlTile, fst);
    stage_push(defer, kStageRlUnique, static_cast<unsigned>(nb), kRlBlock, unq);
    stage_push(defer, kStageRlLabels, lab_blocks, 256, lab);
    return SHMT_OK;
  }
  if (prepared) {
    // the caller's earlier kernels on this stream emptied the table and wrote `total`
  } else if (segs) {
    const int64_t span = l.cap > N ? l.cap : N;
    hipLaunchKernelGGL(rl_fill_concat_kernel, dim3(grid_for(span, 256 * 4)), dim3(256), 0, s,
                       reinterpret_cast<uint4 *>(tbl), l.cap, *segs, const_cast<void *>(total),
                       elem_bytes, n, wide_mark, nonce);
    SHMT_LAUNCH_CHECK();
  } else {
    rc = launch_fill_ones(tbl, l.cap, s);
    if (rc) return rc;
  }
  hipLaunchKernelGGL(rl_insert_kernel, dim3(ins_blocks), dim3(kRlBlock), 0, s, ins);
  SHMT_LAUNCH_CHECK();
  hipLaunchKernelGGL(rl_first_kernel, dim3(static_cast<unsigned>(nb)), dim3(kRlTile), 0, s, fst);
  SHMT_LAUNCH_CHECK();
  if (scanned) {
    rc = launch_scan_partials(partials, nb, s);
    if (rc) return rc;
  }
  hipLaunchKernelGGL(rl_unique_kernel, dim3(static_cast<unsigned>(nb)), dim3(kRlBlock), 0, s, unq);
  SHMT_LAUNCH_CHECK();
  hipLaunchKernelGGL(rl_labels_kernel, dim3(lab_blocks), dim3(256), 0, s, lab);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

}  // extern "C"

namespace shmt {

int relabel_table(int64_t N, bool n_is_loose_bound, int merged_jobs, void *scratch, int64_t scratch_bytes,
                  RelabelTable *out) {
  SHMT_REQUIRE(N >= 1 && N < (1ll << 31), "relabel: N must be in [1, 2^31)");
  const RlLayout l = rl_layout(N);
  if (scratch == nullptr || scratch_bytes < l.total) {
    set_error("relabel: scratch too small (%lld < %lld bytes)", static_cast<long long>(scratch_bytes),
              static_cast<long long>(l.total));
    return SHMT_ENOMEM;
  }
  SHMT_REQUIRE((reinterpret_cast<uintptr_t>(scratch) & 15) == 0, "relabel: scratch must be 16-byte aligned");
  out->slots = static_cast<char *>(scratch) + l.table_off;
  // Small inputs are relabelled in LDS: nothing to empty. When N is a loose bound of the id count (a
  // chained hop sized for every seed the hop before could have produced, typically three times what
  // it did produce) half the slots are used: still one 16-byte slot per id in the worst case, and
  // half as much to empty.
  // Nor is there when the partition passes take the input (rp_plan).
  out->n16 = (N <= kRlSmallMax || rp_plan(N, merged_jobs, n_is_loose_bound).ok) ? 0 : (n_is_loose_bound ? (l.cap / 2 + 7) & ~7ll : l.cap);
  out->wide_mark = reinterpret_cast<uint64_t *>(static_cast<char *>(scratch) + l.flag_off);
  out->nonce = relabel_nonce();
  return SHMT_OK;
}

int launch_relabel_passes(const void *total, int64_t n_bound, int64_t n_fixed, const int64_t *n_fixed_dev,
                          const void *n_extra_dev, int n_extra_bytes, int elem_bytes, void *scratch,
                          int64_t scratch_bytes, void *unique_out, void *labels_out, int64_t *count_out,
                          int64_t *count_copy, const RelabelTable &table, Launcher launcher) {
  return relabel_impl(total, nullptr, n_bound,
                      RlCount{n_fixed, n_fixed_dev, n_extra_dev, n_extra_bytes, n_bound}, elem_bytes,
                      scratch, scratch_bytes, unique_out, labels_out, count_out, launcher, true, table.nonce,
                      count_copy, table.n16);
}

int launch_merged_relabel_stage(int n_jobs, const Stage *const *stages, hipStream_t s) {
  const unsigned threads = stages[0]->threads;
  switch (stages[0]->kind) {
    case kStageRlSmall: {
      Jobs<RlSmallArgs> j;
      jobs_from_stages(n_jobs, stages, &j);
      hipLaunchKernelGGL(rl_small_jobs, dim3(1, n_jobs), dim3(threads), 0, s, j);
      break;
    }
    case kStageRlInsert: {
      Jobs<RlInsertArgs> j;
      const unsigned blocks = jobs_from_stages(n_jobs, stages, &j);
      hipLaunchKernelGGL(rl_insert_jobs, dim3(blocks, n_jobs), dim3(threads), 0, s, j);
      break;
    }
    case kStageRlFirst: {
      Jobs<RlFirstArgs> j;
      const unsigned blocks = jobs_from_stages(n_jobs, stages, &j);
      hipLaunchKernelGGL(rl_first_jobs, dim3(blocks, n_jobs), dim3(threads), 0, s, j);
      break;
    }
    case kStageRlUnique: {
      Jobs<RlUniqueArgs> j;
      const unsigned blocks = jobs_from_stages(n_jobs, stages, &j);
      hipLaunchKernelGGL(rl_unique_jobs, dim3(blocks, n_jobs), dim3(threads), 0, s, j);
      break;
    }
    case kStageRlLabels: {
      Jobs<RlLabelsArgs> j;
      const unsigned blocks = jobs_from_stages(n_jobs, stages, &j);
      hipLaunchKernelGGL(rl_labels_jobs, dim3(blocks, n_jobs), dim3(threads), 0, s, j);
      break;
    }
    case kStageRpCount:
    case kStageRpRows:
    case kStageRpScatter:
    case kStageRpGather:
    case kStageRpBins:
    case kStageRpBins + 1:
    case kStageRpBins + 2: {
      Jobs<RpArgs> j;
      const unsigned blocks = jobs_from_stages(n_jobs, stages, &j);
      int log2P = 0;  // the LDS arrays are sized for the job with the most bins
      for (int i = 0; i < n_jobs; ++i) log2P = j.a[i].log2P > log2P ? j.a[i].log2P : log2P;
      const size_t P = static_cast<size_t>(1) << log2P;
      const dim3 grid(blocks, n_jobs), wg(threads);
      switch (stages[0]->kind) {
        case kStageRpCount: hipLaunchKernelGGL(rp_count_jobs, grid, wg, P * sizeof(uint32_t), s, j); break;
        case kStageRpRows: hipLaunchKernelGGL(rp_rows_jobs, grid, wg, 0, s, j); break;
        case kStageRpScatter: hipLaunchKernelGGL(rp_scatter_jobs, grid, wg, (3 * P + 1) * sizeof(uint32_t), s, j); break;
        case kStageRpGather: hipLaunchKernelGGL(rp_gather_jobs, grid, wg, (2 * P + 1) * sizeof(uint32_t), s, j); break;
        case kStageRpBins: hipLaunchKernelGGL(rp_bins_jobs<14>, grid, wg, 0, s, j); break;
        case kStageRpBins + 1: hipLaunchKernelGGL(rp_bins_jobs<13>, grid, wg, 0, s, j); break;
        default: hipLaunchKernelGGL(rp_bins_jobs<12>, grid, wg, 0, s, j); break;
      }
      break;
    }
    default:
      set_error("internal: stage kind %d has no merged relabel launch", stages[0]->kind);
      return SHMT_EINVAL;
  }
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

}  // namespace shmt

extern "C" {

int shmt_relabel(const void *total, int64_t N, int elem_bytes, void *scratch,
                 int64_t scratch_bytes, void *unique_out, void *labels_out, int64_t *count_out,
                 void *stream) {
  return relabel_impl(total, nullptr, N, RlCount{N, nullptr, nullptr, 8, N}, elem_bytes, scratch, scratch_bytes,
                      unique_out, labels_out, count_out, Launcher{as_stream(stream), nullptr});
}

int shmt_relabel_tuning(int64_t partition_min_ids, int lds_slots_log2, int max_rounds_log2) {
  SHMT_REQUIRE(lds_slots_log2 >= 0 && lds_slots_log2 <= kRpSlotsLog2 && lds_slots_log2 != 1,
               "shmt_relabel_tuning: lds_slots_log2 must be 0 (default) or in [2, %d]", kRpSlotsLog2);
  SHMT_REQUIRE(max_rounds_log2 >= -1 && max_rounds_log2 <= 20,
               "shmt_relabel_tuning: max_rounds_log2 must be -1 (default) or in [0, 20]");
  g_rp_tuning.min_ids = partition_min_ids <= 0 ? kRpDefaultMin : partition_min_ids;
  g_rp_tuning.min_ids_merged = partition_min_ids <= 0 ? kRpMergedMin : (partition_min_ids < kRpMergedMin ? partition_min_ids : kRpMergedMin);
  g_rp_tuning.slots_log2 = lds_slots_log2 == 0 ? kRpSlotsLog2 : lds_slots_log2;
  g_rp_tuning.max_rounds_log2 = max_rounds_log2 < 0 ? kRpMaxRoundsLog2 : max_rounds_log2;
  return SHMT_OK;
}

int shmt_relabel_wide(const void *total, int64_t N, void *scratch, int64_t scratch_bytes, void *unique_out,
                      void *labels_out, int64_t *count_out, void *stream) {
  SHMT_REQUIRE(N >= 0, "shmt_relabel_wide: N must be >= 0");
  SHMT_REQUIRE(count_out != nullptr, "shmt_relabel_wide: count_out is null");
  if (N == 0) {
    hipLaunchKernelGGL(rl_zero_count_kernel, dim3(1), dim3(1), 0, as_stream(stream), count_out,
                       static_cast<int64_t *>(nullptr));
    SHMT_LAUNCH_CHECK();
    return SHMT_OK;
  }
  return relabel_wide_impl(total, N, scratch, scratch_bytes, unique_out, labels_out, count_out, as_stream(stream));
}

int shmt_relabel_segments(const void *const *seg_ptrs, const int64_t *seg_lens, const int *seg_bytes,
                          int nseg, const void *last_len_dev, int last_len_bytes, int elem_bytes,
                          void *total_out, void *scratch, int64_t scratch_bytes, void *unique_out,
                          void *labels_out, int64_t *count_out, void *stream) {
  SHMT_REQUIRE(nseg >= 1 && nseg <= SHMT_RELABEL_MAX_SEGMENTS,
               "shmt_relabel_segments: between 1 and %d segments", SHMT_RELABEL_MAX_SEGMENTS);
  SHMT_REQUIRE(seg_ptrs && seg_lens && seg_bytes, "shmt_relabel_segments: null segment arrays");
  SHMT_REQUIRE(last_len_dev == nullptr || width_ok(last_len_bytes),
               "shmt_relabel_segments: last_len_bytes must be 4 or 8");
  RlSegments segs;
  segs.n = nseg;
  int64_t N = 0;
  for (int i = 0; i < nseg; ++i) {
    SHMT_REQUIRE(seg_lens[i] >= 0, "shmt_relabel_segments: negative segment length");
    SHMT_REQUIRE(width_ok(seg_bytes[i]) && seg_bytes[i] <= elem_bytes,
                 "shmt_relabel_segments: segment width must be 4 or 8 and not wider than the output");
    SHMT_REQUIRE(seg_lens[i] == 0 || seg_ptrs[i] != nullptr, "shmt_relabel_segments: null segment");
    segs.ptr[i] = seg_ptrs[i];
    segs.bytes[i] = seg_bytes[i];
    segs.start[i] = N;
    N += seg_lens[i];
  }
  for (int i = nseg; i <= SHMT_RELABEL_MAX_SEGMENTS; ++i) segs.start[i] = N;
  for (int i = nseg; i < SHMT_RELABEL_MAX_SEGMENTS; ++i) {
    segs.ptr[i] = nullptr;
    segs.bytes[i] = 8;
  }
  SHMT_REQUIRE(N == 0 || total_out != nullptr, "shmt_relabel_segments: total_out is null");
  RlCount n{N, nullptr, nullptr, 8, N};
  if (last_len_dev) {
    // the last segment's true length lives on the device; N stays the bound
    n.fixed = N - seg_lens[nseg - 1];
    n.extra = last_len_dev;
    n.extra_bytes = last_len_bytes;
  }
  return relabel_impl(total_out, &segs, N, n, elem_bytes, scratch, scratch_bytes, unique_out,
                      labels_out, count_out, Launcher{as_stream(stream), nullptr});
}

}  // extern "C"
