// Feature row gather (fetch) and scatter (set) through the HBM cache.
// Replaces the twelve kernels of src/cache_feature_fetch.cu:15-224 and
// src/cache_feature_set.cu:6-207 in the ShmTensor tree with one templated
// kernel.
//
// A wave owns tiles of up to 32 consecutive rows.
// Phase 1 (lane per row): coalesced load of the ids, then the cache slot of
// every row at once: the wave's eight probe groups look the ids up
// cooperatively (one 128-byte bucket line per probe, the first bucket of all
// 32 keys in flight together), or every lane reads its slot from a flat map
// (direct table: one 4-byte load; rank bitmap: one 16-byte load; id range:
// arithmetic), or the mask is loaded. Each lane ends up holding the source
// (fetch) or destination (set) address of its row. A wave with several tiles
// keeps phase 1 of the next tiles in flight while it moves rows.
// Phase 2 (sub-wave group of L lanes per row): the row addresses are
// broadcast with lane shuffles and the rows are moved with the widest vector
// access the row size and base pointers allow (16 bytes per lane when
// aligned). The dependent chain id -> bucket -> row is paid once per tile
// instead of once per row.
//
// A fetch can also go out as two launches (shmt_fetch_cached_part /
// shmt_fetch_missed_part): the rows that hit now, the rows that miss (marked
// in a bitmap) by a small grid that a caller may put on another stream.
//
// Measured on MI355X (1,048,576 rows of 256 B): the kernel is register-lean
// on purpose. Eight resident waves per SIMD with one row in flight
// per lane group beat four waves with eight rows in flight by 25-50 % on
// mixed hit/miss batches, because a wave that waits on a host-link read
// (loads return in issue order) then holds back little other work; setting
// missed rows apart in LDS for dedicated waves was measured slower than this
// and is not done.
#include "common.h"
#include "hashmap.h"
#include "hashmap_dev.h"

namespace shmt {

enum RouteMode : int { kDirect = 0, kMap16 = 1, kMap8 = 2, kMask = 3, kMapFlat = 4 };

struct RowArgs {
  char *miss;          // table addressed by id (pinned host alias or device)
  char *cache;         // table addressed by slot (HBM)
  char *dense;         // fetch: output rows; set: update rows
  const void *indices;
  const void *mask;
  MapView map;
  int64_t Q;
  const int64_t *count;  // when set: only the first min(Q, *count) rows are moved (device memory)
  int64_t *count_seen;   // when set: receives *count as soon as the kernel starts (pinned host memory)
  int64_t row_bytes;
  int idx_bytes;
  int mask_bytes;
  int log2_lanes;      // lanes per row in phase 2 = 1 << log2_lanes, in [8, 64]
  int log2_tile;       // rows per wave tile = 1 << log2_tile, in [64 / lanes, 32]
  uint32_t *miss_bits;  // DEFER: bit (i & 31) of word i / 32 is set when row i missed the cache
};

// Native vector types (the non-temporal builtins do not take HIP's struct vectors).
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Table rows are addressed through integers that travelled across lanes, so
// the compiler cannot tell that they point to global memory; saying so turns
// generic (flat) accesses into global ones.
template <typename VT>
__device__ __forceinline__ VT gload(const char *p) {
  return *reinterpret_cast<const VT __attribute__((address_space(1))) *>(reinterpret_cast<uintptr_t>(p));
}
template <typename VT>
__device__ __forceinline__ void gstore(char *p, VT v) {
  *reinterpret_cast<VT __attribute__((address_space(1))) *>(reinterpret_cast<uintptr_t>(p)) = v;
}

constexpr int kRowsBlock = 256;    // threads per workgroup
constexpr int kRowsWavesPerSimd = 8;  // register budget: 512 / 8 = 64 VGPRs
// Rows a lane group moves concurrently (single-vector rows). Measured on 1,048,576 all-hit rows of
// 256 B: 1 row in flight per group 92 us, 2 rows 96 us, 4 rows 94 us (eight resident waves per SIMD
// already keep the memory system busy; shorter load/store bursts per wave mix reads and writes better).
constexpr int kRowsInFlight = 1;
// Rows per wave tile, at most. 32 measured 2 % faster than 64 on all-hit rows (90 against 92 us) and the
// same on mixed hit / miss batches; 16 gains nothing more and costs the bucket-table probe 15 %.
constexpr int kMaxLog2Tile = 5;

// THROUGH (set only, with a map or mask): rows that hit the cache are written
// to the id-addressed table as well, so that table never goes stale.
// DEFER (fetch only, with a map or mask; tiles of exactly 32 rows): rows that
// miss the cache are not moved; every tile leaves one word of a bitmap that
// marks them for rows_missed_kernel (no counter, no atomics, nothing to clear).
template <typename VT, int MODE, bool SET, bool ONE_VEC, bool THROUGH = false, bool DEFER = false>
__global__ __launch_bounds__(kRowsBlock, ONE_VEC ? kRowsWavesPerSimd : kRowsWavesPerSimd / 2) void rows_kernel(RowArgs a) {
  static_assert(!THROUGH || (SET && MODE != kDirect), "write-through is a cached set");
  static_assert(!DEFER || (!SET && MODE != kDirect), "only a cached fetch sets its misses aside");
  const int lane = lane_id();
  const int L = 1 << a.log2_lanes;
  const int gl = lane & (L - 1);
  const int grp = lane >> a.log2_lanes;
  const int rows_per_step = kWave >> a.log2_lanes;
  const int tile = 1 << a.log2_tile;
  const int64_t waves_per_block = blockDim.x / kWave;
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * waves_per_block + threadIdx.x / kWave;
  const int64_t nwaves = static_cast<int64_t>(gridDim.x) * waves_per_block;
  const int64_t R = a.row_bytes;
  const int64_t step = static_cast<int64_t>(L) * sizeof(VT);
  const int64_t my_off = static_cast<int64_t>(gl) * sizeof(VT);
  int64_t Q = a.Q;
  if (a.count) {
    const int64_t counted = *a.count;
    if (counted < Q) Q = counted;
    if (a.count_seen && blockIdx.x == 0 && threadIdx.x == 0) {
      publish_size(a.count_seen, counted);
    }
  }

  // ---- phase 1, pipelined over the wave's tiles ----
  // Where a row lives takes two dependent loads (its id, then the map entry) before the row itself can be
  // touched. A wave with several tiles to do keeps those loads ahead of the rows: while the rows of tile t
  // move, the map loads of tile t + 1 and the ids of tile t + 2 are in flight, and what is looked at next has
  // long arrived. Measured on the hits of a 1,048,576-row Zipf batch (256-byte rows, hot rows in the caches,
  // 1.28 GB bucket table): 84 us with the three steps one after the other per tile, 72 us with the ids kept
  // ahead; all-hit uniform rows through the rank bitmap 107.6 -> 105 us.
  const int64_t stride = nwaves * tile;
  const int64_t base0 = wave * tile;
  if (base0 >= Q) return;  // (whole waves only: no barrier follows)
  struct Ids {  // step A: the ids of a tile (and its mask entries), one row per lane
    int64_t idx, masked;
    bool live;
  };
  auto load_ids = [&](int64_t base) {
    Ids t;
    const int64_t i = base + lane;
    t.live = lane < tile && i < Q;
    t.idx = t.live ? load_int(a.indices, i, a.idx_bytes) : 0;
    t.masked = -1;
    if (MODE == kMask && t.live) t.masked = load_int(a.mask, i, a.mask_bytes);
    return t;
  };
  struct Lookup {  // step B: the map loads of a tile, in flight
    int64_t idx, key, masked;
    bool live;
    HalfWaveProbe probe;
    FlatPending flat;
  };
  // Map entries are read with the streaming policy (see half_wave_issue) until a tile of this wave shows a
  // repeated id: from then on the wave takes the access for skewed and lets the caches keep what it reads.
  bool stream = streamable(a.map);
  auto start_lookup = [&](const Ids &t, Lookup *l) {
    l->idx = t.idx;
    l->masked = t.masked;
    l->live = t.live;
    l->key = -1;
    if (MODE == kMap16 || MODE == kMap8) {
      constexpr int FMT = MODE == kMap16 ? kSlot16 : kSlot8;
      l->key = t.live ? map_key(a.map, t.idx) : -1;
      if (stream && tile_repeats(l->key, t.live)) stream = false;
      if (stream)
        half_wave_issue<FMT, true>(a.map, l->key, &l->probe);
      else
        half_wave_issue<FMT, false>(a.map, l->key, &l->probe);
    } else if (MODE == kMapFlat) {
      // direct, rank or range form of the map: one load, or arithmetic only
      l->key = t.live ? map_key(a.map, t.idx) : -1;
      if (stream && tile_repeats(l->key, t.live)) stream = false;
      if (stream)
        l->flat = flat_issue<true>(a.map, l->key);
      else
        l->flat = flat_issue<false>(a.map, l->key);
    }
  };
  auto finish_lookup = [&](const Lookup &l) -> int64_t {  // step C: the slot of this lane's row, or -1
    if (MODE == kMask) return l.masked;
    if (MODE == kMap16) return half_wave_finish<kSlot16>(a.map, l.key, l.probe);
    if (MODE == kMap8) return half_wave_finish<kSlot8>(a.map, l.key, l.probe);
    if (MODE == kMapFlat) return l.live ? flat_finish(a.map, l.key, l.flat) : -1;
    return -1;
  };
  // (Bucket maps keep only the ids ahead: four bucket fragments per lane held across the row moves cost more
  // registers than eight resident waves per SIMD leave, and the spills cost more than the overlap gains.)
  constexpr bool kLookupAhead = MODE != kMap16 && MODE != kMap8;
  Ids ids_next = load_ids(base0), ids_after = load_ids(base0 + stride);
  Lookup ahead;
  start_lookup(ids_next, &ahead);
  int64_t slot = finish_lookup(ahead);
  int64_t idx = ahead.idx;
  bool live = ahead.live;
  if (kLookupAhead) {
    if (base0 + stride < Q) start_lookup(ids_after, &ahead);
    ids_after = load_ids(base0 + 2 * stride);
  }

  for (int64_t base = base0; base < Q; base += stride) {
    if (DEFER) {
      const uint64_t missed = __builtin_amdgcn_ballot_w64(live && slot < 0);
      if (lane == 0) a.miss_bits[base >> 5] = static_cast<uint32_t>(missed);
    }
    const int64_t my_table_row =
        DEFER && slot < 0 ? 0 : reinterpret_cast<int64_t>(slot >= 0 ? a.cache + slot * R : a.miss + idx * R);
    // write-through: second destination of a row that hit (0: none)
    const int64_t my_second_row =
        THROUGH && slot >= 0 ? reinterpret_cast<int64_t>(a.miss + idx * R) : 0;
    const int nrows = static_cast<int>(Q - base < tile ? Q - base : tile);

    // ---- phase 2: move the rows ----
    if (ONE_VEC) {
      // row_bytes <= L * sizeof(VT): one vector per lane per row
      const bool in = my_off < R;
      for (int r0 = 0; r0 < nrows; r0 += kRowsInFlight * rows_per_step) {
        VT v[kRowsInFlight];
        char *trow[kRowsInFlight];
        char *second[kRowsInFlight];
        // shuffles run with every lane active: a lane can only read the row
        // address held by a lane that takes part in the same instruction
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
          trow[u] = reinterpret_cast<char *>(
              shfl64(my_table_row, (r0 + u * rows_per_step + grp) & (kWave - 1)));
          second[u] = THROUGH ? reinterpret_cast<char *>(shfl64(
                                    my_second_row, (r0 + u * rows_per_step + grp) & (kWave - 1)))
                              : nullptr;
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
          const int row = r0 + u * rows_per_step + grp;
          if (row < nrows && in && (!DEFER || trow[u])) {
            if (SET)
              v[u] = __builtin_nontemporal_load(
                  reinterpret_cast<const VT *>(a.dense + (base + row) * R + my_off));
            else
              v[u] = gload<VT>(trow[u] + my_off);
          }
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
          const int row = r0 + u * rows_per_step + grp;
          if (row < nrows && in && (!DEFER || trow[u])) {
            if (SET) {
              gstore<VT>(trow[u] + my_off, v[u]);
              if (THROUGH && second[u]) gstore<VT>(second[u] + my_off, v[u]);
            } else
              __builtin_nontemporal_store(
                  v[u], reinterpret_cast<VT *>(a.dense + (base + row) * R + my_off));
          }
        }
      }
    } else {
      for (int r0 = 0; r0 < nrows; r0 += rows_per_step) {
        const int row = r0 + grp;
        char *trow = reinterpret_cast<char *>(shfl64(my_table_row, row & (kWave - 1)));
        char *second =
            THROUGH ? reinterpret_cast<char *>(shfl64(my_second_row, row & (kWave - 1))) : nullptr;
        if (row >= nrows || (DEFER && !trow)) continue;
        char *drow = a.dense + (base + row) * R;
        const char *src = SET ? drow : trow;
        char *dst = SET ? trow : drow;
        int64_t off = my_off;
        for (; off + 3 * step < R; off += 4 * step) {
          const VT v0 = gload<VT>(src + off);
          const VT v1 = gload<VT>(src + off + step);
          const VT v2 = gload<VT>(src + off + 2 * step);
          const VT v3 = gload<VT>(src + off + 3 * step);
          gstore<VT>(dst + off, v0);
          gstore<VT>(dst + off + step, v1);
          gstore<VT>(dst + off + 2 * step, v2);
          gstore<VT>(dst + off + 3 * step, v3);
        }
        for (; off < R; off += step)
          gstore<VT>(dst + off, gload<VT>(src + off));
        if (THROUGH && second) {
          for (off = my_off; off < R; off += step)
            gstore<VT>(second + off, gload<VT>(src + off));
        }
      }
    }
    // ---- the next tile's lookup ends here; the one after starts; the ids of the one after that are asked for ----
    if (base + stride < Q) {
      if (!kLookupAhead) start_lookup(ids_after, &ahead);
      slot = finish_lookup(ahead);
      idx = ahead.idx;
      live = ahead.live;
      if (kLookupAhead) {
        if (base + 2 * stride < Q) start_lookup(ids_after, &ahead);
        ids_after = load_ids(base + 3 * stride);
      } else {
        ids_after = load_ids(base + 2 * stride);
      }
    }
  }
}

// Second half of a fetch whose misses were set aside (rows_kernel with DEFER):
// moves the rows marked in the bitmap from the id-addressed table. These are
// host-link reads when the table lives in pinned host memory. The link is
// saturated by the reads of a few dozen waves, and every read beyond that only
// lengthens the queue that all other link traffic of the GPU (the cold
// adjacency of the next mini-batch's sampling) and, measured, even its HBM
// traffic waits in; so the grid is small by design and the rest of the GPU
// stays free for what other streams have queued.
// A wave takes kMissedChunk bitmap words (32 rows each) per pass: one lane per
// word, a wave scan of the popcounts, the set bits expanded into a position
// list in LDS; then lane groups move kMissedRows rows at a time, all their
// loads issued before the first store.
struct MissedArgs {
  const char *table;
  char *dense;
  const void *indices;
  const uint32_t *bits;
  const int64_t *count;  // optional: only the first min(rows, *count) rows exist
  int64_t rows;
  int64_t row_bytes;
  int idx_bytes;
  int log2_lanes;
};

constexpr int kMissedRows = 2;     // rows a lane group has in flight
constexpr int kMissedChunk = 32;   // bitmap words per wave pass: 1,024 rows
constexpr int kMissedBlocks = 48;  // default grid

__global__ __launch_bounds__(kRowsBlock) void rows_missed_kernel(MissedArgs a) {
  using VT = u32x4;
  __shared__ uint32_t positions[kRowsBlock / kWave][kMissedChunk * 32];
  const int lane = lane_id();
  const int L = 1 << a.log2_lanes;
  const int gl = lane & (L - 1);
  const int grp = lane >> a.log2_lanes;
  const int rows_per_step = kWave >> a.log2_lanes;
  const int per_pass = kMissedRows * rows_per_step;  // <= 16: lane groups hold 8 lanes at least
  const int wave_in_block = threadIdx.x / kWave;
  const int64_t waves_per_block = blockDim.x / kWave;
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * waves_per_block + wave_in_block;
  const int64_t nwaves = static_cast<int64_t>(gridDim.x) * waves_per_block;
  const int64_t R = a.row_bytes;
  const int64_t step = static_cast<int64_t>(L) * sizeof(VT);
  const int64_t my_off = static_cast<int64_t>(gl) * sizeof(VT);
  int64_t Q = a.rows;
  if (a.count) {
    const int64_t counted = *a.count;
    if (counted < Q) Q = counted < 0 ? 0 : counted;
  }
  const int64_t nwords = (Q + 31) >> 5;
  uint32_t *const mine = positions[wave_in_block];
  // Words are dealt to the waves one by one (word w0 + lane * nwaves to lane `lane` of wave w0), not in
  // runs: misses cluster (the first rows of a mini-batch's input nodes are its seeds, mostly cold), and a
  // wave that owned a run of 1,024 such rows would still be moving them long after the others were done.
  for (int64_t w0 = wave; w0 < nwords; w0 += nwaves * kMissedChunk) {
    const int64_t my_word = w0 + lane * nwaves;
    uint32_t word = 0;
    if (lane < kMissedChunk && my_word < nwords) word = a.bits[my_word];
    const uint32_t cnt = __builtin_popcount(word);
    const uint32_t inc = wave_inclusive_scan(cnt);
    const int total = static_cast<int>(wave_last(inc));
    uint32_t at = inc - cnt;
    while (word) {
      mine[at++] = static_cast<uint32_t>(my_word << 5) + static_cast<uint32_t>(__builtin_ctz(word));
      word &= word - 1;
    }
    // the list is written and read by this wave only: order its LDS accesses, no workgroup barrier
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int e0 = 0; e0 < total; e0 += per_pass) {
      int64_t my_src = 0, my_dst = 0;
      if (lane < per_pass && e0 + lane < total) {
        const int64_t pos = mine[e0 + lane];
        const int64_t idx = load_int(a.indices, pos, a.idx_bytes);
        my_src = reinterpret_cast<int64_t>(a.table + idx * R);
        my_dst = reinterpret_cast<int64_t>(a.dense + pos * R);
      }
      const char *src[kMissedRows];
      char *dst[kMissedRows];
#pragma unroll
      for (int u = 0; u < kMissedRows; ++u) {
        src[u] = reinterpret_cast<const char *>(shfl64(my_src, u * rows_per_step + grp));
        dst[u] = reinterpret_cast<char *>(shfl64(my_dst, u * rows_per_step + grp));
      }
      for (int64_t off = my_off; off < R; off += step) {
        VT v[kMissedRows];
#pragma unroll
        for (int u = 0; u < kMissedRows; ++u)
          if (src[u]) v[u] = gload<VT>(src[u] + off);
#pragma unroll
        for (int u = 0; u < kMissedRows; ++u)
          if (src[u]) __builtin_nontemporal_store(v[u], reinterpret_cast<VT *>(dst[u] + off));
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
}

template <bool ONE_VEC>
static void launch_defer(int mode, unsigned grid, hipStream_t s, const RowArgs &a) {
  switch (mode) {
    case kMap16:
      hipLaunchKernelGGL((rows_kernel<u32x4, kMap16, false, ONE_VEC, false, true>), dim3(grid), dim3(kRowsBlock), 0, s, a);
      break;
    case kMap8:
      hipLaunchKernelGGL((rows_kernel<u32x4, kMap8, false, ONE_VEC, false, true>), dim3(grid), dim3(kRowsBlock), 0, s, a);
      break;
    case kMapFlat:
      hipLaunchKernelGGL((rows_kernel<u32x4, kMapFlat, false, ONE_VEC, false, true>), dim3(grid), dim3(kRowsBlock), 0, s, a);
      break;
    default:
      hipLaunchKernelGGL((rows_kernel<u32x4, kMask, false, ONE_VEC, false, true>), dim3(grid), dim3(kRowsBlock), 0, s, a);
      break;
  }
}

static int pick_vector_bytes(int64_t row_bytes, const void *p0, const void *p1, const void *p2) {
  uintptr_t bits = static_cast<uintptr_t>(row_bytes);
  bits |= reinterpret_cast<uintptr_t>(p0) | reinterpret_cast<uintptr_t>(p1) |
          reinterpret_cast<uintptr_t>(p2);
  int v = 16;
  while (v > 1 && (bits & (v - 1))) v >>= 1;
  return v;
}

template <typename VT, bool ONE_VEC>
static void launch_through(int mode, unsigned grid, hipStream_t s, const RowArgs &a) {
  switch (mode) {
    case kMap16:
      hipLaunchKernelGGL((rows_kernel<VT, kMap16, true, ONE_VEC, true>), dim3(grid), dim3(kRowsBlock), 0, s, a);
      break;
    case kMap8:
      hipLaunchKernelGGL((rows_kernel<VT, kMap8, true, ONE_VEC, true>), dim3(grid), dim3(kRowsBlock), 0, s, a);
      break;
    case kMapFlat:
      hipLaunchKernelGGL((rows_kernel<VT, kMapFlat, true, ONE_VEC, true>), dim3(grid), dim3(kRowsBlock), 0, s, a);
      break;
    default:
      hipLaunchKernelGGL((rows_kernel<VT, kMask, true, ONE_VEC, true>), dim3(grid), dim3(kRowsBlock), 0, s, a);
      break;
  }
}

template <typename VT, bool SET, bool ONE_VEC>
static void launch_mode(int mode, unsigned grid, hipStream_t s, const RowArgs &a) {
  switch (mode) {
    case kDirect:
      hipLaunchKernelGGL((rows_kernel<VT, kDirect, SET, ONE_VEC>), dim3(grid), dim3(kRowsBlock), 0, s, a);
      break;
    case kMap16:
      hipLaunchKernelGGL((rows_kernel<VT, kMap16, SET, ONE_VEC>), dim3(grid), dim3(kRowsBlock), 0, s, a);
      break;
    case kMap8:
      hipLaunchKernelGGL((rows_kernel<VT, kMap8, SET, ONE_VEC>), dim3(grid), dim3(kRowsBlock), 0, s, a);
      break;
    case kMapFlat:
      hipLaunchKernelGGL((rows_kernel<VT, kMapFlat, SET, ONE_VEC>), dim3(grid), dim3(kRowsBlock), 0, s, a);
      break;
    default:
      hipLaunchKernelGGL((rows_kernel<VT, kMask, SET, ONE_VEC>), dim3(grid), dim3(kRowsBlock), 0, s, a);
      break;
  }
}

template <typename VT, bool SET>
static void launch_vec(bool one_vec, bool through, int mode, unsigned grid, hipStream_t s,
                       const RowArgs &a) {
  if (SET && through && mode != kDirect) {
    if (one_vec)
      launch_through<VT, true>(mode, grid, s, a);
    else
      launch_through<VT, false>(mode, grid, s, a);
    return;
  }
  if (one_vec)
    launch_mode<VT, SET, true>(mode, grid, s, a);
  else
    launch_mode<VT, SET, false>(mode, grid, s, a);
}

template <bool SET>
static int move_rows(const char *who, void *miss, void *cache, const void *indices, int idx_bytes,
                     const shmt_hashmap_t *map, const void *mask, int mask_bytes, void *dense,
                     int64_t Q, int64_t row_bytes, void *stream, bool through = false,
                     const int64_t *count = nullptr, int64_t *count_seen = nullptr,
                     uint32_t *miss_bits = nullptr) {
  SHMT_REQUIRE(Q >= 0, "%s: Q must be >= 0", who);
  SHMT_REQUIRE(row_bytes > 0, "%s: row_bytes must be > 0", who);
  SHMT_REQUIRE(width_ok(idx_bytes), "%s: ID can only be int32 or int64 (idx_bytes=%d)", who, idx_bytes);
  SHMT_REQUIRE(!(map && mask), "%s: pass a hashmap or a mask, not both", who);
  if (Q == 0) return SHMT_OK;
  SHMT_REQUIRE(indices != nullptr && dense != nullptr, "%s: null indices/rows buffer", who);
  SHMT_REQUIRE(miss != nullptr, "%s: the id-addressed table is null", who);
  int mode = kDirect;
  if (map) {
    mode = map->kind != kKindBuckets ? kMapFlat : (map->fmt == kSlot16 ? kMap16 : kMap8);
    // an empty map never yields a slot, so an empty (null) cache table is fine with it
    SHMT_REQUIRE(cache != nullptr || map->n == 0, "%s: cache table is null", who);
  } else if (mask) {
    mode = kMask;
    SHMT_REQUIRE(width_ok(mask_bytes), "%s: mask can only be int32 or int64", who);
    SHMT_REQUIRE(cache != nullptr, "%s: cache table is null", who);
  }

  RowArgs a;
  a.miss = static_cast<char *>(miss);
  a.cache = static_cast<char *>(cache);
  a.dense = static_cast<char *>(dense);
  a.indices = indices;
  a.mask = mask;
  if (map) a.map = map->view; else a.map = empty_map_view();
  a.Q = Q;
  a.count = count;
  a.count_seen = count_seen;
  a.row_bytes = row_bytes;
  a.idx_bytes = idx_bytes;
  a.mask_bytes = mask_bytes;
  a.miss_bits = miss_bits;

  const int vb = pick_vector_bytes(row_bytes, miss, cache, dense);
  const int64_t nvec = row_bytes / vb;
  int log2_lanes = 3;
  while (log2_lanes < 6 && (1ll << log2_lanes) < nvec) ++log2_lanes;
  a.log2_lanes = log2_lanes;
  // Tile of 64 rows per wave when there are rows enough to occupy the chip
  // (256 CUs x 8 waves); fewer rows per wave otherwise, down to one phase-2 step.
  int log2_tile = kMaxLog2Tile;
  while (log2_tile > 6 - log2_lanes && (Q >> log2_tile) < 2048) --log2_tile;
  if (miss_bits) log2_tile = 5;  // one bitmap word per tile
  a.log2_tile = log2_tile;
  // As many workgroups as the device holds at once (256 units x 8 waves per SIMD): beyond that a wave takes
  // several tiles and keeps the lookups of the next ones in flight while it moves rows.
  const unsigned grid = grid_for(Q, static_cast<int64_t>(kRowsBlock / kWave) << log2_tile, 256 * 8);
  hipStream_t s = as_stream(stream);
  const bool one_vec = nvec <= (1ll << log2_lanes);
  if (miss_bits) {
    SHMT_REQUIRE(!SET && mode != kDirect, "%s: only a fetch through a hashmap or mask sets its misses aside", who);
    SHMT_REQUIRE(vb == 16, "%s: rows and tables must allow 16-byte accesses (row_bytes %lld)", who,
                 static_cast<long long>(row_bytes));
    SHMT_REQUIRE(Q < (1ll << 32), "%s: at most 2^32 - 1 rows", who);
    if (one_vec) launch_defer<true>(mode, grid, s, a); else launch_defer<false>(mode, grid, s, a);
    SHMT_LAUNCH_CHECK();
    return SHMT_OK;
  }
  switch (vb) {
    case 16: launch_vec<u32x4, SET>(one_vec, through, mode, grid, s, a); break;
    case 8: launch_vec<u32x2, SET>(one_vec, through, mode, grid, s, a); break;
    case 4: launch_vec<uint32_t, SET>(one_vec, through, mode, grid, s, a); break;
    case 2: launch_vec<uint16_t, SET>(one_vec, through, mode, grid, s, a); break;
    default: launch_vec<uint8_t, SET>(one_vec, through, mode, grid, s, a); break;
  }
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

}  // namespace shmt

extern "C" {

int shmt_fetch(const void *miss_data, const void *cache_data, const void *indices, int idx_bytes,
               const shmt_hashmap_t *map, const void *mask, int mask_bytes, void *out, int64_t Q,
               int64_t row_bytes, void *stream) {
  return shmt::move_rows<false>("shmt_fetch", const_cast<void *>(miss_data),
                                const_cast<void *>(cache_data), indices, idx_bytes, map, mask,
                                mask_bytes, out, Q, row_bytes, stream);
}

int shmt_fetch_counted(const void *miss_data, const void *cache_data, const void *indices,
                       int idx_bytes, const shmt_hashmap_t *map, const void *mask, int mask_bytes,
                       void *out, int64_t max_rows, const int64_t *count, int64_t *count_seen,
                       int64_t row_bytes, void *stream) {
  SHMT_REQUIRE(count != nullptr, "shmt_fetch_counted: count is null");
  return shmt::move_rows<false>("shmt_fetch_counted", const_cast<void *>(miss_data),
                                const_cast<void *>(cache_data), indices, idx_bytes, map, mask,
                                mask_bytes, out, max_rows, row_bytes, stream, false, count, count_seen);
}

int shmt_fetch_cached_part(const void *miss_data, const void *cache_data, const void *indices, int idx_bytes,
                           const shmt_hashmap_t *map, const void *mask, int mask_bytes, void *out,
                           int64_t max_rows, const int64_t *count, int64_t row_bytes, uint32_t *miss_bits,
                           void *stream) {
  SHMT_REQUIRE(miss_bits != nullptr || max_rows == 0, "shmt_fetch_cached_part: miss_bits is null");
  SHMT_REQUIRE(map != nullptr || mask != nullptr, "shmt_fetch_cached_part: needs a hashmap or a mask");
  return shmt::move_rows<false>("shmt_fetch_cached_part", const_cast<void *>(miss_data),
                                const_cast<void *>(cache_data), indices, idx_bytes, map, mask, mask_bytes, out,
                                max_rows, row_bytes, stream, false, count, nullptr, miss_bits);
}

int shmt_fetch_missed_part(const void *miss_data, const void *indices, int idx_bytes, const uint32_t *miss_bits,
                           void *out, int64_t max_rows, const int64_t *count, int64_t row_bytes, int max_blocks,
                           void *stream) {
  using namespace shmt;
  SHMT_REQUIRE(width_ok(idx_bytes), "shmt_fetch_missed_part: ID can only be int32 or int64 (idx_bytes=%d)", idx_bytes);
  SHMT_REQUIRE(max_rows >= 0 && max_rows < (1ll << 32), "shmt_fetch_missed_part: max_rows must be in [0, 2^32)");
  SHMT_REQUIRE(max_blocks >= 0, "shmt_fetch_missed_part: max_blocks must be >= 0");
  if (max_rows == 0) return SHMT_OK;
  SHMT_REQUIRE(miss_data && indices && miss_bits && out, "shmt_fetch_missed_part: null buffer");
  SHMT_REQUIRE(row_bytes > 0 && pick_vector_bytes(row_bytes, miss_data, out, nullptr) == 16,
               "shmt_fetch_missed_part: rows and tables must allow 16-byte accesses (row_bytes %lld)",
               static_cast<long long>(row_bytes));
  MissedArgs a;
  a.table = static_cast<const char *>(miss_data);
  a.dense = static_cast<char *>(out);
  a.indices = indices;
  a.bits = miss_bits;
  a.count = count;
  a.rows = max_rows;
  a.row_bytes = row_bytes;
  a.idx_bytes = idx_bytes;
  int log2_lanes = 3;
  while (log2_lanes < 6 && (1ll << log2_lanes) < row_bytes / 16) ++log2_lanes;
  a.log2_lanes = log2_lanes;
  const int64_t chunks = ((max_rows + 31) / 32 + kMissedChunk - 1) / kMissedChunk;
  const unsigned grid = grid_for(chunks, kRowsBlock / kWave, max_blocks > 0 ? max_blocks : kMissedBlocks);
  hipLaunchKernelGGL(rows_missed_kernel, dim3(grid), dim3(kRowsBlock), 0, as_stream(stream), a);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

int shmt_set(void *miss_data, void *cache_data, const void *indices, int idx_bytes,
             const shmt_hashmap_t *map, const void *mask, int mask_bytes, const void *update,
             int64_t Q, int64_t row_bytes, void *stream) {
  return shmt::move_rows<true>("shmt_set", miss_data, cache_data, indices, idx_bytes, map, mask,
                               mask_bytes, const_cast<void *>(update), Q, row_bytes, stream);
}

int shmt_set_through(void *miss_data, void *cache_data, const void *indices, int idx_bytes,
                     const shmt_hashmap_t *map, const void *mask, int mask_bytes, const void *update,
                     int64_t Q, int64_t row_bytes, void *stream) {
  return shmt::move_rows<true>("shmt_set_through", miss_data, cache_data, indices, idx_bytes, map, mask,
                               mask_bytes, const_cast<void *>(update), Q, row_bytes, stream, true);
}

}  // extern "C"
