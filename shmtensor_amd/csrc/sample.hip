// Uniform neighbour sampling over a CSR split between an HBM-resident cache
// of hot rows and a cold copy in pinned host memory, and construction of that
// cache. Replaces src/cache_graph_sampling.cu:47-492 in the ShmTensor tree.
//
// plan:  probe the cache map for 64 consecutive seeds per wave (8 cooperative
//        probes at a time), read the two row offsets from the cached or the
//        cold indptr, derive the output count and prefix-sum the counts in the
//        same kernel. Tiles of kPlanBlock (256) seeds: cold row offsets are
//        host-link reads and one compute unit keeps only so many in flight,
//        so small tiles on many units beat one large workgroup. Up to one tile
//        is one launch; beyond that each tile scans locally and the tile
//        offsets are added by two short kernels (or, in the fused hop, by the
//        pick kernel itself).
// pick:  a sub-wave group of G >= k lanes owns a seed. Rows with deg <= k are
//        copied in CSR order. Otherwise the k draws of Floyd's subset
//        algorithm are generated in parallel (one Philox block per lane) and
//        resolved in k ballot steps inside the group, so the cost is O(k) per
//        seed whatever the degree; the reference draws O(deg) numbers per seed
//        (src/cache_graph_sampling.cu:329-336). k > 64 uses one wave per seed
//        with the chosen set staged in LDS.
// hop:   shmt_sample_hop queues plan, pick and the relabel passes of
//        {seeds, sampled ids} as one sequence. The HOP forms of the kernels
//        do the relabel's preparation on the side: plan writes the seeds into
//        the relabel input, pick adds the tile offsets itself (every wave sums
//        the tile totals below its tile; a totals kernel only beyond 1,024
//        tiles) and publishes the total, writes every
//        sampled id into the relabel input too, empties the relabel table and
//        marks whether any id falls outside 32 bits. The number of seeds may
//        itself live in device memory (the count a previous hop produced):
//        launches and buffers are then sized for a bound and every kernel
//        clamps to the true number, so consecutive hops queue without a host
//        wait between them.
#include "common.h"
#include "hashmap.h"
#include "hashmap_dev.h"
#include "launchers.h"
#include "philox.h"
#include "scan_dev.h"

namespace shmt {

constexpr int kPlanBlock = 256;
constexpr int64_t kPlanSingleMax = 256;
constexpr int64_t kCachedTag = 1ll << 62;  // plan.begin carries the source in bit 62
constexpr int64_t kPickSumsTiles = 1024;  // up to this many plan tiles the fused hop needs no totals kernel
constexpr int kWideMaxPicks = 8192;  // chosen set of 8 B entries must fit 64 KiB of LDS

struct SeedPlan {
  int64_t begin;  // first adjacency element, | kCachedTag when it lives in the cache
  int64_t deg;
};

struct PlanArgs {
  const void *indptr;
  const void *cache_indptr;
  const void *seeds;
  void *sub_indptr;
  SeedPlan *plan;
  uint64_t *partials;
  int64_t *nnz_out;
  MapView map;
  int64_t S;
  int64_t k;
  int ptr_bytes;
  int seed_bytes;
  int replace;
  void *seed_copy;      // optional: seeds widened to seed_copy_bytes (head of a relabel input)
  int seed_copy_bytes;
  const int64_t *S_len;  // optional: true number of seeds in device memory, S is then its bound
  uint64_t *total_word;  // optional (single-workgroup form): second copy of the total, in device memory
};

// Number of seeds a kernel works on: the host's figure, or the device-side
// count clamped to it.
// A value every lane holds alike (loaded from one address), moved to scalar registers: what is compared
// with it, counted up to it or fed from it into the random number generator then stays scalar too. (The
// pick kernel needed 104 vector registers with its seed count and RNG seed in vector registers and 73 so.)
__device__ __forceinline__ int64_t wave_uniform(int64_t v) {
  const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(static_cast<uint64_t>(v))));
  const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(static_cast<uint64_t>(v) >> 32)));
  return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
}

__device__ __forceinline__ int64_t seed_count(int64_t bound, const int64_t *len) {
  if (!len) return bound;
  const int64_t n = wave_uniform(*len);
  return n < 0 ? 0 : (n < bound ? n : bound);
}

// MODE 0: no cache; 1: wide map; 2: narrow map.
template <int MODE>
__device__ __forceinline__ int64_t plan_one(const PlanArgs &a, int64_t S, int64_t i) {
  // called by whole waves; lanes past S use a harmless key and produce cnt 0
  const bool live = i < S;
  int64_t node = live ? load_int(a.seeds, i, a.seed_bytes) : -1;
  if (live && a.seed_copy) store_int(a.seed_copy, i, a.seed_copy_bytes, node);
  int64_t slot = -1;
  if (MODE == 1) slot = wave_find<kSlot16>(a.map, map_key(a.map, node));
  if (MODE == 2) slot = wave_find<kSlot8>(a.map, map_key(a.map, node));
  int64_t cnt = 0;
  if (live) {
    // both offsets of the row in flight together (cold rows: two host-link reads)
    int64_t begin, end;
    load_int_pair(slot >= 0 ? a.cache_indptr : a.indptr, slot >= 0 ? slot : node, a.ptr_bytes,
                  &begin, &end);
    const int64_t deg = end - begin;
    a.plan[i].begin = begin | (slot >= 0 ? kCachedTag : 0);
    a.plan[i].deg = deg;
    cnt = a.replace ? (deg > 0 ? a.k : 0) : (deg < a.k ? deg : a.k);
  }
  return cnt;
}

// One workgroup walks all seeds with a running carry and writes final offsets.
template <int MODE>
__device__ __forceinline__ void plan_single_body(const PlanArgs &a) {
  __shared__ uint64_t lds[kPlanBlock / kWave];
  const int64_t S = seed_count(a.S, a.S_len);
  uint64_t carry = 0;
  for (int64_t base = 0; base < S; base += kPlanBlock) {
    const int64_t i = base + threadIdx.x;
    const uint64_t cnt = static_cast<uint64_t>(plan_one<MODE>(a, S, i));
    uint64_t total;
    const uint64_t ex = block_exclusive_scan<uint64_t, kPlanBlock>(cnt, lds, &total);
    if (i < S) store_int(a.sub_indptr, i, a.ptr_bytes, static_cast<int64_t>(carry + ex));
    carry += total;
  }
  if (threadIdx.x == 0) {
    store_int(a.sub_indptr, S, a.ptr_bytes, static_cast<int64_t>(carry));
    if (a.total_word) *a.total_word = carry;
    publish_size(a.nnz_out, static_cast<int64_t>(carry));
  }
}

template <int MODE>
__global__ __launch_bounds__(kPlanBlock) void plan_single_kernel(PlanArgs a) {
  plan_single_body<MODE>(a);
}

// Merged form (see launchers.h): blockIdx.y selects the job.
template <int MODE>
__global__ __launch_bounds__(kPlanBlock) void plan_single_jobs(Jobs<PlanArgs> j) {
  plan_single_body<MODE>(j.a[blockIdx.y]);
}

// Multi-workgroup form: tile-local offsets + one total per tile. (bx, gx):
// this workgroup's index and the number of workgroups of its job.
template <int MODE>
__device__ __forceinline__ void plan_tile_body(unsigned bx, unsigned gx, const PlanArgs &a) {
  __shared__ uint64_t lds[kPlanBlock / kWave];
  const int64_t S = seed_count(a.S, a.S_len);
  if (bx > 0 && static_cast<int64_t>(bx) * kPlanBlock >= S) {  // launched for a bound of S: an empty tile
    if (threadIdx.x == 0) a.partials[bx] = 0;
    return;
  }
  const int64_t i = static_cast<int64_t>(bx) * kPlanBlock + threadIdx.x;
  const uint64_t cnt = static_cast<uint64_t>(plan_one<MODE>(a, S, i));
  uint64_t total;
  const uint64_t ex = block_exclusive_scan<uint64_t, kPlanBlock>(cnt, lds, &total);
  if (i < S) store_int(a.sub_indptr, i, a.ptr_bytes, static_cast<int64_t>(ex));
  if (threadIdx.x == 0) {
    a.partials[bx] = total;
    if (bx == 0) a.partials[gx] = 0;  // becomes the grand total after the scan
  }
}

template <int MODE>
__global__ __launch_bounds__(kPlanBlock) void plan_tile_kernel(PlanArgs a) {
  plan_tile_body<MODE>(blockIdx.x, gridDim.x, a);
}

template <int MODE>
__global__ __launch_bounds__(kPlanBlock) void plan_tile_jobs(Jobs<PlanArgs> j) {
  if (blockIdx.x < j.blocks[blockIdx.y]) plan_tile_body<MODE>(blockIdx.x, j.blocks[blockIdx.y], j.a[blockIdx.y]);
}

// Adds the scanned tile offsets to the tile-local offsets. partials holds
// nb + 1 scanned entries: partials[t] = sum of the tiles before t, and
// partials[nb] = grand total, which becomes data[n] and *total_out.
__global__ __launch_bounds__(256) void add_tile_offsets_kernel(void *data, int eb, int64_t n,
                                                               const uint64_t *partials,
                                                               int64_t tile, int64_t nb,
                                                               int64_t *total_out) {
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (; i <= n; i += stride) {
    if (i < n) {
      store_int(data, i, eb, load_int(data, i, eb) + static_cast<int64_t>(partials[i / tile]));
    } else {
      const int64_t t = static_cast<int64_t>(partials[nb]);
      store_int(data, n, eb, t);
      publish_size(total_out, t);
    }
  }
}

// Fused-hop form of the two kernels above: scans the nb tile totals in place
// (partials[nb] becomes the grand total) and publishes the total; the tile
// offsets themselves are added by the pick kernel.
__global__ __launch_bounds__(1024) void plan_totals_kernel(uint64_t *partials, int64_t nb,
                                                           void *sub_indptr, int ptr_bytes,
                                                           int64_t S_bound, const int64_t *S_len,
                                                           int64_t *nnz_out) {
  __shared__ uint64_t lds[1024 / kWave];
  const int64_t S = seed_count(S_bound, S_len);
  uint64_t carry = 0;
  for (int64_t base = 0; base < nb; base += 1024) {
    const int64_t i = base + threadIdx.x;
    const uint64_t v = i < nb ? partials[i] : 0;
    uint64_t total;
    const uint64_t ex = block_exclusive_scan<uint64_t, 1024>(v, lds, &total);
    if (i < nb) partials[i] = carry + ex;
    carry += total;
  }
  if (threadIdx.x == 0) {
    partials[nb] = carry;
    store_int(sub_indptr, S, ptr_bytes, static_cast<int64_t>(carry));
    publish_size(nnz_out, static_cast<int64_t>(carry));
  }
}

// ---- pick ------------------------------------------------------------------

struct PickArgs {
  const void *indices;
  const void *cache_indices;
  const void *seeds;
  const void *sub_indptr;
  const SeedPlan *plan;
  void *out;
  int64_t S;
  int64_t k;
  uint64_t rng_seed;
  uint32_t rng_stream;
  int idx_bytes;
  int seed_bytes;
  int ptr_bytes;
  int replace;
  int log2_group;  // lanes per seed (narrow kernel)
  int rounds;      // seeds a lane group handles per pass (narrow kernel), 1 .. kPickRounds
  // fused hop only (HOP kernels):
  void *sub_indptr_rw;          // tile-local offsets in, final offsets out
  const uint64_t *tile_prefix;  // totals of the plan's seed tiles, or null when offsets are final: scanned
  int64_t raw_tiles;            // (raw_tiles == 0), or that many raw totals which this kernel sums itself,
  int64_t *nnz_out;             // then also publishing the grand total (sub_indptr[S], total_word, *nnz_out)
  uint64_t *total_word;
  const int64_t *S_len;         // optional: true number of seeds in device memory, S is then its bound
  const uint64_t *rng_seed_dev; // optional: the RNG seed lives in device memory (replayed launch sequences)
  void *copy_out;               // second copy of every sampled id, widened to copy_bytes, at
  int copy_bytes;               // copy_out[number of seeds + offset]: the relabel input after the seeds
  uint4 *clear;                 // clear_n 16-byte words set to all ones (the relabel table)
  int64_t clear_n;
  uint64_t *wide_mark;          // receives wide_nonce when a seed or a sampled id lies outside [0, 2^32)
  uint64_t wide_nonce;
  void *coo_out;                // optional: position of the seed each sampled id belongs to (the destination
  int coo_bytes;                // side of the block's edges in coordinate form), coo_bytes wide
};

__device__ __forceinline__ void note_wide_id(const PickArgs &a, int64_t id) {
  if (a.wide_mark && (static_cast<uint64_t>(id) >> 32)) *a.wide_mark = a.wide_nonce;
}

// Sum of the first `count` raw tile totals, by a whole wave (all lanes active).
__device__ __forceinline__ int64_t wave_sum_tiles(const uint64_t *totals, int64_t count) {
  uint64_t acc = 0;
  for (int64_t t = lane_id(); t < count; t += kWave) acc += totals[t];
  return static_cast<int64_t>(wave_last(wave_inclusive_scan(acc)));
}

// Output offset that precedes the plan tile of seed s (fused hop; wave-uniform s / kPlanBlock,
// all lanes active): the scanned tile total, or the sum of the raw totals below the tile.
__device__ __forceinline__ int64_t pick_tile_base(const PickArgs &a, int64_t s) {
  if (!a.tile_prefix) return 0;
  const int64_t tile = s / kPlanBlock;
  return a.raw_tiles ? wave_sum_tiles(a.tile_prefix, tile) : static_cast<int64_t>(a.tile_prefix[tile]);
}

// With raw tile totals nobody has published the grand total yet: the first wave of the grid does.
__device__ __forceinline__ void pick_publish_total(const PickArgs &a, int64_t S, unsigned bx) {
  if (!a.raw_tiles || bx != 0 || threadIdx.x >= kWave) return;
  const int64_t total = wave_sum_tiles(a.tile_prefix, a.raw_tiles);
  if (threadIdx.x == 0) {
    store_int(a.sub_indptr_rw, S, a.ptr_bytes, total);
    *a.total_word = static_cast<uint64_t>(total);
    publish_size(a.nnz_out, total);
  }
}

// Output offset of seed s. In the fused hop the plan left tile-local offsets:
// the tile's base is added here and the final value written back by `writer`.
template <bool HOP>
__device__ __forceinline__ int64_t pick_offset(const PickArgs &a, int64_t s, int64_t tile_base, bool writer) {
  if (!HOP) return load_int(a.sub_indptr, s, a.ptr_bytes);
  int64_t optr = load_int(a.sub_indptr_rw, s, a.ptr_bytes);
  if (writer && a.wide_mark) note_wide_id(a, load_int(a.seeds, s, a.seed_bytes));
  if (a.tile_prefix) {
    optr += tile_base;
    if (writer) store_int(a.sub_indptr_rw, s, a.ptr_bytes, optr);
  }
  return optr;
}

// s: position of the seed the id was sampled for.
template <bool HOP>
__device__ __forceinline__ void pick_store(const PickArgs &a, int64_t S, int64_t s, int64_t pos, int64_t v) {
  store_int(a.out, pos, a.idx_bytes, v);
  if (HOP && a.copy_out) {
    store_int(a.copy_out, S + pos, a.copy_bytes, v);
    note_wide_id(a, v);
  }
  if (HOP && a.coo_out) store_int(a.coo_out, pos, a.coo_bytes, s);
}

template <bool HOP>
__device__ __forceinline__ void pick_clear(const PickArgs &a, unsigned bx, unsigned gx) {
  if (!HOP) return;
  const uint4 ones = make_uint4(~0u, ~0u, ~0u, ~0u);
  const int64_t stride = static_cast<int64_t>(gx) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(bx) * blockDim.x + threadIdx.x; i < a.clear_n; i += stride)
    a.clear[i] = ones;
}

__device__ __forceinline__ int64_t load_adj(const PickArgs &a, int64_t begin_tagged, int64_t pos) {
  const void *base = (begin_tagged & kCachedTag) ? a.cache_indices : a.indices;
  return load_int(base, (begin_tagged & ~kCachedTag) + pos, a.idx_bytes);
}

// Floyd's subset selection resolved inside a group of G lanes, positions of 32
// bits. Lane j (j < k) brings its draw t_j in [0, top_j], top_j = deg - k + j;
// the chosen position of step j is t_j unless an earlier step already chose
// that value, and top_j then (which no earlier step can have chosen). Steps
// run in order: at step s the choice of lane s is final (it has seen the
// choices of all steps before it) and is handed to the lanes behind it, which
// note whether it equals their own draw. Lanes at or beyond k take no part in
// the result. Groups of 16 and 32 lanes do not walk through the steps at all
// while positions fit 27 bits (see the comment inside); the stepwise forms
// remain for rows beyond that, for groups of 64 (one readlane per step, the
// "already chosen" flags kept as one 64-bit lane mask) and for groups below 16
// (at most seven steps, a lane permute each).
// Sorting network for the resolution below: bitonic sort, ascending, of one
// 32-bit key per lane within every group of G lanes (G = 16 or 32). A stage
// exchanges keys between lanes l and l ^ STRIDE (ds_swizzle in bit mode: no
// memory is touched) and keeps the smaller or the larger one; which lanes keep
// the smaller one is a constant of the stage.
template <int G>
constexpr uint64_t bitonic_keeps_min(int size, int stride) {
  uint64_t m = 0;
  for (int l = 0; l < kWave; ++l) {
    const int gl = l & (G - 1);
    const bool up = (gl & size) == 0, lower = (gl & stride) == 0;
    if (up == lower) m |= 1ull << l;
  }
  return m;
}

template <int G, int SIZE, int STRIDE>
__device__ __forceinline__ uint32_t bitonic_sort_from(uint32_t key) {
  constexpr int kPattern = (STRIDE << 10) | 0x1F;  // bit mode: and 0x1F, or 0, xor STRIDE
  constexpr uint64_t kKeepsMin = bitonic_keeps_min<G>(SIZE, STRIDE);
  const uint32_t other = static_cast<uint32_t>(__builtin_amdgcn_ds_swizzle(static_cast<int>(key), kPattern));
  const uint32_t lo = key < other ? key : other, hi = key < other ? other : key;
  key = __builtin_amdgcn_inverse_ballot_w64(kKeepsMin) ? lo : hi;
  if constexpr (STRIDE > 1) return bitonic_sort_from<G, SIZE, STRIDE / 2>(key);
  else if constexpr (SIZE < G) return bitonic_sort_from<G, SIZE * 2, SIZE>(key);
  else return key;
}

// "Some lane before mine in my group drew the same value": the first of the
// two ways in which a step of Floyd's selection falls back to its J (see
// floyd_resolve32). The draws are sorted together with their
// lane numbers ((t << 5) | gl, which needs t < 2^27 - 1), equal draws then
// stand side by side in lane order, every one but the first is such a repeat,
// and the flag travels back to its lane with one permute. 15 exchange stages
// for 32 lanes (10 for 16) instead of one dependent step per pick: measured
// on 105,000 seeds with 25 picks each, 58.5 -> 52.5 us for the whole kernel.
// (Sorting the draws of the four rounds of a pass stage by stage side by side
// measured 1 us slower than one round after the other.)
template <int G>
__device__ __forceinline__ bool repeats_earlier_draw(uint32_t t, bool live, int gl) {
  static_assert(G == 16 || G == 32, "one swizzle domain holds one or two whole groups");
  const uint32_t key = live ? ((t << 5) | static_cast<uint32_t>(gl)) : (0xFFFFFFE0u | static_cast<uint32_t>(gl));
  const uint32_t sorted = bitonic_sort_from<G, 2, 1>(key);
  const uint32_t before = static_cast<uint32_t>(__shfl_up(static_cast<int>(sorted), 1, kWave));
  const bool repeat = gl != 0 && (before >> 5) == (sorted >> 5) && sorted < 0xFFFFFFE0u;
  const int home = (lane_id() & ~(G - 1)) + static_cast<int>(sorted & 31u);
  return __builtin_amdgcn_ds_permute(home << 2, repeat ? 1 : 0) != 0;
}

template <int G>
__device__ __forceinline__ uint32_t floyd_resolve32(uint32_t t, uint32_t top, int gl, int k) {
  if constexpr (G == 16 || G == 32) {
    // Step j falls back to J = top_j exactly when t_j is among the earlier choices, and that is the case
    // when (a) an earlier lane drew the same value (its choice, or an earlier one, is that value), or
    // (b) t_j is the J of an earlier step i = t_j - (deg - k) < j that fell back itself. (a) needs no
    // step to wait for another; (b) hangs a lane on one earlier lane, needs a draw among the k largest
    // positions (probability about k / deg) and is settled by following those links until nothing
    // changes: a link leads to a smaller lane, so every round settles at least one more lane.
    const uint32_t base = top - static_cast<uint32_t>(gl);  // deg - k, the same for the whole group
    const bool live = gl < k;
    const bool packs = base < (1u << 27) - 64u;
    if (__builtin_amdgcn_ballot_w64(!packs) == 0) {
      bool hit = repeats_earlier_draw<G>(t, live, gl) && live;
      const bool linked = live && t >= base && static_cast<int>(t - base) < gl;
      const int from = (lane_id() & ~(G - 1)) + static_cast<int>(linked ? t - base : 0u);
      if (__builtin_amdgcn_ballot_w64(linked) != 0) {
        for (;;) {
          const uint64_t hits = __builtin_amdgcn_ballot_w64(hit);
          const bool now = hit || (linked && ((hits >> from) & 1ull) != 0);
          if (__builtin_amdgcn_ballot_w64(now != hit) == 0) break;
          hit = now;
        }
      }
      return hit ? top : t;
    }
  }
  if (G == 32) {
    uint64_t hit = 0;
    for (int step = 0; step + 1 < k; ++step) {
      const uint32_t c = __builtin_amdgcn_inverse_ballot_w64(hit) ? top : t;
      const uint32_t c0 = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(c), step));
      const uint32_t c1 = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(c), 32 + step));
      const uint64_t m0 = __builtin_amdgcn_ballot_w64(t == c0), m1 = __builtin_amdgcn_ballot_w64(t == c1);
      const uint32_t behind = 0xFFFFFFFEu << step;  // lanes of a group with gl > step
      hit |= (static_cast<uint64_t>(static_cast<uint32_t>(m1 >> 32) & behind) << 32) |
             (static_cast<uint32_t>(m0) & behind);
    }
    return __builtin_amdgcn_inverse_ballot_w64(hit) ? top : t;
  }
  if (G >= 16) {
    constexpr int kGroups = kWave / G;
    // bit l of `behind`: lane l lies behind the current step in its group (gl > step)
    constexpr uint64_t kLowBits = G == 64 ? 1ull : G == 32 ? 0x0000000100000001ull : 0x0001000100010001ull;
    constexpr uint64_t kGroupLanes = G == 64 ? ~0ull : (1ull << (G % 64)) - 1ull;
    uint64_t behind = ~kLowBits;
    uint64_t hit = 0;
    for (int step = 0; step + 1 < k; ++step) {
      const uint32_t c = __builtin_amdgcn_inverse_ballot_w64(hit) ? top : t;
      uint64_t same = 0;  // lanes whose draw equals the choice their group just made
#pragma unroll
      for (int g = 0; g < kGroups; ++g) {
        const uint32_t chosen = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(c), g * G + step));
        same |= __builtin_amdgcn_ballot_w64(t == chosen) & (kGroupLanes << (g * G));
      }
      hit |= same & behind;
      behind = (behind << 1) & ~kLowBits;
    }
    return __builtin_amdgcn_inverse_ballot_w64(hit) ? top : t;
  }
  bool hit = false;
  for (int step = 0; step + 1 < k; ++step) {
    const uint32_t c = hit ? top : t;
    const uint32_t chosen = static_cast<uint32_t>(__shfl(static_cast<int>(c), (lane_id() & ~(G - 1)) + step, kWave));
    hit |= (gl > step) && (chosen == t);
  }
  return hit ? top : t;
}

// One adjacency element, issued without touching the loaded value: 4-byte
// elements come back zero-extended and are sign-extended by adj_value() when
// they are stored, so that several such loads stay in flight together.
__device__ __forceinline__ int64_t issue_adj(const PickArgs &a, int64_t begin_tagged, int64_t pos) {
  const void *base = (begin_tagged & kCachedTag) ? a.cache_indices : a.indices;
  const int64_t i = (begin_tagged & ~kCachedTag) + pos;
  if (a.idx_bytes == 8) return static_cast<const int64_t *>(base)[i];
  return static_cast<int64_t>(static_cast<const uint32_t *>(base)[i]);
}
__device__ __forceinline__ int64_t adj_value(const PickArgs &a, int64_t raw) {
  return a.idx_bytes == 8 ? raw : static_cast<int64_t>(static_cast<int32_t>(static_cast<uint32_t>(raw)));
}

constexpr int kPickRounds = 4;  // seeds a lane group handles per pass, at most: that many adjacency loads in flight

// k <= 64: group of G = 2^LG >= k lanes per seed. (bx, gx): this workgroup's
// index and the number of workgroups of its job. A wave takes `rounds` x 64 / G
// consecutive seeds per pass (a.rounds <= kPickRounds; they share a plan
// tile): first one lane per seed fetches the seed's plan entry, output offset
// and id in coalesced loads (and finishes the offset: the fused hop's plan
// leaves tile-local offsets), then the lane groups take the seeds round by
// round, choose their positions and issue the adjacency loads of all rounds
// before the first value is stored. The chain of dependent memory round trips
// per pass is plan entry -> adjacency -> store whatever the number of rounds;
// measured on 127,000 seeds with 25 picks each: 98 us with one seed per group
// and pass (four dependent chains per wave one after the other), 79 us so.
// Capping the kernel at 64 registers for eight resident waves per SIMD spills
// and measured 150 us; two rounds per pass instead of four measured the same.
template <bool HOP, int LG>
__device__ __forceinline__ void pick_narrow_body(unsigned bx, unsigned gx, const PickArgs &a) {
  pick_clear<HOP>(a, bx, gx);
  constexpr int G = 1 << LG;
  constexpr int kGroups = kWave / G;
  const int lane = lane_id();
  const int gl = lane & (G - 1);
  const int grp = lane >> LG;
  const int64_t waves_per_block = blockDim.x / kWave;
  const int64_t wave = static_cast<int64_t>(bx) * waves_per_block + threadIdx.x / kWave;
  const int64_t nwaves = static_cast<int64_t>(gx) * waves_per_block;
  const int k = static_cast<int>(a.k);
  const int rounds = a.rounds;
  const int per_pass = rounds * kGroups;  // <= 64 and a divisor of kPlanBlock
  const int64_t S = HOP ? seed_count(a.S, a.S_len) : a.S;
  const uint64_t rng_seed =
      HOP && a.rng_seed_dev ? static_cast<uint64_t>(wave_uniform(static_cast<int64_t>(*a.rng_seed_dev))) : a.rng_seed;
  if (HOP) pick_publish_total(a, S, bx);

  for (int64_t w0 = wave * per_pass; w0 < S; w0 += nwaves * per_pass) {
    const int64_t tile_base = HOP ? pick_tile_base(a, w0) : 0;
    // one lane per seed of the pass
    const int64_t sl = w0 + lane;
    const bool seed_live = lane < per_pass && sl < S;
    SeedPlan pl{0, 0};
    int64_t optr_l = 0, node_l = 0;
    if (seed_live) {
      pl = a.plan[sl];
      node_l = load_int(a.seeds, sl, a.seed_bytes);
      if (!HOP) {
        optr_l = load_int(a.sub_indptr, sl, a.ptr_bytes);
      } else {
        optr_l = load_int(a.sub_indptr_rw, sl, a.ptr_bytes);
        note_wide_id(a, node_l);
        if (a.tile_prefix) {
          optr_l += tile_base;
          store_int(a.sub_indptr_rw, sl, a.ptr_bytes, optr_l);
        }
      }
    }
    int64_t raw[kPickRounds], where[kPickRounds];
#pragma unroll
    for (int r = 0; r < kPickRounds; ++r) {
      where[r] = -1;  // nothing to store for this lane in round r
      if (r >= rounds) continue;
      const int src = r * kGroups + grp;
      const int64_t begin = shfl64(pl.begin, src);
      const int64_t deg = shfl64(pl.deg, src);
      const int64_t optr = shfl64(optr_l, src);
      const int64_t node = shfl64(node_l, src);
      if (w0 + src >= S || deg <= 0) continue;  // uniform within the group
      int64_t pos = -1;  // position in the row this lane reads
      if (a.replace) {
        if (gl < k) pos = static_cast<int64_t>(sample_draw(rng_seed, a.rng_stream, node, gl, static_cast<uint64_t>(deg)));
      } else if (deg <= k) {
        if (gl < deg) pos = gl;
      } else if (deg <= static_cast<int64_t>(0xFFFFFFFFu)) {
        // Floyd with 32-bit positions (every degree met in practice)
        const uint32_t top = static_cast<uint32_t>(deg - k + gl);  // J of this lane's step
        uint32_t t = 0;
        if (gl < k) t = sample_draw32(rng_seed, a.rng_stream, node, gl, top + 1u);
        const uint32_t mine = floyd_resolve32<G>(t, top, gl, k);
        if (gl < k) pos = mine;
      } else {
        // Floyd: for J = deg-k .. deg-1 draw t in [0, J]; take t unless already
        // taken, then take J. Draws in parallel, resolution in k ballot steps.
        int64_t t = 0;
        if (gl < k)
          t = static_cast<int64_t>(sample_draw(rng_seed, a.rng_stream, node, gl,
                                               static_cast<uint64_t>(deg - k + gl + 1)));
        int64_t mine = -1;
        for (int step = 0; step < k; ++step) {
          const int64_t ts = shfl64(t, (lane & ~(G - 1)) + step);
          const bool taken = group_ballot<G>(gl < step && mine == ts) != 0;
          if (gl == step) mine = taken ? (deg - k + step) : ts;
        }
        if (gl < k) pos = mine;
      }
      if (pos >= 0) {
        raw[r] = issue_adj(a, begin, pos);
        where[r] = optr + gl;
      }
    }
#pragma unroll
    for (int r = 0; r < kPickRounds; ++r)
      if (where[r] >= 0) pick_store<HOP>(a, S, w0 + r * kGroups + grp, where[r], adj_value(a, raw[r]));
  }
}

template <bool HOP, int LG>
__global__ __launch_bounds__(256) void pick_narrow_kernel(PickArgs a) {
  pick_narrow_body<HOP, LG>(blockIdx.x, gridDim.x, a);
}

template <int LG>
__global__ __launch_bounds__(256) void pick_narrow_hop_jobs(Jobs<PickArgs> j) {
  if (blockIdx.x < j.blocks[blockIdx.y]) pick_narrow_body<true, LG>(blockIdx.x, j.blocks[blockIdx.y], j.a[blockIdx.y]);
}

// k > 64: one wave (= one 64-thread workgroup) per seed. The chosen positions
// are staged in LDS when k fits (IN_LDS), otherwise in the seed's own output
// segment, which is overwritten by the gathered neighbours at the end
// (positions are < deg and therefore fit the index width).
template <bool IN_LDS, bool HOP>
__global__ __launch_bounds__(64) void pick_wide_kernel(PickArgs a) {
  extern __shared__ int64_t chosen_lds[];
  pick_clear<HOP>(a, blockIdx.x, gridDim.x);
  const int lane = threadIdx.x;
  const int64_t k = a.k;
  const int64_t S = HOP ? seed_count(a.S, a.S_len) : a.S;
  const uint64_t rng_seed =
      HOP && a.rng_seed_dev ? static_cast<uint64_t>(wave_uniform(static_cast<int64_t>(*a.rng_seed_dev))) : a.rng_seed;
  if (HOP) pick_publish_total(a, S, blockIdx.x);
  for (int64_t s = blockIdx.x; s < S; s += gridDim.x) {
    const SeedPlan p = a.plan[s];
    const int64_t deg = p.deg;
    const int64_t optr = pick_offset<HOP>(a, s, HOP ? pick_tile_base(a, s) : 0, lane == 0);
    if (deg <= 0) continue;
    const int64_t node = load_int(a.seeds, s, a.seed_bytes);
    if (a.replace) {
      for (int64_t j = lane; j < k; j += kWave) {
        const uint64_t r = sample_draw(rng_seed, a.rng_stream, node, static_cast<uint32_t>(j),
                                       static_cast<uint64_t>(deg));
        pick_store<HOP>(a, S, s, optr + j, load_adj(a, p.begin, static_cast<int64_t>(r)));
      }
    } else if (deg <= k) {
      for (int64_t j = lane; j < deg; j += kWave) pick_store<HOP>(a, S, s, optr + j, load_adj(a, p.begin, j));
    } else {
      for (int64_t step = 0; step < k; ++step) {
        const int64_t J = deg - k + step;
        const int64_t t = static_cast<int64_t>(sample_draw(
            rng_seed, a.rng_stream, node, static_cast<uint32_t>(step), static_cast<uint64_t>(J + 1)));
        bool taken = false;
        for (int64_t q = lane; q < step; q += kWave) {
          const int64_t c = IN_LDS ? chosen_lds[q] : load_int(a.out, optr + q, a.idx_bytes);
          taken |= (c == t);
        }
        const bool any = __builtin_amdgcn_ballot_w64(taken) != 0;
        if (lane == 0) {
          if (IN_LDS)
            chosen_lds[step] = any ? J : t;
          else
            store_int(a.out, optr + step, a.idx_bytes, any ? J : t);
        }
        __syncthreads();  // single-wave workgroup: orders the staging write before the next reads
      }
      for (int64_t j0 = 0; j0 < k; j0 += kWave) {
        const int64_t j = j0 + lane;
        int64_t c = 0;
        if (j < k) c = IN_LDS ? chosen_lds[j] : load_int(a.out, optr + j, a.idx_bytes);
        __syncthreads();
        if (j < k) pick_store<HOP>(a, S, s, optr + j, load_adj(a, p.begin, c));
      }
      __syncthreads();
    }
  }
}

// ---- cached sub-CSR ----------------------------------------------------------

__global__ __launch_bounds__(256) void subcsr_degree_kernel(const void *indptr, int ptr_bytes,
                                                            const void *seeds, int seed_bytes,
                                                            int64_t C, void *cache_indptr) {
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (; i <= C; i += stride) {
    int64_t d = 0;
    if (i < C) {
      const int64_t v = load_int(seeds, i, seed_bytes);
      d = load_int(indptr, v + 1, ptr_bytes) - load_int(indptr, v, ptr_bytes);
    }
    store_int(cache_indptr, i, ptr_bytes, d);
  }
}

__global__ void copy_total_kernel(const void *data, int eb, int64_t n, int64_t *total_out) {
  publish_size(total_out, load_int(data, n, eb));
}

// Last row r in [lo, hi] with offsets[r] <= e.
__device__ __forceinline__ int64_t row_of(const void *offsets, int eb, int64_t lo, int64_t hi,
                                          int64_t e) {
  while (lo < hi) {
    const int64_t mid = (lo + hi + 1) >> 1;
    if (load_int(offsets, mid, eb) <= e)
      lo = mid;
    else
      hi = mid - 1;
  }
  return lo;
}

constexpr int kCopyChunk = 256 * 8;

// Element-parallel copy: a workgroup owns a contiguous chunk of the output,
// brackets the rows that chunk can touch once, and every element then finds
// its row inside that bracket, so hub rows and empty rows cost the same.
__global__ __launch_bounds__(256) void subcsr_copy_kernel(const void *indptr, const void *indices,
                                                          int ptr_bytes, int idx_bytes,
                                                          const void *seeds, int seed_bytes,
                                                          int64_t C, const void *cache_indptr,
                                                          int64_t nnz, void *cache_indices) {
  __shared__ int64_t bracket[2];
  const int64_t nchunks = (nnz + kCopyChunk - 1) / kCopyChunk;
  for (int64_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
    const int64_t e0 = c * kCopyChunk;
    const int64_t e1 = (e0 + kCopyChunk < nnz ? e0 + kCopyChunk : nnz) - 1;
    if (threadIdx.x < 2)
      bracket[threadIdx.x] = row_of(cache_indptr, ptr_bytes, 0, C - 1, threadIdx.x == 0 ? e0 : e1);
    __syncthreads();
    const int64_t rlo = bracket[0], rhi = bracket[1];
#pragma unroll 2
    for (int j = 0; j < 8; ++j) {
      const int64_t e = e0 + j * 256 + threadIdx.x;
      if (e <= e1) {
        const int64_t r = row_of(cache_indptr, ptr_bytes, rlo, rhi, e);
        const int64_t v = load_int(seeds, r, seed_bytes);
        const int64_t src = load_int(indptr, v, ptr_bytes) + (e - load_int(cache_indptr, r, ptr_bytes));
        store_int(cache_indices, e, idx_bytes, load_int(indices, src, idx_bytes));
      }
    }
    __syncthreads();
  }
}

// rows_out[e] = the row r with offsets[r] <= e < offsets[r + 1], for every e < nnz: the row
// coordinate of each element of a CSR / CSC structure. Element-parallel like the copy above.
__global__ __launch_bounds__(256) void csr_rows_kernel(const void *offsets, int ptr_bytes, int64_t S,
                                                       int64_t nnz, void *rows_out, int out_bytes) {
  __shared__ int64_t bracket[2];
  const int64_t nchunks = (nnz + kCopyChunk - 1) / kCopyChunk;
  for (int64_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
    const int64_t e0 = c * kCopyChunk;
    const int64_t e1 = (e0 + kCopyChunk < nnz ? e0 + kCopyChunk : nnz) - 1;
    if (threadIdx.x < 2)
      bracket[threadIdx.x] = row_of(offsets, ptr_bytes, 0, S - 1, threadIdx.x == 0 ? e0 : e1);
    __syncthreads();
    const int64_t rlo = bracket[0], rhi = bracket[1];
    for (int j = 0; j < 8; ++j) {
      const int64_t e = e0 + j * 256 + threadIdx.x;
      if (e <= e1) store_int(rows_out, e, out_bytes, row_of(offsets, ptr_bytes, rlo, rhi, e));
    }
    __syncthreads();
  }
}

}  // namespace shmt

using namespace shmt;

extern "C" {

int64_t shmt_sample_plan_bytes(int64_t S) {
  if (S < 0) return -1;
  const int64_t nb = (S + kPlanBlock - 1) / kPlanBlock;
  return S * static_cast<int64_t>(sizeof(SeedPlan)) + (nb + 2) * 8;
}

// hop != null: fused-hop form. The seeds are also written, widened, to
// hop->seed_copy, and beyond one tile the offsets stay tile-local: only the
// scanned tile totals and the grand total are produced (*tile_prefix_out), the
// pick kernel adds them.
struct PlanHopExtras {
  void *seed_copy;
  int seed_copy_bytes;
  const int64_t *S_len;             // true number of seeds in device memory, or null
  const uint64_t *tile_prefix_out;
  const uint64_t *total_out;        // where the kernels leave the total (nnz) in device memory
  int64_t raw_tiles_out;            // > 0: tile_prefix_out holds that many raw totals, the pick kernel sums them
};

static int plan_impl(const void *indptr, int ptr_bytes, const void *cache_indptr,
                     const shmt_hashmap_t *map, const void *seeds, int seed_bytes, int64_t S,
                     int64_t k, int replace, void *sub_indptr, void *plan, int64_t plan_bytes,
                     int64_t *nnz_out, Launcher launcher, PlanHopExtras *hop) {
  SHMT_REQUIRE(S >= 0, "shmt_sample_plan: S must be >= 0");
  SHMT_REQUIRE(k >= 0, "shmt_sample_plan: num_picks must be >= 0");
  SHMT_REQUIRE(width_ok(ptr_bytes) && width_ok(seed_bytes),
               "shmt_sample_plan: ID can only be int32 or int64");
  SHMT_REQUIRE(sub_indptr != nullptr && nnz_out != nullptr, "shmt_sample_plan: null output");
  SHMT_REQUIRE(indptr != nullptr, "shmt_sample_plan: indptr is null");
  SHMT_REQUIRE(map == nullptr || cache_indptr != nullptr, "shmt_sample_plan: cache_indptr is null");
  if (S > 0) {
    SHMT_REQUIRE(seeds != nullptr, "shmt_sample_plan: seeds is null");
    if (plan == nullptr || plan_bytes < shmt_sample_plan_bytes(S)) {
      set_error("shmt_sample_plan: plan buffer too small (%lld < %lld bytes)",
                static_cast<long long>(plan_bytes), static_cast<long long>(shmt_sample_plan_bytes(S)));
      return SHMT_ENOMEM;
    }
    SHMT_REQUIRE((reinterpret_cast<uintptr_t>(plan) & 15) == 0,
                 "shmt_sample_plan: plan must be 16-byte aligned");
  }
  hipStream_t s = launcher.stream;
  StageList *const defer = launcher.defer;
  PlanArgs a;
  a.indptr = indptr;
  a.cache_indptr = cache_indptr;
  a.seeds = seeds;
  a.sub_indptr = sub_indptr;
  a.plan = static_cast<SeedPlan *>(plan);
  a.partials = S > 0 ? reinterpret_cast<uint64_t *>(static_cast<char *>(plan) + S * sizeof(SeedPlan))
                     : nullptr;
  a.nnz_out = nnz_out;
  if (map) a.map = map->view; else a.map = empty_map_view();
  a.S = S;
  a.k = k;
  a.ptr_bytes = ptr_bytes;
  a.seed_bytes = seed_bytes;
  a.replace = replace ? 1 : 0;
  a.seed_copy = hop ? hop->seed_copy : nullptr;
  a.seed_copy_bytes = hop ? hop->seed_copy_bytes : 8;
  a.S_len = hop ? hop->S_len : nullptr;
  const int64_t tiles = (S + kPlanBlock - 1) / kPlanBlock;
  a.total_word = hop && S > 0 ? a.partials + tiles : nullptr;  // where plan_totals_kernel leaves it too
  if (hop) {
    hop->tile_prefix_out = nullptr;
    hop->total_out = a.total_word;
    hop->raw_tiles_out = 0;
  }
  const int mode = map ? (map->fmt == kSlot16 ? 1 : 2) : 0;

  if (S <= kPlanSingleMax) {
    if (defer) {
      stage_push(defer, kStagePlanSingle + mode, 1, kPlanBlock, a);
      return SHMT_OK;
    }
    switch (mode) {
      case 0: hipLaunchKernelGGL(plan_single_kernel<0>, dim3(1), dim3(kPlanBlock), 0, s, a); break;
      case 1: hipLaunchKernelGGL(plan_single_kernel<1>, dim3(1), dim3(kPlanBlock), 0, s, a); break;
      default: hipLaunchKernelGGL(plan_single_kernel<2>, dim3(1), dim3(kPlanBlock), 0, s, a); break;
    }
    SHMT_LAUNCH_CHECK();
    return SHMT_OK;
  }
  const int64_t nb = (S + kPlanBlock - 1) / kPlanBlock;
  SHMT_REQUIRE(nb < (1ll << 31), "shmt_sample_plan: too many seeds");
  const dim3 grid(static_cast<unsigned>(nb));
  if (defer) {
    if (!hop || nb > kPickSumsTiles) {
      defer->mergeable = false;
      return SHMT_OK;
    }
    stage_push(defer, kStagePlanTile + mode, static_cast<unsigned>(nb), kPlanBlock, a);
    hop->tile_prefix_out = a.partials;
    hop->raw_tiles_out = nb;
    return SHMT_OK;
  }
  switch (mode) {
    case 0: hipLaunchKernelGGL(plan_tile_kernel<0>, grid, dim3(kPlanBlock), 0, s, a); break;
    case 1: hipLaunchKernelGGL(plan_tile_kernel<1>, grid, dim3(kPlanBlock), 0, s, a); break;
    default: hipLaunchKernelGGL(plan_tile_kernel<2>, grid, dim3(kPlanBlock), 0, s, a); break;
  }
  SHMT_LAUNCH_CHECK();
  if (hop) {
    hop->tile_prefix_out = a.partials;
    if (nb <= kPickSumsTiles) {  // few tiles: every wave of the pick kernel sums the totals below its tile
      hop->raw_tiles_out = nb;
      return SHMT_OK;
    }
    hipLaunchKernelGGL(plan_totals_kernel, dim3(1), dim3(1024), 0, s, a.partials, nb, sub_indptr,
                       ptr_bytes, S, a.S_len, nnz_out);
    SHMT_LAUNCH_CHECK();
    return SHMT_OK;
  }
  int rc = launch_scan_partials(a.partials, nb + 1, s);
  if (rc) return rc;
  hipLaunchKernelGGL(add_tile_offsets_kernel, dim3(grid_for(S + 1, 256)), dim3(256), 0, s,
                     sub_indptr, ptr_bytes, S, a.partials, static_cast<int64_t>(kPlanBlock), nb,
                     nnz_out);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

int shmt_sample_plan(const void *indptr, int ptr_bytes, const void *cache_indptr,
                     const shmt_hashmap_t *map, const void *seeds, int seed_bytes, int64_t S,
                     int64_t k, int replace, void *sub_indptr, void *plan, int64_t plan_bytes,
                     int64_t *nnz_out, void *stream) {
  return plan_impl(indptr, ptr_bytes, cache_indptr, map, seeds, seed_bytes, S, k, replace, sub_indptr,
                   plan, plan_bytes, nnz_out, Launcher{as_stream(stream), nullptr}, nullptr);
}

}  // extern "C"

struct PickHopExtras {
  void *sub_indptr_rw;
  const uint64_t *tile_prefix;
  int64_t raw_tiles;
  int64_t *nnz_out;
  uint64_t *total_word;
  const int64_t *S_len;
  const uint64_t *rng_seed_dev;
  void *copy_out;
  int copy_bytes;
  uint4 *clear;
  int64_t clear_n;
  uint64_t *wide_mark;
  uint64_t wide_nonce;
  void *coo_out;
  int coo_bytes;
};

template <bool HOP>
static void launch_pick_narrow(int lg, unsigned blocks, unsigned threads, hipStream_t s, const PickArgs &a) {
  switch (lg) {
    case 2: hipLaunchKernelGGL((pick_narrow_kernel<HOP, 2>), dim3(blocks), dim3(threads), 0, s, a); break;
    case 3: hipLaunchKernelGGL((pick_narrow_kernel<HOP, 3>), dim3(blocks), dim3(threads), 0, s, a); break;
    case 4: hipLaunchKernelGGL((pick_narrow_kernel<HOP, 4>), dim3(blocks), dim3(threads), 0, s, a); break;
    case 5: hipLaunchKernelGGL((pick_narrow_kernel<HOP, 5>), dim3(blocks), dim3(threads), 0, s, a); break;
    default: hipLaunchKernelGGL((pick_narrow_kernel<HOP, 6>), dim3(blocks), dim3(threads), 0, s, a); break;
  }
}

template <bool HOP>
static int pick_launch(PickArgs a, Launcher launcher) {
  hipStream_t s = launcher.stream;
  StageList *const defer = launcher.defer;
  const int64_t S = a.S, k = a.k;
  if (k <= kWave) {
    // One seed per lane group and pass while all waves of the launch are resident together (4,096: the
    // kernel's registers allow four waves per SIMD); beyond that a group takes 2 or 4 seeds per pass, whose
    // adjacency loads overlap (355,000 picks of 23,000 seeds: 13.9 -> 12.0 us against a limit of 8,192).
    const int groups_per_wave = kWave >> a.log2_group;
    int rounds = 1;
    while (rounds < kPickRounds && (S + groups_per_wave * rounds - 1) / (groups_per_wave * rounds) > 4096) rounds *= 2;
    a.rounds = rounds;
    const int seeds_per_wave = groups_per_wave * rounds;
    // Few seeds: one wave per workgroup, so that the cold rows' host-link reads come from as many
    // compute units as possible (a unit keeps only so many of them in flight).
    int threads = 256;
    int64_t blocks = (S + 4 * seeds_per_wave - 1) / (4 * seeds_per_wave);
    if (blocks < 512) {
      threads = kWave;
      blocks = (S + seeds_per_wave - 1) / seeds_per_wave;
    }
    // the fused form also clears the relabel table: enough threads for that even when S is small
    if (HOP) {
      const int64_t for_clear = (a.clear_n + threads * 4 - 1) / (threads * 4);
      if (blocks < for_clear) blocks = for_clear;
    }
    if (defer) {
      if (HOP)
        stage_push(defer, kStagePickNarrowHop + a.log2_group - 2, grid_for(blocks, 1), threads, a);
      else
        defer->mergeable = false;
      return SHMT_OK;
    }
    launch_pick_narrow<HOP>(a.log2_group, grid_for(blocks, 1), threads, s, a);
  } else if (defer) {
    defer->mergeable = false;  // the one-wave-per-seed forms have no merged launch
    return SHMT_OK;
  } else if (k <= kWideMaxPicks) {
    hipLaunchKernelGGL((pick_wide_kernel<true, HOP>), dim3(grid_for(S, 1, 256 * 32)), dim3(kWave),
                       static_cast<size_t>(k) * sizeof(int64_t), s, a);
  } else {
    hipLaunchKernelGGL((pick_wide_kernel<false, HOP>), dim3(grid_for(S, 1, 256 * 32)), dim3(kWave), 0,
                       s, a);
  }
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

namespace shmt {

int launch_merged_sampling_stage(int n_jobs, const Stage *const *stages, hipStream_t s) {
  const int kind = stages[0]->kind;
  const unsigned threads = stages[0]->threads;
  if (kind >= kStagePickNarrowHop && kind < kStagePickNarrowHop + 5) {
    Jobs<PickArgs> j;
    const unsigned blocks = jobs_from_stages(n_jobs, stages, &j);
    const dim3 grid(blocks, n_jobs), block(threads);
    switch (kind - kStagePickNarrowHop + 2) {
      case 2: hipLaunchKernelGGL(pick_narrow_hop_jobs<2>, grid, block, 0, s, j); break;
      case 3: hipLaunchKernelGGL(pick_narrow_hop_jobs<3>, grid, block, 0, s, j); break;
      case 4: hipLaunchKernelGGL(pick_narrow_hop_jobs<4>, grid, block, 0, s, j); break;
      case 5: hipLaunchKernelGGL(pick_narrow_hop_jobs<5>, grid, block, 0, s, j); break;
      default: hipLaunchKernelGGL(pick_narrow_hop_jobs<6>, grid, block, 0, s, j); break;
    }
  } else if (kind >= kStagePlanSingle && kind < kStagePlanTile + 3) {
    Jobs<PlanArgs> j;
    const unsigned blocks = jobs_from_stages(n_jobs, stages, &j);
    const dim3 grid(blocks, n_jobs), block(threads);
    switch (kind) {
      case kStagePlanSingle + 0: hipLaunchKernelGGL(plan_single_jobs<0>, grid, block, 0, s, j); break;
      case kStagePlanSingle + 1: hipLaunchKernelGGL(plan_single_jobs<1>, grid, block, 0, s, j); break;
      case kStagePlanSingle + 2: hipLaunchKernelGGL(plan_single_jobs<2>, grid, block, 0, s, j); break;
      case kStagePlanTile + 0: hipLaunchKernelGGL(plan_tile_jobs<0>, grid, block, 0, s, j); break;
      case kStagePlanTile + 1: hipLaunchKernelGGL(plan_tile_jobs<1>, grid, block, 0, s, j); break;
      default: hipLaunchKernelGGL(plan_tile_jobs<2>, grid, block, 0, s, j); break;
    }
  } else {
    set_error("internal: stage kind %d has no merged sampling launch", kind);
    return SHMT_EINVAL;
  }
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

}  // namespace shmt

extern "C" {

static int pick_impl(const void *indices, const void *cache_indices, int idx_bytes,
                     const void *seeds, int seed_bytes, int64_t S, int64_t k, int replace,
                     const void *sub_indptr, int ptr_bytes, const void *plan, void *sub_indices,
                     uint64_t rng_seed, uint32_t rng_stream, Launcher launcher, const PickHopExtras *hop) {
  SHMT_REQUIRE(S >= 0 && k >= 0, "shmt_sample_pick: S and num_picks must be >= 0");
  SHMT_REQUIRE(width_ok(idx_bytes) && width_ok(seed_bytes) && width_ok(ptr_bytes),
               "shmt_sample_pick: ID can only be int32 or int64");
  if (S == 0 || k == 0) return SHMT_OK;
  SHMT_REQUIRE(indices && seeds && sub_indptr && plan && sub_indices,
               "shmt_sample_pick: null buffer");
  PickArgs a;
  a.indices = indices;
  a.cache_indices = cache_indices ? cache_indices : indices;
  a.seeds = seeds;
  a.sub_indptr = sub_indptr;
  a.plan = static_cast<const SeedPlan *>(plan);
  a.out = sub_indices;
  a.S = S;
  a.k = k;
  a.rng_seed = rng_seed;
  a.rng_stream = rng_stream;
  a.idx_bytes = idx_bytes;
  a.seed_bytes = seed_bytes;
  a.ptr_bytes = ptr_bytes;
  a.replace = replace ? 1 : 0;
  a.log2_group = 0;
  a.rounds = 1;
  if (k <= kWave) {
    int lg = 2;
    while ((1 << lg) < k) ++lg;
    a.log2_group = lg;
  }
  a.sub_indptr_rw = nullptr;
  a.tile_prefix = nullptr;
  a.raw_tiles = 0;
  a.nnz_out = nullptr;
  a.total_word = nullptr;
  a.S_len = nullptr;
  a.rng_seed_dev = nullptr;
  a.copy_out = nullptr;
  a.copy_bytes = 8;
  a.clear = nullptr;
  a.clear_n = 0;
  a.wide_mark = nullptr;
  a.wide_nonce = 0;
  a.coo_out = nullptr;
  a.coo_bytes = 8;
  if (!hop) return pick_launch<false>(a, launcher);
  a.sub_indptr_rw = hop->sub_indptr_rw;
  a.tile_prefix = hop->tile_prefix;
  a.raw_tiles = hop->raw_tiles;
  a.nnz_out = hop->nnz_out;
  a.total_word = hop->total_word;
  a.S_len = hop->S_len;
  a.rng_seed_dev = hop->rng_seed_dev;
  a.copy_out = hop->copy_out;
  a.copy_bytes = hop->copy_bytes;
  a.clear = hop->clear;
  a.clear_n = hop->clear_n;
  a.wide_mark = hop->wide_mark;
  a.wide_nonce = hop->wide_nonce;
  a.coo_out = hop->coo_out;
  a.coo_bytes = hop->coo_bytes;
  return pick_launch<true>(a, launcher);
}

int shmt_sample_pick(const void *indices, const void *cache_indices, int idx_bytes,
                     const void *seeds, int seed_bytes, int64_t S, int64_t k, int replace,
                     const void *sub_indptr, int ptr_bytes, const void *plan, void *sub_indices,
                     uint64_t rng_seed, uint32_t rng_stream, void *stream) {
  return pick_impl(indices, cache_indices, idx_bytes, seeds, seed_bytes, S, k, replace, sub_indptr,
                   ptr_bytes, plan, sub_indices, rng_seed, rng_stream, Launcher{as_stream(stream), nullptr}, nullptr);
}

int shmt_sample(const void *indptr, int ptr_bytes, const void *indices, int idx_bytes,
                const void *cache_indptr, const void *cache_indices, const shmt_hashmap_t *map,
                const void *seeds, int seed_bytes, int64_t S, int64_t k, int replace, uint64_t rng_seed,
                uint32_t rng_stream, void *sub_indptr, void *sub_indices, void *plan, int64_t plan_bytes,
                int64_t *nnz_out, void *stream) {
  SHMT_REQUIRE(S >= 1 && k >= 1, "shmt_sample: S and num_picks must be >= 1");
  // the fused-hop forms of the kernels without their relabel extras: the pick kernel adds the tile
  // offsets and publishes the total, so plan + pick are two launches whatever the number of seeds
  PlanHopExtras plan_hop{nullptr, 8, nullptr, nullptr, nullptr, 0};
  const Launcher launcher{as_stream(stream), nullptr};
  int rc = plan_impl(indptr, ptr_bytes, cache_indptr, map, seeds, seed_bytes, S, k, replace, sub_indptr, plan,
                     plan_bytes, nnz_out, launcher, &plan_hop);
  if (rc) return rc;
  const PickHopExtras pick_hop{sub_indptr, plan_hop.tile_prefix_out, plan_hop.raw_tiles_out, nnz_out,
                               const_cast<uint64_t *>(plan_hop.total_out), nullptr, nullptr, nullptr, 8,
                               nullptr, 0, nullptr, 0, nullptr, 8};
  return pick_impl(indices, cache_indices, idx_bytes, seeds, seed_bytes, S, k, replace, sub_indptr, ptr_bytes,
                   plan, sub_indices, rng_seed, rng_stream, launcher, &pick_hop);
}

static int hop_impl(const void *indptr, int ptr_bytes, const void *indices, int idx_bytes,
                    const void *cache_indptr, const void *cache_indices, const shmt_hashmap_t *map,
                    const void *seeds, int seed_bytes, int64_t S, const int64_t *S_len, int64_t k,
                    int replace, uint64_t rng_seed, const uint64_t *rng_seed_dev, uint32_t rng_stream,
                    void *sub_indptr,
                    void *sub_indices, void *plan, int64_t plan_bytes, int elem_bytes, void *total_out,
                    void *scratch, int64_t scratch_bytes, void *unique_out, void *labels_out,
                    int64_t *nnz_out, int64_t *count_out, int64_t *count_copy, void *coo_dst, int coo_bytes,
                    Launcher launcher) {
  SHMT_REQUIRE(S >= 1 && k >= 1, "shmt_sample_hop: S and num_picks must be >= 1");
  SHMT_REQUIRE(coo_dst == nullptr || width_ok(coo_bytes), "shmt_sample_hop: coo_bytes must be 4 or 8");
  SHMT_REQUIRE(k <= ((1ll << 31) - 1 - S) / S, "shmt_sample_hop: S * (num_picks + 1) must be < 2^31");
  SHMT_REQUIRE(width_ok(idx_bytes) && width_ok(seed_bytes) && width_ok(ptr_bytes) && width_ok(elem_bytes),
               "shmt_sample_hop: ID can only be int32 or int64");
  SHMT_REQUIRE(elem_bytes >= seed_bytes && elem_bytes >= idx_bytes,
               "shmt_sample_hop: elem_bytes must be the wider of the seed and index widths");
  SHMT_REQUIRE(indices && sub_indices && total_out && unique_out && labels_out && count_out,
               "shmt_sample_hop: null buffer");
  const int64_t n_max = S + S * k;
  RelabelTable table;
  int rc = relabel_table(n_max, S_len != nullptr, launcher.defer ? launcher.defer->jobs : 0, scratch, scratch_bytes,
                         &table);
  if (rc) return rc;
  PlanHopExtras plan_hop{total_out, elem_bytes, S_len, nullptr, nullptr, 0};
  rc = plan_impl(indptr, ptr_bytes, cache_indptr, map, seeds, seed_bytes, S, k, replace, sub_indptr, plan,
                 plan_bytes, nnz_out, launcher, &plan_hop);
  if (rc) return rc;
  const PickHopExtras pick_hop{sub_indptr, plan_hop.tile_prefix_out, plan_hop.raw_tiles_out, nnz_out,
                               const_cast<uint64_t *>(plan_hop.total_out), S_len, rng_seed_dev, total_out, elem_bytes,
                               static_cast<uint4 *>(table.slots), table.n16, table.wide_mark, table.nonce,
                               coo_dst, coo_bytes};
  rc = pick_impl(indices, cache_indices, idx_bytes, seeds, seed_bytes, S, k, replace, sub_indptr, ptr_bytes,
                 plan, sub_indices, rng_seed, rng_stream, launcher, &pick_hop);
  if (rc) return rc;
  // [seeds, sub_indices] is in total_out and the table is empty: the relabel passes follow, with the
  // number of sampled ids (and of seeds, when it is a device-side figure) read from device memory
  return launch_relabel_passes(total_out, n_max, S, S_len, plan_hop.total_out, 8, elem_bytes, scratch,
                               scratch_bytes, unique_out, labels_out, count_out, count_copy, table, launcher);
}

int shmt_sample_hop(const void *indptr, int ptr_bytes, const void *indices, int idx_bytes,
                    const void *cache_indptr, const void *cache_indices, const shmt_hashmap_t *map,
                    const void *seeds, int seed_bytes, int64_t S, int64_t k, int replace,
                    uint64_t rng_seed, uint32_t rng_stream, void *sub_indptr, void *sub_indices,
                    void *plan, int64_t plan_bytes, int elem_bytes, void *total_out, void *scratch,
                    int64_t scratch_bytes, void *unique_out, void *labels_out, int64_t *nnz_out,
                    int64_t *count_out, void *stream) {
  return hop_impl(indptr, ptr_bytes, indices, idx_bytes, cache_indptr, cache_indices, map, seeds, seed_bytes,
                  S, nullptr, k, replace, rng_seed, nullptr, rng_stream, sub_indptr, sub_indices, plan, plan_bytes,
                  elem_bytes, total_out, scratch, scratch_bytes, unique_out, labels_out, nnz_out, count_out,
                  nullptr, nullptr, 8, Launcher{as_stream(stream), nullptr});
}

int shmt_sample_hop_chained(const void *indptr, int ptr_bytes, const void *indices, int idx_bytes,
                            const void *cache_indptr, const void *cache_indices,
                            const shmt_hashmap_t *map, const void *seeds, int seed_bytes,
                            int64_t max_seeds, const int64_t *seeds_len, int64_t k, int replace,
                            uint64_t rng_seed, const uint64_t *rng_seed_dev, uint32_t rng_stream,
                            void *sub_indptr, void *sub_indices,
                            void *plan, int64_t plan_bytes, int elem_bytes, void *total_out,
                            void *scratch, int64_t scratch_bytes, void *unique_out, void *labels_out,
                            int64_t *nnz_out, int64_t *count_out, int64_t *count_dev_out, void *stream) {
  return hop_impl(indptr, ptr_bytes, indices, idx_bytes, cache_indptr, cache_indices, map, seeds, seed_bytes,
                  max_seeds, seeds_len, k, replace, rng_seed, rng_seed_dev, rng_stream, sub_indptr, sub_indices,
                  plan,
                  plan_bytes, elem_bytes, total_out, scratch, scratch_bytes, unique_out, labels_out, nnz_out,
                  count_out, count_dev_out, nullptr, 8, Launcher{as_stream(stream), nullptr});
}

static int hop_job(const shmt_hop_job &j, Launcher launcher) {
  return hop_impl(j.indptr, j.ptr_bytes, j.indices, j.idx_bytes, j.cache_indptr, j.cache_indices, j.map, j.seeds,
                  j.seed_bytes, j.max_seeds, j.seeds_len, j.k, j.replace, j.rng_seed, j.rng_seed_dev, j.rng_stream,
                  j.sub_indptr, j.sub_indices, j.plan, j.plan_bytes, j.elem_bytes, j.total_out, j.scratch,
                  j.scratch_bytes, j.unique_out, j.labels_out, j.nnz_out, j.count_out, j.count_dev_out, j.coo_dst,
                  j.coo_bytes, launcher);
}

int shmt_sample_hops_chained(const shmt_hop_job *jobs, int n_jobs, void *stream) {
  SHMT_REQUIRE(n_jobs >= 0, "shmt_sample_hops_chained: n_jobs must be >= 0");
  SHMT_REQUIRE(n_jobs == 0 || jobs != nullptr, "shmt_sample_hops_chained: jobs is null");
  hipStream_t s = as_stream(stream);
  for (int first = 0; first < n_jobs; first += kMaxJobs) {
    const int n = n_jobs - first < kMaxJobs ? n_jobs - first : kMaxJobs;
    // record every job's launches; merge them when all jobs run the same kernels stage by stage
    StageList lists[kMaxJobs];
    bool merge = n > 1;
    for (int j = 0; j < n && merge; ++j) {
      lists[j].jobs = n;
      const int rc = hop_job(jobs[first + j], Launcher{s, &lists[j]});
      if (rc) return rc;
      merge = lists[j].mergeable && lists[j].n == lists[0].n;
      for (int i = 0; merge && i < lists[j].n; ++i)
        merge = lists[j].stage[i].kind == lists[0].stage[i].kind &&
                lists[j].stage[i].threads == lists[0].stage[i].threads;
    }
    if (!merge) {
      for (int j = 0; j < n; ++j) {
        const int rc = hop_job(jobs[first + j], Launcher{s, nullptr});
        if (rc) return rc;
      }
      continue;
    }
    for (int i = 0; i < lists[0].n; ++i) {
      const Stage *stages[kMaxJobs];
      for (int j = 0; j < n; ++j) stages[j] = &lists[j].stage[i];
      const int rc = stages[0]->kind >= kStageRlSmall ? launch_merged_relabel_stage(n, stages, s)
                                                      : launch_merged_sampling_stage(n, stages, s);
      if (rc) return rc;
    }
  }
  return SHMT_OK;
}

int shmt_csr_rows(const void *offsets, int ptr_bytes, int64_t S, int64_t nnz, void *rows_out,
                  int out_bytes, void *stream) {
  SHMT_REQUIRE(S >= 0 && nnz >= 0, "shmt_csr_rows: S and nnz must be >= 0");
  SHMT_REQUIRE(width_ok(ptr_bytes) && width_ok(out_bytes), "shmt_csr_rows: ID can only be int32 or int64");
  if (nnz == 0) return SHMT_OK;
  SHMT_REQUIRE(S >= 1 && offsets && rows_out, "shmt_csr_rows: null buffer");
  const int64_t nchunks = (nnz + kCopyChunk - 1) / kCopyChunk;
  hipLaunchKernelGGL(csr_rows_kernel, dim3(grid_for(nchunks, 1)), dim3(256), 0, as_stream(stream), offsets,
                     ptr_bytes, S, nnz, rows_out, out_bytes);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

int shmt_subcsr_plan(const void *indptr, int ptr_bytes, const void *seeds, int seed_bytes,
                     int64_t C, void *cache_indptr, void *tmp, int64_t tmp_bytes,
                     int64_t *nnz_out, void *stream) {
  SHMT_REQUIRE(C >= 0, "shmt_subcsr_plan: C must be >= 0");
  SHMT_REQUIRE(width_ok(ptr_bytes) && width_ok(seed_bytes),
               "shmt_subcsr_plan: ID can only be int32 or int64");
  SHMT_REQUIRE(indptr && cache_indptr && nnz_out, "shmt_subcsr_plan: null buffer");
  SHMT_REQUIRE(C == 0 || seeds != nullptr, "shmt_subcsr_plan: seeds is null");
  hipStream_t s = as_stream(stream);
  hipLaunchKernelGGL(subcsr_degree_kernel, dim3(grid_for(C + 1, 256)), dim3(256), 0, s, indptr,
                     ptr_bytes, seeds, seed_bytes, C, cache_indptr);
  SHMT_LAUNCH_CHECK();
  int rc = shmt_exclusive_scan(cache_indptr, C + 1, ptr_bytes, tmp, tmp_bytes, stream);
  if (rc) return rc;
  hipLaunchKernelGGL(copy_total_kernel, dim3(1), dim3(1), 0, s, cache_indptr, ptr_bytes, C, nnz_out);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

int shmt_subcsr_copy(const void *indptr, const void *indices, int ptr_bytes, int idx_bytes,
                     const void *seeds, int seed_bytes, int64_t C, const void *cache_indptr,
                     int64_t nnz, void *cache_indices, void *stream) {
  SHMT_REQUIRE(C >= 0 && nnz >= 0, "shmt_subcsr_copy: C and nnz must be >= 0");
  SHMT_REQUIRE(width_ok(ptr_bytes) && width_ok(idx_bytes) && width_ok(seed_bytes),
               "shmt_subcsr_copy: ID can only be int32 or int64");
  if (C == 0 || nnz == 0) return SHMT_OK;
  SHMT_REQUIRE(indptr && indices && seeds && cache_indptr && cache_indices,
               "shmt_subcsr_copy: null buffer");
  const int64_t nchunks = (nnz + kCopyChunk - 1) / kCopyChunk;
  hipLaunchKernelGGL(subcsr_copy_kernel, dim3(grid_for(nchunks, 1)), dim3(256), 0, as_stream(stream),
                     indptr, indices, ptr_bytes, idx_bytes, seeds, seed_bytes, C, cache_indptr, nnz,
                     cache_indices);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

}  // extern "C"
