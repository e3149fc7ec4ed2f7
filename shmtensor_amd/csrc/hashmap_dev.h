// Device-side view of the static hashmap and the cooperative probe used by
// every kernel that consults it (bulk query, fetch/set, sampling plan).
//
// Layout in HBM: the table is an array of 128-byte buckets, one HBM/L2 line
// each. A probe group of 8 adjacent lanes reads one whole bucket with a
// single coalesced 16-byte-per-lane load and decides hit / miss / continue
// with a ballot, so one memory transaction inspects every slot of the line.
//   wide   (kSlot16): 8 slots {int64 key, int64 value}; used whenever the key
//                     or the value is 8 bytes wide (4-byte members are
//                     sign-extended on insert).
//   narrow (kSlot8) : 16 slots {int32 key, int32 value}; each lane sees two.
// Empty slots hold key = value = -1 (all bits set). Keys probe buckets
// linearly from hash(key) and are always placed in the first bucket of their
// probe sequence that still has a free slot, so a lookup stops at the first
// bucket that contains either the key or an empty slot.
//
// Three flat forms exist beside the bucket table, chosen when the map is built
// from what its keys look like (node ids are dense small integers, caches of
// re-numbered graphs hold an id range, and a cache built in id order numbers
// its rows by rank):
//   direct (kKindDirect): keys lie in [lo, lo + span) with span a small
//                     multiple of their number; the table is int32
//                     value[key - lo], -1 where no key was given. One 4-byte
//                     load per lookup, no probe sequence.
//   range  (kKindRange) : the keys are exactly the ids lo .. lo + span - 1 and
//                     every value is key + delta; lookups are arithmetic and
//                     touch no memory at all.
//   rank   (kKindRank)  : the pairs came in ascending key order with values
//                     v0, v0 + 1, v0 + 2, ...: the value is the key's rank
//                     among the keys (+ delta = v0). The table is a bitmap
//                     with running counts, 16-byte blocks {uint32 keys below
//                     this block, 96 presence bits}: one 16-byte load per
//                     lookup from a table of span / 6 bytes, which stays in
//                     the caches where a 4-byte-per-id table does not.
#pragma once
#include "wave.h"

namespace shmt {

enum SlotFormat : int { kSlot16 = 16, kSlot8 = 8 };

constexpr int kProbeGroup = 8;      // lanes that cooperate on one key
constexpr int kBucketBytes = 128;

enum MapKind : int { kKindBuckets = 0, kKindDirect = 1, kKindRange = 2, kKindRank = 3 };

constexpr int kRankIdsPerBlock = 96;  // presence bits of one 16-byte rank block

struct MapView {
  const uint4 *buckets;   // bucket table: nbuckets * 8 uint4; direct form: int32 values[span];
                          // rank form: one uint4 block per 96 ids
  uint32_t nbuckets;
  int key32;              // 1: keys are int32 -> requests are narrowed before the lookup
  int kind;               // MapKind
  int fits32;             // 1: 64-bit keys stored in narrow slots (they all fit): a request that
                          //    does not fit 32 bits is absent
  int64_t lo;             // flat forms: smallest key
  int64_t span;           // flat forms: keys lie in [lo, lo + span)
  int64_t delta;          // range form: value = key + delta; rank form: value = rank + delta
};

inline MapView empty_map_view() { return MapView{nullptr, 1, 0, kKindBuckets, 0, 0, 0, 0}; }

// Normalise a request to the key domain of the map (what requests.to(key
// dtype) does in the reference): int32-keyed maps see the low 32 bits,
// sign-extended. A request that cannot be a key of a narrow-stored 64-bit
// map becomes the empty sentinel, which every lookup resolves to -1.
__device__ __forceinline__ int64_t map_key(const MapView &m, int64_t req) {
  if (m.key32) return static_cast<int64_t>(static_cast<int32_t>(req));
  if (m.fits32 && req != static_cast<int64_t>(static_cast<int32_t>(req))) return -1;
  return req;
}

// Table entries that will not be looked at again soon (the probe of a row
// fetch) are read with the non-temporal cache policy, so that they do not push
// table rows out of the caches. They go through buffer loads, whose cache
// policy is an operand of the instruction: the same hint as metadata on an
// ordinary load is dropped whenever the optimiser merges the load with its
// plain twin on the other side of a branch. Buffer loads address with 32-bit
// byte offsets, so a table must stay below 4 GiB to be read this way
// (streamable()); larger ones are read with plain loads.
typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));
constexpr int kCachePolicyNonTemporal = 2;  // gfx94x / gfx950: bit 1 of the cache-policy operand

__device__ __forceinline__ __amdgpu_buffer_rsrc_t table_resource(const void *table) {
  // raw buffer over [table, table + 4 GiB): no stride, no swizzle; word 3 as gfx90a .. gfx950 want it for
  // untyped 32-bit data
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(table), 0, -1, 0x00020000);
}

// ... and it must be larger than the L2s together (64 MiB taken as the line): a table that the caches can
// hold is worth keeping there. (A bulk query over a 128 MiB table, which the memory-side cache holds when
// nothing else streams through it, measured 0.38 ms with plain loads and 0.48 ms streaming; the tables of a
// row fetch share that cache with the rows that stream through it, and there streaming wins from 160 MB up.)
__device__ __forceinline__ bool streamable(const MapView &m) {
  if (m.kind == kKindBuckets) return m.nbuckets >= (1u << 19) && m.nbuckets < (1u << 25);  // 128-byte buckets
  if (m.kind == kKindDirect) return m.span >= (1ll << 24) && m.span < (1ll << 30);          // 4-byte entries
  return false;
}

__device__ __forceinline__ uint4 load_bucket_streaming(const MapView &m, uint32_t bucket, int sub) {
  const uint32_t offset = (bucket * kProbeGroup + static_cast<uint32_t>(sub)) * 16u;
  const probe_u32x4 v =
      __builtin_amdgcn_raw_buffer_load_b128(table_resource(m.buckets), offset, 0, kCachePolicyNonTemporal);
  return make_uint4(v.x, v.y, v.z, v.w);
}

// Lookup in a flat map (kind != kKindBuckets); every lane for itself, in two
// steps so that a caller can put other work between the load and its use:
// flat_issue starts the one load a rank or direct map needs, flat_finish turns
// what came back into the value. STREAM: the entry of a direct table is read
// with a non-temporal load (see half_wave_issue for when a row fetch asks for
// that).
struct FlatPending {
  uint4 block;     // rank form: the 16-byte block of the key
  int32_t direct;  // direct form: the table entry
  bool inside;     // the key lies in [lo, lo + span)
};

template <bool STREAM = false>
__device__ __forceinline__ FlatPending flat_issue(const MapView &m, int64_t key) {
  FlatPending p;
  p.block = make_uint4(0, 0, 0, 0);
  p.direct = -1;
  const uint64_t off = static_cast<uint64_t>(key) - static_cast<uint64_t>(m.lo);  // key < lo wraps around
  p.inside = off < static_cast<uint64_t>(m.span);
  if (!p.inside || m.kind == kKindRange) return p;
  if (m.kind == kKindRank) {
    p.block = m.buckets[off / kRankIdsPerBlock];  // x: keys below this block; y, z, w: presence of ids 0-31, 32-63, 64-95
  } else {
    const int32_t *direct = reinterpret_cast<const int32_t *>(m.buckets);
    p.direct = STREAM ? static_cast<int32_t>(__builtin_amdgcn_raw_buffer_load_b32(
                            table_resource(m.buckets), static_cast<uint32_t>(off) * 4u, 0, kCachePolicyNonTemporal))
                      : direct[off];
  }
  return p;
}

__device__ __forceinline__ int64_t flat_finish(const MapView &m, int64_t key, const FlatPending &p) {
  if (!p.inside) return -1;
  if (m.kind == kKindRange) return key + m.delta;
  if (m.kind == kKindRank) {
    const uint64_t off = static_cast<uint64_t>(key) - static_cast<uint64_t>(m.lo);
    const uint32_t r = static_cast<uint32_t>(off % kRankIdsPerBlock);
    const uint4 b = p.block;
    const uint32_t word = r < 32 ? b.y : (r < 64 ? b.z : b.w);
    const uint32_t bit = r & 31;
    if (((word >> bit) & 1u) == 0) return -1;
    uint32_t below = __builtin_popcount(word & ((1u << bit) - 1u));
    if (r >= 32) below += __builtin_popcount(b.y);
    if (r >= 64) below += __builtin_popcount(b.z);
    return static_cast<int64_t>(b.x + below) + m.delta;
  }
  return static_cast<int64_t>(p.direct);
}

template <bool STREAM = false>
__device__ __forceinline__ int64_t flat_find(const MapView &m, int64_t key) {
  return flat_finish(m, key, flat_issue<STREAM>(m, key));
}

__device__ __forceinline__ uint32_t map_bucket(const MapView &m, int64_t key) {
  return reduce_range(hash_id(key), m.nbuckets);
}

// Examine one already-loaded bucket fragment. Returns true when the group is
// done with this key (value written to *val: the mapped value, or -1 when the
// bucket proved the key absent); false when the bucket was full of other keys.
template <int FMT>
__device__ __forceinline__ bool probe_step(const uint4 frag, int64_t key, int64_t *val) {
  const int gbase = lane_id() & ~(kProbeGroup - 1);
  bool match, empty;
  int64_t v;
  if (FMT == kSlot16) {
    int64_t k = static_cast<int64_t>((static_cast<uint64_t>(frag.y) << 32) | frag.x);
    v = static_cast<int64_t>((static_cast<uint64_t>(frag.w) << 32) | frag.z);
    match = (k == key);
    empty = (k == -1);
  } else {
    int32_t k32 = static_cast<int32_t>(key);
    bool m0 = static_cast<int32_t>(frag.x) == k32;
    bool m1 = static_cast<int32_t>(frag.z) == k32;
    match = m0 || m1;
    v = static_cast<int64_t>(static_cast<int32_t>(m0 ? frag.y : frag.w));
    empty = (frag.x == 0xFFFFFFFFu) || (frag.z == 0xFFFFFFFFu);
  }
  uint64_t mm = group_ballot<kProbeGroup>(match);
  if (mm) {
    *val = shfl64(v, gbase + __builtin_ctzll(mm));
    return true;
  }
  if (group_ballot<kProbeGroup>(empty)) {
    *val = -1;
    return true;
  }
  return false;
}

// Cooperative find: the 8 lanes of an aligned probe group call this with the
// same (already normalised) key; all of them receive the value or -1. The
// probe count is bounded by the number of buckets, so a completely full
// table still terminates.
template <int FMT>
__device__ __forceinline__ int64_t group_find(const MapView &m, int64_t key) {
  if (m.kind != kKindBuckets) return flat_find(m, key);
  const int sub = lane_id() & (kProbeGroup - 1);
  uint32_t b = map_bucket(m, key);
  int64_t val = -1;
  for (uint32_t probes = 0; probes < m.nbuckets; ++probes) {
    uint4 frag = m.buckets[static_cast<size_t>(b) * kProbeGroup + sub];
    if (probe_step<FMT>(frag, key, &val)) return val;
    b = (b + 1 == m.nbuckets) ? 0 : b + 1;
  }
  return -1;
}

// Whole-wave find: every lane brings its own (already normalised) key; the
// wave's eight probe groups resolve the 64 keys, eight keys per group. Probing
// proceeds in rounds: in round r every still-unresolved key of a group has its
// (home + r)-th bucket loaded, all loads of the round are issued before any is
// examined, so the number of dependent HBM round trips is the longest probe
// chain among the 64 keys, not the sum. Every lane gets the value for its own
// key (or -1). All 64 lanes must be active; lanes with nothing to look up
// pass -1 (the empty sentinel, which resolves to -1 in one round). Flat maps
// (direct / range form) are answered by every lane for itself.
template <int FMT, int BATCH = kProbeGroup>
__device__ __forceinline__ int64_t wave_find(const MapView &m, int64_t mykey) {
  static_assert(kProbeGroup % BATCH == 0, "BATCH must divide the probe group size");
  if (m.kind != kKindBuckets) return flat_find(m, mykey);  // uniform across the launch
  const int sub = lane_id() & (kProbeGroup - 1);
  const int gbase = lane_id() & ~(kProbeGroup - 1);
  int64_t res = -1;
  // BATCH keys of each group are in flight at a time (fewer live registers
  // for smaller BATCH, at the price of kProbeGroup / BATCH sequential passes)
#pragma unroll
  for (int j0 = 0; j0 < kProbeGroup; j0 += BATCH) {
    uint32_t pending = (1u << BATCH) - 1;  // bit j: key j0 + j of this group unresolved
    for (uint32_t round = 0; round < m.nbuckets; ++round) {
      uint4 frag[BATCH];
#pragma unroll
      for (int j = 0; j < BATCH; ++j) {
        if (pending & (1u << j)) {
          uint32_t b = map_bucket(m, shfl64(mykey, gbase + j0 + j)) + round;
          if (b >= m.nbuckets) b -= m.nbuckets;
          frag[j] = m.buckets[static_cast<size_t>(b) * kProbeGroup + sub];
        }
      }
#pragma unroll
      for (int j = 0; j < BATCH; ++j) {
        if (pending & (1u << j)) {
          int64_t val;
          if (probe_step<FMT>(frag[j], shfl64(mykey, gbase + j0 + j), &val)) {
            pending &= ~(1u << j);
            if (sub == j0 + j) res = val;
          }
        }
      }
      if (pending == 0) break;
    }
  }
  return res;
}

// True (in every lane) when some key of lanes 0 .. 31 also appears in another
// of those lanes at lane distance 1, 2, 4, 8 or 16: under skewed access a
// handful of hot keys take most of the requests and show up twice within 32
// rows nearly every time, under uniform access over a large key set next to
// never. A hint for the cache policy of the lookup, nothing more. All lanes
// must be active; lanes that bring no key pass `has_key` false.
__device__ __forceinline__ bool tile_repeats(int64_t mykey, bool has_key) {
  bool again = false;
#pragma unroll
  for (int d = 1; d < 32; d *= 2) again |= mykey == shfl64(mykey, lane_id() ^ d);
  return __builtin_amdgcn_ballot_w64(again && has_key && lane_id() < 32) != 0;
}

// Find for a wave whose lanes 0 .. 31 bring one (already normalised) key each
// (a fetch tile of 32 rows); lanes 32 .. 63 bring nothing. The keys are dealt
// four to a probe group (group g takes the keys of lanes 4g .. 4g + 3), so all
// eight groups work, the first bucket of every key is in flight at once (32
// lines), and a lookup that ends in its first bucket costs ONE dependent round
// trip; wave_find would leave the upper four groups looking up the empty
// sentinel while the lower four walk through eight keys each in two passes.
// STREAM: read the buckets with non-temporal loads. A
// table far larger than the caches is read once per row and its lines only
// push table rows out: measured on 1,048,576 uniform all-hit rows of 256 B
// through a 640 MB table, 125 us with plain probe loads and 112 us with
// non-temporal ones. Under skewed access the buckets of hot keys are what the
// caches should keep, and there non-temporal probes cost 10 % (Zipf(1.1)
// batch: 112 us plain, 123 us non-temporal). The caller therefore asks for
// streaming only for tiles that show no sign of skew (tile_repeats).
// Every lane below 32 gets the value for its own key (or -1). All 64 lanes
// must be active. Flat maps are answered by every lane for itself.
constexpr int kHalfWaveKeys = 4;  // keys per probe group of a 32-key lookup

// The lookup in two steps, so that a caller can put other work (moving the
// rows of the tile before) between the loads and their use: half_wave_issue
// deals the keys to the groups and starts the load of every key's first
// bucket; half_wave_finish examines what came back and walks on, bucket by
// bucket, for the few keys whose first bucket was full of other keys.
struct HalfWaveProbe {
  uint4 frag[kHalfWaveKeys];  // (the keys are dealt again by half_wave_finish: cheaper than keeping them in registers)
};

template <int FMT, bool STREAM>
__device__ __forceinline__ void half_wave_issue(const MapView &m, int64_t mykey, HalfWaveProbe *p) {
  const int sub = lane_id() & (kProbeGroup - 1);
  const int grp = lane_id() / kProbeGroup;
#pragma unroll
  for (int j = 0; j < kHalfWaveKeys; ++j) {
    const int64_t key = shfl64(mykey, grp * kHalfWaveKeys + j);
    const uint32_t b = map_bucket(m, key);
    p->frag[j] = STREAM ? load_bucket_streaming(m, b, sub) : m.buckets[static_cast<size_t>(b) * kProbeGroup + sub];
  }
}

template <int FMT>
__device__ __forceinline__ int64_t half_wave_finish(const MapView &m, int64_t mykey, const HalfWaveProbe &p) {
  const int lane = lane_id();
  const int sub = lane & (kProbeGroup - 1);
  const int grp = lane / kProbeGroup;
  int64_t res = -1;  // lane 8g + j ends up with the value of key lane 4g + j
  uint32_t pending = 0;
#pragma unroll
  for (int j = 0; j < kHalfWaveKeys; ++j) {
    int64_t val;
    if (probe_step<FMT>(p.frag[j], shfl64(mykey, grp * kHalfWaveKeys + j), &val)) {
      if (sub == j) res = val;
    } else {
      pending |= 1u << j;
    }
  }
  if (__builtin_amdgcn_ballot_w64(pending != 0) != 0) {  // some first bucket was full of other keys: walk on
#pragma unroll
    for (int j = 0; j < kHalfWaveKeys; ++j) {
      const int64_t key = shfl64(mykey, grp * kHalfWaveKeys + j);  // (all lanes take part in the shuffle)
      for (uint32_t round = 1; (pending & (1u << j)) && round < m.nbuckets; ++round) {
        uint32_t b = map_bucket(m, key) + round;
        if (b >= m.nbuckets) b -= m.nbuckets;
        const uint4 frag = m.buckets[static_cast<size_t>(b) * kProbeGroup + sub];
        int64_t val;
        if (probe_step<FMT>(frag, key, &val)) {
          pending &= ~(1u << j);
          if (sub == j) res = val;
        }
      }
    }
  }
  return shfl64(res, (lane / kHalfWaveKeys) * kProbeGroup + (lane & (kHalfWaveKeys - 1)));
}

template <int FMT, bool STREAM>
__device__ __forceinline__ int64_t half_wave_find(const MapView &m, int64_t mykey) {
  if (m.kind != kKindBuckets) return lane_id() < 32 ? flat_find<STREAM>(m, mykey) : -1;
  HalfWaveProbe p;
  half_wave_issue<FMT, STREAM>(m, mykey, &p);
  return half_wave_finish<FMT>(m, mykey, p);
}

}  // namespace shmt
