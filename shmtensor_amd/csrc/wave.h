// Device-side building blocks for gfx950 (wave64): hashing, sub-wave group
// ballots, width-switched integer loads/stores and wavefront/workgroup scans.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace shmt {

constexpr int kWave = 64;

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// ---- hashing -----------------------------------------------------------
// 32-bit avalanche of a 64-bit id (murmur3 finaliser over the folded halves),
// then a multiply-high range reduction so table sizes need not be powers of 2.
__device__ __host__ __forceinline__ uint32_t hash_id(int64_t key) {
  uint32_t lo = static_cast<uint32_t>(static_cast<uint64_t>(key));
  uint32_t hi = static_cast<uint32_t>(static_cast<uint64_t>(key) >> 32);
  uint32_t h = lo ^ (hi * 0x9E3779B1u);
  h ^= h >> 16;
  h *= 0x85EBCA6Bu;
  h ^= h >> 13;
  h *= 0xC2B2AE35u;
  h ^= h >> 16;
  return h;
}

__device__ __host__ __forceinline__ uint32_t reduce_range(uint32_t h, uint32_t n) {
  return static_cast<uint32_t>((static_cast<uint64_t>(h) * n) >> 32);
}

// ---- width-switched integer access --------------------------------------
// Ids, offsets and masks arrive as 4- or 8-byte signed integers; the width is
// uniform across the launch, so the branch is scalar.
// A result size the host is polling for (int64 in pinned host memory, or in
// device memory that the host copies later): one store that bypasses the
// caches, visible to the host as soon as it lands. Not a fence: nothing else
// the kernel wrote is meant to be read by the host before it synchronises, and
// a system-scope fence would write the whole L2 back to make this one word
// visible.
__device__ __forceinline__ void publish_size(int64_t *slot, int64_t value) {
  __hip_atomic_store(slot, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

__device__ __forceinline__ int64_t load_int(const void *p, int64_t i, int bytes) {
  return bytes == 8 ? static_cast<const int64_t *>(p)[i]
                    : static_cast<int64_t>(static_cast<const int32_t *>(p)[i]);
}

// Several independent loads under ONE width branch. load_int() ends in a
// join of its two width paths, which makes the compiler wait for each value
// before the next load is issued; here all N loads of the chosen width are
// issued back to back. Entries with ok[n] false are skipped (out[n] untouched).
template <int N>
__device__ __forceinline__ void load_ints(const void *p, const int64_t (&idx)[N],
                                          const bool (&ok)[N], int bytes, int64_t (&out)[N]) {
  if (bytes == 8) {
    const int64_t *q = static_cast<const int64_t *>(p);
#pragma unroll
    for (int n = 0; n < N; ++n)
      if (ok[n]) out[n] = q[idx[n]];
  } else {
    const int32_t *q = static_cast<const int32_t *>(p);
    int32_t tmp[N];
#pragma unroll
    for (int n = 0; n < N; ++n)
      if (ok[n]) tmp[n] = q[idx[n]];
#pragma unroll
    for (int n = 0; n < N; ++n)
      if (ok[n]) out[n] = static_cast<int64_t>(tmp[n]);
  }
}

// p[i] and p[i + 1] (a CSR row's two offsets) in flight together.
__device__ __forceinline__ void load_int_pair(const void *p, int64_t i, int bytes, int64_t *a,
                                              int64_t *b) {
  if (bytes == 8) {
    const int64_t *q = static_cast<const int64_t *>(p);
    const int64_t x = q[i], y = q[i + 1];
    *a = x;
    *b = y;
  } else {
    const int32_t *q = static_cast<const int32_t *>(p);
    const int32_t x = q[i], y = q[i + 1];
    *a = x;
    *b = y;
  }
}

__device__ __forceinline__ void store_int(void *p, int64_t i, int bytes, int64_t v) {
  if (bytes == 8)
    static_cast<int64_t *>(p)[i] = v;
  else
    static_cast<int32_t *>(p)[i] = static_cast<int32_t>(v);
}

// ---- sub-wave groups -----------------------------------------------------
// Ballot restricted to the aligned group of `G` lanes (G a power of two <= 64)
// that contains the calling lane. Every lane of the group must be active.
template <int G>
__device__ __forceinline__ uint64_t group_ballot(bool pred) {
  uint64_t m = __builtin_amdgcn_ballot_w64(pred);
  if (G == 64) return m;
  int base = lane_id() & ~(G - 1);
  return (m >> base) & ((1ull << (G % 64)) - 1ull);
}

__device__ __forceinline__ uint64_t group_ballot_dyn(bool pred, int G) {
  uint64_t m = __builtin_amdgcn_ballot_w64(pred);
  if (G >= 64) return m;
  int base = lane_id() & ~(G - 1);
  return (m >> base) & ((1ull << G) - 1ull);
}

__device__ __forceinline__ int64_t shfl64(int64_t v, int src_lane) {
  int lo = __shfl(static_cast<int>(static_cast<uint64_t>(v)), src_lane, kWave);
  int hi = __shfl(static_cast<int>(static_cast<uint64_t>(v) >> 32), src_lane, kWave);
  return static_cast<int64_t>((static_cast<uint64_t>(static_cast<uint32_t>(hi)) << 32) |
                              static_cast<uint32_t>(lo));
}

// ---- wavefront scans -----------------------------------------------------
// Inclusive prefix sum across the 64 lanes with DPP row shifts and the two
// gfx9 row broadcasts; lanes shifted in from outside a row read zero
// (bound_ctrl), and the broadcasts are masked to the rows that need them.
__device__ __forceinline__ uint32_t dpp_shr_add(uint32_t v, const int ctrl_sel) {
  // ctrl_sel: 1,2,4,8 -> row_shr; 15 -> row_bcast15 (rows 1,3); 31 -> row_bcast31 (rows 2,3)
  switch (ctrl_sel) {
    case 1:
      return v + __builtin_amdgcn_update_dpp(0u, v, 0x111, 0xf, 0xf, true);
    case 2:
      return v + __builtin_amdgcn_update_dpp(0u, v, 0x112, 0xf, 0xf, true);
    case 4:
      return v + __builtin_amdgcn_update_dpp(0u, v, 0x114, 0xf, 0xf, true);
    case 8:
      return v + __builtin_amdgcn_update_dpp(0u, v, 0x118, 0xf, 0xf, true);
    case 15:
      return v + __builtin_amdgcn_update_dpp(0u, v, 0x142, 0xa, 0xf, false);
    default:
      return v + __builtin_amdgcn_update_dpp(0u, v, 0x143, 0xc, 0xf, false);
  }
}

__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
  v = dpp_shr_add(v, 1);
  v = dpp_shr_add(v, 2);
  v = dpp_shr_add(v, 4);
  v = dpp_shr_add(v, 8);
  v = dpp_shr_add(v, 15);
  v = dpp_shr_add(v, 31);
  return v;
}

// 64-bit variant: the two halves travel through the same DPP pattern and are
// recombined before each add so carries propagate.
__device__ __forceinline__ uint64_t dpp_move64(uint64_t v, const int ctrl_sel) {
  uint32_t lo = static_cast<uint32_t>(v), hi = static_cast<uint32_t>(v >> 32);
  uint32_t mlo, mhi;
  switch (ctrl_sel) {
    case 1:
      mlo = __builtin_amdgcn_update_dpp(0u, lo, 0x111, 0xf, 0xf, true);
      mhi = __builtin_amdgcn_update_dpp(0u, hi, 0x111, 0xf, 0xf, true);
      break;
    case 2:
      mlo = __builtin_amdgcn_update_dpp(0u, lo, 0x112, 0xf, 0xf, true);
      mhi = __builtin_amdgcn_update_dpp(0u, hi, 0x112, 0xf, 0xf, true);
      break;
    case 4:
      mlo = __builtin_amdgcn_update_dpp(0u, lo, 0x114, 0xf, 0xf, true);
      mhi = __builtin_amdgcn_update_dpp(0u, hi, 0x114, 0xf, 0xf, true);
      break;
    case 8:
      mlo = __builtin_amdgcn_update_dpp(0u, lo, 0x118, 0xf, 0xf, true);
      mhi = __builtin_amdgcn_update_dpp(0u, hi, 0x118, 0xf, 0xf, true);
      break;
    case 15:
      mlo = __builtin_amdgcn_update_dpp(0u, lo, 0x142, 0xa, 0xf, false);
      mhi = __builtin_amdgcn_update_dpp(0u, hi, 0x142, 0xa, 0xf, false);
      break;
    default:
      mlo = __builtin_amdgcn_update_dpp(0u, lo, 0x143, 0xc, 0xf, false);
      mhi = __builtin_amdgcn_update_dpp(0u, hi, 0x143, 0xc, 0xf, false);
      break;
  }
  return (static_cast<uint64_t>(mhi) << 32) | mlo;
}

__device__ __forceinline__ uint64_t wave_inclusive_scan(uint64_t v) {
  v += dpp_move64(v, 1);
  v += dpp_move64(v, 2);
  v += dpp_move64(v, 4);
  v += dpp_move64(v, 8);
  v += dpp_move64(v, 15);
  v += dpp_move64(v, 31);
  return v;
}

// Value held by lane 63 (the wave total after an inclusive scan), broadcast.
__device__ __forceinline__ uint32_t wave_last(uint32_t v) {
  return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), 63));
}
__device__ __forceinline__ uint64_t wave_last(uint64_t v) {
  uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(v)), 63));
  uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(v >> 32)), 63));
  return (static_cast<uint64_t>(hi) << 32) | lo;
}

// ---- workgroup scan ------------------------------------------------------
// Exclusive prefix sum of one value per thread across a workgroup of
// BLOCK threads (BLOCK a multiple of 64, <= 1024). `lds` must hold BLOCK/64
// elements of T. Returns the exclusive prefix; *block_total receives the
// workgroup sum in every thread. Contains two barriers.
template <typename T, int BLOCK>
__device__ __forceinline__ T block_exclusive_scan(T v, T *lds, T *block_total) {
  constexpr int NW = BLOCK / kWave;
  T inc = wave_inclusive_scan(v);
  int w = threadIdx.x / kWave;
  if (lane_id() == kWave - 1) lds[w] = inc;
  __syncthreads();
  T wave_prefix = 0, total = 0;
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    T t = lds[i];
    if (i < w) wave_prefix += t;
    total += t;
  }
  __syncthreads();
  *block_total = total;
  return wave_prefix + inc - v;
}

}  // namespace shmt
