// Feature row gather (fetch) and scatter (set) through the HBM cache.
// Replaces the twelve kernels of src/cache_feature_fetch.cu:15-224 and
// src/cache_feature_set.cu:6-207 in the ShmTensor tree with one templated
// kernel: a sub-wave group of L lanes owns one row, the first 8 lanes of the
// group resolve the row's cache slot (cooperative hashmap probe, or a mask
// load), and the group then moves the row with the widest vector access the
// row size and the base pointers allow (16 bytes per lane when aligned).
#include "common.h"
#include "hashmap.h"
#include "hashmap_dev.h"

namespace shmt {

enum RouteMode : int { kDirect = 0, kMap16 = 1, kMap8 = 2, kMask = 3 };

struct RowArgs {
  char *miss;          // table addressed by id (pinned host alias or device)
  char *cache;         // table addressed by slot (HBM)
  char *dense;         // fetch: output rows; set: update rows
  const void *indices;
  const void *mask;
  MapView map;
  int64_t Q;
  int64_t row_bytes;
  int idx_bytes;
  int mask_bytes;
  int log2_lanes;      // lanes per row = 1 << log2_lanes, in [8, 64]
};

template <typename VT, bool SET>
__device__ __forceinline__ void move_vec(char *table_row, char *dense_row, int64_t off) {
  if (SET)
    *reinterpret_cast<VT *>(table_row + off) = *reinterpret_cast<const VT *>(dense_row + off);
  else
    *reinterpret_cast<VT *>(dense_row + off) = *reinterpret_cast<const VT *>(table_row + off);
}

template <typename VT, int MODE, bool SET>
__global__ __launch_bounds__(256) void rows_kernel(RowArgs a) {
  const int lane = lane_id();
  const int L = 1 << a.log2_lanes;
  const int gl = lane & (L - 1);
  const int grp = lane >> a.log2_lanes;
  const int rows_per_wave = kWave >> a.log2_lanes;
  const int64_t waves_per_block = blockDim.x / kWave;
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * waves_per_block + threadIdx.x / kWave;
  const int64_t nwaves = static_cast<int64_t>(gridDim.x) * waves_per_block;
  const int64_t R = a.row_bytes;
  const int64_t step = static_cast<int64_t>(L) * sizeof(VT);

  for (int64_t row0 = wave * rows_per_wave; row0 < a.Q; row0 += nwaves * rows_per_wave) {
    const int64_t row = row0 + grp;
    if (row >= a.Q) continue;  // uniform within the row group
    const int64_t idx = load_int(a.indices, row, a.idx_bytes);
    int64_t slot = -1;
    if (MODE == kMask) {
      slot = load_int(a.mask, row, a.mask_bytes);
    } else if (MODE == kMap16 || MODE == kMap8) {
      int64_t v = -1;
      if (gl < kProbeGroup)
        v = group_find<MODE == kMap16 ? kSlot16 : kSlot8>(a.map, map_key(a.map, idx));
      slot = shfl64(v, lane & ~(L - 1));
    }
    char *table_row = slot >= 0 ? a.cache + slot * R : a.miss + idx * R;
    char *dense_row = a.dense + row * R;

    int64_t off = static_cast<int64_t>(gl) * sizeof(VT);
    // four independent vector moves per lane per trip keep loads in flight
    for (; off + 3 * step < R; off += 4 * step) {
      VT v0, v1, v2, v3;
      const char *src = SET ? dense_row : table_row;
      char *dst = SET ? table_row : dense_row;
      v0 = *reinterpret_cast<const VT *>(src + off);
      v1 = *reinterpret_cast<const VT *>(src + off + step);
      v2 = *reinterpret_cast<const VT *>(src + off + 2 * step);
      v3 = *reinterpret_cast<const VT *>(src + off + 3 * step);
      *reinterpret_cast<VT *>(dst + off) = v0;
      *reinterpret_cast<VT *>(dst + off + step) = v1;
      *reinterpret_cast<VT *>(dst + off + 2 * step) = v2;
      *reinterpret_cast<VT *>(dst + off + 3 * step) = v3;
    }
    for (; off < R; off += step) move_vec<VT, SET>(table_row, dense_row, off);
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

template <typename VT, bool SET>
static void launch_mode(int mode, unsigned grid, hipStream_t s, const RowArgs &a) {
  switch (mode) {
    case kDirect:
      hipLaunchKernelGGL((rows_kernel<VT, kDirect, SET>), dim3(grid), dim3(256), 0, s, a);
      break;
    case kMap16:
      hipLaunchKernelGGL((rows_kernel<VT, kMap16, SET>), dim3(grid), dim3(256), 0, s, a);
      break;
    case kMap8:
      hipLaunchKernelGGL((rows_kernel<VT, kMap8, SET>), dim3(grid), dim3(256), 0, s, a);
      break;
    default:
      hipLaunchKernelGGL((rows_kernel<VT, kMask, SET>), dim3(grid), dim3(256), 0, s, a);
      break;
  }
}

template <bool SET>
static int move_rows(const char *who, void *miss, void *cache, const void *indices, int idx_bytes,
                     const shmt_hashmap_t *map, const void *mask, int mask_bytes, void *dense,
                     int64_t Q, int64_t row_bytes, void *stream) {
  SHMT_REQUIRE(Q >= 0, "%s: Q must be >= 0", who);
  SHMT_REQUIRE(row_bytes > 0, "%s: row_bytes must be > 0", who);
  SHMT_REQUIRE(width_ok(idx_bytes), "%s: ID can only be int32 or int64 (idx_bytes=%d)", who, idx_bytes);
  SHMT_REQUIRE(!(map && mask), "%s: pass a hashmap or a mask, not both", who);
  if (Q == 0) return SHMT_OK;
  SHMT_REQUIRE(indices != nullptr && dense != nullptr, "%s: null indices/rows buffer", who);
  SHMT_REQUIRE(miss != nullptr, "%s: the id-addressed table is null", who);
  int mode = kDirect;
  if (map) {
    mode = map->fmt == kSlot16 ? kMap16 : kMap8;
    SHMT_REQUIRE(cache != nullptr, "%s: cache table is null", who);
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
  if (map) a.map = map->view; else a.map = MapView{nullptr, 1, 0};
  a.Q = Q;
  a.row_bytes = row_bytes;
  a.idx_bytes = idx_bytes;
  a.mask_bytes = mask_bytes;

  const int vb = pick_vector_bytes(row_bytes, miss, cache, dense);
  const int64_t nvec = row_bytes / vb;
  int log2_lanes = 3;
  while (log2_lanes < 6 && (1ll << log2_lanes) < nvec) ++log2_lanes;
  a.log2_lanes = log2_lanes;
  const int rows_per_block = 4 * (kWave >> log2_lanes);
  const unsigned grid = grid_for(Q, rows_per_block);
  hipStream_t s = as_stream(stream);
  switch (vb) {
    case 16: launch_mode<uint4, SET>(mode, grid, s, a); break;
    case 8: launch_mode<uint2, SET>(mode, grid, s, a); break;
    case 4: launch_mode<uint32_t, SET>(mode, grid, s, a); break;
    case 2: launch_mode<uint16_t, SET>(mode, grid, s, a); break;
    default: launch_mode<uint8_t, SET>(mode, grid, s, a); break;
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

int shmt_set(void *miss_data, void *cache_data, const void *indices, int idx_bytes,
             const shmt_hashmap_t *map, const void *mask, int mask_bytes, const void *update,
             int64_t Q, int64_t row_bytes, void *stream) {
  return shmt::move_rows<true>("shmt_set", miss_data, cache_data, indices, idx_bytes, map, mask,
                               mask_bytes, const_cast<void *>(update), Q, row_bytes, stream);
}

}  // extern "C"
