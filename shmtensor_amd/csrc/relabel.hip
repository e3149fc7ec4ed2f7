// Relabel: distinct values in order of first occurrence + position of every
// input element in that list. Replaces TensorRelabel / RelabelHashmap
// (src/tensor_relabel.cu:68-209 in the ShmTensor tree).
//
// Passes over the N inputs (each a separate launch, no host round trip):
//   fill     table slots {key = -1, first = 0xFFFFFFFF}
//   insert   claim a slot per distinct key (64-bit CAS), atomicMin the index
//   first    first[i] = smallest index holding the same key (kept in the
//            labels buffer); per-tile count of i with first[i] == i
//   partials exclusive scan of the per-tile counts
//   unique   rank of every first occurrence; unique[rank] = key; rank_of[i]
//   labels   labels[i] = rank_of[first[i]]
// The table is touched only by `insert` and `first`; the last two passes read
// dense arrays. Slots are 16 bytes {int64 key, uint32 first, pad} at load
// factor <= 0.5 with a mixed hash (the reference hashes with the low bits of
// the id, src/tensor_relabel.cu:111-117).
#include "common.h"
#include "launchers.h"
#include "scan_dev.h"

namespace shmt {

constexpr int kRlBlock = 256;
constexpr int kRlItems = 8;
constexpr int kRlTile = kRlBlock * kRlItems;

struct RlSlot {
  int64_t key;
  uint32_t first;
  uint32_t pad;
};
static_assert(sizeof(RlSlot) == 16, "slot must be 16 bytes");

static int64_t rl_capacity(int64_t N) {
  int64_t cap = 2 * N;
  if (cap < 64) cap = 64;
  return (cap + 7) & ~7ll;
}

struct RlLayout {
  int64_t cap, table_off, rank_off, partial_off, total;
};

static RlLayout rl_layout(int64_t N) {
  RlLayout l;
  l.cap = rl_capacity(N);
  l.table_off = 0;
  l.rank_off = l.cap * 16;
  int64_t rank_bytes = (N * 4 + 127) & ~127ll;
  l.partial_off = l.rank_off + rank_bytes;
  int64_t nb = (N + kRlTile - 1) / kRlTile;
  l.total = l.partial_off + ((nb * 8 + 127) & ~127ll);
  return l;
}

__global__ __launch_bounds__(256) void rl_insert_kernel(RlSlot *tbl, uint32_t cap,
                                                        const void *total, int eb, int64_t N) {
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (; i < N; i += stride) {
    const int64_t key = load_int(total, i, eb);
    uint32_t pos = reduce_range(hash_id(key), cap);
    for (uint32_t probes = 0; probes < cap; ++probes) {
      unsigned long long prev =
          atomicCAS(reinterpret_cast<unsigned long long *>(&tbl[pos].key), ~0ull,
                    static_cast<unsigned long long>(key));
      if (prev == ~0ull || static_cast<int64_t>(prev) == key) {
        atomicMin(&tbl[pos].first, static_cast<uint32_t>(i));
        break;
      }
      pos = (pos + 1 == cap) ? 0 : pos + 1;
    }
  }
}

__device__ __forceinline__ uint32_t rl_find_first(const RlSlot *tbl, uint32_t cap, int64_t key) {
  uint32_t pos = reduce_range(hash_id(key), cap);
  for (uint32_t probes = 0; probes < cap; ++probes) {
    const uint4 s = *reinterpret_cast<const uint4 *>(&tbl[pos]);
    const int64_t k = static_cast<int64_t>((static_cast<uint64_t>(s.y) << 32) | s.x);
    if (k == key) return s.z;
    if (k == -1) break;
    pos = (pos + 1 == cap) ? 0 : pos + 1;
  }
  return 0xFFFFFFFFu;
}

__global__ __launch_bounds__(kRlBlock) void rl_first_kernel(const RlSlot *tbl, uint32_t cap,
                                                            const void *total, int eb, int64_t N,
                                                            void *labels, uint64_t *partials) {
  __shared__ uint64_t lds[kRlBlock / kWave];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kRlTile;
  uint64_t cnt = 0;
#pragma unroll
  for (int j = 0; j < kRlItems; ++j) {
    const int64_t i = base + j * kRlBlock + threadIdx.x;
    if (i < N) {
      const uint32_t f = rl_find_first(tbl, cap, load_int(total, i, eb));
      store_int(labels, i, eb, static_cast<int64_t>(f));
      cnt += (f == static_cast<uint32_t>(i));
    }
  }
  uint64_t tile_total;
  block_exclusive_scan<uint64_t, kRlBlock>(cnt, lds, &tile_total);
  if (threadIdx.x == 0) partials[blockIdx.x] = tile_total;
}

__global__ __launch_bounds__(kRlBlock) void rl_unique_kernel(const void *total, int eb, int64_t N,
                                                             const void *labels,
                                                             const uint64_t *partials,
                                                             void *unique_out, uint32_t *rank_of,
                                                             int64_t *count_out) {
  __shared__ uint32_t lds[kRlBlock / kWave];
  const int64_t first_i = static_cast<int64_t>(blockIdx.x) * kRlTile +
                          static_cast<int64_t>(threadIdx.x) * kRlItems;
  bool win[kRlItems];
  uint32_t mine = 0;
#pragma unroll
  for (int j = 0; j < kRlItems; ++j) {
    const int64_t i = first_i + j;
    win[j] = (i < N) && (load_int(labels, i, eb) == i);
    mine += win[j];
  }
  uint32_t tile_total;
  uint32_t ex = block_exclusive_scan<uint32_t, kRlBlock>(mine, lds, &tile_total);
  uint64_t rank = partials[blockIdx.x] + ex;
#pragma unroll
  for (int j = 0; j < kRlItems; ++j) {
    const int64_t i = first_i + j;
    if (win[j]) {
      store_int(unique_out, static_cast<int64_t>(rank), eb, load_int(total, i, eb));
      rank_of[i] = static_cast<uint32_t>(rank);
      ++rank;
    }
  }
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) {
    *count_out = static_cast<int64_t>(partials[blockIdx.x] + tile_total);
    __threadfence_system();
  }
}

__global__ __launch_bounds__(256) void rl_labels_kernel(void *labels, int eb, int64_t N,
                                                        const uint32_t *rank_of) {
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (; i < N; i += stride) {
    const int64_t f = load_int(labels, i, eb);
    store_int(labels, i, eb, static_cast<int64_t>(rank_of[f]));
  }
}

__global__ void rl_zero_count_kernel(int64_t *count_out) {
  *count_out = 0;
  __threadfence_system();
}

}  // namespace shmt

using namespace shmt;

extern "C" {

int64_t shmt_relabel_scratch_bytes(int64_t N) {
  if (N < 0) return -1;
  return rl_layout(N).total;
}

int shmt_relabel(const void *total, int64_t N, int elem_bytes, void *scratch,
                 int64_t scratch_bytes, void *unique_out, void *labels_out, int64_t *count_out,
                 void *stream) {
  SHMT_REQUIRE(N >= 0, "shmt_relabel: N must be >= 0");
  SHMT_REQUIRE(N < (1ll << 31), "shmt_relabel: N must be < 2^31");
  SHMT_REQUIRE(width_ok(elem_bytes), "shmt_relabel: ID can only be int32 or int64");
  SHMT_REQUIRE(count_out != nullptr, "shmt_relabel: count_out is null");
  hipStream_t s = as_stream(stream);
  if (N == 0) {
    hipLaunchKernelGGL(rl_zero_count_kernel, dim3(1), dim3(1), 0, s, count_out);
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
  uint32_t *rank_of = reinterpret_cast<uint32_t *>(base + l.rank_off);
  uint64_t *partials = reinterpret_cast<uint64_t *>(base + l.partial_off);
  const int64_t nb = (N + kRlTile - 1) / kRlTile;
  const uint32_t cap = static_cast<uint32_t>(l.cap);

  int rc = launch_fill_ones(tbl, l.cap, s);
  if (rc) return rc;
  hipLaunchKernelGGL(rl_insert_kernel, dim3(grid_for(N, 256)), dim3(256), 0, s, tbl, cap, total,
                     elem_bytes, N);
  SHMT_LAUNCH_CHECK();
  hipLaunchKernelGGL(rl_first_kernel, dim3(static_cast<unsigned>(nb)), dim3(kRlBlock), 0, s, tbl,
                     cap, total, elem_bytes, N, labels_out, partials);
  SHMT_LAUNCH_CHECK();
  rc = launch_scan_partials(partials, nb, s);
  if (rc) return rc;
  hipLaunchKernelGGL(rl_unique_kernel, dim3(static_cast<unsigned>(nb)), dim3(kRlBlock), 0, s,
                     total, elem_bytes, N, labels_out, partials, unique_out, rank_of, count_out);
  SHMT_LAUNCH_CHECK();
  hipLaunchKernelGGL(rl_labels_kernel, dim3(grid_for(N, 256)), dim3(256), 0, s, labels_out,
                     elem_bytes, N, rank_of);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

}  // extern "C"
