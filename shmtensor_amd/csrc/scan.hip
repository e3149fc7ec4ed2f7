// Device-wide in-place prefix sums over 4- or 8-byte integers.
// Replaces cub::DeviceScan::ExclusiveSum as used by cub_exclusiveSum
// (src/tensor_relabel.cu:11-26, src/cache_graph_sampling.cu:30-45 in the
// ShmTensor tree) and the exported thrust_scan (src/thrust_scan.cu:9-18).
//
// Wave level: DPP row shifts + row broadcasts (wave.h). Workgroup level: one
// LDS word per wave. Device level: inputs up to kSingleBlockMax elements are
// scanned by one 1024-thread workgroup that walks the array with a running
// carry (one launch). Larger inputs are scanned in ONE pass over the data
// (read once, written once): every workgroup takes the next tile from a
// counter, scans it locally, publishes the tile's sum, and obtains the sum of
// everything before its tile by looking back over the sums (or, where
// available, the finished prefixes) that the tiles before it have published.
// A tile only ever waits for tiles with smaller numbers, which were handed
// out earlier to workgroups that are already running, so the waiting ends.
#include <mutex>

#include "common.h"
#include "launchers.h"
#include "scan_dev.h"

namespace shmt {

constexpr int kScanBlock = 256;
constexpr int kScanItems = 8;
constexpr int kScanTile = kScanBlock * kScanItems;  // 2048 elements per workgroup
constexpr int64_t kSingleBlockMax = 1 << 16;

// One workgroup scans the partials in place (exclusive).
__global__ __launch_bounds__(1024) void scan_partials_kernel(uint64_t *partials, int64_t nb) {
  __shared__ uint64_t lds[1024 / kWave];
  uint64_t carry = 0;
  for (int64_t base = 0; base < nb; base += 1024) {
    int64_t i = base + threadIdx.x;
    uint64_t v = i < nb ? partials[i] : 0;
    uint64_t total;
    uint64_t ex = block_exclusive_scan<uint64_t, 1024>(v, lds, &total);
    if (i < nb) partials[i] = carry + ex;
    carry += total;
  }
}

int launch_scan_partials(uint64_t *partials, int64_t nb, hipStream_t s) {
  hipLaunchKernelGGL(scan_partials_kernel, dim3(1), dim3(1024), 0, s, partials, nb);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

// ---- single-pass device scan ---------------------------------------------------
// What a tile has published so far lives in two 64-bit words per tile, each
// {state : 32 | half of a 64-bit sum : 32}: state 0 = nothing yet, 1 = the
// tile's own sum, 2 = the sum of everything up to and including the tile.
// A reader takes a value only when both words carry the same non-zero state,
// so the two halves always belong together and no fence is needed: the payload
// travels inside the (relaxed, device-scope) atomic accesses themselves.
//
// Tiles are large (128 KiB): finished prefixes spread along the tiles at one
// look-back step (64 tiles) per memory round trip, and with small tiles that
// spreading, not the memory bandwidth, bounds the scan. Measured for
// 16,777,216 int64 (reduce / scan / apply in three launches, which this
// replaces: 125 us): 16 KiB tiles 204 us, 64 KiB 78 us, 128 KiB 64 us, 256 KiB
// 114 us (registers); inspecting 128 or 256 tiles per step gained nothing.
constexpr uint32_t kTileSum = 1, kTilePrefix = 2;
constexpr int64_t kScanHeaderBytes = 64;       // tile counter (+ padding) in front of the tile words
constexpr uint32_t kLookbackSpinLimit = 1u << 24;  // a wait that long means a tile before this one died
constexpr int kLbBlock = 512;                  // threads per tile
constexpr int kLbWaves = kLbBlock / kWave;
constexpr int kLbChunks = 16;                  // 16-byte vectors per lane
constexpr int kLbLook = 1;                     // tiles a lane inspects per look-back step
constexpr int64_t kLbTileBytes = static_cast<int64_t>(kLbWaves) * kLbChunks * kWave * 16;

struct ScanState {
  unsigned long long *counter;  // next tile to hand out
  uint64_t *words;              // 2 per tile
};

__device__ __forceinline__ void tile_publish(const ScanState &st, int64_t tile, uint32_t state, uint64_t sum) {
  const uint64_t tag = static_cast<uint64_t>(state) << 32;
  __hip_atomic_store(&st.words[2 * tile], tag | (sum & 0xFFFFFFFFull), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(&st.words[2 * tile + 1], tag | (sum >> 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Sum of all tiles before `tile` (tile >= 1), by one whole wave: in every step
// lane l looks at the tiles (look - l - 64 j), j < kLbLook; the nearest tile
// that already knows its prefix ends the walk, the own sums of the tiles in
// between are added up.
__device__ __forceinline__ uint64_t tile_lookback(const ScanState &st, int64_t tile) {
  const int lane = lane_id();
  uint64_t prefix = 0;
  uint32_t spins = 0;
  for (int64_t look = tile - 1;; look -= kWave * kLbLook) {
    uint32_t state[kLbLook];
    uint64_t sum[kLbLook];
    for (;;) {
      bool ready = true;
#pragma unroll
      for (int j = 0; j < kLbLook; ++j) {
        const int64_t t = look - lane - kWave * j;
        state[j] = kTilePrefix;  // in front of tile 0: an empty prefix
        sum[j] = 0;
        if (t >= 0) {
          const uint64_t w0 = __hip_atomic_load(&st.words[2 * t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          const uint64_t w1 = __hip_atomic_load(&st.words[2 * t + 1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          state[j] = static_cast<uint32_t>(w0 >> 32);
          ready = ready && state[j] != 0 && state[j] == static_cast<uint32_t>(w1 >> 32);
          sum[j] = (w1 << 32) | (w0 & 0xFFFFFFFFull);
        }
      }
      if (__builtin_amdgcn_ballot_w64(!ready) == 0 || ++spins >= kLookbackSpinLimit) break;
      __builtin_amdgcn_s_sleep(1);
    }
#pragma unroll
    for (int j = 0; j < kLbLook; ++j) {
      const uint64_t done = __builtin_amdgcn_ballot_w64(state[j] == kTilePrefix);
      const int last = done ? __builtin_ctzll(done) : kWave - 1;  // nearest tile with a finished prefix
      prefix += wave_last(wave_inclusive_scan(lane <= last ? sum[j] : static_cast<uint64_t>(0)));
      if (done) return prefix;
    }
  }
}

__global__ __launch_bounds__(256) void scan_state_clear_kernel(uint64_t *p, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = 0;
}

template <typename T>
struct alignas(16) ScanVec {
  T e[16 / sizeof(T)];
};

// One tile per workgroup. A wave owns a contiguous stretch of the tile and
// walks it in kLbChunks steps of 64 lanes x 16 bytes (one coalesced kilobyte
// per step), so the whole tile sits in registers between its single read and
// its single write. `data` is 16-byte aligned: the up to three elements in
// front of the first 16-byte boundary of the caller's array (`head`, n_head of
// them) are scanned by the first thread of tile 0, and their sum starts the
// prefix that the tiles hand on.
template <typename T, bool INCLUSIVE>
__global__ __launch_bounds__(kLbBlock) void scan_lookback_kernel(T *head, int n_head, T *data, int64_t len,
                                                                 ScanState st) {
  constexpr int V = 16 / sizeof(T);
  constexpr int64_t kTileElems = kLbTileBytes / sizeof(T);
  __shared__ uint64_t wave_total[kLbWaves];
  __shared__ uint64_t shared[2];  // tile number, then the sum of everything before the tile
  if (threadIdx.x == 0) shared[0] = atomicAdd(st.counter, 1ull);
  __syncthreads();
  const int64_t tile = static_cast<int64_t>(shared[0]);
  const int wave = threadIdx.x / kWave, lane = lane_id();
  const int64_t lane_base = tile * kTileElems + static_cast<int64_t>(wave) * kLbChunks * kWave * V + lane * V;
  const bool whole = (tile + 1) * kTileElems <= len;
  T v[kLbChunks][V];
  T excl[kLbChunks];  // sum (mod 2^width) of the tile's elements in front of this lane's vector of chunk c
  T carry = 0;  // all in-tile sums are taken in the element type: results are defined modulo its width
#pragma unroll
  for (int c = 0; c < kLbChunks; ++c) {
    const int64_t i = lane_base + static_cast<int64_t>(c) * kWave * V;
    if (whole) {
      const ScanVec<T> x = *reinterpret_cast<const ScanVec<T> *>(data + i);
#pragma unroll
      for (int e = 0; e < V; ++e) v[c][e] = x.e[e];
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) v[c][e] = (i + e < len) ? data[i + e] : static_cast<T>(0);
    }
  }
#pragma unroll
  for (int c = 0; c < kLbChunks; ++c) {
    T mine = 0;
#pragma unroll
    for (int e = 0; e < V; ++e) mine += v[c][e];
    const T inc = wave_inclusive_scan(mine);
    excl[c] = carry + inc - mine;
    carry += wave_last(inc);
  }
  if (lane == 0) wave_total[wave] = carry;
  __syncthreads();
  uint64_t in_tile = 0, total = 0;
#pragma unroll
  for (int w = 0; w < kLbWaves; ++w) {
    const uint64_t t = wave_total[w];
    if (w < wave) in_tile += t;
    total += t;
  }
  if (threadIdx.x < kWave) {  // the first wave talks to the other tiles
    uint64_t before = 0;
    if (tile > 0) {
      if (threadIdx.x == 0) tile_publish(st, tile, kTileSum, total);
      before = tile_lookback(st, tile);
    } else if (threadIdx.x == 0) {
      T run = 0;
      for (int k = 0; k < n_head; ++k) {
        const T x = head[k];
        head[k] = INCLUSIVE ? run + x : run;
        run += x;
      }
      before = static_cast<uint64_t>(run);
    }
    if (threadIdx.x == 0) {
      tile_publish(st, tile, kTilePrefix, before + total);
      shared[1] = before;
    }
  }
  __syncthreads();
  const uint64_t base = shared[1] + in_tile;
#pragma unroll
  for (int c = 0; c < kLbChunks; ++c) {
    const int64_t i = lane_base + static_cast<int64_t>(c) * kWave * V;
    T run = static_cast<T>(base) + excl[c];
    ScanVec<T> out;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      if (INCLUSIVE) run += v[c][e];
      out.e[e] = run;
      if (!INCLUSIVE) run += v[c][e];
    }
    if (whole) {
      *reinterpret_cast<ScanVec<T> *>(data + i) = out;
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e)
        if (i + e < len) data[i + e] = out.e[e];
    }
  }
}

template <typename T, bool INCLUSIVE>
__global__ __launch_bounds__(1024) void scan_single_kernel(T *data, int64_t len) {
  __shared__ T lds[1024 / kWave];
  T carry = 0;
  for (int64_t base = 0; base < len; base += 1024 * kScanItems)
    tile_scan_inplace<T, 1024, kScanItems, INCLUSIVE>(data, base, len, lds, &carry);
}

template <typename T, bool INCLUSIVE>
static int scan_inplace(T *data, int64_t len, void *tmp, int64_t tmp_bytes, hipStream_t s) {
  if (len <= kSingleBlockMax) {
    hipLaunchKernelGGL((scan_single_kernel<T, INCLUSIVE>), dim3(1), dim3(1024), 0, s, data, len);
    SHMT_LAUNCH_CHECK();
    return SHMT_OK;
  }
  // the kernel moves whole 16-byte vectors: up to three elements in front of the first 16-byte boundary
  // are left to tile 0's first thread
  SHMT_REQUIRE((reinterpret_cast<uintptr_t>(data) % sizeof(T)) == 0, "scan: data is not aligned to its element size");
  const int n_head = static_cast<int>(((16 - (reinterpret_cast<uintptr_t>(data) & 15)) & 15) / sizeof(T));
  T *const main_data = data + n_head;
  const int64_t main_len = len - n_head;
  const int64_t tile_elems = kLbTileBytes / static_cast<int64_t>(sizeof(T));
  const int64_t nb = (main_len + tile_elems - 1) / tile_elems;
  const int64_t need = kScanHeaderBytes + nb * 16;
  if (tmp == nullptr || tmp_bytes < need) {
    set_error("scan: tmp buffer too small (%lld < %lld bytes)", static_cast<long long>(tmp_bytes),
              static_cast<long long>(need));
    return SHMT_ENOMEM;
  }
  SHMT_REQUIRE(nb < (1ll << 31), "scan: input too large");
  SHMT_REQUIRE((reinterpret_cast<uintptr_t>(tmp) & 7) == 0, "scan: tmp must be 8-byte aligned");
  ScanState st;
  st.counter = static_cast<unsigned long long *>(tmp);
  st.words = reinterpret_cast<uint64_t *>(static_cast<char *>(tmp) + kScanHeaderBytes);
  // counter and tile words start at zero (a kernel, not a memset, so that the scan can be captured in a graph)
  hipLaunchKernelGGL(scan_state_clear_kernel, dim3(grid_for(need / 8, 256 * 4)), dim3(256), 0, s,
                     static_cast<uint64_t *>(tmp), need / 8);
  SHMT_LAUNCH_CHECK();
  hipLaunchKernelGGL((scan_lookback_kernel<T, INCLUSIVE>), dim3(static_cast<unsigned>(nb)), dim3(kLbBlock), 0, s,
                     data, n_head, main_data, main_len, st);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

// ---- scan without a caller-provided workspace -------------------------------
// The tile counter and tile words of shmt_exclusive_scan_noalloc live in this array, which
// is part of the loaded code object: every GPU the library runs on holds its
// own copy, at its own address, until the process ends. The name below is a
// host-side handle only; kernels are given the device address that
// hipGetSymbolAddress returns for the current device.
constexpr int64_t kStaticScanMaxLen = 1ll << 28;  // 268,435,456 elements
constexpr int64_t kStaticScanTiles = kStaticScanMaxLen / (kLbTileBytes / 8);
constexpr int64_t kStaticScanWords = kScanHeaderBytes / 8 + 2 * kStaticScanTiles;  // 256 KiB + 64 B
static __device__ __align__(256) uint64_t scratch[kStaticScanWords];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static uint64_t *g_scratch_ptr[kMaxDevices];  // device address of `scratch`, per device ordinal

// Device address of this GPU's copy of `scratch` (looked up once per device).
static int static_scan_scratch(uint64_t **out) {
  int dev = -1;
  SHMT_HIP(hipGetDevice(&dev));
  SHMT_REQUIRE(dev >= 0 && dev < kMaxDevices, "shmt_exclusive_scan_noalloc: device ordinal %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void *p = nullptr;
    SHMT_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    SHMT_REQUIRE(p != nullptr, "shmt_exclusive_scan_noalloc: no device address for the static workspace");
    g_scratch_ptr[dev] = static_cast<uint64_t *>(p);
  }
  *out = g_scratch_ptr[dev];
  return SHMT_OK;
}

}  // namespace shmt

using namespace shmt;

extern "C" {

int64_t shmt_scan_tmp_bytes(int64_t len) {
  if (len <= kSingleBlockMax) return 0;
  const int64_t tile_elems = kLbTileBytes / 8;  // tiles of the wider element type: an upper bound for both
  return kScanHeaderBytes + ((len + tile_elems - 1) / tile_elems) * 16;
}

int shmt_exclusive_scan(void *data, int64_t len, int elem_bytes, void *tmp, int64_t tmp_bytes,
                        void *stream) {
  SHMT_REQUIRE(len >= 0, "shmt_exclusive_scan: len must be >= 0");
  SHMT_REQUIRE(width_ok(elem_bytes), "shmt_exclusive_scan: ID can only be int32 or int64");
  if (len == 0) return SHMT_OK;
  SHMT_REQUIRE(data != nullptr, "shmt_exclusive_scan: data is null");
  if (elem_bytes == 8)
    return scan_inplace<uint64_t, false>(static_cast<uint64_t *>(data), len, tmp, tmp_bytes,
                                         as_stream(stream));
  return scan_inplace<uint32_t, false>(static_cast<uint32_t *>(data), len, tmp, tmp_bytes,
                                       as_stream(stream));
}

int shmt_exclusive_scan_noalloc(void *data, int64_t len, int elem_bytes, void *stream) {
  SHMT_REQUIRE(len >= 0, "shmt_exclusive_scan_noalloc: len must be >= 0");
  SHMT_REQUIRE(width_ok(elem_bytes), "shmt_exclusive_scan_noalloc: ID can only be int32 or int64");
  SHMT_REQUIRE(len <= kStaticScanMaxLen,
               "shmt_exclusive_scan_noalloc: len %lld exceeds the static workspace (at most %lld elements); "
               "use shmt_exclusive_scan with a caller-provided workspace",
               static_cast<long long>(len), static_cast<long long>(kStaticScanMaxLen));
  SHMT_REQUIRE(len == 0 || data != nullptr, "shmt_exclusive_scan_noalloc: data is null");
  // also for len == 0, so that an empty call can serve as the set-up call
  uint64_t *partials = nullptr;
  int rc = static_scan_scratch(&partials);
  if (rc) return rc;
  if (len == 0) return SHMT_OK;
  // The workspace keeps what the last call left in it; every call clears the
  // tile counter and the tile words it is going to use before it scans.
  const int64_t tmp_bytes = kStaticScanWords * static_cast<int64_t>(sizeof(uint64_t));
  if (elem_bytes == 8)
    return scan_inplace<uint64_t, false>(static_cast<uint64_t *>(data), len, partials, tmp_bytes,
                                         as_stream(stream));
  return scan_inplace<uint32_t, false>(static_cast<uint32_t *>(data), len, partials, tmp_bytes,
                                       as_stream(stream));
}

int shmt_inclusive_scan_i32(void *data, int64_t len, void *tmp, int64_t tmp_bytes, void *stream) {
  SHMT_REQUIRE(len >= 0, "shmt_inclusive_scan_i32: len must be >= 0");
  if (len == 0) return SHMT_OK;
  SHMT_REQUIRE(data != nullptr, "shmt_inclusive_scan_i32: data is null");
  return scan_inplace<uint32_t, true>(static_cast<uint32_t *>(data), len, tmp, tmp_bytes,
                                      as_stream(stream));
}

}  // extern "C"
