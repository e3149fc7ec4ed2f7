// Device-wide in-place prefix sums over 4- or 8-byte integers.
// Replaces cub::DeviceScan::ExclusiveSum as used by cub_exclusiveSum
// (src/tensor_relabel.cu:11-26, src/cache_graph_sampling.cu:30-45 in the
// ShmTensor tree) and the exported thrust_scan (src/thrust_scan.cu:9-18).
//
// Wave level: DPP row shifts + row broadcasts (wave.h). Workgroup level: one
// LDS word per wave. Device level: inputs up to kSingleBlockMax elements are
// scanned by one 1024-thread workgroup that walks the array with a running
// carry (one launch). Larger inputs are scanned in ONE pass over the data
// (read once, written once) by a grid no larger than the device holds at
// once: a workgroup takes tile numbers from a counter, one after the other,
// scans each tile locally, publishes the tile's sum, and obtains the sum of
// everything before the tile from the sums that the tiles before it have
// published (per tile, per group of 64 tiles, per run of 64 groups). A tile
// only ever waits for tiles with smaller numbers, and a number is only ever
// held by a workgroup that is running (and that never waits for a larger
// one), so the waiting ends whatever else shares the GPU. (Fixed tile
// numbers b, b + grid, ... would not give that: two such kernels on two
// streams could each hold compute units while waiting for workgroups of
// their own that have not been started.)
#include <mutex>

#include "common.h"
#include "launchers.h"
#include "scan_dev.h"

namespace shmt {

constexpr int kScanItems = 8;  // elements per thread and step of the one-workgroup scan
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
// What the tiles publish lives in 64-bit word pairs, each word {state : 32 |
// half of a 64-bit sum : 32}: state 0 = nothing yet, 1 = published. A reader
// takes a value only when both words carry the state, so the two halves
// always belong together and no fence is needed: the payload travels inside
// the (relaxed, device-scope) atomic accesses themselves.
//
// Three levels of sums keep the look-back at two or three dependent steps
// wherever a tile lies: every tile publishes its own sum; the last tile of
// each aligned group of 64 tiles also publishes the group's sum (its own plus
// the 63 before it, which it reads anyway); the last tile of each aligned run
// of 64 groups publishes that run's sum. A tile's prefix is then: tiles before
// it in its group + groups before its group in the run + runs before its run,
// three reads of at most 64 entries that are issued together.
//
// Measured on MI355X, 16,777,216 int64 in place (268 MB of traffic): a
// publish -> read step between workgroups takes tens of microseconds while the
// memory queues are full of tile traffic, so the scan wants few, large tiles
// and few levels (figures for fixed tile numbers): tiles of 16 / 32 / 64 / 128 KiB 216 / 90 / 57 / 52 us
// (256 KiB: 111 us, the tile no longer fits the registers); groups of 16 or 8
// instead of 64 (one level more for the same tiles) 67 / 112 us. Without
// effect: requesting the workgroup's next tile before the look-back, one
// 128-byte line per published entry, 256 instead of 512 workgroups. Fixed
// tile numbers (b, b + grid, ...) instead of the counter: 52 us, but not safe
// beside other kernels (see the top of this file); with the counter 57 us.
// Walking back over single tiles, one tile per workgroup (the earlier form),
// took 64 us.
constexpr uint32_t kPublished = 1;
constexpr uint32_t kLookbackSpinLimit = 1u << 24;  // a wait that long means a tile before this one died
constexpr uint32_t kErrScanWait = 1;               // bit of the error word: a look-back gave up

// Sticky error word of the library, one copy per GPU (part of the loaded code
// object, like the static scan workspace below): a kernel that gives up a
// bounded wait sets a bit here instead of finishing with a wrong result in
// silence. shmt_async_error() reads and clears it.
static __device__ uint32_t async_error_word;
constexpr int kLbBlock = 1024;                 // threads per tile
constexpr int kLbWaves = kLbBlock / kWave;
constexpr int kLbChunks = 8;                   // 16-byte vectors per lane
constexpr int64_t kLbTileBytes = static_cast<int64_t>(kLbWaves) * kLbChunks * kWave * 16;
constexpr int kLbFan = kWave;                  // tiles per group, groups per run

constexpr int64_t kScanHeaderBytes = 64;  // tile counter (+ padding) in front of the published sums

struct ScanState {
  unsigned long long *counter;  // next tile number to hand out; counter[1]: workgroups that are done
  uint32_t *error;              // the GPU's error word
  uint32_t *error_mirror;       // where the host watches for it (device alias of a pinned host word), or null
  int64_t words;                // 64-bit words of the workspace behind the header (tiles, groups, runs)
  uint64_t *tiles;              // 2 words per tile
  uint64_t *groups;             // 2 words per group of 64 tiles
  uint64_t *runs;               // 2 words per run of 64 groups
};

struct ScanTmpLayout {
  int64_t nb, ng, nr, tiles_off, groups_off, runs_off, total;
};

static ScanTmpLayout scan_tmp_layout(int64_t nb) {
  ScanTmpLayout l;
  l.nb = nb;
  l.ng = (nb + kLbFan - 1) / kLbFan;
  l.nr = (l.ng + kLbFan - 1) / kLbFan;
  l.tiles_off = kScanHeaderBytes;
  l.groups_off = l.tiles_off + nb * 16;
  l.runs_off = l.groups_off + l.ng * 16;
  l.total = l.runs_off + l.nr * 16;
  return l;
}

__device__ __forceinline__ void sum_publish(uint64_t *words, int64_t i, uint64_t sum) {
  const uint64_t tag = static_cast<uint64_t>(kPublished) << 32;
  __hip_atomic_store(&words[2 * i], tag | (sum & 0xFFFFFFFFull), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(&words[2 * i + 1], tag | (sum >> 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Reads entry i when `want`; false while it is not published yet.
__device__ __forceinline__ bool sum_read(const uint64_t *words, int64_t i, bool want, uint64_t *sum) {
  *sum = 0;
  if (!want) return true;
  const uint64_t w0 = __hip_atomic_load(&words[2 * i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const uint64_t w1 = __hip_atomic_load(&words[2 * i + 1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  *sum = (w1 << 32) | (w0 & 0xFFFFFFFFull);
  return static_cast<uint32_t>(w0 >> 32) == kPublished && static_cast<uint32_t>(w1 >> 32) == kPublished;
}

__device__ __forceinline__ uint64_t wave_sum_all(uint64_t v) { return wave_last(wave_inclusive_scan(v)); }

// Sum of all tiles before `tile`, by one whole wave; `own` is the tile's own
// sum (already published). Publishes the sums of the group and of the run
// that end with this tile. A tile only waits for entries that tiles with
// smaller numbers publish, which were handed out earlier to workgroups that
// are already running, so the waiting ends.
__device__ __forceinline__ uint64_t tile_lookback(const ScanState &st, int64_t tile, uint64_t own, bool *gave_up) {
  const int lane = lane_id();
  const int64_t group = tile / kLbFan, run = group / kLbFan;
  const int in_group = static_cast<int>(tile % kLbFan), in_run = static_cast<int>(group % kLbFan);
  // A wait ends without its value when it has spun for kLookbackSpinLimit rounds, or as soon as any tile
  // of this GPU has reported such a wait (checked every 256 rounds): the tiles behind a lost one would
  // otherwise each sit out the full limit, one after the other.
  auto hopeless = [&](uint32_t spins) {
    return spins >= kLookbackSpinLimit ||
           ((spins & 255u) == 255u && __hip_atomic_load(st.error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0);
  };
  // runs before this tile's run: at most 64 up to 262,144 tiles, in further steps of 64 beyond
  uint64_t far = 0;
  uint32_t spins = 0;
  bool lost = false;
  for (int64_t first = kWave; first < run; first += kWave) {
    uint64_t part = 0;
    bool ok = false;
    for (;;) {
      if (!ok) ok = sum_read(st.runs, first + lane, first + lane < run, &part);
      if (__builtin_amdgcn_ballot_w64(!ok) == 0) break;
      if (hopeless(++spins)) {
        lost = true;
        break;
      }
      __builtin_amdgcn_s_sleep(8);
    }
    far += part;
  }
  // a lane asks again only for what it has not seen published yet
  uint64_t a = 0, b = 0, c = 0;
  bool ok_a = false, ok_b = false, ok_c = false;
  while (!lost) {
    if (!ok_a) ok_a = sum_read(st.tiles, group * kLbFan + lane, lane < in_group, &a);
    if (!ok_b) ok_b = sum_read(st.groups, run * kLbFan + lane, lane < in_run, &b);
    if (!ok_c) ok_c = sum_read(st.runs, lane, lane < run, &c);
    if (__builtin_amdgcn_ballot_w64(!(ok_a && ok_b && ok_c)) == 0) break;
    if (hopeless(++spins)) lost = true;
    else __builtin_amdgcn_s_sleep(8);
  }
  if (lost) {  // report, publish nothing: the tile is left as it was and so is everything behind it
    if (lane == 0) {
      __hip_atomic_fetch_or(st.error, kErrScanWait, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      // a plain system-scope store: the host only asks whether the word is zero, the bits are in st.error
      if (st.error_mirror) __hip_atomic_store(st.error_mirror, kErrScanWait, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    *gave_up = true;
    return 0;
  }
  c += far;
  const uint64_t tiles_before = wave_sum_all(a), groups_before = wave_sum_all(b), runs_before = wave_sum_all(c);
  if (lane == 0 && in_group == kLbFan - 1) {
    sum_publish(st.groups, group, tiles_before + own);
    if (in_run == kLbFan - 1) sum_publish(st.runs, run, groups_before + tiles_before + own);
  }
  return tiles_before + groups_before + runs_before;
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
template <typename T, int C>
__device__ __forceinline__ void scan_tile_load(const T *data, int64_t len, int64_t lane_base, bool whole,
                                               T (&v)[C][16 / sizeof(T)]) {
  constexpr int V = 16 / sizeof(T);
#pragma unroll
  for (int c = 0; c < C; ++c) {
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
}

template <typename T, bool INCLUSIVE>
__global__ __launch_bounds__(kLbBlock) void scan_lookback_kernel(T *head, int n_head, T *data, int64_t len,
                                                                 int64_t nb, ScanState st) {
  constexpr int V = 16 / sizeof(T);
  constexpr int64_t kTileElems = kLbTileBytes / sizeof(T);
  __shared__ uint64_t wave_total[kLbWaves];
  __shared__ uint64_t shared_before;  // the sum of everything before the tile
  __shared__ uint64_t shared_tile;    // the workgroup's next tile number
  __shared__ int shared_lost;         // the look-back of this tile gave up: leave the tile as it is
  __shared__ int shared_last;         // this workgroup is the last one to finish its look-backs
  const int wave = threadIdx.x / kWave, lane = lane_id();
  const int64_t lane_off = static_cast<int64_t>(wave) * kLbChunks * kWave * V + lane * V;
  T v[kLbChunks][V];
  if (threadIdx.x == 0) {
    shared_tile = atomicAdd(st.counter, 1ull);
    // a workgroup that comes too late for any tile is done with its look-backs at once
    shared_last = shared_tile >= static_cast<uint64_t>(nb) && atomicAdd(st.counter + 1, 1ull) == gridDim.x - 1;
  }
  __syncthreads();
  int64_t tile = static_cast<int64_t>(shared_tile);
  if (tile < nb) scan_tile_load<T, kLbChunks>(data, len, tile * kTileElems + lane_off, (tile + 1) * kTileElems <= len, v);
  while (tile < nb) {
    // The next tile number is asked for now and only looked at after the look-back, which hides the round
    // trip. One number per request: a workgroup that held two would publish the second tile's sum only
    // after it had written the first tile out, and every later tile would wait for that (measured: 2.2 ms).
    unsigned long long next_ticket = 0;
    if (threadIdx.x == 0) next_ticket = atomicAdd(st.counter, 1ull);
    const int64_t lane_base = tile * kTileElems + lane_off;
    const bool whole = (tile + 1) * kTileElems <= len;
    T excl[kLbChunks];  // sum (mod 2^width) of the tile's elements in front of this lane's vector of chunk c
    T carry = 0;  // all in-tile sums are taken in the element type: results are defined modulo its width
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
      bool lost = false;
      if (tile == 0) {
        T run = 0;
        if (threadIdx.x == 0) {
          for (int k = 0; k < n_head; ++k) {
            const T x = head[k];
            head[k] = INCLUSIVE ? run + x : run;
            run += x;
          }
        }
        before = static_cast<uint64_t>(run);  // used by thread 0 only
        if (threadIdx.x == 0) sum_publish(st.tiles, 0, before + total);
      } else {
        if (threadIdx.x == 0) sum_publish(st.tiles, tile, total);
        before = tile_lookback(st, tile, total, &lost);
      }
      if (threadIdx.x == 0) {
        shared_before = before;
        shared_tile = next_ticket;
        shared_lost = lost;
        // no tile left for this workgroup: its look-backs are over; the last workgroup to say so
        // clears the workspace (below), when nobody reads the published words any more
        if (next_ticket >= static_cast<unsigned long long>(nb))
          shared_last = atomicAdd(st.counter + 1, 1ull) == gridDim.x - 1;
      }
    }
    __syncthreads();
    const uint64_t base = shared_before + in_tile;
    const int64_t next = static_cast<int64_t>(shared_tile);
#pragma unroll
    for (int c = 0; c < kLbChunks; ++c) {
      if (shared_lost) break;
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
    if (next < nb) scan_tile_load<T, kLbChunks>(data, len, next * kTileElems + lane_off, (next + 1) * kTileElems <= len, v);
    tile = next;
  }  // the barriers above also order the reuse of the LDS words by the next tile
  // The workgroup that ends its look-backs last leaves the workspace as it found it, all zero: counter,
  // done count and every published word. A workspace that starts clean therefore stays clean from scan to
  // scan and needs no clearing launch in front of the next one (also when this launch is replayed from a
  // graph). shared_last was written before the last barrier above.
  if (shared_last) {
    uint64_t *const words = reinterpret_cast<uint64_t *>(st.counter) + kScanHeaderBytes / 8;
    for (int64_t i = threadIdx.x; i < st.words; i += kLbBlock) words[i] = 0;
    if (threadIdx.x < 2) st.counter[threadIdx.x] = 0;
  }
}

template <typename T, bool INCLUSIVE>
__global__ __launch_bounds__(1024) void scan_single_kernel(T *data, int64_t len) {
  __shared__ T lds[1024 / kWave];
  T carry = 0;
  for (int64_t base = 0; base < len; base += 1024 * kScanItems)
    tile_scan_inplace<T, 1024, kScanItems, INCLUSIVE>(data, base, len, lds, &carry);
}

// Workgroups of `kernel` that the current device holds at once (cached per kernel and device).
static int resident_workgroups(const void *kernel, int *out) {
  static std::mutex mu;
  struct Entry { const void *kernel; int dev, n; };
  static Entry cache[32];
  static int used = 0;
  int dev = -1;
  SHMT_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mu);
  for (int i = 0; i < used; ++i)
    if (cache[i].kernel == kernel && cache[i].dev == dev) { *out = cache[i].n; return SHMT_OK; }
  int per_cu = 0, cus = 0;
  SHMT_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kLbBlock, 0));
  SHMT_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  SHMT_REQUIRE(per_cu >= 1 && cus >= 1, "scan: the device reports no room for the scan kernel");
  const int n = per_cu * cus;
  if (used < 32) cache[used++] = Entry{kernel, dev, n};
  *out = n;
  return SHMT_OK;
}

// Device address of this GPU's error word (looked up once per device).
constexpr int kMaxDevices = 64;
static std::mutex g_symbol_mutex;
static uint32_t *g_error_ptr[kMaxDevices];
static uint32_t *g_mirror_dev[kMaxDevices];            // shmt_async_error_mirror: the pinned word as the GPU addresses it
static volatile uint32_t *g_mirror_host[kMaxDevices];  // and as the host does

static int error_word(uint32_t **out) {
  int dev = -1;
  SHMT_HIP(hipGetDevice(&dev));
  SHMT_REQUIRE(dev >= 0 && dev < kMaxDevices, "scan: device ordinal %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_symbol_mutex);
  if (g_error_ptr[dev] == nullptr) {
    void *p = nullptr;
    SHMT_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(async_error_word)));
    SHMT_REQUIRE(p != nullptr, "scan: no device address for the error word");
    g_error_ptr[dev] = static_cast<uint32_t *>(p);
  }
  *out = g_error_ptr[dev];
  return SHMT_OK;
}

static uint32_t *error_mirror() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_symbol_mutex);
  return g_mirror_dev[dev];
}

// kept: the workspace is all zero (it was cleared once and has only been used by scans since, each of
// which leaves it all zero); otherwise it is cleared first.
template <typename T, bool INCLUSIVE>
static int scan_inplace(T *data, int64_t len, void *tmp, int64_t tmp_bytes, bool kept, hipStream_t s) {
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
  const ScanTmpLayout l = scan_tmp_layout(nb);
  const int64_t need = l.total;
  if (tmp == nullptr || tmp_bytes < need) {
    set_error("scan: tmp buffer too small (%lld < %lld bytes)", static_cast<long long>(tmp_bytes),
              static_cast<long long>(need));
    return SHMT_ENOMEM;
  }
  SHMT_REQUIRE(nb < (1ll << 31), "scan: input too large");
  SHMT_REQUIRE((reinterpret_cast<uintptr_t>(tmp) & 7) == 0, "scan: tmp must be 8-byte aligned");
  ScanState st;
  st.counter = static_cast<unsigned long long *>(tmp);
  int rc = error_word(&st.error);
  if (rc) return rc;
  st.error_mirror = error_mirror();
  st.words = (need - kScanHeaderBytes) / 8;
  st.tiles = reinterpret_cast<uint64_t *>(static_cast<char *>(tmp) + l.tiles_off);
  st.groups = reinterpret_cast<uint64_t *>(static_cast<char *>(tmp) + l.groups_off);
  st.runs = reinterpret_cast<uint64_t *>(static_cast<char *>(tmp) + l.runs_off);
  if (!kept) {
    // counter and words start at zero (a kernel, not a memset, so that the scan can be captured in a graph)
    hipLaunchKernelGGL(scan_state_clear_kernel, dim3(grid_for(need / 8, 256 * 4)), dim3(256), 0, s,
                       static_cast<uint64_t *>(tmp), need / 8);
    SHMT_LAUNCH_CHECK();
  }
  int resident = 0;
  rc = resident_workgroups(reinterpret_cast<const void *>(&scan_lookback_kernel<T, INCLUSIVE>), &resident);
  if (rc) return rc;
  const unsigned grid = static_cast<unsigned>(nb < resident ? nb : resident);
  hipLaunchKernelGGL((scan_lookback_kernel<T, INCLUSIVE>), dim3(grid), dim3(kLbBlock), 0, s,
                     data, n_head, main_data, main_len, nb, st);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

// ---- scan without a caller-provided workspace -------------------------------
// The published sums of shmt_exclusive_scan_noalloc live in this array, which
// is part of the loaded code object: every GPU the library runs on holds its
// own copy, at its own address, until the process ends. The name below is a
// host-side handle only; kernels are given the device address that
// hipGetSymbolAddress returns for the current device.
constexpr int64_t kStaticScanMaxLen = 1ll << 28;  // 268,435,456 elements
constexpr int64_t kStaticScanTiles = kStaticScanMaxLen / (kLbTileBytes / 8);
constexpr int64_t kStaticScanGroups = kStaticScanTiles / kLbFan;
constexpr int64_t kStaticScanRuns = (kStaticScanGroups + kLbFan - 1) / kLbFan;
constexpr int64_t kStaticScanWords =  // header + 256 KiB of tile words + 4 KiB of group words + 64 B of run words
    kScanHeaderBytes / 8 + 2 * (kStaticScanTiles + kStaticScanGroups + kStaticScanRuns);
static __device__ __align__(256) uint64_t scratch[kStaticScanWords];

static uint64_t *g_scratch_ptr[kMaxDevices];  // device address of `scratch`, per device ordinal

// Device address of this GPU's copy of `scratch` (looked up once per device).
static int static_scan_scratch(uint64_t **out) {
  int dev = -1;
  SHMT_HIP(hipGetDevice(&dev));
  SHMT_REQUIRE(dev >= 0 && dev < kMaxDevices, "shmt_exclusive_scan_noalloc: device ordinal %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_symbol_mutex);
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
  return scan_tmp_layout((len + tile_elems - 1) / tile_elems).total;
}

static int exclusive_scan(const char *who, void *data, int64_t len, int elem_bytes, void *tmp, int64_t tmp_bytes,
                          bool kept, void *stream) {
  SHMT_REQUIRE(len >= 0, "%s: len must be >= 0", who);
  SHMT_REQUIRE(width_ok(elem_bytes), "%s: ID can only be int32 or int64", who);
  if (len == 0) return SHMT_OK;
  SHMT_REQUIRE(data != nullptr, "%s: data is null", who);
  if (elem_bytes == 8)
    return scan_inplace<uint64_t, false>(static_cast<uint64_t *>(data), len, tmp, tmp_bytes, kept, as_stream(stream));
  return scan_inplace<uint32_t, false>(static_cast<uint32_t *>(data), len, tmp, tmp_bytes, kept, as_stream(stream));
}

int shmt_exclusive_scan(void *data, int64_t len, int elem_bytes, void *tmp, int64_t tmp_bytes,
                        void *stream) {
  return exclusive_scan("shmt_exclusive_scan", data, len, elem_bytes, tmp, tmp_bytes, false, stream);
}

int shmt_exclusive_scan_kept(void *data, int64_t len, int elem_bytes, void *kept_tmp, int64_t tmp_bytes,
                             void *stream) {
  return exclusive_scan("shmt_exclusive_scan_kept", data, len, elem_bytes, kept_tmp, tmp_bytes, true, stream);
}

int shmt_scan_workspace_clear(void *tmp, int64_t tmp_bytes, void *stream) {
  SHMT_REQUIRE(tmp_bytes >= 0 && (tmp_bytes & 7) == 0, "shmt_scan_workspace_clear: tmp_bytes must be a multiple of 8");
  if (tmp_bytes == 0) return SHMT_OK;
  SHMT_REQUIRE(tmp != nullptr && (reinterpret_cast<uintptr_t>(tmp) & 7) == 0,
               "shmt_scan_workspace_clear: tmp must be 8-byte aligned");
  hipLaunchKernelGGL(scan_state_clear_kernel, dim3(grid_for(tmp_bytes / 8, 256 * 4)), dim3(256), 0, as_stream(stream),
                     static_cast<uint64_t *>(tmp), tmp_bytes / 8);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
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
  uint32_t *err = nullptr;
  rc = error_word(&err);
  if (rc) return rc;
  if (len == 0) return SHMT_OK;
  // The workspace is zero when the library is loaded and every scan leaves it zero again, so no call
  // has anything to clear (calls that overlap on one GPU share the array and race).
  const int64_t tmp_bytes = kStaticScanWords * static_cast<int64_t>(sizeof(uint64_t));
  return exclusive_scan("shmt_exclusive_scan_noalloc", data, len, elem_bytes, partials, tmp_bytes, true, stream);
}

int shmt_inclusive_scan_i32(void *data, int64_t len, void *tmp, int64_t tmp_bytes, void *stream) {
  SHMT_REQUIRE(len >= 0, "shmt_inclusive_scan_i32: len must be >= 0");
  if (len == 0) return SHMT_OK;
  SHMT_REQUIRE(data != nullptr, "shmt_inclusive_scan_i32: data is null");
  return scan_inplace<uint32_t, true>(static_cast<uint32_t *>(data), len, tmp, tmp_bytes, false,
                                      as_stream(stream));
}

int shmt_inclusive_scan_i32_kept(void *data, int64_t len, void *kept_tmp, int64_t tmp_bytes, void *stream) {
  SHMT_REQUIRE(len >= 0, "shmt_inclusive_scan_i32_kept: len must be >= 0");
  if (len == 0) return SHMT_OK;
  SHMT_REQUIRE(data != nullptr, "shmt_inclusive_scan_i32_kept: data is null");
  return scan_inplace<uint32_t, true>(static_cast<uint32_t *>(data), len, kept_tmp, tmp_bytes, true,
                                      as_stream(stream));
}

int shmt_async_error(int *code_out) {
  SHMT_REQUIRE(code_out != nullptr, "shmt_async_error: code_out is null");
  *code_out = 0;
  uint32_t *err = nullptr;
  int rc = error_word(&err);
  if (rc) return rc;
  uint32_t seen = 0;
  SHMT_HIP(hipMemcpy(&seen, err, sizeof(seen), hipMemcpyDeviceToHost));  // waits for the device's queued work
  if (seen != 0) {
    const uint32_t zero = 0;
    SHMT_HIP(hipMemcpy(err, &zero, sizeof(zero), hipMemcpyHostToDevice));
    int dev = -1;
    SHMT_HIP(hipGetDevice(&dev));
    {
      std::lock_guard<std::mutex> lock(g_symbol_mutex);
      if (dev >= 0 && dev < kMaxDevices && g_mirror_host[dev]) *g_mirror_host[dev] = 0;
    }
    set_error("a kernel gave up a bounded wait for another workgroup (error bits 0x%x): %s", seen,
              (seen & kErrScanWait) ? "the look-back of a device-wide scan; the scanned array is incomplete" : "unknown");
  }
  *code_out = static_cast<int>(seen);
  return SHMT_OK;
}

int shmt_async_error_inject(int bits) {
  uint32_t *err = nullptr;
  int rc = error_word(&err);
  if (rc) return rc;
  uint32_t seen = 0;
  SHMT_HIP(hipMemcpy(&seen, err, sizeof(seen), hipMemcpyDeviceToHost));
  seen |= static_cast<uint32_t>(bits);
  SHMT_HIP(hipMemcpy(err, &seen, sizeof(seen), hipMemcpyHostToDevice));
  int dev = -1;
  SHMT_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_symbol_mutex);
  if (bits != 0 && dev >= 0 && dev < kMaxDevices && g_mirror_host[dev]) *g_mirror_host[dev] = seen;
  return SHMT_OK;
}

int shmt_async_error_mirror(void *host_word, void *device_alias) {
  SHMT_REQUIRE((host_word == nullptr) == (device_alias == nullptr),
               "shmt_async_error_mirror: pass both addresses of the word, or null twice");
  SHMT_REQUIRE((reinterpret_cast<uintptr_t>(host_word) & 3) == 0 && (reinterpret_cast<uintptr_t>(device_alias) & 3) == 0,
               "shmt_async_error_mirror: the word must be 4-byte aligned");
  int dev = -1;
  SHMT_HIP(hipGetDevice(&dev));
  SHMT_REQUIRE(dev >= 0 && dev < kMaxDevices, "shmt_async_error_mirror: device ordinal %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_symbol_mutex);
  g_mirror_host[dev] = static_cast<volatile uint32_t *>(host_word);
  g_mirror_dev[dev] = static_cast<uint32_t *>(device_alias);
  if (host_word) *g_mirror_host[dev] = 0;
  return SHMT_OK;
}

}  // extern "C"
