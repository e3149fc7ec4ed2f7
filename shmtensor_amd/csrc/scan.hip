// Device-wide in-place prefix sums over 4- or 8-byte integers.
// Replaces cub::DeviceScan::ExclusiveSum as used by cub_exclusiveSum
// (src/tensor_relabel.cu:11-26, src/cache_graph_sampling.cu:30-45 in the
// ShmTensor tree) and the exported thrust_scan (src/thrust_scan.cu:9-18).
//
// Wave level: DPP row shifts + row broadcasts (wave.h). Workgroup level: one
// LDS word per wave. Device level: inputs up to kSingleBlockMax elements are
// scanned by one 1024-thread workgroup that walks the array with a running
// carry (one launch); larger inputs use reduce -> scan-of-partials -> apply,
// three launches with no inter-workgroup waiting.
#include <mutex>

#include "common.h"
#include "launchers.h"
#include "scan_dev.h"

namespace shmt {

constexpr int kScanBlock = 256;
constexpr int kScanItems = 8;
constexpr int kScanTile = kScanBlock * kScanItems;  // 2048 elements per workgroup
constexpr int64_t kSingleBlockMax = 1 << 16;

// Per-tile sums (as 64-bit; 32-bit scans only use the low half, which is the
// wraparound sum).
template <typename T>
__global__ __launch_bounds__(kScanBlock) void scan_reduce_kernel(const T *data, int64_t len,
                                                                 uint64_t *partials) {
  __shared__ uint64_t lds[kScanBlock / kWave];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kScanTile;
  uint64_t s = 0;
#pragma unroll
  for (int j = 0; j < kScanItems; ++j) {
    int64_t i = base + j * kScanBlock + threadIdx.x;
    if (i < len) s += static_cast<uint64_t>(data[i]);
  }
  uint64_t total;
  block_exclusive_scan<uint64_t, kScanBlock>(s, lds, &total);
  if (threadIdx.x == 0) partials[blockIdx.x] = total;
}

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

template <typename T, bool INCLUSIVE>
__global__ __launch_bounds__(kScanBlock) void scan_apply_kernel(T *data, int64_t len,
                                                                const uint64_t *partials) {
  __shared__ T lds[kScanBlock / kWave];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kScanTile;
  T carry = static_cast<T>(partials[blockIdx.x]);
  tile_scan_inplace<T, kScanBlock, kScanItems, INCLUSIVE>(data, base, len, lds, &carry);
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
  const int64_t nb = (len + kScanTile - 1) / kScanTile;
  if (tmp == nullptr || tmp_bytes < nb * static_cast<int64_t>(sizeof(uint64_t))) {
    set_error("scan: tmp buffer too small (%lld < %lld bytes)", static_cast<long long>(tmp_bytes),
              static_cast<long long>(nb * sizeof(uint64_t)));
    return SHMT_ENOMEM;
  }
  SHMT_REQUIRE(nb < (1ll << 31), "scan: input too large");
  uint64_t *partials = static_cast<uint64_t *>(tmp);
  hipLaunchKernelGGL((scan_reduce_kernel<T>), dim3(static_cast<unsigned>(nb)), dim3(kScanBlock), 0,
                     s, data, len, partials);
  SHMT_LAUNCH_CHECK();
  int rc = launch_scan_partials(partials, nb, s);
  if (rc) return rc;
  hipLaunchKernelGGL((scan_apply_kernel<T, INCLUSIVE>), dim3(static_cast<unsigned>(nb)),
                     dim3(kScanBlock), 0, s, data, len, partials);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

// ---- scan without a caller-provided workspace -------------------------------
// The tile partials of shmt_exclusive_scan_noalloc live in this array, which
// is part of the loaded code object: every GPU the library runs on holds its
// own copy, at its own address, until the process ends. The name below is a
// host-side handle only; kernels are given the device address that
// hipGetSymbolAddress returns for the current device.
constexpr int64_t kStaticScanPartials = 1 << 17;                       // 1 MiB
constexpr int64_t kStaticScanMaxLen = kStaticScanPartials * kScanTile;  // 268,435,456 elements
static __device__ __align__(256) uint64_t scratch[kStaticScanPartials];

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
  return ((len + kScanTile - 1) / kScanTile) * static_cast<int64_t>(sizeof(uint64_t));
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
  // Every partial a launch reads was written by the reduce kernel of the same
  // call, so nothing in the workspace needs clearing between calls.
  const int64_t tmp_bytes = kStaticScanPartials * static_cast<int64_t>(sizeof(uint64_t));
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
