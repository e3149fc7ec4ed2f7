// Workgroup-level tile scan shared by the scan entry points and by kernels
// that fuse a prefix sum with their own work (sampling plan, relabel).
#pragma once
#include "wave.h"

namespace shmt {

// In-place prefix sum of data[base .. base + BLOCK*ITEMS) clipped to len, by
// one workgroup. Thread t owns ITEMS consecutive elements. *carry is the sum
// of everything before `base` on entry and is advanced by the tile total on
// exit (same value in every thread). Contains barriers: call from all threads.
template <typename T, int BLOCK, int ITEMS, bool INCLUSIVE>
__device__ __forceinline__ void tile_scan_inplace(T *data, int64_t base, int64_t len, T *lds,
                                                  T *carry) {
  T v[ITEMS];
  const int64_t first = base + static_cast<int64_t>(threadIdx.x) * ITEMS;
  T sum = 0;
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    v[j] = (first + j < len) ? data[first + j] : static_cast<T>(0);
    sum += v[j];
  }
  T total;
  T run = *carry + block_exclusive_scan<T, BLOCK>(sum, lds, &total);
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    if (INCLUSIVE) run += v[j];
    if (first + j < len) data[first + j] = run;
    if (!INCLUSIVE) run += v[j];
  }
  *carry += total;
}

}  // namespace shmt
