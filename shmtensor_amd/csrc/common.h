// Host-side helpers shared by every translation unit of libshmt.so:
// the thread-local error channel and argument/HIP-status checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "shmt.h"

namespace shmt {

// printf-style; stores the message returned by shmt_last_error().
void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

inline bool width_ok(int bytes) { return bytes == 4 || bytes == 8; }

// Grid size for a grid-stride kernel: enough workgroups to cover `work_items`
// at `items_per_block`, capped at a few resident workgroups per CU of the
// 256-CU part so large inputs loop instead of over-launching.
inline unsigned grid_for(int64_t work_items, int64_t items_per_block,
                         int64_t max_blocks = 256 * 16) {
  int64_t b = (work_items + items_per_block - 1) / items_per_block;
  if (b < 1) b = 1;
  if (b > max_blocks) b = max_blocks;
  return static_cast<unsigned>(b);
}

}  // namespace shmt

#define SHMT_REQUIRE(cond, ...)      \
  do {                               \
    if (!(cond)) {                   \
      shmt::set_error(__VA_ARGS__);  \
      return SHMT_EINVAL;            \
    }                                \
  } while (0)

#define SHMT_HIP(call)                                                     \
  do {                                                                     \
    hipError_t e_ = (call);                                                \
    if (e_ != hipSuccess) {                                                \
      shmt::set_error("%s:%d: %s failed: %s", __FILE__, __LINE__, #call,   \
                      hipGetErrorString(e_));                              \
      return SHMT_EHIP;                                                    \
    }                                                                      \
  } while (0)

// After a kernel launch: report a launch failure without synchronising.
#define SHMT_LAUNCH_CHECK() SHMT_HIP(hipGetLastError())
