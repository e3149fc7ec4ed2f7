// Fill kernel used to initialise hash tables (all-ones = every slot empty).
// A kernel rather than hipMemsetAsync so that callers may capture the build
// into a HIP graph.
#include "common.h"
#include "launchers.h"

namespace shmt {

__global__ __launch_bounds__(256) void fill_ones_kernel(uint4 *p, int64_t n16) {
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const uint4 ones = make_uint4(~0u, ~0u, ~0u, ~0u);
  for (; i < n16; i += stride) p[i] = ones;
}

int launch_fill_ones(void *p, int64_t n16, hipStream_t s) {
  if (n16 <= 0) return SHMT_OK;
  hipLaunchKernelGGL(fill_ones_kernel, dim3(grid_for(n16, 256 * 4)), dim3(256), 0, s,
                     static_cast<uint4 *>(p), n16);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

}  // namespace shmt
