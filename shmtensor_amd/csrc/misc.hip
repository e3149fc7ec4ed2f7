// Fill kernel used to initialise hash tables (all-ones = every slot empty).
// A kernel rather than hipMemsetAsync so that callers may capture the build
// into a HIP graph. Also: the staging kernel and the capture / replay
// wrappers with which a caller turns a queued launch sequence (a mini-batch
// of chained hops) into a HIP graph and feeds it new inputs.
#include "common.h"
#include "launchers.h"
#include "wave.h"

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

namespace shmt {

// Copies the seeds of a mini-batch into the fixed input buffer of a captured
// launch sequence and stores their number and the batch's RNG seed where the
// captured kernels read them.
__global__ __launch_bounds__(256) void stage_seeds_kernel(const void *src, int src_bytes, int64_t n,
                                                          void *dst, int dst_bytes, int64_t *len_dst,
                                                          uint64_t rng_seed, uint64_t *rng_dst) {
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  if (i == 0) {
    *len_dst = n;
    if (rng_dst) *rng_dst = rng_seed;
  }
  for (; i < n; i += stride) store_int(dst, i, dst_bytes, load_int(src, i, src_bytes));
}

}  // namespace shmt

namespace shmt {

// One wave that stays busy for about `ticks` of the 100 MHz wall clock (and at
// most `max_sleeps` sleep instructions, so it ends whatever the clock does).
__global__ __launch_bounds__(64) void busy_wait_kernel(unsigned long long ticks, int max_sleeps) {
  const unsigned long long t0 = wall_clock64();
  for (int i = 0; i < max_sleeps && wall_clock64() - t0 < ticks; ++i) __builtin_amdgcn_s_sleep(64);
}

}  // namespace shmt

using namespace shmt;

extern "C" {

int shmt_busy_wait(void *stream, int microseconds) {
  SHMT_REQUIRE(microseconds >= 0 && microseconds <= 100000, "shmt_busy_wait: 0 .. 100,000 microseconds");
  hipLaunchKernelGGL(busy_wait_kernel, dim3(1), dim3(64), 0, as_stream(stream),
                     static_cast<unsigned long long>(microseconds) * 100ull, microseconds + 16);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

int shmt_stage_seeds(const void *seeds, int seed_bytes, int64_t n, void *staged, int staged_bytes,
                     int64_t *len_out, uint64_t rng_seed, uint64_t *rng_seed_out, void *stream) {
  SHMT_REQUIRE(n >= 0, "shmt_stage_seeds: n must be >= 0");
  SHMT_REQUIRE(width_ok(seed_bytes) && width_ok(staged_bytes) && staged_bytes >= seed_bytes,
               "shmt_stage_seeds: widths must be 4 or 8 and the staged ids not narrower than the seeds");
  SHMT_REQUIRE(len_out != nullptr, "shmt_stage_seeds: len_out is null");
  SHMT_REQUIRE(n == 0 || (seeds != nullptr && staged != nullptr), "shmt_stage_seeds: null buffer");
  hipLaunchKernelGGL(stage_seeds_kernel, dim3(grid_for(n, 256, 1024)), dim3(256), 0, as_stream(stream), seeds,
                     seed_bytes, n, staged, staged_bytes, len_out, rng_seed, rng_seed_out);
  SHMT_LAUNCH_CHECK();
  return SHMT_OK;
}

int shmt_capture_begin(void *stream) {
  SHMT_REQUIRE(stream != nullptr, "shmt_capture_begin: the null stream cannot be captured");
  SHMT_HIP(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal));
  return SHMT_OK;
}

int shmt_capture_end(void *stream, void **graph_exec_out) {
  SHMT_REQUIRE(graph_exec_out != nullptr, "shmt_capture_end: graph_exec_out is null");
  *graph_exec_out = nullptr;
  hipGraph_t graph = nullptr;
  SHMT_HIP(hipStreamEndCapture(as_stream(stream), &graph));
  hipGraphExec_t exec = nullptr;
  const hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (e != hipSuccess) {
    set_error("shmt_capture_end: hipGraphInstantiate failed: %s", hipGetErrorString(e));
    return SHMT_EHIP;
  }
  *graph_exec_out = exec;
  return SHMT_OK;
}

int shmt_graph_launch(void *graph_exec, void *stream) {
  SHMT_REQUIRE(graph_exec != nullptr, "shmt_graph_launch: graph_exec is null");
  SHMT_HIP(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), as_stream(stream)));
  return SHMT_OK;
}

void shmt_graph_destroy(void *graph_exec) {
  if (graph_exec) (void)hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec));
}

}  // extern "C"
