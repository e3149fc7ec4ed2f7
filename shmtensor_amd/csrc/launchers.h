// Small launch helpers shared between translation units of libshmt.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string.h>

namespace shmt {

// ---- merged launches ----------------------------------------------------------
// Several independent jobs that run the same kernel sequence (the hops of
// several mini-batches) can share their launches: instead of being issued, a
// job's launches are recorded as stages, and stage i of all jobs then goes out
// as ONE launch whose blockIdx.y selects the job. The kernels are the same
// device code either way; a sequence that contains a launch without a merged
// form is marked so and the caller issues the jobs one by one instead.
constexpr int kMaxJobs = 8;
constexpr int kStageArgBytes = 256;
constexpr int kMaxStages = 12;

enum StageKind : int {
  kStagePlanSingle = 0,  // + map mode (0: no cache, 1: wide map, 2: narrow map)
  kStagePlanTile = 3,    // + map mode
  kStagePickNarrowHop = 6,  // + log2(lanes per seed) - 2, i.e. 6 .. 10
  kStageRlSmall = 11,
  kStageRlInsert = 12,
  kStageRlFirst = 13,
  kStageRlUnique = 14,
  kStageRlLabels = 15,
  kStageRpCount = 16,
  kStageRpRows = 17,
  kStageRpScatter = 18,
  kStageRpGather = 19,
  kStageRpBins = 20,  // + (largest table - this launch's table), log2 of the slots: 20 .. 22
};

struct Stage {
  int kind;
  unsigned blocks, threads;
  alignas(16) unsigned char args[kStageArgBytes];
};

struct StageList {
  int n = 0;
  int jobs = 1;  // how many jobs the caller means to merge (a job may choose its kernels by it)
  bool mergeable = true;
  Stage stage[kMaxStages];
};

// Where a launch goes: to the stream at once, or (defer != nullptr) into a stage list.
struct Launcher {
  hipStream_t stream;
  StageList *defer;
};

template <typename Args>
inline void stage_push(StageList *list, int kind, unsigned blocks, unsigned threads, const Args &a) {
  static_assert(sizeof(Args) <= kStageArgBytes, "kernel arguments do not fit a stage record");
  if (list->n >= kMaxStages) {
    list->mergeable = false;
    return;
  }
  Stage &s = list->stage[list->n++];
  s.kind = kind;
  s.blocks = blocks;
  s.threads = threads;
  memcpy(s.args, &a, sizeof(Args));
}

// Arguments of `n_jobs` recorded launches of one kernel, as the merged kernel takes them.
template <typename Args>
struct Jobs {
  Args a[kMaxJobs];
  unsigned blocks[kMaxJobs];
};

template <typename Args>
inline unsigned jobs_from_stages(int n_jobs, const Stage *const *stages, Jobs<Args> *out) {
  unsigned max_blocks = 1;
  for (int j = 0; j < kMaxJobs; ++j) {
    const Stage *s = stages[j < n_jobs ? j : 0];
    memcpy(&out->a[j], s->args, sizeof(Args));
    out->blocks[j] = j < n_jobs ? s->blocks : 0;
    if (j < n_jobs && s->blocks > max_blocks) max_blocks = s->blocks;
  }
  return max_blocks;
}

// One merged launch for stage `stages[j]` of jobs j < n_jobs (all of the same kind and block size).
int launch_merged_sampling_stage(int n_jobs, const Stage *const *stages, hipStream_t s);  // sample.hip
int launch_merged_relabel_stage(int n_jobs, const Stage *const *stages, hipStream_t s);   // relabel.hip

// Set n16 consecutive 16-byte words at p (16-byte aligned) to all-ones, i.e.
// every integer field to -1 / its unsigned maximum.
int launch_fill_ones(void *p, int64_t n16, hipStream_t s);

// In-place exclusive scan of nb 64-bit tile totals by one workgroup.
int launch_scan_partials(uint64_t *partials, int64_t nb, hipStream_t s);

// Relabel as the tail of a fused launch sequence. relabel_table() names the
// hash-table part of a relabel scratch buffer sized for N ids (n16 16-byte
// words that must be all ones when the passes start); launch_relabel_passes()
// runs insert -> first -> unique -> labels on `total`, which earlier kernels of
// the same stream have filled, for n_fixed + *n_extra_dev ids (at most n_bound;
// with n_fixed_dev the first part is min(*n_fixed_dev, n_fixed), read on the
// device); those kernels must also have stored `nonce` to *wide_mark if any id
// lies outside [0, 2^32). n16 is 0 when the passes need no table in memory
// (small inputs). count_copy, if set, receives the count as well (device memory).
struct RelabelTable {
  void *slots;
  int64_t n16;
  uint64_t *wide_mark;  // where the earlier kernels store `nonce` when an id lies outside [0, 2^32)
  uint64_t nonce;
};
int relabel_table(int64_t N, bool n_is_loose_bound, int merged_jobs, void *scratch, int64_t scratch_bytes,
                  RelabelTable *out);  // merged_jobs: 0 for a launch sequence of its own
int launch_relabel_passes(const void *total, int64_t n_bound, int64_t n_fixed, const int64_t *n_fixed_dev,
                          const void *n_extra_dev, int n_extra_bytes, int elem_bytes, void *scratch,
                          int64_t scratch_bytes, void *unique_out, void *labels_out, int64_t *count_out,
                          int64_t *count_copy, const RelabelTable &table, Launcher launcher);
uint64_t relabel_nonce();

}  // namespace shmt
