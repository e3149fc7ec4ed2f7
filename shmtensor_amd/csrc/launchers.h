// Small launch helpers shared between translation units of libshmt.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace shmt {

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
int relabel_table(int64_t N, bool n_is_loose_bound, void *scratch, int64_t scratch_bytes, RelabelTable *out);
int launch_relabel_passes(const void *total, int64_t n_bound, int64_t n_fixed, const int64_t *n_fixed_dev,
                          const void *n_extra_dev, int n_extra_bytes, int elem_bytes, void *scratch,
                          int64_t scratch_bytes, void *unique_out, void *labels_out, int64_t *count_out,
                          int64_t *count_copy, const RelabelTable &table, hipStream_t stream);
uint64_t relabel_nonce();

}  // namespace shmt
