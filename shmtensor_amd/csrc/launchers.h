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

}  // namespace shmt
