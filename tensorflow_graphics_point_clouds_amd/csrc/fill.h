// Device-memory helpers shared by the op files (defined in util.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace mccnn {

// Zeroes `bytes` bytes (a multiple of 4) at `ptr` (4-byte aligned) with a fill
// kernel rather than hipMemsetAsync, so that callers may capture the stream
// into a graph.
int fill_zero(hipStream_t stream, void *ptr, size_t bytes);

// In-place scan of counts[0..n): on return counts[i] holds the INCLUSIVE prefix
// sum (the end offset of segment i) and *total_dev the grand total (int64).
// block_sums is scratch for scan_scratch_ints(n) ints.
size_t scan_scratch_ints(int64_t n);
int inclusive_scan_i32(hipStream_t stream, int64_t n, int *counts, int *block_sums,
                       int64_t *total_dev);

}  // namespace mccnn
