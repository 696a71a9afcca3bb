// Error reporting, fill and prefix-sum helpers of libmccnn_hip.so.
#include <stdarg.h>

#include "common.h"
#include "fill.h"

namespace mccnn {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

__global__ void __launch_bounds__(256) fill_zero_kernel(uint32_t *p, size_t words) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < words;
       i += (size_t)gridDim.x * blockDim.x)
    p[i] = 0u;
}

int fill_zero(hipStream_t stream, void *ptr, size_t bytes) {
  if (bytes == 0) return MCCNN_OK;
  size_t words = bytes / 4;
  unsigned grid = (unsigned)((words + 1023) / 1024);
  if (grid > 65535u * 4) grid = 65535u * 4;
  if (grid < 1) grid = 1;
  hipLaunchKernelGGL(fill_zero_kernel, dim3(grid), dim3(256), 0, stream, (uint32_t *)ptr, words);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

// ------------------------------------------------------------ prefix sum ----
// Long inputs take three launches, no inter-block waiting: (1) each block of kScanTile items
// writes its sum, (2) one block scans the block sums, (3) each block rescans its
// tile with the carried-in offset.  The scanned values are int32 (pair counts are
// int32 in the op contract); tile sums and the grand total are formed in 64 bits
// and a tile sum that does not fit saturates, so that a total of 2^31 - 1 or more
// is always reported as at least 2^31 - 1 and the callers can refuse it instead
// of working on wrapped offsets.

constexpr int kScanThreads = 256;
constexpr int kScanItems = 8;
constexpr int kScanTile = kScanThreads * kScanItems;

size_t scan_scratch_ints(int64_t n) { return (size_t)((n + kScanTile - 1) / kScanTile) + 1; }

__device__ __forceinline__ int block_exclusive_scan(int v, int *total) {
  __shared__ int wave_sums[kScanThreads / kWave];
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  const int incl = wave_inclusive_scan(v);
  if (lane == kWave - 1) wave_sums[wave] = incl;
  __syncthreads();
  int carry = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < kScanThreads / kWave; ++w) {
    if (w < wave) carry += wave_sums[w];
    sum += wave_sums[w];
  }
  __syncthreads();
  *total = sum;
  return carry + incl - v;
}

constexpr long long kScanMax = 0x7fffffffLL;

__device__ __forceinline__ int saturate_i32(long long v) {
  return (int)(v > kScanMax ? kScanMax : v);
}

// 64-bit counterpart of block_exclusive_scan for the sums of whole tiles.
template <int kThreads = kScanThreads>
__device__ __forceinline__ long long block_exclusive_scan_i64(long long v, long long *total) {
  __shared__ long long wave_sums[kThreads / kWave];
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  long long incl = v;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const long long t = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += t;
  }
  if (lane == kWave - 1) wave_sums[wave] = incl;
  __syncthreads();
  long long carry = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < kThreads / kWave; ++w) {
    if (w < wave) carry += wave_sums[w];
    sum += wave_sums[w];
  }
  __syncthreads();
  *total = sum;
  return carry + incl - v;
}

__global__ void __launch_bounds__(kScanThreads) scan_tile_sums_kernel(
    int64_t n, const int *__restrict__ counts, int *__restrict__ block_sums) {
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  long long s = 0;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k)
    if (base + k < n) s += counts[base + k];
  long long total;
  block_exclusive_scan_i64(s, &total);
  if (threadIdx.x == 0) block_sums[blockIdx.x] = saturate_i32(total);
}

// Single block: exclusive scan of block_sums[0..nb) in place, total to *total_dev.
__global__ void __launch_bounds__(kScanThreads) scan_block_sums_kernel(int nb, int *block_sums,
                                                                       int64_t *total_dev) {
  long long carry = 0;
  for (int base = 0; base < nb; base += kScanThreads) {
    const int i = base + threadIdx.x;
    const long long v = i < nb ? block_sums[i] : 0;
    long long total;
    const long long ex = block_exclusive_scan_i64(v, &total);
    if (i < nb) block_sums[i] = saturate_i32(carry + ex);
    carry += total;
  }
  if (threadIdx.x == 0) *total_dev = carry;
}

__global__ void __launch_bounds__(kScanThreads) scan_apply_kernel(
    int64_t n, int *__restrict__ counts, const int *__restrict__ block_sums) {
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  int v[kScanItems];
  int s = 0;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) {
    v[k] = base + k < n ? counts[base + k] : 0;
    s += v[k];
  }
  int total;
  int run = block_exclusive_scan(s, &total) + block_sums[blockIdx.x];
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) {
    run += v[k];
    if (base + k < n) counts[base + k] = run;
  }
}

// Short inputs: one block walks the tiles in order and carries the running total,
// one launch instead of three (small clouds are bound by launches, not by bytes).
constexpr int kScanSingleThreads = 1024;
constexpr int kScanSingleTile = kScanSingleThreads * kScanItems;
constexpr int64_t kScanSingleBlockMax = 4 * kScanSingleTile;

__global__ void __launch_bounds__(kScanSingleThreads) scan_single_block_kernel(
    int64_t n, int *counts, int64_t *total_dev) {
  long long carry = 0;
  for (int64_t tile = 0; tile < n; tile += kScanSingleTile) {
    const int64_t base = tile + (int64_t)threadIdx.x * kScanItems;
    int v[kScanItems];
    long long s = 0;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
      v[k] = base + k < n ? counts[base + k] : 0;
      s += v[k];
    }
    long long total;
    long long run = carry + block_exclusive_scan_i64<kScanSingleThreads>(s, &total);
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
      run += v[k];
      if (base + k < n) counts[base + k] = saturate_i32(run);
    }
    carry += total;
  }
  if (threadIdx.x == 0) *total_dev = carry;
}

int inclusive_scan_i32(hipStream_t stream, int64_t n, int *counts, int *block_sums,
                       int64_t *total_dev) {
  const int nb = (int)((n + kScanTile - 1) / kScanTile);
  if (nb == 0) {
    return fill_zero(stream, total_dev, sizeof(int64_t));
  }
  if (n <= kScanSingleBlockMax) {
    hipLaunchKernelGGL(scan_single_block_kernel, dim3(1), dim3(kScanSingleThreads), 0, stream, n,
                       counts, total_dev);
    MCCNN_LAUNCH_CHECK();
    return MCCNN_OK;
  }
  hipLaunchKernelGGL(scan_tile_sums_kernel, dim3(nb), dim3(kScanThreads), 0, stream, n, counts,
                     block_sums);
  MCCNN_LAUNCH_CHECK();
  hipLaunchKernelGGL(scan_block_sums_kernel, dim3(1), dim3(kScanThreads), 0, stream, nb,
                     block_sums, total_dev);
  MCCNN_LAUNCH_CHECK();
  hipLaunchKernelGGL(scan_apply_kernel, dim3(nb), dim3(kScanThreads), 0, stream, n, counts,
                     block_sums);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

}  // namespace mccnn

extern "C" const char *mccnn_last_error(void) { return mccnn::g_error; }
extern "C" int mccnn_abi_version(void) { return 1; }
