// Stable descending radix sort of (cell key, point index) pairs: the sort step
// of the reference's grid construction (pylib/pc/Grid.py:56-64,
// tf.argsort(keys, 'DESCENDING'): equal keys keep ascending original index).
//
// LSD radix sort, 8-bit digits, on the complemented digit so that ascending
// digit order is descending key order while stability keeps equal keys in input
// order.  Per pass: (1) per-tile digit histogram in LDS, written digit-major,
// (2) prefix sum over [256 digits x tiles], (3) stable scatter: ranks inside a
// tile come from wavefront ballots (matching lanes with the same digit) plus
// per-wave LDS counters, never from atomics, so the order is deterministic.
#include "common.h"
#include "fill.h"

namespace mccnn {

constexpr int kSortThreads = 256;
constexpr int kSortItems = 8;
constexpr int kSortTile = kSortThreads * kSortItems;
constexpr int kSortWaves = kSortThreads / kWave;
constexpr int kRadix = 256;

__device__ __forceinline__ int digit_of(int64_t key, int shift) {
  return (int)((~(uint64_t)key >> shift) & (kRadix - 1));
}

__global__ void __launch_bounds__(kSortThreads) sort_hist_kernel(
    int64_t n, int shift, int nb, const int64_t *__restrict__ keys, int *__restrict__ hist) {
  __shared__ int bins[kRadix];
  bins[threadIdx.x] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kSortTile;
#pragma unroll
  for (int k = 0; k < kSortItems; ++k) {
    const int64_t i = base + k * kSortThreads + threadIdx.x;
    if (i < n) atomicAdd(&bins[digit_of(keys[i], shift)], 1);
  }
  __syncthreads();
  hist[(int64_t)threadIdx.x * nb + blockIdx.x] = bins[threadIdx.x];
}

// hist holds the INCLUSIVE prefix sums of the digit-major histogram.
template <bool kFirstPass>
__global__ void __launch_bounds__(kSortThreads) sort_scatter_kernel(
    int64_t n, int shift, int nb, const int64_t *__restrict__ keys_in,
    const int *__restrict__ idx_in, const int *__restrict__ hist,
    int64_t *__restrict__ keys_out, int *__restrict__ idx_out) {
  __shared__ int running[kRadix];              // items of each digit seen in earlier rounds
  __shared__ int wcount[kSortWaves][kRadix];   // per wave, this round
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  running[threadIdx.x] = 0;
#pragma unroll
  for (int w = 0; w < kSortWaves; ++w) wcount[w][threadIdx.x] = 0;
  __syncthreads();

  const int64_t base = (int64_t)blockIdx.x * kSortTile;
  int64_t key[kSortItems];
  int rank[kSortItems];
#pragma unroll
  for (int k = 0; k < kSortItems; ++k) {
    const int64_t i = base + k * kSortThreads + threadIdx.x;
    const bool live = i < n;
    key[k] = live ? keys_in[i] : 0;
    const int d = digit_of(key[k], shift);
    // lanes of this wave holding the same digit (dead lanes match nothing)
    uint64_t same = __ballot(live);
#pragma unroll
    for (int bit = 0; bit < 8; ++bit) {
      const uint64_t b = __ballot((d >> bit) & 1);
      same &= ((d >> bit) & 1) ? b : ~b;
    }
    const int below = __popcll(same & ((1ull << lane) - 1ull));
    if (live && below == 0) wcount[wave][d] = __popcll(same);
    __syncthreads();
    int r = running[d] + below;
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w)
      if (w < wave) r += wcount[w][d];
    rank[k] = r;
    __syncthreads();
    {
      int add = 0;
#pragma unroll
      for (int w = 0; w < kSortWaves; ++w) {
        add += wcount[w][threadIdx.x];
        wcount[w][threadIdx.x] = 0;
      }
      running[threadIdx.x] += add;
    }
    __syncthreads();
  }
  // running[d] is now this tile's count of digit d: global start of the tile's
  // run of digit d = inclusive prefix - count.
  const int start = hist[(int64_t)threadIdx.x * nb + blockIdx.x] - running[threadIdx.x];
  __syncthreads();
  running[threadIdx.x] = start;
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kSortItems; ++k) {
    const int64_t i = base + k * kSortThreads + threadIdx.x;
    if (i < n) {
      const int d = digit_of(key[k], shift);
      const int64_t dst = (int64_t)running[d] + rank[k];
      keys_out[dst] = key[k];
      idx_out[dst] = kFirstPass ? (int)i : idx_in[i];
    }
  }
}

// The whole sort in one launch for small inputs (a cloud of a few thousand points: the
// multi-block passes above cost five launches each, 36 us for three passes of 16 k keys,
// nearly all of it launch latency).  One block of 16 wavefronts runs every pass; wavefront
// w owns the w-th sixteenth of the input, fetched into registers at the start of the pass.
// Counting sweep: digit counts per wavefront with LDS atomics (counts do not depend on the
// order).  Then 256 threads turn the [digit][wavefront] counts into start positions
// (digits ascending, wavefronts ascending inside a digit).  Ranking sweep, without block
// barriers: the wavefront walks its keys in rounds of 64 in input order, a lane's rank among
// the lanes with its digit comes from ballots, the first such lane advances the
// wavefront's start for the digit.  Same stable order as above.  The passes ping-pong
// between two global buffers, which one block keeps coherent with its barriers.
constexpr int kSmallSortThreads = 1024;
constexpr int kSmallSortWaves = kSmallSortThreads / kWave;
constexpr int kSmallSortRounds = 16;                 // keys per lane
constexpr int64_t kSmallSortMax = (int64_t)kSmallSortThreads * kSmallSortRounds;

__global__ void __launch_bounds__(kSmallSortThreads) sort_small_kernel(
    int n, int passes, const int64_t *__restrict__ keys, int64_t *kbuf0, int *ibuf0,
    int64_t *kbuf1, int *ibuf1) {
  __shared__ int start[kSmallSortWaves][kRadix];     // counts, then next free positions
  __shared__ int scan[kRadix];
  const int t = threadIdx.x, lane = lane_id(), wave = t / kWave;
  // the wavefront's chunk: a multiple of 64 keys, so that rounds are whole except the last
  const int per_wave = ((n + kSmallSortWaves - 1) / kSmallSortWaves + kWave - 1) / kWave * kWave;
  const int first = wave * per_wave;
  const int last = first + per_wave < n ? first + per_wave : n;
  const int64_t *kin = keys;
  const int *iin = nullptr;
  for (int p = 0; p < passes; ++p) {
    const int shift = 8 * p;
    int64_t *kout = (p & 1) ? kbuf1 : kbuf0;
    int *iout = (p & 1) ? ibuf1 : ibuf0;
    int64_t key[kSmallSortRounds];
    int idx[kSmallSortRounds];
#pragma unroll
    for (int r = 0; r < kSmallSortRounds; ++r) {
      const int i = first + r * kWave + lane;
      key[r] = i < last ? kin[i] : 0;
      idx[r] = i < last ? (p == 0 ? i : iin[i]) : 0;
    }
    if (t < kRadix) {
#pragma unroll
      for (int w = 0; w < kSmallSortWaves; ++w) start[w][t] = 0;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSmallSortRounds; ++r)
      if (first + r * kWave + lane < last) atomicAdd(&start[wave][digit_of(key[r], shift)], 1);
    __syncthreads();
    // exclusive scan over (digit, wavefront): per-digit totals scanned over the digits
    // (Hillis-Steele in LDS, every thread at every barrier), then spread over the wavefronts
    int total = 0;
    if (t < kRadix) {
#pragma unroll
      for (int w = 0; w < kSmallSortWaves; ++w) total += start[w][t];
    }
    int v = total;
    for (int off = 1; off < kRadix; off <<= 1) {
      if (t < kRadix) scan[t] = v;
      __syncthreads();
      if (t < kRadix && t >= off) v += scan[t - off];
      __syncthreads();
    }
    if (t < kRadix) {
      int run = v - total;
#pragma unroll
      for (int w = 0; w < kSmallSortWaves; ++w) {
        const int c = start[w][t];
        start[w][t] = run;
        run += c;
      }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSmallSortRounds; ++r) {
      if (first + r * kWave >= last) break;              // uniform in the wavefront
      const bool live = first + r * kWave + lane < last;
      const int d = digit_of(key[r], shift);
      uint64_t same = __ballot(live);
#pragma unroll
      for (int bit = 0; bit < 8; ++bit) {
        const uint64_t b = __ballot((d >> bit) & 1);
        same &= ((d >> bit) & 1) ? b : ~b;
      }
      const int below = __popcll(same & ((1ull << lane) - 1ull));
      int dst = 0;
      if (live) dst = start[wave][d] + below;
      wave_lds_sync();                                   // every lane has read its start
      if (live && below == 0) start[wave][d] = dst + __popcll(same);
      wave_lds_sync();
      if (live) {
        kout[dst] = key[r];
        iout[dst] = idx[r];
      }
    }
    __threadfence_block();
    __syncthreads();               // the pass is in memory before the next one reads it
    kin = kout;
    iin = iout;
  }
}

// keys[m] = num_pts - 1 - neighbour id (descending key order = ascending id), and
// the number of pairs of each point.
__global__ void __launch_bounds__(256) transpose_keys_kernel(int64_t m_total, int64_t num_pts,
                                                             const int2 *__restrict__ nbrs,
                                                             int64_t *__restrict__ keys,
                                                             int *__restrict__ counts) {
  for (int64_t m = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; m < m_total;
       m += (int64_t)gridDim.x * blockDim.x) {
    const int n = nbrs[m].x;
    keys[m] = num_pts - 1 - n;
    atomicAdd(&counts[n], 1);
  }
}

struct SortWorkspace {
  int64_t *keys_tmp;
  int *idx_tmp;
  int *hist;
  int *scan_scratch;
  int64_t *total;
  size_t bytes;
};

static SortWorkspace carve_sort_workspace(void *ws, int64_t n) {
  const int64_t nb = (n + kSortTile - 1) / kSortTile;
  char *p = (char *)ws;
  SortWorkspace w;
  size_t off = 0;
  w.keys_tmp = (int64_t *)(p + off);
  off += align256(sizeof(int64_t) * (size_t)n);
  w.idx_tmp = (int *)(p + off);
  off += align256(sizeof(int) * (size_t)n);
  w.hist = (int *)(p + off);
  off += align256(sizeof(int) * (size_t)(kRadix * nb));
  w.scan_scratch = (int *)(p + off);
  off += align256(sizeof(int) * scan_scratch_ints(kRadix * nb));
  w.total = (int64_t *)(p + off);
  off += 256;
  w.bytes = off;
  return w;
}

}  // namespace mccnn

using namespace mccnn;

extern "C" size_t mccnn_sort_keys_workspace_bytes(int64_t num_pts) {
  if (num_pts < 0) num_pts = 0;
  return carve_sort_workspace(nullptr, num_pts).bytes;
}

extern "C" int mccnn_sort_keys_descending(mccnn_stream_t stream, int64_t num_pts, int key_bits,
                                          const int64_t *keys, int64_t *sorted_keys_out,
                                          int32_t *sorted_indices_out, void *workspace,
                                          size_t workspace_bytes) {
  MCCNN_REQUIRE(num_pts >= 0 && num_pts < ((int64_t)1 << 31),
                "sort_keys expects 0 <= num_pts < 2^31");
  MCCNN_REQUIRE(key_bits >= 1 && key_bits <= 64, "sort_keys expects key_bits in [1, 64]");
  if (num_pts == 0) return MCCNN_OK;
  MCCNN_REQUIRE(keys && sorted_keys_out && sorted_indices_out && workspace,
                "sort_keys received a null tensor");
  MCCNN_REQUIRE((const void *)keys != (const void *)sorted_keys_out,
                "sort_keys output must not alias the input");
  const SortWorkspace w = carve_sort_workspace(workspace, num_pts);
  MCCNN_REQUIRE(workspace_bytes >= w.bytes, "sort_keys workspace too small (%zu < %zu)",
                workspace_bytes, w.bytes);
  hipStream_t s = as_stream(stream);
  const int passes = (key_bits + 7) / 8;
  const int nb = (int)((num_pts + kSortTile - 1) / kSortTile);
  // Ping-pong so that the last pass lands in the caller's buffers.
  int64_t *kbuf[2];
  int *ibuf[2];
  if (passes % 2 == 1) {
    kbuf[0] = (int64_t *)sorted_keys_out; ibuf[0] = sorted_indices_out;
    kbuf[1] = w.keys_tmp;                 ibuf[1] = w.idx_tmp;
  } else {
    kbuf[0] = w.keys_tmp;                 ibuf[0] = w.idx_tmp;
    kbuf[1] = (int64_t *)sorted_keys_out; ibuf[1] = sorted_indices_out;
  }
  if (num_pts <= kSmallSortMax) {
    hipLaunchKernelGGL(sort_small_kernel, dim3(1), dim3(kSmallSortThreads), 0, s, (int)num_pts,
                       passes, (const int64_t *)keys, kbuf[0], ibuf[0], kbuf[1], ibuf[1]);
    MCCNN_LAUNCH_CHECK();
    return MCCNN_OK;
  }
  const int64_t *kin = (const int64_t *)keys;
  const int *iin = nullptr;
  for (int p = 0; p < passes; ++p) {
    const int shift = 8 * p;
    int64_t *kout = kbuf[p & 1];
    int *iout = ibuf[p & 1];
    hipLaunchKernelGGL(sort_hist_kernel, dim3(nb), dim3(kSortThreads), 0, s, num_pts, shift, nb,
                       kin, w.hist);
    MCCNN_LAUNCH_CHECK();
    int rc = inclusive_scan_i32(s, (int64_t)kRadix * nb, w.hist, w.scan_scratch, w.total);
    if (rc != MCCNN_OK) return rc;
    if (p == 0)
      hipLaunchKernelGGL(sort_scatter_kernel<true>, dim3(nb), dim3(kSortThreads), 0, s, num_pts,
                         shift, nb, kin, iin, w.hist, kout, iout);
    else
      hipLaunchKernelGGL(sort_scatter_kernel<false>, dim3(nb), dim3(kSortThreads), 0, s, num_pts,
                         shift, nb, kin, iin, w.hist, kout, iout);
    MCCNN_LAUNCH_CHECK();
    kin = kout;
    iin = iout;
  }
  return MCCNN_OK;
}

// ------------------------------------------------- transposed pair lists ----

namespace mccnn {
struct TransposeWorkspace {
  int64_t *keys;
  int64_t *sorted_keys;
  void *sort_ws;
  size_t sort_ws_bytes;
  int *scan_scratch;
  int64_t *total;
  size_t bytes;
};

static TransposeWorkspace carve_transpose_workspace(void *ws, int64_t m, int64_t n) {
  char *p = (char *)ws;
  TransposeWorkspace w;
  size_t off = 0;
  w.keys = (int64_t *)(p + off); off += align256(sizeof(int64_t) * (size_t)m);
  w.sorted_keys = (int64_t *)(p + off); off += align256(sizeof(int64_t) * (size_t)m);
  w.sort_ws = p + off;
  w.sort_ws_bytes = carve_sort_workspace(nullptr, m).bytes;
  off += align256(w.sort_ws_bytes);
  w.scan_scratch = (int *)(p + off); off += align256(sizeof(int) * scan_scratch_ints(n));
  w.total = (int64_t *)(p + off); off += 256;
  w.bytes = off;
  return w;
}
}  // namespace mccnn

extern "C" size_t mccnn_transpose_neighbors_workspace_bytes(int64_t num_neighbors,
                                                            int64_t num_pts) {
  if (num_neighbors < 0) num_neighbors = 0;
  if (num_pts < 0) num_pts = 0;
  return carve_transpose_workspace(nullptr, num_neighbors, num_pts).bytes;
}

extern "C" int mccnn_transpose_neighbors(mccnn_stream_t stream, int64_t num_neighbors,
                                         const int32_t *neighbors, int64_t num_pts,
                                         void *workspace, size_t workspace_bytes,
                                         int32_t *point_ranges_out, int32_t *pair_order_out) {
  MCCNN_REQUIRE(num_neighbors >= 0 && num_neighbors < ((int64_t)1 << 31) && num_pts >= 0 &&
                    num_pts < ((int64_t)1 << 31),
                "transpose_neighbors expects sizes in [0, 2^31)");
  hipStream_t s = as_stream(stream);
  if (num_pts == 0) return MCCNN_OK;
  MCCNN_REQUIRE(point_ranges_out, "transpose_neighbors received a null tensor");
  int rc = fill_zero(s, point_ranges_out, sizeof(int32_t) * (size_t)num_pts);
  if (rc != MCCNN_OK) return rc;
  if (num_neighbors == 0) return MCCNN_OK;
  MCCNN_REQUIRE(neighbors && workspace && pair_order_out,
                "transpose_neighbors received a null tensor");
  const TransposeWorkspace w = carve_transpose_workspace(workspace, num_neighbors, num_pts);
  MCCNN_REQUIRE(workspace_bytes >= w.bytes, "transpose_neighbors workspace too small (%zu < %zu)",
                workspace_bytes, w.bytes);
  int64_t work = num_neighbors > ((int64_t)1 << 26) ? ((int64_t)1 << 26) : num_neighbors;
  hipLaunchKernelGGL(transpose_keys_kernel, dim3(blocks_for(work, 256)), dim3(256), 0, s,
                     num_neighbors, num_pts, (const int2 *)neighbors, w.keys, point_ranges_out);
  MCCNN_LAUNCH_CHECK();
  int bits = 1;
  while (((int64_t)1 << bits) < num_pts) ++bits;
  rc = mccnn_sort_keys_descending(stream, num_neighbors, bits, w.keys, w.sorted_keys,
                                  pair_order_out, w.sort_ws, w.sort_ws_bytes);
  if (rc != MCCNN_OK) return rc;
  return inclusive_scan_i32(s, num_pts, point_ranges_out, w.scan_scratch, w.total);
}
