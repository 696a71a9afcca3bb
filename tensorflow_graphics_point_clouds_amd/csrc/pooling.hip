// Neighbourhood and per-cloud pooling (pylib/pc/layers/Pooling.py:25-166: the
// reference gathers the features of every pair and applies TensorFlow's
// unsorted_segment_max / _mean).  Here a group of lanes owns a centre, strides
// over its channels and walks the pair list, so the [M, C] gathered tensor is
// never materialised.
#include <float.h>

#include "common.h"
#include "fill.h"

namespace mccnn {

constexpr int kPoolThreads = 256;

// blockDim = 256; each centre gets `lanes` threads (a power of two <= 64).
template <bool kMax>
__global__ void __launch_bounds__(kPoolThreads) local_pool_kernel(
    int64_t n_out, int C, int lanes, const float *__restrict__ feat,
    const int2 *__restrict__ nbrs, const int *__restrict__ ranges, float *__restrict__ out) {
  const int per_block = kPoolThreads / lanes;
  const int64_t centre = (int64_t)blockIdx.x * per_block + threadIdx.x / lanes;
  if (centre >= n_out) return;
  const int sub = threadIdx.x % lanes;
  const int a = centre > 0 ? ranges[centre - 1] : 0, b = ranges[centre];
  for (int c = sub; c < C; c += lanes) {
    float acc = kMax ? -FLT_MAX : 0.0f;
    for (int m = a; m < b; ++m) {
      const float v = feat[(int64_t)nbrs[m].x * C + c];
      acc = kMax ? fmaxf(acc, v) : acc + v;
    }
    if (!kMax) acc = acc / (float)(b - a > 0 ? b - a : 1);
    out[centre * C + c] = acc;
  }
}

// One wavefront per centre for C = 4 * 2^q <= 256 channels: a feature row is read
// by C/4 lanes with 16-byte loads, so one load instruction fetches 256/C rows; the
// neighbour indices are read 64 at a time and passed around by lane shuffle, four
// row loads are in flight per lane.  The partial results of the lane groups are
// combined by butterfly shuffles at the end.
template <bool kMax>
__global__ void __launch_bounds__(kPoolThreads) local_pool_rows_kernel(
    int64_t n_out, int C, int lpr_log2, const float *__restrict__ feat,
    const int2 *__restrict__ nbrs, const int *__restrict__ ranges, float *__restrict__ out) {
  const int64_t centre = (int64_t)blockIdx.x * (kPoolThreads / kWave) + threadIdx.x / kWave;
  if (centre >= n_out) return;
  const int lane = lane_id();
  const int lpr = 1 << lpr_log2;                 // lanes per row
  const int slot = lane >> lpr_log2, colv = lane & (lpr - 1);
  const int slots = kWave >> lpr_log2;           // rows per load instruction
  const int a = centre > 0 ? ranges[centre - 1] : 0, b = ranges[centre];
  const float init = kMax ? -FLT_MAX : 0.0f;
  float4 acc = make_float4(init, init, init, init);
  const float *fl = feat + 4 * colv;
  for (int m0 = a; m0 < b; m0 += kWave) {
    const int cnt = b - m0 < kWave ? b - m0 : kWave;
    const int myidx = nbrs[m0 + (lane < cnt ? lane : 0)].x;
    for (int t0 = 0; t0 < cnt; t0 += 4 * slots) {      // uniform trip count: shuffles inside
      float4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int n = t0 + slot + u * slots;
        const int idx = __shfl(myidx, n < cnt ? n : 0, kWave);   // past the end: repeat pair 0
        v[u] = *reinterpret_cast<const float4 *>(fl + (int64_t)idx * C);
        if (!kMax && n >= cnt) v[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        acc.x = kMax ? fmaxf(acc.x, v[u].x) : acc.x + v[u].x;
        acc.y = kMax ? fmaxf(acc.y, v[u].y) : acc.y + v[u].y;
        acc.z = kMax ? fmaxf(acc.z, v[u].z) : acc.z + v[u].z;
        acc.w = kMax ? fmaxf(acc.w, v[u].w) : acc.w + v[u].w;
      }
    }
  }
  for (int off = lpr; off < kWave; off <<= 1) {
    const float x = __shfl_xor(acc.x, off, kWave), y = __shfl_xor(acc.y, off, kWave);
    const float z = __shfl_xor(acc.z, off, kWave), w = __shfl_xor(acc.w, off, kWave);
    acc.x = kMax ? fmaxf(acc.x, x) : acc.x + x;
    acc.y = kMax ? fmaxf(acc.y, y) : acc.y + y;
    acc.z = kMax ? fmaxf(acc.z, z) : acc.z + z;
    acc.w = kMax ? fmaxf(acc.w, w) : acc.w + w;
  }
  if (slot != 0) return;
  if (!kMax) {
    const float inv = 1.0f / (float)(b - a > 0 ? b - a : 1);
    acc.x *= inv; acc.y *= inv; acc.z *= inv; acc.w *= inv;
  }
  *reinterpret_cast<float4 *>(out + centre * C + 4 * colv) = acc;
}

template <bool kMax>
__global__ void __launch_bounds__(kPoolThreads) local_pool_grads_kernel(
    int64_t n_out, int C, int lanes, const float *__restrict__ feat,
    const int2 *__restrict__ nbrs, const int *__restrict__ ranges, const float *__restrict__ out,
    const float *__restrict__ out_grads, float *__restrict__ dfeat) {
  const int per_block = kPoolThreads / lanes;
  const int64_t centre = (int64_t)blockIdx.x * per_block + threadIdx.x / lanes;
  if (centre >= n_out) return;
  const int sub = threadIdx.x % lanes;
  const int a = centre > 0 ? ranges[centre - 1] : 0, b = ranges[centre];
  if (b <= a) return;
  for (int c = sub; c < C; c += lanes) {
    const float g = out_grads[centre * C + c];
    if (kMax) {
      const float top = out[centre * C + c];
      int ties = 0;
      for (int m = a; m < b; ++m) ties += feat[(int64_t)nbrs[m].x * C + c] == top ? 1 : 0;
      const float share = g / (float)(ties > 0 ? ties : 1);
      for (int m = a; m < b; ++m) {
        const int64_t nb = nbrs[m].x;
        if (feat[nb * C + c] == top) unsafeAtomicAdd(&dfeat[nb * C + c], share);
      }
    } else {
      const float share = g / (float)(b - a);
      for (int m = a; m < b; ++m) unsafeAtomicAdd(&dfeat[(int64_t)nbrs[m].x * C + c], share);
    }
  }
}

__device__ __forceinline__ unsigned enc_order(float f) {
  unsigned u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float dec_order(unsigned u) {
  return __uint_as_float((u & 0x80000000u) ? (u & 0x7fffffffu) : ~u);
}

__global__ void global_pool_init_kernel(int count, int batch, bool is_max, unsigned *out,
                                        int *counts) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) out[i] = is_max ? enc_order(-FLT_MAX) : __float_as_uint(0.0f);
  if (i < batch) counts[i] = 0;
}

constexpr int kGlobalChunk = 64;   // points walked by one thread

// Thread (chunk of points, channel): running value per run of equal batch ids,
// flushed with one atomic when the id changes.
template <bool kMax>
__global__ void __launch_bounds__(256) global_pool_kernel(int64_t n, int C,
                                                          const float *__restrict__ feat,
                                                          const int *__restrict__ bids,
                                                          unsigned *out, int *counts) {
  const int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  const int64_t chunk = t / C;
  const int c = (int)(t - chunk * C);
  const int64_t i0 = chunk * kGlobalChunk;
  if (i0 >= n) return;
  const int64_t i1 = i0 + kGlobalChunk < n ? i0 + kGlobalChunk : n;
  int cur = bids[i0], run = 0;
  float acc = kMax ? -FLT_MAX : 0.0f;
  for (int64_t i = i0; i < i1; ++i) {
    const int b = bids[i];
    if (b != cur) {
      if (kMax) atomicMax(&out[(int64_t)cur * C + c], enc_order(acc));
      else unsafeAtomicAdd(reinterpret_cast<float *>(out) + (int64_t)cur * C + c, acc);
      if (c == 0) atomicAdd(&counts[cur], run);
      cur = b;
      run = 0;
      acc = kMax ? -FLT_MAX : 0.0f;
    }
    const float v = feat[i * C + c];
    acc = kMax ? fmaxf(acc, v) : acc + v;
    ++run;
  }
  if (kMax) atomicMax(&out[(int64_t)cur * C + c], enc_order(acc));
  else unsafeAtomicAdd(reinterpret_cast<float *>(out) + (int64_t)cur * C + c, acc);
  if (c == 0) atomicAdd(&counts[cur], run);
}

__global__ void global_pool_finish_kernel(int batch, int C, bool is_max, unsigned *out,
                                          const int *counts) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= batch * C) return;
  float *o = reinterpret_cast<float *>(out);
  if (is_max) {
    o[i] = dec_order(out[i]);
  } else {
    const int cnt = counts[i / C];
    o[i] = o[i] / (float)(cnt > 0 ? cnt : 1);
  }
}

// Max: the points whose feature equals the pooled value share the gradient
// equally; their number per (cloud, channel) is counted first.
__global__ void __launch_bounds__(256) global_pool_ties_kernel(int64_t n, int C,
                                                               const float *__restrict__ feat,
                                                               const int *__restrict__ bids,
                                                               const float *__restrict__ out,
                                                               float *tie_sums) {
  for (int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; t < n * C;
       t += (int64_t)gridDim.x * blockDim.x) {
    const int64_t i = t / C;
    const int c = (int)(t - i * C);
    const int64_t o = (int64_t)bids[i] * C + c;
    if (feat[t] == out[o]) unsafeAtomicAdd(&tie_sums[o], 1.0f);
  }
}

template <bool kMax>
__global__ void __launch_bounds__(256) global_pool_grads_kernel(
    int64_t n, int C, const float *__restrict__ feat, const int *__restrict__ bids,
    const float *__restrict__ out, const int *__restrict__ counts,
    const float *__restrict__ tie_sums, const float *__restrict__ out_grads,
    float *__restrict__ dfeat) {
  for (int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; t < n * C;
       t += (int64_t)gridDim.x * blockDim.x) {
    const int64_t i = t / C;
    const int c = (int)(t - i * C);
    const int b = bids[i];
    const int64_t o = (int64_t)b * C + c;
    if (kMax) dfeat[t] = feat[t] == out[o] ? out_grads[o] / tie_sums[o] : 0.0f;
    else dfeat[t] = out_grads[o] / (float)counts[b];
  }
}

static int lanes_for(int C) {
  int l = 1;
  while (l < C && l < 64) l <<= 1;
  return l;
}

}  // namespace mccnn

using namespace mccnn;

extern "C" int mccnn_local_pool(mccnn_stream_t stream, int kind, int64_t num_pts,
                                int num_features, const float *features, int64_t num_neighbors,
                                const int32_t *neighbors, int64_t num_samples,
                                const int32_t *ranges, float *out) {
  MCCNN_REQUIRE(kind == 0 || kind == 1, "local_pool expects kind 0 (max) or 1 (average)");
  MCCNN_REQUIRE(num_features > 0 && num_pts >= 0 && num_neighbors >= 0 && num_samples >= 0,
                "local_pool expects non-negative sizes and at least one feature");
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(ranges && out && (num_neighbors == 0 || (features && neighbors)),
                "local_pool received a null tensor");
  // C = 4 * 2^q <= 256: row-vectorised kernel, one wavefront per centre
  int lpr_log2 = -1;
  for (int q = 0; q <= 6; ++q)
    if (num_features == (4 << q)) lpr_log2 = q;
  if (lpr_log2 >= 0) {
    const unsigned wgrid = blocks_for(num_samples, kPoolThreads / kWave);
    if (kind == 0)
      hipLaunchKernelGGL(local_pool_rows_kernel<true>, dim3(wgrid), dim3(kPoolThreads), 0,
                         as_stream(stream), num_samples, num_features, lpr_log2, features,
                         (const int2 *)neighbors, ranges, out);
    else
      hipLaunchKernelGGL(local_pool_rows_kernel<false>, dim3(wgrid), dim3(kPoolThreads), 0,
                         as_stream(stream), num_samples, num_features, lpr_log2, features,
                         (const int2 *)neighbors, ranges, out);
    MCCNN_LAUNCH_CHECK();
    return MCCNN_OK;
  }
  const int lanes = lanes_for(num_features);
  const unsigned grid = blocks_for(num_samples, kPoolThreads / lanes);
  if (kind == 0)
    hipLaunchKernelGGL(local_pool_kernel<true>, dim3(grid), dim3(kPoolThreads), 0,
                       as_stream(stream), num_samples, num_features, lanes, features,
                       (const int2 *)neighbors, ranges, out);
  else
    hipLaunchKernelGGL(local_pool_kernel<false>, dim3(grid), dim3(kPoolThreads), 0,
                       as_stream(stream), num_samples, num_features, lanes, features,
                       (const int2 *)neighbors, ranges, out);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_local_pool_grads(mccnn_stream_t stream, int kind, int64_t num_pts,
                                      int num_features, const float *features,
                                      int64_t num_neighbors, const int32_t *neighbors,
                                      int64_t num_samples, const int32_t *ranges,
                                      const float *out, const float *out_grads,
                                      float *feature_grads_out) {
  MCCNN_REQUIRE(kind == 0 || kind == 1, "local_pool_grads expects kind 0 (max) or 1 (average)");
  MCCNN_REQUIRE(num_features > 0 && num_pts >= 0 && num_neighbors >= 0 && num_samples >= 0,
                "local_pool_grads expects non-negative sizes and at least one feature");
  hipStream_t s = as_stream(stream);
  if (num_pts > 0) {
    MCCNN_REQUIRE(feature_grads_out, "local_pool_grads received a null tensor");
    int rc = fill_zero(s, feature_grads_out, sizeof(float) * (size_t)num_pts * num_features);
    if (rc != MCCNN_OK) return rc;
  }
  if (num_samples == 0 || num_neighbors == 0) return MCCNN_OK;
  MCCNN_REQUIRE(ranges && features && neighbors && out && out_grads,
                "local_pool_grads received a null tensor");
  const int lanes = lanes_for(num_features);
  const unsigned grid = blocks_for(num_samples, kPoolThreads / lanes);
  if (kind == 0)
    hipLaunchKernelGGL(local_pool_grads_kernel<true>, dim3(grid), dim3(kPoolThreads), 0, s,
                       num_samples, num_features, lanes, features, (const int2 *)neighbors, ranges,
                       out, out_grads, feature_grads_out);
  else
    hipLaunchKernelGGL(local_pool_grads_kernel<false>, dim3(grid), dim3(kPoolThreads), 0, s,
                       num_samples, num_features, lanes, features, (const int2 *)neighbors, ranges,
                       out, out_grads, feature_grads_out);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_global_pool(mccnn_stream_t stream, int kind, int64_t num_pts,
                                 int num_features, const float *features,
                                 const int32_t *batch_ids, int batch_size, float *out,
                                 int32_t *counts_out) {
  MCCNN_REQUIRE(kind == 0 || kind == 1, "global_pool expects kind 0 (max) or 1 (average)");
  MCCNN_REQUIRE(num_features > 0 && num_pts >= 0 && batch_size > 0,
                "global_pool expects a positive batch size and at least one feature");
  MCCNN_REQUIRE(out && counts_out && (num_pts == 0 || (features && batch_ids)),
                "global_pool received a null tensor");
  hipStream_t s = as_stream(stream);
  const int count = batch_size * num_features;
  const int init = count > batch_size ? count : batch_size;
  hipLaunchKernelGGL(global_pool_init_kernel, dim3(blocks_for(init, 256)), dim3(256), 0, s, count,
                     batch_size, kind == 0, (unsigned *)out, counts_out);
  MCCNN_LAUNCH_CHECK();
  if (num_pts > 0) {
    const int64_t chunks = (num_pts + kGlobalChunk - 1) / kGlobalChunk;
    const unsigned grid = blocks_for(chunks * num_features, 256);
    if (kind == 0)
      hipLaunchKernelGGL(global_pool_kernel<true>, dim3(grid), dim3(256), 0, s, num_pts,
                         num_features, features, batch_ids, (unsigned *)out, counts_out);
    else
      hipLaunchKernelGGL(global_pool_kernel<false>, dim3(grid), dim3(256), 0, s, num_pts,
                         num_features, features, batch_ids, (unsigned *)out, counts_out);
    MCCNN_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(global_pool_finish_kernel, dim3(blocks_for(count, 256)), dim3(256), 0, s,
                     batch_size, num_features, kind == 0, (unsigned *)out, counts_out);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_global_pool_grads(mccnn_stream_t stream, int kind, int64_t num_pts,
                                       int num_features, const float *features,
                                       const int32_t *batch_ids, int batch_size, const float *out,
                                       const int32_t *counts, const float *out_grads,
                                       float *tie_workspace, float *feature_grads_out) {
  MCCNN_REQUIRE(kind == 0 || kind == 1, "global_pool_grads expects kind 0 (max) or 1 (average)");
  MCCNN_REQUIRE(num_features > 0 && num_pts >= 0 && batch_size > 0,
                "global_pool_grads expects a positive batch size and at least one feature");
  if (num_pts == 0) return MCCNN_OK;
  MCCNN_REQUIRE(features && batch_ids && out && counts && out_grads && feature_grads_out &&
                    (kind == 1 || tie_workspace),
                "global_pool_grads received a null tensor");
  hipStream_t s = as_stream(stream);
  int64_t work = num_pts * num_features;
  if (work > (int64_t)1 << 24) work = (int64_t)1 << 24;
  const unsigned grid = blocks_for(work, 256);
  if (kind == 0) {
    int rc = fill_zero(s, tie_workspace, sizeof(float) * (size_t)batch_size * num_features);
    if (rc != MCCNN_OK) return rc;
    hipLaunchKernelGGL(global_pool_ties_kernel, dim3(grid), dim3(256), 0, s, num_pts,
                       num_features, features, batch_ids, out, tie_workspace);
    MCCNN_LAUNCH_CHECK();
    hipLaunchKernelGGL(global_pool_grads_kernel<true>, dim3(grid), dim3(256), 0, s, num_pts,
                       num_features, features, batch_ids, out, counts, tie_workspace, out_grads,
                       feature_grads_out);
  } else {
    hipLaunchKernelGGL(global_pool_grads_kernel<false>, dim3(grid), dim3(256), 0, s, num_pts,
                       num_features, features, batch_ids, out, counts, (const float *)nullptr,
                       out_grads, feature_grads_out);
  }
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}
