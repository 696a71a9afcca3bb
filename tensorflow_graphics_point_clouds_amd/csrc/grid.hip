// Regular-grid stage: bounding boxes and grid shape, cell keys, gathers and the
// 2-D column table.  Integer results must equal the reference's bit for bit, so
// this file is compiled with -ffp-contract=off: every float operation that
// decides a cell index is rounded once, as the op contract states it
// (custom_ops/tfg_custom_ops/shared/cc/kernels/grid_utils.h:63-100).
#include <float.h>

#include "common.h"
#include "fill.h"

namespace mccnn {

// ------------------------------------------------------------------ keys ----

template <int D>
__global__ void __launch_bounds__(256) compute_keys_kernel(
    int64_t n, const float *__restrict__ pts, const int *__restrict__ bids,
    const float *__restrict__ smin, const int *__restrict__ num_cells,
    const float *__restrict__ inv_cell, int64_t *__restrict__ keys) {
  const GridShape<D> g = load_shape<D>(num_cells);
  float ic[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ic[d] = inv_cell[d];
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int b = bids[i];
    float p[D], m[D];
#pragma unroll
    for (int d = 0; d < D; ++d) {
      p[d] = pts[i * D + d];
      m[d] = smin[(int64_t)b * D + d];
    }
    int cell[D];
    cell_of_point<D>(p, m, ic, g, cell);
    keys[i] = key_of_cell<D>(cell, g, b);
  }
}

// --------------------------------------------------------------- gathers ----

template <int D>
__global__ void __launch_bounds__(256) gather_points_kernel(
    int64_t n, const float *__restrict__ pts, const int *__restrict__ bids,
    const int *__restrict__ idx, float *__restrict__ pts_out, int *__restrict__ bids_out) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t j = idx[i];
#pragma unroll
    for (int d = 0; d < D; ++d) pts_out[i * D + d] = pts[j * D + d];
    bids_out[i] = bids[j];
  }
}

__global__ void __launch_bounds__(256) original_ids_kernel(int64_t m,
                                                           const int2 *__restrict__ nbrs,
                                                           const int *__restrict__ sorted_idx,
                                                           int2 *__restrict__ out) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < m;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int2 p = nbrs[i];
    out[i] = make_int2(sorted_idx[p.x], p.y);
  }
}

// Rows of the transposed pair table: out[i] = (centre, point) of pair order[i].
__global__ void __launch_bounds__(256) swapped_pairs_kernel(int64_t m,
                                                            const int2 *__restrict__ nbrs,
                                                            const int *__restrict__ order,
                                                            int2 *__restrict__ out) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < m;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int2 p = nbrs[order[i]];
    out[i] = make_int2(p.y, p.x);
  }
}

__global__ void __launch_bounds__(256) gather_pdf_kernel(int64_t m, const int2 *__restrict__ nbrs,
                                                         int column, const float *__restrict__ pdf,
                                                         float *__restrict__ out) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < m;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int2 p = nbrs[i];
    out[i] = pdf[column == 0 ? p.x : p.y];
  }
}

__global__ void __launch_bounds__(256) gather_i32_kernel(int64_t n, const int *__restrict__ src,
                                                         const int *__restrict__ idx,
                                                         int *__restrict__ out) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x)
    out[i] = src[idx[i]];
}

// out[i, :] = src[idx[i], :] for rows of 4 * row_vecs floats, 16 bytes per lane.
__global__ void __launch_bounds__(256) gather_rows_kernel(int64_t total, int row_vecs,
                                                          const float4 *__restrict__ src,
                                                          const int *__restrict__ idx,
                                                          float4 *__restrict__ out) {
  for (int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; t < total;
       t += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = t / row_vecs;
    const int v = (int)(t - row * row_vecs);
    out[t] = src[(int64_t)idx[row] * row_vecs + v];
  }
}

// ------------------------------------------------------------ grid table ----

// Column of a key in the [B, n0, n1] table: key / prod(n[2:]).
template <int D>
__global__ void __launch_bounds__(256) build_grid_ds_kernel(
    int64_t n, const int64_t *__restrict__ keys, const int *__restrict__ num_cells,
    int2 *__restrict__ ds) {
  int64_t div = 1;
#pragma unroll
  for (int d = 2; d < D; ++d) div *= num_cells[d];
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t col = keys[i] / div;
    if (i > 0 && keys[i - 1] / div != col) ds[col].x = (int)i;
    if (i + 1 == n || keys[i + 1] / div != col) ds[col].y = (int)(i + 1);
  }
}

// ------------------------------------------------ bounding box and shape ----

// Order-preserving map float -> uint32 so that min/max can be taken with
// integer atomics.
__device__ __forceinline__ unsigned enc_float(float f) {
  unsigned u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float dec_float(unsigned u) {
  return __uint_as_float((u & 0x80000000u) ? (u & 0x7fffffffu) : ~u);
}

__global__ void aabb_init_kernel(int count, unsigned *mn, unsigned *mx) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) {
    mn[i] = enc_float(FLT_MAX);
    mx[i] = enc_float(-FLT_MAX);
  }
}

// A wavefront walks a run of points (1024 for a large cloud, down to 64 for a small
// one, so that a few thousand points still spread over many wavefronts).  While the 64 points of an
// iteration belong to one cloud (the usual layout: clouds stored one after
// another) the lanes keep running minima / maxima in registers; they are reduced
// over the wavefront and sent as one atomic per dimension when the cloud changes
// or the run ends.  Iterations that straddle two clouds use one atomic per lane.
constexpr int kAabbRun = 1024;

static int aabb_run(int64_t n) {
  int64_t run = (n / 2048 + kWave - 1) / kWave * kWave;     // aim at ~2048 wavefronts
  return (int)(run < kWave ? kWave : (run > kAabbRun ? kAabbRun : run));
}

template <int D>
__device__ __forceinline__ void aabb_flush(int b, float *lo, float *hi, unsigned *mn,
                                           unsigned *mx) {
#pragma unroll
  for (int d = 0; d < D; ++d) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      lo[d] = fminf(lo[d], __shfl_xor(lo[d], off, kWave));
      hi[d] = fmaxf(hi[d], __shfl_xor(hi[d], off, kWave));
    }
    if (lane_id() == 0) {
      atomicMin(&mn[(int64_t)b * D + d], enc_float(lo[d]));
      atomicMax(&mx[(int64_t)b * D + d], enc_float(hi[d]));
    }
    lo[d] = FLT_MAX;
    hi[d] = -FLT_MAX;
  }
}

template <int D>
__global__ void __launch_bounds__(256) aabb_reduce_kernel(
    int64_t n, int run, const float *__restrict__ pts, const int *__restrict__ bids,
    unsigned *mn, unsigned *mx) {
  const int64_t wave = blockIdx.x * (int64_t)(blockDim.x / kWave) + threadIdx.x / kWave;
  const int64_t first = wave * run;
  const int64_t last = first + run < n ? first + run : n;
  float lo[D], hi[D];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    lo[d] = FLT_MAX;
    hi[d] = -FLT_MAX;
  }
  int cur = -1;                     // cloud of the running minima / maxima (wave-uniform)
  for (int64_t base = first; base < last; base += kWave) {
    const int64_t i = base + lane_id();
    const bool live = i < last;
    const int b = live ? bids[i] : -1;
    float p[D];
#pragma unroll
    for (int d = 0; d < D; ++d) p[d] = live ? pts[i * D + d] : 0.f;
    const int b0 = __shfl(b, 0, kWave);
    const bool uniform = __all(b == b0 || !live) && b0 >= 0;
    if (uniform) {
      if (b0 != cur) {
        if (cur >= 0) aabb_flush<D>(cur, lo, hi, mn, mx);
        cur = b0;
      }
      if (live) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
          lo[d] = fminf(lo[d], p[d]);
          hi[d] = fmaxf(hi[d], p[d]);
        }
      }
    } else if (live) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        atomicMin(&mn[(int64_t)b * D + d], enc_float(p[d]));
        atomicMax(&mx[(int64_t)b * D + d], enc_float(p[d]));
      }
    }
  }
  if (cur >= 0) aabb_flush<D>(cur, lo, hi, mn, mx);
}

// min - 1e-9f, max + 1e-9f, grid shape, scaled minimum and reciprocal cell size,
// in the fp32 expressions of the reference's Python glue.
template <int D>
__global__ void grid_finalize_kernel(int batch, const float *__restrict__ cell,
                                     float *aabb_min, float *aabb_max, int *num_cells,
                                     float *smin, float *inv_cell) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  int nc[D];
#pragma unroll
  for (int d = 0; d < D; ++d) nc[d] = 1;
  for (int b = 0; b < batch; ++b) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const float lo = dec_float(reinterpret_cast<unsigned *>(aabb_min)[b * D + d]) - 1e-9f;
      const float hi = dec_float(reinterpret_cast<unsigned *>(aabb_max)[b * D + d]) + 1e-9f;
      aabb_min[b * D + d] = lo;
      aabb_max[b * D + d] = hi;
      const float size = hi - lo;
      const int c = (int)ceilf(size / cell[d]);
      nc[d] = c > nc[d] ? c : nc[d];
      smin[b * D + d] = lo / cell[d];
    }
  }
#pragma unroll
  for (int d = 0; d < D; ++d) {
    num_cells[d] = nc[d];
    inv_cell[d] = 1.0f / cell[d];
  }
}

}  // namespace mccnn

using namespace mccnn;

extern "C" int mccnn_compute_keys(mccnn_stream_t stream, int64_t num_pts, int num_dims,
                                  const float *points, int64_t batch_ids_len,
                                  const int32_t *batch_ids, int64_t aabb_rows, int aabb_dims,
                                  const float *scaled_aabb_min, int num_cells_len,
                                  const int32_t *num_cells, int inv_cell_sizes_len,
                                  const float *inv_cell_sizes, int64_t *keys_out) {
  MCCNN_REQUIRE(valid_dims(num_dims), "ComputeKeys expects a valid number of dimensions (got %d)",
                num_dims);
  MCCNN_REQUIRE(num_pts >= 0 && aabb_rows >= 0, "ComputeKeys expects non-negative sizes");
  MCCNN_REQUIRE(batch_ids_len == num_pts,
                "ComputeKeys expects the same number of batch ids as number of points");
  MCCNN_REQUIRE(aabb_dims == num_dims,
                "ComputeKeys expects aabb with the same number of dimensions as the points");
  MCCNN_REQUIRE(num_cells_len == num_dims,
                "ComputeKeys expects number of cells with the same number of dimensions as the "
                "points");
  MCCNN_REQUIRE(inv_cell_sizes_len == num_dims,
                "ComputeKeys expects cell sizes with the same number of dimensions as the points");
  if (num_pts == 0) return MCCNN_OK;
  MCCNN_REQUIRE(points && batch_ids && scaled_aabb_min && num_cells && inv_cell_sizes && keys_out,
                "ComputeKeys received a null tensor");
  const unsigned grid = blocks_for(num_pts, 256);
  MCCNN_DIM_SWITCH(num_dims, hipLaunchKernelGGL(compute_keys_kernel<D>, dim3(grid), dim3(256), 0,
                                                as_stream(stream), num_pts, points, batch_ids,
                                                scaled_aabb_min, num_cells, inv_cell_sizes,
                                                (int64_t *)keys_out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_gather_points(mccnn_stream_t stream, int64_t num_pts, int num_dims,
                                   const float *points, const int32_t *batch_ids,
                                   const int32_t *indices, float *points_out,
                                   int32_t *batch_ids_out) {
  MCCNN_REQUIRE(valid_dims(num_dims), "gather_points expects a valid number of dimensions");
  MCCNN_REQUIRE(num_pts >= 0, "gather_points expects a non-negative size");
  if (num_pts == 0) return MCCNN_OK;
  MCCNN_REQUIRE(points && batch_ids && indices && points_out && batch_ids_out,
                "gather_points received a null tensor");
  const unsigned grid = blocks_for(num_pts, 256);
  MCCNN_DIM_SWITCH(num_dims, hipLaunchKernelGGL(gather_points_kernel<D>, dim3(grid), dim3(256), 0,
                                                as_stream(stream), num_pts, points, batch_ids,
                                                indices, points_out, batch_ids_out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_build_grid_ds(mccnn_stream_t stream, int64_t num_pts,
                                   const int64_t *sorted_keys, int num_cells_len,
                                   const int32_t *num_cells, int num_cells_host_len,
                                   const int32_t *num_cells_host, int batch_size,
                                   int32_t *ds_out) {
  MCCNN_REQUIRE(batch_size > 0, "BuildGridDs requires a positive batch size");
  MCCNN_REQUIRE(valid_dims(num_cells_len), "BuildGridDs expects a valid number of dimensions");
  MCCNN_REQUIRE(num_cells_host_len == num_cells_len,
                "BuildGridDs expects number of cells with the same dimensions in both parameters");
  MCCNN_REQUIRE(num_pts >= 0 && num_cells && num_cells_host && ds_out,
                "BuildGridDs received a null tensor");
  MCCNN_REQUIRE(num_cells_host[0] > 0 && num_cells_host[1] > 0,
                "BuildGridDs expects a positive number of cells");
  const int64_t cols = (int64_t)batch_size * num_cells_host[0] * num_cells_host[1];
  MCCNN_REQUIRE(cols * 2 < ((int64_t)1 << 31), "BuildGridDs table too large");
  int rc = fill_zero(as_stream(stream), ds_out, sizeof(int32_t) * 2 * (size_t)cols);
  if (rc != MCCNN_OK) return rc;
  if (num_pts == 0) return MCCNN_OK;
  MCCNN_REQUIRE(sorted_keys, "BuildGridDs received a null tensor");
  const unsigned grid = blocks_for(num_pts, 256);
  MCCNN_DIM_SWITCH(num_cells_len,
                   hipLaunchKernelGGL(build_grid_ds_kernel<D>, dim3(grid), dim3(256), 0,
                                      as_stream(stream), num_pts, (const int64_t *)sorted_keys,
                                      num_cells, (int2 *)ds_out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_grid_setup(mccnn_stream_t stream, int64_t num_pts, int num_dims,
                                const float *points, const int32_t *batch_ids, int batch_size,
                                const float *cell_sizes, float *aabb_min_out, float *aabb_max_out,
                                int32_t *num_cells_out, float *scaled_aabb_min_out,
                                float *inv_cell_sizes_out) {
  MCCNN_REQUIRE(valid_dims(num_dims), "grid_setup expects a valid number of dimensions");
  MCCNN_REQUIRE(batch_size > 0, "grid_setup requires a positive batch size");
  MCCNN_REQUIRE(num_pts >= 0 && cell_sizes && aabb_min_out && aabb_max_out && num_cells_out &&
                    scaled_aabb_min_out && inv_cell_sizes_out,
                "grid_setup received a null tensor");
  const int count = batch_size * num_dims;
  hipLaunchKernelGGL(aabb_init_kernel, dim3(blocks_for(count, 256)), dim3(256), 0,
                     as_stream(stream), count, (unsigned *)aabb_min_out, (unsigned *)aabb_max_out);
  MCCNN_LAUNCH_CHECK();
  if (num_pts > 0) {
    MCCNN_REQUIRE(points && batch_ids, "grid_setup received a null tensor");
    const int run = aabb_run(num_pts);
    MCCNN_DIM_SWITCH(num_dims, hipLaunchKernelGGL(aabb_reduce_kernel<D>,
                                                  dim3(blocks_for(num_pts, 4 * run)),
                                                  dim3(256), 0,
                                                  as_stream(stream), num_pts, run, points, batch_ids,
                                                  (unsigned *)aabb_min_out,
                                                  (unsigned *)aabb_max_out));
    MCCNN_LAUNCH_CHECK();
  }
  MCCNN_DIM_SWITCH(num_dims, hipLaunchKernelGGL(grid_finalize_kernel<D>, dim3(1), dim3(64), 0,
                                                as_stream(stream), batch_size, cell_sizes,
                                                aabb_min_out, aabb_max_out, num_cells_out,
                                                scaled_aabb_min_out, inv_cell_sizes_out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

static unsigned capped_grid(int64_t work) {
  if (work > (int64_t)1 << 26) work = (int64_t)1 << 26;
  return blocks_for(work, 256);
}

extern "C" int mccnn_original_neighbor_ids(mccnn_stream_t stream, int64_t num_neighbors,
                                           const int32_t *neighbors,
                                           const int32_t *sorted_indices,
                                           int32_t *original_neighbors_out) {
  MCCNN_REQUIRE(num_neighbors >= 0, "original_neighbor_ids expects a non-negative size");
  if (num_neighbors == 0) return MCCNN_OK;
  MCCNN_REQUIRE(neighbors && sorted_indices && original_neighbors_out,
                "original_neighbor_ids received a null tensor");
  hipLaunchKernelGGL(original_ids_kernel, dim3(capped_grid(num_neighbors)), dim3(256), 0,
                     as_stream(stream), num_neighbors, (const int2 *)neighbors, sorted_indices,
                     (int2 *)original_neighbors_out);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_swapped_pairs(mccnn_stream_t stream, int64_t num_neighbors,
                                   const int32_t *neighbors, const int32_t *pair_order,
                                   int32_t *swapped_out) {
  MCCNN_REQUIRE(num_neighbors >= 0, "swapped_pairs expects a non-negative size");
  if (num_neighbors == 0) return MCCNN_OK;
  MCCNN_REQUIRE(neighbors && pair_order && swapped_out, "swapped_pairs received a null tensor");
  hipLaunchKernelGGL(swapped_pairs_kernel, dim3(capped_grid(num_neighbors)), dim3(256), 0,
                     as_stream(stream), num_neighbors, (const int2 *)neighbors, pair_order,
                     (int2 *)swapped_out);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_gather_pdf_column(mccnn_stream_t stream, int64_t num_neighbors,
                                       const int32_t *neighbors, int column, const float *pdf,
                                       float *pdf_per_pair_out) {
  MCCNN_REQUIRE(num_neighbors >= 0, "gather_pdf expects a non-negative size");
  MCCNN_REQUIRE(column == 0 || column == 1, "gather_pdf expects column 0 or 1 (got %d)", column);
  if (num_neighbors == 0) return MCCNN_OK;
  MCCNN_REQUIRE(neighbors && pdf && pdf_per_pair_out, "gather_pdf received a null tensor");
  hipLaunchKernelGGL(gather_pdf_kernel, dim3(capped_grid(num_neighbors)), dim3(256), 0,
                     as_stream(stream), num_neighbors, (const int2 *)neighbors, column, pdf,
                     pdf_per_pair_out);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_gather_pdf(mccnn_stream_t stream, int64_t num_neighbors,
                                const int32_t *neighbors, const float *pdf,
                                float *pdf_per_pair_out) {
  return mccnn_gather_pdf_column(stream, num_neighbors, neighbors, 0, pdf, pdf_per_pair_out);
}

extern "C" int mccnn_gather_rows(mccnn_stream_t stream, int64_t num_rows, int num_cols,
                                 const float *src, const int32_t *indices, float *out) {
  MCCNN_REQUIRE(num_rows >= 0, "gather_rows expects a non-negative size");
  MCCNN_REQUIRE(num_cols > 0 && num_cols % 4 == 0,
                "gather_rows expects a row length that is a multiple of 4 (got %d)", num_cols);
  if (num_rows == 0) return MCCNN_OK;
  MCCNN_REQUIRE(src && indices && out, "gather_rows received a null tensor");
  const int64_t total = num_rows * (num_cols / 4);
  hipLaunchKernelGGL(gather_rows_kernel, dim3(capped_grid(total)), dim3(256), 0,
                     as_stream(stream), total, num_cols / 4, (const float4 *)src, indices,
                     (float4 *)out);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_gather_i32(mccnn_stream_t stream, int64_t count, const int32_t *src,
                                const int32_t *indices, int32_t *out) {
  MCCNN_REQUIRE(count >= 0, "gather_i32 expects a non-negative size");
  if (count == 0) return MCCNN_OK;
  MCCNN_REQUIRE(src && indices && out, "gather_i32 received a null tensor");
  hipLaunchKernelGGL(gather_i32_kernel, dim3(capped_grid(count)), dim3(256), 0,
                     as_stream(stream), count, src, indices, out);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

// The grid of pylib/pc/Grid.py:32-64 in one call: bounding boxes and grid shape, keys, the
// host copy of the grid shape (the one synchronisation: it sizes the key width of the sort
// and, for the caller, the grid table), stable descending sort, gathers.  The same
// sequence a caller gets from the five entry points above; small clouds are bound by the
// cost of making calls and launches, and this is one call instead of five.
extern "C" size_t mccnn_build_grid_workspace_bytes(int64_t num_pts) {
  return mccnn_sort_keys_workspace_bytes(num_pts);
}

extern "C" int mccnn_build_grid(mccnn_stream_t stream, int64_t num_pts, int num_dims,
                                const float *points, const int32_t *batch_ids, int batch_size,
                                const float *cell_sizes, float *aabb_min_out,
                                float *aabb_max_out, int32_t *num_cells_out,
                                float *scaled_aabb_min_out, float *inv_cell_sizes_out,
                                int64_t *keys_out, int64_t *sorted_keys_out,
                                int32_t *sorted_indices_out, float *sorted_points_out,
                                int32_t *sorted_batch_ids_out, void *workspace,
                                size_t workspace_bytes, int32_t *num_cells_out_host,
                                int *key_bits_out_host) {
  MCCNN_REQUIRE(valid_dims(num_dims), "build_grid expects a valid number of dimensions");
  MCCNN_REQUIRE(num_cells_out_host && key_bits_out_host,
                "build_grid needs host outputs for the grid shape and the key width");
  int rc = mccnn_grid_setup(stream, num_pts, num_dims, points, batch_ids, batch_size, cell_sizes,
                            aabb_min_out, aabb_max_out, num_cells_out, scaled_aabb_min_out,
                            inv_cell_sizes_out);
  if (rc != MCCNN_OK) return rc;
  rc = mccnn_compute_keys(stream, num_pts, num_dims, points, num_pts, batch_ids, batch_size,
                          num_dims, scaled_aabb_min_out, num_dims, num_cells_out, num_dims,
                          inv_cell_sizes_out, keys_out);
  if (rc != MCCNN_OK) return rc;
  hipStream_t s = as_stream(stream);
  MCCNN_HIP_CHECK(hipMemcpyAsync(num_cells_out_host, num_cells_out, sizeof(int32_t) * num_dims,
                                 hipMemcpyDeviceToHost, s));
  MCCNN_HIP_CHECK(hipStreamSynchronize(s));
  unsigned long long total = (unsigned long long)(batch_size > 0 ? batch_size : 1);
  for (int d = 0; d < num_dims; ++d) total *= (unsigned long long)num_cells_out_host[d];
  int bits = 1;
  while (bits < 64 && (1ull << bits) < total) ++bits;
  *key_bits_out_host = bits;
  rc = mccnn_sort_keys_descending(stream, num_pts, bits, keys_out, sorted_keys_out,
                                  sorted_indices_out, workspace, workspace_bytes);
  if (rc != MCCNN_OK) return rc;
  return mccnn_gather_points(stream, num_pts, num_dims, points, batch_ids, sorted_indices_out,
                             sorted_points_out, sorted_batch_ids_out);
}
