// Point-cloud sampling on the sorted grid
// (custom_ops/tfg_custom_ops/sampling/cc/ops/sampling_ops.cpp:131-194):
// mode 0 Poisson disk (count_sampling_pd_kernels.cu.cc:41-181), mode 1 cell
// average (sampling_avg_kernels.cu.cc:42-88).
//
// Occupied cells are found by flagging key changes and a prefix sum, so the
// cell list and both outputs keep the sorted order (the reference compacts with
// a global atomic counter and leaves the order to chance).  Poisson disk keeps
// the reference's 2^D cell-parity launches; inside a launch one wavefront owns a
// cell and decides its points in order (details at the kernel).  Cell averages are summed serially in sorted order so that the
// result is bit-reproducible (later hierarchy levels derive integer keys from
// these points).
#include "common.h"
#include "fill.h"

namespace mccnn {

// cell_scan[i] = 1 at the first point of each occupied cell (scanned in place
// afterwards into "cells up to and including i").
__global__ void __launch_bounds__(256) flag_cell_starts_kernel(int64_t n,
                                                               const int64_t *__restrict__ keys,
                                                               int *__restrict__ cell_scan) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x)
    cell_scan[i] = (i == 0 || keys[i] != keys[i - 1]) ? 1 : 0;
}

__global__ void __launch_bounds__(256) store_cell_starts_kernel(int64_t n,
                                                                const int64_t *__restrict__ keys,
                                                                const int *__restrict__ cell_scan,
                                                                int *__restrict__ first_idx) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x)
    if (i == 0 || keys[i] != keys[i - 1]) first_idx[cell_scan[i] - 1] = (int)i;
}

// Parity class of every occupied cell: bit d = parity of the cell index in dim d.
template <int D>
__global__ void __launch_bounds__(256) cell_class_kernel(
    const int64_t *__restrict__ num_cells_total /*device*/, const int64_t *__restrict__ keys,
    const int *__restrict__ num_cells, const int *__restrict__ first_idx,
    int *__restrict__ cell_class) {
  const int64_t cells = *num_cells_total;
  for (int64_t u = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; u < cells;
       u += (int64_t)gridDim.x * blockDim.x) {
    // decode the cell index of the key (batch digit dropped)
    int64_t aux = keys[first_idx[u]];
    int cls = 0;
#pragma unroll
    for (int d = D - 1; d >= 0; --d) {
      const int nd = num_cells[d];
      const int cd = (int)(aux % nd);
      aux /= nd;
      cls |= (cd & 1) << d;
    }
    cell_class[u] = cls;
  }
}

// One wavefront per occupied cell of parity class `call`: it visits the cell's
// points in ascending sorted index and spreads each point's neighbour list over its
// lanes; a point is selected unless one of its neighbours already is.  (Cells of one
// class are at least a cell apart, so only the wavefront's own selections can change
// under it during a pass.  Sweeping a cell's whole pair stretch first, to leave only
// a register-level pass for the order-dependent part, was measured and is not
// faster: the passes are bound by the launch of a wavefront per cell and by the
// latency of the sweep, not by the chain from point to point.)
__global__ void __launch_bounds__(256) poisson_pass_kernel(
    int64_t n, int call, const int64_t *__restrict__ num_cells_total /*device*/,
    const int *__restrict__ cell_class, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, const int *__restrict__ first_idx, int *used) {
  const int64_t cells = *num_cells_total;
  const int64_t u = __builtin_amdgcn_readfirstlane(
      (int)((blockIdx.x * (int64_t)blockDim.x + threadIdx.x) / kWave));
  if (u >= cells || cell_class[u] != call) return;
  const int lane = lane_id();
  const int64_t cell_end = u + 1 < cells ? (int64_t)first_idx[u + 1] : n;
  for (int64_t i = first_idx[u]; i < cell_end; ++i) {
    const int a = i > 0 ? ranges[i - 1] : 0, b = ranges[i];
    bool taken = false;
    for (int m = a + lane; m < b; m += kWave) {
      const int nb = nbrs[m].x;
      taken = taken ||
              __hip_atomic_load(&used[nb], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
    }
    if (!__any(taken)) {
      if (lane == 0) __hip_atomic_store(&used[i], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      // Later points of this cell must observe the selection.  They are visited by
      // this same wavefront, and `used` is read and written past the per-CU cache
      // (device-scope atomics), so it is enough that the store has reached L2 before
      // the next loads are issued: a workgroup-scope fence.  A device-scope fence here
      // also writes the whole L2 back, once per selected point; other wavefronts only
      // need the selections in the next launch.
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      // (the compiler relies on the per-CU cache serving a workgroup's accesses in
      // order and emits no wait for this scope; wait for the store's acknowledgement
      // anyway, it costs one round trip per selected point)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    }
  }
}

template <int D>
__global__ void __launch_bounds__(256) store_selected_kernel(
    int64_t n, const float *__restrict__ pts, const int *__restrict__ bids,
    const int *__restrict__ used, const int *__restrict__ sel_scan, float *__restrict__ out_pts,
    int *__restrict__ out_bids, int *__restrict__ out_idx) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    if (used[i]) {
      const int64_t pos = sel_scan[i] - 1;
#pragma unroll
      for (int d = 0; d < D; ++d) out_pts[pos * D + d] = pts[i * D + d];
      out_bids[pos] = bids[i];
      out_idx[pos] = (int)i;
    }
  }
}

template <int D>
__global__ void __launch_bounds__(256) cell_average_kernel(
    int64_t n, int64_t cells, const float *__restrict__ pts, const int64_t *__restrict__ keys,
    const int *__restrict__ num_cells, const int *__restrict__ first_idx,
    float *__restrict__ out_pts, int *__restrict__ out_bids, int *__restrict__ out_idx) {
  int64_t total = 1;
#pragma unroll
  for (int d = 0; d < D; ++d) total *= num_cells[d];
  for (int64_t u = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; u < cells;
       u += (int64_t)gridDim.x * blockDim.x) {
    int64_t i = first_idx[u];
    const int64_t key = keys[i];
    float acc[D];
#pragma unroll
    for (int d = 0; d < D; ++d) acc[d] = 0.0f;
    int cnt = 0;
    while (i < n && keys[i] == key) {
#pragma unroll
      for (int d = 0; d < D; ++d) acc[d] = acc[d] + pts[i * D + d];
      ++cnt;
      ++i;
    }
    const float fc = (float)cnt;
#pragma unroll
    for (int d = 0; d < D; ++d) out_pts[u * D + d] = acc[d] / fc;
    out_bids[u] = (int)(key / total);
    out_idx[u] = first_idx[u];
  }
}

struct SamplingWorkspace {
  int *cell_scan;    // [n]
  int *first_idx;    // [n]
  int *used;         // [n]
  int *sel_scan;     // [n]
  int *scan_scratch;
  int64_t *num_cells_total;
  int64_t *num_selected;
  size_t bytes;
};

static SamplingWorkspace carve_sampling_workspace(void *ws, int64_t n) {
  char *p = (char *)ws;
  SamplingWorkspace w;
  size_t off = 0;
  const size_t arr = align256(sizeof(int) * (size_t)n);
  w.cell_scan = (int *)(p + off); off += arr;
  w.first_idx = (int *)(p + off); off += arr;
  w.used = (int *)(p + off); off += arr;
  w.sel_scan = (int *)(p + off); off += arr;
  w.scan_scratch = (int *)(p + off); off += align256(sizeof(int) * scan_scratch_ints(n));
  w.num_cells_total = (int64_t *)(p + off); off += 256;
  w.num_selected = (int64_t *)(p + off); off += 256;
  w.bytes = off;
  return w;
}

__global__ void __launch_bounds__(256) copy_i32_kernel(int64_t n, const int *__restrict__ src,
                                                       int *__restrict__ dst) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

}  // namespace mccnn

using namespace mccnn;

extern "C" size_t mccnn_sampling_workspace_bytes(int64_t num_pts) {
  if (num_pts < 0) num_pts = 0;
  return carve_sampling_workspace(nullptr, num_pts).bytes;
}

extern "C" int mccnn_sampling_count(mccnn_stream_t stream, int mode, int64_t num_pts, int num_dims,
                                    const float *points, int64_t batch_ids_len,
                                    const int32_t *batch_ids, int64_t point_keys_len,
                                    const int64_t *point_keys, int num_cells_len,
                                    const int32_t *num_cells, int64_t num_neighbors,
                                    int neighbors_rank, int neighbors_cols,
                                    const int32_t *neighbors, int64_t ranges_len,
                                    const int32_t *ranges, void *workspace,
                                    size_t workspace_bytes, int64_t *num_sampled_out_host) {
  MCCNN_REQUIRE(mode >= 0 && mode < 2, "Sampling requires a valid sampling mode");
  MCCNN_REQUIRE(valid_dims(num_dims), "Sampling expects a valid number of dimensions");
  MCCNN_REQUIRE(batch_ids_len == num_pts,
                "Sampling expects the same number of batch ids as number of points");
  MCCNN_REQUIRE(point_keys_len == num_pts,
                "Sampling expects the same number of keys as number of points");
  MCCNN_REQUIRE(num_cells_len == num_dims,
                "Sampling expects a number of dimensions in num_cells equal to the number of "
                "dimensions in the input points");
  MCCNN_REQUIRE(neighbors_rank == 2 && neighbors_cols == 2,
                "Sampling expects a neighbor tensor with 2 dimensions and 2 indices per neighbor");
  MCCNN_REQUIRE(ranges_len == num_pts,
                "Sampling expects the same number of points in ranges as in the points tensor");
  MCCNN_REQUIRE(num_pts >= 0 && num_pts < ((int64_t)1 << 31) && num_neighbors >= 0,
                "Sampling expects sizes in [0, 2^31)");
  MCCNN_REQUIRE(num_sampled_out_host, "Sampling received a null output");
  *num_sampled_out_host = 0;
  if (num_pts == 0) return MCCNN_OK;
  MCCNN_REQUIRE(points && batch_ids && point_keys && num_cells && ranges && workspace &&
                    (neighbors || num_neighbors == 0),
                "Sampling received a null tensor");
  const SamplingWorkspace w = carve_sampling_workspace(workspace, num_pts);
  MCCNN_REQUIRE(workspace_bytes >= w.bytes, "Sampling workspace too small (%zu < %zu)",
                workspace_bytes, w.bytes);
  hipStream_t s = as_stream(stream);
  const unsigned grid = blocks_for(num_pts, 256);
  hipLaunchKernelGGL(flag_cell_starts_kernel, dim3(grid), dim3(256), 0, s, num_pts,
                     (const int64_t *)point_keys, w.cell_scan);
  MCCNN_LAUNCH_CHECK();
  int rc = inclusive_scan_i32(s, num_pts, w.cell_scan, w.scan_scratch, w.num_cells_total);
  if (rc != MCCNN_OK) return rc;
  hipLaunchKernelGGL(store_cell_starts_kernel, dim3(grid), dim3(256), 0, s, num_pts,
                     (const int64_t *)point_keys, w.cell_scan, w.first_idx);
  MCCNN_LAUNCH_CHECK();
  const int64_t *result = w.num_cells_total;
  if (mode == 0) {
    rc = fill_zero(s, w.used, sizeof(int) * (size_t)num_pts);
    if (rc != MCCNN_OK) return rc;
    // at most num_pts occupied cells; the kernels read the true count on device.  The
    // classes live in sel_scan, which is only filled after the passes.
    MCCNN_DIM_SWITCH(num_dims, hipLaunchKernelGGL(cell_class_kernel<D>, dim3(grid), dim3(256), 0, s,
                                                  w.num_cells_total, (const int64_t *)point_keys,
                                                  num_cells, w.first_idx, w.sel_scan));
    MCCNN_LAUNCH_CHECK();
    const unsigned wgrid = blocks_for(num_pts, 256 / kWave);
    for (int call = 0; call < (1 << num_dims); ++call) {
      hipLaunchKernelGGL(poisson_pass_kernel, dim3(wgrid), dim3(256), 0, s, num_pts, call,
                         w.num_cells_total, w.sel_scan, (const int2 *)neighbors, ranges,
                         w.first_idx, w.used);
      MCCNN_LAUNCH_CHECK();
    }
    hipLaunchKernelGGL(copy_i32_kernel, dim3(grid), dim3(256), 0, s, num_pts, w.used, w.sel_scan);
    MCCNN_LAUNCH_CHECK();
    rc = inclusive_scan_i32(s, num_pts, w.sel_scan, w.scan_scratch, w.num_selected);
    if (rc != MCCNN_OK) return rc;
    result = w.num_selected;
  }
  MCCNN_HIP_CHECK(hipMemcpyAsync(num_sampled_out_host, result, sizeof(int64_t),
                                 hipMemcpyDeviceToHost, s));
  MCCNN_HIP_CHECK(hipStreamSynchronize(s));
  return MCCNN_OK;
}

extern "C" int mccnn_sampling_fill(mccnn_stream_t stream, int mode, int64_t num_pts, int num_dims,
                                   const float *points, const int32_t *batch_ids,
                                   const int64_t *point_keys, const int32_t *num_cells,
                                   void *workspace, size_t workspace_bytes, int64_t num_sampled,
                                   float *sample_pts_out, int32_t *sample_batch_ids_out,
                                   int32_t *sample_indices_out) {
  MCCNN_REQUIRE(mode >= 0 && mode < 2, "Sampling requires a valid sampling mode");
  MCCNN_REQUIRE(valid_dims(num_dims), "Sampling expects a valid number of dimensions");
  MCCNN_REQUIRE(num_pts >= 0 && num_sampled >= 0 && num_sampled <= num_pts,
                "Sampling expects 0 <= num_sampled <= num_pts");
  if (num_pts == 0 || num_sampled == 0) return MCCNN_OK;
  MCCNN_REQUIRE(points && batch_ids && point_keys && num_cells && workspace && sample_pts_out &&
                    sample_batch_ids_out && sample_indices_out,
                "Sampling received a null tensor");
  const SamplingWorkspace w = carve_sampling_workspace(workspace, num_pts);
  MCCNN_REQUIRE(workspace_bytes >= w.bytes, "Sampling workspace too small (%zu < %zu)",
                workspace_bytes, w.bytes);
  hipStream_t s = as_stream(stream);
  if (mode == 0) {
    MCCNN_DIM_SWITCH(num_dims, hipLaunchKernelGGL(store_selected_kernel<D>,
                                                  dim3(blocks_for(num_pts, 256)), dim3(256), 0, s,
                                                  num_pts, points, batch_ids, w.used, w.sel_scan,
                                                  sample_pts_out, sample_batch_ids_out,
                                                  sample_indices_out));
  } else {
    MCCNN_DIM_SWITCH(num_dims, hipLaunchKernelGGL(cell_average_kernel<D>,
                                                  dim3(blocks_for(num_sampled, 256)), dim3(256), 0,
                                                  s, num_pts, num_sampled, points,
                                                  (const int64_t *)point_keys, num_cells,
                                                  w.first_idx, sample_pts_out,
                                                  sample_batch_ids_out, sample_indices_out));
  }
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}
