// Radius neighbour search on the sorted regular grid
// (custom_ops/tfg_custom_ops/find_neighbors/cc/ops/find_neighbors_ops.cpp:86-250).
//
// Three stages, all deterministic:
//   ranges  one lane per (centre, cell offset): the column of the 2-D table and
//           a binary search over the descending keys give the contiguous slice
//           of sorted points that lies in the offset cell row
//           (find_ranges_grid_ds_kernels.cu.cc:48-235);
//   count   8 lanes per centre stride over the slices and test
//           |(s - p) * inv_radii| < 1 (count_neighbors_kernels.cu.cc:83-86; as the
//           squared length against 1, which decides identically);
//   fill    same traversal; the slot of a hit is the centre's start offset plus
//           a ballot prefix inside the 8-lane group, so the pairs of a centre
//           come out in ascending sorted-point index without atomics or a sort.
// Offsets are enumerated so that the slices of a centre ascend in index.
// (Keeping the count pass's hit masks for the fill pass, so that it need not load
// and test the candidates again, was measured: what the count pass loses by
// storing them is what the fill pass gains, and crowded centres, whose masks do
// not fit a fixed budget, pay for both.  Letting the count pass find its slices
// itself, 9 of a group's 16 lanes searching, saves a launch and was no faster
// either.)
// Compiled with -ffp-contract=off (the distance test decides integer output).
#include "common.h"
#include "fill.h"

namespace mccnn {

// 8 lanes per centre: with the unreachable cells left out a slice holds one or two cells,
// and a wavefront steps through the union of what its centres need, so narrow groups
// waste fewer lanes (16 lanes: 7 % slower on the dense case, 10 % on clustered clouds;
// 32 lanes: 25 % slower).
constexpr int kGroup = 8;                  // lanes per centre
constexpr int kNbrThreads = 256;
constexpr int kCentresPerBlock = kNbrThreads / kGroup;

// Offsets act on dims 0..max(D-2,1); the last dim is covered by the key search.
template <int D>
struct OffsetInfo {
  static constexpr int kDims = (D - 2 > 1 ? D - 2 : 1) + 1;
  static constexpr int count() {
    int c = 1;
    for (int i = 0; i < kDims; ++i) c *= 3;
    return c;
  }
};

template <int D>
__global__ void __launch_bounds__(256) nbr_ranges_kernel(
    int64_t ns, const float *__restrict__ samples, const int *__restrict__ sbids,
    const int64_t *__restrict__ keys, const int2 *__restrict__ ds,
    const int *__restrict__ num_cells, const float *__restrict__ smin,
    const float *__restrict__ inv_cell, const float *__restrict__ inv_radii,
    int2 *__restrict__ ranges) {
  constexpr int R = OffsetInfo<D>::count();
  constexpr int OD = OffsetInfo<D>::kDims;
  const GridShape<D> g = load_shape<D>(num_cells);
  float ic[D], rho[D];                 // rho: one cell in units of the radius
#pragma unroll
  for (int d = 0; d < D; ++d) {
    ic[d] = inv_cell[d];
    rho[d] = inv_radii[d] / ic[d];
  }
  const int64_t total = ns * R;
  for (int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; t < total;
       t += (int64_t)gridDim.x * blockDim.x) {
    const int64_t c = t / R;
    int r = (int)(t - c * R);
    const int b = sbids[c];
    float p[D], m[D];
#pragma unroll
    for (int d = 0; d < D; ++d) {
      p[d] = samples[c * D + d];
      m[d] = smin[(int64_t)b * D + d];
    }
    int cell[D];
    cell_of_point<D>(p, m, ic, g, cell);
    // The centre in cell units, as the keys were computed, and what rounding can have
    // moved a point across a cell face: a point filed under cell x has a true
    // coordinate within `slack` of [x, x + 1) (outermost cells: unbounded outwards).
    float rel[D], slack[D];
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const float prod = p[d] * ic[d];
      rel[d] = prod - m[d];
      slack[d] = 9.6e-7f * (fabsf(prod) + fabsf(m[d]) + 1.0f);       // 8 float epsilons
    }
    // offset digits, most significant = dim 0, value 1 - digit (descending); g2 = lower
    // bound of the squared scaled distance to any point of the offset cell row, taken
    // over the offset dimensions
    bool inside = true;
    float g2 = 0.0f;
#pragma unroll
    for (int d = OD - 1; d >= 0; --d) {
      const int off = 1 - (r % 3);
      r /= 3;
      float gap = off < 0 ? rel[d] - (float)cell[d]
                          : (off > 0 ? (float)(cell[d] + 1) - rel[d] : 0.0f);
      gap = fmaxf(gap - slack[d], 0.0f) * rho[d];
      g2 += gap * gap;
      cell[d] += off;
      inside = inside && cell[d] >= 0 && cell[d] < g.n[d];
    }
    // Cells that no pair of the exact test can come from are left out: every candidate
    // dropped here has a scaled distance of at least sqrt(1 + 1e-5) > 1, whatever the
    // rounding of the test itself (a few 1e-7), so the pairs found do not change.
    g2 *= 0.99999f;
    inside = inside && g2 < 1.0f;
    int2 out = make_int2(0, 0);
    if (inside) {
      const int64_t col = ((int64_t)b * g.n[0] + cell[0]) * g.n[1] + cell[1];
      const int2 span = ds[col];
      if (span.y > span.x) {
        if (D == 2) {
          out = span;
        } else {
          const int64_t aux = key_of_cell<D>(cell, g, b);
          const int w = cell[D - 1], nw = g.n[D - 1];
          // last dimension: the cells w - 1 .. w + 1 of the reference, cut to those the
          // sphere can reach given the offset in the other dimensions (out-of-range
          // coordinates belong to the outermost cells)
          const float reach = sqrtf(1.0f - g2) / rho[D - 1] * 1.00001f + slack[D - 1];
          int wlo = (int)floorf(fmaxf(rel[D - 1] - reach, -1.0f));
          int whi = (int)floorf(fminf(rel[D - 1] + reach, (float)nw));
          wlo = wlo < 0 ? 0 : (wlo > nw - 1 ? nw - 1 : wlo);
          whi = whi < 0 ? 0 : (whi > nw - 1 ? nw - 1 : whi);
          wlo = wlo > w - 1 ? wlo : (w > 0 ? w - 1 : 0);
          whi = whi < w + 1 ? whi : (w < nw - 1 ? w + 1 : nw - 1);
          const int64_t maxk = aux + (whi - w);
          const int64_t mink = aux + (wlo - w);
          int lo = span.x, hi = span.y;
          while (lo < hi) {                       // first index with key <= maxk
            const int mid = lo + ((hi - lo) >> 1);
            if (keys[mid] > maxk) lo = mid + 1; else hi = mid;
          }
          const int first = lo;
          hi = span.y;
          while (lo < hi) {                       // first index with key < mink
            const int mid = lo + ((hi - lo) >> 1);
            if (keys[mid] >= mink) lo = mid + 1; else hi = mid;
          }
          if (lo > first && whi >= wlo) out = make_int2(first, lo);
        }
      }
    }
    ranges[t] = out;
  }
}

template <int D>
__device__ __forceinline__ bool within_radius(const float *s, const float *__restrict__ pts,
                                              int64_t j, const float *ir) {
  float acc = 0.0f;
#pragma unroll
  for (int d = 0; d < D; ++d) {
    const float diff = s[d] - pts[j * D + d];
    const float sc = diff * ir[d];
    const float sq = sc * sc;
    acc = acc + sq;
  }
  // The reference tests sqrtf(acc) < 1 (count_neighbors_kernels.cu.cc:83-86).  The
  // correctly rounded root is monotonic, sqrtf(1) = 1 and the root of the largest
  // float below 1 is again that float, so acc < 1 decides the same for every
  // float, infinities and NaN included, without the twenty instructions of an
  // IEEE square root per candidate.
  return acc < 1.0f;
}

// kFill == false: counts[c] = number of hits (clamped to max_neighs when > 0).
// kFill == true : writes the pairs of centre c starting at its start offset.
template <int D, bool kFill>
__global__ void __launch_bounds__(kNbrThreads) nbr_visit_kernel(
    int64_t ns, const float *__restrict__ samples, const float *__restrict__ pts,
    const int2 *__restrict__ ranges, const float *__restrict__ inv_radii, int max_neighs,
    int *__restrict__ counts, const int *__restrict__ ends, int2 *__restrict__ nbrs,
    int64_t *__restrict__ truncated = nullptr, int64_t capacity = ((int64_t)1 << 62)) {
  constexpr int R = OffsetInfo<D>::count();
  const int sub = threadIdx.x & (kGroup - 1);
  const int lane = lane_id();
  const uint64_t group_mask = ((1ull << kGroup) - 1ull) << (lane & ~(kGroup - 1));
  const uint64_t below_mask = group_mask & ((1ull << lane) - 1ull);
  float ir[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ir[d] = inv_radii[d];
  const int64_t c = (int64_t)blockIdx.x * kCentresPerBlock + threadIdx.x / kGroup;
  if (c >= ns) return;
  float s[D];
#pragma unroll
  for (int d = 0; d < D; ++d) s[d] = samples[c * D + d];
  const int limit = max_neighs > 0 ? max_neighs : 0x7fffffff;
  int found = 0;                                   // kFill: slots used so far
  int64_t start = 0;
  if (kFill) start = c > 0 ? ends[c - 1] : 0;
  // the slices of the centre, kGroup at a time: lane `sub` fetches one, the group then
  // takes them in turn (one round trip to memory instead of one per slice)
  for (int r0 = 0; r0 < R; r0 += kGroup) {
    const int2 mine = r0 + sub < R ? ranges[c * R + r0 + sub] : make_int2(0, 0);
    const int lim = R - r0 < kGroup ? R - r0 : kGroup;
    for (int r = 0; r < lim; ++r) {
      const int2 span = make_int2(__shfl(mine.x, r, kGroup), __shfl(mine.y, r, kGroup));
      for (int j0 = span.x; j0 < span.y; j0 += kGroup) {
        const int j = j0 + sub;
        const bool hit = j < span.y && within_radius<D>(s, pts, j, ir);
        if (kFill) {
          const uint64_t hits = __ballot(hit) & group_mask;
          const int slot = found + __popcll(hits & below_mask);
          if (hit && slot < limit && start + slot < capacity)
            nbrs[start + slot] = make_int2(j, (int)c);
          found += __popcll(hits);
        } else {
          found += hit ? 1 : 0;
        }
      }
    }
  }
  if (!kFill) {
#pragma unroll
    for (int off = kGroup / 2; off > 0; off >>= 1) found += __shfl_xor(found, off, kWave);
    if (sub == 0) {
      counts[c] = found < limit ? found : limit;
      // some centre lost pairs to max_neighs (every writer stores the same value)
      if (truncated && found > limit) *truncated = 1;
    }
  }
}

struct NbrWorkspace {
  int2 *ranges;
  int *scan_scratch;
  int64_t *total;
  size_t bytes;
};

static int offsets_for(int d) {
  int od = (d - 2 > 1 ? d - 2 : 1) + 1, c = 1;
  for (int i = 0; i < od; ++i) c *= 3;
  return c;
}

static NbrWorkspace carve_nbr_workspace(void *ws, int d, int64_t ns) {
  char *p = (char *)ws;
  NbrWorkspace w;
  size_t off = 0;
  w.ranges = (int2 *)(p + off);
  off += align256(sizeof(int2) * (size_t)ns * offsets_for(d));
  w.scan_scratch = (int *)(p + off);
  off += align256(sizeof(int) * scan_scratch_ints(ns));
  w.total = (int64_t *)(p + off);
  off += 256;
  w.bytes = off;
  return w;
}

// Pair table regrouped for another order of the centres: slot q takes the
// segment of centre order[q].  counts pass, then (after the scan) a copy pass
// with 16 lanes per slot; the centre column is rewritten to the slot.
__global__ void __launch_bounds__(256) segment_counts_kernel(int64_t n, const int *__restrict__ ranges,
                                                             const int *__restrict__ order,
                                                             int *__restrict__ counts) {
  const int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (q >= n) return;
  const int i = order[q];
  counts[q] = ranges[i] - (i > 0 ? ranges[i - 1] : 0);
}

__global__ void __launch_bounds__(256) segment_copy_kernel(int64_t n, const int *__restrict__ ranges,
                                                           const int *__restrict__ order,
                                                           const int2 *__restrict__ pairs,
                                                           const int *__restrict__ ranges_out,
                                                           int2 *__restrict__ pairs_out) {
  const int64_t q = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 4;
  if (q >= n) return;
  const int sub = threadIdx.x & 15;
  const int i = order[q];
  const int src = i > 0 ? ranges[i - 1] : 0, cnt = ranges[i] - src;
  const int dst = ranges_out[q] - cnt;
  for (int t = sub; t < cnt; t += 16) pairs_out[dst + t] = make_int2(pairs[src + t].x, (int)q);
}

}  // namespace mccnn

using namespace mccnn;

extern "C" size_t mccnn_find_neighbors_workspace_bytes(int num_dims, int64_t num_samples) {
  if (!valid_dims(num_dims) || num_samples < 0) return 0;
  return carve_nbr_workspace(nullptr, num_dims, num_samples).bytes;
}

// `facts_out_host` (optional, two values): [0] 1 if some centre lost pairs to max_neighs,
// [1] 1 if the centres are the searched points themselves (same address, same count).
static int find_neighbors_count_impl(
    mccnn_stream_t stream, int64_t num_samples, int num_dims, const float *samples,
    int64_t sample_batch_ids_len, const int32_t *sample_batch_ids, int64_t num_pts, int pts_dims,
    const float *points, int64_t point_keys_len, const int64_t *point_keys, int ds_rank,
    int ds_batch, int ds_nx, int ds_ny, int ds_last, const int32_t *grid_ds, int num_cells_len,
    const int32_t *num_cells, int aabb_dims, const float *scaled_aabb_min, int inv_cell_sizes_len,
    const float *inv_cell_sizes, int inv_radii_len, const float *inv_radii, int max_neighs,
    void *workspace, size_t workspace_bytes, int32_t *ranges_out,
    int64_t *num_neighbors_out_host, int64_t *facts_out_host, bool to_host = true) {
  int64_t unused_total = 0;
  if (!to_host) num_neighbors_out_host = &unused_total;   // the total stays in the workspace
  MCCNN_REQUIRE(valid_dims(num_dims), "FindNeighbors expects a valid number of dimensions");
  MCCNN_REQUIRE(num_cells_len == num_dims,
                "FindNeighbors expects a number of dimensions in num_cells equal to the number of "
                "dimensions in the input points");
  MCCNN_REQUIRE(pts_dims == num_dims,
                "FindNeighbors expects a number of dimensions in points equal to the number of "
                "dimensions in the samples");
  MCCNN_REQUIRE(aabb_dims == num_dims,
                "FindNeighbors expects a number of dimensions in scaled_aabb_min equal to the "
                "number of dimensions in the input points");
  MCCNN_REQUIRE(inv_cell_sizes_len == num_dims,
                "FindNeighbors expects a number of dimensions in inv_cell_sizes equal to the "
                "number of dimensions in the input points");
  MCCNN_REQUIRE(inv_radii_len == num_dims,
                "FindNeighbors expects a number of dimensions in inv_radii equal to the number of "
                "dimensions in the input points");
  MCCNN_REQUIRE(sample_batch_ids_len == num_samples,
                "FindNeighbors expects the same number of batch ids as samples");
  MCCNN_REQUIRE(point_keys_len == num_pts,
                "FindNeighbors expects the same number of keys as points");
  MCCNN_REQUIRE(ds_rank == 4 && ds_last == 2,
                "FindNeighbors expects a grid acceleration data structure with the right format "
                "(B, X, Y, 2)");
  MCCNN_REQUIRE(ds_batch > 0 && ds_nx > 0 && ds_ny > 0,
                "FindNeighbors expects a non-empty grid acceleration data structure");
  MCCNN_REQUIRE(num_samples >= 0 && num_pts >= 0 && num_samples < ((int64_t)1 << 31) &&
                    num_pts < ((int64_t)1 << 31),
                "FindNeighbors expects sizes in [0, 2^31)");
  MCCNN_REQUIRE(num_neighbors_out_host, "FindNeighbors received a null output");
  *num_neighbors_out_host = 0;
  if (facts_out_host) {
    facts_out_host[0] = 0;
    facts_out_host[1] = samples == points && num_samples == num_pts ? 1 : 0;
  }
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(samples && sample_batch_ids && grid_ds && num_cells && scaled_aabb_min &&
                    inv_cell_sizes && inv_radii && ranges_out && workspace,
                "FindNeighbors received a null tensor");
  MCCNN_REQUIRE(num_pts == 0 || (points && point_keys), "FindNeighbors received a null tensor");
  const NbrWorkspace w = carve_nbr_workspace(workspace, num_dims, num_samples);
  MCCNN_REQUIRE(workspace_bytes >= w.bytes, "FindNeighbors workspace too small (%zu < %zu)",
                workspace_bytes, w.bytes);
  hipStream_t s = as_stream(stream);
  const int64_t work = num_samples * offsets_for(num_dims);
  MCCNN_DIM_SWITCH(num_dims,
                   hipLaunchKernelGGL(nbr_ranges_kernel<D>, dim3(blocks_for(work, 256)), dim3(256),
                                      0, s, num_samples, samples, sample_batch_ids,
                                      (const int64_t *)point_keys, (const int2 *)grid_ds,
                                      num_cells, scaled_aabb_min, inv_cell_sizes, inv_radii,
                                      w.ranges));
  MCCNN_LAUNCH_CHECK();
  const unsigned grid = blocks_for(num_samples, kCentresPerBlock);
  // truncation can only happen with max_neighs > 0: only then is the flag cleared and read
  int64_t *truncated = facts_out_host && max_neighs > 0 ? w.total + 1 : nullptr;
  if (truncated) {
    int rc0 = fill_zero(s, truncated, sizeof(int64_t));
    if (rc0 != MCCNN_OK) return rc0;
  }
  MCCNN_DIM_SWITCH(num_dims, hipLaunchKernelGGL((nbr_visit_kernel<D, false>), dim3(grid),
                                                dim3(kNbrThreads), 0, s, num_samples, samples,
                                                points, (const int2 *)w.ranges, inv_radii,
                                                max_neighs, ranges_out, (const int *)nullptr,
                                                (int2 *)nullptr, truncated));
  MCCNN_LAUNCH_CHECK();
  int rc = inclusive_scan_i32(s, num_samples, ranges_out, w.scan_scratch, w.total);
  if (rc != MCCNN_OK) return rc;
  if (!to_host) return MCCNN_OK;
  MCCNN_HIP_CHECK(hipMemcpyAsync(num_neighbors_out_host, w.total, sizeof(int64_t),
                                 hipMemcpyDeviceToHost, s));
  if (truncated)
    MCCNN_HIP_CHECK(hipMemcpyAsync(facts_out_host, truncated, sizeof(int64_t),
                                   hipMemcpyDeviceToHost, s));
  MCCNN_HIP_CHECK(hipStreamSynchronize(s));
  // the scan saturates partial sums at 2^31 - 1, so a total from there on is a lower bound
  MCCNN_REQUIRE(*num_neighbors_out_host < (((int64_t)1 << 31) - 1),
                "FindNeighbors found at least %lld pairs; the int32 offsets of the op contract "
                "hold fewer than 2^31 - 1",
                (long long)*num_neighbors_out_host);
  return MCCNN_OK;
}

extern "C" int mccnn_find_neighbors_count(
    mccnn_stream_t stream, int64_t num_samples, int num_dims, const float *samples,
    int64_t sample_batch_ids_len, const int32_t *sample_batch_ids, int64_t num_pts, int pts_dims,
    const float *points, int64_t point_keys_len, const int64_t *point_keys, int ds_rank,
    int ds_batch, int ds_nx, int ds_ny, int ds_last, const int32_t *grid_ds, int num_cells_len,
    const int32_t *num_cells, int aabb_dims, const float *scaled_aabb_min, int inv_cell_sizes_len,
    const float *inv_cell_sizes, int inv_radii_len, const float *inv_radii, int max_neighs,
    void *workspace, size_t workspace_bytes, int32_t *ranges_out,
    int64_t *num_neighbors_out_host) {
  return find_neighbors_count_impl(
      stream, num_samples, num_dims, samples, sample_batch_ids_len, sample_batch_ids, num_pts,
      pts_dims, points, point_keys_len, point_keys, ds_rank, ds_batch, ds_nx, ds_ny, ds_last,
      grid_ds, num_cells_len, num_cells, aabb_dims, scaled_aabb_min, inv_cell_sizes_len,
      inv_cell_sizes, inv_radii_len, inv_radii, max_neighs, workspace, workspace_bytes, ranges_out,
      num_neighbors_out_host, nullptr);
}

extern "C" int mccnn_find_neighbors_count_facts(
    mccnn_stream_t stream, int64_t num_samples, int num_dims, const float *samples,
    int64_t sample_batch_ids_len, const int32_t *sample_batch_ids, int64_t num_pts, int pts_dims,
    const float *points, int64_t point_keys_len, const int64_t *point_keys, int ds_rank,
    int ds_batch, int ds_nx, int ds_ny, int ds_last, const int32_t *grid_ds, int num_cells_len,
    const int32_t *num_cells, int aabb_dims, const float *scaled_aabb_min, int inv_cell_sizes_len,
    const float *inv_cell_sizes, int inv_radii_len, const float *inv_radii, int max_neighs,
    void *workspace, size_t workspace_bytes, int32_t *ranges_out,
    int64_t *num_neighbors_out_host, int64_t *facts_out_host) {
  MCCNN_REQUIRE(facts_out_host, "FindNeighbors received a null output");
  return find_neighbors_count_impl(
      stream, num_samples, num_dims, samples, sample_batch_ids_len, sample_batch_ids, num_pts,
      pts_dims, points, point_keys_len, point_keys, ds_rank, ds_batch, ds_nx, ds_ny, ds_last,
      grid_ds, num_cells_len, num_cells, aabb_dims, scaled_aabb_min, inv_cell_sizes_len,
      inv_cell_sizes, inv_radii_len, inv_radii, max_neighs, workspace, workspace_bytes, ranges_out,
      num_neighbors_out_host, facts_out_host);
}

extern "C" int mccnn_find_neighbors_fill(
    mccnn_stream_t stream, int64_t num_samples, int num_dims, const float *samples,
    const int32_t *sample_batch_ids, int64_t num_pts, const float *points,
    const int64_t *point_keys, const int32_t *grid_ds, const int32_t *num_cells,
    const float *scaled_aabb_min, const float *inv_cell_sizes, const float *inv_radii,
    int max_neighs, void *workspace, size_t workspace_bytes, const int32_t *ranges,
    int64_t num_neighbors, int32_t *neighbors_out) {
  (void)sample_batch_ids; (void)point_keys; (void)grid_ds; (void)num_cells;
  (void)scaled_aabb_min; (void)inv_cell_sizes; (void)num_pts;
  MCCNN_REQUIRE(valid_dims(num_dims), "FindNeighbors expects a valid number of dimensions");
  MCCNN_REQUIRE(num_samples >= 0 && num_neighbors >= 0, "FindNeighbors expects non-negative sizes");
  if (num_samples == 0 || num_neighbors == 0) return MCCNN_OK;
  MCCNN_REQUIRE(samples && points && inv_radii && ranges && neighbors_out && workspace,
                "FindNeighbors received a null tensor");
  const NbrWorkspace w = carve_nbr_workspace(workspace, num_dims, num_samples);
  MCCNN_REQUIRE(workspace_bytes >= w.bytes, "FindNeighbors workspace too small (%zu < %zu)",
                workspace_bytes, w.bytes);
  const unsigned grid = blocks_for(num_samples, kCentresPerBlock);
  MCCNN_DIM_SWITCH(num_dims, hipLaunchKernelGGL((nbr_visit_kernel<D, true>), dim3(grid),
                                                dim3(kNbrThreads), 0, as_stream(stream),
                                                num_samples, samples, points,
                                                (const int2 *)w.ranges, inv_radii, max_neighs,
                                                (int *)nullptr, ranges, (int2 *)neighbors_out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

// count_out[0] = pairs found, count_out[1] = 1 if they do not fit the capacity
__global__ void publish_neighbor_count_kernel(const int64_t *__restrict__ total, int64_t capacity,
                                              int64_t *__restrict__ count_out) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    count_out[0] = *total;
    count_out[1] = *total > capacity ? 1 : 0;
  }
}

extern "C" int mccnn_find_neighbors_bounded(
    mccnn_stream_t stream, int64_t num_samples, int num_dims, const float *samples,
    const int32_t *sample_batch_ids, int64_t num_pts, const float *points,
    const int64_t *point_keys, int ds_batch, int ds_nx, int ds_ny, const int32_t *grid_ds,
    const int32_t *num_cells, const float *scaled_aabb_min, const float *inv_cell_sizes,
    const float *inv_radii, int max_neighs, void *workspace, size_t workspace_bytes,
    int64_t capacity, int32_t *ranges_out, int32_t *neighbors_out, int64_t *count_out_device) {
  MCCNN_REQUIRE(capacity >= 0 && capacity < ((int64_t)1 << 31),
                "find_neighbors_bounded expects a capacity in [0, 2^31)");
  MCCNN_REQUIRE(count_out_device && (capacity == 0 || neighbors_out),
                "find_neighbors_bounded received a null output");
  int rc = find_neighbors_count_impl(
      stream, num_samples, num_dims, samples, num_samples, sample_batch_ids, num_pts, num_dims,
      points, num_pts, point_keys, 4, ds_batch, ds_nx, ds_ny, 2, grid_ds, num_dims, num_cells,
      num_dims, scaled_aabb_min, num_dims, inv_cell_sizes, num_dims, inv_radii, max_neighs,
      workspace, workspace_bytes, ranges_out, nullptr, nullptr, false);
  if (rc != MCCNN_OK) return rc;
  hipStream_t s = as_stream(stream);
  if (num_samples == 0) return fill_zero(s, count_out_device, 2 * sizeof(int64_t));
  const NbrWorkspace w = carve_nbr_workspace(workspace, num_dims, num_samples);
  hipLaunchKernelGGL(publish_neighbor_count_kernel, dim3(1), dim3(64), 0, s, w.total, capacity,
                     count_out_device);
  MCCNN_LAUNCH_CHECK();
  if (capacity == 0) return MCCNN_OK;
  const unsigned grid = blocks_for(num_samples, kCentresPerBlock);
  MCCNN_DIM_SWITCH(num_dims, hipLaunchKernelGGL((nbr_visit_kernel<D, true>), dim3(grid),
                                                dim3(kNbrThreads), 0, s, num_samples, samples,
                                                points, (const int2 *)w.ranges, inv_radii,
                                                max_neighs, (int *)nullptr, ranges_out,
                                                (int2 *)neighbors_out, (int64_t *)nullptr,
                                                capacity));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" size_t mccnn_reorder_neighbors_workspace_bytes(int64_t num_samples) {
  if (num_samples < 0) return 0;
  return align256(sizeof(int) * scan_scratch_ints(num_samples)) + align256(sizeof(int64_t));
}

extern "C" int mccnn_reorder_neighbors(mccnn_stream_t stream, int64_t num_samples,
                                       const int32_t *ranges, int64_t num_neighbors,
                                       const int32_t *neighbors, const int32_t *centre_order,
                                       void *workspace, size_t workspace_bytes,
                                       int32_t *ranges_out, int32_t *neighbors_out) {
  MCCNN_REQUIRE(num_samples >= 0 && num_neighbors >= 0 && num_neighbors < ((int64_t)1 << 31),
                "reorder_neighbors expects sizes in [0, 2^31)");
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(ranges && centre_order && ranges_out && workspace &&
                    (num_neighbors == 0 || (neighbors && neighbors_out)),
                "reorder_neighbors received a null tensor");
  MCCNN_REQUIRE(workspace_bytes >= mccnn_reorder_neighbors_workspace_bytes(num_samples),
                "reorder_neighbors workspace too small");
  hipStream_t s = as_stream(stream);
  int *scratch = (int *)workspace;
  int64_t *total = (int64_t *)((char *)workspace +
                               align256(sizeof(int) * scan_scratch_ints(num_samples)));
  hipLaunchKernelGGL(segment_counts_kernel, dim3(blocks_for(num_samples, 256)), dim3(256), 0, s,
                     num_samples, ranges, centre_order, ranges_out);
  MCCNN_LAUNCH_CHECK();
  int rc = inclusive_scan_i32(s, num_samples, ranges_out, scratch, total);
  if (rc != MCCNN_OK) return rc;
  if (num_neighbors == 0) return MCCNN_OK;
  hipLaunchKernelGGL(segment_copy_kernel, dim3(blocks_for(num_samples * 16, 256)), dim3(256), 0, s,
                     num_samples, ranges, centre_order, (const int2 *)neighbors, ranges_out,
                     (int2 *)neighbors_out);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}
