/*
 * mccnn_hip.h - C ABI of libmccnn_hip.so, the gfx950 implementation of the
 * Monte-Carlo point-cloud convolution ops.
 *
 * Each entry point replaces one registered op of the reference's native package
 * (custom_ops/tfg_custom_ops) or one piece of caller glue around it; the
 * reference interface it stands for is cited above each declaration.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name ends in _host;
 *     tensors are row-major and contiguous; float = fp32, keys = int64,
 *     indices = int32.  The small per-dimension vectors (num_cells,
 *     inv_cell_sizes, inv_radii, inv_bandwidth) are device tensors as they are
 *     in the reference ops.
 *   - every tensor argument is preceded by the extents the reference op
 *     validates, so the same shape errors can be reported.
 *   - all work is enqueued on `stream` (a hipStream_t).  Only the *_count entry
 *     points, which return a size the caller must allocate, synchronise the
 *     stream (once); nothing else blocks.
 *   - the library never allocates device memory: ops that need scratch take a
 *     caller-owned workspace whose size the matching *_workspace_bytes function
 *     returns.  Workspace contents are private to the library between a
 *     *_count call and the *_fill call that follows it.
 *   - "ranges" are inclusive end offsets: the pairs of centre i are rows
 *     [ranges[i-1], ranges[i]) of the neighbour table, ranges[-1] == 0.
 *   - return value: MCCNN_OK, MCCNN_INVALID_ARGUMENT (shape / attribute
 *     violation; the reference raises errors::InvalidArgument) or
 *     MCCNN_HIP_ERROR (the reference prints and exits,
 *     shared/cc/kernels/tf_gpu_device.cpp:89-100).  mccnn_last_error() returns
 *     the message of the calling thread's last failure.
 *   - re-entrant: no mutable global state; calls on different streams may
 *     overlap.
 */
#ifndef MCCNN_HIP_H_
#define MCCNN_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *mccnn_stream_t; /* hipStream_t */

#define MCCNN_OK 0
#define MCCNN_INVALID_ARGUMENT 1
#define MCCNN_HIP_ERROR 2

#define MCCNN_MIN_DIMENSIONS 2 /* shared/cc/kernels/defines.hpp:25 */
#define MCCNN_MAX_DIMENSIONS 6 /* shared/cc/kernels/defines.hpp:26 */

const char *mccnn_last_error(void);
int mccnn_abi_version(void);

/* ---------------------------------------------------------------- grid ---- */

/* ComputeKeys: compute_keys/cc/ops/compute_keys_ops.cpp:29-121.
 * keys_out[i] = batch_id * prod(num_cells) + row-major index of
 * clamp(floor(p * inv_cell_sizes - scaled_aabb_min[batch_id]), 0, num_cells-1). */
int mccnn_compute_keys(mccnn_stream_t stream, int64_t num_pts, int num_dims,
                       const float *points, int64_t batch_ids_len,
                       const int32_t *batch_ids, int64_t aabb_rows, int aabb_dims,
                       const float *scaled_aabb_min, int num_cells_len,
                       const int32_t *num_cells, int inv_cell_sizes_len,
                       const float *inv_cell_sizes, int64_t *keys_out);

/* The sort step of pylib/pc/Grid.py:56-64 (tf.argsort(keys, 'DESCENDING') and
 * the gathers): stable descending sort, equal keys keep ascending original
 * index.  key_bits = number of significant key bits (keys < 2^key_bits),
 * 1..64.  sorted_keys_out / sorted_indices_out must not alias the inputs. */
size_t mccnn_sort_keys_workspace_bytes(int64_t num_pts);
int mccnn_sort_keys_descending(mccnn_stream_t stream, int64_t num_pts,
                               int key_bits, const int64_t *keys,
                               int64_t *sorted_keys_out,
                               int32_t *sorted_indices_out, void *workspace,
                               size_t workspace_bytes);
int mccnn_gather_points(mccnn_stream_t stream, int64_t num_pts, int num_dims,
                        const float *points, const int32_t *batch_ids,
                        const int32_t *indices, float *points_out,
                        int32_t *batch_ids_out);

/* Per-cloud bounding box, grid shape and op inputs derived from them, the
 * caller glue of pylib/pc/PointCloud.py:38-43, pylib/pc/Grid.py:44-48 and
 * pylib/pc/custom_ops/custom_ops_wrapper.py:37-43:
 *   aabb_min/max_out [B,D] = segment min/max -/+ 1e-9f
 *   num_cells_out [D]      = max(1, max_b ceil((max-min)/cell_sizes))
 *   scaled_aabb_min_out    = aabb_min / cell_sizes
 *   inv_cell_sizes_out     = 1 / cell_sizes
 * cell_sizes is a device vector [D]. */
int mccnn_grid_setup(mccnn_stream_t stream, int64_t num_pts, int num_dims,
                     const float *points, const int32_t *batch_ids,
                     int batch_size, const float *cell_sizes,
                     float *aabb_min_out, float *aabb_max_out,
                     int32_t *num_cells_out, float *scaled_aabb_min_out,
                     float *inv_cell_sizes_out);

/* The whole grid of pylib/pc/Grid.py:32-64 in one call: mccnn_grid_setup,
 * mccnn_compute_keys, the host copy of the grid shape (one synchronisation of the
 * stream; num_cells_out_host [D] and *key_bits_out_host are host memory),
 * mccnn_sort_keys_descending with that key width, mccnn_gather_points.  Same outputs
 * as the five calls; for small clouds, whose cost is the calls and launches
 * themselves.  Workspace: mccnn_build_grid_workspace_bytes(num_pts). */
size_t mccnn_build_grid_workspace_bytes(int64_t num_pts);
int mccnn_build_grid(mccnn_stream_t stream, int64_t num_pts, int num_dims,
                     const float *points, const int32_t *batch_ids, int batch_size,
                     const float *cell_sizes, float *aabb_min_out, float *aabb_max_out,
                     int32_t *num_cells_out, float *scaled_aabb_min_out,
                     float *inv_cell_sizes_out, int64_t *keys_out,
                     int64_t *sorted_keys_out, int32_t *sorted_indices_out,
                     float *sorted_points_out, int32_t *sorted_batch_ids_out,
                     void *workspace, size_t workspace_bytes,
                     int32_t *num_cells_out_host, int *key_bits_out_host);

/* Small gathers of the caller glue:
 *   original ids  out[m] = (sorted_indices[neighbors[m,0]], neighbors[m,1])
 *                 pylib/pc/Neighborhood.py:246-250
 *   pdf per pair  out[m] = pdf[neighbors[m,0]]   pylib/pc/Neighborhood.py:287
 *                 (_column: of either column, for the transposed pair table)
 *   swapped pairs out[i] = (neighbors[order[i],1], neighbors[order[i],0]): the rows of
 *                 the transposed pair table from the order mccnn_transpose_neighbors
 *                 returns (no counterpart: the reference searches again, Neighborhood.py:318-329)
 *   int32 gather  out[i] = src[indices[i]]       pylib/pc/sampling.py:142-146
 *   row gather    out[i,:] = src[indices[i],:]   (tf.gather of feature rows, e.g.
 *                 pylib/pc/layers/utils.py:47; num_cols a multiple of 4, rows 16-byte aligned) */
int mccnn_original_neighbor_ids(mccnn_stream_t stream, int64_t num_neighbors,
                                const int32_t *neighbors,
                                const int32_t *sorted_indices,
                                int32_t *original_neighbors_out);
int mccnn_gather_pdf(mccnn_stream_t stream, int64_t num_neighbors,
                     const int32_t *neighbors, const float *pdf,
                     float *pdf_per_pair_out);
int mccnn_swapped_pairs(mccnn_stream_t stream, int64_t num_neighbors,
                        const int32_t *neighbors, const int32_t *pair_order,
                        int32_t *swapped_out);
int mccnn_gather_pdf_column(mccnn_stream_t stream, int64_t num_neighbors,
                            const int32_t *neighbors, int column, const float *pdf,
                            float *pdf_per_pair_out);
int mccnn_gather_i32(mccnn_stream_t stream, int64_t count, const int32_t *src,
                     const int32_t *indices, int32_t *out);
int mccnn_gather_rows(mccnn_stream_t stream, int64_t num_rows, int num_cols, const float *src,
                      const int32_t *indices, float *out);

/* BuildGridDs: build_grid_ds/cc/ops/build_grid_ds_ops.cpp:27-115.
 * ds_out is int32 [batch_size, num_cells[0], num_cells[1], 2]: (first, last+1)
 * index of each column in the sorted arrays, (0,0) when empty.  num_cells is
 * passed twice as in the reference: device copy and host copy. */
int mccnn_build_grid_ds(mccnn_stream_t stream, int64_t num_pts,
                        const int64_t *sorted_keys, int num_cells_len,
                        const int32_t *num_cells, int num_cells_host_len,
                        const int32_t *num_cells_host, int batch_size,
                        int32_t *ds_out);

/* ----------------------------------------------------------- neighbours --- */

/* FindNeighbors: find_neighbors/cc/ops/find_neighbors_ops.cpp:42-259, split
 * where the reference synchronises to size its second output
 * (find_neighbors/cc/kernels/scan_alg_kernels.cu.cc:259-265).
 *
 * _count writes ranges_out [num_samples] (inclusive end offsets), stores
 * the total pair count in *num_neighbors_out_host and synchronises `stream`.
 * _fill writes neighbors_out [M,2] rows (sorted point index, centre index),
 * grouped by centre, ascending point index inside a centre.
 * max_neighs > 0 keeps the first max_neighs pairs of each centre in that order
 * (the reference picks a wall-clock-seeded random subset,
 * store_neighbors_kernels.cu.cc:216). */
size_t mccnn_find_neighbors_workspace_bytes(int num_dims, int64_t num_samples);
int mccnn_find_neighbors_count(
    mccnn_stream_t stream, int64_t num_samples, int num_dims,
    const float *samples, int64_t sample_batch_ids_len,
    const int32_t *sample_batch_ids, int64_t num_pts, int pts_dims,
    const float *points, int64_t point_keys_len, const int64_t *point_keys,
    int ds_rank, int ds_batch, int ds_nx, int ds_ny, int ds_last,
    const int32_t *grid_ds, int num_cells_len, const int32_t *num_cells,
    int aabb_dims, const float *scaled_aabb_min, int inv_cell_sizes_len,
    const float *inv_cell_sizes, int inv_radii_len, const float *inv_radii,
    int max_neighs, void *workspace, size_t workspace_bytes,
    int32_t *ranges_out, int64_t *num_neighbors_out_host);
/* _count with two facts about the table it sizes, read back in the same synchronisation:
 * facts_out_host[0] = 1 if some centre lost pairs to max_neighs, [1] = 1 if the centres are
 * the searched points themselves (same address and count).  With [0] == 0 and [1] == 1 the
 * table is symmetric (j in N(c) <=> c in N(j)) and mccnn_compute_pdf_pt_grads_symmetric
 * applies.  No counterpart in the reference. */
int mccnn_find_neighbors_count_facts(
    mccnn_stream_t stream, int64_t num_samples, int num_dims,
    const float *samples, int64_t sample_batch_ids_len,
    const int32_t *sample_batch_ids, int64_t num_pts, int pts_dims,
    const float *points, int64_t point_keys_len, const int64_t *point_keys,
    int ds_rank, int ds_batch, int ds_nx, int ds_ny, int ds_last,
    const int32_t *grid_ds, int num_cells_len, const int32_t *num_cells,
    int aabb_dims, const float *scaled_aabb_min, int inv_cell_sizes_len,
    const float *inv_cell_sizes, int inv_radii_len, const float *inv_radii,
    int max_neighs, void *workspace, size_t workspace_bytes,
    int32_t *ranges_out, int64_t *num_neighbors_out_host,
    int64_t *facts_out_host);
/* The search without a host round trip, for callers that enqueue a whole step (or record it
 * in a HIP graph): count, scan and fill in one call on the stream.  The pair table has room
 * for `capacity` rows; pairs beyond it are dropped, ranges_out holds the true end offsets,
 * count_out_device[0] the true number of pairs and count_out_device[1] 1 if it exceeds the
 * capacity (the caller checks that flag when it next reads from the device, e.g. once per
 * step).  Rows [0, min(count, capacity)) equal those of the _count / _fill pair; the rest of
 * the table is not written.  Same workspace as _count.  No counterpart in the reference,
 * whose op returns a tensor of the exact size (find_neighbors_ops.cpp:217-259). */
int mccnn_find_neighbors_bounded(
    mccnn_stream_t stream, int64_t num_samples, int num_dims,
    const float *samples, const int32_t *sample_batch_ids, int64_t num_pts,
    const float *points, const int64_t *point_keys, int ds_batch, int ds_nx,
    int ds_ny, const int32_t *grid_ds, const int32_t *num_cells,
    const float *scaled_aabb_min, const float *inv_cell_sizes,
    const float *inv_radii, int max_neighs, void *workspace,
    size_t workspace_bytes, int64_t capacity, int32_t *ranges_out,
    int32_t *neighbors_out, int64_t *count_out_device);
int mccnn_find_neighbors_fill(
    mccnn_stream_t stream, int64_t num_samples, int num_dims,
    const float *samples, const int32_t *sample_batch_ids, int64_t num_pts,
    const float *points, const int64_t *point_keys, const int32_t *grid_ds,
    const int32_t *num_cells, const float *scaled_aabb_min,
    const float *inv_cell_sizes, const float *inv_radii, int max_neighs,
    void *workspace, size_t workspace_bytes, const int32_t *ranges,
    int64_t num_neighbors, int32_t *neighbors_out);

/* ------------------------------------------------------------------ pdf --- */

/* ComputePdf / ComputePdfWithPtGrads: compute_pdf/cc/ops/compute_pdf_ops.cpp:28-161.
 * pdf_out[i] = sum over the pairs of centre i of
 *   prod_d bw_d * exp(-0.5 * ((p_j - p_i)_d * bw_d * inv_radii_d)^2) * 0.39894228
 * with bw = inv_bandwidth (mode 0) or sqrt(num_pts) (mode 1, as the reference
 * computes it).  Centres are the points themselves: num_samples == num_pts. */
int mccnn_compute_pdf(mccnn_stream_t stream, int64_t num_pts, int num_dims,
                      const float *points, int64_t num_neighbors,
                      int neighbors_rank, int neighbors_cols,
                      const int32_t *neighbors, int64_t num_samples,
                      const int32_t *ranges, int inv_bandwidth_len,
                      const float *inv_bandwidth, int inv_radii_len,
                      const float *inv_radii, int mode, float *pdf_out);

/* ComputePdfPtGrads: compute_pdf/cc/ops/compute_pdf_ops.cpp:163-259.
 * pt_grads_out [num_pts, D] = d(sum_i pdf_grads_i * pdf_i) / d(points).  The table must be
 * a self-neighbourhood (centre c is point c: num_samples == num_pts, as the op requires,
 * compute_pdf_ops.cpp:205-207) in which no pair occurs twice -- what find_neighbors writes,
 * truncated by max_neighs or not, in any order inside a centre.  Where the reverse of a
 * pair is in the table too (always, in an untruncated self-neighbourhood) its term is
 * gathered instead of scattered, so atomics are used only for pairs without a reverse.
 * (A repeated pair would be gathered once per occurrence of its reverse; the reference's
 * atomics weight every occurrence.) */
int mccnn_compute_pdf_pt_grads(mccnn_stream_t stream, int64_t num_pts,
                               int num_dims, const float *points,
                               int64_t num_neighbors, int neighbors_rank,
                               int neighbors_cols, const int32_t *neighbors,
                               int64_t num_samples, const int32_t *ranges,
                               int inv_bandwidth_len, const float *inv_bandwidth,
                               int inv_radii_len, const float *inv_radii,
                               int64_t pdf_grads_len, const float *pdf_grads,
                               int mode, float *pt_grads_out);

/* ComputePdfPtGrads for a symmetric pair table (j in N(c) <=> c in N(j)), which
 * an untruncated self-neighbourhood is: the same gradient as a pure gather,
 *   grad[c] = sum_{j in N(c)} (pdf_grads_c + pdf_grads_j) * d k_cj / d x_c,
 * without atomics and in a fixed summation order.  The caller vouches for the
 * symmetry; same arguments as mccnn_compute_pdf_pt_grads.  No counterpart in
 * the reference, whose kernel scatters with atomics
 * (compute_pdf_kernels.cu.cc:193-199). */
int mccnn_compute_pdf_pt_grads_symmetric(
    mccnn_stream_t stream, int64_t num_pts, int num_dims, const float *points,
    int64_t num_neighbors, int neighbors_rank, int neighbors_cols,
    const int32_t *neighbors, int64_t num_samples, const int32_t *ranges,
    int inv_bandwidth_len, const float *inv_bandwidth, int inv_radii_len,
    const float *inv_radii, int64_t pdf_grads_len, const float *pdf_grads,
    int mode, float *pt_grads_out);

/* ----------------------------------------------------------- basis_proj --- */

/* BasisProj: basis_proj/cc/ops/basis_proj_ops.cpp:25-131.
 * out [num_samples, C, K]: out[i,c,k] = sum_m features[neighbors[m,0], c] *
 * basis[m,k] over the pairs m of centre i.  K in {8,16,32,64}; C < 8 or a
 * multiple of 8.  neighbors[:,0] indexes `features` (original point ids). */
int mccnn_basis_proj(mccnn_stream_t stream, int64_t basis_rows, int num_basis,
                     const float *basis, int64_t num_pts, int num_features,
                     const float *features, int64_t num_neighbors,
                     int neighbors_rank, int neighbors_cols,
                     const int32_t *neighbors, int64_t num_samples,
                     const int32_t *ranges, float *out);

/* BasisProjGrads: basis_proj/cc/ops/basis_proj_ops.cpp:133-227.
 * basis_grads_out [M,K], feature_grads_out [num_pts, C] for upstream gradient
 * in_grads [num_samples, C, K] (its three extents are validated). */
int mccnn_basis_proj_grads(mccnn_stream_t stream, int64_t basis_rows,
                           int num_basis, const float *basis, int64_t num_pts,
                           int num_features, const float *features,
                           int64_t num_neighbors, int neighbors_rank,
                           int neighbors_cols, const int32_t *neighbors,
                           int64_t num_samples, const int32_t *ranges,
                           int in_grads_rank, int64_t in_grads_dim0,
                           int64_t in_grads_dim1, int64_t in_grads_dim2,
                           const float *in_grads, float *basis_grads_out,
                           float *feature_grads_out);

/* The two ops above with a visiting order for the centres: centre_order
 * [num_samples] is a permutation of the centre indices (NULL = natural order).
 * Results are identical; only the schedule changes.  Passing the centres in
 * spatial order (e.g. sorted by grid cell key) keeps the feature rows shared by
 * neighbouring centres in L2.  No counterpart in the reference, whose kernels
 * always walk the centres in index order. */
int mccnn_basis_proj_ordered(mccnn_stream_t stream, int64_t basis_rows,
                             int num_basis, const float *basis, int64_t num_pts,
                             int num_features, const float *features,
                             int64_t num_neighbors, int neighbors_rank,
                             int neighbors_cols, const int32_t *neighbors,
                             int64_t num_samples, const int32_t *ranges,
                             const int32_t *centre_order, float *out);
int mccnn_basis_proj_grads_ordered(
    mccnn_stream_t stream, int64_t basis_rows, int num_basis, const float *basis,
    int64_t num_pts, int num_features, const float *features,
    int64_t num_neighbors, int neighbors_rank, int neighbors_cols,
    const int32_t *neighbors, int64_t num_samples, const int32_t *ranges,
    const int32_t *centre_order, int in_grads_rank, int64_t in_grads_dim0,
    int64_t in_grads_dim1, int64_t in_grads_dim2, const float *in_grads,
    float *basis_grads_out, float *feature_grads_out);

/* Pair lists grouped by neighbour point, the transposed view of a pair table:
 * point_ranges_out [num_pts] (inclusive end offsets) and pair_order_out [M], the
 * pair indices sorted by neighbours[:,0], ties in ascending pair index.  No
 * counterpart in the reference (whose backward scatters with atomics); it is
 * built once per neighbourhood and reused by every backward pass. */
size_t mccnn_transpose_neighbors_workspace_bytes(int64_t num_neighbors,
                                                 int64_t num_pts);
int mccnn_transpose_neighbors(mccnn_stream_t stream, int64_t num_neighbors,
                              const int32_t *neighbors, int64_t num_pts,
                              void *workspace, size_t workspace_bytes,
                              int32_t *point_ranges_out, int32_t *pair_order_out);

/* The pair table regrouped for another order of the centres: slot q of the
 * outputs holds the pairs of centre centre_order[q] (centre_order is a
 * permutation of 0..num_samples-1), in their original order, with the centre
 * column rewritten to q; ranges_out are the inclusive end offsets per slot.
 * With centre_order = the centres sorted by grid cell this gives the table in
 * which neighbouring slots share their neighbours, the layout the layer kernels
 * run on.  No counterpart in the reference. */
size_t mccnn_reorder_neighbors_workspace_bytes(int64_t num_samples);
int mccnn_reorder_neighbors(mccnn_stream_t stream, int64_t num_samples,
                            const int32_t *ranges, int64_t num_neighbors,
                            const int32_t *neighbors, const int32_t *centre_order,
                            void *workspace, size_t workspace_bytes,
                            int32_t *ranges_out, int32_t *neighbors_out);

/* BasisProjGrads without atomics: the feature gradient of each pair is written
 * to pair_rows_workspace [M, C] and then summed per point over the lists of
 * mccnn_transpose_neighbors, in a fixed order (bit-reproducible, unlike the
 * atomic scatter of the reference, basis_proj_grads_kernels.cu.cc:120-140).
 * K in {16, 32}, C in {16, 32, 64, 128} (C >= 32 for K = 32). */
int mccnn_basis_proj_grads_gathered(
    mccnn_stream_t stream, int64_t basis_rows, int num_basis, const float *basis,
    int64_t num_pts, int num_features, const float *features,
    int64_t num_neighbors, int neighbors_rank, int neighbors_cols,
    const int32_t *neighbors, int64_t num_samples, const int32_t *ranges,
    int in_grads_rank, int64_t in_grads_dim0, int64_t in_grads_dim1,
    int64_t in_grads_dim2, const float *in_grads, const int32_t *point_ranges,
    const int32_t *pair_order, float *pair_rows_workspace,
    float *basis_grads_out, float *feature_grads_out);

/* ------------------------------------------------------------- sampling --- */

/* Sampling: sampling/cc/ops/sampling_ops.cpp:33-204, split at the host
 * synchronisation that sizes the outputs.  mode 0 = Poisson disk (2^D cell
 * parity passes, count_sampling_pd_kernels.cu.cc:156-181), mode 1 = cell average.
 * Inputs are the SORTED points / batch ids / keys and the self-neighbourhood.
 * _count stores S in *num_sampled_out_host and synchronises; _fill writes
 * sample_pts_out [S,D], sample_batch_ids_out [S], sample_indices_out [S]
 * (mode 0: selected sorted indices, ascending; mode 1: first sorted index of
 * each occupied cell, cells in sorted-key order). */
size_t mccnn_sampling_workspace_bytes(int64_t num_pts);
int mccnn_sampling_count(mccnn_stream_t stream, int mode, int64_t num_pts,
                         int num_dims, const float *points,
                         int64_t batch_ids_len, const int32_t *batch_ids,
                         int64_t point_keys_len, const int64_t *point_keys,
                         int num_cells_len, const int32_t *num_cells,
                         int64_t num_neighbors, int neighbors_rank,
                         int neighbors_cols, const int32_t *neighbors,
                         int64_t ranges_len, const int32_t *ranges,
                         void *workspace, size_t workspace_bytes,
                         int64_t *num_sampled_out_host);
int mccnn_sampling_fill(mccnn_stream_t stream, int mode, int64_t num_pts,
                        int num_dims, const float *points,
                        const int32_t *batch_ids, const int64_t *point_keys,
                        const int32_t *num_cells, void *workspace,
                        size_t workspace_bytes, int64_t num_sampled,
                        float *sample_pts_out, int32_t *sample_batch_ids_out,
                        int32_t *sample_indices_out);

/* -------------------------------------------------------------- pooling --- */

/* Local pooling over neighbourhoods, pylib/pc/layers/Pooling.py:107-166
 * (tf.math.unsorted_segment_max / _mean over the pairs).  kind 0 = max,
 * 1 = average.  out [num_samples, C]; a centre without pairs gets -FLT_MAX
 * (max) or 0 (average), as the TensorFlow segment ops give.  neighbors holds
 * ORIGINAL point ids in column 0. */
int mccnn_local_pool(mccnn_stream_t stream, int kind, int64_t num_pts,
                     int num_features, const float *features,
                     int64_t num_neighbors, const int32_t *neighbors,
                     int64_t num_samples, const int32_t *ranges, float *out);

/* Gradient of the above.  Max: every pair whose feature equals the pooled value
 * receives out_grads / (number of such pairs), the rule of TensorFlow's
 * unsorted_segment_max gradient; average: out_grads / (pairs of the centre).
 * `out` is the forward result.  feature_grads_out [num_pts, C] is overwritten. */
int mccnn_local_pool_grads(mccnn_stream_t stream, int kind, int64_t num_pts,
                           int num_features, const float *features,
                           int64_t num_neighbors, const int32_t *neighbors,
                           int64_t num_samples, const int32_t *ranges,
                           const float *out, const float *out_grads,
                           float *feature_grads_out);

/* Global pooling per cloud, pylib/pc/layers/Pooling.py:25-104.  out [B, C];
 * counts_out [B] (int32) receives the number of points of each cloud. */
int mccnn_global_pool(mccnn_stream_t stream, int kind, int64_t num_pts,
                      int num_features, const float *features,
                      const int32_t *batch_ids, int batch_size, float *out,
                      int32_t *counts_out);
/* Gradient of the above with the tie rule of mccnn_local_pool_grads.
 * tie_workspace is [B, C] floats of scratch (kind 0 only, may be NULL for 1). */
int mccnn_global_pool_grads(mccnn_stream_t stream, int kind, int64_t num_pts,
                            int num_features, const float *features,
                            const int32_t *batch_ids, int batch_size,
                            const float *out, const int32_t *counts,
                            const float *out_grads, float *tie_workspace,
                            float *feature_grads_out);

/* --------------------------------------------------- layer composition --- */

#define MCCNN_ACT_RELU 0
#define MCCNN_ACT_LEAKY_RELU 1 /* slope 0.2 */
#define MCCNN_ACT_ELU 2

/* Per-pair basis of the Monte-Carlo convolution,
 * pylib/pc/layers/MCConv.py:163-171 and :264-269 for a one-hidden-layer kernel:
 *   delta_m = (points_in[nbr_m] - points_out[ctr_m]) * inv_radius     (fp32)
 *   basis[m, l*H + h] = act(delta_m . W[l,:,h] + b[l,h]) / pdf[m]
 * neighbors holds ORIGINAL ids (point, centre).  weights [L, D, H], biases
 * [L, H] with L*H = num_basis. */
int mccnn_mc_basis(mccnn_stream_t stream, int64_t num_neighbors, int num_dims,
                   int num_basis, int activation, const float *points_in,
                   const float *points_out, const int32_t *neighbors,
                   const float *inv_radii, const float *weights,
                   const float *biases, int num_mlps, const float *pdf,
                   float *basis_out);

/* Gradient of the above w.r.t. weights and biases (accumulated over all pairs)
 * for upstream basis_grads [M, num_basis].  weight_grads_out [L,D,H] and
 * bias_grads_out [L,H] are overwritten.  partials is a workspace of
 * mccnn_mc_basis_grads_workspace_bytes() bytes. */
size_t mccnn_mc_basis_grads_workspace_bytes(int num_dims, int num_basis);
int mccnn_mc_basis_grads(mccnn_stream_t stream, int64_t num_neighbors,
                         int num_dims, int num_basis, int activation,
                         const float *points_in, const float *points_out,
                         const int32_t *neighbors, const float *inv_radii,
                         const float *weights, const float *biases,
                         int num_mlps, const float *pdf,
                         const float *basis_grads, void *workspace,
                         size_t workspace_bytes, float *weight_grads_out,
                         float *bias_grads_out);

/* mccnn_mc_basis_grads without a workspace argument and without any allocation:
 * the per-block partial sums live in a static device array of the library
 * (1.75 MiB per device, enough for the largest shape the op accepts: 6
 * dimensions, 64 basis functions; anything larger is refused with status 1).
 * No counterpart in the reference.  It is for callers that cannot allocate:
 * code under HIP graph capture, serving loops, harnesses that forbid
 * hipMalloc.  Same arguments, results bit-identical to mccnn_mc_basis_grads.
 * All calls on one device share that device's array: calls that overlap on
 * one device (two streams, two threads) race; serialise them.  The first call
 * on a device looks the array's address up (hipGetSymbolAddress, no
 * allocation); make one call before starting a graph capture. */
int mccnn_mc_basis_grads_static(mccnn_stream_t stream, int64_t num_neighbors,
                                int num_dims, int num_basis, int activation,
                                const float *points_in, const float *points_out,
                                const int32_t *neighbors,
                                const float *inv_radii, const float *weights,
                                const float *biases, int num_mlps,
                                const float *pdf, const float *basis_grads,
                                float *weight_grads_out,
                                float *bias_grads_out);

/* Fused Monte-Carlo convolution projection: mccnn_mc_basis followed by
 * mccnn_basis_proj (MCConv.py:163-177) in one kernel that evaluates the basis in
 * registers, and the matching backward (gradients of features, kernel weights
 * and biases from the upstream [N_out, C, K] gradient).  Same results as the
 * separate entry points up to fp32 summation order; the [M, K] basis and its
 * gradient are never written.  mccnn_mc_conv_supported() tells whether a shape
 * is covered (D in {2,3}, K = 16, C in {16,32,64,128}; see the two queries below
 * for the wider shapes of the forward and of the weights-only backward); other
 * shapes return
 * MCCNN_INVALID_ARGUMENT and must use the separate entry points.  out_rows
 * (optional permutation of 0..N_out-1) makes the forward write the projection of
 * centre i to row out_rows[i] of out, so that a caller working on re-ordered
 * centres gets its result back in the original order for free.  The last three
 * inputs of the backward select the atomic-free feature gradient of
 * mccnn_basis_proj_grads_gathered (all NULL = atomics); a NULL
 * feature_grads_out skips the feature gradient (a layer obtains it without any
 * scatter as the projection of its output gradient over the transposed pair
 * table: mccnn_mc_conv_project with the roles of the two point sets swapped and
 * negated inv_radii, followed by a product with the re-indexed weights).  No
 * counterpart among the reference's ops, which materialise the basis in
 * TensorFlow. */
int mccnn_mc_conv_supported(int num_dims, int num_features, int num_basis);
/* ... for the backward without the feature gradient (feature_grads_out NULL):
 * also K = 32 and K = 64 ... */
int mccnn_mc_conv_weight_grads_supported(int num_dims, int num_features, int num_basis);
/* ... and for the forward alone (also mccnn_kp_conv_project, K = 16 there): any
 * multiple of 16 channels up to 512, K in {16, 32, 64}. */
int mccnn_mc_conv_project_supported(int num_dims, int num_features, int num_basis);
int mccnn_mc_conv_project(mccnn_stream_t stream, int num_dims, int64_t num_pts,
                          const float *points_in, int num_features,
                          const float *features, int64_t num_samples,
                          const float *points_out, int64_t num_neighbors,
                          const int32_t *neighbors, const int32_t *ranges,
                          const float *inv_radii, int num_basis, int num_mlps,
                          int activation, const float *weights,
                          const float *biases, const float *pdf,
                          const int32_t *out_rows, float *out);
size_t mccnn_mc_conv_project_grads_workspace_bytes(int num_dims, int num_basis,
                                                   int64_t num_samples);
int mccnn_mc_conv_project_grads(
    mccnn_stream_t stream, int num_dims, int64_t num_pts, const float *points_in,
    int num_features, const float *features, int64_t num_samples,
    const float *points_out, int64_t num_neighbors, const int32_t *neighbors,
    const int32_t *ranges, const float *inv_radii, int num_basis, int num_mlps,
    int activation, const float *weights, const float *biases, const float *pdf,
    const float *in_grads, void *workspace, size_t workspace_bytes,
    const int32_t *point_ranges, const int32_t *pair_order,
    float *pair_rows_workspace, float *feature_grads_out,
    float *weight_grads_out, float *bias_grads_out);

/* The weights-only backward of the fused projection that also returns the gradient
 * with respect to every pair's scale 1/pdf[m]:
 *   pair_scale_grads_out [K/16, M]: slab s, pair m = sum over the basis columns
 *   16 s .. 16 s + 15 of dbasis[m, k] * act(z[m, k])
 * (the slabs are summed by the consumer).  A layer whose per-pair density is itself
 * a function of trainable parameters (PointConv.py:176-190) needs it; shapes as
 * for mccnn_mc_conv_weight_grads_supported.  No counterpart among the reference's
 * ops. */
int mccnn_mc_conv_weight_and_scale_grads(
    mccnn_stream_t stream, int num_dims, int64_t num_pts, const float *points_in,
    int num_features, const float *features, int64_t num_samples,
    const float *points_out, int64_t num_neighbors, const int32_t *neighbors,
    const int32_t *ranges, const float *inv_radii, int num_basis, int num_mlps,
    int activation, const float *weights, const float *biases, const float *pdf,
    const float *in_grads, void *workspace, size_t workspace_bytes,
    float *weight_grads_out, float *bias_grads_out, float *pair_scale_grads_out);

/* Density transform of PointConv (pylib/pc/layers/PointConv.py:176-190), per pair:
 *   rel = pdf[point] / max_pdf[centre],
 *   density_out[m] = biases_2 + sum_j weights_2[j] * relu(rel * weights_1[j] + biases_1[j]),
 * 16 hidden units.  neighbors[m][point_column] indexes pdf, the other column
 * max_pdf (point_column 1 serves a transposed pair table).  density_out takes the
 * place of pdf in the projection entry points above.  _grads turns the pair scale
 * gradients of mccnn_mc_conv_weight_and_scale_grads into param_grads_out [49]:
 * weights_1 [16], biases_1 [16], weights_2 [16], biases_2.  The reference forms
 * the [M, 16] hidden layer with TensorFlow ops. */
int mccnn_pointconv_density(mccnn_stream_t stream, int64_t num_neighbors,
                            const int32_t *neighbors, int point_column,
                            const float *pdf, const float *max_pdf,
                            const float *weights_1, const float *biases_1,
                            const float *weights_2, const float *biases_2,
                            float *density_out);
size_t mccnn_pointconv_density_grads_workspace_bytes(int64_t num_neighbors);
int mccnn_pointconv_density_grads(
    mccnn_stream_t stream, int64_t num_neighbors, const int32_t *neighbors,
    int point_column, const float *pdf, const float *max_pdf,
    const float *weights_1, const float *biases_1, const float *weights_2,
    const float *biases_2, const float *density, int num_slabs,
    const float *pair_scale_grads, void *workspace, size_t workspace_bytes,
    float *param_grads_out);

/* Rigid kernel-point convolution projection (KPConv.py:193-224): kp_basis
 * followed by basis_proj in one kernel, the correlation weights
 *   kind 0: max(1 - d/sigma, 0),  kind 1: exp(-(d/(sigma/3))^2),
 *   d = || delta - kernel_points[k] ||,  delta = (p_in[nbr] - p_out[centre]) * inv_radii
 * evaluated in registers.  out [N_out, C, 16] for up to 16 kernel points and
 * [N_out, C, 32] for 17..32; columns >= num_kernel_points are zero (the padding
 * the reference slices off).  out_rows as for mccnn_mc_conv_project.  D in
 * {2,3}, C a multiple of 16 up to 512, 1..32 kernel points.
 * No counterpart among the reference's ops. */
int mccnn_kp_conv_project(mccnn_stream_t stream, int num_dims, int64_t num_pts,
                          const float *points_in, int num_features,
                          const float *features, int64_t num_samples,
                          const float *points_out, int64_t num_neighbors,
                          const int32_t *neighbors, const int32_t *ranges,
                          const float *inv_radii, int num_kernel_points,
                          const float *kernel_points, int kind, float sigma,
                          const int32_t *out_rows, float *out);

/* Projection of the deformable kernel-point convolution (KPConv.py:317-392):
 * mccnn_kp_conv_project with the kernel points of every centre shifted by its row
 * of offsets [N_centres, num_kernel_points, D] (at most 16 kernel points).  With
 * offsets_follow_points != 0 the pair table is the transposed one (rows grouped
 * by point) and the shifts are those of the gathered side of each pair, which is
 * how the layer backward obtains its feature gradient.  No counterpart among the
 * reference's ops (kp_basis in TensorFlow + BasisProj). */
int mccnn_kp_deform_project(mccnn_stream_t stream, int num_dims, int64_t num_pts,
                            const float *points_in, int num_features,
                            const float *features, int64_t num_samples,
                            const float *points_out, int64_t num_neighbors,
                            const int32_t *neighbors, const int32_t *ranges,
                            const float *inv_radii, int num_kernel_points,
                            const float *kernel_points, int kind, float sigma,
                            const float *offsets, int offsets_follow_points,
                            const int32_t *out_rows, float *out);

/* Gradient of that projection with respect to the offsets for an upstream
 * gradient in_grads [N_out, C, 16]: offset_grads_out [N_out, num_kernel_points, D]
 * (overwritten).  The [M, 16] basis gradient is formed tile by tile on the matrix
 * cores and folded in registers; no atomics, fixed summation order.  D in {2,3},
 * C in {16,32,64,128}.  No counterpart among the reference's ops (TensorFlow
 * autodiff of KPConv.py:193-224 + BasisProjGrads). */
int mccnn_kp_deform_offset_grads_supported(int num_dims, int num_features);
int mccnn_kp_deform_offset_grads(mccnn_stream_t stream, int num_dims, int64_t num_pts,
                                 const float *points_in, int num_features,
                                 const float *features, int64_t num_samples,
                                 const float *points_out, int64_t num_neighbors,
                                 const int32_t *neighbors, const int32_t *ranges,
                                 const float *inv_radii, int num_kernel_points,
                                 const float *kernel_points, int kind, float sigma,
                                 const float *offsets, const float *in_grads,
                                 float *offset_grads_out);

/* The whole Monte-Carlo convolution (MCConv.py:137-194) in one kernel:
 *   out[i, f] = sum_{c,k} proj[i, c, k] * final_weights[c*K + k, f]
 * with proj as produced by mccnn_mc_conv_project; the projection is handed from
 * the matrix-core accumulators to the final product through LDS and reaches HBM
 * only when proj_out [N_out, C, K] is not NULL.  final_weights is the dense
 * [C*K, F] matrix, kept in registers by every block for the whole launch.
 * out_rows (optional, a permutation of 0..N_out-1) names the row of out (and of
 * proj_out) that centre i is written to.  Covered shapes
 * (mccnn_mc_conv_layer_supported): D in {2,3}, K = 16, C in {16,32,64}, F in
 * {16,32,64,128}, C*K*F <= 65536.  Results are bit-reproducible.  No
 * counterpart among the reference's ops, which run the projection and
 * tf.matmul separately. */
int mccnn_mc_conv_layer_supported(int num_dims, int num_features, int num_basis,
                                  int num_out_features);
int mccnn_mc_conv_layer(mccnn_stream_t stream, int num_dims, int64_t num_pts,
                        const float *points_in, int num_features,
                        const float *features, int64_t num_samples,
                        const float *points_out, int64_t num_neighbors,
                        const int32_t *neighbors, const int32_t *ranges,
                        const float *inv_radii, int num_basis, int num_mlps,
                        int activation, const float *weights, const float *biases,
                        const float *pdf, int num_out_features,
                        const float *final_weights, const int32_t *out_rows,
                        float *proj_out, float *out);

/* The same for the rigid kernel-point convolution (KPConv.py:165-232): the
 * projection of mccnn_kp_conv_project (up to 16 kernel points, 16 basis columns,
 * the columns past the last kernel point zero) times final_weights [C*16, F].
 * Shapes as for mccnn_mc_conv_layer. */
int mccnn_kp_conv_layer(mccnn_stream_t stream, int num_dims, int64_t num_pts,
                        const float *points_in, int num_features,
                        const float *features, int64_t num_samples,
                        const float *points_out, int64_t num_neighbors,
                        const int32_t *neighbors, const int32_t *ranges,
                        const float *inv_radii, int num_kernel_points,
                        const float *kernel_points, int kind, float sigma,
                        int num_out_features, const float *final_weights,
                        const int32_t *out_rows, float *proj_out, float *out);

/* out[out_rows[n] or n, :] = x[n, :] * w: the product of a layer with its final
 * weights (the tf.matmul of MCConv.py:187 / KPConv.py:226-230) for x [N, R] in
 * HBM and w [R, F].  One block per compute unit keeps all of w in registers and
 * streams x through LDS tiles of 16 rows, reading it exactly once; sums in a
 * fixed order (bit-reproducible).  One launch covers a block of up to 1024 rows
 * and up to 128 columns of w with at most 65536 weights; larger w (R a multiple
 * of 256 up to 8192, F a multiple of 16 up to 1024) take one launch per block,
 * x being read once per column block and the later row blocks adding to what
 * the earlier ones wrote, in launch order.  No counterpart among the
 * reference's ops (TensorFlow's matmul). */
int mccnn_final_product_supported(int num_cols_in, int num_cols_out);
int mccnn_final_product(mccnn_stream_t stream, int64_t num_rows, int num_cols_in,
                        const float *x, int num_cols_out, const float *w,
                        const int32_t *out_rows, float *out);

/* The same product with the weights handed over transposed, wt [F, R] (the rows of
 * wt run along the reduction, like the rows of x): the tiled product for weight
 * matrices beyond a block's registers (the 128 -> 128 layers, R = 2048), 128 x 128
 * or 256 x 64 output tiles per block of four wavefronts, reduction in steps of 32
 * through LDS.  Supported: R a multiple of 32, F a multiple of 64.  mccnn_final_product
 * itself switches to the same tiles (fetching w as it is, about a tenth slower) when
 * R*F > 65536 and the tiles fill the device. */
int mccnn_final_product_wt_supported(int num_cols_in, int num_cols_out);
int mccnn_final_product_wt(mccnn_stream_t stream, int64_t num_rows, int num_cols_in,
                           const float *x, int num_cols_out, const float *wt,
                           const int32_t *out_rows, float *out);

/* out[c, r] = sum_n x[n, c] * y[n, r]: the gradient of a layer's final weights
 * (the backward of the tf.matmul of MCConv.py:187 / KPConv.py:226-230), a product
 * with a reduction over all points and a small [C, R] output.  y is read from
 * HBM exactly once; per-slice partial sums in the workspace are added in a fixed
 * order (bit-reproducible).  Supported: C in {16,32,64,128}, R a multiple of 256
 * up to 4096.  No counterpart among the reference's ops (TensorFlow's matmul
 * gradient). */
int mccnn_weight_grad_product_supported(int num_rows_out, int num_cols_out);
size_t mccnn_weight_grad_product_workspace_bytes(int num_rows_out, int num_cols_out);
int mccnn_weight_grad_product(mccnn_stream_t stream, int64_t num_pts,
                              int num_rows_out, const float *x, int num_cols_out,
                              const float *y, void *workspace,
                              size_t workspace_bytes, float *out);

/* One layer of a kernel MLP per neighbour pair: y[m, :] = act(x[m, :] * weights + biases)
 * for x [num_rows, num_cols_in], weights [num_cols_in, num_cols_out] (both widths 1..64),
 * biases [num_cols_out] or NULL; activation -1 (none) or MCCNN_ACT_*.  The reference
 * evaluates its kernel MLPs with tf.matmul on [M, .] tensors (MCConv.py:163-168,
 * PointConv.py:168-190); these are the same layers as memory-bound kernels, used for kernel
 * MLPs of several layers and where the kernel input stays differentiable.
 * _grads: from the layer's output y and the upstream gradient dy, dx [num_rows,
 * num_cols_in] (NULL to skip), dweights and dbiases (NULL to skip); partial sums per slice
 * of the rows in the workspace, added in a fixed order. */
int mccnn_pair_dense(mccnn_stream_t stream, int64_t num_rows, int num_cols_in,
                     const float *x, int num_cols_out, const float *weights,
                     const float *biases, int activation, float *y);
size_t mccnn_pair_dense_grads_workspace_bytes(int64_t num_rows, int num_cols_in,
                                              int num_cols_out);
int mccnn_pair_dense_grads(mccnn_stream_t stream, int64_t num_rows, int num_cols_in,
                           const float *x, int num_cols_out, const float *weights,
                           const float *y, const float *dy, int activation,
                           void *workspace, size_t workspace_bytes, float *dx,
                           float *dweights, float *dbiases);

/* The dense products of the layers (final product, projection gradient, final-weight
 * gradient) run on the bf16 matrix pipe with float32 accuracy: every float32 operand is
 * split into three bfloat16 parts and six of the nine part products are accumulated in
 * float32 (the three left out are below 2^-24 of the term).  mccnn_set_split_products(0)
 * switches the process back to the float32 matrix instructions (returns the previous
 * setting); MCCNN_DENSE_FP32=1 in the environment does the same from the start.  No
 * counterpart in the reference (TensorFlow picks its own GEMM). */
int mccnn_set_split_products(int enabled);
int mccnn_split_products_enabled(void);

/* out[n, r] = sum_f x[n, f] * w[r, f]: the gradient of the projection entering a
 * layer's final product (x = output gradient [N, F], w = final weights [R, F],
 * out [N, R]); write-bound, each wavefront keeps its slice of w in registers.
 * Supported: F in {16,32,64} with R a multiple of 256, F = 128 with R a multiple
 * of 128, F = 256 with R a multiple of 64.  No counterpart among the reference's
 * ops (TensorFlow's matmul gradient). */
int mccnn_projection_grad_product_supported(int num_cols_in, int num_cols_out);
int mccnn_projection_grad_product(mccnn_stream_t stream, int64_t num_pts,
                                  int num_cols_in, const float *x,
                                  int num_cols_out, const float *w, float *out);

/* Per-pair kernel-point weights, pylib/pc/layers/KPConv.py:29-57,193-213:
 *   d[m,k] = || delta_m - (kernel_points[k] + offsets[ctr_m,k]) ||
 *   kind 0: max(1 - d/sigma, 0);  kind 1: exp(-(d/(sigma/3))^2)
 * written to basis_out [M, num_basis] with columns >= num_kernel_points zero.
 * offsets [num_samples, num_kernel_points, D] may be NULL (rigid).  dist_out
 * [M, num_kernel_points] may be NULL. */
int mccnn_kp_basis(mccnn_stream_t stream, int64_t num_neighbors, int num_dims,
                   int num_kernel_points, int num_basis, int kind, float sigma,
                   const float *points_in, const float *points_out,
                   const int32_t *neighbors, const float *inv_radii,
                   const float *kernel_points, const float *offsets,
                   float *basis_out, float *dist_out);

/* Gradient of mccnn_kp_basis with respect to the per-centre kernel-point
 * offsets (deformable KPConv, pylib/pc/layers/KPConv.py:193-198 differentiated):
 * offsets_grads_out [num_samples, num_kernel_points, D] for upstream basis_grads
 * [M, num_basis].  The pairs of a centre are summed in order, without atomics. */
int mccnn_kp_basis_grads(mccnn_stream_t stream, int64_t num_neighbors,
                         int num_dims, int num_kernel_points, int num_basis,
                         int kind, float sigma, const float *points_in,
                         const float *points_out, const int32_t *neighbors,
                         int64_t num_samples, const int32_t *ranges,
                         const float *inv_radii, const float *kernel_points,
                         const float *offsets, const float *basis_grads,
                         float *offsets_grads_out);

/* Regularisation terms of deformable kernel points,
 * pylib/pc/layers/KPConv.py:394-429: fit_out [num_samples, KP] = min over the
 * pairs of the centre of (dist / sigma)^2 with the attaining pair in argmin_out
 * (0 and -1 for a centre without pairs), repulsion_out [num_samples, KP] =
 * sum over the other kernel points of the correlation weight of their distance.
 * The loss is sum(fit) + sum(repulsion). */
int mccnn_kp_regularization(mccnn_stream_t stream, int64_t num_neighbors,
                            int num_dims, int num_kernel_points, int kind,
                            float sigma, const float *points_in,
                            const float *points_out, const int32_t *neighbors,
                            int64_t num_samples, const int32_t *ranges,
                            const float *inv_radii, const float *kernel_points,
                            const float *offsets, float *fit_out,
                            int32_t *argmin_out, float *repulsion_out);

/* offsets_grads_out = loss_grad * d(sum(fit) + sum(repulsion)) / d(offsets). */
int mccnn_kp_regularization_grads(mccnn_stream_t stream, int64_t num_neighbors,
                                  int num_dims, int num_kernel_points, int kind,
                                  float sigma, float loss_grad,
                                  const float *points_in, const float *points_out,
                                  const int32_t *neighbors, int64_t num_samples,
                                  const float *inv_radii,
                                  const float *kernel_points, const float *offsets,
                                  const int32_t *argmin, float *offsets_grads_out);

#ifdef __cplusplus
}
#endif
#endif /* MCCNN_HIP_H_ */
