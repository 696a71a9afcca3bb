"""Object-level adapters of the ops, with the names and argument meaning of
the reference's dispatch module (pylib/pc/custom_ops/__init__.py:20-39,
custom_ops_wrapper.py:20-198): they take `PointCloud`, `Grid` and
`Neighborhood` instances and forward to the positional op entry points of
`tfg_custom_ops`.  There is no second implementation to fall back to: the HIP
library is the only backend."""
import torch

from . import tfg_custom_ops


def compute_keys(point_cloud, num_cells, cell_size):
    """Cell key per point, int64 [N] (custom_ops_wrapper.py:20-43)."""
    aabb = point_cloud.get_AABB()
    return tfg_custom_ops.compute_keys(
        point_cloud._points, point_cloud._batch_ids, (aabb._aabb_min / cell_size).contiguous(),
        num_cells, torch.reciprocal(cell_size))


def build_grid_ds(sorted_keys, num_cells, batch_size):
    """[batch_size, num_cells[0], num_cells[1], 2] first / last+1 index per
    column of the sorted keys (custom_ops_wrapper.py:47-66)."""
    return tfg_custom_ops.build_grid_ds(sorted_keys, num_cells, num_cells, batch_size)


def find_neighbors(grid, point_cloud_centers, radii, max_neighbors=0):
    """-> (ranges [N_out] inclusive end offsets, neighbors [M, 2] rows (sorted
    point index, centre index)) (custom_ops_wrapper.py:70-104)."""
    return tfg_custom_ops.find_neighbors(
        point_cloud_centers._points, point_cloud_centers._batch_ids, grid._sorted_points,
        grid._sorted_keys, grid.get_DS(), grid._num_cells, grid._scaled_aabb_min,
        grid._inv_cell_sizes, torch.reciprocal(radii), max_neighbors)


def sampling(neighborhood, sample_mode):
    """-> (points [S, D], batch ids [S], indices into the grid's sorted points [S]);
    `sample_mode` 0 Poisson disk, 1 cell average as the op defines them
    (sampling_ops.cpp:33-53; the wrapper's docstring has the two the other way
    round, custom_ops_wrapper.py:114-115)."""
    g = neighborhood._grid
    return tfg_custom_ops.sampling(g._sorted_points, g._sorted_batch_ids, g._sorted_keys,
                                   g._num_cells, neighborhood._neighbors,
                                   neighborhood._samples_neigh_ranges, sample_mode)


def compute_pdf(neighborhood, bandwidth, mode):
    """Density per sorted point of the neighbourhood's grid, differentiable with
    respect to the points (custom_ops_wrapper.py:136-169)."""
    return tfg_custom_ops.compute_pdf_with_pt_grads(
        neighborhood._grid._sorted_points, neighborhood._neighbors,
        neighborhood._samples_neigh_ranges, torch.reciprocal(bandwidth),
        torch.reciprocal(neighborhood._radii), mode)


def basis_proj(neigh_basis, features, neighborhood):
    """[N_out, C, H] sum of feature (outer) basis over the pairs of every centre,
    differentiable in both (custom_ops_wrapper.py:172-198)."""
    return tfg_custom_ops.basis_proj(neigh_basis, features, neighborhood._original_neigh_ids,
                                     neighborhood._samples_neigh_ranges)
