"""The eight entry points of the reference's native op package
(custom_ops/tfg_custom_ops/__init__.py:16-26), on torch GPU tensors, with the
positional argument order of the reference's REGISTER_OP declarations.  Each
function forwards to one or two C-ABI calls of libmccnn_hip.so on torch's
current stream; nothing is computed in Python or torch.

Gradients mirror custom_ops_wrapper.py:159-169 and :192-198: `basis_proj` and
`compute_pdf_with_pt_grads` are differentiable (basis and features / points),
the other ops are not.
"""
import torch

from .. import _lib
from .._lib import InvalidArgumentError, cint, i64, ptr, stream, vptr

__all__ = ["compute_keys", "build_grid_ds", "find_neighbors", "sampling",
           "compute_pdf_with_pt_grads", "compute_pdf_pt_grads", "basis_proj",
           "basis_proj_grads", "transpose_neighbors", "InvalidArgumentError"]

_F32, _I32, _I64 = torch.float32, torch.int32, torch.int64


def _dim(t, axis, default=-1):
    return t.shape[axis] if t.dim() > axis else default


def compute_keys(points, batch_ids, scaled_aabb_min, num_cells, inv_cell_sizes):
    """ComputeKeys (compute_keys_ops.cpp:29-41): int64 cell key per point."""
    keys = torch.empty(points.shape[0], dtype=_I64, device=points.device)
    _lib.call("compute_keys", stream(), i64(points.shape[0]), cint(_dim(points, 1)), ptr(points, _F32),
        i64(batch_ids.shape[0]), ptr(batch_ids, _I32),
        i64(scaled_aabb_min.shape[0]), cint(_dim(scaled_aabb_min, 1)),
        ptr(scaled_aabb_min, _F32), cint(num_cells.shape[0]), ptr(num_cells, _I32),
        cint(inv_cell_sizes.shape[0]), ptr(inv_cell_sizes, _F32), ptr(keys))
    return keys


def build_grid_ds(sorted_keys, num_cells, num_cells_host, batch_size):
    """BuildGridDs (build_grid_ds_ops.cpp:27-40): [B, n0, n1, 2] column table.
    `num_cells_host` is the host copy (list / CPU tensor / numpy) that sizes it."""
    host = [int(v) for v in (num_cells_host.tolist() if hasattr(num_cells_host, "tolist")
                             else num_cells_host)]
    if batch_size <= 0:
        raise InvalidArgumentError("BuildGridDs requires a positive batch size")
    if len(host) < 2:
        raise InvalidArgumentError("BuildGridDs expects a valid number of dimensions")
    import ctypes
    host_arr = (ctypes.c_int32 * len(host))(*host)
    ds = torch.empty((batch_size, host[0], host[1], 2), dtype=_I32, device=sorted_keys.device)
    _lib.call("build_grid_ds", stream(), i64(sorted_keys.shape[0]), ptr(sorted_keys, _I64), cint(num_cells.shape[0]),
        ptr(num_cells, _I32), cint(len(host)), host_arr, cint(batch_size), ptr(ds))
    return ds


def find_neighbors(samples, samples_batch_ids, points, point_keys, grid_acc_ds, num_cells,
                   scaled_aabb_min, inv_cell_sizes, inv_radii, max_neighs=0):
    """FindNeighbors (find_neighbors_ops.cpp:42-61) -> (ranges [N_out] inclusive
    end offsets, neighbors [M, 2] rows (sorted point index, centre index))."""
    import ctypes
    L = _lib.lib()
    ns, nd = samples.shape[0], _dim(samples, 1)
    dev = samples.device
    ws_bytes = L.mccnn_find_neighbors_workspace_bytes(cint(nd), i64(ns))
    ws = _lib.workspace(ws_bytes, dev)
    ranges = torch.empty(ns, dtype=_I32, device=dev)
    total, total_ptr = _lib.host_count()
    dsr = grid_acc_ds.dim()
    _lib.call("find_neighbors_count_facts", stream(), i64(ns), cint(nd), ptr(samples, _F32), i64(samples_batch_ids.shape[0]),
        ptr(samples_batch_ids, _I32), i64(points.shape[0]), cint(_dim(points, 1)),
        ptr(points, _F32), i64(point_keys.shape[0]), ptr(point_keys, _I64), cint(dsr),
        cint(_dim(grid_acc_ds, 0)), cint(_dim(grid_acc_ds, 1)), cint(_dim(grid_acc_ds, 2)),
        cint(_dim(grid_acc_ds, 3)), ptr(grid_acc_ds, _I32), cint(num_cells.shape[0]),
        ptr(num_cells, _I32), cint(_dim(scaled_aabb_min, 1)), ptr(scaled_aabb_min, _F32),
        cint(inv_cell_sizes.shape[0]), ptr(inv_cell_sizes, _F32), cint(inv_radii.shape[0]),
        ptr(inv_radii, _F32), cint(max_neighs), ptr(ws), _lib.csize(ws.numel()), ptr(ranges),
        total_ptr, _lib.vptr(total.data_ptr() + 8), timed_as="find_neighbors_count")
    m = int(total[0])
    symmetric = int(total[1]) == 0 and int(total[2]) == 1
    neighbors = torch.empty((m, 2), dtype=_I32, device=dev)
    _lib.call("find_neighbors_fill", stream(), i64(ns), cint(nd), ptr(samples, _F32), ptr(samples_batch_ids, _I32),
        i64(points.shape[0]), ptr(points, _F32), ptr(point_keys, _I64), ptr(grid_acc_ds, _I32),
        ptr(num_cells, _I32), ptr(scaled_aabb_min, _F32), ptr(inv_cell_sizes, _F32),
        ptr(inv_radii, _F32), cint(max_neighs), ptr(ws), _lib.csize(ws.numel()), ptr(ranges),
        i64(m), ptr(neighbors))
    if symmetric:
        _remember_symmetric(neighbors)
    return ranges, neighbors


def find_neighbors_bounded(samples, samples_batch_ids, points, point_keys, grid_acc_ds, num_cells,
                           scaled_aabb_min, inv_cell_sizes, inv_radii, max_neighs, capacity,
                           out=None):
    """find_neighbors without a host round trip: (ranges [N_out], neighbors [capacity, 2],
    count [2] = (pairs found, 1 if they exceed the capacity), all on the device).  Rows of the
    table past the count are not written.  `out` = (ranges, neighbors, count) reuses tensors
    of a previous call, so that the call allocates nothing and can be recorded in a HIP
    graph."""
    ns, nd = samples.shape[0], _dim(samples, 1)
    dev = samples.device
    L = _lib.lib()
    if out is None:
        out = (torch.empty(ns, dtype=_I32, device=dev),
               torch.empty((capacity, 2), dtype=_I32, device=dev),
               torch.zeros(2, dtype=_I64, device=dev),
               torch.empty(max(int(L.mccnn_find_neighbors_workspace_bytes(cint(nd), i64(ns))), 1),
                           dtype=torch.uint8, device=dev))
    ranges, neighbors, count, ws = out
    _lib.call("find_neighbors_bounded", stream(), i64(ns), cint(nd), ptr(samples, _F32),
              ptr(samples_batch_ids, _I32), i64(points.shape[0]), ptr(points, _F32),
              ptr(point_keys, _I64), cint(_dim(grid_acc_ds, 0)), cint(_dim(grid_acc_ds, 1)),
              cint(_dim(grid_acc_ds, 2)), ptr(grid_acc_ds, _I32), ptr(num_cells, _I32),
              ptr(scaled_aabb_min, _F32), ptr(inv_cell_sizes, _F32), ptr(inv_radii, _F32),
              cint(max_neighs), ptr(ws), _lib.csize(ws.numel()), i64(neighbors.shape[0]),
              ptr(ranges), ptr(neighbors), ptr(count))
    return out


def sampling(points, batch_ids, point_keys, num_cells, neighbors, sample_neigh_indices, mode):
    """Sampling (sampling_ops.cpp:33-53): mode 0 Poisson disk, mode 1 cell average.
    -> (sample_pts [S, D], sample_batch_ids [S], sample_indices [S])."""
    import ctypes
    L = _lib.lib()
    n, nd = points.shape[0], _dim(points, 1)
    dev = points.device
    ws = _lib.workspace(L.mccnn_sampling_workspace_bytes(i64(n)), dev)
    total, total_ptr = _lib.host_count()
    _lib.call("sampling_count", stream(), cint(mode), i64(n), cint(nd), ptr(points, _F32), i64(batch_ids.shape[0]),
        ptr(batch_ids, _I32), i64(point_keys.shape[0]), ptr(point_keys, _I64),
        cint(num_cells.shape[0]), ptr(num_cells, _I32), i64(neighbors.shape[0]),
        cint(neighbors.dim()), cint(_dim(neighbors, 1)), ptr(neighbors, _I32),
        i64(sample_neigh_indices.shape[0]), ptr(sample_neigh_indices, _I32), ptr(ws),
        _lib.csize(ws.numel()), total_ptr)
    s = int(total[0])
    out_pts = torch.empty((s, nd), dtype=_F32, device=dev)
    out_bids = torch.empty(s, dtype=_I32, device=dev)
    out_idx = torch.empty(s, dtype=_I32, device=dev)
    _lib.call("sampling_fill", stream(), cint(mode), i64(n), cint(nd), ptr(points, _F32), ptr(batch_ids, _I32),
        ptr(point_keys, _I64), ptr(num_cells, _I32), ptr(ws), _lib.csize(ws.numel()), i64(s),
        ptr(out_pts), ptr(out_bids), ptr(out_idx))
    return out_pts, out_bids, out_idx


def _compute_pdf_raw(points, neighbors, ranges, inv_bandwidth, inv_radii, mode):
    pdf = torch.empty(ranges.shape[0], dtype=_F32, device=points.device)
    _lib.call("compute_pdf", stream(), i64(points.shape[0]), cint(_dim(points, 1)), ptr(points, _F32),
        i64(neighbors.shape[0]), cint(neighbors.dim()), cint(_dim(neighbors, 1)),
        ptr(neighbors, _I32), i64(ranges.shape[0]), ptr(ranges, _I32),
        cint(inv_bandwidth.shape[0]), ptr(inv_bandwidth, _F32), cint(inv_radii.shape[0]),
        ptr(inv_radii, _F32), cint(mode), ptr(pdf))
    return pdf


# Pair tables that find_neighbors reported as untruncated self-neighbourhoods (symmetric:
# j in N(c) <=> c in N(j)), by the identity of the tensor it returned; the entry dies with it.
_symmetric_tables = {}


def _remember_symmetric(neighbors):
    """To be called once the table has been filled: its version counter then only moves if
    somebody writes to the tensor in place, which voids the record."""
    import weakref
    key = id(neighbors)
    _symmetric_tables[key] = (weakref.ref(neighbors, lambda _, k=key: _symmetric_tables.pop(k, None)),
                              neighbors._version)


def is_symmetric_table(neighbors):
    """True for a pair table that `find_neighbors` returned for the points as their own
    centres without cutting any neighbourhood at max_neighs, and that has not been written
    to since."""
    entry = _symmetric_tables.get(id(neighbors))
    return entry is not None and entry[0]() is neighbors and entry[1] == neighbors._version


def compute_pdf_pt_grads(points, neighbors, sample_neigh_indices, inv_bandwidth, inv_radii,
                         pdf_grads, mode, symmetric=False):
    """ComputePdfPtGrads (compute_pdf_ops.cpp:58-74): [N, D] gradient of
    sum(pdf_grads * pdf) with respect to the points.  `symmetric=True` (the caller
    vouches that j in N(c) <=> c in N(j)) selects the atomic-free gather; a table that
    `find_neighbors` itself reported as an untruncated self-neighbourhood takes it
    without being told."""
    symmetric = symmetric or is_symmetric_table(neighbors)
    out = torch.empty_like(points)
    _lib.call("compute_pdf_pt_grads_symmetric" if symmetric else "compute_pdf_pt_grads", stream(), i64(points.shape[0]), cint(_dim(points, 1)), ptr(points, _F32),
        i64(neighbors.shape[0]), cint(neighbors.dim()), cint(_dim(neighbors, 1)),
        ptr(neighbors, _I32), i64(sample_neigh_indices.shape[0]),
        ptr(sample_neigh_indices, _I32), cint(inv_bandwidth.shape[0]),
        ptr(inv_bandwidth, _F32), cint(inv_radii.shape[0]), ptr(inv_radii, _F32),
        i64(pdf_grads.shape[0]), ptr(pdf_grads, _F32), cint(mode), ptr(out))
    return out


class _ComputePdf(torch.autograd.Function):
    @staticmethod
    def forward(ctx, points, neighbors, ranges, inv_bandwidth, inv_radii, mode, symmetric):
        ctx.save_for_backward(points, neighbors, ranges, inv_bandwidth, inv_radii)
        ctx.mode, ctx.symmetric = mode, symmetric
        return _compute_pdf_raw(points, neighbors, ranges, inv_bandwidth, inv_radii, mode)

    @staticmethod
    def backward(ctx, grad):
        points, neighbors, ranges, inv_bandwidth, inv_radii = ctx.saved_tensors
        g = compute_pdf_pt_grads(points, neighbors, ranges, inv_bandwidth, inv_radii,
                                 grad.contiguous(), ctx.mode, ctx.symmetric)
        return g, None, None, None, None, None, None


def compute_pdf_with_pt_grads(points, neighbors, sample_neigh_indices, inv_bandwidth,
                              inv_radii, mode, symmetric=False):
    """ComputePdfWithPtGrads (compute_pdf_ops.cpp:43-56): Gaussian KDE per point
    over its neighbour list; differentiable with respect to `points`.
    `symmetric`: see `compute_pdf_pt_grads`."""
    return _ComputePdf.apply(points, neighbors, sample_neigh_indices, inv_bandwidth,
                             inv_radii, mode, symmetric)


def _basis_proj_raw(basis, features, neighbors, ranges, centre_order=None):
    out = torch.empty((ranges.shape[0], _dim(features, 1), _dim(basis, 1)), dtype=_F32,
                      device=features.device)
    _lib.call("basis_proj_ordered", stream(), i64(basis.shape[0]), cint(_dim(basis, 1)),
              ptr(basis, _F32), i64(features.shape[0]), cint(_dim(features, 1)),
              ptr(features, _F32), i64(neighbors.shape[0]), cint(neighbors.dim()),
              cint(_dim(neighbors, 1)), ptr(neighbors, _I32), i64(ranges.shape[0]),
              ptr(ranges, _I32), ptr(centre_order, _I32 if centre_order is not None else None),
              ptr(out))
    return out


def gathered_grads_supported(num_features, num_basis):
    """Shapes for which the atomic-free feature gradient exists."""
    if num_basis == 16:
        return num_features in (16, 32, 64, 128)
    if num_basis == 32:
        return num_features in (32, 64, 128)
    return False


def basis_proj_grads(basis_neighbors, pt_features, neighbors, sample_neigh_indices,
                     in_gradients, centre_order=None, transposed=None):
    """BasisProjGrads (basis_proj_ops.cpp:40-53) -> (basis_gradients [M, K],
    feat_gradients [N_in, C]).  `transposed` = (point_ranges, pair_order) from
    `transpose_neighbors` selects the atomic-free, bit-reproducible feature
    gradient (needs an [M, C] scratch tensor)."""
    dbasis = torch.empty_like(basis_neighbors)
    dfeat = torch.empty_like(pt_features)
    g = in_gradients
    head = (stream(), i64(basis_neighbors.shape[0]), cint(_dim(basis_neighbors, 1)),
            ptr(basis_neighbors, _F32), i64(pt_features.shape[0]), cint(_dim(pt_features, 1)),
            ptr(pt_features, _F32), i64(neighbors.shape[0]), cint(neighbors.dim()),
            cint(_dim(neighbors, 1)), ptr(neighbors, _I32), i64(sample_neigh_indices.shape[0]),
            ptr(sample_neigh_indices, _I32))
    gdims = (cint(g.dim()), i64(_dim(g, 0)), i64(_dim(g, 1)), i64(_dim(g, 2)), ptr(g, _F32))
    if transposed is not None and gathered_grads_supported(_dim(pt_features, 1),
                                                           _dim(basis_neighbors, 1)):
        rows = torch.empty((neighbors.shape[0], pt_features.shape[1]), dtype=_F32,
                           device=pt_features.device)
        _lib.call("basis_proj_grads_gathered", *head, *gdims, ptr(transposed[0], _I32),
                  ptr(transposed[1], _I32), ptr(rows), ptr(dbasis), ptr(dfeat))
    else:
        _lib.call("basis_proj_grads_ordered", *head,
                  ptr(centre_order, _I32 if centre_order is not None else None), *gdims,
                  ptr(dbasis), ptr(dfeat))
    return dbasis, dfeat


def transpose_neighbors(neighbors, num_pts):
    """Pair lists grouped by neighbour point: (point_ranges [num_pts] inclusive end
    offsets, pair_order [M] pair indices sorted by neighbors[:, 0], stable)."""
    L = _lib.lib()
    L.mccnn_transpose_neighbors_workspace_bytes.restype = _lib.csize
    m, dev = neighbors.shape[0], neighbors.device
    ws = _lib.workspace(L.mccnn_transpose_neighbors_workspace_bytes(i64(m), i64(num_pts)), dev)
    point_ranges = torch.empty(num_pts, dtype=_I32, device=dev)
    pair_order = torch.empty(m, dtype=_I32, device=dev)
    _lib.call("transpose_neighbors", stream(), i64(m), ptr(neighbors, _I32), i64(num_pts),
              ptr(ws), _lib.csize(ws.numel()), ptr(point_ranges), ptr(pair_order))
    return point_ranges, pair_order


class _BasisProj(torch.autograd.Function):
    @staticmethod
    def forward(ctx, basis, features, neighbors, ranges, centre_order, transposed):
        ctx.save_for_backward(basis, features, neighbors, ranges)
        ctx.centre_order, ctx.transposed = centre_order, transposed
        return _basis_proj_raw(basis, features, neighbors, ranges, centre_order)

    @staticmethod
    def backward(ctx, grad):
        basis, features, neighbors, ranges = ctx.saved_tensors
        dbasis, dfeat = basis_proj_grads(basis, features, neighbors, ranges, grad.contiguous(),
                                         ctx.centre_order, ctx.transposed)
        return dbasis, dfeat, None, None, None, None


def basis_proj(basis_neighbors, pt_features, neighbors, sample_neigh_indices,
               centre_order=None, transposed=None):
    """BasisProj (basis_proj_ops.cpp:25-38): [N_out, C, K] sum over the pairs of
    each centre of feature (outer) basis; differentiable in basis and features.
    `centre_order` (optional int32 permutation of the centres) only changes the
    order in which centres are processed; `transposed` (optional, see
    `basis_proj_grads`) selects the atomic-free backward."""
    return _BasisProj.apply(basis_neighbors, pt_features, neighbors, sample_neigh_indices,
                            centre_order, transposed)
