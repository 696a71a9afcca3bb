"""Thin counterparts of the reference's callers of the op path, on torch GPU
tensors: `PointCloud` (segmented and padded forms), `Grid`, `Neighborhood`, `sample`
and `PointHierarchy` (pylib/pc/PointCloud.py, Grid.py, Neighborhood.py,
sampling.py, PointHierarchy.py).  They only arrange arguments: bounding boxes,
grid shape, sort and gathers are kernels of libmccnn_hip.so as well.
"""
import ctypes
import enum
import threading
import math

import numpy as np

import torch

from . import _lib, tfg_custom_ops
from ._lib import cint, i64, ptr, stream

_F32, _I32, _I64 = torch.float32, torch.int32, torch.int64


class KDEMode(enum.Enum):
    """pylib/pc/Neighborhood.py: constant bandwidth, bandwidth from the number of
    points, or no density estimate."""
    constant = 0
    num_points = 1
    no_pdf = 2


_vector_cache = {}       # (bytes of the host values, dims, device) -> shared device vector
_shared = {}             # id of a shared vector -> (the vector itself, its host values)
_derived_cache = {}      # (operation, id of a shared vector) -> shared result


def _share(t, values):
    """Registers a small read-only device vector under its own identity.  The entry keeps
    the tensor alive, so the id (and the memory behind it) cannot be handed to another
    tensor while the entry exists."""
    _shared[id(t)] = (t, values)
    return t


def _as_vector(value, dims, device):
    """`value` (a number, a sequence or a tensor) as a float32 [dims] tensor on
    `device`.  Host numbers are uploaded once per (value, dims, device) and the
    tensor is shared read-only afterwards: radii and cell sizes repeat in every
    layer of a network."""
    if isinstance(value, torch.Tensor):
        t = value.to(dtype=_F32).reshape(-1)
        if t.numel() == 1:
            t = t.repeat(dims)
        return t.to(device).contiguous()
    host = np.asarray(value, dtype=np.float32).reshape(-1)
    key = (host.tobytes(), int(dims), str(device))
    t = _vector_cache.get(key)
    if t is None:
        t = torch.as_tensor(host)
        if t.numel() == 1:
            t = t.repeat(dims)
        t = t.to(device).contiguous()
        if len(_vector_cache) < 4096:
            _vector_cache[key] = _share(t, tuple(float(v) for v in t.tolist()))
    return t


def _derived(op, fn, t):
    """fn(t) for a small device vector; the vectors `_as_vector` keeps (shared,
    read-only) and what was derived from them get the result once instead of one
    kernel launch per use.  Shared vectors are recognised by object identity, never by
    address: a caller's own tensor always takes fn(t)."""
    entry = _shared.get(id(t))
    if entry is None or entry[0] is not t:
        return fn(t)
    r = _derived_cache.get((op, id(t)))
    if r is None:
        r = _derived_cache[(op, id(t))] = _share(fn(t), None)
    return r


def _reciprocal(t):
    return _derived("reciprocal", torch.reciprocal, t)


def _negative(t):
    return _derived("negative", torch.neg, t)


def _host_values(t):
    """The entries of a small device vector as a tuple of floats; no device round
    trip for the vectors `_as_vector` keeps."""
    entry = _shared.get(id(t))
    if entry is not None and entry[0] is t and entry[1] is not None and \
            len(entry[1]) == t.numel():
        return entry[1]
    return tuple(float(v) for v in t.tolist())


class AABB:
    """Axis-aligned bounding box per cloud (pylib/pc/PointCloud.py:23-66)."""

    def __init__(self, point_cloud):
        pts, ids = point_cloud._points.detach(), point_cloud._batch_ids.long()
        b, d = point_cloud._batch_size, pts.shape[1]
        index = ids[:, None].expand(-1, d)
        self._batch_shape = point_cloud._batch_shape
        self._aabb_min = torch.zeros((b, d), dtype=_F32, device=pts.device).scatter_reduce(
            0, index, pts, "amin", include_self=False) - 1e-9
        self._aabb_max = torch.zeros((b, d), dtype=_F32, device=pts.device).scatter_reduce(
            0, index, pts, "amax", include_self=False) + 1e-9

    def get_diameter(self, ord="euclidean"):
        """Norm of the box extent per cloud, [A1, ..., An] (or [B])."""
        extent = self._aabb_max - self._aabb_min
        diam = torch.linalg.vector_norm(extent, ord=2 if ord == "euclidean" else ord, dim=-1)
        return diam if self._batch_shape is None else diam.reshape(self._batch_shape)


class PointCloud:
    """Points with a cloud id per point (pylib/pc/PointCloud.py:68-290).

    points     [N, D] with `batch_ids` [N] or `sizes` (sum = N), or padded
               [A1, ..., An, V, D] with optional `sizes` [A1, ..., An] (the first
               sizes[a] rows of each cloud are real, the rest padding)
    batch_size number of clouds (default: from batch_ids / sizes / batch shape)

    Internally always the segmented form `_points` [N, D], `_batch_ids` [N]."""

    def __init__(self, points, batch_ids=None, batch_size=None, sizes=None):
        points = torch.as_tensor(points, dtype=_F32)
        dev = points.device
        self._sizes = None if sizes is None else torch.as_tensor(sizes, dtype=_I32, device=dev)
        self._batch_shape = None
        if points.dim() < 2:
            raise ValueError("expected points [N, D] or [A1, ..., An, V, D]")
        if points.dim() > 2:                                  # PointCloud.py:122-138
            self._batch_shape = tuple(points.shape[:-2])
            clouds, v = int(math.prod(self._batch_shape)), points.shape[-2]
            if self._sizes is None:
                self._sizes = torch.full(self._batch_shape, v, dtype=_I32, device=dev)
            if tuple(self._sizes.shape) != self._batch_shape:
                raise ValueError("sizes must have the batch shape %s" % (self._batch_shape,))
            flat_sizes = self._sizes.reshape(-1).long()
            if bool((flat_sizes > v).any()) or bool((flat_sizes < 0).any()):
                raise ValueError("sizes must lie in [0, V]")
            if batch_size is None:
                batch_size = clouds
            keep = (torch.arange(v, device=dev)[None, :] < flat_sizes[:, None]).reshape(-1)
            self._points = points.reshape(clouds * v, -1)[keep].contiguous()
            self._batch_ids = torch.repeat_interleave(
                torch.arange(clouds, dtype=_I32, device=dev), flat_sizes)
        else:                                                 # PointCloud.py:140-149
            self._points = points.contiguous()
            if batch_ids is None:
                if self._sizes is None:
                    raise ValueError("points [N, D] need batch_ids or sizes")
                flat_sizes = self._sizes.reshape(-1).long()
                if batch_size is None:
                    batch_size = flat_sizes.numel()
                batch_ids = torch.repeat_interleave(
                    torch.arange(flat_sizes.numel(), dtype=_I32, device=dev), flat_sizes)
            self._batch_ids = torch.as_tensor(batch_ids, dtype=_I32, device=dev).contiguous()
            if self._batch_ids.shape[0] != self._points.shape[0]:
                raise ValueError("expected one batch id (or sizes summing to one) per point")
            if batch_size is None:
                batch_size = int(self._batch_ids.max().item()) + 1 if self._points.shape[0] else 0
        self._batch_size = int(batch_size)
        self._dimension = self._points.shape[1]

    def get_AABB(self):
        """The bounding boxes, computed on the first call (PointCloud.py:235-247)."""
        if getattr(self, "_aabb", None) is None:
            self._aabb = AABB(self)
        return self._aabb

    def get_sizes(self):
        """Points per cloud, in the batch shape if one is set (PointCloud.py:184-204)."""
        if self._sizes is None:
            self._sizes = torch.bincount(self._batch_ids.long(),
                                         minlength=self._batch_size).to(_I32)
            if self._batch_shape is not None:
                self._sizes = self._sizes.reshape(self._batch_shape)
        return self._sizes

    def set_batch_shape(self, batch_shape):
        """PointCloud.py:262-290."""
        if batch_shape is None:
            self._batch_shape = None
            return
        batch_shape = tuple(int(b) for b in batch_shape)
        if int(math.prod(batch_shape)) != self._batch_size:
            raise ValueError("Incompatible batch size. Must be %d but is %d" %
                             (self._batch_size, int(math.prod(batch_shape))))
        self._batch_shape = batch_shape
        if self._sizes is not None:
            self._sizes = self._sizes.reshape(batch_shape)

    def get_unflatten(self, max_num_points=None):
        """data [N, ...] -> zero-padded [A1, ..., An, V, ...] (PointCloud.py:206-235):
        the rows of each cloud in their stored order."""
        sizes = self.get_sizes().reshape(-1).long()
        v = int(sizes.max().item()) if sizes.numel() else 0
        if max_num_points is not None:
            if max_num_points < v:
                raise ValueError("max_num_points must be at least the largest cloud")
            v = int(max_num_points)
        order = torch.argsort(self._batch_ids.long(), stable=True)
        starts = torch.cumsum(sizes, 0) - sizes
        sorted_ids = self._batch_ids.long()[order]
        slot = sorted_ids * v + (torch.arange(order.numel(), device=order.device) -
                                 starts[sorted_ids])
        shape = self._batch_shape if self._batch_shape is not None else (self._batch_size,)

        def unflatten(data):
            out = torch.zeros((self._batch_size * v,) + tuple(data.shape[1:]), dtype=data.dtype,
                              device=data.device)
            out[slot] = data[order]
            return out.reshape(tuple(shape) + (v,) + tuple(data.shape[1:]))

        return unflatten

    def flatten_features(self, features):
        """Features [N, C] (returned unchanged) or padded [A1, ..., An, V, C] ->
        [N, C] in the order of the stored points (pylib/pc/utils.py:75-94)."""
        features = torch.as_tensor(features, dtype=_F32, device=self._points.device)
        if features.dim() == 2:
            if features.shape[0] != self._points.shape[0]:
                raise ValueError("expected one feature row per point")
            return features
        sizes = self.get_sizes().reshape(-1).long()
        v, c = features.shape[-2], features.shape[-1]
        keep = (torch.arange(v, device=features.device)[None, :] < sizes[:, None]).reshape(-1)
        by_cloud = features.reshape(-1, c)[keep]          # rows grouped by cloud
        order = torch.argsort(self._batch_ids.long(), stable=True)
        out = torch.empty_like(by_cloud)
        out[order] = by_cloud
        return out

    def format_output(self, features, return_sorted=False, return_padded=False):
        """Layer output [N, C] as is, sorted by cloud id, or zero-padded to
        [A1, ..., An, V, C] (pylib/pc/layers/utils.py:22-49)."""
        if return_padded:
            return self.get_unflatten()(features)
        if return_sorted:
            return features[torch.argsort(self._batch_ids.long(), stable=True)]
        return features

    def get_points(self, id=None, max_num_points=None):
        """The points of cloud `id` (an int or an index into the batch shape), or all
        of them padded to [A1, ..., An, V, D] (PointCloud.py:151-182)."""
        if id is None:
            return self.get_unflatten(max_num_points)(self._points)
        if not isinstance(id, int):
            shape = self._batch_shape if self._batch_shape is not None else (self._batch_size,)
            id = int(torch.arange(self._batch_size).reshape(shape)[tuple(id)].item())
        if id >= self._batch_size or id < -self._batch_size:
            raise IndexError("batch index out of range")
        return self._points[self._batch_ids == id % self._batch_size]


def _sort_keys(keys, key_bits):
    """Stable descending sort -> (sorted keys, int32 permutation)."""
    n, dev = keys.shape[0], keys.device
    sorted_keys = torch.empty(n, dtype=_I64, device=dev)
    sorted_indices = torch.empty(n, dtype=_I32, device=dev)
    ws = _lib.workspace(_lib.lib().mccnn_sort_keys_workspace_bytes(i64(n)), dev)
    _lib.call("sort_keys_descending", stream(), i64(n), cint(key_bits), ptr(keys, _I64),
              ptr(sorted_keys), ptr(sorted_indices), ptr(ws), _lib.csize(ws.numel()))
    return sorted_keys, sorted_indices


_ONE_CALL_GRID = 16384     # points up to which a grid is built by the single-call entry point
_pinned_shape = threading.local()


class Grid:
    """Regular grid over a point cloud (pylib/pc/Grid.py:32-84): grid shape from
    the per-cloud bounding boxes, cell keys, stable descending sort, gathers."""

    def __init__(self, point_cloud, cell_sizes, aabb=None):
        # `aabb` is accepted for the reference's signature; like the reference
        # (Grid.py:42-44) the grid always takes the cloud's own bounding boxes
        L = _lib.lib()
        pc = point_cloud
        dev, n, d, b = pc._points.device, pc._points.shape[0], pc._dimension, pc._batch_size
        self._point_cloud = pc
        self._batch_size = b
        self._cell_sizes = _as_vector(cell_sizes, d, dev)
        self._aabb_min = torch.empty((b, d), dtype=_F32, device=dev)
        self._aabb_max = torch.empty((b, d), dtype=_F32, device=dev)
        self._num_cells = torch.empty(d, dtype=_I32, device=dev)
        self._scaled_aabb_min = torch.empty((b, d), dtype=_F32, device=dev)
        self._inv_cell_sizes = torch.empty(d, dtype=_F32, device=dev)
        self._fast_DS = None
        self._sorted_positions = None
        self._self_neighborhoods = {}
        if 0 < n <= _ONE_CALL_GRID:
            # small clouds are bound by calls and launches: the same five steps in one call
            self._cur_keys = torch.empty(n, dtype=_I64, device=dev)
            self._sorted_keys = torch.empty(n, dtype=_I64, device=dev)
            self._sorted_indices = torch.empty(n, dtype=_I32, device=dev)
            self._sorted_points = torch.empty_like(pc._points)
            self._sorted_batch_ids = torch.empty_like(pc._batch_ids)
            ws = _lib.workspace(L.mccnn_build_grid_workspace_bytes(i64(n)), dev)
            # the grid shape comes back through pinned host memory (one allocation, reused)
            # (per host thread: two threads may build grids at the same time)
            pinned = getattr(_pinned_shape, "buffer", None)
            if pinned is None:
                pinned = _pinned_shape.buffer = torch.empty(16, dtype=_I32, pin_memory=True)
            cells_host = (ctypes.c_int32 * d).from_address(pinned.data_ptr())
            bits_host = ctypes.c_int.from_address(pinned.data_ptr() + 32)
            _lib.call("build_grid", stream(), i64(n), cint(d), ptr(pc._points, _F32),
                      ptr(pc._batch_ids, _I32), cint(b), ptr(self._cell_sizes),
                      ptr(self._aabb_min), ptr(self._aabb_max), ptr(self._num_cells),
                      ptr(self._scaled_aabb_min), ptr(self._inv_cell_sizes), ptr(self._cur_keys),
                      ptr(self._sorted_keys), ptr(self._sorted_indices), ptr(self._sorted_points),
                      ptr(self._sorted_batch_ids), ptr(ws), _lib.csize(ws.numel()), cells_host,
                      ctypes.byref(bits_host))
            self._num_cells_host = [int(v) for v in cells_host]
            self._key_bits = int(bits_host.value)
            return
        _lib.call("grid_setup", stream(), i64(n), cint(d), ptr(pc._points, _F32), ptr(pc._batch_ids, _I32), cint(b),
            ptr(self._cell_sizes), ptr(self._aabb_min), ptr(self._aabb_max),
            ptr(self._num_cells), ptr(self._scaled_aabb_min), ptr(self._inv_cell_sizes))
        self._cur_keys = tfg_custom_ops.compute_keys(
            pc._points, pc._batch_ids, self._scaled_aabb_min, self._num_cells,
            self._inv_cell_sizes)
        # host copy of the grid shape: sizes the key width and the column table
        self._num_cells_host = [int(v) for v in self._num_cells.tolist()]
        total = b
        for v in self._num_cells_host:
            total *= v
        self._key_bits = max(1, (total - 1).bit_length())
        self._sorted_keys, self._sorted_indices = _sort_keys(self._cur_keys, self._key_bits)
        self._sorted_points = torch.empty_like(pc._points)
        self._sorted_batch_ids = torch.empty_like(pc._batch_ids)
        _lib.call("gather_points", stream(), i64(n), cint(d), ptr(pc._points), ptr(pc._batch_ids),
            ptr(self._sorted_indices), ptr(self._sorted_points), ptr(self._sorted_batch_ids))

    def sorted_positions(self):
        """Inverse of the sort: position of every original point in the sorted order."""
        if self._sorted_positions is None:
            n, dev = self._sorted_indices.shape[0], self._sorted_indices.device
            inv = torch.empty(n, dtype=_I32, device=dev)
            inv[self._sorted_indices.long()] = torch.arange(n, dtype=_I32, device=dev)
            self._sorted_positions = inv
        return self._sorted_positions

    def self_neighborhood(self, radii, max_neighbors=0):
        """The neighbourhood of the grid's sorted points among themselves for these
        radii, built once and shared (densities, grid-ordered view, same-cloud
        convolutions)."""
        key = (_host_values(radii), int(max_neighbors))
        if key not in self._self_neighborhoods:
            self._self_neighborhoods[key] = Neighborhood(self, radii, None, max_neighbors)
        return self._self_neighborhoods[key]

    def get_DS(self):
        if self._fast_DS is None:
            self._fast_DS = tfg_custom_ops.build_grid_ds(
                self._sorted_keys, self._num_cells, self._num_cells_host, self._batch_size)
        return self._fast_DS


class _SortedView:
    """A neighbourhood with input points and centres both numbered in grid-cell
    order, the layout the layer kernels run on: consecutive centres then share
    their neighbours and every neighbour list is a few contiguous index runs, so
    the feature gathers hit in L2 instead of walking the whole table at random.

    points_in / points_out   coordinates in that order
    point_order [N_in]       position -> original point id (the grid's sort)
    centre_order [N_out]     slot -> original centre id, None if the centres
                             already are the grid's sorted points
    table [M,2], ranges      pairs (point position, centre slot) grouped by slot
    table_t [M,2], ranges_t  pairs (centre slot, point position) grouped by point
    """

    def __init__(self, nbh):
        grid, samples = nbh._grid, nbh._point_cloud_sampled
        self.points_in = grid._sorted_points
        self.point_rows = grid._sorted_indices           # int32, for kernels
        self._point_order = self._centre_order = None    # their int64 forms, on first use
        n_out = samples._points.shape[0]
        if nbh._equal_samples:
            self.centre_rows = None
            self.points_out = grid._sorted_points
            self.table, self.ranges = nbh._neighbors, nbh._samples_neigh_ranges
        elif nbh._self_neighborhood is not None:     # same cloud: the shared sorted search
            own = nbh._self_neighborhood
            self.centre_rows = grid._sorted_indices
            self.points_out = grid._sorted_points
            self.table, self.ranges = own._neighbors, own._samples_neigh_ranges
        else:
            order = nbh.compute_centre_order()
            self.centre_rows = order
            self.points_out = samples._points[self.centre_order].contiguous()
            L = _lib.lib()
            L.mccnn_reorder_neighbors_workspace_bytes.restype = _lib.csize
            dev = nbh._neighbors.device
            ws = _lib.workspace(L.mccnn_reorder_neighbors_workspace_bytes(i64(n_out)), dev)
            self.ranges = torch.empty_like(nbh._samples_neigh_ranges)
            self.table = torch.empty_like(nbh._neighbors)
            _lib.call("reorder_neighbors", stream(), i64(n_out),
                      ptr(nbh._samples_neigh_ranges, _I32), i64(nbh._neighbors.shape[0]),
                      ptr(nbh._neighbors, _I32), ptr(order, _I32), ptr(ws),
                      _lib.csize(ws.numel()), ptr(self.ranges), ptr(self.table))
        if (nbh._equal_samples or nbh._self_neighborhood is not None) and nbh.max_neighbors == 0:
            # An untruncated self-neighbourhood is symmetric (the distance test is exact
            # under negation): the rows (x, p) of segment p are at once "x is a neighbour
            # of centre p" and "p is a neighbour of centre x", so the table is its own
            # transpose.
            self.table_t, self.ranges_t = self.table, self.ranges
        else:
            self.ranges_t, pair_order = tfg_custom_ops.transpose_neighbors(
                self.table, self.points_in.shape[0])
            self.table_t = torch.empty_like(self.table)
            _lib.call("swapped_pairs", stream(), i64(self.table.shape[0]), ptr(self.table, _I32),
                      ptr(pair_order, _I32), ptr(self.table_t))
        self._pdf_key, self.pdf, self.pdf_t = None, None, None

    @property
    def point_order(self):
        """position -> original point id as int64 (for torch indexing)."""
        if self._point_order is None:
            self._point_order = self.point_rows.long()
        return self._point_order

    @property
    def centre_order(self):
        """slot -> original centre id as int64, None if the centres are the sorted points."""
        if self._centre_order is None and self.centre_rows is not None:
            self._centre_order = self.centre_rows.long()
        return self._centre_order

    def pair_pdf(self, nbh):
        """Per-pair densities of `table` and `table_t` (the neighbour point's)."""
        per_point = nbh._pdf_per_point
        # compute_pdf bumps the generation: a key made of the density tensor's address
        # could match a later tensor that the allocator put in the same place
        key = nbh._pdf_generation
        if self.pdf is None or key != self._pdf_key:
            m, dev = self.table.shape[0], self.table.device
            if per_point is None:
                self.pdf = self.pdf_t = torch.ones(m, dtype=_F32, device=dev)
            else:
                per_point = per_point.detach()
                self.pdf = torch.empty(m, dtype=_F32, device=dev)
                self.pdf_t = torch.empty(m, dtype=_F32, device=dev)
                for out, table, column in ((self.pdf, self.table, 0), (self.pdf_t, self.table_t, 1)):
                    _lib.call("gather_pdf_column", stream(), i64(m), ptr(table, _I32), cint(column),
                              ptr(per_point, _F32), ptr(out))
                if nbh._pdf_normalize:
                    # Neighborhood.py:288-293: divided by the size of the pair's
                    # neighbourhood, i.e. the pair count of its centre (column 1 of
                    # `table`, column 0 of `table_t`)
                    ends = self.ranges.long()
                    counts = (ends - torch.cat([ends.new_zeros(1), ends[:-1]])).to(_F32)
                    self.pdf = self.pdf / counts[self.table[:, 1].long()]
                    self.pdf_t = self.pdf_t / counts[self.table_t[:, 0].long()]
            self._pdf_key = key
        return self.pdf, self.pdf_t


class Neighborhood:
    """Neighbour pairs of the centres `point_cloud_sample` (default: the grid's
    own sorted points) inside `grid` (pylib/pc/Neighborhood.py:218-311)."""

    def __init__(self, grid, radius, point_cloud_sample=None, max_neighbors=0, lazy=False):
        """`lazy` puts the search off until the pair table is first read (a cell-average
        hierarchy keeps a neighbourhood per level that it never reads itself)."""
        d = grid._point_cloud._dimension
        dev = grid._sorted_points.device
        self._radii = _as_vector(radius, d, dev)
        self._grid = grid
        if point_cloud_sample is None:
            self._equal_samples = True
            self._point_cloud_sampled = PointCloud(grid._sorted_points, grid._sorted_batch_ids,
                                                   grid._batch_size)
        else:
            self._equal_samples = False
            self._point_cloud_sampled = point_cloud_sample
        self.max_neighbors = max_neighbors
        self._inv_radii = _reciprocal(self._radii)
        s = self._point_cloud_sampled
        self._self_neighborhood = None
        self._table = self._ranges = self._original = None
        if point_cloud_sample is grid._point_cloud:
            # The centres are the grid's own points in the caller's order: search once
            # from the sorted points (consecutive centres then walk the same cells;
            # the same search also serves the densities and the grid-ordered view of
            # the layers).  The table in the caller's centre order is the same
            # segments regrouped (the pairs of a centre depend on its coordinates
            # only); it is built when somebody asks for it, which the layers on the
            # grid-ordered view never do.
            self._self_neighborhood = grid.self_neighborhood(self._radii, max_neighbors)
        elif not lazy:
            self._search()
        self._pdf = None
        self._pdf_per_point = None
        self._pdf_args = None
        self._pdf_normalize = False
        self._pdf_generation = 0
        # optional visiting order of the centres for the projection kernels
        self._centre_order = None
        self._transposed_pairs = None
        self._sorted_view = None
        self._transposed = None

    def _search(self):
        s, grid = self._point_cloud_sampled, self._grid
        self._ranges, self._table = tfg_custom_ops.find_neighbors(
            s._points, s._batch_ids, grid._sorted_points, grid._sorted_keys, grid.get_DS(),
            grid._num_cells, grid._scaled_aabb_min, grid._inv_cell_sizes, self._inv_radii,
            self.max_neighbors)

    def _regroup(self):
        if self._self_neighborhood is None:      # a search that was put off
            return self._search()
        own, grid = self._self_neighborhood, self._grid
        n = self._point_cloud_sampled._points.shape[0]
        dev = own._neighbors.device
        L = _lib.lib()
        ws = _lib.workspace(L.mccnn_reorder_neighbors_workspace_bytes(i64(n)), dev)
        self._ranges = torch.empty_like(own._samples_neigh_ranges)
        self._table = torch.empty_like(own._neighbors)
        _lib.call("reorder_neighbors", stream(), i64(n), ptr(own._samples_neigh_ranges, _I32),
                  i64(own._neighbors.shape[0]), ptr(own._neighbors, _I32),
                  ptr(grid.sorted_positions(), _I32), ptr(ws), _lib.csize(ws.numel()),
                  ptr(self._ranges), ptr(self._table))

    @property
    def _neighbors(self):
        """[M, 2] pairs (sorted point index, centre index), grouped by centre."""
        if self._table is None:
            self._regroup()
        return self._table

    @property
    def _samples_neigh_ranges(self):
        """[N_out] inclusive end offset of every centre's pairs."""
        if self._ranges is None:
            self._regroup()
        return self._ranges

    @property
    def _original_neigh_ids(self):
        """The pairs addressed by original point ids (Neighborhood.py:246-250);
        built on first use."""
        if self._original is None:
            nb = self._neighbors
            self._original = torch.empty_like(nb)
            _lib.call("original_neighbor_ids", stream(), i64(nb.shape[0]), ptr(nb, _I32),
                      ptr(self._grid._sorted_indices, _I32), ptr(self._original))
        return self._original

    def transposed_pairs(self):
        """(point_ranges, pair_order): the pairs grouped by neighbour point, used by
        the atomic-free feature gradients; built on first use and kept."""
        if self._transposed_pairs is None:
            self._transposed_pairs = tfg_custom_ops.transpose_neighbors(
                self._original_neigh_ids, self._grid._point_cloud._points.shape[0])
        return self._transposed_pairs

    def get_grid(self):
        """The grid used for the neighbour search (Neighborhood.py:313-316)."""
        return self._grid

    def transpose(self):
        """The neighbourhood with centres and neighbour points switched
        (Neighborhood.py:318-329): itself for a self-neighbourhood, otherwise a
        grid over the centres searched from the original points; built once."""
        if self._transposed is None:
            if self._equal_samples:
                self._transposed = self
            else:
                grid = Grid(self._point_cloud_sampled, self._radii)
                self._transposed = Neighborhood(grid, self._radii, self._grid._point_cloud)
        return self._transposed

    def sorted_view(self):
        """The neighbourhood re-expressed in grid order on both sides (built on
        first use and kept): see `_SortedView`."""
        if self._sorted_view is None:
            self._sorted_view = _SortedView(self)
        return self._sorted_view

    def compute_centre_order(self):
        """Rank the centres by their cell key in the grid (a scheduling hint for
        `basis_proj`; the grid's own sorted points already are in that order)."""
        s, grid = self._point_cloud_sampled, self._grid
        if not self._equal_samples and s._points.shape[0] > 0:
            keys = tfg_custom_ops.compute_keys(s._points, s._batch_ids, grid._scaled_aabb_min,
                                               grid._num_cells, grid._inv_cell_sizes)
            self._centre_order = _sort_keys(keys, grid._key_bits)[1]
        return self._centre_order

    def compute_pdf(self, bandwidth=0.2, mode=KDEMode.constant, normalize=False):
        """Densities of the grid's points from their self-neighbourhood
        (Neighborhood.py:257-293); the per-pair values follow on `get_pdf()`."""
        d = self._grid._point_cloud._dimension
        dev = self._grid._sorted_points.device
        self._pdf = None
        self._pdf_args = (bandwidth, mode)
        self._pdf_normalize = bool(normalize)
        self._pdf_generation += 1
        if mode == KDEMode.no_pdf:
            self._pdf_per_point = None
            return
        nbh = self if self._equal_samples else self._grid.self_neighborhood(self._radii)
        bw = _as_vector(bandwidth, d, dev)
        self._pdf_per_point = tfg_custom_ops.compute_pdf_with_pt_grads(
            self._grid._sorted_points, nbh._neighbors, nbh._samples_neigh_ranges,
            _reciprocal(bw), nbh._inv_radii, mode.value,
            symmetric=nbh._equal_samples and nbh.max_neighbors == 0)

    def point_pdf(self, **kwargs):
        """Density per sorted point (None with KDEMode.no_pdf), computed on first use
        with `kwargs` as for `compute_pdf`."""
        if self._pdf_args is None:
            self.compute_pdf(**kwargs)
        return self._pdf_per_point

    def get_pdf(self, **kwargs):
        """Density of the neighbour point of every pair of `_neighbors`
        (Neighborhood.py:287)."""
        per_point = self.point_pdf(**kwargs)
        if self._pdf is None:
            nb = self._neighbors
            if per_point is None:
                self._pdf = torch.ones(nb.shape[0], dtype=_F32, device=nb.device)
            else:
                self._pdf = torch.empty(nb.shape[0], dtype=_F32, device=nb.device)
                _lib.call("gather_pdf", stream(), i64(nb.shape[0]), ptr(nb, _I32),
                          ptr(per_point.detach(), _F32), ptr(self._pdf))
            if self._pdf_normalize:       # divided by the size of the pair's neighbourhood
                ends = self._samples_neigh_ranges.long()
                counts = (ends - torch.cat([ends.new_zeros(1), ends[:-1]])).to(_F32)
                self._pdf = self._pdf / counts[nb[:, 1].long()]
        return self._pdf


_SAMPLE_MODES = {"average": 1, "cell average": 1, "cell_average": 1,
                 "poisson": 0, "poisson disk": 0, "poisson_disk": 0}


def sample(neighborhood, sample_mode="poisson"):
    """pylib/pc/sampling.py:123-150 -> (PointCloud, original indices or None)."""
    mode = _SAMPLE_MODES[sample_mode.lower()]
    g = neighborhood._grid
    if mode == 1:
        # cell averages read the keys only: no reason to run the neighbour search that
        # the (lazily built) pair table of `neighborhood` would cost
        dev = g._sorted_points.device
        pairs = torch.empty((0, 2), dtype=_I32, device=dev)
        ranges = torch.zeros(g._sorted_points.shape[0], dtype=_I32, device=dev)
    else:
        pairs, ranges = neighborhood._neighbors, neighborhood._samples_neigh_ranges
    pts, bids, idx = tfg_custom_ops.sampling(
        g._sorted_points, g._sorted_batch_ids, g._sorted_keys, g._num_cells, pairs, ranges, mode)
    original = None
    if mode == 0:
        original = torch.empty_like(idx)
        _lib.call("gather_i32", stream(), i64(idx.shape[0]), ptr(g._sorted_indices, _I32), ptr(idx, _I32),
            ptr(original))
    return PointCloud(pts, bids, g._batch_size), original


def poisson_disk_sampling(point_cloud, radius=None, neighborhood=None, return_ids=False):
    """Poisson-disk sample of a point cloud (pylib/pc/sampling.py:31-78) -> PointCloud
    (and the original indices of the kept points).  The reference passes the mode
    of the other sampler here (:67, and :114 below); this follows the names."""
    if radius is None and neighborhood is None:
        raise ValueError("Missing Argument! Either radius or neighborhood must be given!")
    if neighborhood is None:
        radii = _as_vector(radius, point_cloud._dimension, point_cloud._points.device)
        neighborhood = Neighborhood(Grid(point_cloud, radii), radii)
    cloud, ids = sample(neighborhood, "poisson")
    return (cloud, ids) if return_ids else cloud


def cell_average_sampling(point_cloud, cell_sizes=None, grid=None):
    """One point per occupied cell, the mean of the cell's points
    (pylib/pc/sampling.py:81-120) -> PointCloud."""
    if cell_sizes is None and grid is None:
        raise ValueError("Missing Argument! Either cell_sizes or grid must be given!")
    if grid is None:
        grid = Grid(point_cloud, _as_vector(cell_sizes, point_cloud._dimension,
                                            point_cloud._points.device))
    return sample(Neighborhood(grid, grid._cell_sizes, lazy=True), "average")[0]


class PointHierarchy:
    """Successively sampled point clouds (pylib/pc/PointHierarchy.py:40-98)."""

    def __init__(self, point_cloud, cell_sizes, sample_mode="poisson"):
        self._point_clouds = [point_cloud]
        self._cell_sizes = []
        self._neighborhoods = []
        self._sample_indices = []
        cur = point_cloud
        for cs in cell_sizes:
            cs = _as_vector(cs, point_cloud._dimension, point_cloud._points.device)
            self._cell_sizes.append(cs)
            grid = Grid(cur, cs)
            nbh = Neighborhood(grid, cs, lazy=_SAMPLE_MODES[sample_mode.lower()] == 1)
            cur, idx = sample(nbh, sample_mode)
            self._neighborhoods.append(nbh)
            self._point_clouds.append(cur)
            self._sample_indices.append(idx)

    def get_neighborhood(self, i=None, transposed=False):
        """Neighbourhood between level i and i+1, or all of them
        (PointHierarchy.py:159-183); `transposed` gives level i+1 -> i."""
        if i is None:
            return [nb.transpose() for nb in self._neighborhoods] if transposed \
                else self._neighborhoods
        return self._neighborhoods[i].transpose() if transposed else self._neighborhoods[i]

    def get_points(self, batch_id=None, max_num_points=None):
        """Per level: the points of cloud `batch_id`, or all of them padded
        (PointHierarchy.py:100-122)."""
        return [c.get_points(batch_id, max_num_points) for c in self._point_clouds]

    def get_sizes(self):
        """Per level: points per cloud (PointHierarchy.py:124-138)."""
        return [c.get_sizes() for c in self._point_clouds]

    def set_batch_shape(self, batch_shape):
        """PointHierarchy.py:140-157."""
        for c in self._point_clouds:
            c.set_batch_shape(batch_shape)

    def __getitem__(self, index):
        return self._point_clouds[index]

    def __len__(self):
        return len(self._point_clouds)
