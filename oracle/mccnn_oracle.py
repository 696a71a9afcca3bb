"""numpy front-end of the CPU oracle.  TEST INFRASTRUCTURE ONLY.

Loads ``libmccnn_oracle.so`` (built from ``mccnn_oracle.c`` by the Makefile in
this directory) and adds the caller-side glue of the reference in numpy, with
the same fp32 expressions in the same order:

* bounding boxes            pylib/pc/PointCloud.py:38-43
* grid shape, keys, sort    pylib/pc/Grid.py:44-64
* scaled box / reciprocals  pylib/pc/custom_ops/custom_ops_wrapper.py:37-43,95-104
* neighbourhoods            pylib/pc/Neighborhood.py:218-250
* pdf per pair              pylib/pc/Neighborhood.py:281-287
* layers                    pylib/pc/layers/MCConv.py:137-194, KPConv.py:165-232,
                            Pooling.py:25-166

Only tests, the smoke check and the cpu-baseline leg of the benchmark may import
this module; the product never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_i64 = ctypes.c_int64
_int = ctypes.c_int


def build():
    """Compile the C oracle with gcc (a few seconds)."""
    subprocess.run(["make", "-C", _HERE, "-s", "-B"], check=True)


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libmccnn_oracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
        _LIB.orc_find_neighbors_count.restype = _i64
        _LIB.orc_unique_keys.restype = _i64
        _LIB.orc_sampling_poisson.restype = _i64
    return _LIB


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


# --------------------------------------------------------------------------- ops


def compute_keys(points, batch_ids, scaled_aabb_min, num_cells, inv_cell_sizes):
    points, batch_ids = _f32(points), _i32(batch_ids)
    smin, nc, ic = _f32(scaled_aabb_min), _i32(num_cells), _f32(inv_cell_sizes)
    n, d = points.shape
    keys = np.empty(n, dtype=np.int64)
    lib().orc_compute_keys(_int(d), _i64(n), _ptr(points), _ptr(batch_ids),
                           _ptr(smin), _ptr(nc), _ptr(ic), _ptr(keys))
    return keys


def sort_keys_descending(keys):
    """tf.argsort(keys, 'DESCENDING') (Grid.py:56-57): ties keep the lower index."""
    idx = np.argsort(-np.asarray(keys, dtype=np.int64), kind="stable").astype(np.int32)
    return idx


def build_grid_ds(sorted_keys, num_cells, batch_size):
    sorted_keys = np.ascontiguousarray(sorted_keys, dtype=np.int64)
    nc = _i32(num_cells)
    ds = np.empty((batch_size, nc[0], nc[1], 2), dtype=np.int32)
    lib().orc_build_grid_ds(_int(len(nc)), _i64(len(sorted_keys)), _ptr(sorted_keys),
                            _ptr(nc), _int(batch_size), _ptr(ds))
    return ds


def find_neighbors(samples, sample_batch_ids, points, point_keys, grid_ds, num_cells,
                   scaled_aabb_min, inv_cell_sizes, inv_radii, max_neighs=0):
    samples, sb = _f32(samples), _i32(sample_batch_ids)
    points = _f32(points)
    keys = np.ascontiguousarray(point_keys, dtype=np.int64)
    ds, nc = _i32(grid_ds), _i32(num_cells)
    smin, ic, ir = _f32(scaled_aabb_min), _f32(inv_cell_sizes), _f32(inv_radii)
    ns, d = samples.shape
    ranges = np.empty(ns, dtype=np.int32)
    args = (_int(d), _i64(ns), _ptr(samples), _ptr(sb), _i64(len(points)), _ptr(points),
            _ptr(keys), _ptr(ds), _ptr(nc), _ptr(smin), _ptr(ic), _ptr(ir),
            _int(max_neighs))
    m = lib().orc_find_neighbors_count(*args, _ptr(ranges))
    if m >= 2 ** 31 - 1:        # the int32 end offsets of the op contract have wrapped
        raise ValueError("find_neighbors: %d pairs do not fit the int32 offsets" % m)
    nbrs = np.empty((m, 2), dtype=np.int32)
    lib().orc_find_neighbors_fill(*args, _ptr(ranges), _ptr(nbrs))
    return ranges, nbrs


def compute_pdf(points, neighbors, ranges, inv_bandwidth, inv_radii, mode=0):
    points, nb, rg = _f32(points), _i32(neighbors), _i32(ranges)
    ib, ir = _f32(inv_bandwidth), _f32(inv_radii)
    n, d = points.shape
    pdf = np.empty(n, dtype=np.float64)
    lib().orc_compute_pdf(_int(d), _i64(n), _ptr(points), _ptr(nb), _ptr(rg), _ptr(ib),
                          _ptr(ir), _int(mode), _ptr(pdf))
    return pdf


def compute_pdf_pt_grads(points, neighbors, ranges, inv_bandwidth, inv_radii,
                         pdf_grads, mode=0):
    points, nb, rg = _f32(points), _i32(neighbors), _i32(ranges)
    ib, ir, pg = _f32(inv_bandwidth), _f32(inv_radii), _f32(pdf_grads)
    n, d = points.shape
    out = np.empty((n, d), dtype=np.float64)
    lib().orc_compute_pdf_pt_grads(_int(d), _i64(n), _ptr(points), _ptr(nb), _ptr(rg),
                                   _ptr(ib), _ptr(ir), _ptr(pg), _int(mode), _ptr(out))
    return out


def basis_proj(basis, features, neighbors, ranges, with_magnitude=False):
    basis, features = _f32(basis), _f32(features)
    nb, rg = _i32(neighbors), _i32(ranges)
    n_out, (c, k) = len(rg), (features.shape[1], basis.shape[1])
    out = np.empty((n_out, c, k), dtype=np.float64)
    mag = np.empty((n_out, c, k), dtype=np.float64) if with_magnitude else None
    lib().orc_basis_proj(_i64(n_out), _int(c), _int(k), _ptr(basis), _ptr(features),
                         _ptr(nb), _ptr(rg), _ptr(out),
                         _ptr(mag) if with_magnitude else None)
    return (out, mag) if with_magnitude else out


def basis_proj_grads(basis, features, neighbors, ranges, in_grad):
    basis, features, in_grad = _f32(basis), _f32(features), _f32(in_grad)
    nb, rg = _i32(neighbors), _i32(ranges)
    n_out, (c, k) = len(rg), (features.shape[1], basis.shape[1])
    dbasis = np.zeros(basis.shape, dtype=np.float64)
    dfeat = np.empty(features.shape, dtype=np.float64)
    lib().orc_basis_proj_grads(_i64(len(features)), _i64(n_out), _int(c), _int(k),
                               _ptr(basis), _ptr(features), _ptr(nb), _ptr(rg),
                               _ptr(in_grad), _ptr(dbasis), _ptr(dfeat))
    return dbasis, dfeat


def basis_proj_f32(basis, features, neighbors, ranges):
    basis, features = _f32(basis), _f32(features)
    nb, rg = _i32(neighbors), _i32(ranges)
    n_out, (c, k) = len(rg), (features.shape[1], basis.shape[1])
    out = np.empty((n_out, c, k), dtype=np.float32)
    lib().orc_basis_proj_f32(_i64(n_out), _int(c), _int(k), _ptr(basis), _ptr(features),
                             _ptr(nb), _ptr(rg), _ptr(out))
    return out


def basis_proj_grads_f32(basis, features, neighbors, ranges, in_grad):
    basis, features, in_grad = _f32(basis), _f32(features), _f32(in_grad)
    nb, rg = _i32(neighbors), _i32(ranges)
    n_out, (c, k) = len(rg), (features.shape[1], basis.shape[1])
    dbasis = np.zeros(basis.shape, dtype=np.float32)
    dfeat = np.empty(features.shape, dtype=np.float32)
    lib().orc_basis_proj_grads_f32(_i64(len(features)), _i64(n_out), _int(c), _int(k),
                                   _ptr(basis), _ptr(features), _ptr(nb), _ptr(rg),
                                   _ptr(in_grad), _ptr(dbasis), _ptr(dfeat))
    return dbasis, dfeat


def sampling(points, batch_ids, point_keys, num_cells, neighbors, ranges, mode):
    """sampling_ops.cpp:131-194.  mode 0: Poisson disk, mode 1: cell average.

    Returns (points [S,D], batch ids [S], indices [S]); the indices refer to the
    sorted order.  In mode 1 the third value is the first index of each cell
    (custom_ops_tf.py:318); the reference's native op leaves it unset.
    """
    points, bids = _f32(points), _i32(batch_ids)
    keys = np.ascontiguousarray(point_keys, dtype=np.int64)
    nc, nb, rg = _i32(num_cells), _i32(neighbors), _i32(ranges)
    n, d = points.shape
    if mode not in (0, 1):
        raise ValueError("sampling mode must be 0 or 1")
    n_cells = lib().orc_unique_keys(_i64(n), _ptr(keys), None)
    first = np.empty(n_cells, dtype=np.int32)
    lib().orc_unique_keys(_i64(n), _ptr(keys), _ptr(first))
    if mode == 1:
        out_pts = np.empty((n_cells, d), dtype=np.float32)
        out_b = np.empty(n_cells, dtype=np.int32)
        lib().orc_sampling_avg(_int(d), _i64(n), _i64(n_cells), _ptr(points), _ptr(keys),
                               _ptr(nc), _ptr(first), _ptr(out_pts), _ptr(out_b))
        return out_pts, out_b, first
    used = np.empty(n, dtype=np.int32)
    lib().orc_sampling_poisson(_int(d), _i64(n), _i64(n_cells), _ptr(keys), _ptr(nc),
                               _ptr(nb), _ptr(rg), _ptr(first), _ptr(used))
    sel = np.nonzero(used)[0].astype(np.int32)
    return points[sel], bids[sel], sel


# -------------------------------------------------------------------- caller glue


class Grid:
    """pylib/pc/Grid.py:32-84 in numpy (fp32 expressions kept in order)."""

    def __init__(self, points, batch_ids, batch_size, cell_sizes):
        points, batch_ids = _f32(points), _i32(batch_ids)
        d = points.shape[1]
        cell = _f32(np.broadcast_to(np.asarray(cell_sizes, dtype=np.float32).reshape(-1)
                                    if np.ndim(cell_sizes) else
                                    np.float32(cell_sizes), (d,)))
        amin = np.full((batch_size, d), np.inf, dtype=np.float32)
        amax = np.full((batch_size, d), -np.inf, dtype=np.float32)
        np.minimum.at(amin, batch_ids, points)
        np.maximum.at(amax, batch_ids, points)
        # PointCloud.py:38-43
        self.aabb_min = (amin - np.float32(1e-9)).astype(np.float32)
        self.aabb_max = (amax + np.float32(1e-9)).astype(np.float32)
        # Grid.py:44-48
        sizes = (self.aabb_max - self.aabb_min).astype(np.float32)
        per_batch = np.ceil((sizes / cell).astype(np.float32)).astype(np.int32)
        self.num_cells = np.maximum(per_batch.max(axis=0), 1).astype(np.int32)
        self.cell_sizes = cell
        self.batch_size = batch_size
        self.points, self.batch_ids = points, batch_ids
        # custom_ops_wrapper.py:37-43
        self.scaled_aabb_min = (self.aabb_min / cell).astype(np.float32)
        self.inv_cell_sizes = (np.float32(1.0) / cell).astype(np.float32)
        self.keys = compute_keys(points, batch_ids, self.scaled_aabb_min,
                                 self.num_cells, self.inv_cell_sizes)
        self.sorted_indices = sort_keys_descending(self.keys)
        self.sorted_keys = self.keys[self.sorted_indices]
        self.sorted_points = points[self.sorted_indices]
        self.sorted_batch_ids = batch_ids[self.sorted_indices]
        self._ds = None

    def get_ds(self):
        if self._ds is None:
            self._ds = build_grid_ds(self.sorted_keys, self.num_cells, self.batch_size)
        return self._ds


class Neighborhood:
    """pylib/pc/Neighborhood.py:218-293 in numpy."""

    def __init__(self, grid, radii, samples=None, sample_batch_ids=None, max_neighbors=0):
        d = grid.points.shape[1]
        self.radii = _f32(np.broadcast_to(np.asarray(radii, dtype=np.float32).reshape(-1),
                                          (d,)))
        self.grid = grid
        self.equal_samples = samples is None
        if samples is None:
            samples, sample_batch_ids = grid.sorted_points, grid.sorted_batch_ids
        self.samples, self.sample_batch_ids = _f32(samples), _i32(sample_batch_ids)
        self.inv_radii = (np.float32(1.0) / self.radii).astype(np.float32)
        self.ranges, self.neighbors = find_neighbors(
            self.samples, self.sample_batch_ids, grid.sorted_points, grid.sorted_keys,
            grid.get_ds(), grid.num_cells, grid.scaled_aabb_min, grid.inv_cell_sizes,
            self.inv_radii, max_neighbors)
        self._original = None

    @property
    def original_neigh_ids(self):
        """Neighborhood.py:246-250: the pairs with the points' ids before the sort (built
        on first use: the gather takes seconds at 10^8 pairs)."""
        if self._original is None:
            self._original = np.empty_like(self.neighbors)
            self._original[:, 0] = np.take(self.grid.sorted_indices, self.neighbors[:, 0])
            self._original[:, 1] = self.neighbors[:, 1]
        return self._original

    def pdf_per_pair(self, bandwidth=0.2, mode=0):
        d = self.grid.points.shape[1]
        bw = _f32(np.broadcast_to(np.asarray(bandwidth, dtype=np.float32).reshape(-1),
                                  (d,)))
        inv_bw = (np.float32(1.0) / bw).astype(np.float32)
        nbh = self if self.equal_samples else Neighborhood(self.grid, self.radii)
        pdf = compute_pdf(self.grid.sorted_points, nbh.neighbors, nbh.ranges, inv_bw,
                          nbh.inv_radii, mode)
        return pdf[self.neighbors[:, 0]]


def segment_starts(ranges):
    ranges = np.asarray(ranges)
    return np.concatenate([[0], ranges[:-1]]).astype(np.int64)


_ACT = {
    "relu": lambda x: np.maximum(x, 0.0),
    "leaky_relu": lambda x: np.where(x > 0, x, 0.2 * x),
    "elu": lambda x: np.where(x > 0, x, np.expm1(np.minimum(x, 0.0))),
}


def mc_basis(points_diff, pdf, weights, biases, activation="relu"):
    """MCConv.py:163-171 for a one-hidden-layer kernel: [M, num_mlps*H] in float64."""
    x = np.asarray(points_diff, dtype=np.float64)
    w = np.asarray(weights, dtype=np.float64)      # [num_mlps, D, H]
    b = np.asarray(biases, dtype=np.float64)       # [num_mlps, 1, H]
    h = _ACT[activation](np.einsum("md,ldh->lmh", x, w) + b)
    h = np.transpose(h, (1, 0, 2)).reshape(x.shape[0], -1)
    return h / np.asarray(pdf, dtype=np.float64).reshape(-1, 1)


def mc_conv_forward(features, points_in, points_out, nbh, pdf_pair, weights, biases,
                    final_weights, radius, activation="relu"):
    """MCConv.py:137-194 and :264-274 in float64; returns (out, basis, projected)."""
    orig = nbh.original_neigh_ids
    d = points_in.shape[1]
    radii = np.full(d, np.float32(radius), dtype=np.float32)
    diff = (_f32(points_in)[orig[:, 0]] - _f32(points_out)[orig[:, 1]]) / radii
    basis = mc_basis(diff, pdf_pair, weights, biases, activation)
    proj = basis_proj(basis.astype(np.float32), features, orig, nbh.ranges)
    num_mlps, _, hidden = np.asarray(weights).shape
    c = features.shape[1]
    p = proj.reshape(-1, c, num_mlps, hidden).transpose(2, 0, 1, 3)
    p = p.reshape(num_mlps, -1, c * hidden)
    out = np.einsum("lnk,lko->lno", p, np.asarray(final_weights, dtype=np.float64))
    out = out.transpose(1, 0, 2).reshape(proj.shape[0], -1)
    return out, basis, proj


def kp_basis(points_diff, kernel_points, sigma, kind="linear", offsets=None):
    """KPConv.py:29-57,193-198: [M, K] kernel-point weights in float64."""
    x = np.asarray(points_diff, dtype=np.float64)[:, None, :]
    kp = np.asarray(kernel_points, dtype=np.float64)[None, :, :]
    if offsets is not None:
        kp = kp + np.asarray(offsets, dtype=np.float64)
    dist = np.linalg.norm(x - kp, axis=2)
    if kind == "linear":
        return np.maximum(1.0 - dist / sigma, 0.0), dist
    s = sigma / 3.0
    return np.exp(-(dist / s) ** 2), dist


def local_pool(features, original_neigh_ids, n_out, kind="max"):
    """Pooling.py:150-161: unsorted_segment_max / _mean over the neighbour pairs."""
    f = np.asarray(features, dtype=np.float64)[original_neigh_ids[:, 0]]
    seg = original_neigh_ids[:, 1]
    if kind == "max":
        out = np.full((n_out, f.shape[1]), np.finfo(np.float32).min, dtype=np.float64)
        np.maximum.at(out, seg, f)
        return out
    out = np.zeros((n_out, f.shape[1]), dtype=np.float64)
    np.add.at(out, seg, f)
    cnt = np.bincount(seg, minlength=n_out).astype(np.float64)
    return out / np.maximum(cnt, 1.0)[:, None]


def global_pool(features, batch_ids, batch_size, kind="max"):
    """Pooling.py:54-57, 93-96."""
    f = np.asarray(features, dtype=np.float64)
    if kind == "max":
        out = np.full((batch_size, f.shape[1]), np.finfo(np.float32).min,
                      dtype=np.float64)
        np.maximum.at(out, batch_ids, f)
        return out
    out = np.zeros((batch_size, f.shape[1]), dtype=np.float64)
    np.add.at(out, batch_ids, f)
    cnt = np.bincount(batch_ids, minlength=batch_size).astype(np.float64)
    return out / np.maximum(cnt, 1.0)[:, None]
