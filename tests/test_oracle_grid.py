"""Pins the integer half of the CPU oracle (keys, sort order, grid table,
neighbour lists) against independent statements of the same results: the numpy
formulas the reference's own tests use, closed-form lattice answers, brute force
and scipy's k-d tree.  No GPU needed."""
import numpy as np
import pytest
from scipy.spatial import cKDTree


def _cloud(rng, batch, n, d, scale=1.0):
    pts = (rng.random((n, d)) * scale).astype(np.float32)
    bids = rng.integers(0, batch, n).astype(np.int32)
    bids[:batch] = np.arange(batch)
    return pts, bids


@pytest.mark.parametrize("d", [2, 3, 4, 6])
@pytest.mark.parametrize("batch", [1, 5, 32])
def test_keys_match_float64_formula_on_dyadic_cells(oracle, d, batch):
    """compute_keys_tf_test.py:59-70 / compute_keys_ops_test.py:81-91: with a cell
    size that is a power of two, p/cell and min/cell are exact, so the fp32 op and
    the float64 formula must agree on every point."""
    rng = np.random.default_rng(7 + d + batch)
    pts, bids = _cloud(rng, batch, 4000, d, scale=4.0)
    cell = np.float32(0.25)
    g = oracle.Grid(pts, bids, batch, cell)
    amin = np.stack([pts[bids == b].min(axis=0) for b in range(batch)]).astype(np.float64)
    cells = np.floor((pts.astype(np.float64) - amin[bids]) / 0.25).astype(np.int64)
    cells = np.clip(cells, 0, g.num_cells.astype(np.int64) - 1)
    mult = np.concatenate([np.cumprod(g.num_cells[::-1].astype(np.int64))[::-1], [1]])
    expect = bids.astype(np.int64) * mult[0] + (cells * mult[1:]).sum(axis=1)
    assert np.array_equal(g.keys, expect)
    total = int(np.prod(g.num_cells.astype(np.int64)))
    assert g.keys.min() >= 0 and g.keys.max() < batch * total
    assert np.array_equal(g.keys // total, bids)


def test_keys_hand_computed(oracle):
    # one cloud, grid 4 x 2 x 3, cell 1: key = x*6 + y*3 + z ; second cloud adds 24
    pts = np.array([[0.5, 0.5, 0.5], [3.5, 1.5, 2.5], [2.25, 0.75, 1.5],
                    [9.0, 9.0, 9.0], [-4.0, 0.1, 0.1]], dtype=np.float32)
    bids = np.array([0, 0, 0, 1, 1], dtype=np.int32)
    smin = np.zeros((2, 3), dtype=np.float32)
    keys = oracle.compute_keys(pts, bids, smin, [4, 2, 3], [1.0, 1.0, 1.0])
    # clamping: (9,9,9) -> (3,1,2); (-4,.1,.1) -> (0,0,0)
    assert keys.tolist() == [0, 3 * 6 + 1 * 3 + 2, 2 * 6 + 0 + 1, 24 + 23, 24]


def test_sort_is_descending_and_stable(oracle):
    rng = np.random.default_rng(3)
    keys = rng.integers(0, 50, 5000).astype(np.int64)
    idx = oracle.sort_keys_descending(keys)
    assert np.array_equal(keys[idx], np.flip(np.sort(keys)))      # grid_test.py:69-71
    same = keys[idx][1:] == keys[idx][:-1]
    assert np.all(idx[1:][same] > idx[:-1][same])                 # ties: lower index first


@pytest.mark.parametrize("d", [2, 3, 4])
def test_grid_table_matches_numpy_loop(oracle, d):
    """build_grid_ds_tf_test.py:61-93: first / last+1 per (b, x, y) column."""
    rng = np.random.default_rng(11 + d)
    batch = 3
    pts, bids = _cloud(rng, batch, 3000, d)
    g = oracle.Grid(pts, bids, batch, 0.2)
    ds = g.get_ds()
    nc = g.num_cells.astype(np.int64)
    per_col = int(np.prod(nc[2:])) if d > 2 else 1
    expect = np.zeros((batch * nc[0] * nc[1], 2), dtype=np.int64)
    seen = {}
    for i, k in enumerate(g.sorted_keys):
        col = int(k) // per_col
        if col not in seen:
            seen[col] = True
            expect[col, 0] = i
        expect[col, 1] = i + 1
    assert np.array_equal(ds.reshape(-1, 2), expect)


@pytest.mark.parametrize("radius,expected", [(0.05, 1), (0.11, 7), (0.142, 19), (0.174, 27)])
def test_lattice_known_answer(oracle, radius, expected):
    """find_neighbors_tf_test.py:28-61: a 10^3 lattice of spacing 0.1 and 4^3 centres
    on lattice nodes have exactly 1 / 7 / 19 / 27 neighbours."""
    t = np.linspace(0, 1, 10, endpoint=False)
    pts = np.array(np.meshgrid(t, t, t)).T.reshape(-1, 3).astype(np.float32)
    t2 = np.linspace(1 / 5, 1, 4, endpoint=False)
    ctr = np.array(np.meshgrid(t2, t2, t2)).T.reshape(-1, 3).astype(np.float32)
    g = oracle.Grid(pts, np.zeros(len(pts), np.int32), 1, radius)
    nbh = oracle.Neighborhood(g, radius, ctr, np.zeros(len(ctr), np.int32))
    counts = np.diff(np.concatenate([[0], nbh.ranges]))
    assert np.all(counts == expected)


def _brute_force(samples, sb, pts, pb, radius):
    out = []
    for i in range(len(samples)):
        diff = (samples[i] - pts).astype(np.float32)
        sc = (diff * (np.float32(1.0) / np.float32(radius))).astype(np.float32)
        acc = np.zeros(len(pts), dtype=np.float32)
        for k in range(pts.shape[1]):
            acc = (acc + (sc[:, k] * sc[:, k]).astype(np.float32)).astype(np.float32)
        hit = np.nonzero((np.sqrt(acc) < 1.0) & (pb == sb[i]))[0]
        out.append(hit)
    return out


@pytest.mark.parametrize("d", [2, 3, 4, 5])
@pytest.mark.parametrize("self_nbh", [True, False])
def test_neighbours_match_brute_force(oracle, d, self_nbh):
    """neighbors_test.py:57-76 (find_neighbors_no_grid semantics): with cell >=
    radius the grid search returns every same-cloud point closer than the radius,
    listed per centre in ascending sorted index."""
    rng = np.random.default_rng(100 + d)
    batch = 3
    radius = {2: 0.08, 3: 0.2, 4: 0.35, 5: 0.5}[d]
    pts, bids = _cloud(rng, batch, 1500, d)
    g = oracle.Grid(pts, bids, batch, radius)
    if self_nbh:
        nbh = oracle.Neighborhood(g, radius)
    else:
        ctr, cb = _cloud(rng, batch, 300, d, scale=1.2)
        ctr -= 0.1
        nbh = oracle.Neighborhood(g, radius, ctr, cb)
    ref = _brute_force(nbh.samples, nbh.sample_batch_ids, g.sorted_points,
                       g.sorted_batch_ids, radius)
    starts = oracle.segment_starts(nbh.ranges)
    assert nbh.ranges[-1] == len(nbh.neighbors) == sum(len(r) for r in ref)
    for i, r in enumerate(ref):
        seg = nbh.neighbors[starts[i]:nbh.ranges[i]]
        assert np.array_equal(seg[:, 0], r)
        assert np.all(seg[:, 1] == i)
    if self_nbh:   # every point is its own neighbour
        assert np.all(np.diff(np.concatenate([[0], nbh.ranges])) >= 1)
    # original ids address the unsorted cloud (Neighborhood.py:246-250)
    assert np.array_equal(g.points[nbh.original_neigh_ids[:, 0]],
                          g.sorted_points[nbh.neighbors[:, 0]])


def test_neighbours_match_kdtree(oracle):
    """Library cross-check in float64 on inputs kept away from the radius sphere."""
    rng = np.random.default_rng(5)
    pts = rng.random((4000, 3)).astype(np.float32)
    radius = 0.07
    g = oracle.Grid(pts, np.zeros(len(pts), np.int32), 1, radius)
    nbh = oracle.Neighborhood(g, radius)
    sp = g.sorted_points.astype(np.float64)
    tree = cKDTree(sp)
    near = tree.query_ball_point(sp, radius * (1 + 1e-5))
    far = tree.query_ball_point(sp, radius * (1 - 1e-5))
    starts = oracle.segment_starts(nbh.ranges)
    for i in range(len(sp)):
        got = set(nbh.neighbors[starts[i]:nbh.ranges[i], 0].tolist())
        assert set(far[i]) <= got <= set(near[i])


def test_max_neighbours_keeps_first_in_canonical_order(oracle):
    rng = np.random.default_rng(9)
    pts = rng.random((2000, 3)).astype(np.float32)
    g = oracle.Grid(pts, np.zeros(len(pts), np.int32), 1, 0.15)
    full = oracle.Neighborhood(g, 0.15)
    lim = oracle.Neighborhood(g, 0.15, max_neighbors=5)
    fs, ls = oracle.segment_starts(full.ranges), oracle.segment_starts(lim.ranges)
    for i in range(len(pts)):
        a = full.neighbors[fs[i]:full.ranges[i]][:5]
        b = lim.neighbors[ls[i]:lim.ranges[i]]
        assert np.array_equal(a, b)


def test_empty_cells_and_single_point(oracle):
    pts = np.array([[0.0, 0.0, 0.0], [1.0, 1.0, 1.0]], dtype=np.float32)
    g = oracle.Grid(pts, np.array([0, 0], np.int32), 1, 0.1)
    assert g.num_cells.tolist() == [10, 10, 10]
    ds = g.get_ds()
    assert ds.sum() == (0 + 1) + (1 + 2)           # two occupied columns
    nbh = oracle.Neighborhood(g, 0.1)
    assert nbh.ranges.tolist() == [1, 2]
    g1 = oracle.Grid(pts[:1], np.array([0], np.int32), 1, 0.1)
    assert g1.num_cells.tolist() == [1, 1, 1]
    assert oracle.Neighborhood(g1, 0.1).neighbors.tolist() == [[0, 0]]


def test_radius_test_on_the_squared_length_decides_identically():
    """The HIP kernels compare the squared scaled distance with 1 where the reference
    compares its square root (count_neighbors_kernels.cu.cc:83-86).  In float32 the
    two agree for every value: checked on the 2^20 floats on either side of 1 (the
    correctly rounded root is monotonic, so no other value can differ) and on the
    special values."""
    below = np.float32(1.0) - np.arange(1 << 20, dtype=np.float32) * np.float32(2.0 ** -24)
    above = np.float32(1.0) + np.arange(1 << 20, dtype=np.float32) * np.float32(2.0 ** -23)
    special = np.array([0.0, np.finfo(np.float32).tiny, 1e-45, np.inf, np.nan], np.float32)
    with np.errstate(invalid="ignore"):
        for x in (below, above, special):
            assert x.dtype == np.float32
            assert np.array_equal(np.sqrt(x) < 1, x < 1)
