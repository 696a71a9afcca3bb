"""Parity of the HIP ops against the CPU oracle, through the C ABI of
libmccnn_hip.so (via the torch binding).  Integer outputs must be bit-exact;
float outputs are held to 1e-5 relative, stated per test."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

pytestmark = pytest.mark.gpu

REL = 1e-5


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from tensorflow_graphics_point_clouds_amd import tfg_custom_ops, _lib
    _lib.lib()   # raises if the HIP library is not built
    return tfg_custom_ops


def dev(a, dtype=None):
    t = torch.as_tensor(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda().contiguous()


def _cloud(rng, batch, n, d, scale=1.0):
    pts = (rng.random((n, d)) * scale).astype(np.float32)
    bids = rng.integers(0, batch, n).astype(np.int32)
    bids[:batch] = np.arange(batch)
    return pts, bids


def assert_rel(got, expect, mag=None, tol=REL):
    """|got - expect| <= tol * mag elementwise, where mag is the sum of the
    absolute values of the terms of each sum (default |expect|)."""
    got, expect = np.asarray(got, np.float64), np.asarray(expect, np.float64)
    mag = np.abs(expect) if mag is None else np.asarray(mag, np.float64)
    err = np.abs(got - expect)
    bad = err > tol * mag + 1e-30
    assert not bad.any(), "max err/mag = %g at %d entries" % (
        (err / np.maximum(mag, 1e-300)).max(), int(bad.sum()))


def assert_normwise(got, expect, tol=REL):
    """max |got - expect| <= tol * max |expect| (sums with cancellation)."""
    got, expect = np.asarray(got, np.float64), np.asarray(expect, np.float64)
    scale = np.abs(expect).max() if expect.size else 1.0
    assert np.abs(got - expect).max(initial=0.0) <= tol * scale


# ------------------------------------------------------------------ grid ----

@pytest.mark.parametrize("d", [2, 3, 4, 5, 6])
@pytest.mark.parametrize("batch,n,cell", [(1, 1000, 0.13), (5, 20000, 0.05), (32, 50000, 0.21)])
def test_keys_sort_table_bit_exact(ops, oracle, d, batch, n, cell):
    from tensorflow_graphics_point_clouds_amd import pc
    rng = np.random.default_rng(1 + d + batch)
    if d >= 5:
        cell = max(cell, 0.21)
    pts, bids = _cloud(rng, batch, n, d)
    g = oracle.Grid(pts, bids, batch, cell)
    keys = ops.compute_keys(dev(pts), dev(bids), dev(g.scaled_aabb_min), dev(g.num_cells),
                            dev(g.inv_cell_sizes))
    assert np.array_equal(keys.cpu().numpy(), g.keys)
    # the glue kernels reproduce the grid set-up, the sort and the gathers
    grid = pc.Grid(pc.PointCloud(dev(pts), dev(bids), batch), cell)
    assert np.array_equal(grid._aabb_min.cpu().numpy(), g.aabb_min)
    assert np.array_equal(grid._aabb_max.cpu().numpy(), g.aabb_max)
    assert np.array_equal(grid._num_cells.cpu().numpy(), g.num_cells)
    assert np.array_equal(grid._scaled_aabb_min.cpu().numpy(), g.scaled_aabb_min)
    assert np.array_equal(grid._inv_cell_sizes.cpu().numpy(), g.inv_cell_sizes)
    assert np.array_equal(grid._sorted_indices.cpu().numpy(), g.sorted_indices)
    assert np.array_equal(grid._sorted_keys.cpu().numpy(), g.sorted_keys)
    assert np.array_equal(grid._sorted_points.cpu().numpy(), g.sorted_points)
    assert np.array_equal(grid._sorted_batch_ids.cpu().numpy(), g.sorted_batch_ids)
    assert np.array_equal(grid.get_DS().cpu().numpy(), g.get_ds())


@pytest.mark.parametrize("n", [70001, 16384, 16385, 1025, 1, 4097])
@pytest.mark.parametrize("bits", [1, 7, 8, 9, 20, 33, 63])
def test_sort_key_widths_and_ties(ops, bits, n):
    """Stable descending order for every pass count, with many equal keys; sizes on both
    sides of the single-block path (up to 16384 keys) and at its round boundaries."""
    from tensorflow_graphics_point_clouds_amd import _lib
    from tensorflow_graphics_point_clouds_amd._lib import cint, i64, ptr, stream
    rng = np.random.default_rng(bits + n)
    hi = min(2 ** bits, 2 ** 62)
    keys = rng.integers(0, hi, n, dtype=np.int64)
    keys[::3] = keys[0]
    k = dev(keys)
    out_k = torch.empty_like(k)
    out_i = torch.empty(n, dtype=torch.int32, device="cuda")
    L = _lib.lib()
    ws = _lib.workspace(L.mccnn_sort_keys_workspace_bytes(i64(n)), k.device)
    _lib.check(L.mccnn_sort_keys_descending(stream(), i64(n), cint(bits), ptr(k), ptr(out_k),
                                            ptr(out_i), ptr(ws), _lib.csize(ws.numel())))
    expect = np.argsort(-keys, kind="stable")
    assert np.array_equal(out_i.cpu().numpy(), expect)
    assert np.array_equal(out_k.cpu().numpy(), keys[expect])


# ------------------------------------------------------------- neighbours ----

def _gpu_neighbors(ops, g, samples, sbids, radii, max_neighs=0):
    inv_r = (np.float32(1.0) / radii).astype(np.float32)
    return ops.find_neighbors(dev(samples), dev(sbids), dev(g.sorted_points), dev(g.sorted_keys),
                              dev(g.get_ds()), dev(g.num_cells), dev(g.scaled_aabb_min),
                              dev(g.inv_cell_sizes), dev(inv_r), max_neighs)


@pytest.mark.parametrize("d,radius", [(2, 0.03), (3, 0.08), (3, 0.3), (4, 0.3), (5, 0.5), (6, 0.6)])
@pytest.mark.parametrize("self_nbh", [True, False])
def test_neighbors_bit_exact(ops, oracle, d, radius, self_nbh):
    rng = np.random.default_rng(10 * d + int(self_nbh))
    batch, n = 4, 6000 if d < 5 else 2500
    pts, bids = _cloud(rng, batch, n, d)
    g = oracle.Grid(pts, bids, batch, radius)
    if self_nbh:
        nbh = oracle.Neighborhood(g, radius)
    else:
        ctr, cb = _cloud(rng, batch, 1500, d, scale=1.2)
        ctr -= 0.1                               # some centres outside the grid box
        nbh = oracle.Neighborhood(g, radius, ctr, cb)
    ranges, nbrs = _gpu_neighbors(ops, g, nbh.samples, nbh.sample_batch_ids, nbh.radii)
    assert np.array_equal(ranges.cpu().numpy(), nbh.ranges)
    assert np.array_equal(nbrs.cpu().numpy(), nbh.neighbors)


@pytest.mark.parametrize("radius,expected", [(0.05, 1), (0.11, 7), (0.142, 19), (0.174, 27)])
def test_neighbors_lattice_known_answer(ops, oracle, radius, expected):
    t = np.linspace(0, 1, 10, endpoint=False)
    pts = np.array(np.meshgrid(t, t, t)).T.reshape(-1, 3).astype(np.float32)
    t2 = np.linspace(1 / 5, 1, 4, endpoint=False)
    ctr = np.array(np.meshgrid(t2, t2, t2)).T.reshape(-1, 3).astype(np.float32)
    g = oracle.Grid(pts, np.zeros(len(pts), np.int32), 1, radius)
    ranges, _ = _gpu_neighbors(ops, g, ctr, np.zeros(len(ctr), np.int32),
                               np.full(3, radius, np.float32))
    counts = np.diff(np.concatenate([[0], ranges.cpu().numpy()]))
    assert np.all(counts == expected)


def test_neighbors_max_neighs_and_anisotropic_radii(ops, oracle):
    rng = np.random.default_rng(77)
    pts, bids = _cloud(rng, 2, 5000, 3)
    radii = np.array([0.1, 0.05, 0.08], np.float32)
    g = oracle.Grid(pts, bids, 2, radii)
    for limit in (0, 4):
        nbh = oracle.Neighborhood(g, radii, max_neighbors=limit)
        ranges, nbrs = _gpu_neighbors(ops, g, nbh.samples, nbh.sample_batch_ids, radii, limit)
        assert np.array_equal(ranges.cpu().numpy(), nbh.ranges)
        assert np.array_equal(nbrs.cpu().numpy(), nbh.neighbors)


@pytest.mark.parametrize("n", [50000, 66000])
def test_neighbors_refuses_pair_counts_beyond_int32(ops, oracle, n):
    """Every point within reach of every other: n^2 pairs, 2.5e9 (past 2^31) and
    4.36e9 (past 2^32, which a wrapped 32-bit total would report as 6.1e7).  The
    offsets of the op contract are int32, so the op has to refuse, not wrap."""
    rng = np.random.default_rng(n)
    pts = (rng.random((n, 3)) * 0.1).astype(np.float32)
    bids = np.zeros(n, np.int32)
    g = oracle.Grid(pts, bids, 1, 1.0)
    with pytest.raises(ValueError, match="pairs"):
        _gpu_neighbors(ops, g, pts, bids, np.full(3, 1.0, np.float32))
    # the library is usable afterwards
    ranges, _ = _gpu_neighbors(ops, g, pts[:100], bids[:100], np.full(3, 1.0, np.float32))
    assert np.array_equal(ranges.cpu().numpy(), n * np.arange(1, 101))


def test_neighbors_clustered_cloud(ops, oracle):
    """Heavy-tailed neighbour counts (blobs + noise), the shape of the scene-scale
    configuration at 1/50 of its size."""
    from tensorflow_graphics_point_clouds_amd import synthetic
    cfg = synthetic.config3(scale=0.02)
    g = oracle.Grid(cfg["points"], cfg["batch_ids"], cfg["batch_size"], cfg["radius"])
    nbh = oracle.Neighborhood(g, cfg["radius"])
    ranges, nbrs = _gpu_neighbors(ops, g, nbh.samples, nbh.sample_batch_ids, nbh.radii)
    assert np.array_equal(ranges.cpu().numpy(), nbh.ranges)
    assert np.array_equal(nbrs.cpu().numpy(), nbh.neighbors)


def test_find_neighbors_bounded_matches_two_phase_and_replays_from_a_graph(ops, oracle):
    """The search without a host round trip (count, scan and fill enqueued in one call, the pair
    count left on the device): the first min(count, capacity) rows and the end offsets equal the
    two-phase op bit for bit, an insufficient capacity raises the flag, and the call -- which
    allocates nothing when given its outputs -- replays from a captured HIP graph on changed
    centres with eager calls in between, every replay equal to the two-phase result."""
    rng = np.random.default_rng(123)
    pts, bids = _cloud(rng, 3, 5000, 3)
    g = oracle.Grid(pts, bids, 3, 0.1)
    grid_args = (dev(g.sorted_points), dev(g.sorted_keys), dev(g.get_ds()), dev(g.num_cells),
                 dev(g.scaled_aabb_min), dev(g.inv_cell_sizes),
                 dev(np.full(3, 1 / np.float32(0.1), np.float32)))

    def centres(seed):
        r = np.random.default_rng(seed)
        c, cb = _cloud(r, 3, 1200, 3, scale=1.1)
        return (c - 0.05).astype(np.float32), cb

    ctr, cb = centres(1)
    t_ctr, t_cb = dev(ctr), dev(cb)
    for limit in (0, 5):
        ranges, nbrs = ops.find_neighbors(t_ctr, t_cb, *grid_args, limit)
        m = nbrs.shape[0]
        nbh = oracle.Neighborhood(g, 0.1, ctr, cb, max_neighbors=limit)
        assert np.array_equal(nbrs.cpu().numpy(), nbh.neighbors)
        for capacity in (m + 1000, m, m - 7, 0):
            r2, n2, count, _ = ops.find_neighbors_bounded(t_ctr, t_cb, *grid_args, limit, capacity)
            assert count.tolist() == [m, int(m > capacity)]
            assert torch.equal(r2, ranges)
            keep = min(m, capacity)
            assert torch.equal(n2[:keep], nbrs[:keep])
    # graph: outputs allocated once, centres rewritten in place between replays
    capacity = m + 4000
    out = ops.find_neighbors_bounded(t_ctr, t_cb, *grid_args, 0, capacity)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.find_neighbors_bounded(t_ctr, t_cb, *grid_args, 0, capacity, out=out)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.find_neighbors_bounded(t_ctr, t_cb, *grid_args, 0, capacity, out=out)
    for seed in (2, 3, 4):
        ctr2, cb2 = centres(seed)
        t_ctr.copy_(dev(ctr2))
        t_cb.copy_(dev(cb2))
        graph.replay()
        torch.cuda.synchronize()
        ranges, nbrs = ops.find_neighbors(t_ctr, t_cb, *grid_args, 0)     # eager work in between
        count = out[2].tolist()
        assert count == [nbrs.shape[0], 0]
        assert torch.equal(out[0], ranges) and torch.equal(out[1][:count[0]], nbrs)


# -------------------------------------------------------------------- pdf ----

@pytest.mark.parametrize("d", [2, 3, 4])
@pytest.mark.parametrize("mode", [0, 1])
def test_pdf_and_point_grads(ops, oracle, d, mode):
    rng = np.random.default_rng(20 + d)
    pts, bids = _cloud(rng, 3, 4000, d)
    radius = {2: 0.05, 3: 0.15, 4: 0.3}[d]
    g = oracle.Grid(pts, bids, 3, radius)
    nbh = oracle.Neighborhood(g, radius)
    inv_bw = np.full(d, 1 / np.float32(0.2), np.float32)
    expect = oracle.compute_pdf(g.sorted_points, nbh.neighbors, nbh.ranges, inv_bw,
                                nbh.inv_radii, mode)
    sp = dev(g.sorted_points).requires_grad_(True)
    pdf = ops.compute_pdf_with_pt_grads(sp, dev(nbh.neighbors), dev(nbh.ranges), dev(inv_bw),
                                        dev(nbh.inv_radii), mode)
    assert_rel(pdf.detach().cpu().numpy(), expect)       # all terms positive: 1e-5 relative
    up = rng.standard_normal(len(pts)).astype(np.float32)
    pdf.backward(dev(up))
    gexp = oracle.compute_pdf_pt_grads(g.sorted_points, nbh.neighbors, nbh.ranges, inv_bw,
                                       nbh.inv_radii, up, mode)
    assert_normwise(sp.grad.cpu().numpy(), gexp)
    # the atomic-free form for symmetric pair tables (a self-neighbourhood is one)
    sym = ops.compute_pdf_pt_grads(sp.detach(), dev(nbh.neighbors), dev(nbh.ranges), dev(inv_bw),
                                   dev(nbh.inv_radii), dev(up), mode, symmetric=True)
    assert_normwise(sym.cpu().numpy(), gexp)


def test_find_neighbors_reports_symmetric_tables(ops, oracle):
    """find_neighbors marks the table it returns as symmetric exactly when the centres are the
    searched points themselves and no neighbourhood was cut at max_neighs; compute_pdf_pt_grads
    then takes the atomic-free form by itself and must still give the oracle's gradient."""
    rng = np.random.default_rng(91)
    pts, bids = _cloud(rng, 2, 3000, 3)
    g = oracle.Grid(pts, bids, 2, 0.15)
    sp, sb = dev(g.sorted_points), dev(g.sorted_batch_ids)
    args = (dev(g.sorted_keys), dev(g.get_ds()), dev(g.num_cells), dev(g.scaled_aabb_min),
            dev(g.inv_cell_sizes), dev(np.full(3, 1 / np.float32(0.15), np.float32)))
    largest = int(np.diff(np.concatenate([[0], oracle.Neighborhood(g, 0.15).ranges])).max())
    inv_bw = np.full(3, 1 / np.float32(0.2), np.float32)
    up = rng.standard_normal(len(pts)).astype(np.float32)
    for limit, same, expect in ((0, True, True), (largest, True, True), (largest - 1, True, False),
                                (6, True, False), (0, False, False)):
        centres = sp if same else sp.clone()
        ranges, nbrs = ops.find_neighbors(centres, sb, sp, *args, limit)
        assert ops.is_symmetric_table(nbrs) == expect, (limit, same)
        assert not ops.is_symmetric_table(nbrs.clone())
        if expect:          # an in-place write voids the record
            other = nbrs.clone()
            ranges2, edited = ops.find_neighbors(centres, sb, sp, *args, limit)
            assert ops.is_symmetric_table(edited)
            edited[0, 0] = edited[0, 0]
            assert not ops.is_symmetric_table(edited) and torch.equal(edited, other)
        nbh = oracle.Neighborhood(g, 0.15, max_neighbors=limit)
        assert np.array_equal(nbrs.cpu().numpy(), nbh.neighbors)
        for mode in (0, 1):
            gexp = oracle.compute_pdf_pt_grads(g.sorted_points, nbh.neighbors, nbh.ranges, inv_bw,
                                               nbh.inv_radii, up, mode)
            got = ops.compute_pdf_pt_grads(sp, nbrs, ranges, dev(inv_bw), dev(nbh.inv_radii),
                                           dev(up), mode)
            assert_normwise(got.cpu().numpy(), gexp)


@pytest.mark.parametrize("variant", ["truncated", "shuffled", "truncated+shuffled"])
def test_pdf_point_grads_on_asymmetric_and_unordered_tables(ops, oracle, variant):
    """compute_pdf_pt_grads looks the reverse of every pair up in the neighbour's list: lists
    cut by max_neighbors (reverse pairs missing: their terms are scattered) and lists in
    another order than find_neighbors writes (the binary search misses and the linear scan
    decides) must give the oracle's gradient (normwise 1e-5)."""
    rng = np.random.default_rng(77)
    pts, bids = _cloud(rng, 2, 3000, 3)
    g = oracle.Grid(pts, bids, 2, 0.15)
    nbh = oracle.Neighborhood(g, 0.15, max_neighbors=6 if "truncated" in variant else 0)
    pairs, ranges = nbh.neighbors.copy(), nbh.ranges
    if "shuffled" in variant:              # every centre's list in random order
        start = 0
        for end in ranges:
            pairs[start:end] = pairs[start:end][rng.permutation(end - start)]
            start = end
    if "truncated" in variant:             # the table really is asymmetric
        have = set(map(tuple, pairs.tolist()))
        assert any((c, j) not in have for j, c in have)
    inv_bw = np.full(3, 1 / np.float32(0.2), np.float32)
    up = rng.standard_normal(len(pts)).astype(np.float32)
    for mode in (0, 1):
        gexp = oracle.compute_pdf_pt_grads(g.sorted_points, pairs, ranges, inv_bw, nbh.inv_radii,
                                           up, mode)
        got = ops.compute_pdf_pt_grads(dev(g.sorted_points), dev(pairs), dev(ranges), dev(inv_bw),
                                       dev(nbh.inv_radii), dev(up), mode)
        assert_normwise(got.cpu().numpy(), gexp)


# ------------------------------------------------------------- basis_proj ----

@pytest.mark.parametrize("c,k", [(1, 8), (3, 16), (5, 32), (8, 8), (16, 16), (32, 32),
                                 (64, 16), (128, 32), (24, 64), (64, 64)])
def test_basis_proj_forward_and_grads(ops, oracle, c, k):
    rng = np.random.default_rng(c * 100 + k)
    n = 3000
    pts, bids = _cloud(rng, 2, n, 3)
    g = oracle.Grid(pts, bids, 2, 0.12)
    ctr, cb = _cloud(rng, 2, 700, 3)
    nbh = oracle.Neighborhood(g, 0.12, ctr, cb)
    ids = nbh.original_neigh_ids
    m = len(ids)
    basis = rng.random((m, k)).astype(np.float32)
    feat = rng.standard_normal((n, c)).astype(np.float32)
    expect, mag = oracle.basis_proj(basis, feat, ids, nbh.ranges, with_magnitude=True)
    tb, tf = dev(basis).requires_grad_(True), dev(feat).requires_grad_(True)
    out = ops.basis_proj(tb, tf, dev(ids), dev(nbh.ranges))
    assert out.shape == (700, c, k)
    assert_rel(out.detach().cpu().numpy(), expect, mag)
    up = rng.standard_normal((700, c, k)).astype(np.float32)
    out.backward(dev(up))
    db, df = oracle.basis_proj_grads(basis, feat, ids, nbh.ranges, up)
    assert_normwise(tb.grad.cpu().numpy(), db)
    assert_normwise(tf.grad.cpu().numpy(), df)


def test_basis_proj_empty_neighbourhoods(ops, oracle):
    """Centres without pairs give zero rows; a centre list with no pairs at all works."""
    feat = np.ones((10, 8), np.float32)
    ranges = np.array([0, 2, 2, 3], np.int32)
    ids = np.array([[1, 1], [4, 1], [9, 3]], np.int32)
    basis = np.arange(24, dtype=np.float32).reshape(3, 8)
    out = ops.basis_proj(dev(basis), dev(feat), dev(ids), dev(ranges)).cpu().numpy()
    expect = oracle.basis_proj(basis, feat, ids, ranges)
    assert np.array_equal(out, expect.astype(np.float32))
    none = ops.basis_proj(dev(np.zeros((0, 8), np.float32)), dev(feat),
                          dev(np.zeros((0, 2), np.int32)), dev(np.zeros(4, np.int32)))
    assert none.shape == (4, 8, 8) and float(none.abs().sum()) == 0.0


def test_op_validation_errors(ops):
    """The reference ops reject these with InvalidArgument."""
    f = lambda *s: torch.zeros(*s, device="cuda")
    i = lambda *s: torch.zeros(*s, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):      # 7 dimensions
        ops.compute_keys(f(4, 7), i(4), f(1, 7), i(7), f(7))
    with pytest.raises(ValueError):      # batch ids do not match
        ops.compute_keys(f(4, 3), i(5), f(1, 3), i(3), f(3))
    with pytest.raises(ValueError):      # K = 12
        ops.basis_proj(f(5, 12), f(4, 8), i(5, 2), i(3))
    with pytest.raises(ValueError):      # C = 12
        ops.basis_proj(f(5, 8), f(4, 12), i(5, 2), i(3))
    with pytest.raises(ValueError):      # basis rows != pairs
        ops.basis_proj(f(6, 8), f(4, 8), i(5, 2), i(3))
    with pytest.raises(ValueError):      # pairs need two columns
        ops.basis_proj(f(5, 8), f(4, 8), i(5, 3), i(3))
    with pytest.raises(ValueError):      # mode 2
        ops.compute_pdf_with_pt_grads(f(4, 3), i(4, 2), i(4), f(3), f(3), 2)
    with pytest.raises(ValueError):      # samples != points
        ops.compute_pdf_with_pt_grads(f(4, 3), i(4, 2), i(5), f(3), f(3), 0)
    with pytest.raises(ValueError):      # sampling mode
        ops.sampling(f(4, 3), i(4), torch.zeros(4, dtype=torch.int64, device="cuda"), i(3),
                     i(4, 2), i(4), 2)
    with pytest.raises(ValueError):      # non-positive batch size
        ops.build_grid_ds(torch.zeros(4, dtype=torch.int64, device="cuda"), i(3), [1, 1, 1], 0)
    with pytest.raises(ValueError):      # grid table of the wrong rank
        ops.find_neighbors(f(4, 3), i(4), f(4, 3), torch.zeros(4, dtype=torch.int64, device="cuda"),
                           i(1, 1, 2), i(3), f(1, 3), f(3), f(3), 0)


# --------------------------------------------------------------- sampling ----

@pytest.mark.parametrize("d,batch,cell", [(2, 1, 0.04), (3, 4, 0.1), (3, 1, 0.3), (4, 3, 0.3)])
@pytest.mark.parametrize("mode", [0, 1])
def test_sampling_bit_exact(ops, oracle, d, batch, cell, mode):
    rng = np.random.default_rng(33 + d + batch)
    pts, bids = _cloud(rng, batch, 5000, d)
    g = oracle.Grid(pts, bids, batch, cell)
    nbh = oracle.Neighborhood(g, cell)
    ep, eb, ei = oracle.sampling(g.sorted_points, g.sorted_batch_ids, g.sorted_keys, g.num_cells,
                                 nbh.neighbors, nbh.ranges, mode)
    gp, gb, gi = ops.sampling(dev(g.sorted_points), dev(g.sorted_batch_ids), dev(g.sorted_keys),
                              dev(g.num_cells), dev(nbh.neighbors), dev(nbh.ranges), mode)
    assert np.array_equal(gi.cpu().numpy(), ei)
    assert np.array_equal(gb.cpu().numpy(), eb)
    assert np.array_equal(gp.cpu().numpy(), ep)     # serial fp32 sums: same bits


@pytest.mark.parametrize("n_sqrt,scale", [(6, 1), (100, 5)])
def test_poisson_collinear_known_answer(ops, oracle, n_sqrt, scale):
    from tensorflow_graphics_point_clouds_amd import pc
    t = np.linspace(0, scale, num=n_sqrt)
    pts = np.array(np.meshgrid(t, t)).T.reshape(-1, 2).astype(np.float32)
    bids = np.repeat(np.arange(n_sqrt), n_sqrt).astype(np.int32)
    cell = (scale * np.array([2, 2], dtype=np.float32) / n_sqrt).astype(np.float32)
    cloud = pc.PointCloud(dev(pts), dev(bids), n_sqrt)
    nbh = pc.Neighborhood(pc.Grid(cloud, cell), cell)
    sampled, idx = pc.sample(nbh, "poisson")
    assert sampled._points.shape[0] == n_sqrt ** 2 // 2
    assert np.array_equal(pts[idx.cpu().numpy()], sampled._points.cpu().numpy())


def test_point_hierarchy_matches_oracle(ops, oracle):
    """Three cell-average levels (the ModelNet-shaped configuration): every level's
    points, batch ids and neighbourhoods equal the oracle's, bit for bit."""
    from tensorflow_graphics_point_clouds_amd import pc, synthetic
    cfg = synthetic.config2(batch=4, points_per_cloud=512)
    hier = pc.PointHierarchy(pc.PointCloud(dev(cfg["points"]), dev(cfg["batch_ids"]),
                                           cfg["batch_size"]), cfg["radii"], "cell average")
    pts, bids = cfg["points"], cfg["batch_ids"]
    for level, r in enumerate(cfg["radii"]):
        g = oracle.Grid(pts, bids, cfg["batch_size"], r)
        nbh = oracle.Neighborhood(g, r)
        gn = hier._neighborhoods[level]
        assert np.array_equal(gn._neighbors.cpu().numpy(), nbh.neighbors)
        pts, bids, _ = oracle.sampling(g.sorted_points, g.sorted_batch_ids, g.sorted_keys,
                                       g.num_cells, nbh.neighbors, nbh.ranges, 1)
        assert np.array_equal(hier._point_clouds[level + 1]._points.cpu().numpy(), pts)
        assert np.array_equal(hier._point_clouds[level + 1]._batch_ids.cpu().numpy(), bids)


def test_neighborhood_transpose_holds_the_same_pairs(ops, oracle):
    """transpose() (Neighborhood.py:318-329): the pair set of the transposed
    neighbourhood, mapped back to original ids, is the pair set of the original
    with the two columns swapped; a self-neighbourhood is its own transpose."""
    from tensorflow_graphics_point_clouds_amd import pc
    rng = np.random.default_rng(77)
    pts, bids = _cloud(rng, 3, 3000, 3)
    ctr, cb = _cloud(rng, 3, 700, 3)
    cloud, centres = pc.PointCloud(dev(pts), dev(bids), 3), pc.PointCloud(dev(ctr), dev(cb), 3)
    grid = pc.Grid(cloud, 0.12)
    nbh = pc.Neighborhood(grid, 0.12, centres)
    t = nbh.transpose()
    assert t is nbh.transpose() and t.get_grid()._point_cloud is centres
    a = nbh._original_neigh_ids.cpu().numpy()            # (point, centre)
    b = t._original_neigh_ids.cpu().numpy()              # (centre, point)
    assert len(a) == len(b)
    assert np.array_equal(np.unique(a, axis=0), np.unique(b[:, ::-1], axis=0))
    og = oracle.Grid(ctr, cb, 3, 0.12)
    on = oracle.Neighborhood(og, 0.12, pts, bids)
    assert np.array_equal(t._neighbors.cpu().numpy(), on.neighbors)
    own = pc.Neighborhood(grid, 0.12)
    assert own.transpose() is own


@pytest.mark.parametrize("max_neighbors", [0, 5])
def test_same_cloud_neighborhood_equals_direct_search(ops, oracle, max_neighbors):
    """Centres = the grid's own cloud (one sorted search + regrouped segments):
    ranges, pairs and original ids equal the oracle's direct search bit for bit,
    and the grid-ordered view describes the same pair set."""
    from tensorflow_graphics_point_clouds_amd import pc
    rng = np.random.default_rng(31)
    pts, bids = _cloud(rng, 3, 5000, 3)
    cloud = pc.PointCloud(dev(pts), dev(bids), 3)
    grid = pc.Grid(cloud, 0.09)
    nbh = pc.Neighborhood(grid, 0.09, cloud, max_neighbors)
    g = oracle.Grid(pts, bids, 3, 0.09)
    on = oracle.Neighborhood(g, 0.09, pts, bids, max_neighbors)
    assert np.array_equal(nbh._samples_neigh_ranges.cpu().numpy(), on.ranges)
    assert np.array_equal(nbh._neighbors.cpu().numpy(), on.neighbors)
    assert np.array_equal(nbh._original_neigh_ids.cpu().numpy(), on.original_neigh_ids)
    view = nbh.sorted_view()
    order = view.centre_order.cpu().numpy()
    table = view.table.cpu().numpy()
    back = np.stack((table[:, 0], order[table[:, 1]]), axis=1)     # (sorted point, original centre)
    assert np.array_equal(np.unique(back, axis=0), np.unique(on.neighbors, axis=0))
    tt = view.table_t.cpu().numpy()                                 # (centre slot, point position)
    assert np.array_equal(np.unique(tt[:, ::-1], axis=0), np.unique(table, axis=0))
    rt = view.ranges_t.cpu().numpy()
    assert np.all(np.diff(rt) >= 0) and rt[-1] == len(tt)
    seg = np.repeat(np.arange(len(rt)), np.diff(np.concatenate(([0], rt))))
    assert np.array_equal(seg, tt[:, 1])


def test_basis_proj_visiting_order_does_not_change_results(ops, oracle):
    """The *_ordered entry points only reschedule: forward and basis gradients
    are bit-identical for any permutation of the centres, feature gradients (float
    atomics) agree normwise."""
    rng = np.random.default_rng(123)
    n, c, k = 4000, 64, 16
    pts, bids = _cloud(rng, 2, n, 3)
    g = oracle.Grid(pts, bids, 2, 0.1)
    nbh = oracle.Neighborhood(g, 0.1, pts, bids)
    ids = nbh.original_neigh_ids
    basis = rng.random((len(ids), k)).astype(np.float32)
    feat = rng.standard_normal((n, c)).astype(np.float32)
    up = rng.standard_normal((n, c, k)).astype(np.float32)
    order = dev(rng.permutation(n).astype(np.int32))
    args = (dev(basis), dev(feat), dev(ids), dev(nbh.ranges))
    a = ops._basis_proj_raw(*args)
    b = ops._basis_proj_raw(*args, order)
    assert torch.equal(a, b)
    da, fa = ops.basis_proj_grads(*args, dev(up))
    db, fb = ops.basis_proj_grads(*args, dev(up), order)
    assert torch.equal(da, db)
    assert_normwise(fb.cpu().numpy(), fa.cpu().numpy())


def test_full_size_invariants(ops):
    """Scene-scale batch at its real size (8 clouds, ~760k points): properties
    that need no oracle.  Sortedness and permutation of the grid sort, the column
    table against the keys, ranges non-decreasing with last == M, pairs grouped by
    centre and ascending inside a centre, every point its own neighbour, the
    neighbourhood symmetric, and linearity / adjointness of basis_proj."""
    from tensorflow_graphics_point_clouds_amd import pc, synthetic
    cfg = synthetic.config3()
    cloud = pc.PointCloud(dev(cfg["points"]), dev(cfg["batch_ids"]), cfg["batch_size"])
    grid = pc.Grid(cloud, cfg["radius"])
    n = cloud._points.shape[0]
    keys = grid._sorted_keys
    assert bool((keys[1:] <= keys[:-1]).all())
    assert torch.equal(torch.sort(grid._sorted_indices.long()).values,
                       torch.arange(n, device="cuda"))
    assert torch.equal(grid._cur_keys[grid._sorted_indices.long()], keys)
    ties = keys[1:] == keys[:-1]
    assert bool((grid._sorted_indices[1:][ties] > grid._sorted_indices[:-1][ties]).all())
    nc = grid._num_cells_host
    ds = grid.get_DS().reshape(-1, 2).long()
    col = torch.div(keys, nc[2], rounding_mode="floor")
    occupied = torch.unique(col)
    counts = torch.bincount(col, minlength=ds.shape[0])
    assert torch.equal((ds[:, 1] - ds[:, 0]), counts)
    assert bool((col[ds[occupied, 0]] == occupied).all())

    nbh = pc.Neighborhood(grid, cfg["radius"])          # centres = sorted points
    ranges, nbrs = nbh._samples_neigh_ranges.long(), nbh._neighbors.long()
    m = nbrs.shape[0]
    assert int(ranges[-1]) == m and bool((ranges[1:] >= ranges[:-1]).all())
    starts = torch.cat([ranges.new_zeros(1), ranges[:-1]])
    centre_of_pair = torch.repeat_interleave(torch.arange(n, device="cuda"), ranges - starts)
    assert torch.equal(nbrs[:, 1], centre_of_pair)
    same = nbrs[1:, 1] == nbrs[:-1, 1]
    assert bool((nbrs[1:, 0][same] > nbrs[:-1, 0][same]).all())
    assert int((nbrs[:, 0] == nbrs[:, 1]).sum()) == n                     # self pairs
    assert bool((grid._sorted_batch_ids[nbrs[:, 0]] == grid._sorted_batch_ids[nbrs[:, 1]]).all())
    fwd = nbrs[:, 0] * n + nbrs[:, 1]
    bwd = nbrs[:, 1] * n + nbrs[:, 0]
    assert torch.equal(torch.sort(fwd).values, torch.sort(bwd).values)    # symmetry
    d = (grid._sorted_points[nbrs[:, 0]] - grid._sorted_points[nbrs[:, 1]]).norm(dim=1)
    assert float(d.max()) < cfg["radius"] * (1 + 1e-6)

    # basis_proj: linear in the features, and <up, proj(B, F)> == <dB, B> == <dF, F>
    gen = torch.Generator(device="cuda").manual_seed(0)
    ids = nbh._original_neigh_ids
    basis = torch.rand((m, 16), device="cuda", generator=gen)
    f1 = torch.randn((n, 64), device="cuda", generator=gen)
    f2 = torch.randn((n, 64), device="cuda", generator=gen)
    r32 = nbh._samples_neigh_ranges
    p1 = ops._basis_proj_raw(basis, f1, ids, r32)
    p2 = ops._basis_proj_raw(basis, f2, ids, r32)
    p12 = ops._basis_proj_raw(basis, f1 + 2 * f2, ids, r32)
    assert float((p12 - (p1 + 2 * p2)).abs().max()) <= 1e-5 * float(p12.abs().max())
    up = torch.randn(p1.shape, device="cuda", generator=gen)
    db, df = ops.basis_proj_grads(basis, f1, ids, r32, up)
    lhs = float((up.double() * p1.double()).sum())
    assert abs(float((db.double() * basis.double()).sum()) - lhs) <= 1e-5 * abs(lhs) + 1e-3
    assert abs(float((df.double() * f1.double()).sum()) - lhs) <= 1e-5 * abs(lhs) + 1e-3


@pytest.mark.parametrize("c,k", [(16, 16), (64, 16), (128, 16), (32, 32), (128, 32)])
def test_gathered_feature_gradient(ops, oracle, c, k):
    """Transposed pair lists equal a stable argsort by neighbour id, and the
    atomic-free feature gradient matches the oracle and is bit-reproducible."""
    rng = np.random.default_rng(c + k)
    n = 3000
    pts, bids = _cloud(rng, 2, n, 3)
    g = oracle.Grid(pts, bids, 2, 0.12)
    ctr, cb = _cloud(rng, 2, 900, 3)
    nbh = oracle.Neighborhood(g, 0.12, ctr, cb)
    ids = nbh.original_neigh_ids
    t_ranges, t_order = ops.transpose_neighbors(dev(ids), n)
    expect_order = np.argsort(ids[:, 0], kind="stable")
    assert np.array_equal(t_order.cpu().numpy(), expect_order)
    assert np.array_equal(t_ranges.cpu().numpy(), np.cumsum(np.bincount(ids[:, 0], minlength=n)))
    # the rows of the transposed table: (centre, point) of the pairs in that order
    from tensorflow_graphics_point_clouds_amd import _lib
    from tensorflow_graphics_point_clouds_amd._lib import i64, ptr, stream
    swapped = torch.empty((len(ids), 2), dtype=torch.int32, device="cuda")
    _lib.call("swapped_pairs", stream(), i64(len(ids)), ptr(dev(ids)), ptr(t_order), ptr(swapped))
    assert np.array_equal(swapped.cpu().numpy(), ids[expect_order][:, ::-1])
    basis = rng.random((len(ids), k)).astype(np.float32)
    feat = rng.standard_normal((n, c)).astype(np.float32)
    up = rng.standard_normal((900, c, k)).astype(np.float32)
    args = (dev(basis), dev(feat), dev(ids), dev(nbh.ranges), dev(up))
    db1, df1 = ops.basis_proj_grads(*args, transposed=(t_ranges, t_order))
    db2, df2 = ops.basis_proj_grads(*args, transposed=(t_ranges, t_order))
    assert torch.equal(df1, df2) and torch.equal(db1, db2)
    edb, edf = oracle.basis_proj_grads(basis, feat, ids, nbh.ranges, up)
    assert_normwise(db1.cpu().numpy(), edb)
    assert_normwise(df1.cpu().numpy(), edf)
    # points that are nobody's neighbour get an exact zero row
    unused = np.setdiff1d(np.arange(n), ids[:, 0])
    assert len(unused) > 0 and float(df1[dev(unused).long()].abs().sum()) == 0.0


def test_sampling_wrappers_hierarchy_accessors_and_normalised_pdf(ops, oracle):
    """poisson_disk_sampling / cell_average_sampling (sampling.py:31-120) against the
    oracle's sampler, the per-level accessors of the hierarchy, and densities
    divided by the size of their neighbourhood (Neighborhood.py:288-293)."""
    from tensorflow_graphics_point_clouds_amd import pc
    rng = np.random.default_rng(8)
    pts, bids = _cloud(rng, 3, 4000, 3)
    cloud = pc.PointCloud(dev(pts), dev(bids), 3)
    r = np.float32(0.07)
    g = oracle.Grid(pts, bids, 3, r)
    nbh = oracle.Neighborhood(g, r)
    for mode, fn in ((0, lambda: pc.poisson_disk_sampling(cloud, float(r), return_ids=True)),
                     (1, lambda: (pc.cell_average_sampling(cloud, float(r)), None))):
        spts, sbids, sidx = oracle.sampling(g.sorted_points, g.sorted_batch_ids, g.sorted_keys,
                                            g.num_cells, nbh.neighbors, nbh.ranges, mode)
        got, ids = fn()
        assert np.array_equal(got._points.cpu().numpy(), spts)
        assert np.array_equal(got._batch_ids.cpu().numpy(), sbids)
        if mode == 0:
            assert np.array_equal(ids.cpu().numpy(), g.sorted_indices[sidx])
            assert np.array_equal(pts[ids.cpu().numpy()], spts)
    with pytest.raises(ValueError):
        pc.poisson_disk_sampling(cloud)
    with pytest.raises(ValueError):
        pc.cell_average_sampling(cloud)

    hier = pc.PointHierarchy(cloud, [0.1, 0.2], "cell average")
    sizes = hier.get_sizes()
    assert [int(s.sum()) for s in sizes] == [c._points.shape[0] for c in hier._point_clouds]
    padded = hier.get_points()
    assert [tuple(p.shape[:1]) for p in padded] == [(3,)] * 3
    assert [p.shape[1] for p in padded] == [int(s.max()) for s in sizes]
    assert hier.get_points(1)[2].shape[0] == int(sizes[2][1])
    hier.set_batch_shape([3, 1])
    assert all(tuple(s.shape) == (3, 1) for s in hier.get_sizes())

    ctr, cb = _cloud(rng, 3, 500, 3)
    gn = pc.Neighborhood(pc.Grid(cloud, float(r) * 2), float(r) * 2, pc.PointCloud(dev(ctr), dev(cb), 3))
    plain = gn.get_pdf(bandwidth=0.2).clone()
    gn.compute_pdf(bandwidth=0.2, normalize=True)
    ends = gn._samples_neigh_ranges.long()
    counts = ends - torch.cat([ends.new_zeros(1), ends[:-1]])
    expect = plain / counts[gn._neighbors[:, 1].long()].float()
    assert torch.allclose(gn.get_pdf(), expect, rtol=1e-6)


def test_object_level_adapters_match_the_callers(ops):
    """custom_ops (the wrapper layer of custom_ops_wrapper.py:20-198) gives what the
    Grid / Neighborhood callers compute through the positional ops."""
    from tensorflow_graphics_point_clouds_amd import custom_ops, pc
    rng = np.random.default_rng(12)
    pts, bids = _cloud(rng, 3, 5000, 3)
    ctr, cb = _cloud(rng, 3, 700, 3)
    cloud, centres = pc.PointCloud(dev(pts), dev(bids), 3), pc.PointCloud(dev(ctr), dev(cb), 3)
    radii = dev(np.full(3, 0.08, np.float32))
    grid = pc.Grid(cloud, radii)
    assert torch.equal(custom_ops.compute_keys(cloud, grid._num_cells, grid._cell_sizes),
                       grid._cur_keys)
    assert torch.equal(custom_ops.build_grid_ds(grid._sorted_keys, grid._num_cells, 3),
                       grid.get_DS())
    nbh = pc.Neighborhood(grid, radii, centres)
    ranges, nbrs = custom_ops.find_neighbors(grid, centres, radii)
    assert torch.equal(ranges, nbh._samples_neigh_ranges) and torch.equal(nbrs, nbh._neighbors)
    own = pc.Neighborhood(grid, radii)
    for mode, name in ((0, "poisson"), (1, "average")):
        spts, sbids, _ = custom_ops.sampling(own, mode)
        expect = pc.sample(own, name)[0]
        assert torch.equal(spts, expect._points) and torch.equal(sbids, expect._batch_ids)
    bw = dev(np.full(3, 0.2, np.float32))
    assert torch.equal(custom_ops.compute_pdf(own, bw, 0), own.point_pdf(bandwidth=0.2))
    basis = torch.rand((nbrs.shape[0], 8), device="cuda")
    feat = torch.randn((5000, 8), device="cuda")
    assert torch.equal(custom_ops.basis_proj(basis, feat, nbh),
                       ops.basis_proj(basis, feat, nbh._original_neigh_ids, ranges))


def test_pipeline_on_the_reference_sample_cloud(ops, oracle):
    """Real data instead of uniform noise: the first 256 points of the reference's
    sample scan (positions; the normals serve as features), radius 0.05: keys, sort,
    grid table and pairs bit-exact, densities and the projection within 1e-5."""
    import os
    from tensorflow_graphics_point_clouds_amd import pc
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                        "shrec15_cloud0_first256.txt")
    data = np.loadtxt(path, delimiter=",", dtype=np.float32)
    pts, normals = np.ascontiguousarray(data[:, :3]), np.ascontiguousarray(data[:, 3:6])
    bids = np.zeros(len(pts), np.int32)
    radius = np.float32(0.05)
    g = oracle.Grid(pts, bids, 1, radius)
    nbh = oracle.Neighborhood(g, radius, pts, bids)
    cloud = pc.PointCloud(dev(pts), dev(bids), 1)
    grid = pc.Grid(cloud, float(radius))
    got = pc.Neighborhood(grid, float(radius), cloud)
    assert np.array_equal(grid._sorted_keys.cpu().numpy(), g.sorted_keys)
    assert np.array_equal(grid._sorted_indices.cpu().numpy(), g.sorted_indices)
    assert np.array_equal(grid.get_DS().cpu().numpy(), g.get_ds())
    assert np.array_equal(got._samples_neigh_ranges.cpu().numpy(), nbh.ranges)
    assert np.array_equal(got._neighbors.cpu().numpy(), nbh.neighbors)
    assert np.array_equal(got._original_neigh_ids.cpu().numpy(), nbh.original_neigh_ids)
    assert len(nbh.neighbors) > 2 * len(pts)          # the radius reaches beyond the point itself
    pdf = nbh.pdf_per_pair(0.2)
    np.testing.assert_allclose(got.get_pdf(bandwidth=0.2).cpu().numpy(), pdf, rtol=1e-5)
    rng = np.random.default_rng(0)
    basis = rng.random((len(nbh.neighbors), 16)).astype(np.float32)
    feat = np.concatenate([normals, np.ones((len(pts), 1), np.float32)], axis=1)   # C = 4
    out = ops.basis_proj(dev(basis), dev(feat), got._original_neigh_ids, got._samples_neigh_ranges)
    expect, mag = oracle.basis_proj(basis, feat, nbh.original_neigh_ids, nbh.ranges, with_magnitude=True)
    assert_rel(out.cpu().numpy(), expect, mag)


def test_two_host_threads_on_their_own_streams(ops, oracle):
    """The library keeps no state between calls (error text and the pinned size
    word are per thread, workspaces per call): two host threads, each on its own
    stream, build grids and neighbourhoods and project at the same time and get
    what the oracle gets."""
    import threading
    from tensorflow_graphics_point_clouds_amd import pc
    jobs = []
    for seed in (1, 2):
        rng = np.random.default_rng(seed)
        pts, bids = _cloud(rng, 3, 20000 + 3000 * seed, 3)
        radius = np.float32(0.04 + 0.01 * seed)
        g = oracle.Grid(pts, bids, 3, radius)
        nbh = oracle.Neighborhood(g, radius, pts, bids)
        basis = rng.random((len(nbh.neighbors), 16)).astype(np.float32)
        feat = rng.standard_normal((len(pts), 16)).astype(np.float32)
        expect, mag = oracle.basis_proj(basis, feat, nbh.original_neigh_ids, nbh.ranges,
                                        with_magnitude=True)
        jobs.append(dict(pts=dev(pts), bids=dev(bids), radius=float(radius), nbh=nbh,
                         basis=dev(basis), feat=dev(feat), expect=expect, mag=mag, out=None,
                         error=None))
    torch.cuda.synchronize()

    def work(job):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(3):
                    cloud = pc.PointCloud(job["pts"], job["bids"], 3)
                    got = pc.Neighborhood(pc.Grid(cloud, job["radius"]), job["radius"], cloud)
                    out = ops.basis_proj(job["basis"], job["feat"], got._original_neigh_ids,
                                         got._samples_neigh_ranges)
                stream.synchronize()
            job["out"] = (got._neighbors.cpu().numpy(), out.cpu().numpy())
        except Exception as exc:                      # surfaced by the main thread
            job["error"] = exc

    threads = [threading.Thread(target=work, args=(job,)) for job in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for job in jobs:
        assert job["error"] is None, job["error"]
        pairs, out = job["out"]
        assert np.array_equal(pairs, job["nbh"].neighbors)
        assert_rel(out, job["expect"], job["mag"])


def test_ops_without_a_host_round_trip_replay_from_a_captured_graph(ops):
    """The entry points that size no output enqueue kernels only (zero-fills are
    kernels too), so a caller may capture them: basis_proj with both gradients and
    compute_pdf recorded in a HIP graph, replayed three times on changed inputs with
    eager work and synchronisations in between, every replay equal to the eager
    result on the same inputs (the atomic feature gradient within 1e-5)."""
    gen = torch.Generator(device="cuda").manual_seed(9)
    n, n_out, c, k, per = 3000, 1200, 32, 16, 9
    ranges = (torch.arange(1, n_out + 1, device="cuda") * per).int()
    m = n_out * per
    nbrs = torch.stack((torch.randint(0, n, (m,), device="cuda", generator=gen),
                        torch.arange(n_out, device="cuda").repeat_interleave(per)), 1).int()
    basis = torch.rand((m, k), device="cuda", generator=gen)
    feat = torch.randn((n, c), device="cuda", generator=gen)
    up = torch.randn((n_out, c, k), device="cuda", generator=gen)
    pts = torch.rand((n_out, 3), device="cuda", generator=gen)
    self_pairs = torch.stack((torch.randint(0, n_out, (m,), device="cuda", generator=gen),
                              torch.arange(n_out, device="cuda").repeat_interleave(per)), 1).int()
    inv = torch.full((3,), 5.0, device="cuda")

    def run():
        out = ops._basis_proj_raw(basis, feat, nbrs, ranges, None)
        dbasis, dfeat = ops.basis_proj_grads(basis, feat, nbrs, ranges, up, None)
        pdf = ops.compute_pdf_with_pt_grads(pts, self_pairs, ranges, inv, inv, 0)
        return out, dbasis, dfeat, pdf

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run()
    for rep in range(3):
        feat.copy_(torch.randn((n, c), device="cuda", generator=gen))
        basis.copy_(torch.rand((m, k), device="cuda", generator=gen))
        pts.copy_(torch.rand((n_out, 3), device="cuda", generator=gen))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        eager = run()
        torch.cuda.synchronize()
        assert torch.equal(got[0], eager[0]) and torch.equal(got[1], eager[1]), rep
        assert torch.equal(got[3], eager[3]), rep
        scale = float(eager[2].abs().max())
        assert float((got[2] - eager[2]).abs().max()) <= 1e-5 * scale, rep


def test_row_and_density_gathers(ops):
    """The glue gathers the layers use: feature rows by int32 index (any row length
    that is a multiple of 4) and per-pair densities from either column of a pair
    table."""
    from tensorflow_graphics_point_clouds_amd import _lib
    from tensorflow_graphics_point_clouds_amd._lib import cint, i64, ptr, stream
    gen = torch.Generator(device="cuda").manual_seed(0)
    for n, c, m in ((1000, 4, 3000), (5000, 64, 777), (300, 132, 300), (7, 8, 0)):
        x = torch.randn((n, c), device="cuda", generator=gen)
        rows = torch.randint(0, n, (m,), device="cuda", generator=gen, dtype=torch.int32)
        out = torch.empty((m, c), device="cuda")
        _lib.call("gather_rows", stream(), i64(m), cint(c), ptr(x), ptr(rows), ptr(out))
        assert torch.equal(out, x[rows.long()])
    with pytest.raises(ValueError):
        _lib.call("gather_rows", stream(), i64(4), cint(6), ptr(x), ptr(rows), ptr(out))
    pairs = torch.randint(0, 500, (4000, 2), device="cuda", generator=gen, dtype=torch.int32)
    pdf = torch.rand(500, device="cuda", generator=gen)
    for column in (0, 1):
        out = torch.empty(4000, device="cuda")
        _lib.call("gather_pdf_column", stream(), i64(4000), ptr(pairs), cint(column), ptr(pdf),
                  ptr(out))
        assert torch.equal(out, pdf[pairs[:, column].long()])
