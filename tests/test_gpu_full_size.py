"""The integer pipeline at the benchmark's own sizes, table against table.

keys, sort permutation, sorted keys, column table, ranges, pair table (sorted and original
point ids) and the Poisson-disk index set of the GPU path are compared with the CPU
oracle's with `array_equal` / `torch.equal` on

* the scene-scale batch (8 clouds, 763 063 points, radius 0.15, 28.2 M pairs);
* the dense batch (4 x 200 000 uniform points) at radii 0.02, 0.04 and 0.06 (6.0 M, 41.8 M
  and 136 M pairs);
* clouds far from the origin (coordinates around 1000 with radius 0.01 to 0.05, where one
  float32 step is 6e-5), and centres that lie outside the grid's bounding box.

These are the cases that exercise the cell-row pruning of the neighbour search (rows the
sphere cannot reach are dropped from a slack estimate in float32) at the coordinate
magnitudes and cell counts of the benchmark.  The large tables are compared on the
device (the oracle's table is uploaded)."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.as_tensor(np.ascontiguousarray(a)).cuda().contiguous()


def _same(got, expect, what):
    """torch.equal of a device tensor with a host array, with a useful message."""
    want = dev(expect)
    assert tuple(got.shape) == tuple(want.shape), "%s: shape %s vs %s" % (
        what, tuple(got.shape), tuple(want.shape))
    if not torch.equal(got, want):
        bad = (got != want).reshape(got.shape[0], -1).any(dim=1).nonzero()
        raise AssertionError("%s differs in %d rows, first at row %d" % (
            what, bad.numel(), int(bad[0])))


def _check_grid_and_self_neighbourhood(oracle, points, batch_ids, batch_size, radius,
                                       poisson=False):
    from tensorflow_graphics_point_clouds_amd import pc
    r = np.float32(radius)
    g = oracle.Grid(points, batch_ids, batch_size, r)
    nbh = oracle.Neighborhood(g, r)

    cloud = pc.PointCloud(dev(points), dev(batch_ids), batch_size)
    grid = pc.Grid(cloud, radius)
    assert grid._num_cells_host == [int(v) for v in g.num_cells]
    _same(grid._num_cells, g.num_cells, "grid shape")
    _same(grid._cur_keys, g.keys, "keys")
    _same(grid._sorted_indices, g.sorted_indices, "sort permutation")
    _same(grid._sorted_keys, g.sorted_keys, "sorted keys")
    _same(grid._sorted_points, g.sorted_points, "sorted points")
    _same(grid._sorted_batch_ids, g.sorted_batch_ids, "sorted batch ids")
    _same(grid.get_DS(), g.get_ds(), "column table")

    got = pc.Neighborhood(grid, radius)
    assert got._neighbors.shape[0] == len(nbh.neighbors)
    _same(got._samples_neigh_ranges, nbh.ranges, "ranges")
    _same(got._neighbors, nbh.neighbors, "pair table")
    # original ids: the oracle's sorted ids through the oracle's permutation, on the device
    want = dev(nbh.neighbors)
    want[:, 0] = dev(g.sorted_indices)[want[:, 0].long()]
    assert torch.equal(got._original_neigh_ids, want), "pair table with original ids"
    del want
    # the search without a host round trip: same end offsets and rows, count on the device
    from tensorflow_graphics_point_clouds_amd import tfg_custom_ops as ops
    m = len(nbh.neighbors)
    for capacity in (m + 3, m - 1):
        ranges, table, count, _ = ops.find_neighbors_bounded(
            grid._sorted_points, grid._sorted_batch_ids, grid._sorted_points, grid._sorted_keys,
            grid.get_DS(), grid._num_cells, grid._scaled_aabb_min, grid._inv_cell_sizes,
            got._inv_radii, 0, capacity)
        assert count.tolist() == [m, int(m > capacity)]
        assert torch.equal(ranges, got._samples_neigh_ranges), "bounded search: ranges"
        keep = min(m, capacity)
        assert torch.equal(table[:keep], got._neighbors[:keep]), "bounded search: pair table"
        del ranges, table
    if poisson:
        pts, bids, sel = oracle.sampling(g.sorted_points, g.sorted_batch_ids, g.sorted_keys,
                                         g.num_cells, nbh.neighbors, nbh.ranges, 0)
        sampled, ids = pc.sample(got, "poisson")
        _same(sampled._points, pts, "Poisson-disk points")
        _same(sampled._batch_ids, bids, "Poisson-disk batch ids")
        _same(ids, g.sorted_indices[sel], "Poisson-disk original indices")
    return len(nbh.neighbors)


def test_scene_scale_batch_integer_pipeline_equals_oracle(oracle):
    """Configuration 3 at its real size: 763 063 clustered points in a 10 x 10 x 3 box,
    radius 0.15 (93 x 93 x 28 cells: the blobs reach beyond the box), 28.2 M pairs."""
    from tensorflow_graphics_point_clouds_amd import synthetic
    cfg = synthetic.config3()
    m = _check_grid_and_self_neighbourhood(oracle, cfg["points"], cfg["batch_ids"],
                                           cfg["batch_size"], cfg["radius"])
    assert m == 28225813


@pytest.mark.parametrize("radius,pairs", [(0.02, 6036492), (0.04, 41786012), (0.06, 135977048)])
def test_dense_batch_integer_pipeline_equals_oracle(oracle, radius, pairs):
    """Configuration 4 at its real size (4 x 200 000 uniform points; 50^3, 25^3 and 17^3
    cells per cloud) with the Poisson-disk sample at the same radius."""
    from tensorflow_graphics_point_clouds_amd import synthetic
    cfg = synthetic.config4()
    m = _check_grid_and_self_neighbourhood(oracle, cfg["points"], cfg["batch_ids"],
                                           cfg["batch_size"], radius, poisson=True)
    assert m == pairs


@pytest.mark.parametrize("origin,extent,radius", [(1000.0, 1.0, 0.01), (-2500.0, 2.0, 0.05),
                                                  (300.0, 0.5, 0.013)])
def test_clouds_far_from_the_origin_equal_oracle(oracle, origin, extent, radius):
    """Bounding boxes far from the origin: the scaled coordinates the search prunes on are
    of the order 10^4..10^5 cells, so the slack of the row test is thousands of times
    larger in absolute terms than inside the unit cube."""
    rng = np.random.default_rng(int(abs(origin)))
    n, batch = 120000, 3
    pts = (origin + extent * rng.random((n, 3))).astype(np.float32)
    bids = np.sort(rng.integers(0, batch, n)).astype(np.int32)
    _check_grid_and_self_neighbourhood(oracle, pts, bids, batch, radius, poisson=True)


@pytest.mark.parametrize("d", [2, 3, 4])
def test_centres_outside_the_grid_equal_oracle(oracle, d):
    """Foreign centres scattered over a box twice as large as the cloud's: those outside
    take the clamped border cell (grid_utils.h:63-80) and may still reach points inside.
    Cell sizes differ per axis and the radius is anisotropic."""
    from tensorflow_graphics_point_clouds_amd import pc
    rng = np.random.default_rng(40 + d)
    n, n_ctr, batch = 60000, 40000, 2
    pts = rng.random((n, d)).astype(np.float32)
    bids = np.sort(rng.integers(0, batch, n)).astype(np.int32)
    ctr = (rng.random((n_ctr, d)) * 2.0 - 0.5).astype(np.float32)
    cb = np.sort(rng.integers(0, batch, n_ctr)).astype(np.int32)
    radii = (np.array([0.05, 0.08, 0.06, 0.3][:d]) * (2.0 if d == 4 else 1.0)).astype(np.float32)
    g = oracle.Grid(pts, bids, batch, radii)
    nbh = oracle.Neighborhood(g, radii, ctr, cb)
    grid = pc.Grid(pc.PointCloud(dev(pts), dev(bids), batch), dev(radii))
    got = pc.Neighborhood(grid, dev(radii), pc.PointCloud(dev(ctr), dev(cb), batch))
    outside = ((ctr < 0) | (ctr > 1)).any(axis=1)
    starts = oracle.segment_starts(nbh.ranges)
    assert int(((nbh.ranges - starts)[outside] > 0).sum()) > 100     # the case is exercised
    _same(got._samples_neigh_ranges, nbh.ranges, "ranges")
    _same(got._neighbors, nbh.neighbors, "pair table")


# ------------------------------------------------- configuration 2 at 16 x 1024 ----

def test_modelnet_shaped_batch_hierarchy_equals_oracle_at_full_size(oracle):
    """16 x 1024 points (16 384 keys: the upper edge of the single-launch sort and of the
    one-call grid): every level's grid, neighbourhood and cell-average points bit for bit."""
    from tensorflow_graphics_point_clouds_amd import pc, synthetic
    cfg = synthetic.config2()
    assert len(cfg["points"]) == 16384
    hier = pc.PointHierarchy(pc.PointCloud(dev(cfg["points"]), dev(cfg["batch_ids"]),
                                           cfg["batch_size"]), cfg["radii"], "cell average")
    pts, bids = cfg["points"], cfg["batch_ids"]
    for level, r in enumerate(cfg["radii"]):
        g = oracle.Grid(pts, bids, cfg["batch_size"], np.float32(r))
        nbh = oracle.Neighborhood(g, np.float32(r))
        gn = hier._neighborhoods[level]
        _same(gn._grid._sorted_indices, g.sorted_indices, "sort permutation")
        _same(gn._grid._sorted_keys, g.sorted_keys, "sorted keys")
        _same(gn._samples_neigh_ranges, nbh.ranges, "ranges")
        _same(gn._neighbors, nbh.neighbors, "pair table")
        pts, bids, _ = oracle.sampling(g.sorted_points, g.sorted_batch_ids, g.sorted_keys,
                                       g.num_cells, nbh.neighbors, nbh.ranges, 1)
        _same(hier._point_clouds[level + 1]._points, pts, "cell-average points")
        _same(hier._point_clouds[level + 1]._batch_ids, bids, "cell-average batch ids")


def test_modelnet_shaped_batch_chain_forward_backward_at_full_size(oracle):
    """Configuration 2 at its real size: 3 -> 64 -> 128 -> 256 Monte-Carlo convolutions
    down a three-level cell-average hierarchy of 16 x 1024 points, forward and backward
    through the whole chain.  Reference: the same chain in float64 on the oracle's
    hierarchy, pairs and densities (torch autograd), with leaky-ReLU between the levels.
    Bound: |got - expect| <= 1e-5 * mag elementwise for every level's output and for the
    gradients of every level's kernel weights, biases, final weights and of the input
    features.  mag is the same sum taken over the absolute values of its terms: a second
    chain is built from the absolute values of every operand (activation slopes entering as
    the factors they are), and its autograd gradients for the upstream |up| are the sums of
    absolute values of the terms of the true gradients."""
    from tensorflow_graphics_point_clouds_amd import layers, pc, synthetic
    cfg = synthetic.config2()
    rng = np.random.default_rng(2)
    pts, bids, batch = cfg["points"], cfg["batch_ids"], cfg["batch_size"]
    hier = pc.PointHierarchy(pc.PointCloud(dev(pts), dev(bids), batch), cfg["radii"],
                             "cell average")
    widths = [3, 64, 128, 256]
    f64 = dict(dtype=torch.float64, device="cuda")
    leaf = lambda a: torch.tensor(np.asarray(a, np.float64), device="cuda", requires_grad=True)
    slope_of = lambda z: torch.where(z > 0, torch.ones_like(z), torch.full_like(z, 0.2))
    t_in, m_in = leaf(pts), leaf(np.abs(pts))
    g_in = dev(pts).requires_grad_(True)
    ref, mag, got = t_in, m_in, g_in
    params, mag_params, convs = [], [], []
    cur_pts, cur_bids = pts, bids
    for level, r in enumerate(cfg["radii"]):
        conv_r = np.float32(1.5 * r)
        g = oracle.Grid(cur_pts, cur_bids, batch, np.float32(r))
        nbh = oracle.Neighborhood(g, np.float32(r))
        nxt_pts, nxt_bids, _ = oracle.sampling(g.sorted_points, g.sorted_batch_ids, g.sorted_keys,
                                               g.num_cells, nbh.neighbors, nbh.ranges, 1)
        cg = oracle.Grid(cur_pts, cur_bids, batch, conv_r)
        cn = oracle.Neighborhood(cg, conv_r, nxt_pts, nxt_bids)
        pdf = torch.tensor(cn.pdf_per_pair(0.2), device="cuda")
        ids = torch.tensor(cn.original_neigh_ids, device="cuda").long()
        radii = np.full(3, conv_r, np.float32)
        delta = torch.tensor(((cur_pts[cn.original_neigh_ids[:, 0]]
                               - nxt_pts[cn.original_neigh_ids[:, 1]]) / radii).astype(np.float64),
                             device="cuda")
        w, b, wo = synthetic.mcconv_weights(rng, 3, widths[level], widths[level + 1], 16, 1)
        b = (0.1 * rng.standard_normal(b.shape)).astype(np.float32)
        tw, tb, two = leaf(w), leaf(b), leaf(wo)
        n_out = len(nxt_pts)

        def chain(feat, basis, final):
            rows = feat[ids[:, 0]][:, :, None] * basis[:, None, :]
            proj = torch.zeros((n_out, feat.shape[1], 16), **f64).index_add(0, ids[:, 1], rows)
            return proj.reshape(n_out, -1) @ final

        z = delta @ tw[0] + tb[0]
        basis = torch.nn.functional.leaky_relu(z, 0.2) / pdf[:, None]
        ref = chain(ref, basis, two[0])
        # the chain of magnitudes: value |basis|, derivative with respect to the kernel
        # weights |delta| * slope / pdf and to the bias slope / pdf
        mw, mb, mwo = leaf(np.abs(w)), leaf(np.abs(b)), leaf(np.abs(wo))
        lin = (delta.abs() @ mw[0] + mb[0]) * slope_of(z.detach()) / pdf[:, None]
        mag_basis = basis.detach().abs() + (lin - lin.detach())
        mag = chain(mag, mag_basis, mwo[0])
        conv = layers.MCConv(widths[level], widths[level + 1], 3, num_mlps=1, mlp_size=[16],
                             non_linearity_type="leaky_relu", weights=dev(w), biases=dev(b),
                             final_weights=dev(wo))
        got = conv(got, hier[level], hier[level + 1], float(conv_r), bandwidth=0.2)
        err = (got.detach().double() - ref.detach()).abs()
        assert bool((err <= 1e-5 * mag.detach() + 1e-30).all()), \
            "level %d output: max err/mag %g" % (level, float((err / mag.detach().clamp(min=1e-300)).max()))
        params.append((tw, tb, two))
        mag_params.append((mw, mb, mwo))
        convs.append(conv)
        if level < 2:
            mag = mag * slope_of(ref.detach())
            ref = torch.nn.functional.leaky_relu(ref, 0.2)
            got = torch.nn.functional.leaky_relu(got, 0.2)
        cur_pts, cur_bids = nxt_pts, nxt_bids

    up = torch.randn(got.shape, generator=torch.Generator(device="cuda").manual_seed(3),
                     device="cuda")
    got.backward(up)
    grads = torch.autograd.grad((ref * up.double()).sum(),
                                [t_in] + [p for trio in params for p in trio])
    mags = torch.autograd.grad((mag * up.double().abs()).sum(),
                               [m_in] + [p for trio in mag_params for p in trio])
    cases = [(g_in.grad, grads[0], mags[0], "input features")]
    for level, conv in enumerate(convs):
        mine = (conv.weights.grad, conv.biases.grad, conv.final_weights.grad)
        names = ("kernel weights", "kernel biases", "final weights")
        for j in range(3):
            cases.append((mine[j], grads[1 + 3 * level + j], mags[1 + 3 * level + j],
                          "level %d %s" % (level, names[j])))
    for mine, want, bound, what in cases:
        assert bool((bound >= want.abs() * (1 - 1e-9)).all()), what     # it is a magnitude
        err = (mine.double() - want).abs()
        assert bool((err <= 1e-5 * bound + 1e-30).all()), "%s: max err/mag %g" % (
            what, float((err / bound.clamp(min=1e-300)).max()))
