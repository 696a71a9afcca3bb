#!/usr/bin/env python3
"""Benchmark of the MCCNN hot path on one MI355X.

A step is one forward + backward pass of a Monte-Carlo convolution layer
(64 -> 64 channels, 16-unit kernel MLP, radius 0.15) over the scene-scale batch:
8 clustered clouds of 50k-150k points.  Grid, neighbourhood and densities are
built once before the timed region (their times are reported separately);
inputs are resident in HBM when timing starts.

Prints ONE JSON line: points/sec (centre points per second of fwd+bwd), the
roofline of the dominant kernel of the step (HIP events around every op call on
the launch stream), per-op figures, the isolated basis_proj figures on the
dense-neighbourhood case (C=128, K=32), and the host-CPU figure of the oracle on
a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
FP32_MATRIX_PEAK_TFLOPS = 157.3


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def op_bytes(name, M, N_in, N_out, C, K, D):
    """Operand bytes of one launch of each op (fp32, int32 pair table): every per-pair
    gather counted at full width (a feature row per pair).  On grid-ordered inputs
    most of the gathers are served by L2, so this figure can exceed what HBM moves; it is
    reported as `operand_GBps`, never as a roofline fraction."""
    if name == "basis_proj":
        return 4 * (M * K + M * C + N_out * C * K) + 8 * M + 4 * N_out
    if name == "basis_proj_grads":
        return 4 * (2 * M * K + M * C + N_out * C * K + N_in * C) + 8 * M + 4 * N_out
    if name == "mc_basis":
        return M * (8 + 2 * 4 * D + 4) + 4 * M * K
    if name == "mc_basis_grads":
        return M * (8 + 2 * 4 * D + 4) + 4 * M * K
    if name == "mc_conv_project":        # basis evaluated in registers: no [M, K] traffic
        return M * (8 + 4 * D + 4) + 4 * (M * C + N_out * C * K) + 4 * N_out * (1 + D)
    if name == "mc_conv_project_grads":  # kernel-MLP gradients only (no feature gradient)
        return M * (8 + 4 * D + 4) + 4 * (M * C + N_out * C * K) + 4 * N_out * (1 + D)
    return None


def compulsory_bytes(name, M, N_in, N_out, C, K, D):
    """HBM bytes one launch cannot avoid: every tensor counted once, whatever the number
    of times its rows are gathered.  The roofline fraction of an op is this figure over
    its launch time and the HBM peak, so it cannot exceed 1.

      pair stream   8 M (table) [+ 4 M densities] [+ 4 M K basis rows]
      coordinates   4 D (N_in + N_out)
      features      4 N_in C        read once (not 4 M C)
      projection    4 N_out C K     written (or read, for the gradient ops)
      ranges        4 N_out
    """
    pairs = 8 * M
    coords = 4 * D * (N_in + N_out)
    feats = 4 * N_in * C
    proj = 4 * N_out * C * K
    if name == "basis_proj":
        return pairs + 4 * M * K + feats + proj + 4 * N_out
    if name == "basis_proj_grads":       # + basis gradient written, feature gradient written
        return pairs + 2 * 4 * M * K + feats + proj + 4 * N_in * C + 4 * N_out
    if name in ("mc_conv_project", "kp_conv_project"):
        return pairs + (4 * M if name == "mc_conv_project" else 0) + coords + feats + proj + \
            4 * N_out
    if name == "mc_conv_project_grads":
        return pairs + 4 * M + coords + feats + proj + 4 * N_out
    if name in ("mc_basis", "mc_basis_grads"):
        return pairs + 4 * M + coords + 4 * M * K
    if name == "compute_pdf":
        return pairs + 4 * D * N_in + 4 * N_out + 4 * N_out
    if name == "compute_pdf_pt_grads":
        return pairs + 4 * D * N_in + 8 * N_out + 4 * D * N_in
    if name == "local_pool":
        return pairs + feats + 4 * N_out * C + 4 * N_out
    return None


def roofline_entry(by, operand_by, ms, calls=1.0):
    """GB/s and fraction of the HBM peak from compulsory bytes; `operand_GBps` beside it."""
    gbps = by * calls / ms / 1e6
    entry = {"GBps": round(gbps, 1), "frac_hbm_peak": round(gbps / HBM_PEAK_GBS, 4),
             "compulsory_bytes": by}
    if operand_by:
        entry["operand_GBps"] = round(operand_by * calls / ms / 1e6, 1)
        entry["operand_bytes"] = operand_by
    if entry["frac_hbm_peak"] > 1.0:
        entry["flag"] = "fraction above 1: the byte model counts more than HBM can have moved"
    return entry


def product_figures(name, N, C, K, CO):
    """(bytes, flops) of the dense products of the layer, one launch each."""
    flops = 2 * N * C * K * CO
    if name == "final_product":               # [N, C*K] x [C*K, CO] and [N, CO*K] x [CO*K, C]
        return 4 * (N * C * K + N * CO + C * K * CO), flops
    if name == "gemm_out":                    # [N, C*K] x [C*K, CO]
        return 4 * (N * C * K + N * CO + C * K * CO), flops
    if name == "gemm_dfeat":                  # [N, CO*K] x [CO*K, C]
        return 4 * (N * CO * K + N * C + C * K * CO), flops
    if name in ("projection_grad_product", "gemm_dproj"):   # [N, CO] x [CO, C*K]
        return 4 * (N * CO + N * C * K + C * K * CO), flops
    if name in ("weight_grad_product", "gemm_dfinal"):      # [C, N] x [N, CO*K]
        return 4 * (N * C + N * CO * K + C * K * CO), flops
    return None


def _source_digest(files):
    import hashlib
    h = hashlib.sha256()
    for f in files:
        with open(os.path.join(ROOT, "tensorflow_graphics_point_clouds_amd", "csrc", f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def measured_traffic(op, workload):
    """HBM-side bytes per launch from the committed counter summary (scaled FETCH_SIZE +
    WRITE_SIZE) -> (bytes, file) or (None, reason).  A summary names the kernel sources
    it was taken from and their digest (`sources <digest> <file> ...`); when the sources
    in the tree differ, the number belongs to another build and is not reported."""
    for fname in ("mcconv_layer_config3_hbm_traffic.txt",
                  "basis_proj_dense_case_hbm_traffic.txt"):
        path = os.path.join(ROOT, "profiles", fname)
        try:
            lines = open(path).read().splitlines()
        except OSError:
            continue
        digest = files = None
        for line in lines:
            parts = line.split()
            if len(parts) >= 3 and parts[0] == "sources":
                digest, files = parts[1], parts[2:]
        for line in lines:
            parts = line.split()
            if len(parts) == 4 and parts[0] == "traffic_bytes" and parts[1] == op \
                    and parts[2] == workload:
                if digest is None:
                    return None, "profiles/%s names no kernel sources" % fname
                try:
                    current = _source_digest(files)
                except OSError:
                    return None, "kernel sources of profiles/%s are missing" % fname
                if current != digest:
                    return None, ("profiles/%s was taken from other kernel sources (digest %s, "
                                  "tree has %s)" % (fname, digest, current))
                return int(parts[3]), "profiles/" + fname
    return None, "no counter summary for %s on %s" % (op, workload)


def build_scene(torch, pc, synthetic, scale):
    import numpy as np
    cfg = synthetic.config3(scale=scale)
    dev = lambda a: torch.as_tensor(np.ascontiguousarray(a)).cuda()
    cloud = pc.PointCloud(dev(cfg["points"]), dev(cfg["batch_ids"]), cfg["batch_size"])
    return cfg, cloud


def time_build(torch, pc, cloud, radius, reps=3):
    """Grid + neighbourhood + density + grid-ordered view build as the layer uses
    them, best of `reps` (ms).  `caller_order_tables_ms` is the extra cost of the
    pair table in the caller's centre order with original point ids, which only
    the op-level API (basis_proj, pooling) reads; it is not part of the sum."""
    out = {}
    best = extra = None
    for _ in range(reps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        grid = pc.Grid(cloud, radius)
        grid.get_DS()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        nbh = pc.Neighborhood(grid, radius, cloud)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        nbh.point_pdf(bandwidth=0.2)
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        nbh.sorted_view().pair_pdf(nbh)
        torch.cuda.synchronize()
        t4 = time.perf_counter()
        nbh._original_neigh_ids
        torch.cuda.synchronize()
        t5 = time.perf_counter()
        cur = dict(grid_ms=(t1 - t0) * 1e3, neighbors_ms=(t2 - t1) * 1e3,
                   pdf_ms=(t3 - t2) * 1e3, view_ms=(t4 - t3) * 1e3)
        if best is None or sum(cur.values()) < sum(best.values()):
            best = cur
        extra = (t5 - t4) * 1e3 if extra is None else min(extra, (t5 - t4) * 1e3)
    out.update(best)
    out["caller_order_tables_ms"] = extra
    return grid, nbh, out


def _set_cpu_threads(orc, n):
    """Threads of the oracle's OpenMP loops and of numpy's BLAS."""
    try:
        orc.lib().omp_set_num_threads(int(n))
    except AttributeError:
        os.environ["OMP_NUM_THREADS"] = str(n)
    try:
        from threadpoolctl import threadpool_limits
        return threadpool_limits(limits=int(n))
    except Exception:
        return None


def cpu_baseline(synthetic):
    """MCConv fwd+bwd of the oracle (C with OpenMP, numpy GEMMs) on the host cores:
    the whole configuration-3 workload with all cores, and one of its clouds with a
    single thread (bounded so that the default run stays within minutes)."""
    import numpy as np
    from oracle import mccnn_oracle as orc

    def prepare(cfg):
        pts, bids = cfg["points"], cfg["batch_ids"]
        n = len(pts)
        r = np.float32(cfg["radius"])
        t0 = time.perf_counter()
        g = orc.Grid(pts, bids, cfg["batch_size"], r)
        nbh = orc.Neighborhood(g, r, pts, bids)
        pdf = nbh.pdf_per_pair(0.2).astype(np.float32)
        build_s = time.perf_counter() - t0
        ids = nbh.original_neigh_ids
        rng = np.random.default_rng(0)
        C, K, CO = cfg["c_in"], cfg["hidden"], cfg["c_out"]
        w, b, wo = synthetic.mcconv_weights(rng, 3, C, CO, K, 1)
        feat = rng.standard_normal((n, C)).astype(np.float32)
        up = rng.standard_normal((n, CO)).astype(np.float32)
        inv_r = np.float32(1.0) / r

        def step():
            diff = (pts[ids[:, 0]] - pts[ids[:, 1]]) * inv_r
            z = diff @ w[0] + b[0]
            basis = (np.maximum(z, 0) / pdf[:, None]).astype(np.float32)
            proj = orc.basis_proj_f32(basis, feat, ids, nbh.ranges)
            out = proj.reshape(n, C * K) @ wo[0]
            dproj = (up @ wo[0].T).reshape(n, C, K)
            dwo = proj.reshape(n, C * K).T @ up
            dbasis, dfeat = orc.basis_proj_grads_f32(basis, feat, ids, nbh.ranges, dproj)
            dz = dbasis * (z > 0) / pdf[:, None]
            dw = diff.T @ dz
            db = dz.sum(axis=0)
            return out, dwo, dfeat, dw, db

        return n, len(ids), build_s, step

    def timed(step, budget_s, min_reps):
        step()
        times = []
        t_start = time.perf_counter()
        while len(times) < min_reps or time.perf_counter() - t_start < budget_s:
            t0 = time.perf_counter()
            step()
            times.append(time.perf_counter() - t0)
            if time.perf_counter() - t_start > 2.5 * budget_s:
                break
        return times

    cores = int(os.environ.get("OMP_NUM_THREADS", "0")) or len(os.sched_getaffinity(0))
    limit = _set_cpu_threads(orc, cores)
    n, m, build_s, step = prepare(synthetic.config3(scale=1.0))
    times = timed(step, 10.0, 2)
    all_cores = {"points_per_s": n / (sum(times) / len(times)), "cores": cores,
                 "ms_per_step_mean": 1e3 * sum(times) / len(times),
                 "ms_per_step_min": 1e3 * min(times), "passes": len(times),
                 "build_s": round(build_s, 2), "points": n, "pairs": m}
    del step
    limit = _set_cpu_threads(orc, 1)
    n1, m1, build1_s, step1 = prepare(synthetic.config3(scale=1.0, batch=1))
    times1 = timed(step1, 8.0, 1)
    one_thread = {"points_per_s": n1 / (sum(times1) / len(times1)), "cores": 1,
                  "ms_per_step_mean": 1e3 * sum(times1) / len(times1),
                  "ms_per_step_min": 1e3 * min(times1), "passes": len(times1),
                  "points": n1, "pairs": m1,
                  "sample": "the first cloud of the configuration-3 generator"}
    del step1
    limit = _set_cpu_threads(orc, cores)

    # configuration 1, the case the reference's own CPU path is quoted on: 2 x 1024
    # points, grid + neighbours + densities + one MCConv 8 -> 16 forward
    c1 = synthetic.config1()
    r1 = np.float32(c1["radius"])

    def c1_step():
        g1 = orc.Grid(c1["points"], c1["batch_ids"], c1["batch_size"], r1)
        n1_ = orc.Neighborhood(g1, r1, c1["points"], c1["batch_ids"])
        return orc.mc_conv_forward(c1["features"], c1["points"], c1["points"], n1_,
                                   n1_.pdf_per_pair(c1["bandwidth"]), c1["weights"], c1["biases"],
                                   c1["final_weights"], r1)

    c1_step()
    t0 = time.perf_counter()
    for _ in range(10):
        c1_step()
    c1_ms = (time.perf_counter() - t0) * 100.0
    return {"value": all_cores["points_per_s"], "unit": "points/s", "cores": cores,
            "kind": "port",
            "sample": "the whole configuration-3 workload (%d points, %d pairs), %d fwd+bwd "
                      "passes of the C/OpenMP oracle with numpy GEMMs on %d threads; "
                      "`one_thread` is the same on one cloud with a single thread"
                      % (n, m, len(times), cores),
            "all_cores": all_cores, "one_thread": one_thread,
            "config1_forward_with_build_ms": c1_ms,
            "config1_points_per_s": len(c1["points"]) / (c1_ms * 1e-3)}


def config1_forward(torch, pc, layers, synthetic, steps=50):
    """Configuration 1 on the GPU: 2 x 1024 points, grid + neighbours + densities +
    one MCConv 8 -> 16 forward, everything rebuilt every step."""
    import numpy as np
    cfg = synthetic.config1()
    dev = lambda a: torch.as_tensor(np.ascontiguousarray(a)).cuda()
    pts, bids, feats = dev(cfg["points"]), dev(cfg["batch_ids"]), dev(cfg["features"])
    conv = layers.MCConv(8, 16, 3, num_mlps=1, mlp_size=[16], non_linearity_type="relu",
                         weights=dev(cfg["weights"]), biases=dev(cfg["biases"]),
                         final_weights=dev(cfg["final_weights"]))

    def step():
        cloud = pc.PointCloud(pts, bids, cfg["batch_size"])
        with torch.no_grad():
            return conv(feats, cloud, cloud, cfg["radius"], bandwidth=cfg["bandwidth"])

    for _ in range(5):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    return {"workload": "config 1: 2 x 1024 points, r=0.1, MCConv 8->16, K=16, forward only, "
                        "grid, neighbourhood and densities rebuilt every step",
            "ms_per_step": ms, "points_per_s": int(pts.shape[0]) / (ms * 1e-3)}


def kpconv_config5(torch, pc, layers, synthetic, _lib, steps=5):
    """Kernel-point convolution 128 -> 128, 15 kernel points (padded to 16), fwd+bwd
    on the scene-scale geometry (configuration 5): rigid with the linear and the
    Gaussian correlation (sigma = 0.3 r), and deformable (offsets from a rigid
    convolution, scaled to a spread of 0.01 r) with its regularisation loss."""
    import numpy as np
    cfg = synthetic.config5()
    dev = lambda a: torch.as_tensor(np.ascontiguousarray(a)).cuda()
    cloud = pc.PointCloud(dev(cfg["points"]), dev(cfg["batch_ids"]), cfg["batch_size"])
    r = cfg["radius"]
    nbh = pc.Neighborhood(pc.Grid(cloud, r), r, cloud)
    N, M, C, CO = cloud._points.shape[0], nbh._neighbors.shape[0], cfg["c_in"], cfg["c_out"]
    gen = torch.Generator(device="cuda").manual_seed(5)
    feats = torch.randn((N, C), device="cuda", generator=gen).requires_grad_(True)
    up = torch.randn((N, CO), device="cuda", generator=gen)

    def measure(conv, influence, regularised):
        def step():
            out = conv(feats, cloud, cloud, r, neighborhood=nbh, kernel_influence_dist=influence)
            if regularised:
                torch.autograd.backward([out, conv.regularization_loss()],
                                        [up, torch.ones((), device="cuda")])
            else:
                out.backward(up)
            feats.grad = None
            for p in conv.parameters():
                p.grad = None

        for _ in range(2):
            step()
        torch.cuda.synchronize()
        _lib.start_timing()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        ops = {k.replace("_ordered", ""): round(sum(v) / steps, 3)
               for k, v in _lib.collect_timing().items()}
        return {"ms_per_step": ms, "points_per_s": N / (ms * 1e-3), "ops_ms": ops}

    kp = cfg["kernel_points"] / 0.75
    res = {"workload": "config 5: KPConv %d->%d, 15 kernel points, radius %.2f, %d points, "
                       "%d pairs, fwd+bwd" % (C, CO, r, N, M)}
    res.update(measure(layers.KPConv(C, CO, custom_kernel_points=kp, kp_interpolation="linear",
                                     seed=5), None, False))
    res["gaussian"] = measure(layers.KPConv(C, CO, custom_kernel_points=kp,
                                            kp_interpolation="gaussian", seed=5), 0.3 * r, False)
    conv = layers.KPConv(C, CO, custom_kernel_points=kp, kp_interpolation="linear",
                         deformable=True, seed=5)
    with torch.no_grad():
        conv.offset_weights.normal_(0.0, 1.0, generator=gen)
        conv(feats, cloud, cloud, r, neighborhood=nbh)
        conv.offset_weights.mul_(0.01 / float(conv._last[0].std()))
    res["deformable_with_regularisation_loss"] = measure(conv, None, True)
    return res


def config2_network(torch, pc, layers, synthetic, steps=20):
    """Configuration 2: 16 x 1024 points on random primitives, cell-average hierarchy
    at radii 0.1 / 0.2 / 0.4, one Monte-Carlo convolution per level (3 -> 64 -> 128 ->
    256, convolution radius 1.5 x the level's), fwd+bwd; once with the hierarchy,
    grids, neighbourhoods and densities rebuilt every step, once with them reused."""
    import numpy as np
    cfg = synthetic.config2()
    dev = lambda a: torch.as_tensor(np.ascontiguousarray(a)).cuda()
    pts, bids, batch = dev(cfg["points"]), dev(cfg["batch_ids"]), cfg["batch_size"]
    widths = cfg["channels"]
    convs = [layers.MCConv(widths[i], widths[i + 1], 3, num_mlps=1, mlp_size=[16],
                           non_linearity_type="leaky_relu", seed=i) for i in range(3)]
    params = [p for c in convs for p in c.parameters()]
    state = {}

    def step(build):
        if build or "hier" not in state:
            state["hier"] = pc.PointHierarchy(pc.PointCloud(pts, bids, batch), cfg["radii"],
                                              "cell average")
            state["nbh"] = [None] * 3
        hier, feat = state["hier"], pts
        for level, r in enumerate(cfg["radii"]):
            feat = torch.relu(convs[level](feat, hier[level], hier[level + 1], 1.5 * r,
                                           bandwidth=0.2, neighborhood=state["nbh"][level]))
            if not build:
                state["nbh"][level] = convs[level].last_neighborhood
        feat.sum().backward()
        for p in params:
            p.grad = None

    def timed(build):
        for _ in range(3):
            step(build)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step(build)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    n = int(pts.shape[0])
    with_build = timed(True)
    reused = timed(False)

    # the prebuilt step enqueues kernels only: recorded once in a HIP graph and replayed
    def graph_step():
        hier, feat = state["hier"], pts
        for level, r in enumerate(cfg["radii"]):
            feat = torch.relu(convs[level](feat, hier[level], hier[level + 1], 1.5 * r,
                                           bandwidth=0.2, neighborhood=state["nbh"][level]))
        feat.sum().backward()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            graph_step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for p in params:
        p.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        graph_step()
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    replayed = (time.perf_counter() - t0) * 1e3 / steps
    return {"workload": "config 2: 16 x 1024 points, 3-level cell-average hierarchy, MCConv "
                        "3->64->128->256, fwd+bwd",
            "ms_per_step_with_build": with_build, "points_per_s_with_build": n / (with_build * 1e-3),
            "ms_per_step_prebuilt": reused, "points_per_s_prebuilt": n / (reused * 1e-3),
            "ms_per_step_prebuilt_graph_replay": replayed,
            "points_per_s_prebuilt_graph_replay": n / (replayed * 1e-3)}


def pointconv_config3(torch, pc, layers, synthetic, _lib, steps=5):
    """PointConv 64 -> 64 with 32 hidden units (the reference's default) on the clouds
    of configuration 3, fwd+bwd, neighbourhood and densities prebuilt."""
    cfg, cloud = build_scene(torch, pc, synthetic, 1.0)
    r = cfg["radius"]
    nbh = pc.Neighborhood(pc.Grid(cloud, r), r, cloud)
    n = int(cloud._points.shape[0])
    conv = layers.PointConv(64, 64, 3, size_hidden=32)
    gen = torch.Generator(device="cuda").manual_seed(6)
    feats = torch.randn((n, 64), device="cuda", generator=gen).requires_grad_(True)
    up = torch.randn((n, 64), device="cuda", generator=gen)

    def step():
        conv(feats, cloud, cloud, r, neighborhood=nbh).backward(up)
        feats.grad = None
        for p in conv.parameters():
            p.grad = None

    for _ in range(2):
        step()
    torch.cuda.synchronize()
    _lib.start_timing()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    ops = {k: round(sum(v) / steps, 3) for k, v in _lib.collect_timing().items()}
    return {"workload": "PointConv 64->64, 32 hidden units, radius %.2f, %d points, %d pairs, "
                        "fwd+bwd" % (r, n, int(nbh._neighbors.shape[0])),
            "ms_per_step": ms, "points_per_s": n / (ms * 1e-3), "ops_ms": ops}


def per_op_times(torch, pc, layers, synthetic, _lib, radius=0.04, reps=5):
    """Every op of the path on the dense case (4 x 200k uniform points, radius
    0.04): average milliseconds from HIP events around each C-ABI call, with
    algorithmic GB/s where a byte count is defined.  Dynamic-size ops include
    their one host synchronisation."""
    import numpy as np
    cfg = synthetic.config4()
    dev = lambda a: torch.as_tensor(np.ascontiguousarray(a)).cuda()
    cloud = pc.PointCloud(dev(cfg["points"]), dev(cfg["batch_ids"]), cfg["batch_size"])
    N, D, B = cloud._points.shape[0], 3, cfg["batch_size"]
    feats = torch.randn((N, 64), device="cuda")

    def run():
        grid = pc.Grid(cloud, radius)
        grid.get_DS()
        nbh = pc.Neighborhood(grid, radius)                    # self neighbourhood
        nbh.compute_pdf(bandwidth=0.2)
        g = torch.ones(N, device="cuda")
        pts = grid._sorted_points
        from tensorflow_graphics_point_clouds_amd import tfg_custom_ops as tfg
        # a table that find_neighbors reported as an untruncated self-neighbourhood takes the
        # symmetric kernel by itself: the general one is timed on a view of the same table
        tfg.compute_pdf_pt_grads(pts, nbh._neighbors.view(-1, 2), nbh._samples_neigh_ranges,
                                 torch.full((3,), 5.0, device="cuda"), nbh._inv_radii, g, 0)
        tfg.compute_pdf_pt_grads(pts, nbh._neighbors, nbh._samples_neigh_ranges,
                                 torch.full((3,), 5.0, device="cuda"), nbh._inv_radii, g, 0,
                                 symmetric=True)
        pc.sample(nbh, "poisson")
        pc.sample(nbh, "average")
        layers.MaxPooling()(feats, cloud, None, radius, neighborhood=nbh)
        layers.AveragePooling()(feats, cloud, None, radius, neighborhood=nbh)
        layers.GlobalMaxPooling()(feats, cloud)
        return grid, nbh

    run()
    torch.cuda.synchronize()
    _lib.start_timing()
    for _ in range(reps):
        grid, nbh = run()
    t = _lib.collect_timing()
    M = nbh._neighbors.shape[0]
    ncol = B * grid._num_cells_host[0] * grid._num_cells_host[1]
    passes = (grid._key_bits + 7) // 8
    by = {
        "compute_keys": N * (4 * D + 4 + 8),
        "sort_keys_descending": passes * 2 * 12 * N,
        "gather_points": 2 * N * (4 * D + 4) + 4 * N,
        "build_grid_ds": 8 * N + 8 * ncol,
        "find_neighbors_count": N * (4 * D + 4) + N * (4 * D + 8) + 8 * ncol + 4 * N,
        "find_neighbors_fill": N * (4 * D) + N * (4 * D) + 8 * M,
        "compute_pdf": N * 4 * D + 8 * M + 4 * N + M * 4 * D + 4 * N,
        "compute_pdf_pt_grads": N * 4 * D + 8 * M + 8 * N + M * 4 * D + 2 * N * 4 * D,
        "compute_pdf_pt_grads_symmetric": N * 4 * D + 8 * M + 8 * N + M * (4 * D + 4) + N * 4 * D,
        "local_pool": 4 * M * 64 + 8 * M + 4 * N * 64,
    }
    out = {"workload": "4x200k uniform, r=%.2f, self neighbourhood, %d pairs; pooling C=64"
                       % (radius, M)}
    # ops whose operand count includes per-pair gathers: the roofline uses the compulsory bytes
    compulsory = {name: compulsory_bytes(name, M, N, N, 64, 1, D)
                  for name in ("compute_pdf", "compute_pdf_pt_grads", "local_pool")}
    compulsory["compute_pdf_pt_grads_symmetric"] = compulsory["compute_pdf_pt_grads"]
    for name, vals in sorted(t.items()):
        ms = sum(vals) / reps
        calls = len(vals) // reps
        entry = {"ms": round(ms, 4), "calls_per_pass": calls}
        if name in compulsory:
            entry.update(roofline_entry(compulsory[name], by[name], ms, calls))
        elif name in by:
            entry.update(roofline_entry(by[name], None, ms, calls))
        out[name] = entry
    return out


def isolated_basis_proj(torch, pc, synthetic, tfg, _lib, radius=0.04, steps=5, gathered=False):
    """basis_proj forward and gradients alone on 4 x 200k uniform points,
    C=128, K=32 (the dense-neighbourhood case)."""
    import numpy as np
    cfg = synthetic.config4()
    dev = lambda a: torch.as_tensor(np.ascontiguousarray(a)).cuda()
    cloud = pc.PointCloud(dev(cfg["points"]), dev(cfg["batch_ids"]), cfg["batch_size"])
    grid = pc.Grid(cloud, radius)
    nbh = pc.Neighborhood(grid, radius, cloud)
    ids, ranges = nbh._original_neigh_ids, nbh._samples_neigh_ranges
    M, N, C, K = ids.shape[0], cloud._points.shape[0], cfg["c_in"], cfg["basis"]
    gen = torch.Generator(device="cuda").manual_seed(4)
    basis = torch.rand((M, K), device="cuda", generator=gen)
    feat = torch.randn((N, C), device="cuda", generator=gen)
    up = torch.randn((N, C, K), device="cuda", generator=gen)
    res = {"workload": "4x200k uniform, r=%.2f, C=%d, K=%d" % (radius, C, K), "pairs": M}

    def run(tag, ids, ranges, feat):
        for _ in range(2):
            out = tfg._basis_proj_raw(basis, feat, ids, ranges, None)
            tfg.basis_proj_grads(basis, feat, ids, ranges, up, None)
        del out
        _lib.start_timing()
        for _ in range(steps):
            tfg._basis_proj_raw(basis, feat, ids, ranges, None)
            tfg.basis_proj_grads(basis, feat, ids, ranges, up, None)
        t = {k.replace("_ordered", ""): v for k, v in _lib.collect_timing().items()}
        for name in ("basis_proj", "basis_proj_grads"):
            ms = sum(t[name]) / len(t[name])
            by = op_bytes(name, M, N, N, C, K, 3)
            entry = {"ms": ms}
            entry.update(roofline_entry(compulsory_bytes(name, M, N, N, C, K, 3), by, ms))
            # the metric's own definition: operand bytes (4*C per pair for the feature rows)
            # over kernel time; with the pairs in the caller's order those rows do come from
            # HBM (counter traffic 0.99x this figure), in grid order L2 serves most of them
            entry["operand_frac_hbm_peak"] = round(by / ms / 1e6 / HBM_PEAK_GBS, 4)
            # (the workload tag of the counter summary: r = 0.04 carries no radius suffix)
            workload = "dense_C%d_K%d%s%s" % (C, K, tag, "" if radius == 0.04 else "_r%.2f" % radius)
            traffic, source = measured_traffic(name, workload)
            entry["traffic"], entry["traffic_source"] = traffic, source
            if traffic:
                entry["traffic_frac"] = round(traffic / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
            res[name + tag] = entry
        # the atomic-free variant: per-pair rows of the feature gradient written to a
        # [M, C] workspace and summed per point over the transposed pair lists (built once
        # per neighbourhood, timed separately)
        if gathered and tfg.gathered_grads_supported(C, K):
            tr = tfg.transpose_neighbors(ids, N)
            tfg.basis_proj_grads(basis, feat, ids, ranges, up, None, transposed=tr)
            _lib.start_timing()
            for _ in range(steps):
                tr = tfg.transpose_neighbors(ids, N)
                tfg.basis_proj_grads(basis, feat, ids, ranges, up, None, transposed=tr)
            t = _lib.collect_timing()
            ms = sum(t["basis_proj_grads_gathered"]) / steps
            by = op_bytes("basis_proj_grads", M, N, N, C, K, 3)
            entry = {"ms": ms, "transpose_neighbors_ms": sum(t["transpose_neighbors"]) / steps,
                     "workspace_bytes": 4 * M * C}
            entry.update(roofline_entry(compulsory_bytes("basis_proj_grads", M, N, N, C, K, 3), by, ms))
            res["basis_proj_grads_gathered" + tag] = entry

    # the reference's call pattern: pairs address the features by original point id
    # (custom_ops_wrapper.py:185-189), points and centres in the caller's (random) order
    run("", ids, ranges, feat)
    # the same pairs with points and centres renumbered in grid-cell order
    view = nbh.sorted_view()
    run("_grid_order", view.table, view.ranges, feat[view.point_order].contiguous())
    del basis, up, feat
    # the density estimate and Poisson-disk sampling at the same radius (self neighbourhood)
    self_nbh = pc.Neighborhood(grid, radius)
    for timed in (False, True):
        if timed:
            _lib.start_timing()
        for _ in range(steps if timed else 1):
            self_nbh.compute_pdf(bandwidth=0.2)
            sampled, _ = pc.sample(self_nbh, "poisson")
    t = _lib.collect_timing()
    ms = sum(t["compute_pdf"]) / steps
    by = N * 4 * 3 + 8 * M + 4 * N + M * 4 * 3 + 4 * N
    res["compute_pdf"] = {"ms": ms}
    res["compute_pdf"].update(roofline_entry(compulsory_bytes("compute_pdf", M, N, N, 1, 1, 3), by, ms))
    res["poisson_disk_sampling"] = {"ms": (sum(t["sampling_count"]) + sum(t["sampling_fill"])) / steps,
                                    "selected": int(sampled._points.shape[0])}
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--scale", type=float, default=1.0, help="shrink the point counts (tests)")
    ap.add_argument("--fuse-final", action="store_true",
                    help="run the product with the final weights inside the projection kernel")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline")
    ap.add_argument("--no-isolated", action="store_true", help="skip the isolated basis_proj case")
    ap.add_argument("--no-sweep", action="store_true",
                    help="skip the other two radii (0.02, 0.06) of the dense case")
    ap.add_argument("--no-small-configs", action="store_true",
                    help="skip configurations 1 (2 x 1024 points, forward) and 2 (16 x 1024 "
                         "points, three-level network, fwd+bwd): they launch the layer's kernels "
                         "on tiny shapes and blur the per-kernel averages of a profile")
    ap.add_argument("--extra-configs", action="store_true",
                    help="also time PointConv on the scene-scale clouds and the atomic-free "
                         "variant of the basis_proj gradients")
    ap.add_argument("--only-dense-radius", type=float, default=None,
                    help="only run the isolated basis_proj case at this radius and exit (counter "
                         "runs for the radii of the sweep)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a 1 GiB device copy three times (reference point for the "
                         "FETCH_SIZE / WRITE_SIZE counters) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py measures one GPU: this build has no multi-GPU path (clouds would be "
            "sharded whole across GPUs with no exchange in the forward pass); run with --gpus 1")
        sys.exit(2)

    import numpy as np
    import torch
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.calibrate_copy:
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")      # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "3 device copies of 1 GiB (2^30 bytes read, 2^30 written "
                                         "each)"}))
        return
    from tensorflow_graphics_point_clouds_amd import _lib, layers, pc, synthetic, tfg_custom_ops
    _lib.lib()
    torch.backends.cuda.matmul.allow_tf32 = False
    if args.only_dense_radius is not None:
        print(json.dumps(isolated_basis_proj(torch, pc, synthetic, tfg_custom_ops, _lib,
                                             radius=args.only_dense_radius, steps=2)))
        return

    cfg, cloud = build_scene(torch, pc, synthetic, args.scale)
    radius = cfg["radius"]
    grid, nbh, build_ms = time_build(torch, pc, cloud, radius)
    N = cloud._points.shape[0]
    M = nbh._neighbors.shape[0]
    C, CO, K, D = cfg["c_in"], cfg["c_out"], cfg["hidden"], 3
    log("scene: %d points, %d pairs (mean %.1f per point), build %s" % (N, M, M / N, build_ms))

    conv = layers.MCConv(C, CO, D, num_mlps=1, mlp_size=[K], non_linearity_type="leaky_relu",
                         seed=3, fuse_final=args.fuse_final)
    gen = torch.Generator(device="cuda").manual_seed(3)
    feats = torch.randn((N, C), device="cuda", generator=gen).requires_grad_(True)
    up = torch.randn((N, CO), device="cuda", generator=gen)

    def step():
        out = conv(feats, cloud, cloud, radius, neighborhood=nbh)
        out.backward(up)
        feats.grad = None
        for p in conv.parameters():
            p.grad = None

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # the timed region: exactly `steps` steps with nothing recorded inside a step (one event
    # after each step gives the median and the minimum)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(args.steps):
        step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt * 1e3 / args.steps
    step_ms = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    # a second region of the same length with a pair of events around every op call: the
    # per-op times (about 14 event records per step)
    _lib.start_timing()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step_instrumented = (time.perf_counter() - t0) * 1e3 / args.steps
    per_op = {k.replace("_ordered", ""): v for k, v in _lib.collect_timing().items()}

    ops = {}
    for name, vals in per_op.items():
        ms = sum(vals) / args.steps            # per step, over all calls of the op
        calls = len(vals) / args.steps
        by = compulsory_bytes(name, M, N, N, C, K, D)
        ops[name] = {"ms": round(ms, 4), "calls_per_step": calls}
        if by:
            ops[name].update(roofline_entry(by, op_bytes(name, M, N, N, C, K, D), ms, calls))
        fig = product_figures(name, N, C, K, CO)
        if fig:                           # dense products: matrix-core and HBM figures
            pby, flops = fig
            ops[name].update(flops=flops, TFLOPs=round(flops * calls / ms / 1e9, 1),
                             frac_fp32_matrix_peak=round(flops * calls / ms / 1e9 /
                                                         FP32_MATRIX_PEAK_TFLOPS, 4),
                             compulsory_bytes=pby, GBps_dense=round(pby * calls / ms / 1e6, 1),
                             library="hipBLASLt via torch.matmul" if name.startswith("gemm_")
                             else "hand-written")
        if name in ("permute_rows", "gather_rows"):
            ops[name].update(GBps_copy=round(8 * N * C * calls / ms / 1e6, 1))
    kernel_ms = sum(v["ms"] for v in ops.values())
    ops["host_gaps_and_small_kernels"] = {"ms": round(ms_per_step_instrumented - kernel_ms, 4)}
    dominant = max((n for n in ops if "GBps" in ops[n]), key=lambda n: ops[n]["ms"])
    launch_ms = ops[dominant]["ms"] / ops[dominant]["calls_per_step"]
    traffic, traffic_source = (measured_traffic(dominant, "config3_C%d_K%d" % (C, K))
                               if args.scale == 1.0 else (None, "reduced scale"))
    roof = {"kernel": dominant, "bound": "hbm", "achieved": ops[dominant]["GBps"],
            "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": ops[dominant]["frac_hbm_peak"],
            "traffic": traffic, "traffic_source": traffic_source,
            "launch_ms": round(launch_ms, 4),
            "launches_per_step": ops[dominant]["calls_per_step"],
            "compulsory_bytes": ops[dominant]["compulsory_bytes"],
            "operand_GBps": ops[dominant].get("operand_GBps"),
            "matrix_TFLOPs": round(2.0 * M * C * K / launch_ms / 1e9, 1),
            "matrix_frac_fp32_peak": round(2.0 * M * C * K / launch_ms / 1e9 /
                                           FP32_MATRIX_PEAK_TFLOPS, 4),
            "note": "achieved = compulsory HBM bytes of one launch (pair table and densities, "
                    "coordinates, the feature table once, the [N, C, K] output) over the launch "
                    "time from HIP events; `operand_GBps` counts every per-pair feature-row read "
                    "(4*C per pair, served mostly by L2 on the grid-ordered view); `traffic` is "
                    "what the HBM counters saw per launch, `traffic_frac` that over launch time "
                    "and peak; `matrix_*` is the segmented C x K contraction against the fp32 "
                    "matrix peak"}
    if traffic:
        roof["traffic_frac"] = round(traffic / (launch_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
    # the step as a whole against the fp32 matrix peak: four dense products [N, C*K] x
    # [C*K, C_out] (forward, feature gradient, projection gradient, final-weight gradient) and
    # three projection-shaped contractions over the pairs
    step_flops = 4 * 2.0 * N * C * K * CO + 3 * 2.0 * M * C * K
    roof["step_flops"] = step_flops
    roof["step_matrix_TFLOPs"] = round(step_flops / ms_per_step / 1e9, 1)
    roof["step_matrix_frac"] = round(step_flops / ms_per_step / 1e9 / FP32_MATRIX_PEAK_TFLOPS, 4)
    # what this box's HBM delivers to a plain device-to-device copy of 1 GiB (2^30 bytes read and
    # 2^30 written per copy): a measured ceiling beside the published 8 TB/s that `peak` uses
    src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")
    dst = torch.empty_like(src)
    for _ in range(2):
        dst.copy_(src)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        dst.copy_(src)
    e1.record()
    torch.cuda.synchronize()
    roof["measured_copy_GBps"] = round(5 * 2.0 * (1 << 30) / (e0.elapsed_time(e1) * 1e-3) / 1e9, 1)
    del src, dst

    result = {
        "metric": "MCConv layer fwd+bwd points/sec", "value": N / (ms_per_step * 1e-3),
        "unit": "points/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "ms_per_step_median": step_ms[len(step_ms) // 2],
        "ms_per_step_min": step_ms[0], "ms_per_step_instrumented": ms_per_step_instrumented,
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "dense_products": ("bf16 matrix pipe, three-way operand splits, float32 accumulation "
                           "(float32-accurate)" if _lib.lib().mccnn_split_products_enabled()
                           else "float32 matrix instructions"),
        "config": {"workload": "config 3: 8 clustered clouds of 50k-150k points (seed 1003), "
                               "MCConv 64->64, 16-unit kernel MLP, radius 0.15, fp32, fwd+bwd, "
                               "neighbourhood and densities prebuilt",
                   "points": N, "pairs": M, "scale": args.scale},
        "roofline": roof, "ops": ops, "build_ms": {k: round(v, 3) for k, v in build_ms.items()},
        "points_per_s_with_build": N / ((ms_per_step + sum(
            v for k, v in build_ms.items() if k != "caller_order_tables_ms")) * 1e-3),
    }
    if not args.no_isolated and args.scale == 1.0:
        del feats, up
        torch.cuda.empty_cache()
        # (the atomic-free gradient variant is timed with --extra-configs only: it launches
        # the same gradient kernel in another mode and would blur its average in a profile)
        result["basis_proj_isolated"] = isolated_basis_proj(torch, pc, synthetic, tfg_custom_ops,
                                                            _lib, gathered=args.extra_configs)
        torch.cuda.empty_cache()
        # the other two radii of the dense case's sweep (about 7 and 180 pairs per point)
        result["dense_radius_sweep"] = {}
        for radius in (() if args.no_sweep else (0.02, 0.06)):
            result["dense_radius_sweep"]["r=%.2f" % radius] = isolated_basis_proj(
                torch, pc, synthetic, tfg_custom_ops, _lib, radius=radius, steps=3)
            torch.cuda.empty_cache()
        result["per_op_dense_case"] = per_op_times(torch, pc, layers, synthetic, _lib)
        torch.cuda.empty_cache()
        result["kpconv_config5"] = kpconv_config5(torch, pc, layers, synthetic, _lib)
    if not args.no_small_configs and args.scale == 1.0:
        # the two small configurations, bound by launches and host round trips rather than bytes
        # (profile commands pass --no-small-configs: the layer's kernels on these tiny shapes
        # would blur the per-kernel averages)
        torch.cuda.empty_cache()
        result["config1_forward"] = config1_forward(torch, pc, layers, synthetic)
        result["config2_network"] = config2_network(torch, pc, layers, synthetic)
    if args.extra_configs:
        result["pointconv_config3"] = pointconv_config3(torch, pc, layers, synthetic, _lib)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(synthetic)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
