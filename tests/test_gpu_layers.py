"""Layer-level parity on the GPU: Monte-Carlo and kernel-point convolutions and
pooling against the oracle's float64 restatements (forward) and float64 autograd
of the same expressions (backward).  Outputs and gradients of the convolutions are
held elementwise to 1e-5 of the magnitude of their sums (`elementwise`); where a
test says "normwise" the bound is max |got - expect| <= tol * max |expect|."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.as_tensor(np.ascontiguousarray(a)).cuda().contiguous()


def normwise(got, expect, tol=1e-5):
    got, expect = np.asarray(got, np.float64), np.asarray(expect, np.float64)
    assert np.abs(got - expect).max() <= tol * np.abs(expect).max(), \
        np.abs(got - expect).max() / np.abs(expect).max()


def elementwise(got, expect, mag, tol=1e-5):
    """|got - expect| <= tol * mag for every entry, mag = the sum of the absolute values
    of the terms of that entry's sum."""
    got, expect, mag = (np.asarray(a, np.float64) for a in (got, expect, mag))
    assert got.shape == expect.shape == mag.shape, (got.shape, expect.shape, mag.shape)
    err = np.abs(got - expect)
    bad = err > tol * mag + 1e-30
    assert not bad.any(), "max err/mag = %g at %d of %d entries" % (
        (err / np.maximum(mag, 1e-300)).max(), int(bad.sum()), err.size)


def _leaky_basis_magnitude(diff, pdf, w, b):
    """Magnitude of the rounding error of one-layer leaky-ReLU basis values
    act(diff . w + b) / pdf: the slope carries the error of the pre-activation (sum of the
    absolute values of its terms), the value itself its own rounding."""
    z = diff.astype(np.float64) @ np.asarray(w, np.float64)[0] + np.asarray(b, np.float64).reshape(-1)
    mz = np.abs(diff).astype(np.float64) @ np.abs(np.asarray(w, np.float64)[0]) + \
        np.abs(np.asarray(b, np.float64).reshape(-1))
    slope = np.where(z > 0, 1.0, 0.2)
    return (slope * mz + np.abs(slope * z)) / np.asarray(pdf, np.float64).reshape(-1, 1)


def _setup(oracle, rng, n=3000, n_out=800, batch=2, radius=0.15):
    pts = rng.random((n, 3)).astype(np.float32)
    bids = np.sort(rng.integers(0, batch, n)).astype(np.int32)
    ctr = rng.random((n_out, 3)).astype(np.float32)
    cb = np.sort(rng.integers(0, batch, n_out)).astype(np.int32)
    g = oracle.Grid(pts, bids, batch, np.float32(radius))
    nbh = oracle.Neighborhood(g, np.float32(radius), ctr, cb)
    return pts, bids, ctr, cb, nbh


_T_ACT = {"relu": torch.relu, "leaky_relu": lambda x: torch.nn.functional.leaky_relu(x, 0.2),
          "elu": torch.nn.functional.elu}


@pytest.mark.parametrize("fused,gathered,transposed,fuse_final",
                         [(True, True, True, True), (True, True, True, False),
                          (True, True, False, False), (True, False, False, False),
                          (False, True, False, False), (False, False, False, False)])
@pytest.mark.parametrize("c_in,c_out,hidden,num_mlps,act",
                         [(8, 16, 16, 1, "relu"), (3, 8, 8, 1, "leaky_relu"),
                          (16, 32, 8, 4, "elu"), (64, 64, 16, 1, "leaky_relu"),
                          (32, 16, 8, 2, "relu"), (16, 8, 16, 1, "elu"),
                          (128, 32, 16, 1, "leaky_relu"), (3, 64, 16, 1, "relu"),
                          (64, 256, 16, 1, "leaky_relu"), (24, 40, 4, 4, "elu"),
                          (32, 32, 8, 4, "leaky_relu"), (16, 64, 8, 8, "relu"),
                          (64, 16, 32, 1, "elu"), (128, 24, 16, 2, "relu"),
                          # 8 basis columns: hidden units padded with zero columns to 16
                          (16, 16, 8, 1, "elu"), (32, 32, 4, 2, "leaky_relu"),
                          # 128 output channels: the transposed single-kernel layer of the
                          # backward is not covered, the layer has to take the two-kernel form
                          (16, 128, 16, 1, "relu"), (32, 128, 16, 1, "elu")])
def test_mcconv_forward_backward(oracle, c_in, c_out, hidden, num_mlps, act, fused, gathered,
                                 transposed, fuse_final):
    from tensorflow_graphics_point_clouds_amd import layers, pc, synthetic
    rng = np.random.default_rng(c_in + hidden)
    batch, radius = 2, 0.15
    pts, bids, ctr, cb, nbh = _setup(oracle, rng, batch=batch, radius=radius)
    feat = rng.standard_normal((len(pts), c_in)).astype(np.float32)
    w, b, wo = synthetic.mcconv_weights(rng, 3, c_in, c_out, hidden, num_mlps)
    b = (0.1 * rng.standard_normal(b.shape)).astype(np.float32)
    pdf = nbh.pdf_per_pair(0.2)
    expect, basis, proj = oracle.mc_conv_forward(feat, pts, ctr, nbh, pdf, w, b, wo,
                                                 np.float32(radius), act)

    conv = layers.MCConv(c_in, c_out, 3, num_mlps=num_mlps, mlp_size=[hidden],
                         non_linearity_type=act, weights=dev(w), biases=dev(b),
                         final_weights=dev(wo), fused=fused, gathered_grads=gathered,
                         transposed_grads=transposed, fuse_final=fuse_final)
    tfeat = dev(feat).requires_grad_(True)
    out = conv(tfeat, pc.PointCloud(dev(pts), dev(bids), batch),
               pc.PointCloud(dev(ctr), dev(cb), batch), radius, bandwidth=0.2)
    nb = conv.last_neighborhood
    assert np.array_equal(nb._neighbors.cpu().numpy(), nbh.neighbors)
    assert np.array_equal(nb._original_neigh_ids.cpu().numpy(), nbh.original_neigh_ids)
    np.testing.assert_allclose(nb.get_pdf().cpu().numpy(), pdf, rtol=1e-5)
    normwise(out.detach().cpu().numpy(), expect)

    up = rng.standard_normal(expect.shape).astype(np.float32)
    out.backward(dev(up))

    # float64 autograd of the same expression, neighbour lists and pdf held fixed
    ids = torch.tensor(nbh.original_neigh_ids).long()
    tw = torch.tensor(w.astype(np.float64), requires_grad=True)
    tb = torch.tensor(b.astype(np.float64), requires_grad=True)
    two = torch.tensor(wo.astype(np.float64), requires_grad=True)
    tf = torch.tensor(feat.astype(np.float64), requires_grad=True)
    radii = np.full(3, np.float32(radius), np.float32)
    diff = torch.tensor(((pts[ids[:, 0]] - ctr[ids[:, 1]]) / radii).astype(np.float64))
    hid = _T_ACT[act](torch.einsum("md,ldh->lmh", diff, tw) + tb)
    bas = hid.permute(1, 0, 2).reshape(len(ids), -1) / torch.tensor(pdf).reshape(-1, 1)
    per_pair = tf[ids[:, 0]][:, :, None] * bas[:, None, :]
    pj = torch.zeros(len(ctr), c_in, num_mlps * hidden, dtype=torch.float64).index_add(
        0, ids[:, 1], per_pair)
    pj = pj.reshape(-1, c_in, num_mlps, hidden).permute(2, 0, 1, 3).reshape(
        num_mlps, -1, c_in * hidden)
    ref = torch.bmm(pj, two).permute(1, 0, 2).reshape(len(ctr), -1)
    (ref * torch.tensor(up.astype(np.float64))).sum().backward()
    # Elementwise bound: every gradient is a sum of products; `mag` is the same sum over
    # the absolute values of its terms (the derivative of the activation enters as it is).
    with torch.no_grad():
        aup = torch.tensor(np.abs(up).astype(np.float64))
        abas, afeat = bas.abs(), tf.abs()
        n_out = len(ctr)

        def blocks(x):                                   # [n, C, L*H] -> [L, n, C*H]
            return x.reshape(-1, c_in, num_mlps, hidden).permute(2, 0, 1, 3).reshape(
                num_mlps, -1, c_in * hidden)

        apj = torch.zeros(n_out, c_in, num_mlps * hidden, dtype=torch.float64).index_add(
            0, ids[:, 1], afeat[ids[:, 0]][:, :, None] * abas[:, None, :])
        aup_l = aup.reshape(n_out, num_mlps, -1).permute(1, 0, 2)             # [L, n, G]
        mag_out = torch.bmm(blocks(apj), two.abs()).permute(1, 0, 2).reshape(n_out, -1)
        mag_final = torch.bmm(blocks(apj).transpose(1, 2), aup_l)
        adproj = torch.bmm(aup_l, two.abs().transpose(1, 2))                  # [L, n, C*H]
        adproj = adproj.reshape(num_mlps, n_out, c_in, hidden).permute(1, 2, 0, 3).reshape(
            n_out, c_in, num_mlps * hidden)
        mag_feat = torch.zeros_like(tf).index_add(
            0, ids[:, 0], torch.einsum("mck,mk->mc", adproj[ids[:, 1]], abas))
        mag_dbasis = torch.einsum("mck,mc->mk", adproj[ids[:, 1]], afeat[ids[:, 0]])
        z = (torch.einsum("md,ldh->lmh", diff, tw) + tb).permute(1, 0, 2).reshape(len(ids), -1)
        slope = {"relu": (z > 0).double(), "leaky_relu": torch.where(z > 0, 1.0, 0.2),
                 "elu": torch.where(z > 0, torch.ones_like(z), torch.exp(z))}[act]
        mag_dz = (mag_dbasis * slope / torch.tensor(pdf).reshape(-1, 1)).reshape(
            len(ids), num_mlps, hidden)
        mag_b = mag_dz.sum(0).reshape(num_mlps, 1, hidden)
        mag_w = torch.einsum("md,mlh->ldh", diff.abs(), mag_dz)
    elementwise(out.detach().cpu().numpy(), expect, mag_out.numpy())
    elementwise(tfeat.grad.cpu().numpy(), tf.grad.numpy(), mag_feat.numpy())
    elementwise(conv.final_weights.grad.cpu().numpy(), two.grad.numpy(), mag_final.numpy())
    elementwise(conv.weights.grad.cpu().numpy(), tw.grad.numpy(), mag_w.numpy())
    elementwise(conv.biases.grad.cpu().numpy(), tb.grad.numpy(), mag_b.numpy())


@pytest.mark.parametrize("hidden,act,fused", [(8, "relu", True), (8, "elu", False), (16, "elu", True),
                                              (32, "leaky_relu", True), (32, "leaky_relu", False)])
def test_pointconv_forward_backward(oracle, hidden, act, fused):
    """PointConv against the numpy expressions of point_conv_test.py:75-117 evaluated
    in float64 on the oracle's pairs and densities, gradients by float64 autograd."""
    from tensorflow_graphics_point_clouds_amd import layers, pc
    rng = np.random.default_rng(hidden)
    batch, radius, c_in, c_out = 2, 0.2, 8, 12
    pts, bids, ctr, cb, nbh = _setup(oracle, rng, n=1500, n_out=300, batch=batch, radius=radius)
    feat = rng.random((len(pts), c_in)).astype(np.float32)
    pdf = nbh.pdf_per_pair(0.2)
    ids = torch.tensor(nbh.original_neigh_ids).long()
    par = dict(weights=rng.standard_normal((3, hidden)) * 0.6,
               biases=rng.standard_normal((1, hidden)) * 0.1,
               final_weights=rng.standard_normal((hidden * c_in, c_out)) * 0.1,
               pw1=np.abs(rng.standard_normal((1, 16))) + 0.2, pw2=np.abs(rng.standard_normal((16, 1))) + 0.2,
               pb1=np.abs(rng.standard_normal((1, 16))) * 0.1, pb2=np.full((1, 1), 0.5))
    par = {k: v.astype(np.float32) for k, v in par.items()}
    conv = layers.PointConv(c_in, c_out, 3, size_hidden=hidden, non_linearity_type=act,
                            weights=par["weights"], biases=par["biases"],
                            final_weights=par["final_weights"],
                            pdf_weights=(par["pw1"], par["pw2"]), pdf_biases=(par["pb1"], par["pb2"]),
                            fused=fused)
    tfeat = dev(feat).requires_grad_(True)
    out = conv(tfeat, pc.PointCloud(dev(pts), dev(bids), batch),
               pc.PointCloud(dev(ctr), dev(cb), batch), radius, bandwidth=0.2)

    t = {k: torch.tensor(v.astype(np.float64), requires_grad=True) for k, v in par.items()}
    tf = torch.tensor(feat.astype(np.float64), requires_grad=True)
    diff = torch.tensor((pts[ids[:, 0]] - ctr[ids[:, 1]]).astype(np.float64))
    # the float64 restatement is oracle/layers_f64.point_conv, pinned on the CPU against the
    # per-centre loop of point_conv_test.py:75-117 (tests/test_oracle_float.py)
    from oracle import layers_f64
    tpdf = torch.tensor(pdf.astype(np.float64))
    ref, basis, cur, rel = layers_f64.point_conv(
        diff, ids, len(ctr), tf, tpdf, t["weights"], t["biases"], t["final_weights"],
        t["pw1"], t["pb1"], t["pw2"], t["pb2"], _T_ACT[act])
    hid = basis * cur
    up = rng.standard_normal(ref.shape).astype(np.float32)
    out.backward(dev(up))
    (ref * torch.tensor(up.astype(np.float64))).sum().backward()
    # Elementwise bound |err| <= 1e-5 * mag, mag = the same sum over the absolute values of
    # its terms (activation slopes and the density network's relu mask enter as they are).
    with torch.no_grad():
        n_out = len(ctr)
        aup = torch.tensor(np.abs(up).astype(np.float64))
        abas, afeat, afw = basis.abs(), tf.abs(), t["final_weights"].abs()
        apj = torch.zeros(n_out, c_in, hidden, dtype=torch.float64).index_add(
            0, ids[:, 1], afeat[ids[:, 0]][:, :, None] * abas[:, None, :]).reshape(n_out, -1)
        mag_out = apj @ afw
        mag_final = apj.T @ aup
        adproj = (aup @ afw.T).reshape(n_out, c_in, hidden)
        mag_feat = torch.zeros_like(tf).index_add(
            0, ids[:, 0], torch.einsum("mck,mk->mc", adproj[ids[:, 1]], abas))
        mag_dbasis = torch.einsum("mck,mc->mk", adproj[ids[:, 1]], afeat[ids[:, 0]])
        z = diff @ t["weights"] + t["biases"]
        slope = {"relu": (z > 0).double(), "leaky_relu": torch.where(z > 0, 1.0, 0.2),
                 "elu": torch.where(z > 0, torch.ones_like(z), torch.exp(z))}[act]
        mag_dz = mag_dbasis * slope / cur.abs()
        mag_b = mag_dz.sum(0, keepdim=True)
        mag_w = diff.abs().T @ mag_dz
        mag_dcur = (mag_dbasis * hid.abs()).sum(1, keepdim=True) / cur ** 2          # [M, 1]
        pre = rel @ t["pw1"] + t["pb1"]
        h1, on = torch.relu(pre), (pre > 0).double()
        mag_pb2 = mag_dcur.sum(0, keepdim=True)
        mag_pw2 = h1.T @ mag_dcur
        mag_pb1 = (mag_dcur * on * t["pw2"].abs().T).sum(0, keepdim=True)
        mag_pw1 = (mag_dcur * on * t["pw2"].abs().T * rel).sum(0, keepdim=True)
    elementwise(out.detach().cpu().numpy(), ref.detach().numpy(), mag_out.numpy())
    elementwise(tfeat.grad.cpu().numpy(), tf.grad.numpy(), mag_feat.numpy())
    elementwise(conv.final_weights.grad.cpu().numpy(), t["final_weights"].grad.numpy(),
                mag_final.numpy())
    elementwise(conv.weights.grad.cpu().numpy(), t["weights"].grad.numpy(), mag_w.numpy())
    elementwise(conv.biases.grad.cpu().numpy(), t["biases"].grad.numpy(), mag_b.numpy())
    elementwise(conv.pdf_weights_1.grad.cpu().numpy(), t["pw1"].grad.numpy(), mag_pw1.numpy())
    elementwise(conv.pdf_weights_2.grad.cpu().numpy(), t["pw2"].grad.numpy(), mag_pw2.numpy())
    elementwise(conv.pdf_biases_1.grad.cpu().numpy(), t["pb1"].grad.numpy(), mag_pb1.numpy())
    elementwise(conv.pdf_biases_2.grad.cpu().numpy(), t["pb2"].grad.numpy(), mag_pb2.numpy())


@pytest.mark.parametrize("column", [0, 1])
def test_pointconv_density_transform_and_parameter_gradients(column):
    """The per-pair density transform of PointConv (PointConv.py:176-190) and the
    gradients of its 49 parameters against float64 torch autograd, for a pair table
    read in either orientation; two slabs of scale gradients."""
    from tensorflow_graphics_point_clouds_amd import _lib
    from tensorflow_graphics_point_clouds_amd._lib import cint, csize, i64, ptr, stream
    gen = torch.Generator(device="cuda").manual_seed(column)
    m, n_pts, n_ctr = 70001, 900, 400
    pairs = torch.stack((torch.randint(0, n_pts, (m,), device="cuda", generator=gen),
                         torch.randint(0, n_ctr, (m,), device="cuda", generator=gen)), 1).int()
    if column == 1:
        pairs = pairs.flip(1).contiguous()
    pdf = torch.rand(n_pts, device="cuda", generator=gen) + 0.1
    mx = torch.rand(n_ctr, device="cuda", generator=gen) + 1.0
    par = [torch.randn(s, device="cuda", generator=gen) for s in (16, 16, 16, 1)]
    par[3] += 3.0
    y = torch.empty(m, device="cuda")
    _lib.call("pointconv_density", stream(), i64(m), ptr(pairs), cint(column), ptr(pdf), ptr(mx),
              ptr(par[0]), ptr(par[1]), ptr(par[2]), ptr(par[3]), ptr(y))
    ref = [p.double().cpu().requires_grad_(True) for p in par]
    pt, ctr = pairs[:, column].long().cpu(), pairs[:, 1 - column].long().cpu()
    rel = (pdf.double().cpu()[pt] / mx.double().cpu()[ctr]).reshape(-1, 1)
    yr = torch.relu(rel * ref[0] + ref[1]) @ ref[2] + ref[3]
    normwise(y.cpu().numpy(), yr.detach().numpy(), tol=1e-5)
    # gradient of sum_m t[m] / y[m] for two slabs of scale gradients t
    t = torch.randn((2, m), device="cuda", generator=gen)
    L = _lib.lib()
    ws = _lib.workspace(L.mccnn_pointconv_density_grads_workspace_bytes(i64(m)), y.device)
    grads = torch.empty(49, device="cuda")
    _lib.call("pointconv_density_grads", stream(), i64(m), ptr(pairs), cint(column), ptr(pdf),
              ptr(mx), ptr(par[0]), ptr(par[1]), ptr(par[2]), ptr(par[3]), ptr(y), cint(2),
              ptr(t), ptr(ws), csize(ws.numel()), ptr(grads))
    (t.double().cpu().sum(0) / yr).sum().backward()
    expect = torch.cat([r.grad.reshape(-1) for r in ref]).numpy()
    scale = torch.cat([(t.double().cpu().sum(0).abs() / yr.detach() ** 2).sum().reshape(1)] * 49)
    assert np.abs(grads.cpu().numpy() - expect).max() <= 1e-5 * float(scale[0])
    with pytest.raises(ValueError):
        _lib.call("pointconv_density", stream(), i64(m), ptr(pairs), cint(2), ptr(pdf), ptr(mx),
                  ptr(par[0]), ptr(par[1]), ptr(par[2]), ptr(par[3]), ptr(y))


@pytest.mark.parametrize("c_in,c_out,transposed,kpn", [(16, 24, True, 15), (16, 24, False, 15),
                                                       (64, 32, True, 15), (8, 16, True, 15),
                                                       (16, 16, True, 5), (32, 8, True, 18),
                                                       (16, 8, False, 18), (8, 8, True, 7)])
@pytest.mark.parametrize("kind,influence", [("linear", None), ("gaussian", 0.3 * 0.15)])
def test_kpconv_forward_backward(oracle, kind, influence, c_in, c_out, transposed, kpn):
    """Rigid kernel-point convolution for the reference's kernel sizes (5 and 7 points
    padded to 16 basis columns, 15 to 16, 18 to 32; KPConv.py:199-213)."""
    from tensorflow_graphics_point_clouds_amd import layers, pc, synthetic
    rng = np.random.default_rng(5)
    batch, radius = 2, 0.15
    pts, bids, ctr, cb, nbh = _setup(oracle, rng, batch=batch, radius=radius)
    feat = rng.standard_normal((len(pts), c_in)).astype(np.float32)
    kp = synthetic.spherical_kernel_points(kpn, rotate=False) * 0.8     # * 0.75 inside the layer = 0.6
    if kpn == 13:
        kp = kp / 1.902
    wts = (rng.standard_normal((kpn * c_in, c_out)) * 0.1).astype(np.float32)
    sigma = 1.0 if influence is None else influence / radius
    ids = nbh.original_neigh_ids
    radii = np.full(3, np.float32(radius), np.float32)
    diff = (pts[ids[:, 0]] - ctr[ids[:, 1]]) / radii
    basis, _ = oracle.kp_basis(diff, kp.astype(np.float64) * 0.75, sigma, kind)
    kpad = 16 if kpn <= 16 else 32
    padded = np.zeros((len(ids), kpad), np.float32)
    padded[:, :kpn] = basis
    proj = oracle.basis_proj(padded, feat, ids, nbh.ranges)[:, :, :kpn]
    expect = proj.reshape(len(ctr), -1) @ wts.astype(np.float64)

    conv = layers.KPConv(c_in, c_out, custom_kernel_points=kp, kp_interpolation=kind,
                         weights=dev(wts),
                         transposed_grads=transposed)
    tfeat = dev(feat).requires_grad_(True)
    out = conv(tfeat, pc.PointCloud(dev(pts), dev(bids), batch),
               pc.PointCloud(dev(ctr), dev(cb), batch), radius, kernel_influence_dist=influence)
    w64, up = wts.astype(np.float64), rng.standard_normal(expect.shape).astype(np.float32)
    _, pmag = oracle.basis_proj(padded, np.abs(feat), ids, nbh.ranges, with_magnitude=True)
    pmag = pmag[:, :, :kpn].reshape(len(ctr), -1)
    elementwise(out.detach().cpu().numpy(), expect, pmag @ np.abs(w64),
                tol=1e-5 if kind == "linear" else 2e-5)       # (see below)
    out.backward(dev(up))
    up64 = up.astype(np.float64)
    dpad = np.zeros((len(ctr), c_in, kpad), np.float32)
    dmag = np.zeros((len(ctr), c_in, kpad), np.float32)
    dpad[:, :, :kpn] = (up64 @ w64.T).reshape(len(ctr), c_in, kpn)
    dmag[:, :, :kpn] = (np.abs(up64) @ np.abs(w64).T).reshape(len(ctr), c_in, kpn)
    _, dfeat = oracle.basis_proj_grads(padded, feat, ids, nbh.ranges, dpad)
    _, fmag = oracle.basis_proj_grads(padded, feat, ids, nbh.ranges, dmag)
    # (the oracle takes the upstream gradient rounded to float32: 2^-24 of the magnitude)
    # The Gaussian with sigma = 0.3 falls off as exp(-(d / 0.1)^2): one unit in the last
    # place of a scaled offset (the kernels multiply by 1/r, the reference divides by r)
    # changes a weight at d = 0.5 by 2 * 5 * 6e-8 / 0.1 = 6e-6 of its value, which the
    # bound has to leave room for; the linear correlation is held to 1e-5.
    tol = 1e-5 if kind == "linear" else 2e-5
    elementwise(tfeat.grad.cpu().numpy(), dfeat, fmag, tol=tol + 1e-7)
    elementwise(conv.weights.grad.cpu().numpy(), proj.reshape(len(ctr), -1).T @ up64,
                pmag.T @ np.abs(up64), tol=tol)


@pytest.mark.parametrize("c_in,c_out", [(16, 8), (8, 16), (32, 32), (16, 16), (8, 32), (8, 8),
                                        (32, 64), (64, 16), (64, 64)])
@pytest.mark.parametrize("kind", ["linear", "gaussian"])
def test_deformable_kpconv_and_regularization(oracle, kind, c_in, c_out):
    """Deformable kernel points (offsets predicted by a rigid convolution) and the
    regularisation loss, forward and backward, against float64 autograd of the
    expressions of KPConv.py:165-232, 317-429 on the oracle's neighbour pairs; foreign
    centres; 16 and 32 input channels take the kernels with the weights in registers, 8
    the materialising ops.  Offsets and output elementwise at 1e-5 of the sum of the
    absolute values of their terms, the reference evaluated at the layer's own offsets;
    normwise 1e-5 for the gradients (non-smooth points of the correlation and of the
    fitting minimum are handled as the helper describes)."""
    from tensorflow_graphics_point_clouds_amd import synthetic
    from tests.deformable_reference import check_deformable_kpconv
    rng = np.random.default_rng(17)
    batch, radius, kpn = 2, 0.2, 15
    pts, bids, ctr, cb, nbh = _setup(oracle, rng, n=1500, n_out=400, batch=batch, radius=radius)
    feat = rng.standard_normal((len(pts), c_in)).astype(np.float32)
    kp = synthetic.spherical_kernel_points(15, rotate=False) * 0.8
    wts = (rng.standard_normal((kpn * c_in, c_out)) * 0.1).astype(np.float32)
    # offsets of about N(0, 0.02): enough to separate the layout's two coincident pairs
    woff = (rng.standard_normal((kpn * c_in, kpn * 3)) * 2.0 / c_in).astype(np.float32)
    check_deformable_kpconv(pts, bids, ctr, cb, batch, nbh.original_neigh_ids, radius, feat, kp,
                            wts, woff, 0.5 * radius, kind)


@pytest.mark.parametrize("kpn", [5, 15, 16, 20])
@pytest.mark.parametrize("dims", [2, 3])
@pytest.mark.parametrize("kind", [0, 1])
def test_kp_regularization_terms(oracle, kpn, dims, kind):
    """The per-(centre, kernel point) terms of the regularisation loss (KPConv.py:394-429) as
    the op returns them -- fitting distance, the pair that attains it, repulsion -- against a
    float64 evaluation on the oracle's pairs; up to 16 kernel points take the kernel with a
    quarter of a wavefront per centre, more the one with a thread per term.  Centres without
    pairs report 0 and -1."""
    from tensorflow_graphics_point_clouds_amd import _lib
    from tensorflow_graphics_point_clouds_amd._lib import cfloat, cint, i64, ptr, stream
    rng = np.random.default_rng(100 * kpn + 10 * dims + kind)
    n, n_out, batch, radius, sigma = 1500, 420, 2, 0.2, 0.45
    pts = rng.random((n, dims)).astype(np.float32)
    bids = np.sort(rng.integers(0, batch, n)).astype(np.int32)
    ctr = (rng.random((n_out, dims)) * 2.0 - 0.5).astype(np.float32)    # some far from every point
    cb = np.sort(rng.integers(0, batch, n_out)).astype(np.int32)
    g = oracle.Grid(pts, bids, batch, np.float32(radius))
    nbh = oracle.Neighborhood(g, np.float32(radius), ctr, cb)
    ids, ranges = nbh.original_neigh_ids, nbh.ranges
    counts = np.diff(np.concatenate([[0], ranges]))
    assert (counts == 0).any() and counts.max() > 16
    kp = (rng.standard_normal((kpn, dims)) * 0.5).astype(np.float32)
    off = (rng.standard_normal((n_out, kpn, dims)) * 0.05).astype(np.float32)
    inv_r = np.full(dims, 1 / np.float32(radius), np.float32)
    fit = torch.empty((n_out, kpn), dtype=torch.float32, device="cuda")
    rep = torch.empty_like(fit)
    argmin = torch.empty((n_out, kpn), dtype=torch.int32, device="cuda")
    # the device copies stay referenced until the results have been read back
    t_pts, t_ctr, t_ids, t_ranges = dev(pts), dev(ctr), dev(ids), dev(ranges)
    t_inv_r, t_kp, t_off = dev(inv_r), dev(kp), dev(off)
    assert t_ids.dtype == torch.int32 and t_ranges.dtype == torch.int32
    assert t_ids.shape == (int(ranges[-1]), 2) and int(ids[:, 0].max()) < n
    _lib.call("kp_regularization", stream(), i64(len(ids)), cint(dims), cint(kpn), cint(kind),
              cfloat(sigma), ptr(t_pts), ptr(t_ctr), ptr(t_ids), i64(n_out), ptr(t_ranges),
              ptr(t_inv_r), ptr(t_kp), ptr(t_off), ptr(fit), ptr(argmin), ptr(rep))
    fit, rep, argmin = fit.cpu().numpy(), rep.cpu().numpy(), argmin.cpu().numpy()
    del t_pts, t_ctr, t_ids, t_ranges, t_inv_r, t_kp, t_off
    moved = kp.astype(np.float64)[None] + off.astype(np.float64)            # [n_out, kpn, dims]
    delta = (pts.astype(np.float64)[ids[:, 0]] - ctr.astype(np.float64)[ids[:, 1]]) * inv_r
    sq = ((delta[:, None, :] - moved[ids[:, 1]]) ** 2).sum(-1)              # [M, kpn]
    start = 0
    for c, end in enumerate(ranges):
        if end == start:
            assert (fit[c] == 0).all() and (argmin[c] == -1).all()
            continue
        seg = sq[start:end]
        best = seg.min(0)
        # differences of coordinates of order 1 are squared: absolute float32 error ~1e-7
        np.testing.assert_allclose(fit[c], best / sigma ** 2, rtol=1e-5, atol=2e-6)
        assert ((argmin[c] >= start) & (argmin[c] < end)).all()
        # the reported pair attains the minimum (ties and near-ties: to float32 accuracy)
        np.testing.assert_allclose(sq[argmin[c], np.arange(kpn)], best, rtol=1e-5, atol=1e-6)
        start = end
    dist = np.sqrt(((moved[:, :, None, :] - moved[:, None, :, :]) ** 2).sum(-1))
    wgt = np.maximum(1 - dist / sigma, 0) if kind == 0 else np.exp(-(dist / (sigma / 3)) ** 2)
    wgt[:, np.arange(kpn), np.arange(kpn)] = 0
    np.testing.assert_allclose(rep, wgt.sum(-1), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("c", [1, 4, 5, 16, 64, 100, 128, 256])
def test_local_and_global_pooling(oracle, c):
    from tensorflow_graphics_point_clouds_amd import layers, pc
    rng = np.random.default_rng(c)
    batch = 3
    pts, bids, ctr, cb, nbh = _setup(oracle, rng, batch=batch, radius=0.08, n_out=600)
    feat = rng.standard_normal((len(pts), c)).astype(np.float32)
    ids = nbh.original_neigh_ids
    cin = pc.PointCloud(dev(pts), dev(bids), batch)
    cout = pc.PointCloud(dev(ctr), dev(cb), batch)
    for layer, kind in ((layers.MaxPooling(), "max"), (layers.AveragePooling(), "avg")):
        t = dev(feat).requires_grad_(True)
        out = layer(t, cin, cout, 0.08)
        expect = oracle.local_pool(feat, ids, len(ctr), kind)
        if kind == "max":
            assert np.array_equal(out.detach().cpu().numpy(), expect.astype(np.float32))
        else:
            np.testing.assert_allclose(out.detach().cpu().numpy(), expect, rtol=1e-5, atol=1e-6)
        up = rng.standard_normal(expect.shape).astype(np.float32)
        out.backward(dev(up))
        tf = torch.tensor(feat.astype(np.float64), requires_grad=True)
        gathered = tf[torch.tensor(ids[:, 0]).long()]
        seg = torch.tensor(ids[:, 1]).long()
        if kind == "max":
            ref = torch.full((len(ctr), c), float(np.finfo(np.float32).min), dtype=torch.float64)
            ref = ref.scatter_reduce(0, seg[:, None].expand(-1, c), gathered, "amax")
        else:
            ref = torch.zeros((len(ctr), c), dtype=torch.float64).index_add(0, seg, gathered)
            cnt = torch.bincount(seg, minlength=len(ctr)).clamp(min=1)
            ref = ref / cnt[:, None]
        (ref * torch.tensor(up.astype(np.float64))).sum().backward()
        normwise(t.grad.cpu().numpy(), tf.grad.numpy())
    for layer, kind in ((layers.GlobalMaxPooling(), "max"), (layers.GlobalAveragePooling(), "avg")):
        t = dev(feat).requires_grad_(True)
        out = layer(t, cin)
        expect = oracle.global_pool(feat, bids, batch, kind)
        np.testing.assert_allclose(out.detach().cpu().numpy(), expect, rtol=1e-5, atol=1e-6)
        up = rng.standard_normal(expect.shape).astype(np.float32)
        out.backward(dev(up))
        if kind == "avg":
            cnt = np.bincount(bids, minlength=batch)
            gexp = up[bids] / cnt[bids][:, None]
        else:
            gexp = np.where(feat == expect.astype(np.float32)[bids], up[bids], 0.0)
        normwise(t.grad.cpu().numpy(), gexp)


def _wide_range(shape, gen):
    """Standard-normal values times 10^U(-3, 3): operands whose magnitudes span six decades,
    so that an operand split that loses low-order bits of small entries would show."""
    return torch.randn(shape, device="cuda", generator=gen) * \
        10.0 ** (6.0 * torch.rand(shape, device="cuda", generator=gen) - 3.0)


@pytest.fixture(params=[True, False], ids=["split-bf16", "fp32-mfma"])
def dense_mode(request):
    """Runs a test once with the dense products on the bf16 matrix pipe (three-way operand
    splits, the default) and once with the float32 matrix instructions."""
    from tensorflow_graphics_point_clouds_amd import _lib
    before = _lib.lib().mccnn_set_split_products(1 if request.param else 0)
    yield request.param
    _lib.lib().mccnn_set_split_products(before)


@pytest.mark.parametrize("n,c,r", [(1, 16, 256), (4099, 64, 1024), (20000, 128, 512),
                                   (777, 32, 2048), (0, 64, 256), (100003, 64, 1024),
                                   (50001, 128, 2048), (33, 128, 128), (257, 32, 256)])
def test_weight_grad_product_matches_float64(n, c, r, dense_mode):
    """x^T y with the long reduction over the points, elementwise against float64:
    |got - expect| <= 1e-5 * (|x|^T |y|), on operands whose magnitudes span six decades;
    equal bits on a second call (the partial sums are added in a fixed order)."""
    from tensorflow_graphics_point_clouds_amd import layers
    gen = torch.Generator(device="cuda").manual_seed(n + c)
    x = _wide_range((n, c), gen)
    y = _wide_range((n, r), gen)
    got = layers._weight_grad_product(x, y)
    assert got.shape == (c, r)
    assert torch.equal(got, layers._weight_grad_product(x, y))
    expect = x.double().t() @ y.double()
    mag = x.double().abs().t() @ y.double().abs()
    err = (got.double() - expect).abs()
    assert bool((err <= 1e-5 * mag).all()), float((err / mag.clamp(min=1e-300)).max())


@pytest.mark.parametrize("n,f,r", [(1, 16, 256), (4099, 64, 1024), (20000, 32, 512), (0, 64, 256),
                                   (4099, 128, 1024), (3001, 128, 2048), (1500, 256, 4096),
                                   (17, 256, 64), (33, 128, 128), (31, 64, 256), (70001, 64, 1024),
                                   (5000, 32, 1024), (65, 128, 256), (70001, 128, 2048),
                                   (2081, 128, 384)])
def test_projection_grad_product_matches_float64(n, f, r, dense_mode):
    """x w^T elementwise against float64: |got - expect| <= 1e-5 * (|x| |w|^T), on operands
    whose magnitudes span six decades; equal bits on a second call."""
    from tensorflow_graphics_point_clouds_amd import layers
    gen = torch.Generator(device="cuda").manual_seed(n + f)
    x = _wide_range((n, f), gen)
    w = _wide_range((r, f), gen)
    got = layers._projection_grad_product(x, w)
    assert got.shape == (n, r)
    assert torch.equal(got, layers._projection_grad_product(x, w))
    expect = x.double() @ w.double().t()
    mag = x.double().abs() @ w.double().abs().t()
    err = (got.double() - expect).abs()
    assert bool((err <= 1e-5 * mag).all()), float((err / mag).max()) if n else 0.0
    if n:       # the split path is as accurate as float32 accumulation, far inside the bound
        assert float((err / mag).max()) <= 2e-6


@pytest.mark.parametrize("n,r,f", [(1, 256, 16), (15, 256, 128), (4099, 1024, 64), (20000, 512, 128),
                                   (333, 1024, 32), (5000, 512, 32), (0, 1024, 64), (70001, 1024, 16),
                                   (4099, 2048, 128), (3001, 1024, 128), (1500, 4096, 256),
                                   (777, 2048, 48), (2000, 768, 192), (9000, 2048, 64),
                                   (33000, 1024, 128), (66100, 2048, 64)])
def test_final_product_matches_float64(n, r, f):
    """x w with a block of w in the registers of each block of wavefronts (the blocks of a
    larger w walked inside one launch, later row blocks adding to the earlier ones; the last
    two shapes are large enough for the tiled product on w as it is),
    elementwise against float64 with the magnitude sum |x| |w| (1e-5), row permutation
    included; a second call must return the same bits."""
    from tensorflow_graphics_point_clouds_amd import _lib
    from tensorflow_graphics_point_clouds_amd._lib import cint, i64, ptr, stream
    assert _lib.lib().mccnn_final_product_supported(r, f) == 1
    assert _lib.lib().mccnn_final_product_supported(2048 + 128, 64) == 0
    assert _lib.lib().mccnn_final_product_supported(1024, 24) == 0
    gen = torch.Generator(device="cuda").manual_seed(n + f)
    x = torch.randn((n, r), device="cuda", generator=gen)
    w = torch.randn((r, f), device="cuda", generator=gen)
    rows = torch.randperm(n, device="cuda", generator=gen).int()
    outs = []
    for perm in (None, rows, rows):
        out = torch.full((n, f), float("nan"), device="cuda")
        _lib.call("final_product", stream(), i64(n), cint(r), ptr(x), cint(f), ptr(w), ptr(perm),
                  ptr(out))
        outs.append(out)
    expect = x.double() @ w.double()
    mag = x.double().abs() @ w.double().abs()
    assert bool(((outs[0].double() - expect).abs() <= 1e-5 * mag).all())
    assert torch.equal(outs[1], outs[2])
    if n:
        assert torch.equal(outs[1][rows.long()], outs[0])
    with pytest.raises(ValueError):
        _lib.call("final_product", stream(), i64(n), cint(2048 + 128), ptr(x), cint(64), ptr(w),
                  ptr(None), ptr(outs[0]))


@pytest.mark.parametrize("n,r,f", [(40001, 2048, 128), (70000, 1024, 64), (33000, 512, 192),
                                   (129, 64, 64), (1, 32, 128), (0, 2048, 128),
                                   (131101, 512, 128), (66003, 256, 256)])
def test_final_product_with_transposed_weights_matches_float64(n, r, f):
    """The tiled product on wt [F, R] (128 x 128 and 256 x 64 tiles, 256 x 128 once those fill
    the device twice over -- the last two shapes --, partial last tiles, row
    permutation), elementwise against float64 with the magnitude sum |x| |w| (1e-5); equal
    bits on a second call; and the layer-level product, which picks the tiles for the large
    shapes, against the same reference."""
    from tensorflow_graphics_point_clouds_amd import _lib, layers
    from tensorflow_graphics_point_clouds_amd._lib import cint, i64, ptr, stream
    assert _lib.lib().mccnn_final_product_wt_supported(r, f) == 1
    assert _lib.lib().mccnn_final_product_wt_supported(r, 48) == 0
    gen = torch.Generator(device="cuda").manual_seed(n + f)
    x = torch.randn((n, r), device="cuda", generator=gen)
    w = torch.randn((r, f), device="cuda", generator=gen)
    wt = w.t().contiguous()
    rows = torch.randperm(n, device="cuda", generator=gen).int()
    outs = []
    for perm in (None, rows, rows):
        out = torch.full((n, f), float("nan"), device="cuda")
        _lib.call("final_product_wt", stream(), i64(n), cint(r), ptr(x), cint(f), ptr(wt),
                  ptr(perm), ptr(out))
        outs.append(out)
    expect = x.double() @ w.double()
    mag = x.double().abs() @ w.double().abs()
    assert bool(((outs[0].double() - expect).abs() <= 1e-5 * mag).all())
    assert torch.equal(outs[1], outs[2])
    if n:
        assert torch.equal(outs[1][rows.long()], outs[0])
    got = layers._final_product(x, w)
    assert bool(((got.double() - expect).abs() <= 1e-5 * mag).all())


def test_layers_accept_padded_input_and_return_padded_output():
    """Padded point clouds / features ([A, V, D], [A, V, C], sizes) give the same
    result as the segmented form, re-padded on request (layers/utils.py:22-49,
    pc/utils.py:75-94)."""
    from tensorflow_graphics_point_clouds_amd import layers, pc
    rng = np.random.default_rng(11)
    sizes, v, c = [700, 400, 900], 900, 16
    pts = rng.random((3, v, 3)).astype(np.float32)
    feat = rng.standard_normal((3, v, c)).astype(np.float32)
    padded = pc.PointCloud(dev(pts), sizes=sizes)
    flat_pts = np.concatenate([pts[b, :n] for b, n in enumerate(sizes)])
    flat_feat = np.concatenate([feat[b, :n] for b, n in enumerate(sizes)])
    bids = np.repeat(np.arange(3), sizes).astype(np.int32)
    flat = pc.PointCloud(dev(flat_pts), dev(bids), 3)
    conv = layers.MCConv(c, 16, 3, num_mlps=1, mlp_size=[16], seed=4)
    a = conv(dev(feat), padded, padded, 0.2, return_padded=True).detach()
    b = conv(dev(flat_feat), flat, flat, 0.2)
    assert a.shape == (3, v, 16)
    for i, n in enumerate(sizes):
        start = sum(sizes[:i])
        assert torch.equal(a[i, :n], b[start:start + n])
        assert float(a[i, n:].abs().sum()) == 0.0
    pool = layers.MaxPooling()(dev(feat), padded, padded, 0.2, return_sorted=True)
    assert torch.equal(pool, layers.MaxPooling()(dev(flat_feat), flat, flat, 0.2))


def test_three_level_mcconv_network_matches_oracle(oracle):
    """The ModelNet-shaped configuration (cell-average hierarchy at three radii, one
    Monte-Carlo convolution per level, 3 -> 64 -> 128 -> 256 features with the point
    coordinates as input features): every level's output against the oracle's
    float64 chain on the oracle's own hierarchy."""
    from tensorflow_graphics_point_clouds_amd import layers, pc, synthetic
    cfg = synthetic.config2(batch=4, points_per_cloud=512)
    rng = np.random.default_rng(2)
    pts, bids, batch = cfg["points"], cfg["batch_ids"], cfg["batch_size"]
    hier = pc.PointHierarchy(pc.PointCloud(dev(pts), dev(bids), batch), cfg["radii"],
                             "cell average")
    widths = [3, 64, 128, 256]
    feat_ref = pts.astype(np.float64)
    feat = dev(pts)
    cur_pts, cur_bids = pts, bids
    for level, r in enumerate(cfg["radii"]):
        conv_r = np.float32(1.5 * r)
        g = oracle.Grid(cur_pts, cur_bids, batch, np.float32(r))
        nbh = oracle.Neighborhood(g, np.float32(r))
        nxt_pts, nxt_bids, _ = oracle.sampling(g.sorted_points, g.sorted_batch_ids, g.sorted_keys,
                                               g.num_cells, nbh.neighbors, nbh.ranges, 1)
        cg = oracle.Grid(cur_pts, cur_bids, batch, conv_r)
        cn = oracle.Neighborhood(cg, conv_r, nxt_pts, nxt_bids)
        pdf = cn.pdf_per_pair(0.2)
        w, b, wo = synthetic.mcconv_weights(rng, 3, widths[level], widths[level + 1], 16, 1)
        expect, _, _ = oracle.mc_conv_forward(feat_ref.astype(np.float32), cur_pts, nxt_pts, cn,
                                              pdf, w, b, wo, conv_r, "leaky_relu")
        conv = layers.MCConv(widths[level], widths[level + 1], 3, num_mlps=1, mlp_size=[16],
                             non_linearity_type="leaky_relu", weights=dev(w), biases=dev(b),
                             final_weights=dev(wo))
        out = conv(feat, hier[level], hier[level + 1], float(conv_r), bandwidth=0.2)
        assert np.array_equal(hier[level + 1]._points.cpu().numpy(), nxt_pts)
        normwise(out.detach().cpu().numpy(), expect, tol=1e-5)
        # elementwise, against the sum of the absolute values of every entry's terms
        ids = cn.original_neigh_ids
        diff = (cur_pts[ids[:, 0]] - nxt_pts[ids[:, 1]]) / conv_r
        bmag = _leaky_basis_magnitude(diff, pdf, w, b)
        pmag = oracle.basis_proj(bmag.astype(np.float32), np.abs(feat_ref).astype(np.float32), ids,
                                 cn.ranges)
        elementwise(out.detach().cpu().numpy(), expect,
                    pmag.reshape(len(nxt_pts), -1) @ np.abs(wo[0].astype(np.float64)))
        # feed the oracle's (float32-rounded) result to both sides of the next level
        feat_ref = np.maximum(expect, 0.0)
        feat = dev(feat_ref.astype(np.float32))
        cur_pts, cur_bids = nxt_pts, nxt_bids


@pytest.mark.parametrize("d,c,n_out,radius", [(3, 64, 803, 0.3), (2, 32, 517, 0.12), (3, 128, 99, 0.35),
                                              (3, 16, 5, 0.3)])
def test_projection_runs_with_empty_and_crowded_centres(oracle, d, c, n_out, radius):
    """The projection kernel walks runs of 8 consecutive centres in chunks of 64
    pairs: centre counts that are no multiple of 8, neighbourhoods of several
    chunks, empty centres (a whole empty run first, single ones in between, the
    last centres), two channel chunks (C = 128) and D = 2, with and without row
    indirection, against the oracle's basis and projection."""
    from tensorflow_graphics_point_clouds_amd import layers
    rng = np.random.default_rng(d * 100 + c)
    n, batch = 3000, 2
    pts = rng.random((n, d)).astype(np.float32)
    bids = np.sort(rng.integers(0, batch, n)).astype(np.int32)
    ctr = rng.random((n_out, d)).astype(np.float32)
    cb = np.sort(rng.integers(0, batch, n_out)).astype(np.int32)
    far = np.zeros(n_out, bool)
    far[:min(9, n_out - 2)] = True
    far[-2:] = True
    far[rng.random(n_out) < 0.2] = True
    far[n_out // 2] = False
    ctr[far] += 5.0                                        # no neighbours out there
    g = oracle.Grid(pts, bids, batch, np.float32(radius))
    nbh = oracle.Neighborhood(g, np.float32(radius), ctr, cb)
    counts = np.diff(np.concatenate([[0], nbh.ranges]))
    assert counts[far].max() == 0 and (counts.max() > 64 or d == 2)
    pdf = (0.5 + rng.random(len(nbh.neighbors))).astype(np.float32)
    w = (rng.standard_normal((1, d, 16)) * 0.7).astype(np.float32)
    b = (rng.standard_normal((1, 1, 16)) * 0.1).astype(np.float32)
    feat = rng.standard_normal((n, c)).astype(np.float32)
    ids = nbh.original_neigh_ids
    diff = (pts[ids[:, 0]] - ctr[ids[:, 1]]) / np.float32(radius)
    basis = oracle.mc_basis(diff, pdf, w, b, "leaky_relu")
    expect = oracle.basis_proj(basis.astype(np.float32), feat, ids, nbh.ranges)
    inv = dev(np.full(d, 1.0 / np.float32(radius), np.float32))
    args = (dev(w), dev(b.reshape(-1)), dev(feat), dev(pts), dev(ctr), dev(ids), dev(nbh.ranges), inv,
            dev(pdf), 1)
    out = layers._mc_project(*args)
    normwise(out.cpu().numpy(), expect)
    bmag = _leaky_basis_magnitude(diff, pdf, w, b)
    elementwise(out.cpu().numpy(), expect,
                oracle.basis_proj(bmag.astype(np.float32), np.abs(feat), ids, nbh.ranges))
    assert float(out[dev(far)].abs().max()) == 0.0
    rows = rng.permutation(n_out).astype(np.int32)
    moved = layers._mc_project(*args, out_rows=dev(rows))
    assert torch.equal(moved[dev(rows).long()], out)


def test_mcconv_layer_at_full_scene_size():
    """The benchmark configuration at its real size (8 clouds, 763 k points, 28 M
    pairs, 64 -> 64 channels): rows of the output and of the feature gradient at
    sampled points against float64 on the layer's own pair table and densities (whose
    integer parity is pinned elsewhere), every entry within 1e-5 of the sum of the
    absolute values of its terms, and two properties over
    the whole tensors: linearity in the features and <up, conv(x)> == <dfeat, x>."""
    from tensorflow_graphics_point_clouds_amd import layers, pc, synthetic
    cfg = synthetic.config3()
    cloud = pc.PointCloud(dev(cfg["points"]), dev(cfg["batch_ids"]), cfg["batch_size"])
    radius, c = cfg["radius"], 64
    n = cloud._points.shape[0]
    conv = layers.MCConv(c, c, 3, num_mlps=1, mlp_size=[16], non_linearity_type="leaky_relu", seed=3)
    gen = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn((n, c), device="cuda", generator=gen).requires_grad_(True)
    y = torch.randn((n, c), device="cuda", generator=gen)
    up = torch.randn((n, c), device="cuda", generator=gen)
    out = conv(x, cloud, cloud, radius, bandwidth=0.2)
    nbh = conv.last_neighborhood
    out.backward(up)
    dfeat = x.grad

    with torch.no_grad():
        out_y = conv(y, cloud, cloud, radius, neighborhood=nbh)
        out_xy = conv(x.detach() + 2 * y, cloud, cloud, radius, neighborhood=nbh)
        assert float((out_xy - (out + 2 * out_y)).abs().max()) <= 2e-5 * float(out_xy.abs().max())
    lhs = float((up.double() * out.detach().double()).sum())
    rhs = float((dfeat.double() * x.detach().double()).sum())
    assert abs(lhs - rhs) <= 1e-5 * (float((up.double() * out.detach().double()).abs().sum()))

    # sampled rows in float64
    ids = nbh._original_neigh_ids.long()
    ranges = nbh._samples_neigh_ranges.long()
    pdf = nbh.get_pdf().double()
    w = conv.weights.detach().double()[0]                # [3, 16]
    b = conv.biases.detach().double().reshape(1, 16)
    final = conv.final_weights.detach().double()[0]      # [C*16, C]
    pts = cloud._points.double()
    rng = np.random.default_rng(0)
    picks = torch.as_tensor(rng.choice(n, 200, replace=False), device="cuda")
    starts = torch.where(picks > 0, ranges[(picks - 1).clamp(min=0)], torch.zeros_like(picks))

    def basis_of(seg):                                   # pairs seg -> [len, 16]
        diff = (pts[ids[seg, 0]] - pts[ids[seg, 1]]) / radius
        return torch.nn.functional.leaky_relu(diff @ w + b, 0.2) / pdf[seg].reshape(-1, 1)

    xs, ups = x.detach().double(), up.double()
    for centre, a, e in zip(picks.tolist(), starts.tolist(), ranges[picks].tolist()):
        seg = torch.arange(a, e, device="cuda")
        assert bool((ids[seg, 1] == centre).all())
        bas = basis_of(seg)
        proj = torch.einsum("mc,mk->ck", xs[ids[seg, 0]], bas).reshape(1, -1)
        pmag = torch.einsum("mc,mk->ck", xs[ids[seg, 0]].abs(), bas.abs()).reshape(1, -1)
        elementwise(out[centre].detach().cpu().numpy(), (proj @ final).cpu().numpy()[0],
                    (pmag @ final.abs()).cpu().numpy()[0])
    # the feature gradient of point j collects the pairs (j, i); the pairs of the
    # self-neighbourhood are symmetric, so they are found through j's own segment
    pair_key = ids[:, 0] * n + ids[:, 1]
    order = torch.argsort(pair_key)
    sorted_key = pair_key[order]
    w3 = final.reshape(c, 16, c)
    for j, a, e in list(zip(picks.tolist(), starts.tolist(), ranges[picks].tolist()))[:60]:
        centres = ids[torch.arange(a, e, device="cuda"), 0]          # by symmetry: the i with j in N(i)
        pos = torch.searchsorted(sorted_key, j * n + centres)
        seg = order[pos]
        assert bool((ids[seg, 0] == j).all()) and bool((ids[seg, 1] == centres).all())
        dproj = torch.einsum("mf,ckf->mck", ups[centres], w3)         # [len, C, 16]
        bas = basis_of(seg)
        expect = torch.einsum("mck,mk->c", dproj, bas)
        mag = torch.einsum("mck,mk->c", torch.einsum("mf,ckf->mck", ups[centres].abs(), w3.abs()),
                           bas.abs())
        elementwise(dfeat[j].cpu().numpy(), expect.cpu().numpy(), mag.cpu().numpy())


@pytest.mark.parametrize("layer", ["mcconv", "kpconv", "pointconv"])
def test_fused_layers_in_two_dimensions(layer):
    """The three convolutions on planar clouds (D = 2 takes its own instantiation of
    every fused kernel): outputs and gradients against float64 torch autograd of the
    reference expressions on the layer's own pair table and densities."""
    from tensorflow_graphics_point_clouds_amd import layers, pc
    rng = np.random.default_rng(21)
    n, n_out, batch, radius, c_in, c_out = 2600, 700, 2, 0.07, 16, 32
    pts = rng.random((n, 2)).astype(np.float32)
    bids = np.sort(rng.integers(0, batch, n)).astype(np.int32)
    ctr = rng.random((n_out, 2)).astype(np.float32)
    cb = np.sort(rng.integers(0, batch, n_out)).astype(np.int32)
    feat = rng.standard_normal((n, c_in)).astype(np.float32)
    cin, cout = pc.PointCloud(dev(pts), dev(bids), batch), pc.PointCloud(dev(ctr), dev(cb), batch)
    if layer == "mcconv":
        conv = layers.MCConv(c_in, c_out, 2, num_mlps=1, mlp_size=[16],
                             non_linearity_type="leaky_relu", seed=1)
    elif layer == "kpconv":
        ang = np.linspace(0, 2 * np.pi, 6, endpoint=False)
        kp = np.concatenate([np.zeros((1, 2)), 0.8 * np.stack([np.cos(ang), np.sin(ang)], 1)])
        conv = layers.KPConv(c_in, c_out, num_kernel_points=7, num_dims=2,
                             custom_kernel_points=kp.astype(np.float32), seed=2)
    else:
        conv = layers.PointConv(c_in, c_out, 2, size_hidden=16, seed=3)
        with torch.no_grad():      # a density MLP away from its kinks and from zero
            conv.pdf_weights_1.abs_().add_(0.2)
            conv.pdf_weights_2.abs_().add_(0.2)
            conv.pdf_biases_2.fill_(0.5)
    tfeat = dev(feat).requires_grad_(True)
    out = conv(tfeat, cin, cout, radius)
    up = rng.standard_normal(out.shape).astype(np.float32)
    out.backward(dev(up))

    nb = conv.last_neighborhood
    ids = nb._original_neigh_ids.cpu().long()
    f64 = lambda t: t.detach().cpu().double()
    x = torch.tensor(feat.astype(np.float64), requires_grad=True)
    delta = torch.tensor((pts[ids[:, 0]] - ctr[ids[:, 1]]).astype(np.float64))
    ref_params = {}

    def leaf(name, t):
        ref_params[name] = f64(t).requires_grad_(True)
        return ref_params[name]

    if layer == "mcconv":
        pdf = f64(nb.get_pdf()).reshape(-1, 1)
        hid = torch.nn.functional.leaky_relu(
            (delta / radius) @ leaf("weights", conv.weights)[0] + leaf("biases", conv.biases)[0], 0.2)
        basis = hid / pdf
        final = leaf("final_weights", conv.final_weights)[0]
    elif layer == "kpconv":
        kpt = torch.tensor(kp * 0.75)
        dist = ((delta / radius)[:, None, :] - kpt[None]).norm(dim=2)
        basis = torch.relu(1.0 - dist)
        final = leaf("weights", conv.weights)
    else:
        pdf = f64(nb.get_pdf())
        mx = torch.zeros(n_out, dtype=torch.float64).scatter_reduce(0, ids[:, 1], pdf, "amax",
                                                                    include_self=False)
        rel = (pdf / mx[ids[:, 1]]).reshape(-1, 1)
        y = torch.relu(rel @ leaf("pdf_weights_1", conv.pdf_weights_1) +
                       leaf("pdf_biases_1", conv.pdf_biases_1)) @ \
            leaf("pdf_weights_2", conv.pdf_weights_2) + leaf("pdf_biases_2", conv.pdf_biases_2)
        basis = torch.relu(delta @ leaf("weights", conv.weights) + leaf("biases", conv.biases)) / y
        final = leaf("final_weights", conv.final_weights)
    per_pair = x[ids[:, 0]][:, :, None] * basis[:, None, :]
    proj = torch.zeros(n_out, c_in, basis.shape[1], dtype=torch.float64).index_add(
        0, ids[:, 1], per_pair)
    ref = proj.reshape(n_out, -1) @ final.reshape(-1, c_out)
    normwise(out.detach().cpu().numpy(), ref.detach().numpy(), tol=1e-5)
    (ref * torch.tensor(up.astype(np.float64))).sum().backward()
    normwise(tfeat.grad.cpu().numpy(), x.grad.numpy(), tol=1e-5)
    for name, t in ref_params.items():
        normwise(getattr(conv, name).grad.cpu().numpy(), t.grad.numpy(), tol=1e-5)
    # output, feature gradient and final-weight gradient elementwise: the same sums over the
    # absolute values of their terms (the basis values enter with their own magnitude)
    mx = x.detach().abs().requires_grad_(True)
    mfinal = final.detach().abs().requires_grad_(True)
    mproj = torch.zeros(n_out, c_in, basis.shape[1], dtype=torch.float64).index_add(
        0, ids[:, 1], mx[ids[:, 0]][:, :, None] * basis.detach().abs()[:, None, :])
    mout = mproj.reshape(n_out, -1) @ mfinal.reshape(-1, c_out)
    elementwise(out.detach().cpu().numpy(), ref.detach().numpy(), mout.detach().numpy())
    gx, gfinal = torch.autograd.grad((mout * torch.tensor(np.abs(up).astype(np.float64))).sum(),
                                     [mx, mfinal])
    elementwise(tfeat.grad.cpu().numpy(), x.grad.numpy(), gx.numpy())
    fname = "weights" if layer == "kpconv" else "final_weights"
    elementwise(getattr(conv, fname).grad.cpu().numpy().reshape(gfinal.shape),
                ref_params[fname].grad.numpy().reshape(gfinal.shape), gfinal.numpy())


def test_mcconv_step_replays_from_a_captured_graph():
    """With its neighbourhood built, a Monte-Carlo convolution enqueues kernels and
    library products only: forward + backward recorded in a HIP graph, replayed on
    changed features with eager steps in between; outputs and every gradient equal
    the eager ones bit for bit (the layer path has no atomics)."""
    from tensorflow_graphics_point_clouds_amd import layers, pc
    gen = torch.Generator(device="cuda").manual_seed(3)
    n = 4000
    pts = torch.rand((n, 3), device="cuda", generator=gen)
    bids = (torch.arange(n, device="cuda") % 2).int()
    cloud = pc.PointCloud(pts, bids, 2)
    conv = layers.MCConv(32, 48, 3, num_mlps=1, mlp_size=[16], seed=4)
    feat = torch.randn((n, 32), device="cuda", generator=gen).requires_grad_(True)
    up = torch.randn((n, 48), device="cuda", generator=gen)
    nbh = pc.Neighborhood(pc.Grid(cloud, 0.12), 0.12, cloud)
    params = list(conv.parameters())

    def step():
        feat.grad = None
        for p in params:
            p.grad = None
        out = conv(feat, cloud, cloud, 0.12, neighborhood=nbh)
        out.backward(up)
        return out

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    feat.grad = None
    for p in params:
        p.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = conv(feat, cloud, cloud, 0.12, neighborhood=nbh)
        out.backward(up)
    captured = [out, feat.grad] + [p.grad for p in params]
    for rep in range(3):
        with torch.no_grad():
            feat.copy_(torch.randn((n, 32), device="cuda", generator=gen))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        eager_out = step()
        torch.cuda.synchronize()
        eager = [eager_out, feat.grad] + [p.grad for p in params]
        for a, b in zip(got, eager):
            assert torch.equal(a, b), rep
        # the eager step re-created the gradient tensors; point the graph's at fresh zeros
        feat.grad = captured[1]
        for p, g in zip(params, captured[2:]):
            p.grad = g


def _slope(act, z):
    if act == "relu":
        return (z > 0).double()
    if act == "leaky_relu":
        return torch.where(z > 0, 1.0, 0.2)
    if act == "elu":
        return torch.where(z > 0, torch.ones_like(z), torch.exp(z))
    return torch.ones_like(z)


@pytest.mark.parametrize("rows,i,o,act", [(1, 3, 8, "relu"), (70001, 3, 16, "leaky_relu"),
                                          (5000, 8, 16, "elu"), (333, 16, 64, "relu"),
                                          (40000, 64, 64, "elu"), (129, 1, 16, "relu"),
                                          (2049, 16, 1, None), (0, 3, 8, "relu"),
                                          (10000, 5, 49, "leaky_relu")])
def test_pair_dense_layer_matches_float64(rows, i, o, act):
    """One per-pair layer of a kernel MLP, y = act(x w + b), and its three gradients against
    float64 autograd, elementwise: |got - expect| <= 1e-5 * mag with mag the same sum over
    the absolute values of its terms; the weight and bias gradients (sums over all rows,
    added in a fixed order) come out bit-equal on a second call."""
    from tensorflow_graphics_point_clouds_amd import layers
    gen = torch.Generator(device="cuda").manual_seed(rows + i + o)
    x = torch.randn((rows, i), device="cuda", generator=gen).requires_grad_(True)
    w = (torch.randn((i, o), device="cuda", generator=gen) / max(i, 1) ** 0.5).requires_grad_(True)
    b = (0.3 * torch.randn((1, o), device="cuda", generator=gen)).requires_grad_(True)
    up = torch.randn((rows, o), device="cuda", generator=gen)
    code = {None: -1, "relu": 0, "leaky_relu": 1, "elu": 2}[act]
    y = layers._pair_dense(x, w, b, code)
    grads = torch.autograd.grad((y * up).sum(), [x, w, b])
    again = torch.autograd.grad((layers._pair_dense(x, w, b, code) * up).sum(), [x, w, b])
    for a, c in zip(grads, again):
        assert torch.equal(a, c)
    xd, wd, bd = (t.detach().double().requires_grad_(True) for t in (x, w, b))
    z = xd @ wd + bd
    ref = z if act is None else _T_ACT[act](z)
    mag_z = xd.detach().abs() @ wd.detach().abs() + bd.detach().abs()
    slope = _slope(act, z.detach())
    assert bool(((y.double() - ref).abs() <= 1e-5 * (slope * mag_z + ref.detach().abs()) + 1e-30).all())
    want = torch.autograd.grad((ref * up.double()).sum(), [xd, wd, bd])
    dz = (up.double() * slope).abs()
    mags = (dz @ wd.detach().abs().t(), xd.detach().abs().t() @ dz, dz.sum(0, keepdim=True))
    for got, expect, mag, what in zip(grads, want, mags, ("dx", "dw", "db")):
        err = (got.double() - expect).abs()
        assert bool((err <= 1e-5 * mag + 1e-30).all()), what


@pytest.mark.parametrize("mlp_size,num_mlps,act", [([8, 16], 1, "relu"), ([4, 8, 8], 2, "elu"),
                                                   ([16, 32], 1, "leaky_relu")])
def test_mcconv_with_deeper_kernel_mlp(oracle, mlp_size, num_mlps, act):
    """Kernel MLPs of several layers (MCConv.py:163-171): forward and all gradients
    against float64 autograd of the same expressions on the oracle's pairs and
    densities.  Elementwise: |got - expect| <= 1e-5 * mag, where mag comes from a second
    chain built on the absolute values of every operand -- through an activation a
    magnitude m of the pre-activation becomes slope * m + |act(z)| (the slope carries the
    error of z, the second term the rounding of the activation itself) -- and, for the
    gradients, from autograd of that chain with the upstream |up|."""
    from tensorflow_graphics_point_clouds_amd import layers, pc
    rng = np.random.default_rng(len(mlp_size))
    batch, radius, c_in, c_out = 2, 0.2, 8, 12
    pts, bids, ctr, cb, nbh = _setup(oracle, rng, n=1500, n_out=300, batch=batch, radius=radius)
    feat = rng.standard_normal((len(pts), c_in)).astype(np.float32)
    pdf = nbh.pdf_per_pair(0.2)
    conv = layers.MCConv(c_in, c_out, 3, num_mlps=num_mlps, mlp_size=mlp_size,
                         non_linearity_type=act, seed=4)
    with torch.no_grad():
        for b in [conv.biases] + list(conv.deep_biases):
            b.copy_(dev((0.1 * rng.standard_normal(tuple(b.shape))).astype(np.float32)))
    tfeat = dev(feat).requires_grad_(True)
    out = conv(tfeat, pc.PointCloud(dev(pts), dev(bids), batch),
               pc.PointCloud(dev(ctr), dev(cb), batch), radius, bandwidth=0.2)
    up = rng.standard_normal(tuple(out.shape)).astype(np.float32)
    out.backward(dev(up))

    ids = torch.tensor(nbh.original_neigh_ids).long()
    params = [conv.weights] + list(conv.deep_weights) + [conv.biases] + list(conv.deep_biases) + \
        [conv.final_weights]
    ref = [p.detach().cpu().double().requires_grad_(True) for p in params]
    mref = [p.detach().cpu().double().abs().requires_grad_(True) for p in params]
    depth = len(mlp_size)
    tf = torch.tensor(feat.astype(np.float64), requires_grad=True)
    mf = torch.tensor(np.abs(feat).astype(np.float64), requires_grad=True)
    diff = torch.tensor(((pts[ids[:, 0]] - ctr[ids[:, 1]]) / np.float32(radius)).astype(np.float64))
    cur = diff.unsqueeze(0).expand(num_mlps, -1, -1)
    mag = cur.abs()
    for w, b, mw, mb in zip(ref[:depth], ref[depth:2 * depth], mref[:depth], mref[depth:2 * depth]):
        z = torch.bmm(cur, w) + b
        cur = _T_ACT[act](z)
        mag = _slope(act, z.detach()) * (torch.bmm(mag, mw) + mb) + cur.detach().abs()
    h = mlp_size[-1]
    tpdf = torch.tensor(pdf.astype(np.float64)).reshape(-1, 1)

    def rest(hidden, f, final):
        bas = hidden.permute(1, 0, 2).reshape(len(ids), -1) / tpdf
        per_pair = f[ids[:, 0]][:, :, None] * bas[:, None, :]
        pj = torch.zeros(len(ctr), c_in, num_mlps * h, dtype=torch.float64).index_add(
            0, ids[:, 1], per_pair)
        pj = pj.reshape(-1, c_in, num_mlps, h).permute(2, 0, 1, 3).reshape(num_mlps, -1, c_in * h)
        return torch.bmm(pj, final).permute(1, 0, 2).reshape(len(ctr), -1)

    expect = rest(cur, tf, ref[-1])
    bound = rest(mag, mf, mref[-1])
    elementwise(out.detach().cpu().numpy(), expect.detach().numpy(), bound.detach().numpy())
    tup = torch.tensor(up.astype(np.float64))
    want = torch.autograd.grad((expect * tup).sum(), [tf] + ref)
    mags = torch.autograd.grad((bound * tup.abs()).sum(), [mf] + mref)
    got = [tfeat.grad] + [p.grad for p in params]
    for g, e, m in zip(got, want, mags):
        elementwise(g.cpu().numpy(), e.numpy(), m.numpy())


def test_mcconv_gradient_with_respect_to_points(oracle):
    """Point coordinates that require a gradient (monte_carlo_conv_test.py:196-230
    checks this Jacobian): the layer output depends on them through the kernel
    inputs and through the densities.  Against float64 autograd of the whole
    expression, Gaussian KDE included, on the oracle's pair tables."""
    from tensorflow_graphics_point_clouds_amd import layers, pc
    rng = np.random.default_rng(5)
    n, batch, radius, bw, c_in, c_out, hidden = 600, 2, 0.25, 0.2, 4, 6, 8
    pts = rng.random((n, 3)).astype(np.float32)
    bids = np.sort(rng.integers(0, batch, n)).astype(np.int32)
    feat = rng.standard_normal((n, c_in)).astype(np.float32)
    g = oracle.Grid(pts, bids, batch, np.float32(radius))
    own = oracle.Neighborhood(g, np.float32(radius))                 # sorted self-neighbourhood
    nbh = oracle.Neighborhood(g, np.float32(radius), pts, bids)     # centres in the caller's order
    conv = layers.MCConv(c_in, c_out, 3, num_mlps=1, mlp_size=[hidden], non_linearity_type="elu",
                         seed=2)
    tpts = dev(pts).requires_grad_(True)
    cloud = pc.PointCloud(tpts, dev(bids), batch)
    out = conv(dev(feat), cloud, cloud, radius, bandwidth=bw)
    up = rng.standard_normal(tuple(out.shape)).astype(np.float32)
    out.backward(dev(up))

    p = torch.tensor(pts.astype(np.float64), requires_grad=True)
    order = torch.tensor(g.sorted_indices).long()
    on = torch.tensor(own.neighbors).long()
    u = (p[order][on[:, 0]] - p[order][on[:, 1]]) / (bw * radius)
    u.retain_grad()
    kde = torch.prod(torch.exp(-0.5 * u * u) * (0.3989422804014327 / bw), dim=1)
    per_point = torch.zeros(n, dtype=torch.float64).index_add(0, on[:, 1], kde)
    ids = torch.tensor(nbh.original_neigh_ids).long()
    pdf = per_point[torch.tensor(nbh.neighbors[:, 0]).long()]
    w, b = conv.weights.detach().cpu().double()[0], conv.biases.detach().cpu().double()[0]
    diff = (p[ids[:, 0]] - p[ids[:, 1]]) / radius
    diff.retain_grad()
    basis = torch.nn.functional.elu(diff @ w + b) / pdf[:, None]
    per_pair = torch.tensor(feat.astype(np.float64))[ids[:, 0]][:, :, None] * basis[:, None, :]
    proj = torch.zeros(n, c_in, hidden, dtype=torch.float64).index_add(0, ids[:, 1], per_pair)
    ref = proj.reshape(n, -1) @ conv.final_weights.detach().cpu().double()[0]
    normwise(out.detach().cpu().numpy(), ref.detach().numpy(), tol=1e-5)
    (ref * torch.tensor(up.astype(np.float64))).sum().backward()
    normwise(tpts.grad.cpu().numpy(), p.grad.numpy(), tol=1e-5)
    # per coordinate: the gradient of a point is a signed sum of per-pair terms (through the
    # kernel input of every pair it belongs to, as point or as centre, and through every
    # density term it enters); the error is held to 1e-5 of the sum of their absolute values
    mag = _point_gradient_magnitude(n, [(diff.grad / radius, ids[:, 0], ids[:, 1]),
                                        (u.grad / (bw * radius), order[on[:, 0]], order[on[:, 1]])])
    elementwise(tpts.grad.cpu().numpy(), p.grad.numpy(), mag.numpy())


def _point_gradient_magnitude(n, paths, n_centres=None):
    """Sum of the absolute values of the per-pair terms that a coordinate gradient adds up:
    every path is (gradient with respect to a per-pair difference `a - b`, index of a, index
    of b).  Returns the magnitude for the `a` side ([n, D]) and, if the `b` side is another
    point set of `n_centres` points, for that side too."""
    first = torch.zeros((n, paths[0][0].shape[1]), dtype=torch.float64)
    second = first if n_centres is None else torch.zeros((n_centres, first.shape[1]),
                                                         dtype=torch.float64)
    for grad, a, b, *same in paths:
        first.index_add_(0, a, grad.abs())
        (first if same and same[0] else second).index_add_(0, b, grad.abs())
    return first if n_centres is None else (first, second)


@pytest.mark.parametrize("layer", ["kp_linear", "kp_gaussian_deformable", "pointconv"])
def test_kpconv_and_pointconv_gradient_with_respect_to_points(oracle, layer):
    """kernel_point_conv_test.py:218-260 and point_conv_test.py:218-260 check the
    Jacobian with respect to the point coordinates; here both clouds require a
    gradient and the result is compared with float64 autograd of the same
    expressions (kernel-point correlation, offsets of the deformable kernel,
    relative densities and their MLP)."""
    from tensorflow_graphics_point_clouds_amd import layers, pc, synthetic
    rng = np.random.default_rng(11)
    batch, radius, c_in, c_out, bw = 2, 0.25, 4, 6, 0.2
    pts, bids, ctr, cb, nbh = _setup(oracle, rng, n=700, n_out=150, batch=batch, radius=radius)
    feat = rng.standard_normal((len(pts), c_in)).astype(np.float32)
    ids = torch.tensor(nbh.original_neigh_ids).long()
    tpts, tctr = dev(pts).requires_grad_(True), dev(ctr).requires_grad_(True)
    cin, cout = pc.PointCloud(tpts, dev(bids), batch), pc.PointCloud(tctr, dev(cb), batch)
    p = torch.tensor(pts.astype(np.float64), requires_grad=True)
    q = torch.tensor(ctr.astype(np.float64), requires_grad=True)
    f64 = lambda t: t.detach().cpu().double()
    tf = torch.tensor(feat.astype(np.float64))

    def project(basis):
        per_pair = tf[ids[:, 0]][:, :, None] * basis[:, None, :]
        return torch.zeros(len(ctr), c_in, basis.shape[1], dtype=torch.float64).index_add(
            0, ids[:, 1], per_pair).reshape(len(ctr), -1)

    paths = []      # (per-pair difference a - b, scale of the difference, index of a, index of b)
    if layer == "pointconv":
        conv = layers.PointConv(c_in, c_out, 3, size_hidden=8, non_linearity_type="elu", seed=3)
        with torch.no_grad():
            conv.pdf_biases_2.fill_(0.7)
        out = conv(dev(feat), cin, cout, radius, bandwidth=bw)
        g = oracle.Grid(pts, bids, batch, np.float32(radius))
        own = oracle.Neighborhood(g, np.float32(radius))
        order, on = torch.tensor(g.sorted_indices).long(), torch.tensor(own.neighbors).long()
        u = (p[order][on[:, 0]] - p[order][on[:, 1]]) / (bw * radius)
        u.retain_grad()
        kde = torch.prod(torch.exp(-0.5 * u * u) * (0.3989422804014327 / bw), dim=1)
        per_sorted = torch.zeros(len(p), dtype=torch.float64).index_add(0, on[:, 1], kde)
        pdf = per_sorted[torch.tensor(nbh.neighbors[:, 0]).long()]
        paths.append((u, 1.0 / (bw * radius), order[on[:, 0]], order[on[:, 1]], True))
        mx = torch.zeros(len(ctr), dtype=torch.float64).scatter_reduce(0, ids[:, 1], pdf, "amax",
                                                                       include_self=False)
        rel = (pdf / mx[ids[:, 1]]).reshape(-1, 1)
        cur = torch.relu(rel @ f64(conv.pdf_weights_1) + f64(conv.pdf_biases_1))
        cur = cur @ f64(conv.pdf_weights_2) + f64(conv.pdf_biases_2)
        diff = p[ids[:, 0]] - q[ids[:, 1]]
        diff.retain_grad()
        paths.append((diff, 1.0, ids[:, 0], ids[:, 1]))
        hid = torch.nn.functional.elu(diff @ f64(conv.weights) + f64(conv.biases))
        ref = project(hid / cur) @ f64(conv.final_weights)
    else:
        deform = layer.endswith("deformable")
        kp = synthetic.spherical_kernel_points(15, rotate=False) * 0.8
        conv = layers.KPConv(c_in, c_out, custom_kernel_points=kp, deformable=deform,
                             kp_interpolation="gaussian" if deform else "linear", seed=3)
        if deform:
            with torch.no_grad():
                conv.offset_weights.mul_(0.05)
        sigma = 0.6
        out = conv(dev(feat), cin, cout, radius, kernel_influence_dist=sigma * radius)
        tkp = torch.tensor(kp.astype(np.float64) * 0.75)
        diff = (p[ids[:, 0]] - q[ids[:, 1]]) / radius
        diff.retain_grad()
        paths.append((diff, 1.0 / radius, ids[:, 0], ids[:, 1]))

        def correlation(offsets):
            delta = diff[:, None, :] - tkp[None] - (0 if offsets is None else offsets[ids[:, 1]])
            dist = torch.sqrt((delta * delta).sum(2) + 1e-20)
            if deform:
                return torch.exp(-(dist / (sigma / 3)) ** 2)
            return torch.relu(1 - dist / sigma)

        offsets = None
        if deform:
            offsets = (project(correlation(None)) @ f64(conv.offset_weights)).reshape(-1, 15, 3)
        ref = project(correlation(offsets)) @ f64(conv.weights)
    normwise(out.detach().cpu().numpy(), ref.detach().numpy(), tol=1e-5)
    up = rng.standard_normal(tuple(out.shape)).astype(np.float32)
    out.backward(dev(up))
    (ref * torch.tensor(up.astype(np.float64))).sum().backward()
    normwise(tpts.grad.cpu().numpy(), p.grad.numpy(), tol=1e-5)
    normwise(tctr.grad.cpu().numpy(), q.grad.numpy(), tol=1e-5)
    # per coordinate, against the sum of the absolute per-pair terms of its signed sum.  The
    # kernel-point terms carry a condition number of their own (the unit vector delta / dist of
    # a pair close to a kernel point amplifies the rounding of delta), which this magnitude
    # does not contain: 5e-5 there (1.9e-5 and 4.2e-5 measured), 1e-5 for PointConv.
    mag_p, mag_q = _point_gradient_magnitude(
        len(pts), [(t.grad * scale, a, b, *same) for t, scale, a, b, *same in paths], len(ctr))
    tol = 1e-5 if layer == "pointconv" else 5e-5
    elementwise(tpts.grad.cpu().numpy(), p.grad.numpy(), mag_p.numpy(), tol=tol)
    elementwise(tctr.grad.cpu().numpy(), q.grad.numpy(), mag_q.numpy(), tol=tol)


@pytest.mark.parametrize("layer", ["mcconv", "kpconv", "pointconv", "pool"])
def test_layers_on_degenerate_neighbourhoods(layer):
    """No pair at all (every centre out of reach) and clouds of one point each: the
    convolutions return zeros where nothing is in reach (max pooling the lowest
    float, Pooling.py:54), finite values otherwise, and gradients of the right
    shapes."""
    from tensorflow_graphics_point_clouds_amd import layers, pc
    rng = np.random.default_rng(1)
    pts = rng.random((64, 3)).astype(np.float32)
    bids = np.repeat(np.arange(4), 16).astype(np.int32)
    cloud = pc.PointCloud(dev(pts), dev(bids), 4)
    far = pc.PointCloud(dev(pts[:20] + 9.0), dev(bids[:20]), 4)
    single = pc.PointCloud(dev(pts[:4]), dev(np.arange(4, dtype=np.int32)), 4)
    feat = torch.randn((64, 16), device="cuda", requires_grad=True)
    make = {"mcconv": lambda: layers.MCConv(16, 16, 3, num_mlps=1, mlp_size=[16]),
            "kpconv": lambda: layers.KPConv(16, 16),
            "pointconv": lambda: layers.PointConv(16, 16, 3, size_hidden=8),
            "pool": lambda: layers.MaxPooling()}[layer]
    conv = make()
    out = conv(feat, cloud, far, 0.2)
    assert out.shape == (20, 16)
    if layer == "pool":     # an empty maximum is the lowest float, as tf.math.unsorted_segment_max gives
        assert bool((out.detach() == torch.finfo(torch.float32).min).all())
    else:
        assert float(out.detach().abs().max()) == 0.0
        assert conv.last_neighborhood._neighbors.shape[0] == 0
    out.sum().backward()
    assert feat.grad is not None and float(feat.grad.abs().max()) == 0.0
    conv = make()
    f1 = torch.randn((4, 16), device="cuda", requires_grad=True)
    out = conv(f1, single, single, 0.2)                       # every point its own only neighbour
    assert out.shape == (4, 16) and bool(torch.isfinite(out).all())
    out.sum().backward()
    assert f1.grad.shape == (4, 16) and bool(torch.isfinite(f1.grad).all())
