"""Feature-space layers, residual blocks and the classification network on the
GPU.  The blocks are compositions: their spatial convolutions are pinned one by
one in test_gpu_layers.py, so here the whole block is compared with a float64
torch chain of the same expressions (batch statistics, activation, Monte-Carlo
convolution on the block's own pair tables and densities, skip connection),
outputs and gradients.  Tolerance 1e-5 normwise (max error over max |expected|) over several fp32 convolutions and
normalisations in a row."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

pytestmark = pytest.mark.gpu

TOL = 1e-5


def dev(a):
    return torch.as_tensor(np.ascontiguousarray(a)).cuda().contiguous()


def normwise(got, expect, tol=TOL):
    got, expect = np.asarray(got, np.float64), np.asarray(expect, np.float64)
    assert np.abs(got - expect).max() <= tol * np.abs(expect).max(), \
        np.abs(got - expect).max() / np.abs(expect).max()


def f64(t):
    return t.detach().cpu().double()


def batch_norm_ref(x, eps=1e-3):
    return (x - x.mean(0)) / torch.sqrt(x.var(0, unbiased=False) + eps)


def mc_conv_ref(conv, feat, pts_in, pts_out, radius, final=None):
    """float64 Monte-Carlo convolution with the layer's parameters on the pair
    table and densities the layer used in its last call."""
    nb = conv.last_neighborhood
    ids = nb._original_neigh_ids.cpu().long()
    pdf = f64(nb.get_pdf()).reshape(-1, 1)
    w, b = f64(conv.weights), f64(conv.biases)
    final = f64(conv.final_weights) if final is None else final
    l, _, h = w.shape
    c = feat.shape[1]
    diff = (f64(pts_in)[ids[:, 0]] - f64(pts_out)[ids[:, 1]]) / radius
    hid = torch.nn.functional.leaky_relu(torch.einsum("md,ldh->lmh", diff, w) + b, 0.2)
    basis = hid.permute(1, 0, 2).reshape(len(ids), -1) / pdf
    per_pair = feat[ids[:, 0]][:, :, None] * basis[:, None, :]
    proj = torch.zeros(len(pts_out), c, l * h, dtype=torch.float64).index_add(0, ids[:, 1], per_pair)
    proj = proj.reshape(-1, c, l, h).permute(2, 0, 1, 3).reshape(l, -1, c * h)
    return torch.bmm(proj, final).permute(1, 0, 2).reshape(len(pts_out), -1)


def conv1x1_ref(layer, x):
    return x @ f64(layer.weights) + f64(layer.bias)


def _cloud(rng, n=1500, batch=2):
    pts = rng.random((n, 3)).astype(np.float32)
    bids = rng.integers(0, batch, n).astype(np.int32)
    bids[:batch] = np.arange(batch)
    return pts, bids


def test_conv1x1_and_batch_norm():
    from tensorflow_graphics_point_clouds_amd import blocks, pc
    rng = np.random.default_rng(0)
    pts, bids = _cloud(rng, 700, 3)
    cloud = pc.PointCloud(dev(pts), dev(bids), 3)
    feat = rng.standard_normal((700, 12)).astype(np.float32)
    layer = blocks.Conv1x1(12, 20, seed=3)
    with torch.no_grad():
        layer.bias.copy_(dev(rng.standard_normal((1, 20)).astype(np.float32)))
    out = layer(dev(feat), cloud)
    expect = conv1x1_ref(layer, torch.tensor(feat.astype(np.float64)))
    normwise(out.detach().cpu().numpy(), expect.numpy(), tol=1e-5)
    # truncated-normal initial weights of scale sqrt(2 / C_in) (Conv1x1.py:52-59)
    w = layer.weights.detach().cpu().numpy()
    assert np.abs(w).max() <= 2.0 * np.sqrt(2.0 / 12) + 1e-6
    # padded input and output
    padded = cloud.get_unflatten()(dev(feat))
    out_p = layer(padded, cloud, return_padded=True)
    assert torch.equal(out_p, cloud.get_unflatten()(out))
    assert blocks.Conv1x1(4, 4, use_bias=False).bias is None
    # per-call training flag; Keras' momentum and epsilon
    bn = blocks.BatchNorm(12)
    assert abs(bn.momentum - 0.01) < 1e-12 and bn.eps == 1e-3
    bn.eval()
    y = bn(dev(feat), training=True)
    normwise(y.detach().cpu().numpy(), batch_norm_ref(torch.tensor(feat.astype(np.float64))).numpy(),
             tol=1e-5)
    assert not bn.training and float(bn.running_mean.abs().max()) > 0.0
    z = bn(dev(feat), training=False)
    assert float((z - y).detach().abs().max()) > 1e-3       # running statistics, not the batch's


@pytest.mark.parametrize("shortcut", [False, True])
def test_point_resnet(shortcut):
    from tensorflow_graphics_point_clouds_amd import blocks, pc
    rng = np.random.default_rng(1)
    pts, bids = _cloud(rng)
    cloud = pc.PointCloud(dev(pts), dev(bids), 2)
    c, radius = 16, 0.2
    net = blocks.PointResNet(c, 2, 3, projection_shortcuts=shortcut, num_mlps=1, mlp_size=[8])
    feat = rng.standard_normal((len(pts), c)).astype(np.float32)
    tfeat = dev(feat).requires_grad_(True)
    out = net(tfeat, cloud, radius, training=True)
    up = rng.standard_normal(out.shape).astype(np.float32)
    out.backward(dev(up))

    x = torch.tensor(feat.astype(np.float64), requires_grad=True)
    final0 = f64(net._conv_layers[0].final_weights).requires_grad_(True)
    cur = x
    for i in range(2):
        skip = cur
        for j in (2 * i, 2 * i + 1):
            cur = torch.relu(batch_norm_ref(cur))
            cur = mc_conv_ref(net._conv_layers[j], cur, cloud._points, cloud._points, radius,
                              final0 if j == 0 else None)
        if shortcut:
            skip = conv1x1_ref(net._projection_layers[i], skip)
        cur = cur + skip
    normwise(out.detach().cpu().numpy(), cur.detach().numpy())
    (cur * torch.tensor(up.astype(np.float64))).sum().backward()
    normwise(tfeat.grad.cpu().numpy(), x.grad.numpy())
    normwise(net._conv_layers[0].final_weights.grad.cpu().numpy(), final0.grad.numpy())
    # one neighbourhood serves all four convolutions
    assert len({id(l.last_neighborhood) for l in net._conv_layers}) == 1


def test_point_resnet_bottleneck():
    from tensorflow_graphics_point_clouds_amd import blocks, pc
    rng = np.random.default_rng(2)
    pts, bids = _cloud(rng)
    cloud = pc.PointCloud(dev(pts), dev(bids), 2)
    c, inner, radius = 32, 8, 0.2
    net = blocks.PointResNetBottleNeck(c, inner, 2, 3, projection_shortcuts=True, num_mlps=2,
                                       mlp_size=[8])
    feat = rng.standard_normal((len(pts), c)).astype(np.float32)
    tfeat = dev(feat).requires_grad_(True)
    out = net(tfeat, cloud, radius, training=True)
    up = rng.standard_normal(out.shape).astype(np.float32)
    out.backward(dev(up))

    x = torch.tensor(feat.astype(np.float64), requires_grad=True)
    cur = x
    for i in range(2):
        skip = cur
        cur = conv1x1_ref(net._downsampling_layers[i], torch.relu(batch_norm_ref(cur)))
        cur = mc_conv_ref(net._conv_layers[i], torch.relu(batch_norm_ref(cur)), cloud._points,
                          cloud._points, radius)
        cur = conv1x1_ref(net._upsampling_layers[i], torch.relu(batch_norm_ref(cur)))
        cur = cur + conv1x1_ref(net._projection_layers[i], skip)
    normwise(out.detach().cpu().numpy(), cur.detach().numpy())
    (cur * torch.tensor(up.astype(np.float64))).sum().backward()
    normwise(tfeat.grad.cpu().numpy(), x.grad.numpy())


@pytest.mark.parametrize("radii", [(0.2, 0.3, 0.2), (0.2, 0.3, 0.25)])
def test_point_resnet_spatial_bottleneck(radii):
    """Down onto a cell-average sample, inside it, and back up; with equal first and
    last radius the way up is the transposed neighbourhood of the way down."""
    from tensorflow_graphics_point_clouds_amd import blocks, pc
    rng = np.random.default_rng(3)
    pts, bids = _cloud(rng)
    cloud = pc.PointCloud(dev(pts), dev(bids), 2)
    small = pc.PointHierarchy(cloud, [0.1], "cell average")[1]
    c = 16
    net = blocks.PointResNetSpatialBottleNeck(c, 1, 3, num_mlps=1, mlp_size=[8])
    feat = rng.standard_normal((len(pts), c)).astype(np.float32)
    tfeat = dev(feat).requires_grad_(True)
    out = net(tfeat, cloud, small, radii, training=True)
    assert out.shape == (len(pts), c)
    up = rng.standard_normal(out.shape).astype(np.float32)
    out.backward(dev(up))

    x = torch.tensor(feat.astype(np.float64), requires_grad=True)
    clouds = [(cloud, small), (small, small), (small, cloud)]
    cur = x
    for stage in range(3):
        cur = torch.relu(batch_norm_ref(cur))
        cur = mc_conv_ref(net._stage_layers[stage], cur, clouds[stage][0]._points,
                          clouds[stage][1]._points, radii[stage])
    cur = cur + x
    normwise(out.detach().cpu().numpy(), cur.detach().numpy())
    (cur * torch.tensor(up.astype(np.float64))).sum().backward()
    normwise(tfeat.grad.cpu().numpy(), x.grad.numpy())
    down, back = net._stage_layers[0].last_neighborhood, net._stage_layers[2].last_neighborhood
    assert (back is down.transpose()) == (radii[0] == radii[2])
    # the pairs of the way up are those of a direct search from the small cloud
    direct = pc.Neighborhood(pc.Grid(small, radii[2]), radii[2], cloud)
    a = back._original_neigh_ids.cpu().numpy()
    b = direct._original_neigh_ids.cpu().numpy()
    assert np.array_equal(np.unique(a, axis=0), np.unique(b, axis=0))


@pytest.mark.parametrize("layer_type", ["MCConv", "KPConv", "PointConv"])
def test_classification_net_learns_primitives(layer_type):
    """A two-level network of every layer type on the four-class primitive set: the
    training loss falls over a few RMSprop steps, evaluation mode runs, every
    parameter receives a finite gradient."""
    from tensorflow_graphics_point_clouds_amd import models, synthetic, train_classification
    pts, labels = synthetic.labelled_primitives(32, 256, seed=5)
    torch.manual_seed(0)
    net = models.ClassificationNet([16, 32, 32, 4], np.array([0.15, 0.3]), np.array([0.3, 0.6]),
                                   layer_type=layer_type, dropout_rate=0.0, seed=1)
    opt = torch.optim.RMSprop(net.parameters(), lr=1e-3, alpha=0.9, eps=1e-7)
    rng = np.random.default_rng(0)
    first = train_classification.run_epoch(net, pts, labels, 16, rng, opt)
    for _ in range(5):
        last = train_classification.run_epoch(net, pts, labels, 16, rng, opt)
    assert np.isfinite(last[0]) and last[0] < first[0]
    for name, p in net.named_parameters():
        assert p.grad is not None and bool(torch.isfinite(p.grad).all()), name
    loss, acc = train_classification.run_epoch(net, pts, labels, 16, rng)
    assert np.isfinite(loss) and 0.0 <= acc <= 1.0
    logits = net(dev(pts[:4]), training=False)
    assert logits.shape == (4, 4)
