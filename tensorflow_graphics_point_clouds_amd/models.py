"""The classification network of the reference's training script
(modelnet40.py:128-398): a point hierarchy, one initial convolution, a strided
and a plain residual block per level, global average pooling and a two-layer
head.  Dense parts are stock torch; the spatial parts are the HIP-backed layers."""
import numpy as np
import torch

from . import blocks, layers, pc


def _spatial_conv(layer_type, c_in, c_out, device, seed):
    # modelnet40.py:156-179
    if layer_type == "MCConv":
        return layers.MCConv(c_in, c_out, num_dims=3, num_mlps=1, mlp_size=[16], device=device,
                             seed=seed)
    if layer_type == "PointConv":
        return layers.PointConv(c_in, c_out, num_dims=3, size_hidden=32, device=device, seed=seed)
    if layer_type == "KPConv":
        return layers.KPConv(c_in, c_out, num_dims=3, num_kernel_points=15, device=device,
                             seed=seed)
    raise ValueError("Unknown layer type!")


class ConvBlock(torch.nn.Module):
    """Residual block (modelnet40.py:128-260): batch norm + leaky ReLU before a
    1x1 reduction to a quarter of the output width, the spatial convolution and
    a 1x1 expansion; the skip branch max-pools onto the output cloud when
    `strided` and is re-projected when the widths differ."""

    def __init__(self, num_features_in, num_features_out, layer_type, strided=False,
                 device="cuda", seed=0):
        super().__init__()
        inner = num_features_out // 4
        bn = lambda c: blocks.BatchNorm(c, momentum=0.9, device=device)
        self.norms = torch.nn.ModuleList([bn(num_features_in), bn(inner), bn(inner)])
        self.reduce = blocks.Conv1x1(num_features_in, inner, device=device, seed=seed)
        self.conv = _spatial_conv(layer_type, inner, inner, device, seed + 1)
        self.expand = blocks.Conv1x1(inner, num_features_out, device=device, seed=seed + 2)
        self.pool = layers.MaxPooling() if strided else None
        self.skip_norm = self.skip_conv = None
        if num_features_in != num_features_out:
            self.skip_norm = bn(num_features_in)
            self.skip_conv = blocks.Conv1x1(num_features_in, num_features_out, device=device,
                                            seed=seed + 3)
        self.act = torch.nn.LeakyReLU(0.3)          # Keras' default slope

    def forward(self, features, point_cloud_in, point_cloud_out, conv_radius, pool_radius=None,
                training=None):
        # the convolution and the pooling of a strided block look at the same pairs
        # when their radii agree (modelnet40.py:373-379 passes the pooling radius twice)
        shared = None
        if self.pool is not None and pool_radius is not None and \
                float(conv_radius) == float(pool_radius):
            radii = pc._as_vector(conv_radius, 3, point_cloud_in._points.device)
            shared = pc.Neighborhood(pc.Grid(point_cloud_in, radii), radii, point_cloud_out)
        res = self.reduce(self.act(self.norms[0](features, training)), point_cloud_in)
        res = self.conv(self.act(self.norms[1](res, training)), point_cloud_in, point_cloud_out,
                        conv_radius, shared)
        res = self.expand(self.act(self.norms[2](res, training)), point_cloud_out)
        skip = features
        if self.pool is not None:
            skip = self.pool(skip, point_cloud_in, point_cloud_out, pool_radius, shared)
        if self.skip_conv is not None:
            skip = self.skip_conv(self.act(self.skip_norm(skip, training)), point_cloud_out)
        return res + skip


class ClassificationNet(torch.nn.Module):
    """modelnet40.py:263-398.  `feature_sizes` has one width per level, then the
    hidden width of the head and the number of classes; `pool_radii` and
    `conv_radii` one radius per level.  The input feature is the constant 1 on
    the first sampled level."""

    def __init__(self, feature_sizes, pool_radii, conv_radii, layer_type="MCConv",
                 sampling_method="cell average", dropout_rate=0.0, device="cuda", seed=0):
        super().__init__()
        self.sampling_method = sampling_method
        self.pool_radii = [float(r) for r in np.asarray(pool_radii).reshape(-1)]
        self.conv_radii = [float(r) for r in np.asarray(conv_radii).reshape(-1)]
        self.num_levels = len(self.pool_radii)
        if len(feature_sizes) != self.num_levels + 2 or len(self.conv_radii) != self.num_levels:
            raise ValueError("expected one feature size and one convolution radius per level, "
                             "then the head width and the class count")
        self.init_conv = _spatial_conv(layer_type, 1, feature_sizes[0], device, seed)
        self.strided_conv_blocks = torch.nn.ModuleList(
            ConvBlock(feature_sizes[i - 1], feature_sizes[i], layer_type, strided=True,
                      device=device, seed=seed + 10 * i) for i in range(1, self.num_levels))
        self.conv_blocks = torch.nn.ModuleList(
            ConvBlock(feature_sizes[i], feature_sizes[i], layer_type, device=device,
                      seed=seed + 10 * i + 5) for i in range(self.num_levels))
        self.global_pooling = layers.GlobalAveragePooling()
        last, hidden, classes = feature_sizes[self.num_levels - 1], feature_sizes[-2], \
            feature_sizes[-1]
        self.head_norms = torch.nn.ModuleList([
            blocks.BatchNorm(last, momentum=0.9, device=device),
            blocks.BatchNorm(hidden, momentum=0.9, device=device)])
        self.head_dense = torch.nn.ModuleList([
            torch.nn.Linear(last, hidden, device=device),
            torch.nn.Linear(hidden, classes, device=device)])
        self.dropout_rate = float(dropout_rate)
        self.act = torch.nn.LeakyReLU(0.3)

    def forward(self, points, sizes=None, training=None, batch_ids=None, batch_size=None):
        """points [B, V, 3] with `sizes` [B] (or [N, 3] with `batch_ids`) ->
        logits [B, classes]."""
        cloud = pc.PointCloud(points, batch_ids=batch_ids, batch_size=batch_size, sizes=sizes)
        hierarchy = pc.PointHierarchy(cloud, self.pool_radii, self.sampling_method)
        first = hierarchy[1]
        features = torch.ones((first._points.shape[0], 1), dtype=torch.float32,
                              device=first._points.device)
        for i in range(self.num_levels):
            if i == 0:
                features = self.init_conv(features, first, first, self.conv_radii[0])
            else:
                features = self.strided_conv_blocks[i - 1](
                    features, hierarchy[i], hierarchy[i + 1], self.pool_radii[i],
                    self.pool_radii[i], training=training)
            features = self.conv_blocks[i](features, hierarchy[i + 1], hierarchy[i + 1],
                                           self.conv_radii[i], training=training)
        features = self.global_pooling(features, hierarchy[-1])
        dropping = self.training if training is None else bool(training)
        drop = lambda x: torch.nn.functional.dropout(x, self.dropout_rate, dropping)
        features = self.head_dense[0](drop(self.act(self.head_norms[0](features, training))))
        features = self.act(drop(self.head_norms[1](features, training)))
        return self.head_dense[1](features)
