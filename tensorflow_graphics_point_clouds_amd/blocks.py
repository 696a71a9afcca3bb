"""Feature-space layers and residual blocks around the point convolutions
(pylib/pc/layers/Conv1x1.py:24-101, pylib/pc/layers/network_blocks.py:27-465).
Everything here is dense per-point work (a GEMM, batch normalisation, an
activation) on stock torch; the spatial convolutions inside the blocks are the
layers of `layers.py`."""
import math

import torch

from . import layers, pc

_F32 = torch.float32

layer_types = {"mcconv": layers.MCConv, "mc": layers.MCConv, "mc_conv": layers.MCConv,
               "kpconv": layers.KPConv, "kp": layers.KPConv, "kp_conv": layers.KPConv,
               "pointconv": layers.PointConv, "point_conv": layers.PointConv}


def _identity(features, *args, **kwargs):
    return features


class BatchNorm(torch.nn.BatchNorm1d):
    """Batch normalisation over the points with Keras' defaults (moving-average
    momentum 0.99, epsilon 1e-3; torch counts the momentum from the other side).
    `training`, when given, overrides the module's train/eval mode, as the
    reference passes it per call."""

    def __init__(self, num_features, momentum=0.99, eps=1e-3, device="cuda"):
        super().__init__(num_features, eps=eps, momentum=1.0 - momentum, device=device)

    def forward(self, features, training=None):
        if training is None or bool(training) == self.training:
            return super().forward(features)
        mode = self.training
        self.train(bool(training))
        try:
            return super().forward(features)
        finally:
            self.train(mode)


class Conv1x1(torch.nn.Module):
    """Per-point linear map features [N, C_in] -> [N, C_out] with a bias
    (Conv1x1.py:24-101): truncated-normal weights of scale sqrt(2 / C_in), zero
    bias."""

    def __init__(self, num_features_in, num_features_out, use_bias=True, device="cuda", seed=0):
        super().__init__()
        gen = torch.Generator().manual_seed(seed)
        w = layers._truncated_normal((num_features_in, num_features_out),
                                     math.sqrt(2.0 / float(num_features_in)), gen, device)
        self.weights = torch.nn.Parameter(w)
        self.bias = torch.nn.Parameter(torch.zeros((1, num_features_out), dtype=_F32,
                                                   device=device)) if use_bias else None

    def forward(self, features, point_cloud, return_sorted=False, return_padded=False):
        features = point_cloud.flatten_features(features)
        out = features @ self.weights
        if self.bias is not None:
            out = out + self.bias
        return point_cloud.format_output(out, return_sorted, return_padded)


def _own_neighborhood(point_cloud, radius, num_dims):
    radii = pc._as_vector(radius, num_dims, point_cloud._points.device)
    return pc.Neighborhood(pc.Grid(point_cloud, radii), radii, point_cloud)


class PointResNet(torch.nn.Module):
    """Pre-activation residual blocks of two point convolutions on one cloud
    (network_blocks.py:27-151).  `kwargs` go to the convolution layers."""

    def __init__(self, num_features, num_blocks, num_dims, layer_type="MCConv",
                 projection_shortcuts=False, activation=torch.relu, device="cuda", **kwargs):
        super().__init__()
        self._num_dims, self._num_blocks, self._activation = num_dims, num_blocks, activation
        conv = layer_types[layer_type.lower()]
        self._batch_norm_layers = torch.nn.ModuleList(
            BatchNorm(num_features, device=device) for _ in range(2 * num_blocks))
        self._conv_layers = torch.nn.ModuleList(
            conv(num_features, num_features, num_dims=num_dims, device=device, seed=i, **kwargs)
            for i in range(2 * num_blocks))
        self._projection_layers = torch.nn.ModuleList(
            Conv1x1(num_features, num_features, device=device, seed=100 + i)
            for i in range(num_blocks)) if projection_shortcuts else None

    def forward(self, features, point_cloud, radius, training=None, neighborhood=None,
                return_sorted=False, return_padded=False, **kwargs):
        features = point_cloud.flatten_features(features)
        if neighborhood is None:
            neighborhood = _own_neighborhood(point_cloud, radius, self._num_dims)
        for i in range(self._num_blocks):
            skip = features
            for j in (2 * i, 2 * i + 1):
                features = self._activation(self._batch_norm_layers[j](features, training))
                features = self._conv_layers[j](features, point_cloud, point_cloud, radius,
                                                neighborhood, **kwargs)
            if self._projection_layers is not None:
                skip = self._projection_layers[i](skip, point_cloud)
            features = features + skip
        return point_cloud.format_output(features, return_sorted, return_padded)


class PointResNetBottleNeck(torch.nn.Module):
    """Residual blocks whose point convolution runs on fewer channels: 1x1 down,
    convolution, 1x1 up, each after batch normalisation and the activation
    (network_blocks.py:153-298)."""

    def __init__(self, num_features, bottle_neck_num_features, num_blocks, num_dims,
                 layer_type="MCConv", projection_shortcuts=False, activation=torch.relu,
                 device="cuda", **kwargs):
        super().__init__()
        self._num_dims, self._num_blocks, self._activation = num_dims, num_blocks, activation
        conv = layer_types[layer_type.lower()]
        inner = bottle_neck_num_features
        widths = (num_features, inner, inner)
        self._batch_norm_layers = torch.nn.ModuleList(
            BatchNorm(widths[j % 3], device=device) for j in range(3 * num_blocks))
        self._downsampling_layers = torch.nn.ModuleList(
            Conv1x1(num_features, inner, device=device, seed=200 + i) for i in range(num_blocks))
        self._conv_layers = torch.nn.ModuleList(
            conv(inner, inner, num_dims=num_dims, device=device, seed=i, **kwargs)
            for i in range(num_blocks))
        self._upsampling_layers = torch.nn.ModuleList(
            Conv1x1(inner, num_features, device=device, seed=300 + i) for i in range(num_blocks))
        self._projection_layers = torch.nn.ModuleList(
            Conv1x1(num_features, num_features, device=device, seed=100 + i)
            for i in range(num_blocks)) if projection_shortcuts else None

    def forward(self, features, point_cloud, radius, training=None, neighborhood=None,
                return_sorted=False, return_padded=False, **kwargs):
        features = point_cloud.flatten_features(features)
        if neighborhood is None:
            neighborhood = _own_neighborhood(point_cloud, radius, self._num_dims)
        bn, act = self._batch_norm_layers, self._activation
        for i in range(self._num_blocks):
            skip = features
            features = self._downsampling_layers[i](act(bn[3 * i](features, training)),
                                                    point_cloud)
            features = self._conv_layers[i](act(bn[3 * i + 1](features, training)), point_cloud,
                                            point_cloud, radius, neighborhood, **kwargs)
            features = self._upsampling_layers[i](act(bn[3 * i + 2](features, training)),
                                                  point_cloud)
            if self._projection_layers is not None:
                skip = self._projection_layers[i](skip, point_cloud)
            features = features + skip
        return point_cloud.format_output(features, return_sorted, return_padded)


class PointResNetSpatialBottleNeck(torch.nn.Module):
    """Residual blocks with a bottleneck in space: a convolution onto a
    down-sampled cloud, one inside it, one back onto the full cloud
    (network_blocks.py:300-465).  `conv_radii` holds the three radii in that
    order; `neighborhoods`, when given, the three matching neighbourhoods.  When
    the first and the last radius agree the way back is the transpose of the way
    down and no third search is made."""

    def __init__(self, num_features, num_blocks, num_dims, layer_type="MCConv",
                 projection_shortcuts=False, activation=torch.relu, device="cuda", **kwargs):
        super().__init__()
        self._num_dims, self._num_blocks, self._activation = num_dims, num_blocks, activation
        conv = layer_types[layer_type.lower()]
        self._batch_norm_layers = torch.nn.ModuleList(
            BatchNorm(num_features, device=device) for _ in range(3 * num_blocks))
        self._stage_layers = torch.nn.ModuleList(
            conv(num_features, num_features, num_dims=num_dims, device=device, seed=i, **kwargs)
            for i in range(3 * num_blocks))
        self._projection_layers = torch.nn.ModuleList(
            Conv1x1(num_features, num_features, device=device, seed=100 + i)
            for i in range(num_blocks)) if projection_shortcuts else None

    def forward(self, features, point_cloud, point_cloud_downsampled, conv_radii, training=None,
                neighborhoods=None, return_sorted=False, return_padded=False, **kwargs):
        features = point_cloud.flatten_features(features)
        radii = [float(r) for r in torch.as_tensor(conv_radii).reshape(-1).tolist()]
        if len(radii) != 3:
            raise ValueError("conv_radii holds three radii: down, inside, up")
        d, dev = self._num_dims, features.device
        if neighborhoods is None:
            vec = [pc._as_vector(r, d, dev) for r in radii]
            down = pc.Neighborhood(pc.Grid(point_cloud, vec[0]), vec[0], point_cloud_downsampled)
            inside = pc.Neighborhood(pc.Grid(point_cloud_downsampled, vec[1]), vec[1],
                                     point_cloud_downsampled)
            if radii[0] == radii[2]:
                up = down.transpose()
            else:
                up = pc.Neighborhood(pc.Grid(point_cloud_downsampled, vec[2]), vec[2],
                                     point_cloud)
            neighborhoods = [down, inside, up]
        clouds = [(point_cloud, point_cloud_downsampled),
                  (point_cloud_downsampled, point_cloud_downsampled),
                  (point_cloud_downsampled, point_cloud)]
        for i in range(self._num_blocks):
            skip = features
            for stage in range(3):
                j = 3 * i + stage
                features = self._activation(self._batch_norm_layers[j](features, training))
                features = self._stage_layers[j](features, clouds[stage][0], clouds[stage][1],
                                                 radii[stage], neighborhoods[stage], **kwargs)
            if self._projection_layers is not None:
                skip = self._projection_layers[i](skip, point_cloud)
            features = features + skip
        return point_cloud.format_output(features, return_sorted, return_padded)
