"""Float64 restatements of the reference's layer compositions that need gradients.
TEST INFRASTRUCTURE ONLY (same rule as mccnn_oracle.py: tests, the smoke check and the
cpu-baseline leg of the benchmark may import this module; the product never does).

Written with torch in float64 so that torch.autograd differentiates them; every
function works on whatever device its arguments live on (the CPU tests pin them on the
CPU with hand-computed cases, the GPU tests evaluate the same functions on the device
for speed).  Each function follows the reference lines it cites:

* kernel-point correlation            pylib/pc/layers/KPConv.py:29-57
* basis projection                    custom_ops/.../basis_proj_kernels.cu.cc:29-116,
                                      pylib/pc/custom_ops/custom_ops_tf.py:423-446
* rigid / deformable KPConv           pylib/pc/layers/KPConv.py:165-232, 317-392
* regularisation loss                 pylib/pc/layers/KPConv.py:394-429
* PointConv density transform, layer  pylib/pc/layers/PointConv.py:143-202
"""
import numpy as np
import torch

FLT_MAX = float(np.finfo(np.float32).max)


def kp_weight(dist, sigma, kind):
    """KPConv.py:29-57: linear relu(1 - d / sigma), Gaussian exp(-(d / (sigma / 3))^2)."""
    if kind == "linear":
        return torch.relu(1.0 - dist / sigma)
    if kind == "gaussian":
        return torch.exp(-(dist / (sigma / 3.0)) ** 2)
    raise ValueError("kind must be 'linear' or 'gaussian'")


def project(basis, features, pairs, n_out):
    """basis_proj: out[i, c, k] = sum over the pairs (j, i) of features[j, c] * basis[m, k]
    (custom_ops_tf.py:423-446).  pairs: int64 [M, 2] rows (point, centre)."""
    c, k = features.shape[1], basis.shape[1]
    rows = features[pairs[:, 0]][:, :, None] * basis[:, None, :]
    return torch.zeros((n_out, c, k), dtype=basis.dtype, device=basis.device).index_add(
        0, pairs[:, 1], rows)


def kp_distances(delta, pairs, kernel_points, offsets=None):
    """KPConv.py:193-197: |delta[m] - (kp[k] + offsets[centre(m), k])| for every pair and
    kernel point, [M, K].  `kernel_points` already carry the reference's scaling
    (KPConv.py:131); `offsets` is [N_out, K, D] or None (rigid)."""
    kp = kernel_points[None]
    if offsets is not None:
        kp = kp + offsets[pairs[:, 1]]
    return (delta[:, None, :] - kp).norm(dim=2)


def kp_conv(delta, pairs, n_out, features, kernel_points, weights, sigma, kind, offsets=None):
    """KPConv.py:165-232: correlation -> basis_proj -> [N, C*K] x [C*K, C_out].
    Returns (output [N_out, C_out], distances [M, K])."""
    dist = kp_distances(delta, pairs, kernel_points, offsets)
    proj = project(kp_weight(dist, sigma, kind), features, pairs, n_out)
    return proj.reshape(n_out, -1) @ weights, dist


def kp_offsets(delta, pairs, n_out, features, kernel_points, offset_weights, sigma, kind):
    """KPConv.py:317-392: the offsets of a deformable layer are a rigid convolution with
    K*D outputs, reshaped to [N_out, K, D]."""
    k, d = kernel_points.shape
    out, _ = kp_conv(delta, pairs, n_out, features, kernel_points, offset_weights, sigma, kind)
    return out.reshape(n_out, k, d)


def kp_regularization_loss(dist, pairs, n_out, kernel_points, offsets, sigma, kind,
                           empty_value=FLT_MAX):
    """KPConv.py:394-429.  Fitting term: per centre and kernel point the minimum over the
    centre's pairs of (dist / sigma)^2, summed (tf.math.unsorted_segment_min: a centre
    without pairs contributes the largest float32, `empty_value`).  Repulsion: the
    correlation of every ordered pair of distinct deformed kernel points of a centre,
    summed (the diagonal is set to zero, each unordered pair therefore counts twice).
    Returns (fit_sum, repulsion_sum)."""
    k = kernel_points.shape[0]
    sq = (dist / sigma) ** 2
    index = pairs[:, 1][:, None].expand(-1, k)
    fit = torch.full((n_out, k), float("inf"), dtype=dist.dtype, device=dist.device)
    fit = fit.scatter_reduce(0, index, sq, "amin")
    fit = torch.where(torch.isinf(fit), torch.full_like(fit, empty_value), fit)
    moved = kernel_points[None] + offsets                       # [N_out, K, D]
    # (the 1e-300 keeps the norm differentiable on the diagonal, which is masked out)
    between = (moved[:, None] - moved[:, :, None] + 1e-300).norm(dim=3)
    off_diagonal = 1.0 - torch.eye(k, dtype=dist.dtype, device=dist.device)
    rep = kp_weight(between, sigma, kind) * off_diagonal[None]
    return fit.sum(), rep.sum()


def pointconv_density(pdf_pair, pairs, n_out, pw1, pb1, pw2, pb2):
    """PointConv.py:176-190: density of a pair relative to the largest density in its
    centre's neighbourhood, through the 1 -> 16 -> 1 network (relu hidden layer).
    Returns (transformed density [M, 1], relative density [M, 1])."""
    top = torch.zeros(n_out, dtype=pdf_pair.dtype, device=pdf_pair.device).scatter_reduce(
        0, pairs[:, 1], pdf_pair, "amax", include_self=False)
    rel = (pdf_pair / top[pairs[:, 1]]).reshape(-1, 1)
    return torch.relu(rel @ pw1 + pb1) @ pw2 + pb2, rel


def point_conv(diff, pairs, n_out, features, pdf_pair, weights, biases, final_weights,
               pw1, pb1, pw2, pb2, activation):
    """PointConv.py:143-202: act(diff W + b) / density transform -> basis_proj -> final
    product.  `diff` is NOT divided by the radius (PointConv.py:268-272).
    Returns (output, basis [M, H], transformed density [M, 1], relative density)."""
    hidden = activation(diff @ weights + biases)
    cur, rel = pointconv_density(pdf_pair, pairs, n_out, pw1, pb1, pw2, pb2)
    basis = hidden / cur
    proj = project(basis, features, pairs, n_out)
    return proj.reshape(n_out, -1) @ final_weights, basis, cur, rel
