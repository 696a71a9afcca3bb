"""Convolution and pooling layers composed from the HIP ops, with the call
signatures of the reference's layers (pylib/pc/layers/MCConv.py, KPConv.py,
Pooling.py).  Per-pair basis evaluation, basis projection, pooling and all
their gradients are kernels of libmccnn_hip.so, and so are the dense
[N, C*K] x [C*K, C_out] product and its two gradient products for channel
counts that are multiples of 16 (other shapes of the dense products fall back to
torch.matmul inside `_final_product`, `_weight_grad_product` and
`_projection_grad_product`, nowhere else)."""
import math

import numpy as np
import torch

from . import _lib, pc, tfg_custom_ops
from .kernel_points import cube_kernel_points, spherical_kernel_points
from ._lib import cfloat, cint, i64, ptr, stream

_F32, _I32 = torch.float32, torch.int32

_ACTIVATIONS = {"relu": 0, "lrelu": 1, "leakyrelu": 1, "leaky_relu": 1, "elu": 2}


class _MCBasis(torch.autograd.Function):
    """basis[m, l*H + h] = act(delta_m . W[l,:,h] + b[l,h]) / pdf[m]
    (MCConv.py:163-171); differentiable in the kernel weights and biases."""

    @staticmethod
    def forward(ctx, weights, biases, points_in, points_out, neighbors, inv_radii, pdf, act):
        num_mlps, dims, hidden = weights.shape
        k = num_mlps * hidden
        basis = torch.empty((neighbors.shape[0], k), dtype=_F32, device=weights.device)
        _lib.call("mc_basis", stream(), i64(neighbors.shape[0]), cint(dims), cint(k), cint(act),
            ptr(points_in, _F32), ptr(points_out, _F32), ptr(neighbors, _I32),
            ptr(inv_radii, _F32), ptr(weights, _F32), ptr(biases, _F32), cint(num_mlps),
            ptr(pdf, _F32), ptr(basis))
        ctx.save_for_backward(weights, biases, points_in, points_out, neighbors, inv_radii, pdf)
        ctx.act = act
        return basis

    @staticmethod
    def backward(ctx, grad):
        weights, biases, points_in, points_out, neighbors, inv_radii, pdf = ctx.saved_tensors
        num_mlps, dims, hidden = weights.shape
        k = num_mlps * hidden
        L = _lib.lib()
        ws = _lib.workspace(L.mccnn_mc_basis_grads_workspace_bytes(cint(dims), cint(k)),
                            weights.device)
        dw, db = torch.empty_like(weights), torch.empty_like(biases)
        _lib.call("mc_basis_grads", stream(), i64(neighbors.shape[0]), cint(dims), cint(k), cint(ctx.act),
            ptr(points_in, _F32), ptr(points_out, _F32), ptr(neighbors, _I32),
            ptr(inv_radii, _F32), ptr(weights, _F32), ptr(biases, _F32), cint(num_mlps),
            ptr(pdf, _F32), ptr(grad.contiguous(), _F32), ptr(ws), _lib.csize(ws.numel()),
            ptr(dw), ptr(db))
        return dw, db, None, None, None, None, None, None


class _MCConvProject(torch.autograd.Function):
    """mc_basis followed by basis_proj in one kernel (the basis is evaluated in
    registers); differentiable in the kernel weights, biases and the features."""

    @staticmethod
    def forward(ctx, weights, biases, features, points_in, points_out, neighbors, ranges,
                inv_radii, pdf, act, transposed):
        num_mlps, dims, hidden = weights.shape
        k = num_mlps * hidden
        out = torch.empty((ranges.shape[0], features.shape[1], k), dtype=_F32,
                          device=features.device)
        _lib.call("mc_conv_project", stream(), cint(dims), i64(features.shape[0]),
                  ptr(points_in, _F32), cint(features.shape[1]), ptr(features, _F32),
                  i64(ranges.shape[0]), ptr(points_out, _F32), i64(neighbors.shape[0]),
                  ptr(neighbors, _I32), ptr(ranges, _I32), ptr(inv_radii, _F32), cint(k),
                  cint(num_mlps), cint(act), ptr(weights, _F32), ptr(biases, _F32),
                  ptr(pdf, _F32), ptr(None), ptr(out))
        ctx.save_for_backward(weights, biases, features, points_in, points_out, neighbors,
                              ranges, inv_radii, pdf)
        ctx.act, ctx.transposed = act, transposed
        return out

    @staticmethod
    def backward(ctx, grad):
        (weights, biases, features, points_in, points_out, neighbors, ranges, inv_radii,
         pdf) = ctx.saved_tensors
        num_mlps, dims, hidden = weights.shape
        k = num_mlps * hidden
        L = _lib.lib()
        ws = _lib.workspace(L.mccnn_mc_conv_project_grads_workspace_bytes(
            cint(dims), cint(k), i64(ranges.shape[0])), weights.device)
        dfeat = torch.empty_like(features)
        dw, db = torch.empty_like(weights), torch.empty_like(biases)
        t_ranges = t_order = rows = None
        if ctx.transposed is not None:
            t_ranges, t_order = ctx.transposed
            rows = torch.empty((neighbors.shape[0], features.shape[1]), dtype=_F32,
                               device=features.device)
        _lib.call("mc_conv_project_grads", stream(), cint(dims), i64(features.shape[0]),
                  ptr(points_in, _F32), cint(features.shape[1]), ptr(features, _F32),
                  i64(ranges.shape[0]), ptr(points_out, _F32), i64(neighbors.shape[0]),
                  ptr(neighbors, _I32), ptr(ranges, _I32), ptr(inv_radii, _F32), cint(k),
                  cint(num_mlps), cint(ctx.act), ptr(weights, _F32), ptr(biases, _F32),
                  ptr(pdf, _F32), ptr(grad.contiguous(), _F32), ptr(ws), _lib.csize(ws.numel()),
                  ptr(t_ranges), ptr(t_order), ptr(rows), ptr(dfeat), ptr(dw), ptr(db))
        return dw, db, dfeat, None, None, None, None, None, None, None, None


def _mc_project(weights, biases, features, points_in, points_out, neighbors, ranges, inv_radii,
                pdf, act, out_rows=None):
    num_mlps, dims, hidden = weights.shape
    k = num_mlps * hidden
    out = torch.empty((ranges.shape[0], features.shape[1], k), dtype=_F32,
                      device=features.device)
    _lib.call("mc_conv_project", stream(), cint(dims), i64(features.shape[0]),
              ptr(points_in, _F32), cint(features.shape[1]), ptr(features, _F32),
              i64(ranges.shape[0]), ptr(points_out, _F32), i64(neighbors.shape[0]),
              ptr(neighbors, _I32), ptr(ranges, _I32), ptr(inv_radii, _F32), cint(k),
              cint(num_mlps), cint(act), ptr(weights, _F32), ptr(biases, _F32),
              ptr(pdf, _F32), ptr(out_rows), ptr(out))
    return out


def _mc_layer(weights, biases, features, points_in, points_out, neighbors, ranges, inv_radii,
              pdf, act, dense_weights, out_rows=None, want_proj=False):
    """Fused projection + product with the dense [C*K, F] final weights; rows of the
    result (and of the projection, if asked for) go to `out_rows`."""
    num_mlps, dims, hidden = weights.shape
    k, c, f = num_mlps * hidden, features.shape[1], dense_weights.shape[1]
    out = torch.empty((ranges.shape[0], f), dtype=_F32, device=features.device)
    proj = None
    if want_proj:
        proj = torch.empty((ranges.shape[0], c, k), dtype=_F32, device=features.device)
    _lib.call("mc_conv_layer", stream(), cint(dims), i64(features.shape[0]),
              ptr(points_in, _F32), cint(c), ptr(features, _F32), i64(ranges.shape[0]),
              ptr(points_out, _F32), i64(neighbors.shape[0]), ptr(neighbors, _I32),
              ptr(ranges, _I32), ptr(inv_radii, _F32), cint(k), cint(num_mlps), cint(act),
              ptr(weights, _F32), ptr(biases, _F32), ptr(pdf, _F32), cint(f),
              ptr(dense_weights.contiguous(), _F32), ptr(out_rows), ptr(proj), ptr(out))
    return out, proj


def _gather_rows(x, rows):
    """x[rows] for x [N, C] and int32 row indices."""
    x = x.contiguous()
    if x.shape[1] % 4 != 0:
        return x.index_select(0, rows.long())
    out = torch.empty((rows.shape[0], x.shape[1]), dtype=_F32, device=x.device)
    _lib.call("gather_rows", stream(), i64(rows.shape[0]), cint(x.shape[1]), ptr(x, _F32),
              ptr(rows, _I32), ptr(out))
    return out


def _weight_grad_product(x, y):
    """x^T y for [N, C] and [N, R] operands with the long reduction over N."""
    c, r = x.shape[1], y.shape[1]
    L = _lib.lib()
    if not L.mccnn_weight_grad_product_supported(cint(c), cint(r)):
        with _lib.region("gemm_dfinal"):
            return x.t() @ y
    L.mccnn_weight_grad_product_workspace_bytes.restype = _lib.csize
    ws = _lib.workspace(L.mccnn_weight_grad_product_workspace_bytes(cint(c), cint(r)), x.device)
    out = torch.empty((c, r), dtype=_F32, device=x.device)
    _lib.call("weight_grad_product", stream(), i64(x.shape[0]), cint(c), ptr(x, _F32), cint(r),
              ptr(y, _F32), ptr(ws), _lib.csize(ws.numel()), ptr(out))
    return out


def _projection_grad_product(x, w):
    """x w^T for x [N, F] and w [R, F]."""
    f, r = x.shape[1], w.shape[0]
    if not _lib.lib().mccnn_projection_grad_product_supported(cint(f), cint(r)):
        with _lib.region("gemm_dproj"):
            return x @ w.t()
    out = torch.empty((x.shape[0], r), dtype=_F32, device=x.device)
    _lib.call("projection_grad_product", stream(), i64(x.shape[0]), cint(f), ptr(x, _F32),
              cint(r), ptr(w.contiguous(), _F32), ptr(out))
    return out


_cu_count = {}


def _compute_units(device):
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if idx not in _cu_count:
        _cu_count[idx] = torch.cuda.get_device_properties(idx).multi_processor_count
    return _cu_count[idx]


def _tiles(n, f):
    """Blocks of the tiled product: 128 x 128 tiles, 256 x 64 for odd multiples of 64."""
    return (n + 127) // 128 * (f // 128) if f % 128 == 0 else (n + 255) // 256 * (f // 64)


def _padded_columns(cols):
    """Output columns of a layer whose count the kernels do not cover, with zero columns
    added: a multiple of 16, and of 64 beyond 32 (the tiled product and the 64-channel
    kernels of the backward take 64 columns in less time than the blocked product takes 48:
    [825 274, 2048] x [2048, 48] 3.4 ms, x [2048, 64] 1.9 ms)."""
    return -(-cols // 64) * 64 if cols > 32 else -(-cols // 16) * 16


def _final_product(x, w):
    """x w for x [N, R] and the final weights w [R, F]."""
    r, f = w.shape
    L = _lib.lib()
    out = torch.empty((x.shape[0], f), dtype=_F32, device=x.device)
    # Weights beyond the registers of a block of wavefronts (R * F > 65536) take the tiled
    # product, which reads both operands along the reduction: w is handed over transposed
    # (a copy of at most a few MB).  Only when its 128-row tiles give every compute unit
    # one; smaller inputs take the register-resident product in blocks of w.  With the dense
    # products on the bf16 pipe the tiled kernel is also the faster one for smaller weights
    # once there are one and a half tiles per compute unit ([763 063, 1024] x [1024, 64]:
    # 0.82 against 0.93 ms inside the layer step; [30 000, 1024] x [1024, 64]: 0.087 against
    # 0.049 ms, which is why the register-resident float32 kernel keeps the small inputs).
    tiles, units = _tiles(x.shape[0], f), _compute_units(x.device)
    if L.mccnn_final_product_wt_supported(cint(r), cint(f)) and (
            (r * f > _TILED_ABOVE and tiles >= units) or
            (L.mccnn_split_products_enabled() and 2 * tiles >= 3 * units)):
        _lib.call("final_product_wt", stream(), i64(x.shape[0]), cint(r), ptr(x, _F32), cint(f),
                  ptr(w.t().contiguous(), _F32), ptr(None), ptr(out), timed_as="final_product")
        return out
    if not L.mccnn_final_product_supported(cint(r), cint(f)):
        with _lib.region("gemm_final"):
            return x @ w
    _lib.call("final_product", stream(), i64(x.shape[0]), cint(r), ptr(x, _F32), cint(f),
              ptr(w.contiguous(), _F32), ptr(None), ptr(out))
    return out


_TILED_ABOVE = 65536      # weights that fit the registers of a block of wavefronts


class _DenseProduct(torch.autograd.Function):
    """x w for x [N, R], w [R, F] on the library's dense kernels, differentiable in both:
    dx = dout w^T (projection-gradient product), dw = x^T dout (final-weight-gradient
    product); shapes the kernels do not cover fall back to torch inside the three helpers."""

    @staticmethod
    def forward(ctx, x, w):
        ctx.save_for_backward(x, w)
        return _final_product(x.contiguous(), w)

    @staticmethod
    def backward(ctx, dout):
        x, w = ctx.saved_tensors
        dout = dout.contiguous()
        dx = _projection_grad_product(dout, w.contiguous()) if ctx.needs_input_grad[0] else None
        # x^T dout with the reduction over the rows: the kernel takes the narrow operand first
        dw = None
        if ctx.needs_input_grad[1]:
            if _lib.lib().mccnn_weight_grad_product_supported(cint(dout.shape[1]), cint(x.shape[1])):
                dw = _weight_grad_product(dout, x.contiguous()).t()
            else:
                dw = _weight_grad_product(x.contiguous(), dout)
        return dx, dw


def _dense_product(x, w):
    return _DenseProduct.apply(x, w)


class _PairDense(torch.autograd.Function):
    """One layer of a kernel MLP per neighbour pair, y = act(x w + b) for x [M, I] with
    I, O <= 64 (MCConv.py:163-168, PointConv.py:168-190), forward and all gradients on the
    library's memory-bound kernels (mccnn_pair_dense, mccnn_pair_dense_grads)."""

    @staticmethod
    def forward(ctx, x, w, b, act):
        x, w = x.contiguous(), w.contiguous()
        ctx.bias_shape = None if b is None else tuple(b.shape)
        b = None if b is None else b.reshape(-1).contiguous()
        y = torch.empty((x.shape[0], w.shape[1]), dtype=_F32, device=x.device)
        _lib.call("pair_dense", stream(), i64(x.shape[0]), cint(w.shape[0]), ptr(x, _F32),
                  cint(w.shape[1]), ptr(w, _F32), ptr(b, _F32), cint(act), ptr(y))
        ctx.save_for_backward(x, w, y)
        ctx.act = act
        return y

    @staticmethod
    def backward(ctx, dy):
        x, w, y = ctx.saved_tensors
        rows, i, o = x.shape[0], w.shape[0], w.shape[1]
        L = _lib.lib()
        ws = _lib.workspace(L.mccnn_pair_dense_grads_workspace_bytes(i64(rows), cint(i), cint(o)),
                            x.device)
        dx = torch.empty_like(x) if ctx.needs_input_grad[0] else None
        dw = torch.empty_like(w)
        db = torch.empty(o, dtype=_F32, device=x.device) if ctx.bias_shape is not None else None
        _lib.call("pair_dense_grads", stream(), i64(rows), cint(i), ptr(x, _F32), cint(o),
                  ptr(w, _F32), ptr(y, _F32), ptr(dy.contiguous(), _F32), cint(ctx.act), ptr(ws),
                  _lib.csize(ws.numel()), ptr(dx), ptr(dw), ptr(db))
        return dx, dw, None if db is None else db.reshape(ctx.bias_shape), None


def _pair_dense(x, w, b, act):
    """act(x w + b) per pair; `act` -1 for none.  Widths beyond 64 take torch."""
    if w.shape[0] > 64 or w.shape[1] > 64:
        z = x @ w if b is None else x @ w + b.reshape(1, -1)
        return z if act < 0 else _activate(z, act)
    return _PairDense.apply(x, w, b, act)


def _dense_final_weights(final_weights, c):
    """[L, C*H, G] per-MLP blocks -> dense [C*(L*H), L*G] with zero off-diagonal blocks."""
    l, ch, g = final_weights.shape
    if l == 1:
        return final_weights[0]
    h = ch // c
    dense = torch.zeros((c, l, h, l, g), dtype=_F32, device=final_weights.device)
    blocks = final_weights.reshape(l, c, h, g)
    for i in range(l):
        dense[:, i, :, i, :] = blocks[i]
    return dense.reshape(c * l * h, l * g)


class _MCConvLayer(torch.autograd.Function):
    """The whole Monte-Carlo convolution (MCConv.py:137-194), run on the
    neighbourhood's grid-ordered view (features and output gradients are permuted
    into grid order once per pass so that the gathers of neighbouring centres hit
    in L2).  Forward: fused basis + projection, product with the final weights
    (inside the same kernel with `fuse_final`).  Backward: the feature gradient
    is the same convolution run from the centres back to the points over the
    transposed pair table (no scatter):
        Q[j, f, k]  = sum_{i in T(j)} basis[ij, k] dout[i, f]
        dfeat[j, c] = sum_{f,k} Q[j, f, k] W[c, k, f]
        dW[c, k, f] = sum_j feat[j, c] Q[j, f, k]
    and the kernel-MLP gradients come from dproj = dout W^T through the weight
    half of the fused projection backward."""

    @staticmethod
    def forward(ctx, weights, biases, final_weights, features, neighborhood, inv_radii, act,
                fuse_final):
        view = neighborhood.sorted_view()
        pdf, _ = view.pair_pdf(neighborhood)
        feats = _gather_rows(features, view.point_rows)
        dense = _dense_final_weights(final_weights, features.shape[1])
        if fuse_final:
            out, _ = _mc_layer(weights, biases, feats, view.points_in, view.points_out,
                               view.table, view.ranges, inv_radii, pdf, act, dense,
                               view.centre_rows)
        else:
            # rows of the projection go straight to the centres' original positions
            proj = _mc_project(weights, biases, feats, view.points_in, view.points_out,
                               view.table, view.ranges, inv_radii, pdf, act,
                               view.centre_rows)
            out = _final_product(proj.reshape(proj.shape[0], -1), dense)
        ctx.save_for_backward(weights, biases, final_weights, feats, features, inv_radii)
        ctx.neighborhood, ctx.act, ctx.fuse_final = neighborhood, act, fuse_final
        return out

    @staticmethod
    def backward(ctx, dout):
        weights, biases, final_weights, feats, features, inv_radii = ctx.saved_tensors
        nbh = ctx.neighborhood
        view = nbh.sorted_view()
        pdf, pdf_t = view.pair_pdf(nbh)
        l, dims, h = weights.shape
        k, n, c = l * h, view.ranges.shape[0], feats.shape[1]
        g = final_weights.shape[2]
        f = g * l
        if view.centre_rows is not None:
            dout = _gather_rows(dout, view.centre_rows)
        else:
            dout = dout.contiguous()
        dense = _dense_final_weights(final_weights, c)               # [C*K, F]
        # kernel-MLP gradients
        dproj = _projection_grad_product(dout, dense)
        L = _lib.lib()
        ws = _lib.workspace(L.mccnn_mc_conv_project_grads_workspace_bytes(
            cint(dims), cint(k), i64(n)), weights.device)
        dw, db = torch.empty_like(weights), torch.empty_like(biases)
        _lib.call("mc_conv_project_grads", stream(), cint(dims), i64(feats.shape[0]),
                  ptr(view.points_in, _F32), cint(c), ptr(feats, _F32), i64(n),
                  ptr(view.points_out, _F32), i64(view.table.shape[0]), ptr(view.table, _I32),
                  ptr(view.ranges, _I32), ptr(inv_radii, _F32), cint(k), cint(l), cint(ctx.act),
                  ptr(weights, _F32), ptr(biases, _F32), ptr(pdf, _F32), ptr(dproj, _F32),
                  ptr(ws), _lib.csize(ws.numel()), ptr(None), ptr(None), ptr(None), ptr(None),
                  ptr(dw), ptr(db))
        del dproj
        # feature and final-weight gradients from the transposed convolution
        w2 = dense.reshape(c, k, f).permute(2, 1, 0).reshape(f * k, c)
        neg = pc._negative(inv_radii)
        if ctx.fuse_final:
            # rows of Q and of dfeat go straight to the points' original positions
            dfeat, q = _mc_layer(weights, biases, dout, view.points_out, view.points_in,
                                 view.table_t, view.ranges_t, neg, pdf_t, ctx.act, w2,
                                 view.point_rows, want_proj=True)
            ddense = _weight_grad_product(features, q.reshape(features.shape[0], f * k))
        else:
            # rows of Q (and so of dfeat) go straight to the points' original positions
            q = _mc_project(weights, biases, dout, view.points_out, view.points_in,
                            view.table_t, view.ranges_t, neg, pdf_t, ctx.act, view.point_rows)
            dfeat = _final_product(q.reshape(q.shape[0], f * k), w2)
            ddense = _weight_grad_product(features, q.reshape(features.shape[0], f * k))
        ddense = ddense.reshape(c, f, k).permute(0, 2, 1)            # [C, K, F]
        if l == 1:
            dfinal = ddense.reshape(1, c * k, f)
        else:
            blocks = ddense.reshape(c, l, h, l, g)
            dfinal = torch.stack([blocks[:, i, :, i, :].reshape(c * h, g) for i in range(l)])
        return dw, db, dfinal, dfeat, None, None, None, None


def _truncated_normal(shape, std, generator, device):
    t = torch.empty(shape, dtype=_F32)
    torch.nn.init.trunc_normal_(t, mean=0.0, std=std, a=-2 * std, b=2 * std,
                                generator=generator)
    return t.to(device)


class MCConv(torch.nn.Module):
    """Monte-Carlo convolution (pylib/pc/layers/MCConv.py:35-278) with a
    one-hidden-layer kernel MLP per output group."""

    def __init__(self, num_features_in, num_features_out, num_dims, num_mlps=4, mlp_size=(8,),
                 non_linearity_type="leaky_relu", weights=None, biases=None,
                 final_weights=None, device="cuda", seed=0, fused=True, gathered_grads=True,
                 transposed_grads=True, fuse_final=False):
        super().__init__()
        if num_features_out % num_mlps != 0:
            raise ValueError("The number of output features must be divisible by the number"
                             " of kernel MLPs")
        if len(mlp_size) < 1:
            raise ValueError("mlp_size needs at least one layer")
        first, hidden = int(mlp_size[0]), int(mlp_size[-1])
        self._num_features_in, self._num_features_out = num_features_in, num_features_out
        self._num_dims, self._num_mlps, self._hidden = num_dims, num_mlps, hidden
        self._act = _ACTIVATIONS[non_linearity_type.lower()]
        gen = torch.Generator().manual_seed(seed)
        if weights is None:      # MCConv.py:100-135: truncated normal, He scale
            weights = _truncated_normal((num_mlps, num_dims, first),
                                        math.sqrt(2.0 / num_dims), gen, device)
        if biases is None:
            biases = torch.zeros((num_mlps, 1, first), dtype=_F32, device=device)
        # Kernel MLPs with further layers (MCConv.py:100-120: scale sqrt(1 / fan-in)):
        # the HIP kernels evaluate one-layer kernels in registers; deeper ones are
        # evaluated per pair with dense products and handed to basis_proj.
        self.deep_weights = torch.nn.ParameterList()
        self.deep_biases = torch.nn.ParameterList()
        for prev, cur in zip(mlp_size[:-1], mlp_size[1:]):
            self.deep_weights.append(torch.nn.Parameter(_truncated_normal(
                (num_mlps, int(prev), int(cur)), math.sqrt(1.0 / int(prev)), gen, device)))
            self.deep_biases.append(torch.nn.Parameter(
                torch.zeros((num_mlps, 1, int(cur)), dtype=_F32, device=device)))
        if final_weights is None:
            final_weights = _truncated_normal(
                (num_mlps, hidden * num_features_in, num_features_out // num_mlps),
                math.sqrt(2.0 / (hidden * num_features_in)), gen, device)
        self.weights = torch.nn.Parameter(weights.to(_F32).contiguous())
        self.biases = torch.nn.Parameter(biases.to(_F32).contiguous())
        self.final_weights = torch.nn.Parameter(final_weights.to(_F32).contiguous())
        self.last_neighborhood = None
        # evaluate the kernel MLP inside the projection kernel when the shape allows
        self.fused = fused
        # feature gradient by per-pair rows + ordered gather instead of float atomics
        self.gathered_grads = gathered_grads
        # feature gradient as a convolution over the transposed pair table (fused path)
        self.transposed_grads = transposed_grads
        # product with the final weights inside the projection kernel (out of LDS)
        self.fuse_final = fuse_final

    def forward(self, features, point_cloud_in, point_cloud_out, radius, neighborhood=None,
                bandwidth=0.2, return_sorted=False, return_padded=False):
        features = point_cloud_in.flatten_features(features)
        out = self._convolve(features, point_cloud_in, point_cloud_out, radius, neighborhood,
                             bandwidth)
        return point_cloud_out.format_output(out, return_sorted, return_padded)

    def _convolve_deep(self, features, point_cloud_in, point_cloud_out, radii, neighborhood,
                       pdf=None):
        """The layer as the reference composes it (MCConv.py:163-194), differentiable
        in everything: per-pair offsets through the layers of the kernel MLPs as
        batched dense products, divided by the densities, then basis_proj and the
        final product.  Used for kernel MLPs of several layers and for point
        clouds whose coordinates require a gradient; the [M, K] basis is
        materialised, as in the reference."""
        ids = neighborhood._original_neigh_ids.long()
        l, c, h = self._num_mlps, self._num_features_in, self._hidden
        diff = (point_cloud_in._points[ids[:, 0]] - point_cloud_out._points[ids[:, 1]]) / radii
        layers_w = [self.weights] + list(self.deep_weights)
        layers_b = [self.biases] + list(self.deep_biases)
        columns = []
        for mlp in range(l):             # every kernel MLP is a chain of per-pair layers
            cur = diff
            for w, b in zip(layers_w, layers_b):
                cur = _pair_dense(cur, w[mlp], b[mlp], self._act)
            columns.append(cur)
        pdf = neighborhood.get_pdf() if pdf is None else pdf
        basis = (columns[0] if l == 1 else torch.cat(columns, dim=1)) / pdf.reshape(-1, 1)
        proj = tfg_custom_ops.basis_proj(basis.contiguous(), features.contiguous(),
                                         neighborhood._original_neigh_ids,
                                         neighborhood._samples_neigh_ranges)
        n = proj.shape[0]
        if l == 1:
            return _dense_product(proj.reshape(n, c * h), self.final_weights[0])
        p = proj.reshape(n, c, l, h).permute(2, 0, 1, 3).reshape(l, n, c * h)
        return torch.cat([_dense_product(p[mlp].contiguous(), self.final_weights[mlp])
                          for mlp in range(l)], dim=1)

    def _convolve_on_view(self, features, neighborhood, radii, biases, k):
        """The fused path on the grid-ordered view; channel counts it does not cover
        are zero-padded (features, rows / columns of the final weights) and the
        result is cut back.  None if the shape is out of reach."""
        d, c, f, l, h = (self._num_dims, self._num_features_in, self._num_features_out,
                         self._num_mlps, self._hidden)
        if d not in (2, 3):
            return None
        # hidden units per kernel MLP padded with zero columns until the layer has 16, 32 or
        # 64 basis columns (every activation maps 0 to 0, and the rows of the final weights
        # that meet the padding are zero too): `MCConv(c, f, 3, 1, [8])` then runs on the
        # 16-column kernels
        h_pad = next((v // l for v in (16, 32, 64) if v % l == 0 and v // l >= h), None)
        pad = _layer_padding(c, f, l)
        if pad is None or h_pad is None:
            return None
        c_pad, g_pad = pad
        g = f // l
        weights = self.weights
        if h_pad != h:
            weights = torch.nn.functional.pad(weights, (0, h_pad - h))
            biases = torch.nn.functional.pad(biases, (0, h_pad - h))
            k = l * h_pad
        # the backward runs the same single-kernel layer transposed (output channels as its
        # input channels), so both directions have to be covered
        supported = _lib.lib().mccnn_mc_conv_layer_supported
        fuse_final = (self.fuse_final
                      and bool(supported(cint(d), cint(c_pad), cint(k), cint(g_pad * l)))
                      and bool(supported(cint(d), cint(g_pad * l), cint(k), cint(c_pad))))
        final = self.final_weights
        if c_pad != c or g_pad != g or h_pad != h:
            final = torch.nn.functional.pad(final.reshape(l, c, h, g),
                                            (0, g_pad - g, 0, h_pad - h, 0, c_pad - c))
            final = final.reshape(l, c_pad * h_pad, g_pad)
            features = torch.nn.functional.pad(features, (0, c_pad - c))
            h = h_pad
        inv_radii = pc._reciprocal(radii)
        per = 16 // h if h <= 16 and 16 % h == 0 else 0       # kernel MLPs per 16 basis columns
        if k > 16 and per > 0 and l % per == 0 and (per * g_pad) % 16 == 0:
            # Kernel MLPs do not share final weights (MCConv.py:180-194), so the layer is
            # l / per independent convolutions of 16 basis columns, each with its own
            # slice of the output: the dense products then cost l / per times less than on
            # the block-diagonal [C*K, F] matrix (default constructor, 4 x 8: 16.5 -> 12 ms
            # per step on the scene-scale batch).
            outs = [_MCConvLayer.apply(weights[t:t + per].contiguous(),
                                       biases[t:t + per].contiguous(), final[t:t + per],
                                       features, neighborhood, inv_radii, self._act, False)
                    for t in range(0, l, per)]
            out = torch.cat(outs, dim=1)
        else:
            out = _MCConvLayer.apply(weights.contiguous(), biases.contiguous(), final, features,
                                     neighborhood, inv_radii, self._act, fuse_final)
        if g_pad != g:
            out = out.reshape(-1, l, g_pad)[:, :, :g].reshape(-1, f)
        return out

    def _convolve(self, features, point_cloud_in, point_cloud_out, radius, neighborhood,
                  bandwidth):
        d = self._num_dims
        dev = features.device
        radii = pc._as_vector(radius, d, dev)
        if neighborhood is None:
            grid = pc.Grid(point_cloud_in, radii)
            neighborhood = pc.Neighborhood(grid, radii, point_cloud_out)
        self.last_neighborhood = neighborhood
        neighborhood.point_pdf(bandwidth=bandwidth, mode=pc.KDEMode.constant)
        moving = _moving(point_cloud_in, point_cloud_out)
        if len(self.deep_weights) > 0 or moving:
            pdf = _differentiable_pdf(neighborhood, bandwidth) if moving else None
            return self._convolve_deep(features, point_cloud_in, point_cloud_out, radii,
                                       neighborhood, pdf)
        biases = self.biases.reshape(self._num_mlps, self._hidden)
        k = self._num_mlps * self._hidden
        fused = self.fused and _lib.lib().mccnn_mc_conv_supported(
            cint(d), cint(self._num_features_in), cint(k))
        if self.fused and self.transposed_grads:
            out = self._convolve_on_view(features, neighborhood, radii, biases, k)
            if out is not None:
                return out
        pdf = neighborhood.get_pdf()
        transposed = None
        if self.gathered_grads and features.requires_grad and \
                tfg_custom_ops.gathered_grads_supported(self._num_features_in, k):
            transposed = neighborhood.transposed_pairs()
        if fused:
            proj = _MCConvProject.apply(self.weights, biases, features.contiguous(),
                                        point_cloud_in._points, point_cloud_out._points,
                                        neighborhood._original_neigh_ids,
                                        neighborhood._samples_neigh_ranges,
                                        pc._reciprocal(radii), pdf, self._act, transposed)
        else:
            basis = _MCBasis.apply(self.weights, biases, point_cloud_in._points,
                                   point_cloud_out._points, neighborhood._original_neigh_ids,
                                   pc._reciprocal(radii), pdf, self._act)
            proj = tfg_custom_ops.basis_proj(basis, features.contiguous(),
                                             neighborhood._original_neigh_ids,
                                             neighborhood._samples_neigh_ranges,
                                             neighborhood._centre_order, transposed)
        n, c, l, h = proj.shape[0], self._num_features_in, self._num_mlps, self._hidden
        if l == 1:
            return _dense_product(proj.reshape(n, c * h), self.final_weights[0])
        p = proj.reshape(n, c, l, h).permute(2, 0, 1, 3).reshape(l, n, c * h)
        return torch.cat([_dense_product(p[mlp].contiguous(), self.final_weights[mlp])
                          for mlp in range(l)], dim=1)


def _differentiable_pdf(neighborhood, bandwidth):
    """Per-pair densities as a function of the grid cloud's point coordinates
    (the gradient registered for ComputePdfWithPtGrads,
    custom_ops_wrapper.py:159-169), for point clouds whose coordinates require a
    gradient."""
    grid = neighborhood._grid
    points = grid._point_cloud._points
    d, dev = points.shape[1], points.device
    mode = pc.KDEMode.constant
    if neighborhood._pdf_args is not None:       # the settings of an earlier compute_pdf
        bandwidth, mode = neighborhood._pdf_args
    nb = neighborhood._neighbors
    if mode == pc.KDEMode.no_pdf:
        return torch.ones(nb.shape[0], dtype=_F32, device=dev)
    own = neighborhood if neighborhood._equal_samples else \
        grid.self_neighborhood(neighborhood._radii)
    per_point = tfg_custom_ops.compute_pdf_with_pt_grads(
        points[grid._sorted_indices.long()], own._neighbors, own._samples_neigh_ranges,
        pc._reciprocal(pc._as_vector(bandwidth, d, dev)), own._inv_radii,
        mode.value, symmetric=own._equal_samples and own.max_neighbors == 0)
    pdf = per_point[nb[:, 0].long()]
    if neighborhood._pdf_normalize:              # Neighborhood.py:288-293
        ends = neighborhood._samples_neigh_ranges.long()
        counts = (ends - torch.cat([ends.new_zeros(1), ends[:-1]])).to(_F32)
        pdf = pdf / counts[nb[:, 1].long()]
    return pdf


def _moving(*clouds):
    return any(c._points.requires_grad for c in clouds)


def _activate(x, act):
    if act == 0:
        return torch.relu(x)
    if act == 1:
        return torch.nn.functional.leaky_relu(x, 0.2)
    return torch.nn.functional.elu(x)


def _layer_padding(c, f, num_mlps):
    """Channel counts the grid-ordered layer path runs on, or None: C rounded up to
    16/32/64/128, and per kernel MLP as many output columns G' >= G as make the
    total a multiple of 16 (at most 512)."""
    c_pad = next((v for v in (16, 32, 64, 128) if v >= c), None)
    step = 16 // math.gcd(16, num_mlps)
    g = f // num_mlps
    g_pad = -(-g // step) * step
    if c_pad is None or g_pad * num_mlps > 512:
        return None
    return c_pad, g_pad


class _PointConvLayer(torch.autograd.Function):
    """PointConv (PointConv.py:143-202) on the neighbourhood's grid-ordered view with
    the kernels of the Monte-Carlo convolution: the transformed density of a pair,
        y = mlp(pdf[point] / max pdf of the centre's neighbourhood),
    is computed once per pair (forward and transposed order) and takes the place
    of the density in the fused projection, which runs on the unscaled offsets
    (unit radii).  Backward as for the Monte-Carlo convolution (transposed
    convolution for the features, no scatter); the gradient of the four density
    parameters comes from the per-pair gradient of the scale 1/y that the
    kernel-MLP backward returns beside the weight gradients."""

    @staticmethod
    def forward(ctx, weights, biases, final_weights, pw1, pb1, pw2, pb2, features,
                neighborhood, act):
        view = neighborhood.sorted_view()
        dev = features.device
        per_point = neighborhood._pdf_per_point.detach()
        m, dims = view.table.shape[0], weights.shape[1]
        max_pdf = torch.empty((view.ranges.shape[0], 1), dtype=_F32, device=dev)
        _lib.call("local_pool", stream(), cint(0), i64(per_point.shape[0]), cint(1),
                  ptr(per_point, _F32), i64(m), ptr(view.table, _I32),
                  i64(view.ranges.shape[0]), ptr(view.ranges, _I32), ptr(max_pdf))
        mlp = [t.detach().reshape(-1).contiguous() for t in (pw1, pb1, pw2, pb2)]

        def density(table, point_column):
            out = torch.empty(m, dtype=_F32, device=dev)
            _lib.call("pointconv_density", stream(), i64(m), ptr(table, _I32), cint(point_column),
                      ptr(per_point, _F32), ptr(max_pdf, _F32), ptr(mlp[0], _F32),
                      ptr(mlp[1], _F32), ptr(mlp[2], _F32), ptr(mlp[3], _F32), ptr(out))
            return out

        y = density(view.table, 0)
        y_t = density(view.table_t, 1)
        ones = torch.ones(dims, dtype=_F32, device=dev)
        feats = _gather_rows(features, view.point_rows)
        proj = _mc_project(weights, biases, feats, view.points_in, view.points_out, view.table,
                           view.ranges, ones, y, act, view.centre_rows)
        out = _final_product(proj.reshape(proj.shape[0], -1), final_weights[0])
        ctx.save_for_backward(weights, biases, final_weights, feats, features, per_point, max_pdf,
                              y, y_t, ones, *mlp)
        ctx.neighborhood, ctx.act = neighborhood, act
        return out

    @staticmethod
    def backward(ctx, dout):
        (weights, biases, final_weights, feats, features, per_point, max_pdf, y, y_t, ones,
         w1, b1, w2, b2) = ctx.saved_tensors
        view = ctx.neighborhood.sorted_view()
        dev = feats.device
        _, dims, k = weights.shape
        n, c, m = view.ranges.shape[0], feats.shape[1], view.table.shape[0]
        dense = final_weights[0]                                      # [C*K, F]
        f = dense.shape[1]
        if view.centre_rows is not None:
            dout = _gather_rows(dout, view.centre_rows)
        else:
            dout = dout.contiguous()
        # kernel-MLP gradients and, per pair, the gradient of the scale 1/y
        dproj = _projection_grad_product(dout, dense)
        L = _lib.lib()
        ws = _lib.workspace(L.mccnn_mc_conv_project_grads_workspace_bytes(
            cint(dims), cint(k), i64(n)), dev)
        dw, db = torch.empty_like(weights), torch.empty_like(biases)
        slabs = k // 16
        scale_grads = torch.empty((slabs, m), dtype=_F32, device=dev)
        _lib.call("mc_conv_weight_and_scale_grads", stream(), cint(dims), i64(feats.shape[0]),
                  ptr(view.points_in, _F32), cint(c), ptr(feats, _F32), i64(n),
                  ptr(view.points_out, _F32), i64(m), ptr(view.table, _I32),
                  ptr(view.ranges, _I32), ptr(ones, _F32), cint(k), cint(1), cint(ctx.act),
                  ptr(weights, _F32), ptr(biases, _F32), ptr(y, _F32), ptr(dproj, _F32),
                  ptr(ws), _lib.csize(ws.numel()), ptr(dw), ptr(db), ptr(scale_grads))
        del dproj
        ws2 = _lib.workspace(L.mccnn_pointconv_density_grads_workspace_bytes(i64(m)), dev)
        dmlp = torch.empty(49, dtype=_F32, device=dev)
        _lib.call("pointconv_density_grads", stream(), i64(m), ptr(view.table, _I32), cint(0),
                  ptr(per_point, _F32), ptr(max_pdf, _F32), ptr(w1, _F32), ptr(b1, _F32),
                  ptr(w2, _F32), ptr(b2, _F32), ptr(y, _F32), cint(slabs),
                  ptr(scale_grads, _F32), ptr(ws2), _lib.csize(ws2.numel()), ptr(dmlp))
        # feature and final-weight gradients from the transposed convolution
        q = _mc_project(weights, biases, dout, view.points_out, view.points_in, view.table_t,
                        view.ranges_t, -ones, y_t, ctx.act, view.point_rows)
        q = q.reshape(q.shape[0], f * k)
        dfeat = None
        if ctx.needs_input_grad[7]:
            w_t = dense.reshape(c, k, f).permute(2, 1, 0).reshape(f * k, c)
            dfeat = _final_product(q, w_t)
        ddense = _weight_grad_product(features, q).reshape(c, f, k).permute(0, 2, 1)
        dfinal = ddense.reshape(1, c * k, f)
        return (dw, db, dfinal, dmlp[0:16].reshape(1, 16), dmlp[16:32].reshape(1, 16),
                dmlp[32:48].reshape(16, 1), dmlp[48:49].reshape(1, 1), dfeat, None, None)


class PointConv(torch.nn.Module):
    """PointConv-style Monte-Carlo convolution (pylib/pc/layers/PointConv.py:34-292):
    one kernel MLP with a single hidden layer on the unscaled point offsets, the
    densities normalised by their maximum in each neighbourhood and passed
    through a 1 -> 16 -> 1 MLP before they divide the basis."""

    def __init__(self, num_features_in, num_features_out, num_dims, size_hidden=32,
                 non_linearity_type="relu", device="cuda", seed=0, weights=None, biases=None,
                 final_weights=None, pdf_weights=None, pdf_biases=None, fused=True):
        super().__init__()
        self.fused = fused
        if size_hidden not in (8, 16, 32):
            raise ValueError("size_hidden must be 8, 16 or 32")
        self._num_features_in, self._num_features_out = num_features_in, num_features_out
        self._num_dims, self._size_hidden = num_dims, size_hidden
        self._act = _ACTIVATIONS[non_linearity_type.lower()]
        gen = torch.Generator().manual_seed(seed)

        def glorot(fan_in, fan_out):          # GlorotNormal, PointConv.py:83-85
            return (torch.randn((fan_in, fan_out), generator=gen) *
                    math.sqrt(2.0 / (fan_in + fan_out))).to(device)

        def param(value, default):
            value = default() if value is None else torch.as_tensor(value).to(device)
            return torch.nn.Parameter(value.to(_F32).contiguous())

        self.weights = param(weights, lambda: glorot(num_dims, size_hidden))
        self.biases = param(biases, lambda: torch.zeros((1, size_hidden), device=device))
        self.final_weights = param(final_weights, lambda: glorot(size_hidden * num_features_in,
                                                                 num_features_out))
        pw = pdf_weights or (None, None)
        pb = pdf_biases or (None, None)
        self.pdf_weights_1 = param(pw[0], lambda: glorot(1, 16))
        self.pdf_weights_2 = param(pw[1], lambda: glorot(16, 1))
        self.pdf_biases_1 = param(pb[0], lambda: torch.zeros((1, 16), device=device))
        self.pdf_biases_2 = param(pb[1], lambda: torch.zeros((1, 1), device=device))
        self.last_neighborhood = None

    def forward(self, features, point_cloud_in, point_cloud_out, radius, neighborhood=None,
                bandwidth=0.2, return_sorted=False, return_padded=False):
        features = point_cloud_in.flatten_features(features)
        out = self._convolve(features, point_cloud_in, point_cloud_out, radius, neighborhood,
                             bandwidth)
        return point_cloud_out.format_output(out, return_sorted, return_padded)

    def _convolve_on_view(self, features, neighborhood, bandwidth):
        """The fused path on the grid-ordered view (channels zero-padded as for the
        Monte-Carlo convolution); None if the shape is out of its reach."""
        d, c, f, h = (self._num_dims, self._num_features_in, self._num_features_out,
                      self._size_hidden)
        pad = _layer_padding(c, f, 1)
        if not self.fused or d not in (2, 3) or pad is None:
            return None
        if neighborhood.point_pdf(bandwidth=bandwidth, mode=pc.KDEMode.constant) is None:
            return None
        c_pad, f_pad = pad
        h_pad = max(h, 16)       # 8 hidden units: zero columns (every activation maps 0 to 0)
        weights, biases = self.weights, self.biases
        final = self.final_weights.reshape(1, c * h, f)
        if h_pad != h:
            weights = torch.nn.functional.pad(weights, (0, h_pad - h))
            biases = torch.nn.functional.pad(biases, (0, h_pad - h))
        if c_pad != c or f_pad != f or h_pad != h:
            final = torch.nn.functional.pad(final.reshape(1, c, h, f),
                                            (0, f_pad - f, 0, h_pad - h, 0, c_pad - c))
            final = final.reshape(1, c_pad * h_pad, f_pad)
            features = torch.nn.functional.pad(features, (0, c_pad - c))
        h = h_pad
        out = _PointConvLayer.apply(weights.reshape(1, d, h), biases.reshape(1, h),
                                    final, self.pdf_weights_1, self.pdf_biases_1,
                                    self.pdf_weights_2, self.pdf_biases_2,
                                    features.contiguous(), neighborhood, self._act)
        return out[:, :f] if f_pad != f else out

    def _convolve(self, features, point_cloud_in, point_cloud_out, radius, neighborhood,
                  bandwidth):
        d, dev = self._num_dims, features.device
        radii = pc._as_vector(radius, d, dev)
        if neighborhood is None:
            grid = pc.Grid(point_cloud_in, radii)
            neighborhood = pc.Neighborhood(grid, radii, point_cloud_out)
        self.last_neighborhood = neighborhood
        ids, ranges = neighborhood._original_neigh_ids, neighborhood._samples_neigh_ranges
        m, n_out = ids.shape[0], ranges.shape[0]
        if _moving(point_cloud_in, point_cloud_out):
            # coordinates that require a gradient: the same expressions in torch
            pdf = _differentiable_pdf(neighborhood, bandwidth)
            diff = point_cloud_in._points[ids[:, 0].long()] - \
                point_cloud_out._points[ids[:, 1].long()]
            hidden = _pair_dense(diff, self.weights, self.biases, self._act)
        else:
            out = self._convolve_on_view(features, neighborhood, bandwidth)
            if out is not None:
                return out
            pdf = neighborhood.get_pdf(bandwidth=bandwidth, mode=pc.KDEMode.constant)
            # hidden layer on the unscaled offsets (PointConv.py:268-272): unit radii, unit pdf
            ones_d = torch.ones(d, dtype=_F32, device=dev)
            hidden = _MCBasis.apply(self.weights.reshape(1, d, self._size_hidden),
                                    self.biases.reshape(1, self._size_hidden),
                                    point_cloud_in._points, point_cloud_out._points, ids, ones_d,
                                    torch.ones(m, dtype=_F32, device=dev), self._act)
        # densities relative to the largest of their neighbourhood, then the pdf MLP
        # (PointConv.py:166-177)
        centre = ids[:, 1].long()
        max_pdf = torch.zeros(n_out, dtype=_F32, device=dev).scatter_reduce(
            0, centre, pdf, "amax", include_self=False)
        rel = (pdf / max_pdf[centre]).reshape(-1, 1)
        cur = _pair_dense(rel, self.pdf_weights_1, self.pdf_biases_1, 0)
        cur = _pair_dense(cur, self.pdf_weights_2, self.pdf_biases_2, -1)
        basis = hidden / cur
        proj = tfg_custom_ops.basis_proj(basis, features.contiguous(), ids, ranges)
        return _dense_product(proj.reshape(n_out, -1), self.final_weights)


def _padded_basis_count(num_kernel_points):
    """Basis columns for a kernel of this many points (KPConv.py:199-213 pads to 8,
    16, 32 or 64; 16 is the narrowest tile of the projection kernels, so kernels
    of up to 8 points are padded to 16 here, with zero columns either way)."""
    for k in (16, 32, 64):
        if num_kernel_points <= k:
            return k
    raise ValueError("at most 64 kernel points are supported")


class _KPBasis(torch.autograd.Function):
    """Kernel-point correlation weights per pair, zero-padded to `k` columns
    (KPConv.py:29-57, 193-213); differentiable in the per-centre offsets."""

    @staticmethod
    def forward(ctx, offsets, points_in, points_out, neighbors, ranges, inv_radii,
                kernel_points, k, kind, sigma):
        kp, dims = kernel_points.shape
        basis = torch.empty((neighbors.shape[0], k), dtype=_F32, device=points_in.device)
        _lib.call("kp_basis", stream(), i64(neighbors.shape[0]), cint(dims), cint(kp), cint(k),
                  cint(kind), cfloat(sigma), ptr(points_in, _F32), ptr(points_out, _F32),
                  ptr(neighbors, _I32), ptr(inv_radii, _F32), ptr(kernel_points, _F32),
                  ptr(offsets), ptr(basis), ptr(None))
        ctx.save_for_backward(offsets, points_in, points_out, neighbors, ranges, inv_radii,
                              kernel_points)
        ctx.k, ctx.kind, ctx.sigma = k, kind, sigma
        return basis

    @staticmethod
    def backward(ctx, grad):
        (offsets, points_in, points_out, neighbors, ranges, inv_radii,
         kernel_points) = ctx.saved_tensors
        if offsets is None:
            return (None,) * 10
        kp, dims = kernel_points.shape
        doff = torch.empty_like(offsets)
        _lib.call("kp_basis_grads", stream(), i64(neighbors.shape[0]), cint(dims), cint(kp),
                  cint(ctx.k), cint(ctx.kind), cfloat(ctx.sigma), ptr(points_in, _F32),
                  ptr(points_out, _F32), ptr(neighbors, _I32), i64(ranges.shape[0]),
                  ptr(ranges, _I32), ptr(inv_radii, _F32), ptr(kernel_points, _F32),
                  ptr(offsets, _F32), ptr(grad.contiguous(), _F32), ptr(doff))
        return (doff,) + (None,) * 9


class _KPRegularization(torch.autograd.Function):
    """sum(fit) + sum(repulsion) of the deformed kernel points (KPConv.py:394-429)."""

    @staticmethod
    def forward(ctx, offsets, points_in, points_out, neighbors, ranges, inv_radii,
                kernel_points, kind, sigma):
        kp, dims = kernel_points.shape
        n_out = ranges.shape[0]
        fit = torch.empty((n_out, kp), dtype=_F32, device=offsets.device)
        rep = torch.empty((n_out, kp), dtype=_F32, device=offsets.device)
        argmin = torch.empty((n_out, kp), dtype=_I32, device=offsets.device)
        _lib.call("kp_regularization", stream(), i64(neighbors.shape[0]), cint(dims), cint(kp),
                  cint(kind), cfloat(sigma), ptr(points_in, _F32), ptr(points_out, _F32),
                  ptr(neighbors, _I32), i64(n_out), ptr(ranges, _I32), ptr(inv_radii, _F32),
                  ptr(kernel_points, _F32), ptr(offsets, _F32), ptr(fit), ptr(argmin), ptr(rep))
        ctx.save_for_backward(offsets, points_in, points_out, neighbors, inv_radii,
                              kernel_points, argmin)
        ctx.kind, ctx.sigma = kind, sigma
        return fit.sum() + rep.sum()

    @staticmethod
    def backward(ctx, grad):
        offsets, points_in, points_out, neighbors, inv_radii, kernel_points, argmin = \
            ctx.saved_tensors
        kp, dims = kernel_points.shape
        doff = torch.empty_like(offsets)
        _lib.call("kp_regularization_grads", stream(), i64(neighbors.shape[0]), cint(dims),
                  cint(kp), cint(ctx.kind), cfloat(ctx.sigma), cfloat(1.0),
                  ptr(points_in, _F32), ptr(points_out, _F32), ptr(neighbors, _I32),
                  i64(offsets.shape[0]), ptr(inv_radii, _F32), ptr(kernel_points, _F32),
                  ptr(offsets, _F32), ptr(argmin, _I32), ptr(doff))
        return (doff * grad,) + (None,) * 8


def _kp_basis_raw(points_in, points_out, neighbors, inv_radii, kernel_points, k, kind, sigma):
    kp, dims = kernel_points.shape
    basis = torch.empty((neighbors.shape[0], k), dtype=_F32, device=points_in.device)
    _lib.call("kp_basis", stream(), i64(neighbors.shape[0]), cint(dims), cint(kp), cint(k),
              cint(kind), cfloat(sigma), ptr(points_in, _F32), ptr(points_out, _F32),
              ptr(neighbors, _I32), ptr(inv_radii, _F32), ptr(kernel_points, _F32), ptr(None),
              ptr(basis), ptr(None))
    return basis


def _kp_project(features, points_in, points_out, neighbors, ranges, inv_radii, kernel_points, k,
                kind, sigma, out_rows=None):
    """Kernel-point weights + projection -> [N_out, C, k]: one kernel (weights in
    registers) when the shape is covered, else kp_basis followed by basis_proj."""
    kp, dims = kernel_points.shape
    c = features.shape[1]
    if k in (16, 32) and _lib.lib().mccnn_mc_conv_project_supported(cint(dims), cint(c), cint(k)):
        out = torch.empty((ranges.shape[0], c, k), dtype=_F32, device=features.device)
        _lib.call("kp_conv_project", stream(), cint(dims), i64(features.shape[0]),
                  ptr(points_in, _F32), cint(c), ptr(features, _F32), i64(ranges.shape[0]),
                  ptr(points_out, _F32), i64(neighbors.shape[0]), ptr(neighbors, _I32),
                  ptr(ranges, _I32), ptr(inv_radii, _F32), cint(kp), ptr(kernel_points, _F32),
                  cint(kind), cfloat(sigma), ptr(out_rows), ptr(out))
        return out
    basis = _kp_basis_raw(points_in, points_out, neighbors, inv_radii, kernel_points, k, kind,
                          sigma)
    out = tfg_custom_ops._basis_proj_raw(basis, features, neighbors, ranges)
    if out_rows is not None:
        out = torch.empty_like(out).index_copy_(0, out_rows.long(), out)
    return out


class _KPConvRigidLayer(torch.autograd.Function):
    """Rigid kernel-point convolution (KPConv.py:165-232) on the neighbourhood's
    grid-ordered view.  As for the Monte-Carlo convolution, the feature gradient is
    the same convolution run from the centres back to the points over the
    transposed pair table, with the kernel-point weights re-evaluated there
    (offset negated), and the weight gradient is feat^T Q; nothing is scattered and
    the basis gradient, which a rigid kernel does not need, is never formed."""

    @staticmethod
    def forward(ctx, dense_weights, features, neighborhood, inv_radii, kernel_points, k, kind,
                sigma, rows_in_view_order):
        view = neighborhood.sorted_view()
        feats = _gather_rows(features, view.point_rows)
        # rows of the projection go straight to the centres' original positions (or stay
        # in the view's order, for a consumer that works on the view itself)
        proj = _kp_project(feats, view.points_in, view.points_out, view.table, view.ranges,
                           inv_radii, kernel_points, k, kind, sigma,
                           None if rows_in_view_order else view.centre_rows)
        out = _final_product(proj.reshape(proj.shape[0], -1), dense_weights)
        ctx.save_for_backward(dense_weights, feats, features, inv_radii, kernel_points)
        ctx.neighborhood, ctx.k, ctx.kind, ctx.sigma = neighborhood, k, kind, sigma
        ctx.rows_in_view_order = rows_in_view_order
        return out

    @staticmethod
    def backward(ctx, dout):
        dense, feats, features, inv_radii, kernel_points = ctx.saved_tensors
        view = ctx.neighborhood.sorted_view()
        k, c, f = ctx.k, feats.shape[1], dense.shape[1]
        if view.centre_rows is not None and not ctx.rows_in_view_order:
            dout = _gather_rows(dout, view.centre_rows)
        else:
            dout = dout.contiguous()
        # rows of Q (and so of dfeat) go straight to the points' original positions
        q = _kp_project(dout, view.points_out, view.points_in, view.table_t, view.ranges_t,
                        pc._negative(inv_radii), kernel_points, k, ctx.kind, ctx.sigma,
                        view.point_rows)
        q = q.reshape(feats.shape[0], f * k)
        dfeat = ddense = None
        if ctx.needs_input_grad[1]:
            w2 = dense.reshape(c, k, f).permute(2, 1, 0).reshape(f * k, c)
            dfeat = _final_product(q, w2)
        if ctx.needs_input_grad[0]:
            ddense = _weight_grad_product(features, q).reshape(c, f, k).permute(0, 2, 1)
            ddense = ddense.reshape(c * k, f)
        return ddense, dfeat, None, None, None, None, None, None, None


def _kp_deform_project(features, points_in, points_out, neighbors, ranges, inv_radii,
                       kernel_points, kind, sigma, offsets, offsets_follow_points, out_rows=None):
    """Projection with per-centre kernel-point offsets -> [N_out, C, 16]."""
    kp, dims = kernel_points.shape
    c = features.shape[1]
    out = torch.empty((ranges.shape[0], c, 16), dtype=_F32, device=features.device)
    _lib.call("kp_deform_project", stream(), cint(dims), i64(features.shape[0]),
              ptr(points_in, _F32), cint(c), ptr(features, _F32), i64(ranges.shape[0]),
              ptr(points_out, _F32), i64(neighbors.shape[0]), ptr(neighbors, _I32),
              ptr(ranges, _I32), ptr(inv_radii, _F32), cint(kp), ptr(kernel_points, _F32),
              cint(kind), cfloat(sigma), ptr(offsets, _F32), cint(1 if offsets_follow_points else 0),
              ptr(out_rows), ptr(out))
    return out


class _KPConvDeformLayer(torch.autograd.Function):
    """Deformable kernel-point convolution (KPConv.py:317-392) on the neighbourhood's
    grid-ordered view, given the per-centre offsets in the view's centre order.  The
    kernel-point weights are evaluated in registers in the forward projection, in the
    transposed projection that yields the feature and weight gradients (there the
    offsets belong to the gathered side of a pair), and in the offset-gradient kernel,
    which forms the basis gradient tile by tile from dproj = dout W^T; the [M, K] basis
    and its gradient never reach memory and nothing is scattered."""

    @staticmethod
    def forward(ctx, dense_weights, offsets, features, neighborhood, inv_radii, kernel_points,
                kind, sigma):
        view = neighborhood.sorted_view()
        feats = _gather_rows(features, view.point_rows)
        offsets = offsets.contiguous()
        proj = _kp_deform_project(feats, view.points_in, view.points_out, view.table,
                                  view.ranges, inv_radii, kernel_points, kind, sigma, offsets,
                                  False, view.centre_rows)
        out = _final_product(proj.reshape(proj.shape[0], -1), dense_weights)
        ctx.save_for_backward(dense_weights, offsets, feats, features, inv_radii, kernel_points)
        ctx.neighborhood, ctx.kind, ctx.sigma = neighborhood, kind, sigma
        return out

    @staticmethod
    def backward(ctx, dout):
        dense, offsets, feats, features, inv_radii, kernel_points = ctx.saved_tensors
        view = ctx.neighborhood.sorted_view()
        kp, dims = kernel_points.shape
        k, c, f = 16, feats.shape[1], dense.shape[1]
        n_out = view.ranges.shape[0]
        if view.centre_rows is not None:
            dout = _gather_rows(dout, view.centre_rows)
        else:
            dout = dout.contiguous()
        dfeat = ddense = doff = None
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[2]:
            q = _kp_deform_project(dout, view.points_out, view.points_in, view.table_t,
                                   view.ranges_t, pc._negative(inv_radii), kernel_points, ctx.kind, ctx.sigma,
                                   offsets, True, view.point_rows)
            q = q.reshape(feats.shape[0], f * k)
            if ctx.needs_input_grad[2]:
                w2 = dense.reshape(c, k, f).permute(2, 1, 0).reshape(f * k, c)
                dfeat = _final_product(q, w2)
            if ctx.needs_input_grad[0]:
                ddense = _weight_grad_product(features, q).reshape(c, f, k).permute(0, 2, 1)
                ddense = ddense.reshape(c * k, f)
        if ctx.needs_input_grad[1]:
            dproj = _projection_grad_product(dout, dense)            # [N_out, C*16]
            doff = torch.empty((n_out, kp, dims), dtype=_F32, device=dout.device)
            _lib.call("kp_deform_offset_grads", stream(), cint(dims), i64(feats.shape[0]),
                      ptr(view.points_in, _F32), cint(c), ptr(feats, _F32), i64(n_out),
                      ptr(view.points_out, _F32), i64(view.table.shape[0]),
                      ptr(view.table, _I32), ptr(view.ranges, _I32), ptr(inv_radii, _F32),
                      cint(kp), ptr(kernel_points, _F32), cint(ctx.kind), cfloat(ctx.sigma),
                      ptr(offsets, _F32), ptr(dproj, _F32), ptr(doff))
        return ddense, doff, dfeat, None, None, None, None, None


class KPConv(torch.nn.Module):
    """Kernel-point convolution, rigid or deformable
    (pylib/pc/layers/KPConv.py:60-429).  The kernel points are one of the
    spherical layouts, randomly rotated (seeded), or `custom_kernel_points`
    [K, D] in units of the convolution radius (required when num_dims != 3,
    :117-128); either is scaled by 0.75 as in the reference (:131).  With
    `deformable=True` a rigid kernel-point convolution predicts a per-centre
    offset for every kernel point (:317-392) and `regularization_loss()` returns
    the fitting + repulsive loss (:394-429)."""

    def __init__(self, num_features_in, num_features_out, num_kernel_points=15, num_dims=3,
                 deformable=False, kp_interpolation="linear", custom_kernel_points=None,
                 weights=None, offset_weights=None, device="cuda", seed=0,
                 transposed_grads=True):
        super().__init__()
        if custom_kernel_points is None:
            if num_dims != 3:
                raise ValueError("For dimension not 3 custom kernel points must be provided!")
            custom_kernel_points = spherical_kernel_points(
                num_kernel_points, rotate=True, rng=np.random.default_rng(seed))
        kp = torch.as_tensor(np.asarray(custom_kernel_points, dtype=np.float32)).to(device) * 0.75
        self._kernel_points = kp.contiguous()
        self._num_kernel_points = kp.shape[0]
        self._num_basis = _padded_basis_count(kp.shape[0])
        self._kind = {"linear": 0, "gaussian": 1}[kp_interpolation]
        self._num_features_in, self._num_features_out = num_features_in, num_features_out
        self._num_dims = num_dims
        gen = torch.Generator().manual_seed(seed)

        def glorot(fan_in, fan_out):      # Glorot normal as KPConv.py:133-160
            return (torch.randn((fan_in, fan_out), generator=gen) *
                    math.sqrt(2.0 / (fan_in + fan_out))).to(device)

        fan_in = self._num_kernel_points * num_features_in
        if weights is None:
            weights = glorot(fan_in, num_features_out)
        self.weights = torch.nn.Parameter(weights.to(_F32).contiguous())
        self.deformable = deformable
        # rigid kernels: feature gradient as a convolution over the transposed pair table
        self.transposed_grads = transposed_grads
        if deformable:
            if offset_weights is None:
                offset_weights = glorot(fan_in, self._num_kernel_points * num_dims)
            self.offset_weights = torch.nn.Parameter(offset_weights.to(_F32).contiguous())
        self.last_neighborhood = None
        self._last = None
        self.last_offsets = None      # [N_out, K, D] offsets of the last deformable call

    def _padded(self, w):
        """[C*KP, F] -> [C*K, F] with zero rows for the padded basis columns."""
        c, kp, k = self._num_features_in, self._num_kernel_points, self._num_basis
        if k == kp:
            return w
        return torch.nn.functional.pad(w.reshape(c, kp, -1), (0, 0, 0, k - kp)).reshape(c * k, -1)

    def forward(self, features, point_cloud_in, point_cloud_out, conv_radius, neighborhood=None,
                kernel_influence_dist=None, return_sorted=False, return_padded=False):
        features = point_cloud_in.flatten_features(features)
        out = self._convolve(features, point_cloud_in, point_cloud_out, conv_radius,
                             neighborhood, kernel_influence_dist)
        return point_cloud_out.format_output(out, return_sorted, return_padded)

    def _convolve(self, features, point_cloud_in, point_cloud_out, conv_radius, neighborhood,
                  kernel_influence_dist):
        d, dev = self._num_dims, features.device
        sigma = 1.0 if kernel_influence_dist is None else float(kernel_influence_dist) / float(
            conv_radius)
        radii = pc._as_vector(conv_radius, d, dev)
        if neighborhood is None:
            grid = pc.Grid(point_cloud_in, radii)
            neighborhood = pc.Neighborhood(grid, radii, point_cloud_out)
        self.last_neighborhood = neighborhood
        kp, k, c = self._num_kernel_points, self._num_basis, self._num_features_in
        features = features.contiguous()
        if _moving(point_cloud_in, point_cloud_out):
            return self._convolve_moving(features, point_cloud_in, point_cloud_out, radii,
                                         neighborhood, sigma)
        if not self.deformable and self.transposed_grads:
            return _KPConvRigidLayer.apply(self._padded(self.weights), features, neighborhood,
                                           pc._reciprocal(radii), self._kernel_points, k,
                                           self._kind, sigma, False)
        if self.deformable and self.transposed_grads and k == 16 and d in (2, 3) and \
                _lib.lib().mccnn_kp_deform_offset_grads_supported(cint(d), cint(c)):
            return self._convolve_deformed_on_view(features, neighborhood, radii, sigma)
        ids, ranges = neighborhood._original_neigh_ids, neighborhood._samples_neigh_ranges
        transposed = None
        if features.requires_grad and tfg_custom_ops.gathered_grads_supported(c, k):
            transposed = neighborhood.transposed_pairs()
        geometry = (point_cloud_in._points, point_cloud_out._points, ids, ranges,
                    pc._reciprocal(radii), self._kernel_points)

        def project(basis):
            return tfg_custom_ops.basis_proj(basis, features, ids, ranges,
                                             neighborhood._centre_order, transposed)

        offsets = None
        if self.deformable:       # KPConv.py:317-392: offsets from a rigid convolution
            w_off = self._padded(self.offset_weights)
            if self.transposed_grads and k in (16, 32):
                # the rigid layer's kernels, output columns padded (45 -> 64)
                cols = kp * d
                w_off = torch.nn.functional.pad(w_off, (0, _padded_columns(cols) - cols))
                offsets = _KPConvRigidLayer.apply(w_off, features, neighborhood,
                                                  pc._reciprocal(radii), self._kernel_points, k,
                                                  self._kind, sigma, False)[:, :cols]
            else:
                rigid = _KPBasis.apply(None, *geometry, k, self._kind, sigma)
                offsets = _dense_product(project(rigid).reshape(-1, c * k), w_off)
            offsets = offsets.reshape(-1, kp, d).contiguous()
        self._last = (offsets, geometry, sigma)
        self.last_offsets = offsets
        basis = _KPBasis.apply(offsets, *geometry, k, self._kind, sigma)
        return _dense_product(project(basis).reshape(-1, c * k), self._padded(self.weights))

    def _convolve_deformed_on_view(self, features, neighborhood, radii, sigma):
        """KPConv.py:317-392 on the grid-ordered view: a rigid convolution predicts the
        offsets (rows in the caller's centre order, `last_offsets`), which are brought
        into the view's centre order for the deformed convolution and for the
        regularisation loss."""
        kp, k, d = self._num_kernel_points, self._num_basis, self._num_dims
        view = neighborhood.sorted_view()
        inv_radii = pc._reciprocal(radii)
        cols = kp * d
        w_off = torch.nn.functional.pad(self._padded(self.offset_weights),
                                        (0, _padded_columns(cols) - cols))
        offsets = _KPConvRigidLayer.apply(w_off, features, neighborhood, inv_radii,
                                          self._kernel_points, k, self._kind, sigma,
                                          False)[:, :cols]
        offsets = offsets.reshape(-1, kp, d)
        self.last_offsets = offsets
        on_view = offsets if view.centre_order is None else \
            offsets.index_select(0, view.centre_order)
        on_view = on_view.contiguous()
        geometry = (view.points_in, view.points_out, view.table, view.ranges, inv_radii,
                    self._kernel_points)
        self._last = (on_view, geometry, sigma)
        # output columns padded to a multiple of 16 (the transposed projection runs on them)
        f = self._num_features_out
        dense = torch.nn.functional.pad(self._padded(self.weights), (0, -f % 16))
        out = _KPConvDeformLayer.apply(dense, on_view, features, neighborhood, inv_radii,
                                       self._kernel_points, self._kind, sigma)
        return out[:, :f] if f % 16 else out

    def _convolve_moving(self, features, point_cloud_in, point_cloud_out, radii, neighborhood,
                         sigma):
        """KPConv.py:165-232, 317-392 with the kernel-point correlation written in
        torch, for point clouds whose coordinates require a gradient (the norm is
        taken with a floor of 1e-10 so that a point sitting on a kernel point has
        a finite gradient)."""
        kp, k, c, d = self._num_kernel_points, self._num_basis, self._num_features_in, \
            self._num_dims
        ids, ranges = neighborhood._original_neigh_ids, neighborhood._samples_neigh_ranges
        centre = ids[:, 1].long()
        diff = (point_cloud_in._points[ids[:, 0].long()] - point_cloud_out._points[centre]) / radii

        def correlation(offsets):
            delta = diff[:, None, :] - self._kernel_points[None]
            if offsets is not None:
                delta = delta - offsets[centre]
            dist = torch.sqrt((delta * delta).sum(dim=2) + 1e-20)
            if self._kind == 0:
                wgt = torch.relu(1.0 - dist / sigma)
            else:
                wgt = torch.exp(-(dist / (sigma / 3.0)) ** 2)
            return torch.nn.functional.pad(wgt, (0, k - kp)).contiguous()

        def project(basis):
            return tfg_custom_ops.basis_proj(basis, features, ids, ranges).reshape(-1, c * k)

        offsets = None
        if self.deformable:
            offsets = _dense_product(project(correlation(None)), self._padded(self.offset_weights))
            offsets = offsets.reshape(-1, kp, d)
        self._last = None
        self.last_offsets = offsets
        if self.deformable:
            geometry = (point_cloud_in._points.detach(), point_cloud_out._points.detach(), ids,
                        ranges, pc._reciprocal(radii), self._kernel_points)
            self._last = (offsets, geometry, sigma)
        return _dense_product(project(correlation(offsets)), self._padded(self.weights))

    def regularization_loss(self):
        """Fitting + repulsive loss of the last deformable call (KPConv.py:394-429)."""
        if not self.deformable or self._last is None:
            raise RuntimeError("regularization_loss needs a preceding deformable forward pass")
        offsets, geometry, sigma = self._last
        return _KPRegularization.apply(offsets, *geometry, self._kind, sigma)


class _LocalPool(torch.autograd.Function):
    @staticmethod
    def forward(ctx, features, neighbors, ranges, kind):
        out = torch.empty((ranges.shape[0], features.shape[1]), dtype=_F32,
                          device=features.device)
        _lib.call("local_pool", stream(), cint(kind), i64(features.shape[0]), cint(features.shape[1]),
            ptr(features, _F32), i64(neighbors.shape[0]), ptr(neighbors, _I32),
            i64(ranges.shape[0]), ptr(ranges, _I32), ptr(out))
        ctx.save_for_backward(features, neighbors, ranges, out)
        ctx.kind = kind
        return out

    @staticmethod
    def backward(ctx, grad):
        features, neighbors, ranges, out = ctx.saved_tensors
        dfeat = torch.empty_like(features)
        _lib.call("local_pool_grads", stream(), cint(ctx.kind), i64(features.shape[0]), cint(features.shape[1]),
            ptr(features, _F32), i64(neighbors.shape[0]), ptr(neighbors, _I32),
            i64(ranges.shape[0]), ptr(ranges, _I32), ptr(out, _F32),
            ptr(grad.contiguous(), _F32), ptr(dfeat))
        return dfeat, None, None, None


class _LocalPointPooling:
    kind = 0

    def __call__(self, features, point_cloud_in, point_cloud_out, pooling_radius,
                 neighborhood=None, return_sorted=False, return_padded=False):
        features = point_cloud_in.flatten_features(features)
        if neighborhood is None:
            radii = pc._as_vector(pooling_radius, point_cloud_in._dimension, features.device)
            grid = pc.Grid(point_cloud_in, radii)
            neighborhood = pc.Neighborhood(grid, radii, point_cloud_out)
        if point_cloud_out is None:          # centres of a self-neighbourhood: the sorted points
            point_cloud_out = neighborhood._point_cloud_sampled
        out = _LocalPool.apply(features.contiguous(), neighborhood._original_neigh_ids,
                               neighborhood._samples_neigh_ranges, self.kind)
        return point_cloud_out.format_output(out, return_sorted, return_padded)


class MaxPooling(_LocalPointPooling):
    """pylib/pc/layers/Pooling.py:169-206."""
    kind = 0


class AveragePooling(_LocalPointPooling):
    """pylib/pc/layers/Pooling.py:209-246."""
    kind = 1


class _GlobalPool(torch.autograd.Function):
    @staticmethod
    def forward(ctx, features, batch_ids, batch_size, kind):
        out = torch.empty((batch_size, features.shape[1]), dtype=_F32, device=features.device)
        counts = torch.empty(batch_size, dtype=_I32, device=features.device)
        _lib.call("global_pool", stream(), cint(kind), i64(features.shape[0]), cint(features.shape[1]),
            ptr(features, _F32), ptr(batch_ids, _I32), cint(batch_size), ptr(out), ptr(counts))
        ctx.save_for_backward(features, batch_ids, out, counts)
        ctx.kind, ctx.batch_size = kind, batch_size
        return out

    @staticmethod
    def backward(ctx, grad):
        features, batch_ids, out, counts = ctx.saved_tensors
        dfeat = torch.empty_like(features)
        tie = torch.empty_like(out) if ctx.kind == 0 else None
        _lib.call("global_pool_grads", stream(), cint(ctx.kind), i64(features.shape[0]), cint(features.shape[1]),
            ptr(features, _F32), ptr(batch_ids, _I32), cint(ctx.batch_size), ptr(out, _F32),
            ptr(counts, _I32), ptr(grad.contiguous(), _F32), ptr(tie), ptr(dfeat))
        return dfeat, None, None, None


class GlobalMaxPooling:
    """pylib/pc/layers/Pooling.py:25-61."""

    def __call__(self, features, point_cloud, return_padded=False):
        features = point_cloud.flatten_features(features)
        out = _GlobalPool.apply(features.contiguous(), point_cloud._batch_ids,
                                point_cloud._batch_size, 0)
        if return_padded and point_cloud._batch_shape is not None:   # Pooling.py:58-61
            out = out.reshape(tuple(point_cloud._batch_shape) + (-1,))
        return out


class GlobalAveragePooling:
    """pylib/pc/layers/Pooling.py:64-104."""

    def __call__(self, features, point_cloud, return_padded=False):
        features = point_cloud.flatten_features(features)
        out = _GlobalPool.apply(features.contiguous(), point_cloud._batch_ids,
                                point_cloud._batch_size, 1)
        if return_padded and point_cloud._batch_shape is not None:   # Pooling.py:101-104
            out = out.reshape(tuple(point_cloud._batch_shape) + (-1,))
        return out
