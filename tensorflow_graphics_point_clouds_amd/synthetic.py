"""Seeded synthetic inputs for the benchmark and parity configurations.

Every generator is numpy-only, takes a seed (``1000 + configuration id`` by
default) and returns fp32 points and int32 batch ids in cloud order.  ``scale``
shrinks the point counts so the same shapes can be used in CPU-sized tests.
"""
import numpy as np

from .kernel_points import spherical_kernel_points


def _batch_ids(sizes):
    return np.repeat(np.arange(len(sizes), dtype=np.int32), sizes)


def truncated_normal(rng, shape, std):
    """Normal(0, std) re-drawn outside two standard deviations."""
    x = rng.standard_normal(shape)
    bad = np.abs(x) > 2.0
    while bad.any():
        x[bad] = rng.standard_normal(int(bad.sum()))
        bad = np.abs(x) > 2.0
    return (x * std).astype(np.float32)


def mcconv_weights(rng, num_dims, c_in, c_out, hidden=16, num_mlps=1):
    """Kernel-MLP and output weights with the reference's initial scale
    (pylib/pc/layers/MCConv.py:100-135)."""
    w = truncated_normal(rng, (num_mlps, num_dims, hidden), np.sqrt(2.0 / num_dims))
    b = np.zeros((num_mlps, 1, hidden), dtype=np.float32)
    wo = truncated_normal(rng, (num_mlps, hidden * c_in, c_out // num_mlps),
                          np.sqrt(2.0 / (hidden * c_in)))
    return w, b, wo


def uniform_clouds(batch, points_per_cloud, dims=3, seed=0):
    rng = np.random.default_rng(seed)
    pts = rng.random((batch * points_per_cloud, dims), dtype=np.float32)
    return pts, _batch_ids([points_per_cloud] * batch)


def config1(seed=1001):
    """2 x 1024 uniform points, 8 -> 16 channels, radius 0.1."""
    rng = np.random.default_rng(seed)
    pts = rng.random((2048, 3), dtype=np.float32)
    bids = _batch_ids([1024, 1024])
    feat = rng.standard_normal((2048, 8)).astype(np.float32)
    w, b, wo = mcconv_weights(rng, 3, 8, 16, hidden=16)
    return dict(points=pts, batch_ids=bids, batch_size=2, features=feat, weights=w,
                biases=b, final_weights=wo, radius=0.1, bandwidth=0.2)


def _random_rotation(rng):
    q, r = np.linalg.qr(rng.standard_normal((3, 3)))
    q = q * np.sign(np.diag(r))
    if np.linalg.det(q) < 0:
        q[:, 0] = -q[:, 0]
    return q


def _primitive(rng, n, kind=None):
    if kind is None:
        kind = rng.integers(0, 4)
    if kind == 0:      # sphere
        v = rng.standard_normal((n, 3))
        p = v / np.linalg.norm(v, axis=1, keepdims=True)
    elif kind == 1:    # box surface, area-uniform
        half = rng.uniform(0.5, 1.0, 3)
        area = np.array([half[1] * half[2], half[0] * half[2], half[0] * half[1]])
        face = rng.choice(3, size=n, p=area / area.sum())
        p = rng.uniform(-1, 1, (n, 3)) * half
        sign = rng.choice([-1.0, 1.0], size=n)
        p[np.arange(n), face] = sign * half[face]
    elif kind == 2:    # torus
        big, small = 1.0, rng.uniform(0.2, 0.5)
        u = rng.uniform(0, 2 * np.pi, n)
        # rejection sampling for area-uniformity in the minor angle
        v = np.empty(n)
        filled = 0
        while filled < n:
            cand = rng.uniform(0, 2 * np.pi, n)
            keep = cand[rng.uniform(0, 1, n) < (big + small * np.cos(cand)) / (big + small)]
            take = min(n - filled, len(keep))
            v[filled:filled + take] = keep[:take]
            filled += take
        p = np.stack([(big + small * np.cos(v)) * np.cos(u),
                      (big + small * np.cos(v)) * np.sin(u), small * np.sin(v)], axis=1)
    else:              # capped cylinder
        rad, half = rng.uniform(0.3, 1.0), rng.uniform(0.3, 1.0)
        side, cap = 2 * np.pi * rad * 2 * half, 2 * np.pi * rad * rad
        on_side = rng.uniform(0, 1, n) < side / (side + cap)
        ang = rng.uniform(0, 2 * np.pi, n)
        rr = np.where(on_side, rad, rad * np.sqrt(rng.uniform(0, 1, n)))
        z = np.where(on_side, rng.uniform(-half, half, n),
                     rng.choice([-half, half], size=n))
        p = np.stack([rr * np.cos(ang), rr * np.sin(ang), z], axis=1)
    p = p * rng.uniform(0.5, 1.0) @ _random_rotation(rng).T
    p = p - p.mean(axis=0)
    return p / np.linalg.norm(p, axis=1).max()


def config2(seed=1002, batch=16, points_per_cloud=1024):
    """ModelNet-shaped clouds: points on random primitives in the unit sphere."""
    rng = np.random.default_rng(seed)
    pts = np.concatenate([_primitive(rng, points_per_cloud) for _ in range(batch)])
    return dict(points=pts.astype(np.float32),
                batch_ids=_batch_ids([points_per_cloud] * batch), batch_size=batch,
                radii=(0.1, 0.2, 0.4), channels=(3, 64, 128, 256))


def labelled_primitives(count, points_per_cloud=1024, seed=0):
    """A four-class stand-in for a shape-classification set: `count` clouds of
    points on spheres, boxes, tori and cylinders (class 0..3) of random size and
    orientation inside the unit sphere -> (points [count, P, 3], labels [count])."""
    rng = np.random.default_rng(seed)
    labels = rng.integers(0, 4, count)
    pts = np.stack([_primitive(rng, points_per_cloud, int(k)) for k in labels])
    return pts.astype(np.float32), labels.astype(np.int64)


def config3(seed=1003, scale=1.0, batch=8):
    """Scene-scale clustered clouds of uneven size; radius 0.15.

    Per cloud: 20 Gaussian blobs inside a 10 x 10 x 3 box plus 10 % uniform
    noise.  The blob spread is 0.05 of the box extent per axis (0.5, 0.5, 0.15):
    that is the reading under which radius 0.15 gives the stated mean of about 30
    neighbours; an absolute spread of 0.05 would put thousands of points inside
    every radius and overflow the int32 pair offsets of the op contract."""
    rng = np.random.default_rng(seed)
    sizes = rng.integers(int(50000 * scale), int(150000 * scale) + 1, size=batch)
    box = np.array([10.0, 10.0, 3.0])
    chunks = []
    for n in sizes:
        centres = rng.uniform(0, 1, (20, 3)) * box
        n_noise = n // 10
        n_blob = n - n_noise
        which = rng.integers(0, 20, n_blob)
        blob = centres[which] + 0.05 * box * rng.standard_normal((n_blob, 3))
        noise = rng.uniform(0, 1, (n_noise, 3)) * box
        p = np.concatenate([blob, noise])
        chunks.append(p[rng.permutation(n)])
    pts = np.concatenate(chunks).astype(np.float32)
    return dict(points=pts, batch_ids=_batch_ids(sizes), batch_size=batch, radius=0.15,
                c_in=64, c_out=64, hidden=16, sizes=sizes)


def config4(seed=1004, scale=1.0, batch=4):
    """Dense uniform clouds; radii 0.02 / 0.04 / 0.06; C=128, K=32."""
    n = int(200000 * scale)
    pts, bids = uniform_clouds(batch, n, 3, seed)
    return dict(points=pts, batch_ids=bids, batch_size=batch, radii=(0.02, 0.04, 0.06),
                c_in=128, basis=32)


def config5(seed=1005, scale=1.0, batch=8):
    """KPConv on the scene-scale geometry: 15 kernel points at 0.6 r, 128 -> 128."""
    cfg = config3(seed=seed, scale=scale, batch=batch)
    cfg.update(c_in=128, c_out=128, kernel_points=spherical_kernel_points(15, rotate=False) * 0.6)
    return cfg
