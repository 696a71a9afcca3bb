"""Kernel-point layouts for the kernel-point convolution
(pylib/pc/layers/utils.py:52-238), as numpy arrays in units of the convolution
radius.  The layers scale them by 0.75 (pylib/pc/layers/KPConv.py:131)."""
import numpy as np

_SUPPORTED = (5, 7, 13, 15, 18)
_POLES = np.array([[0.0, 0.0, 0.0], [0.0, 0.0, 1.0], [0.0, 0.0, -1.0]])


def _ring(rows, scale, height):
    pts = np.asarray(rows, dtype=np.float64) * scale
    pts[:, 2] += height
    return pts


def _hexagon(scale, height):
    # utils.py:79-100.  The sixth row repeats the fourth instead of closing the
    # ring at (-0.5, -h); kept, because it is the data the reference convolves with.
    h = np.sqrt(3.0) / 2.0
    return _ring([[0, 1, 0], [0, -1, 0], [0.5, h, 0], [0.5, -h, 0], [-0.5, h, 0], [0.5, -h, 0]],
                 scale, height)


def _pentagon(scale, height):
    # utils.py:103-124
    c1, c2 = (np.sqrt(5.0) - 1.0) / 4.0, (np.sqrt(5.0) + 1.0) / 4.0
    s1, s2 = np.sqrt(10.0 + 2.0 * np.sqrt(5.0)) / 4.0, np.sqrt(10.0 - 2.0 * np.sqrt(5.0)) / 4.0
    return _ring([[1, 0, 0], [c1, s1, 0], [c1, -s1, 0], [-c2, s2, 0], [-c2, -s2, 0]],
                 scale, height)


def random_rotation(points, rng=None):
    """Rotates [N, 3] points by three angles drawn uniformly from [0, 2 pi), one
    per axis, composed as x, then y, then z (utils.py:52-76)."""
    rng = np.random.default_rng() if rng is None else rng
    ax, ay, az = rng.uniform(0.0, 2.0 * np.pi, 3)

    def about(axis, angle):
        c, s = np.cos(angle), np.sin(angle)
        m = np.eye(3)
        i, j = [(1, 2), (2, 0), (0, 1)][axis]
        m[i, i], m[i, j], m[j, i], m[j, j] = c, s, -s, c
        return m

    rot = about(0, ax) @ about(1, ay) @ about(2, az)
    return (np.asarray(points, dtype=np.float64) @ rot).astype(np.float32)


def spherical_kernel_points(num_points, rotate=True, rng=None):
    """[num_points, 3] kernel points of the unit sphere: centre plus the
    vertices of a tetrahedron (5), octahedron (7), icosahedron (13), two
    hexagons and the poles (15), three pentagons and the poles (18)
    (utils.py:149-222).  The icosahedron is not normalised, as in the reference."""
    if num_points not in _SUPPORTED:
        raise ValueError("KPConv currently only supports kernel sizes [5, 7, 13, 15, 18]")
    if num_points == 5:
        a, b, c = np.sqrt(8.0 / 9.0), np.sqrt(2.0 / 9.0), np.sqrt(2.0 / 3.0)
        pts = np.array([[0, 0, 0], [0, 0, 1], [a, 0, -1 / 3], [-b, c, -1 / 3], [-b, -c, -1 / 3]])
    elif num_points == 7:
        pts = np.concatenate([np.zeros((1, 3)), np.eye(3)[[0, 0, 1, 1, 2, 2]] *
                              np.array([1, -1, 1, -1, 1, -1])[:, None]])
    elif num_points == 13:
        g = (1.0 + np.sqrt(5.0)) / 2.0
        pts = np.array([[0, 0, 0],
                        [0, 1, g], [0, 1, -g], [0, -1, g], [0, -1, -g],
                        [1, g, 0], [1, -g, 0], [-1, g, 0], [-1, -g, 0],
                        [g, 0, 1], [-g, 0, 1], [g, 0, -1], [-g, 0, -1]])
    elif num_points == 15:
        h = np.sqrt(3.0) / 2.0
        # second ring: mirrored, x and y exchanged (a quarter turn about z)
        pts = np.concatenate([_POLES, _hexagon(0.5, h), _hexagon(-0.5, h)[:, [1, 0, 2]]])
    else:
        r = 1.0 / np.sqrt(2.0)
        pts = np.concatenate([_POLES, _pentagon(r, 0.5), -_pentagon(1.0, 0.0), _pentagon(-r, 0.5)])
    pts = pts.astype(np.float32)
    return random_rotation(pts, rng) if rotate else pts


def cube_kernel_points(cbrt_num_points):
    """[cbrt_num_points^3, 3] regular lattice of the unit cube (utils.py:225-238;
    `meshgrid` order: y varies slowest, then x, then z)."""
    t = np.linspace(0.0, 1.0, cbrt_num_points)
    x, y, z = np.meshgrid(t, t, t)
    return np.stack((x.ravel(), y.ravel(), z.ravel()), axis=1).astype(np.float32)
