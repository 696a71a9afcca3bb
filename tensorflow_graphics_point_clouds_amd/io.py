"""Point-cloud file loaders (pylib/io/points.py:24-222): ASCII files with one
point per line, `x,y,z[,features...]`, and the vertices of Wavefront .obj
meshes.  Parsing is host work; the batch loaders return torch tensors on the
requested device, zero-padded to the largest cloud, with the per-cloud sizes."""
import os

import numpy as np
import torch


def _check_file(filename):
    if not isinstance(filename, str):
        raise TypeError("'filename' must be of type 'string'")
    if not os.path.exists(filename):
        raise FileNotFoundError(f"No such file: {filename}")


def load_points_from_file_to_numpy(filename, delimiter=",", dimension=3, max_num_points=None,
                                   dtype=np.float32):
    """-> (points [N, dimension], features [N, columns - dimension]); at most
    `max_num_points` lines are read, all of them when it is None
    (points.py:72-120)."""
    _check_file(filename)
    rows = []
    with open(filename, "r") as handle:
        for line in handle:
            if max_num_points is not None and len(rows) >= max_num_points:
                break
            line = line.strip()
            if line:
                rows.append(line.split(delimiter))
    if not rows:
        return np.zeros((0, dimension), dtype), np.zeros((0, 0), dtype)
    width = len(rows[0])
    if any(len(r) != width for r in rows):
        raise ValueError(f"{filename}: lines differ in their number of columns")
    table = np.asarray(rows, dtype=np.float64).astype(dtype)
    return table[:, :dimension], table[:, dimension:]


def load_points_from_file_to_tensor(filename, delimiter=",", dimension=3, dtype=torch.float32,
                                    device="cpu"):
    """points.py:24-69, as torch tensors."""
    pts, feat = load_points_from_file_to_numpy(filename, delimiter, dimension, None, np.float64)
    return (torch.as_tensor(pts).to(dtype).to(device), torch.as_tensor(feat).to(dtype).to(device))


def _pad_and_stack(arrays, batch_shape, dtype, device):
    sizes = [len(a) for a in arrays]
    batch = len(arrays)
    shape = list(batch_shape)
    if shape != [-1] and int(np.prod(shape)) != batch:
        raise ValueError(f"Invalid batch shape {batch_shape} for batch size {batch}")
    if shape == [-1]:
        shape = [batch]
    v, width = max(sizes) if sizes else 0, arrays[0].shape[1] if arrays else 0
    out = np.zeros((batch, v, width), dtype=np.float64)
    for i, a in enumerate(arrays):
        out[i, :len(a)] = a
    out = torch.as_tensor(out).to(dtype).to(device).reshape(shape + [v, width])
    return out, torch.as_tensor(sizes, dtype=torch.int32, device=device).reshape(shape)


def load_batch_of_points(filenames, batch_shape=(-1,), delimiter=",", point_dimension=3,
                         dtype=torch.float32, device="cpu"):
    """-> (points [A1..An, V, D1], features [A1..An, V, D2], sizes [A1..An])
    (points.py:123-177)."""
    loaded = [load_points_from_file_to_numpy(f, delimiter, point_dimension, None, np.float64)
              for f in filenames]
    pts, sizes = _pad_and_stack([p for p, _ in loaded], batch_shape, dtype, device)
    feat, _ = _pad_and_stack([f for _, f in loaded], batch_shape, dtype, device)
    return pts, feat, sizes


def load_obj_vertices(filename, dtype=np.float32):
    """The `v x y z` records of a Wavefront .obj file, in file order, [N, 3].
    No vertex merging or other mesh processing is applied."""
    _check_file(filename)
    rows = []
    with open(filename, "r") as handle:
        for line in handle:
            if line.startswith("v ") or line.startswith("v\t"):
                rows.append(line.split()[1:4])
    return np.asarray(rows, dtype=np.float64).reshape(-1, 3).astype(dtype)


def load_batch_of_meshes(filenames, batch_shape=(-1,), file_type=None, dtype=torch.float32,
                         device="cpu"):
    """-> (points [A1..An, V, 3], sizes [A1..An]) from the vertices of mesh files
    (points.py:180-222).  Only the .obj format is read."""
    for f in filenames:
        kind = (file_type or os.path.splitext(f)[1].lstrip(".")).lower()
        if kind != "obj":
            raise ValueError(f"unsupported mesh file type '{kind}': only obj is read")
    return _pad_and_stack([load_obj_vertices(f, np.float64) for f in filenames], batch_shape,
                          dtype, device)
