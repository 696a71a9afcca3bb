"""Host-side logic of PointCloud (no GPU, no native library): the padded and
sizes-based constructors, sizes, unflattening and per-cloud access, following the
cases of the reference's point_cloud_test.py (flatten -> unflatten round trip,
construction from sizes, batch-shape handling)."""
import numpy as np
import pytest
import torch

from tensorflow_graphics_point_clouds_amd import pc


def test_padded_input_is_flattened_with_sizes():
    rng = np.random.default_rng(0)
    pts = rng.random((3, 5, 3)).astype(np.float32)
    sizes = [5, 2, 4]
    cloud = pc.PointCloud(pts, sizes=sizes)
    assert cloud._batch_size == 3 and cloud._dimension == 3
    expect = np.concatenate([pts[b, :n] for b, n in enumerate(sizes)])
    assert np.array_equal(cloud._points.numpy(), expect)
    assert cloud._batch_ids.tolist() == [0] * 5 + [1] * 2 + [2] * 4
    assert cloud.get_sizes().tolist() == sizes
    back = cloud.get_points()
    assert back.shape == (3, 5, 3)
    for b, n in enumerate(sizes):
        assert np.array_equal(back[b, :n].numpy(), pts[b, :n])
        assert float(back[b, n:].abs().sum()) == 0.0
        assert np.array_equal(cloud.get_points(b).numpy(), pts[b, :n])


def test_padded_input_without_sizes_and_with_batch_shape():
    pts = torch.arange(2 * 2 * 3 * 2, dtype=torch.float32).reshape(2, 2, 3, 2)
    cloud = pc.PointCloud(pts)
    assert cloud._batch_size == 4 and cloud._points.shape == (12, 2)
    assert cloud.get_sizes().shape == (2, 2) and int(cloud.get_sizes().sum()) == 12
    assert torch.equal(cloud.get_points(), pts)
    assert torch.equal(cloud.get_points((1, 0)), pts[1, 0])
    assert cloud.get_points(max_num_points=5).shape == (2, 2, 5, 2)


def test_segmented_input_from_sizes_and_unsorted_batch_ids():
    rng = np.random.default_rng(1)
    pts = rng.random((7, 2)).astype(np.float32)
    cloud = pc.PointCloud(pts, sizes=[3, 0, 4])
    assert cloud._batch_ids.tolist() == [0, 0, 0, 2, 2, 2, 2] and cloud._batch_size == 3
    ids = np.array([2, 0, 1, 0, 2, 2, 1], np.int32)
    cloud = pc.PointCloud(pts, ids)
    assert cloud.get_sizes().tolist() == [2, 2, 3]
    padded = cloud.get_points()
    assert padded.shape == (3, 3, 2)
    assert np.array_equal(padded[0, :2].numpy(), pts[[1, 3]])
    assert np.array_equal(padded[2].numpy(), pts[[0, 4, 5]])
    feats = torch.arange(7, dtype=torch.float32).reshape(7, 1)
    assert cloud.get_unflatten()(feats)[1, :, 0].tolist() == [2.0, 6.0, 0.0]
    cloud.set_batch_shape((3, 1))
    assert cloud.get_points().shape == (3, 1, 3, 2)
    with pytest.raises(ValueError):
        cloud.set_batch_shape((2, 2))


def test_invalid_point_cloud_inputs_raise():
    pts = np.zeros((4, 3), np.float32)
    with pytest.raises(ValueError):
        pc.PointCloud(pts)                               # neither batch ids nor sizes
    with pytest.raises(ValueError):
        pc.PointCloud(pts, np.zeros(3, np.int32))        # wrong number of ids
    with pytest.raises(ValueError):
        pc.PointCloud(np.zeros((2, 3, 3), np.float32), sizes=[4, 1])    # size above V
    with pytest.raises(ValueError):
        pc.PointCloud(np.zeros((2, 3, 3), np.float32), sizes=[1, 1, 1])  # wrong batch shape
    with pytest.raises(IndexError):
        pc.PointCloud(pts, np.zeros(4, np.int32)).get_points(3)


def test_flatten_features_and_format_output_round_trip():
    rng = np.random.default_rng(2)
    ids = np.array([1, 0, 1, 2, 0, 1], np.int32)
    cloud = pc.PointCloud(rng.random((6, 3)).astype(np.float32), ids)
    feats = torch.arange(12, dtype=torch.float32).reshape(6, 2)
    padded = cloud.format_output(feats, return_padded=True)
    assert padded.shape == (3, 3, 2)
    assert torch.equal(padded[1], feats[[0, 2, 5]])
    assert torch.equal(cloud.flatten_features(padded), feats)       # inverse of the padding
    assert torch.equal(cloud.format_output(feats, return_sorted=True), feats[[1, 4, 0, 2, 5, 3]])
    assert cloud.flatten_features(feats) is feats
    with pytest.raises(ValueError):
        cloud.flatten_features(feats[:4])


def test_bounding_boxes_and_diameter():
    """aabb_test.py:30-78: per-cloud minima / maxima and the norms of the extent."""
    rng = np.random.default_rng(3)
    pts = rng.random((500, 3)).astype(np.float32) * np.array([2.0, 1.0, 0.5], np.float32)
    bids = rng.integers(0, 4, 500).astype(np.int32)
    bids[:4] = np.arange(4)
    cloud = pc.PointCloud(torch.as_tensor(pts), torch.as_tensor(bids), 4)
    box = cloud.get_AABB()
    assert cloud.get_AABB() is box
    for b in range(4):
        sel = pts[bids == b]
        assert np.allclose(box._aabb_min[b].numpy(), sel.min(0) - 1e-9)
        assert np.allclose(box._aabb_max[b].numpy(), sel.max(0) + 1e-9)
    extent = np.stack([pts[bids == b].max(0) - pts[bids == b].min(0) for b in range(4)])
    assert np.allclose(box.get_diameter().numpy(), np.linalg.norm(extent, axis=1), rtol=1e-6)
    assert np.allclose(box.get_diameter(ord=1).numpy(), extent.sum(1), rtol=1e-6)
    assert np.allclose(box.get_diameter(ord=np.inf).numpy(), extent.max(1), rtol=1e-6)
    cloud.set_batch_shape([2, 2])
    assert pc.AABB(cloud).get_diameter().shape == (2, 2)
