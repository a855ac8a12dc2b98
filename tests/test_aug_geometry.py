"""RoI construction and box transforms of the augmentation layer (CPU: numpy only).

Expected values are worked out by hand from the definition "window (start, end), scaled about its
centre by 1/s, moved by -extent * shift / s, turned by the angle", not by re-running the code's
formula."""
import math
import random

import numpy as np
import pytest

from medvision_amd.aug_cuda import geometry
from medvision_amd.aug_cuda import spatial


def test_frame_and_window_rois():
    r = geometry.frame_rois((4, 6, 8), 2)
    assert r.dtype == np.float32 and r.shape == (2, 10)
    assert r.tolist() == [[0, 4, 3, 2, 8, 6, 4, 0, 0, 0], [1, 4, 3, 2, 8, 6, 4, 0, 0, 0]]
    # 3-D: scale 1.25 -> the sampled box shrinks to 8/1.25 = 6.4 etc.; shift +0.1 of the width
    # moves the box centre by -8 * 0.1 / 1.25 = -0.64; the angle goes to the last column
    r = geometry.window_rois(3, [0, 0, 0], [8, 6, 4], [1.25] * 3, [0.1, 0.0, -0.1], [0.3])
    want = [0, 4 - 0.64, 3, 2 + 0.32, 6.4, 4.8, 3.2, 0, 0, 0.3]
    assert np.allclose(r[0], want, atol=1e-6)
    # 2-D rows have one angle; per-sample tables
    r = geometry.window_rois(2, [[0, 0], [2, 2]], [[8, 6], [10, 8]], [[2, 2], [1, 1]],
                             [[0, 0.5], [0, 0]], [[0.3], [-0.1]])
    assert np.allclose(r, [[0, 4, 3 - 1.5, 4, 3, 0.3], [1, 6, 5, 8, 6, -0.1]], atol=1e-6)


def test_map_and_clip_boxes():
    frame = (40.0, 30.0, 20.0)
    box = np.array([[10., 9., 8., 20., 15., 12., 1., 0.9]])
    same = geometry.map_boxes(3, box, frame, [1, 1, 1], [0, 0, 0], [0.0])
    assert np.allclose(same, box)
    # shift by +0.25 of the width: content (and boxes) move +10 voxels along x
    moved = geometry.map_boxes(3, box, frame, [1, 1, 1], [0.25, 0, 0], [0.0])
    assert np.allclose(moved[0, [0, 3]], [20, 30]) and np.allclose(moved[0, [1, 2, 4, 5]], box[0, [1, 2, 4, 5]])
    # scale 2 about the image centre (20, 15, 10)
    big = geometry.map_boxes(3, box, frame, [2, 2, 2], [0, 0, 0], [0.0])
    assert np.allclose(big[0, :6], [0, 3, 6, 20, 15, 14])
    # quarter turn of a rectangle centred on the image centre swaps its x and y extents; z stays
    cen = np.array([[20 - 6., 15 - 2., 5., 20 + 6., 15 + 2., 9., 0., 0.]])
    turned = geometry.map_boxes(3, cen, frame, [1, 1, 1], [0, 0, 0], [math.pi / 2])
    assert np.allclose(turned[0, :6], [20 - 2, 15 - 6, 5, 20 + 2, 15 + 6, 9])
    # a crop window starting at (5, 4, 3) moves boxes by -start
    crop = geometry.map_boxes(3, box, (16., 16., 16.), [1, 1, 1], [0, 0, 0], [0.0], start_xyz=(5, 4, 3))
    assert np.allclose(crop[0, :6], [5, 5, 5, 15, 11, 9])
    # clip: into [0, size-1]; boxes that collapse are dropped; extra columns survive
    boxes = np.array([[-3., 2., 1., 50., 10., 5., 7., 0.5], [45., 2., 1., 60., 10., 5., 3., 0.1]])
    kept = geometry.clip_boxes(boxes, (20, 30, 40))
    assert kept.tolist() == [[0., 2., 1., 39., 10., 5., 7., 0.5]]
    assert geometry.clip_boxes(np.zeros((0, 8)), (20, 30, 40)).shape == (0, 8)


def test_parameter_draws_follow_numpy_random_in_the_documented_order():
    import torch
    result = {"img": torch.zeros(1, 8, 9, 10), "img_dim": 3}
    stage = spatial.CudaCropRandomWithAffine((4, 5, 6), scale=0.2, shift=0.1, rotate=30)
    np.random.seed(7)
    stage._forward_params(result)
    np.random.seed(7)
    start = [np.random.randint(0, 8 - 4 + 1), np.random.randint(0, 9 - 5 + 1), np.random.randint(0, 10 - 6 + 1)]
    scale = 1 + np.random.uniform(-0.2, 0.2)
    shifts = [np.random.uniform(-0.1, 0.1) for _ in range(3)]
    angle = math.pi * np.random.uniform(-30, 30) / 180
    p = result["CudaCropRandomWithAffine_params"]
    assert tuple(p["start"]) == tuple(start[::-1]) and tuple(p["end"]) == (start[2] + 6, start[1] + 5, start[0] + 4)
    assert p["_scales"] == [scale] * 3 and p["_shifts"] == shifts and p["_rotate"] == [angle]
    rois = stage._rois()
    assert rois.shape == (1, 10) and rois[0, 9] == np.float32(angle) and rois[0, 7] == 0 and rois[0, 8] == 0
    # batch stage: one row of parameters per sample
    bstage = spatial.BatchCudaRandomAffine(1.0, scale=0.1, shift=0.1, rotate=10)
    bresult = {"img": torch.zeros(3, 1, 8, 9), "img_dim": 2}
    bstage._forward_params(bresult)
    bp = bresult["BatchCudaRandomAffine_params"]
    assert bp["scales"].shape == (3, 2) and bp["shifts"].shape == (3, 2) and bp["rotate"].shape == (3, 1)
    assert bstage._rois().shape == (3, 6) and bstage._rois()[:, 0].tolist() == [0, 1, 2]


def test_elastic_control_grid_and_gate():
    import torch
    stage = spatial.CudaRandomElasticDeformation(p=1.0, num_control_points=7, max_displacement=0.5)
    result = {"img": torch.zeros(1, 24, 30, 36), "img_dim": 3}
    np.random.seed(3)
    stage._forward_params(result)
    grid = result["CudaRandomElasticDeformation_params"]
    assert grid.shape == (7, 7, 7, 3) and grid.dtype == np.float32
    inner = grid[2:-2, 2:-2, 2:-2]
    assert np.all(grid[:2] == 0) and np.all(grid[:, -2:] == 0) and np.all(grid[:, :, :2] == 0)
    assert np.any(inner != 0)
    # |displacement| <= max_displacement * cell / 2 with cell = size / (points - 1), per component z, y, x
    limit = 0.5 * np.array([24, 30, 36]) / 6 / 2
    assert np.all(np.abs(inner) <= limit + 1e-6) and np.abs(inner[..., 2]).max() > limit[0]
    # the probability gate uses random.random(): p * latitude = 0 never fires
    gate = spatial.CudaRandomShift(p=0.5, shift=0.1)
    gate.setLatitude(0.0)
    random.seed(0)
    out = gate({"img": torch.zeros(1, 4, 4), "img_dim": 2, "img_fields": ["img"]})
    assert out["history"] == ["CudaRandomShift"] and "CudaRandomShift_params" not in out
    with pytest.raises(AssertionError):
        spatial.CudaRandomShift(p=0.0, shift=0.1)({"img": torch.zeros(1, 4, 4), "img_dim": 2})
