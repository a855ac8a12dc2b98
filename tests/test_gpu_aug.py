"""GPU tests of the augmentation stages: each stage's output against the oracle run on the rois
the stage built, plus checks that do not depend on the roi formula at all (identity parameters ==
plain slicing, boxes follow the image content, resize round trip, batch == per-sample)."""
import math
import random

import numpy as np
import pytest
import torch

from parity import FWD_TOL, assert_close
import workloads as wl

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def aug():
    import medvision_amd.aug_cuda as aug_
    from medvision_amd import _lib
    _lib.load()
    return aug_


def _sample(g, shape, boxes=None, dtype=torch.float32):
    dim = len(shape)
    img = torch.randn(2, *shape, generator=g).to(dtype)
    seg = torch.randint(0, 4, (1, *shape), generator=g, dtype=torch.int32)
    res = {"img": img.to(DEV), "gt_seg": seg.to(DEV), "img_dim": dim, "img_shape": tuple(img.shape),
           "img_spacing": (1.0,) * dim, "img_fields": ["img"], "seg_fields": ["gt_seg"], "det_fields": []}
    if boxes is not None:
        res["gt_det"] = torch.tensor(boxes, dtype=torch.float64, device=DEV)
        res["det_fields"] = ["gt_det"]
    return res, img, seg


@pytest.mark.parametrize("shape,factor,order,ties", [
    ((12, 16, 20), (1.5, 0.75, 1.25), 1, True), ((12, 16, 20), (2.0, 2.0, 2.0), 3, True),
    ((18, 22), (0.5, 1.5), 1, True),
    ((12, 15, 21), (16, 10, 14), 1, False)])   # target shape; no nearest-neighbour coordinate on a .5 tie
def test_resize(aug, oracle, shape, factor, order, ties):
    g = wl.gen(200)
    dim = len(shape)
    box = [[2, 3, 4, 10, 9, 8, 1, 1]] if dim == 3 else [[2, 3, 10, 9, 1, 1]]
    res, img, seg = _sample(g, shape, box)
    if ties:
        stage = aug.CudaResize(factor=factor, order=order)
    else:
        stage, factor = aug.CudaResize(scale=factor, order=order), tuple(o / s for o, s in zip(factor, shape))
    out = stage(res)
    new_shape = tuple(int(round(s * f)) if not ties else int(s * f) for s, f in zip(shape, factor))
    assert out["img"].shape == (2, *new_shape) and out["img_shape"] == (2, *new_shape)
    assert np.allclose(out["img_spacing"], [1 / f for f in factor])
    centre, ext = [s / 2 for s in shape[::-1]], list(shape[::-1])
    roi = torch.tensor([[0, *centre, *ext, *([0.0] * (2 * dim - 3))]])
    want = oracle.roi_align_forward(img[None], roi, new_shape, 1.0, 1, True, order, True)[0]
    assert_close(out["img"], want, FWD_TOL[torch.float32], "resized image")
    want_seg = oracle.roi_align_forward(seg[None].float(), roi, new_shape, 1.0, 1, True, 0, True)[0]
    assert out["gt_seg"].dtype == torch.int32 and out["gt_seg"].shape == (1, *new_shape)
    if not ties:   # on exact .5 ties the last bit of the coordinate decides; compared elsewhere
        assert torch.equal(out["gt_seg"].cpu().double(), want_seg)
    scale_xyz = list(factor[::-1]) * 2
    assert np.allclose(out["gt_det"][0, :2 * dim].cpu(), np.array(box[0][:2 * dim]) * scale_xyz)
    # undo: same shape and spacing as before (content is low-pass filtered, not identical)
    back = stage(out, forward=False)
    assert back["img"].shape == (2, *shape) and np.allclose(back["img_spacing"], 1.0)
    assert back["history"] == []


def test_crop_with_identity_affine_is_slicing(aug):
    """scale / shift / rotate ranges of 0: the patch is exactly image[start:end] (and the boxes
    move by -start), whatever the roi formula looks like."""
    g = wl.gen(201)
    res, img, seg = _sample(g, (14, 18, 22), [[8, 6, 4, 15, 12, 9, 1, 1]])
    stage = aug.CudaCropRandomWithAffine((8, 10, 12), scale=0, shift=0, rotate=0)
    np.random.seed(5)
    out = stage(res)
    x0, y0, z0 = out["CudaCropRandomWithAffine_params"]["start"]
    assert torch.equal(out["img"].cpu(), img[:, z0:z0 + 8, y0:y0 + 10, x0:x0 + 12])
    assert torch.equal(out["gt_seg"].cpu(), seg[:, z0:z0 + 8, y0:y0 + 10, x0:x0 + 12])
    want = np.clip(np.array([8 - x0, 6 - y0, 4 - z0, 15 - x0, 12 - y0, 9 - z0]), 0, [11, 9, 7] * 2)
    if len(out["gt_det"]):
        assert np.allclose(out["gt_det"][0, :6].cpu(), want)
    centre = aug.CudaCropCenterWithAffine((8, 10, 12), scale=0, shift=0, rotate=0)
    res2, img2, _ = _sample(g, (14, 18, 22))
    out2 = centre(res2)
    assert torch.equal(out2["img"].cpu(), img2[:, 3:11, 4:14, 5:17])
    # times > 1: a list of independent patches
    many = aug.CudaCropRandomWithAffine((8, 10, 12), scale=0.1, shift=0.05, rotate=10, times=3)
    res3, _, _ = _sample(g, (14, 18, 22))
    outs = many(res3)
    assert len(outs) == 3 and all(o["img"].shape == (2, 8, 10, 12) for o in outs)


@pytest.mark.parametrize("dim", [2, 3])
def test_affine_boxes_follow_the_content(aug, oracle, dim):
    """A bright block and its box go through RandomAffine together: the block's support in the
    output lies inside the transformed box and fills it (up to interpolation blur / rotation hull)."""
    shape = (40, 48)[:dim] if dim == 2 else (16, 40, 48)
    img = torch.zeros(1, *shape)
    if dim == 2:
        img[0, 14:24, 18:34] = 1.0
        box = [[18, 14, 34, 24, 1, 1]]
    else:
        img[0, 5:11, 14:24, 18:34] = 1.0
        box = [[18, 14, 5, 34, 24, 11, 1, 1]]
    for seed, (scale, shift, rot) in enumerate([(0.0, 0.1, 0.0), ([0.2, 0.2], 0.0, 0.0), (0.0, 0.0, [20, 20]),
                                                ([-0.1, -0.1], 0.08, [-15, -15])]):
        res = {"img": img.to(DEV), "img_dim": dim, "img_fields": ["img"], "seg_fields": [],
               "det_fields": ["gt_det"], "gt_det": torch.tensor(box, dtype=torch.float64, device=DEV)}
        stage = aug.CudaRandomAffine(1.0, scale, shift, rot)
        np.random.seed(seed)
        random.seed(seed)
        out = stage(res)
        p = out["CudaRandomAffine_params"]
        rois = torch.from_numpy(stage._rois())
        want = oracle.roi_align_forward(img[None], rois, shape, 1.0, 1, True, 1, True)[0]
        assert_close(out["img"], want, FWD_TOL[torch.float32], "affine image")
        got = out["gt_det"][0].cpu().numpy()
        on = (out["img"][0] > 0.5).nonzero().cpu().numpy()      # voxels well inside the block
        lo, hi = on.min(0)[::-1], on.max(0)[::-1] + 1               # x, y[, z]
        slack = 1.01
        assert np.all(lo >= got[:dim] - slack) and np.all(hi <= got[dim:2 * dim] + slack), (p, lo, hi, got)
        if p["_rotate"][0] == 0.0:   # no rotation hull: the box is tight
            assert np.all(np.abs(lo - got[:dim]) <= slack) and np.all(np.abs(hi - got[dim:2 * dim]) <= slack)


def test_subclasses_and_batch_equal_per_sample(aug, oracle):
    g = wl.gen(203)
    vol = torch.randn(3, 2, 10, 14, 18, generator=g).half()
    res = {"img": vol.to(DEV), "img_dim": 3, "img_fields": ["img"], "seg_fields": [], "det_fields": []}
    stage = aug.BatchCudaRandomAffine(1.0, scale=0.2, shift=0.1, rotate=25)
    np.random.seed(11)
    out = stage(res)
    p = out["BatchCudaRandomAffine_params"]
    assert out["img"].shape == vol.shape
    want = oracle.roi_align_forward(vol, torch.from_numpy(stage._rois()), (10, 14, 18), 1.0, 1, True, 1, True)
    assert_close(out["img"], want, FWD_TOL[torch.float16], "batch affine")
    for b in range(3):   # the per-sample stage with sample b's parameters gives sample b
        single = aug.CudaRandomAffine(1.0, 0, 0, 0)
        single._init_params({"img": vol[b].to(DEV), "img_dim": 3})
        single.params = {"_scales": list(p["scales"][b]), "_shifts": list(p["shifts"][b]), "_rotate": list(p["rotate"][b])}
        r = {"img": vol[b].to(DEV), "img_fields": ["img"]}
        single.apply_to_img(r)
        assert torch.equal(r["img"], out["img"][b])
    crop = aug.BatchCudaCropCenterWithAffine((6, 8, 10), scale=0, shift=0, rotate=0)
    out = crop({"img": vol.to(DEV), "img_dim": 3, "img_fields": ["img"], "seg_fields": [], "det_fields": []})
    assert torch.equal(out["img"].cpu(), vol[:, :, 2:8, 3:11, 4:14])
    bres = aug.BatchCudaResize(scale=(20, -1, 9))({"img": vol.to(DEV), "img_dim": 3, "img_fields": ["img"]})
    assert bres["img"].shape == (3, 2, 20, 14, 9)
    # the named subclasses only narrow the ranges
    s = aug.CudaRandomScale(1.0, 0.3)
    assert (s.shift, s.rotate) == (0, 0)
    r = aug.CudaRandomRotate(1.0, 30)
    np.random.seed(1)
    o = r({"img": vol[0].to(DEV), "img_dim": 3, "img_fields": ["img"]})
    assert o["CudaRandomRotate_params"]["_scales"] == [1.0] * 3 and o["CudaRandomRotate_params"]["_shifts"] == [0.0] * 3


@pytest.mark.parametrize("dim", [2, 3])
def test_elastic(aug, oracle, dim):
    g = wl.gen(204 + dim)
    shape = (40, 48) if dim == 2 else (24, 28, 32)
    box = [[10, 12, 30, 33, 1, 1]] if dim == 2 else [[8, 9, 7, 22, 20, 18, 1, 1]]
    res, img, seg = _sample(g, shape, box)
    stage = aug.CudaRandomElasticDeformation(1.0, num_control_points=7, max_displacement=0.9)
    np.random.seed(21)
    out = stage(res)
    grid = out["CudaRandomElasticDeformation_params"]
    # dense field = order-3 resampling of the halved control grid over the window [1.5, n - 1.5]
    coarse = torch.from_numpy(grid).permute(dim, *range(dim))[None] / 2
    roi = torch.tensor([[0, *([3.5] * dim), *([4.0] * dim), *([0.0] * (2 * dim - 3))]])
    field = oracle.roi_align_forward(coarse, roi, shape, 1.0, 1, True, 3, True)
    assert_close(stage.tmp_params, field[0], FWD_TOL[torch.float32], "dense field")
    assert float(field.abs().max()) > 0.5
    field32 = stage.tmp_params.cpu()[None]
    assert_close(out["img"], oracle.deform_warp(img[None], field32, 1)[0], FWD_TOL[torch.float32], "warped image")
    want_seg = oracle.deform_warp(seg[None].float(), field32, 0)[0]
    assert out["gt_seg"].dtype == torch.int32 and torch.equal(out["gt_seg"].cpu().double(), want_seg)
    # boxes: every corner moves against the displacement found at its voxel
    b = np.array(box[0][:2 * dim], dtype=np.float64)
    f = field32[0].numpy()
    lo = f[(slice(None), *np.int64(b[:dim])[::-1])][::-1]
    got = out["gt_det"][0, :2 * dim].cpu().numpy()
    assert np.all(np.abs(got - b) <= np.abs(f).max() + 1e-6) and abs(got[0] - (b[0] - lo[0])) < np.abs(f).max() * 2
    # locked borders: the outermost voxels barely move
    assert float(stage.tmp_params[:, 0].abs().max()) < 0.3
    # undo pushes the stored grid back with the opposite sign
    back = stage(out, forward=False)
    assert back["img"].shape == img.shape and "CudaRandomElasticDeformation_params" not in back
    # zero displacement = identity
    still = aug.CudaRandomElasticDeformation(1.0, 7, 0.0)
    res2, img2, _ = _sample(g, shape)
    assert torch.equal(still(res2)["img"].cpu(), img2)


@pytest.mark.parametrize("dim", [2, 3])
def test_batch_elastic_equals_per_sample(aug, oracle, dim):
    """The batch stage draws one control grid per sample in sample order and warps the batch in one
    call: sample b must equal the per-sample stage run on that grid, and the oracle."""
    g = wl.gen(230 + dim)
    shape = (36, 44) if dim == 2 else (20, 24, 28)
    B = 3
    img = torch.randn(B, 2, *shape, generator=g)
    seg = torch.randint(0, 4, (B, 1, *shape), generator=g, dtype=torch.int32)
    res = {"img": img.to(DEV), "gt_seg": seg.to(DEV), "img_dim": dim, "img_fields": ["img"], "seg_fields": ["gt_seg"],
           "det_fields": []}
    stage = aug.BatchCudaRandomElasticDeformation(1.0, num_control_points=7, max_displacement=0.9)
    np.random.seed(31)
    out = stage(res)
    grids = out["BatchCudaRandomElasticDeformation_params"]
    assert grids.shape == (B, *([7] * dim), dim)
    np.random.seed(31)   # the same draws, one sample at a time
    for b in range(B):
        want_grid = 2 * np.random.rand(*([7] * dim), dim).astype(np.float32) - 1
        inner = tuple(slice(2, 5) for _ in range(dim))
        assert np.all(grids[b][inner] != 0) and np.count_nonzero(grids[b]) == 3 ** dim * dim
        assert np.allclose(np.sign(grids[b][inner]), np.sign(want_grid[inner]))
        coarse = torch.from_numpy(grids[b]).permute(dim, *range(dim))[None] / 2
        roi = torch.tensor([[0, *([3.5] * dim), *([4.0] * dim), *([0.0] * (2 * dim - 3))]])
        field = oracle.roi_align_forward(coarse, roi, shape, 1.0, 1, True, 3, True)
        assert_close(stage.tmp_params[b], field[0], FWD_TOL[torch.float32], "dense field of sample %d" % b)
        f32 = stage.tmp_params[b].cpu()[None]
        assert_close(out["img"][b], oracle.deform_warp(img[b][None], f32, 1)[0], FWD_TOL[torch.float32], "warped image")
        assert torch.equal(out["gt_seg"][b].cpu().double(), oracle.deform_warp(seg[b][None].float(), f32, 0)[0])
    assert float((stage.tmp_params[0] - stage.tmp_params[1]).abs().max()) > 0.1   # samples differ
    with pytest.raises(NotImplementedError):
        stage.apply_to_det({"det_fields": ["gt_det"], "gt_det": torch.zeros(1, 6)})


def test_batch_crops_around_boxes_and_foreground(aug):
    """The windows of the detection / foreground crop stages contain the box or component they were
    drawn around (plus the border where the patch has room); identity affine == slicing."""
    g = wl.gen(240)
    B, shape, patch = 3, (24, 28, 32), (12, 14, 16)
    img = torch.randn(B, 1, *shape, generator=g)
    seg = torch.zeros(B, 1, *shape, dtype=torch.int32)
    blobs = [(3, 4, 5), (10, 12, 20), (18, 20, 6)]
    for b, (z, y, x) in enumerate(blobs):
        seg[b, 0, z:z + 3, y:y + 4, x:x + 5] = 1
    det = torch.tensor([[6., 5., 4., 11., 9., 7., 1., 1.], [20., 12., 10., 25., 16., 13., 1., 1.]], dtype=torch.float64)
    base = {"img_dim": 3, "img_fields": ["img"], "seg_fields": ["gt_seg"], "det_fields": []}
    random.seed(5)
    np.random.seed(5)
    fg = aug.BatchCudaCropForegroundWithAffine(border=2, patch_size=patch, scale=0, shift=0, rotate=0)
    out = fg({**base, "img": img.to(DEV), "gt_seg": seg.to(DEV)})
    p = out["BatchCudaCropForegroundWithAffine_params"]
    for b, (z, y, x) in enumerate(blobs):
        sx, sy, sz = p["start"][b]
        assert sz <= z and z + 3 <= sz + patch[0] and sy <= y and y + 4 <= sy + patch[1] and sx <= x and x + 5 <= sx + patch[2]
        assert torch.equal(out["img"][b].cpu(), img[b, :, sz:sz + patch[0], sy:sy + patch[1], sx:sx + patch[2]])
        assert int(out["gt_seg"][b].sum()) == 60
    first = aug.BatchCudaCropFirstDetWithAffine(border=1, patch_size=patch, scale=0, shift=0, rotate=0)
    out = first({**base, "seg_fields": [], "img": img.to(DEV), "gt_det": det.to(DEV)})
    for b in range(B):
        sx, sy, sz = out["BatchCudaCropFirstDetWithAffine_params"]["start"][b]
        assert sx <= 6 and 11 <= sx + patch[2] and sy <= 5 and 9 <= sy + patch[1] and sz <= 4 and 7 <= sz + patch[0]
    turns = aug.BatchCudaCropDetWithAffine(border=1, patch_size=patch, scale=0, shift=0, rotate=0, times=2)
    turns._init_params({"img": img.to(DEV), "img_dim": 3})
    picks = []
    for _ in range(4):
        sz, sy, sx = turns._crop_start({"gt_det": det.to(DEV)}, 0)
        picks.append(0 if sx <= 6 and 11 <= sx + patch[2] else 1)
    assert picks == [0, 1, 0, 1]


@pytest.mark.parametrize("dim,size,out", [(3, (40, 48, 56), (40, 48, 56)), (3, (20, 24, 28), (9, 10, 11)),
                                          (2, (96, 128), (96, 128)), (2, (30, 40), (12, 14))])
def test_int32_label_maps_are_sampled_as_they_are(dim, size, out):
    """Order 0 on int32 label maps through the affine engines: the library loads and stores the integers
    itself (tiled kernel for large outputs, general kernel for small ones) and must pick the very voxels of
    the float copy that such maps used to be resampled through (the reference's `.float()` ... `.int()`):
    rotated, shifted and scaled rois that reach past the map, labels from -5 to 2^24 - 1."""
    import medvision_amd.ops as ops
    g = wl.gen(77 + dim + out[0])
    n = 3
    seg = torch.randint(-5, 40, (n, 2, *size), generator=g, dtype=torch.int32)
    seg[0, 0].view(-1)[::7] = 2 ** 24 - 1
    xyz = torch.tensor(size[::-1], dtype=torch.float32)
    ctr = xyz / 2 + (torch.rand(n, dim, generator=g) * 2 - 1) * 6
    ext = xyz * (0.7 + torch.rand(n, dim, generator=g) * 0.7)
    ang = (torch.rand(n, 3 if dim == 3 else 1, generator=g) * 2 - 1) * 0.5
    rois = torch.cat([torch.arange(n).float().view(n, 1), ctr, ext, ang], 1).to(DEV)
    fn = ops.affine_3d if dim == 3 else ops.affine_2d
    got = fn(seg.to(DEV), rois, out, 1.0, 1, True, 0)
    want = fn(seg.to(DEV).float(), rois, out, 1.0, 1, True, 0).int()
    assert got.dtype == torch.int32 and torch.equal(got, want)
    assert int((got != 0).sum()) > got.numel() // 4
    with pytest.raises((RuntimeError, AssertionError)):
        fn(seg.to(DEV), rois, out, 1.0, 1, True, 1)    # int32 at order 1
