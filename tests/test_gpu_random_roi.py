"""Random RoIAlign / RoIAlignRotated problems against the fp64 oracle: every dispatch branch of the
forward and backward entry points (tiled, pooled, channels-last, box tiles, general) is reached by
shape alone, so shapes are drawn at random - dimensions, plain / rotated, types, orders, fixed and
adaptive sampling grids, scales, output sizes from one cell to resampling size, boxes partly or wholly
outside the volume.  A longer run of the same generator (tens of thousands of cases) found a 16-byte
over-read of the pooled backward that only showed with NaN behind the tensor."""
import math
import random

import pytest
import torch

from parity import BWD_TOL, FWD_TOL, assert_nearest, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    import medvision_amd.ops as ops_
    from medvision_amd import _lib
    _lib.load()
    return ops_


def make_case(seed):
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    ndim = rng.choice([2, 3, 3])
    rotated = rng.random() < 0.5
    dtype = rng.choice([torch.float32, torch.float16, torch.bfloat16])
    order = rng.choice([1, 1, 1, 0])
    sr = 1 if order == 0 else rng.choice([0, 1, 1, 2, 2, 3, 4, 5])
    aligned = rng.random() < 0.7
    N, C = rng.choice([1, 2, 3]), rng.choice([1, 2, 3, 5, 16, 24, 64])
    kind = rng.choice(["small", "small", "medium", "large"])
    size = [rng.randint(4, 40) for _ in range(3)] if ndim == 3 else [rng.randint(6, 150) for _ in range(2)]
    if rng.random() < 0.3:
        size[-1] = max(4, size[-1] // 4 * 4)
    if kind == "small":
        out, R = [rng.randint(1, 9) for _ in range(ndim)], rng.choice([1, 7, 60, 300])
    elif kind == "medium":
        out, R = [rng.randint(8, 20) for _ in range(ndim)], rng.choice([1, 5, 30])
    else:
        out = [rng.randint(12, 40) for _ in range(ndim)]
        out[-1] = rng.randint(16, 48)
        R, C = rng.choice([1, 2, 4]), min(C, 3)
        if ndim == 2:
            out = [rng.randint(40, 120), rng.randint(64, 128)]
    grid = sr if sr > 0 else 3
    while R * C * math.prod(out) * grid ** ndim > 3e7 and C > 1:
        C = max(1, C // 2)
    while R * C * math.prod(out) * grid ** ndim > 3e7 and R > 1:
        R = max(1, R // 2)
    scale = rng.choice([1.0, 1.0, 0.5, 0.25, 2.0])
    xyz = torch.tensor(size[::-1], dtype=torch.float32) / scale
    b = torch.randint(0, N, (R, 1), generator=g).float()
    ext = torch.exp(torch.rand(R, ndim, generator=g) * math.log(60.0)) * 0.5 / scale * (3 if kind == "large" else 1)
    if rotated:
        ctr = (torch.rand(R, ndim, generator=g) * 1.2 - 0.1) * xyz
        ang = (torch.rand(R, 1 if ndim == 2 else 3, generator=g) * 2 - 1) * rng.choice([0.0, 0.3, 1.0, 3.14])
        rois = torch.cat([b, ctr, torch.minimum(ext, xyz * 1.3), ang], 1)
    else:
        lo = (torch.rand(R, ndim, generator=g) * 1.2 - 0.15) * xyz
        rois = torch.cat([b, lo, lo + ext], 1)
    feat = torch.randn(N, C, *size, generator=g).to(dtype)
    what = (f"seed={seed} ndim={ndim} rotated={rotated} {dtype} order={order} sr={sr} aligned={aligned} "
            f"N={N} C={C} size={size} out={out} R={R} scale={scale}")
    return dict(g=g, feat=feat, rois=rois, out=tuple(out), scale=scale, sr=sr, aligned=aligned if rotated else True,
                order=order, rotated=rotated, dtype=dtype, what=what)


@pytest.mark.parametrize("block", range(4))
def test_random_problems_vs_oracle(ops, oracle, block):
    for seed in range(900000 + block * 150, 900000 + (block + 1) * 150):
        c = make_case(seed)
        feat, rois, out, dtype = c["feat"], c["rois"], c["out"], c["dtype"]
        args = (out, c["scale"], c["sr"], c["aligned"])
        x = feat.to(DEV).requires_grad_(True)
        mod = ops.RoIAlignRotated(*args) if c["rotated"] else ops.RoIAlign(*args[:3])
        got = mod(x, rois.to(DEV), c["order"])
        want = oracle.roi_align_forward(feat, rois, out, c["scale"], c["sr"], c["aligned"], c["order"], c["rotated"])
        # distance of a cell's samples from a decision of the sampler: a 0.5 tie (order 0) or the edge
        # of [-1, size], where a sample turns void (both orders)
        margin = oracle.roi_decision_margin(feat.shape, rois, out, c["scale"], c["sr"], c["aligned"], c["rotated"])
        if c["order"] == 0:
            assert_nearest(got, want, margin, dtype, c["what"])
            continue
        keep = (margin > (2e-5 if dtype != torch.float32 else 1e-9)).unsqueeze(1).to(torch.float64)
        e = rel_err(got.detach().cpu().double() * keep, want * keep)
        assert e <= FWD_TOL[dtype], f"{c['what']}: forward rel err {e:.3e}"
        gy = (torch.randn(got.shape, generator=c["g"]) * keep.float()).to(dtype)
        got.backward(gy.to(DEV))
        gwant = oracle.roi_align_backward(gy, rois, feat.shape, c["scale"], c["sr"], c["aligned"], 1, c["rotated"])
        e = rel_err(x.grad, gwant)
        assert e <= BWD_TOL[dtype], f"{c['what']}: backward rel err {e:.3e}"
