"""Pins the oracle's RoI geometry G and its adjoint.

Known answers come from the reference's own test script (test/ops_test_RoIAlign.py): the 2-D roi
[0,161.5,111.5,417.5,367.5] -> image[112:368,162:418] (:68,86); the 3-D roi
[0,9.5,9.5,59.5,187.5,187.5,89.5] with out (30,178,178) -> vol[60:90,10:188,10:188] (:121,131);
the rotated roi [0,99,99,75,178,178,30,0,0,0] (aligned) -> the same crop (:124).  The sample
volumes are missing from the checkout, so seeded synthetic ones of sufficient size are used.
Everything else is an identity the mathematics fixes, or the independent torch formulation in
torch_ref.py (grid_sample + textbook Euler matrix), or autograd for the adjoint.
"""
import math

import pytest
import torch

import torch_ref


def _rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


def test_reference_crop_identity_2d(oracle):
    img = _rand(2, 1, 400, 440)
    rois = torch.tensor([[0, 161.5, 111.5, 417.5, 367.5]])
    out = oracle.roi_align_forward(img, rois, (256, 256), 1.0, 1)
    assert torch.equal(out[0, 0], img[0, 0, 112:368, 162:418])
    # rotated flavour of the same test (ops_test_RoIAlign.py:73-75): centre 290,240 size 256
    rr = torch.tensor([[0, 290., 240., 256., 256., 0.0]])
    out = oracle.roi_align_forward(img, rr, (256, 256), 1.0, 1, aligned=True, rotated=True)
    assert torch.allclose(out[0, 0], img[0, 0, 112:368, 162:418], atol=1e-12)


def test_reference_crop_identity_3d(oracle):
    vol = _rand(1, 1, 95, 192, 190, seed=1)
    rois = torch.tensor([[0, 9.5, 9.5, 59.5, 187.5, 187.5, 89.5]])
    out = oracle.roi_align_forward(vol, rois, (30, 178, 178), 1.0, 1)
    assert torch.equal(out[0, 0], vol[0, 0, 60:90, 10:188, 10:188])
    rr = torch.tensor([[0, 99., 99., 75., 178, 178, 30, 0, 0, 0]])
    out = oracle.roi_align_forward(vol, rr, (30, 178, 178), 1.0, 1, aligned=True, rotated=True)
    assert torch.allclose(out[0, 0], vol[0, 0, 60:90, 10:188, 10:188], atol=1e-12)
    # nearest (order 0) gives the same crop because samples sit on voxel centres
    out = oracle.roi_align_forward(vol, rr, (30, 178, 178), 1.0, 1, aligned=True, order=0,
                                   rotated=True)
    assert torch.equal(out[0, 0], vol[0, 0, 60:90, 10:188, 10:188])


def test_rotated_identity_shift_and_quarter_turns(oracle):
    vol = _rand(2, 3, 8, 10, 12, seed=2)
    D, H, W = 8, 10, 12
    full = [W / 2, H / 2, D / 2, W, H, D]
    ident = torch.tensor([[1, *full, 0, 0, 0]])
    out = oracle.roi_align_forward(vol, ident, (D, H, W), 1.0, 1, rotated=True)
    assert torch.allclose(out[0], vol[1], atol=1e-12)
    # integer shift by (+2 x, -1 y, +3 z): replicate within one voxel of the border, zero beyond
    sh = torch.tensor([[0, full[0] + 2, full[1] - 1, full[2] + 3, W, H, D, 0, 0, 0]])
    out = oracle.roi_align_forward(vol, sh, (D, H, W), 1.0, 1, rotated=True)[0]
    want = torch.zeros_like(vol[0])
    for z in range(D):
        for y in range(H):
            for x in range(W):
                sz, sy, sx = z + 3, y - 1, x + 2
                if -1 <= sz <= D and -1 <= sy <= H and -1 <= sx <= W:
                    want[:, z, y, x] = vol[0, :, min(max(sz, 0), D - 1), min(max(sy, 0), H - 1),
                                           min(max(sx, 0), W - 1)]
    assert torch.allclose(out, want, atol=1e-12)
    # quarter turn about z on a cube: out[z,y,x] = vol[z, x, S-1-y]  (x' = -y, y' = x)
    cube = _rand(1, 1, 6, 6, 6, seed=3)
    r = torch.tensor([[0, 3, 3, 3, 6, 6, 6, 0, 0, math.pi / 2]], dtype=torch.float64)
    out = oracle.roi_align_forward(cube, r, (6, 6, 6), 1.0, 1, rotated=True)[0, 0]
    want = cube[0, 0].permute(0, 2, 1).flip(1)
    assert torch.allclose(out, want, atol=1e-9)
    # quarter turn about x (gamma): y' = -z, z' = y  -> out[z,y,x] = vol[y, S-1-z, x]
    r = torch.tensor([[0, 3, 3, 3, 6, 6, 6, math.pi / 2, 0, 0]], dtype=torch.float64)
    out = oracle.roi_align_forward(cube, r, (6, 6, 6), 1.0, 1, rotated=True)[0, 0]
    want = cube[0, 0].permute(1, 0, 2).flip(0)
    assert torch.allclose(out, want, atol=1e-9)
    # quarter turn about y (beta): x' = z, z' = -x -> out[z,y,x] = vol[S-1-x, y, z]
    r = torch.tensor([[0, 3, 3, 3, 6, 6, 6, 0, math.pi / 2, 0]], dtype=torch.float64)
    out = oracle.roi_align_forward(cube, r, (6, 6, 6), 1.0, 1, rotated=True)[0, 0]
    want = cube[0, 0].permute(2, 1, 0).flip(2)
    assert torch.allclose(out, want, atol=1e-9)


def test_plain_vs_rotated_and_aligned_relations(oracle):
    f = _rand(2, 2, 9, 11, 13, seed=4)
    # angles 0, aligned=False  ==  plain RoIAlign of centre +- size/2
    plain = torch.tensor([[1, 2.25, 1.5, 0.75, 9.75, 8.0, 6.25]])
    c = (plain[0, 1:4] + plain[0, 4:7]) / 2
    s = plain[0, 4:7] - plain[0, 1:4]
    rot = torch.tensor([[1, *c, *s, 0, 0, 0]])
    a = oracle.roi_align_forward(f, plain, (3, 4, 5), 1.0, 2)
    b = oracle.roi_align_forward(f, rot, (3, 4, 5), 1.0, 2, aligned=False, rotated=True)
    assert torch.allclose(a, b, atol=1e-12)
    # aligned=True == aligned=False with the centre moved by -0.5 (sizes >= 1)
    rot2 = rot.clone()
    rot2[0, 1:4] += 0.5
    b2 = oracle.roi_align_forward(f, rot2, (3, 4, 5), 1.0, 2, aligned=True, rotated=True)
    assert torch.allclose(a, b2, atol=1e-12)
    # spatial_scale just rescales the box
    a2 = oracle.roi_align_forward(f, torch.cat([plain[:, :1], plain[:, 1:] * 4], 1), (3, 4, 5),
                                  0.25, 2)
    assert torch.allclose(a, a2, atol=1e-12)
    # sampling_ratio g == mean over the g^3 sub-bins sampled once each
    fine = oracle.roi_align_forward(f, plain, (6, 8, 10), 1.0, 1)
    pooled = fine.reshape(1, 2, 3, 2, 4, 2, 5, 2).mean(dim=(3, 5, 7))
    assert torch.allclose(a, pooled, atol=1e-12)
    # adaptive grid (sampling_ratio <= 0) == explicit ceil(size / cells) when equal on all axes
    box = torch.tensor([[0, 1.0, 1.0, 1.0, 8.5, 8.5, 8.5]])  # 7.5 / 3 -> ceil = 3
    assert torch.allclose(oracle.roi_align_forward(f, box, (3, 3, 3), 1.0, 0),
                          oracle.roi_align_forward(f, box, (3, 3, 3), 1.0, 3), atol=1e-12)
    # constant input -> constant output where all samples are in range; linearity
    ones = torch.ones_like(f)
    assert torch.allclose(oracle.roi_align_forward(ones, plain, (3, 4, 5), 1.0, 2),
                          torch.ones(1, 2, 3, 4, 5, dtype=torch.float64))
    g = _rand(2, 2, 9, 11, 13, seed=5)
    lhs = oracle.roi_align_forward(2 * f - 3 * g, plain, (3, 4, 5), 1.0, 2)
    rhs = 2 * a - 3 * oracle.roi_align_forward(g, plain, (3, 4, 5), 1.0, 2)
    assert torch.allclose(lhs, rhs, atol=1e-12)


@pytest.mark.parametrize("ndim,rotated,aligned,sr", [
    (3, True, True, 2), (3, True, False, 0), (3, False, True, 2), (3, False, True, -1),
    (2, True, True, 3), (2, True, False, 0), (2, False, True, 2), (2, False, True, 0)])
def test_against_torch_formulation_and_autograd(oracle, ndim, rotated, aligned, sr):
    g = torch.Generator().manual_seed(10 + ndim + 2 * rotated + 4 * aligned + sr)
    size = (7, 9, 11)[3 - ndim:]
    feat = torch.randn(2, 3, *size, generator=g, dtype=torch.float64, requires_grad=True)
    R = 6
    rois = torch.zeros(R, {(2, False): 5, (3, False): 7, (2, True): 6, (3, True): 10}[(ndim, rotated)])
    rois[:, 0] = torch.randint(0, 2, (R,), generator=g)
    ext = torch.tensor(size[::-1], dtype=torch.float32)
    if rotated:
        rois[:, 1:1 + ndim] = torch.rand(R, ndim, generator=g) * ext * 2.0     # scale 0.5 below
        rois[:, 1 + ndim:1 + 2 * ndim] = (torch.rand(R, ndim, generator=g) * 0.9 + 0.05) * ext * 2.4
        rois[:, 1 + 2 * ndim:] = (torch.rand(R, rois.shape[1] - 1 - 2 * ndim, generator=g) - 0.5) * 2.0
        rois[0, 1 + ndim:1 + 2 * ndim] = 0.3   # degenerate extent (< 1 voxel)
    else:
        lo = (torch.rand(R, ndim, generator=g) * 1.2 - 0.2) * ext * 2.0
        rois[:, 1:1 + ndim] = lo
        rois[:, 1 + ndim:] = lo + torch.rand(R, ndim, generator=g) * ext * 1.6
        rois[0, 1 + ndim:] = rois[0, 1:1 + ndim] + 0.4
    out_size = (3, 4, 5)[3 - ndim:]
    ref = torch_ref.roi_align(feat, rois, out_size, 0.5, sr, aligned, rotated)
    got = oracle.roi_align_forward(feat, rois, out_size, 0.5, sr, aligned, 1, rotated)
    assert torch.allclose(got, ref.detach(), atol=1e-11, rtol=0)
    gy = torch.randn(ref.shape, generator=g, dtype=torch.float64)
    (gref,) = torch.autograd.grad(ref, feat, gy)
    ggot = oracle.roi_align_backward(gy, rois, feat.shape, 0.5, sr, aligned, 1, rotated)
    assert torch.allclose(ggot, gref, atol=1e-11, rtol=0)


@pytest.mark.parametrize("order", [0, 1])
def test_backward_is_adjoint_of_forward(oracle, order):
    g = torch.Generator().manual_seed(77)
    x = torch.randn(2, 2, 6, 7, 8, generator=g, dtype=torch.float64)
    rois = torch.tensor([[0, 4.2, 3.1, 2.9, 7.5, 6.0, 5.2, 0.3, -0.2, 0.5],
                         [1, 1.0, 6.0, 3.0, 9.0, 3.0, 4.0, -0.7, 0.1, 0.0]])
    sr = 1 if order == 0 else 2
    y = torch.randn(2, 2, 3, 3, 4, generator=g, dtype=torch.float64)
    ax = oracle.roi_align_forward(x, rois, (3, 3, 4), 1.0, sr, True, order, True)
    aty = oracle.roi_align_backward(y, rois, x.shape, 1.0, sr, True, order, True)
    assert abs(float((ax * y).sum() - (x * aty).sum())) < 1e-10
    # total gradient mass = sum over outputs of gO * (fraction of in-range samples)
    frac = oracle.roi_align_forward(torch.ones_like(x), rois, (3, 3, 4), 1.0, sr, True, order, True)
    assert abs(float(aty.sum() - (y * frac).sum())) < 1e-10


def test_two_d_matches_textbook_detectron_roialign(oracle):
    """ops_test_RoIAlign.py:24 -- "2d is exactly the same with RoIAlignTorchvision" (aligned=False):
    restated densely: bin sample positions y = y1 + ph*bh + (iy+.5)*bh/g, bilinear with the
    [-1, S] rule, average."""
    g = torch.Generator().manual_seed(5)
    f = torch.randn(1, 2, 12, 14, generator=g, dtype=torch.float64)
    x1, y1, x2, y2 = 2.3, 1.7, 11.9, 9.4
    ph_n, pw_n, sr = 3, 4, 2
    bh, bw = (y2 - y1) / ph_n, (x2 - x1) / pw_n
    want = torch.zeros(2, ph_n, pw_n, dtype=torch.float64)
    for ph in range(ph_n):
        for pw in range(pw_n):
            for iy in range(sr):
                for ix in range(sr):
                    y = y1 + ph * bh + (iy + .5) * bh / sr
                    x = x1 + pw * bw + (ix + .5) * bw / sr
                    y0, x0 = int(y), int(x)
                    ly, lx = y - y0, x - x0
                    want[:, ph, pw] += ((1 - ly) * (1 - lx) * f[0, :, y0, x0] + (1 - ly) * lx * f[0, :, y0, x0 + 1]
                                        + ly * (1 - lx) * f[0, :, y0 + 1, x0] + ly * lx * f[0, :, y0 + 1, x0 + 1])
    want /= sr * sr
    got = oracle.roi_align_forward(f, torch.tensor([[0, x1, y1, x2, y2]]), (ph_n, pw_n), 1.0, sr)
    assert torch.allclose(got[0], want, atol=1e-12)
