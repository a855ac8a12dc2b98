"""Pins the restated torch-function RoIAlign (CPU baseline of config 1) with its closed form."""
import torch

import torch_ref


def test_closed_form_aligned_false():
    from oracle.torchfun_roi_align import torchfun_roi_align
    g = torch.Generator().manual_seed(3)
    feat = torch.randn(2, 3, 8, 10, 12, generator=g)
    rois = torch.tensor([[1, 2.0, 1.0, 1.5, 9.0, 7.5, 6.0], [0, 0.5, 3.0, 2.0, 11.0, 9.0, 7.0]])
    out_size = (3, 4, 5)
    scale = 0.5
    got = torchfun_roi_align(feat, rois, out_size, scale)
    assert got.shape == (2, 3, 3, 4, 5) and got.dtype == torch.float32
    for r, roi in enumerate(rois):
        b = int(roi[0])
        coords = []
        for axis in range(3):                      # x, y, z
            S = feat.shape[4 - axis]
            n = out_size[2 - axis]
            x1, x2 = float(roi[1 + axis]) / scale, float(roi[4 + axis]) / scale
            j = torch.arange(n, dtype=torch.float64)
            coords.append((x1 + x2) / 2 + ((2 * j + 1) / n - 1) * (x2 - x1) / 2 * S / (S - 1))
        X = coords[0][None, None, :].expand(out_size)
        Y = coords[1][None, :, None].expand(out_size)
        Z = coords[2][:, None, None].expand(out_size)
        want = torch_ref.sample_zeros(feat[b].double(), Z, Y, X)
        assert torch.allclose(got[r].double(), want, atol=2e-5)


def test_closed_form_aligned_true():
    """align_corners=True: base points linspace(-1, 1, n), pixel = (g + 1) / 2 * (S - 1)."""
    from oracle.torchfun_roi_align import torchfun_roi_align
    g = torch.Generator().manual_seed(5)
    feat = torch.randn(2, 2, 7, 9, 8, generator=g)
    rois = torch.tensor([[0, 1.0, 2.0, 0.5, 6.0, 7.5, 5.0], [1, 0.0, 0.0, 0.0, 7.0, 8.0, 6.0]])
    out_size = (4, 3, 5)
    got = torchfun_roi_align(feat, rois, out_size, 1.0, aligned=True)
    for r, roi in enumerate(rois):
        coords = []
        for axis in range(3):
            S, n = feat.shape[4 - axis], out_size[2 - axis]
            x1, x2 = float(roi[1 + axis]), float(roi[4 + axis])
            base = torch.linspace(-1, 1, n, dtype=torch.float64)
            coords.append((S - 1) / S * ((x1 + x2) / 2 + base * (x2 - x1) / 2))
        X = coords[0][None, None, :].expand(out_size)
        Y = coords[1][None, :, None].expand(out_size)
        Z = coords[2][:, None, None].expand(out_size)
        want = torch_ref.sample_zeros(feat[int(roi[0])].double(), Z, Y, X)
        assert torch.allclose(got[r].double(), want, atol=2e-5)


def test_against_vectors_of_the_reference_class():
    """tests/golden/torchfun_roi_align.npz holds what the reference's own class returned (written
    by tests/golden/make_torchfun_vectors.py in the build container): both ``aligned`` settings,
    order 0 and 1, images and volumes, boxes that leave the map."""
    import os
    import numpy as np
    from oracle.torchfun_roi_align import torchfun_roi_align
    data = np.load(os.path.join(os.path.dirname(__file__), "golden", "torchfun_roi_align.npz"))
    for name in ("2d", "3d"):
        feat, rois = torch.from_numpy(data[name + "_feat"]), torch.from_numpy(data[name + "_rois"])
        size, scale = tuple(int(v) for v in data[name + "_size"]), float(data[name + "_scale"])
        for aligned in (False, True):
            for order in (0, 1):
                want = torch.from_numpy(data["%s_aligned%d_order%d" % (name, int(aligned), order)])
                got = torchfun_roi_align(feat, rois, size, scale, aligned=aligned, order=order)
                assert got.shape == want.shape
                # order 0 picks voxels (exact); order 1 may differ in the last bits between CPU types
                ok = torch.equal(got, want) if order == 0 else torch.allclose(got, want, rtol=0, atol=1e-5)
                assert ok, (name, aligned, order, (got - want).abs().max())
