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
