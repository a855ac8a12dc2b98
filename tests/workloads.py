"""Seeded synthetic inputs shaped like the five benchmark configurations (and reduced twins)."""
import math

import torch


def gen(seed):
    return torch.Generator().manual_seed(seed)


def roi3d_detection(g, n_rois, batch, in_size, extent=(4.0, 24.0), log_uniform=False):
    """Plain 3-D boxes (b, x1,y1,z1, x2,y2,z2) in input space; in_size = (W, H, D)."""
    size = torch.tensor(in_size, dtype=torch.float32)
    b = torch.randint(0, batch, (n_rois, 1), generator=g).float()
    u = torch.rand(n_rois, 3, generator=g)
    if log_uniform:
        e = torch.exp(math.log(extent[0]) + u * (math.log(extent[1]) - math.log(extent[0])))
    else:
        e = extent[0] + u * (extent[1] - extent[0])
    lo = torch.rand(n_rois, 3, generator=g) * (size - e).clamp(min=0)
    hi = torch.minimum(lo + e, size)
    return torch.cat([b, lo, hi], 1)


def affine_rois(g, batch, size, max_angle_deg=30.0, scale=(0.8, 1.2), shift=10.0):
    """One full-volume rotated roi per sample, RandomAffine-style; size = (W, H, D)."""
    size = torch.tensor(size, dtype=torch.float32)
    ang = (torch.rand(batch, 3, generator=g) * 2 - 1) * math.radians(max_angle_deg)
    s = scale[0] + torch.rand(batch, 1, generator=g) * (scale[1] - scale[0])
    sh = (torch.rand(batch, 3, generator=g) * 2 - 1) * shift
    idx = torch.arange(batch, dtype=torch.float32)[:, None]
    return torch.cat([idx, size / 2 + sh, size / s, ang], 1)


def ct_like(g, shape, dtype=torch.float16):
    """Hounsfield-like volume: 30% air (-1000), 60% tissue N(40,30), 10% bone N(700,200)."""
    u = torch.rand(shape, generator=g)
    n = torch.randn(shape, generator=g)
    v = torch.where(u < 0.3, torch.full(shape, -1000.0),
                    torch.where(u < 0.9, 40.0 + 30.0 * n, 700.0 + 200.0 * n))
    return v.to(dtype)


def dcn_inputs(g, B, Cin, Cout, size, k=3, dg=1, groups=1, dtype=torch.float32, stride=1, pad=1,
               dil=1, modulated=True, offset_std=2.0):
    """Inputs of a deformable convolution; ``size`` with two entries gives the 2-D layer."""
    nd = len(size)
    x = torch.randn(B, Cin, *size, generator=g)
    K = k ** nd
    bound = 1.0 / math.sqrt(Cin // groups * K)
    w = (torch.rand(Cout, Cin // groups, *([k] * nd), generator=g) * 2 - 1) * bound
    bias = (torch.rand(Cout, generator=g) * 2 - 1) * bound
    out = [(s + 2 * pad - (dil * (k - 1) + 1)) // stride + 1 for s in size]
    off = torch.randn(B, dg * nd * K, *out, generator=g) * offset_std
    mask = torch.sigmoid(torch.randn(B, dg * K, *out, generator=g)) if modulated else None
    cast = lambda t: None if t is None else t.to(dtype)
    return cast(x), cast(off), cast(mask), cast(w), cast(bias)
