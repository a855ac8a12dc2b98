"""Independent fp64 torch formulations used to pin the C oracle (CPU tests only).

They lean on library routines whose conventions are documented by torch itself:
``F.grid_sample(align_corners=True)`` with ``padding_mode='border'`` (== clamped sampler S on
[0, S-1]) or ``'zeros'`` (== the DCN zero-padded sampler), ``F.conv3d`` and autograd.
"""
import math

import torch
import torch.nn.functional as F


def _norm(coord, size):
    # align_corners=True: pixel i <-> -1 + 2 i / (size - 1); a size-1 axis maps everything to 0
    if size == 1:
        return torch.zeros_like(coord)
    return 2.0 * coord / (size - 1) - 1.0


def sample_border(plane, z, y, x):
    """Clamped trilinear sampler S (order 1) for coordinate tensors of equal shape.

    plane [C, D, H, W] fp64 -> [C, *z.shape].  Zero outside the closed interval [-1, S].
    """
    C, D, H, W = plane.shape
    shp = z.shape
    inside = ((z >= -1) & (z <= D) & (y >= -1) & (y <= H) & (x >= -1) & (x <= W))
    zc, yc, xc = z.clamp(0, D - 1), y.clamp(0, H - 1), x.clamp(0, W - 1)
    grid = torch.stack([_norm(xc, W), _norm(yc, H), _norm(zc, D)], -1).reshape(1, 1, 1, -1, 3)
    val = F.grid_sample(plane[None], grid, mode="bilinear", padding_mode="border",
                        align_corners=True)
    return (val.reshape(C, -1) * inside.reshape(1, -1).to(plane.dtype)).reshape(C, *shp)


def sample_zeros(plane, z, y, x):
    """Zero-padded trilinear sampler of the DCN kernels: grid_sample(zeros, align_corners=True).

    The DCN gate -1 < p < S is implied: beyond it all 8 corners are out of bounds.
    """
    C, D, H, W = plane.shape
    shp = z.shape
    grid = torch.stack([_norm(x, W), _norm(y, H), _norm(z, D)], -1).reshape(1, 1, 1, -1, 3)
    val = F.grid_sample(plane[None], grid, mode="bilinear", padding_mode="zeros",
                        align_corners=True)
    return val.reshape(C, *shp)


def euler_zyx(gamma, beta, alpha):
    """Rz(alpha) @ Ry(beta) @ Rx(gamma) acting on (x, y, z) column vectors (textbook form)."""
    cg, sg, cb, sb, ca, sa = (math.cos(gamma), math.sin(gamma), math.cos(beta), math.sin(beta),
                              math.cos(alpha), math.sin(alpha))
    rx = torch.tensor([[1, 0, 0], [0, cg, -sg], [0, sg, cg]], dtype=torch.float64)
    ry = torch.tensor([[cb, 0, sb], [0, 1, 0], [-sb, 0, cb]], dtype=torch.float64)
    rz = torch.tensor([[ca, -sa, 0], [sa, ca, 0], [0, 0, 1]], dtype=torch.float64)
    return rz @ ry @ rx


def roi_align(features, rois, output_size, spatial_scale=1.0, sampling_ratio=0, aligned=True,
              rotated=False):
    """Differentiable order-1 RoIAlign / RoIAlignRotated in fp64 (2-D or 3-D).

    Sample positions are built as whole tensors (bin centres via linspace-like arithmetic and a
    matrix product with the textbook Euler matrix) and handed to ``sample_border``.
    """
    ndim = features.dim() - 2
    f = features.to(torch.float64)
    if ndim == 2:
        f = f[:, :, None]
    rois = rois.detach().to(torch.float64)
    scale = float(torch.tensor(spatial_scale, dtype=torch.float32))
    if isinstance(output_size, int):
        output_size = (output_size,) * ndim
    out_zyx = ((1,) + tuple(output_size)) if ndim == 2 else tuple(output_size)
    outs = []
    for roi in rois:
        b = int(roi[0])
        if rotated:
            centre = roi[1:1 + ndim] * scale - (0.5 if aligned else 0.0)
            ext = roi[1 + ndim:1 + 2 * ndim] * scale
            if not aligned:
                ext = ext.clamp(min=1.0)
            start = -ext / 2
            if ndim == 3:
                rot = euler_zyx(float(roi[7]), float(roi[8]), float(roi[9]))
            else:
                rot = euler_zyx(0.0, 0.0, float(roi[5]))
        else:
            start = roi[1:1 + ndim] * scale
            ext = (roi[1 + ndim:1 + 2 * ndim] * scale - start).clamp(min=1.0)
            centre = torch.zeros(ndim, dtype=torch.float64)
            rot = torch.eye(3, dtype=torch.float64)
        axes = []  # local sample coordinates per axis (x, y, z), shape [cells, grid]
        for a in range(3):
            if a >= ndim:
                axes.append(torch.zeros(1, 1, dtype=torch.float64))
                continue
            cells = out_zyx[2 - a]
            g = sampling_ratio if sampling_ratio > 0 else int(math.ceil(float(ext[a]) / cells))
            binsz = ext[a] / cells
            cell = torch.arange(cells, dtype=torch.float64)[:, None]
            sub = torch.arange(g, dtype=torch.float64)[None, :]
            axes.append(start[a] + cell * binsz + (sub + 0.5) * binsz / max(g, 1))
        px, py, pz = axes
        # [od, gz, oh, gy, ow, gx]
        X = px[None, None, None, None, :, :].expand(pz.shape[0], pz.shape[1], py.shape[0],
                                                    py.shape[1], px.shape[0], px.shape[1])
        Y = py[None, None, :, :, None, None].expand_as(X)
        Z = pz[:, :, None, None, None, None].expand_as(X)
        c3 = torch.zeros(3, dtype=torch.float64)
        c3[:ndim] = centre
        P = torch.stack([X, Y, Z], -1) @ rot.T + c3
        if ndim == 2:
            P = torch.stack([P[..., 0], P[..., 1], torch.zeros_like(P[..., 2])], -1)
        vals = sample_border(f[b], P[..., 2], P[..., 1], P[..., 0])
        cnt = max(px.shape[1] * py.shape[1] * pz.shape[1], 1)
        outs.append(vals.sum(dim=(2, 4, 6)) / cnt)
    out = torch.stack(outs) if outs else f.new_zeros((0, f.shape[1]) + out_zyx)
    return out[:, :, 0] if ndim == 2 else out


def sample_border_open(plane, z, y, x):
    """Clamped trilinear sampler on the OPEN interval (-1, S): what the augmentation DCN evaluates."""
    _, D, H, W = plane.shape
    inside = (z > -1) & (z < D) & (y > -1) & (y < H) & (x > -1) & (x < W)
    return sample_border(plane, z, y, x) * inside.to(plane.dtype)


def dcn3d(x, offset, mask, weight, bias=None, stride=1, padding=0, dilation=1, groups=1,
          deformable_groups=1, sampler=sample_zeros):
    """Differentiable fp64 DCN 3-D (v1 if mask is None) from grid_sample + einsum."""
    t3 = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v,) * 3
    s, p, d = t3(stride), t3(padding), t3(dilation)
    B, Cin, D, H, W = x.shape
    Cout, cpg, kd, kh, kw = weight.shape
    K = kd * kh * kw
    Do, Ho, Wo = [(S + 2 * pp - (dd * (k - 1) + 1)) // ss + 1
                  for S, pp, dd, k, ss in zip((D, H, W), p, d, (kd, kh, kw), s)]
    qd = (torch.arange(Do, dtype=x.dtype) * s[0] - p[0])[:, None, None]
    qh = (torch.arange(Ho, dtype=x.dtype) * s[1] - p[1])[None, :, None]
    qw = (torch.arange(Wo, dtype=x.dtype) * s[2] - p[2])[None, None, :]
    cpd = Cin // deformable_groups
    cols = []
    for b in range(B):
        per_dg = []
        for g in range(deformable_groups):
            xs = x[b, g * cpd:(g + 1) * cpd]
            taps = []
            for k in range(K):
                i, j, kk = k // (kh * kw), (k // kw) % kh, k % kw
                o = offset[b, g * 3 * K + 3 * k: g * 3 * K + 3 * k + 3]
                v = sampler(xs, qd + i * d[0] + o[0], qh + j * d[1] + o[1],
                            qw + kk * d[2] + o[2])
                if mask is not None:
                    v = v * mask[b, g * K + k][None]
                taps.append(v)
            per_dg.append(torch.stack(taps, 1))  # [cpd, K, Do, Ho, Wo]
        cols.append(torch.cat(per_dg, 0))  # [Cin, K, ...]
    col = torch.stack(cols)  # [B, Cin, K, Do, Ho, Wo]
    col = col.reshape(B, groups, Cin // groups, K, Do, Ho, Wo)
    wg = weight.reshape(groups, Cout // groups, cpg, K)
    y = torch.einsum("bgckdhw,gock->bgodhw", col, wg).reshape(B, Cout, Do, Ho, Wo)
    if bias is not None:
        y = y + bias.view(1, -1, 1, 1, 1)
    return y


def dcn2d(x, offset, mask, weight, bias=None, stride=1, padding=0, dilation=1, groups=1,
          deformable_groups=1):
    """Differentiable fp64 DCN 2-D (v1 if mask is None): bilinear, zero-padded sampling with torch's
    2-D grid_sample; offset channel 2k = row, 2k+1 = column displacement of tap k = i*kw + j."""
    t2 = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v,) * 2
    s, p, d = t2(stride), t2(padding), t2(dilation)
    B, Cin, H, W = x.shape
    Cout, cpg, kh, kw = weight.shape
    K = kh * kw
    Ho, Wo = [(S + 2 * pp - (dd * (k - 1) + 1)) // ss + 1
              for S, pp, dd, k, ss in zip((H, W), p, d, (kh, kw), s)]
    qh = (torch.arange(Ho, dtype=x.dtype) * s[0] - p[0])[:, None]
    qw = (torch.arange(Wo, dtype=x.dtype) * s[1] - p[1])[None, :]
    cpd = Cin // deformable_groups
    col = []
    for b in range(B):
        per_dg = []
        for g in range(deformable_groups):
            xs = x[b:b + 1, g * cpd:(g + 1) * cpd]
            taps = []
            for k in range(K):
                i, j = k // kw, k % kw
                ph = qh + i * d[0] + offset[b, (g * K + k) * 2]
                pw = qw + j * d[1] + offset[b, (g * K + k) * 2 + 1]
                grid = torch.stack([2 * pw / max(W - 1, 1) - 1, 2 * ph / max(H - 1, 1) - 1], -1)
                v = F.grid_sample(xs, grid[None], mode="bilinear", padding_mode="zeros",
                                  align_corners=True)[0]
                if mask is not None:
                    v = v * mask[b, g * K + k][None]
                taps.append(v)
            per_dg.append(torch.stack(taps, 1))
        col.append(torch.cat(per_dg, 0))
    col = torch.stack(col).reshape(B, groups, Cin // groups, K, Ho, Wo)
    wg = weight.reshape(groups, Cout // groups, cpg, K)
    y = torch.einsum("bgckhw,gock->bgohw", col, wg).reshape(B, Cout, Ho, Wo)
    if bias is not None:
        y = y + bias.view(1, -1, 1, 1)
    return y
