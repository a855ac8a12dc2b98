"""Seeded random sweeps of the hot path against the fp64 oracle: shapes, roi geometry, sampling
grids, orders, layer hyper-parameters and dtypes are drawn per case (odd sizes, rois partly or
wholly outside, degenerate extents, 16-byte and ragged rows, channel counts on either side of the
matrix-core kernels' limits).  Each sweep runs a few hundred tiny cases in a few seconds."""
import math
import random

import pytest
import torch

from parity import BWD_TOL, FWD_TOL, NEAREST_EPS, assert_nearest, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.float16, torch.bfloat16, torch.float64]


@pytest.fixture(scope="module")
def ops():
    import medvision_amd.ops as ops_
    from medvision_amd import _lib
    _lib.load()
    return ops_


def _warp_margin(shape, off):
    """Distance of every warped sample q + off[q] from a decision of the nearest sampler (a 0.5 tie
    or the edge of the open interval (-1, S)), [B, *spatial]; same rule as the oracle's
    ``roi_decision_margin``."""
    spatial = shape[2:]
    grids = torch.meshgrid(*[torch.arange(n, dtype=torch.float64) for n in spatial], indexing="ij")
    inside = torch.full((shape[0], *spatial), 1e300, dtype=torch.float64)
    outside = torch.zeros_like(inside)
    for a, n in enumerate(spatial):
        v = grids[a][None] + off[:, a].double()
        edge = torch.minimum((v + 1).abs(), (v - n).abs())
        out = (v <= -1) | (v >= n)
        vc = v.clamp(min=0)
        base = vc.floor()
        tie = torch.where(base < n - 1, (vc - base - 0.5).abs(), torch.full_like(v, 1e300))
        inside = torch.minimum(inside, torch.where(out, torch.full_like(v, 1e300), torch.minimum(edge, tie)))
        outside = torch.maximum(outside, torch.where(out, edge, torch.zeros_like(v)))
    return torch.where(outside > 0, outside, inside)


def _roi_case(seed):
    rnd = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    ndim = rnd.choice([2, 3])
    rotated = rnd.random() < 0.6
    big = rnd.random() < 0.25
    size = [rnd.randint(1, 70 if big else 24) for _ in range(ndim)]
    batch = rnd.randint(1, 3)
    channels = rnd.choice([1, 2]) if big else rnd.choice([1, 1, 2, 3, 5, 33])
    dtype = rnd.choice(DTYPES)
    out = [rnd.randint(1, 40 if big else 12) for _ in range(ndim)]
    n = rnd.randint(1, 5)
    scale = rnd.choice([0.25, 0.5, 1.0, 1.0, 2.0])
    sr = rnd.choice([-1, 0, 1, 1, 2, 3])
    order = rnd.choice([0, 1, 1, 1])
    aligned = rnd.random() < 0.6
    feat = torch.randn(batch, channels, *size, generator=g).to(dtype)
    ext = torch.tensor(size[::-1], dtype=torch.float32) / scale
    cols = {(2, False): 5, (3, False): 7, (2, True): 6, (3, True): 10}[(ndim, rotated)]
    rois = torch.zeros(n, cols)
    rois[:, 0] = torch.randint(0, batch, (n,), generator=g)
    if rotated:
        rois[:, 1:1 + ndim] = (torch.rand(n, ndim, generator=g) * 1.6 - 0.3) * ext
        rois[:, 1 + ndim:1 + 2 * ndim] = torch.rand(n, ndim, generator=g) * ext * rnd.choice([0.3, 1.0, 1.5, 2.5])
        rois[:, 1 + 2 * ndim:] = (torch.rand(n, cols - 1 - 2 * ndim, generator=g) - 0.5) * rnd.choice([0.0, 0.5, 2.0, 6.3])
    else:
        lo = (torch.rand(n, ndim, generator=g) * 1.4 - 0.3) * ext
        rois[:, 1:1 + ndim] = lo
        rois[:, 1 + ndim:] = lo + torch.rand(n, ndim, generator=g) * ext * rnd.choice([0.2, 0.8, 1.6])
    if rnd.random() < 0.2:   # a roi of zero extent
        rois[0, 1 + ndim:1 + 2 * ndim] = 0.0 if rotated else rois[0, 1:1 + ndim]
    return g, ndim, rotated, feat, rois, tuple(out), scale, sr, order, aligned, dtype


def test_roi_sweep(ops, oracle):
    for seed in range(7000, 7300):
        g, ndim, rotated, feat, rois, out, scale, sr, order, aligned, dtype = _roi_case(seed)
        mod = ops.RoIAlignRotated(out, scale, sr, aligned) if rotated else ops.RoIAlign(out, scale, sr)
        fg = feat.to(DEV).requires_grad_(True)
        got = mod(fg, rois.to(DEV), order=order)
        eff = 1 if order == 0 else sr
        want = oracle.roi_align_forward(feat, rois, out, scale, eff, aligned, order, rotated)
        what = f"seed {seed}: {ndim}-D rotated={rotated} {tuple(feat.shape)} -> {out} sr={sr} order={order} {dtype}"
        if order == 0:
            margin = oracle.roi_decision_margin(feat.shape, rois, out, scale, eff, aligned, rotated)
            assert_nearest(got, want, margin, dtype, what)
            continue
        assert rel_err(got, want) <= FWD_TOL[dtype], what
        gy = torch.randn(got.shape, generator=g).to(dtype)
        got.backward(gy.to(DEV))
        gwant = oracle.roi_align_backward(gy, rois, feat.shape, scale, eff, aligned, order, rotated)
        assert rel_err(fg.grad, gwant) <= BWD_TOL[dtype], what + " (backward)"


def test_pooled_many_rois_sweep(ops, oracle):
    """fp16 heads with many rois on small maps: the matrix-core pooled forward from the input and from
    the blocked copy of the features (widths that are and are not multiples of four, channel counts
    around the tile and chunk sizes, 2-D and 3-D, boxes inside, across and outside the volume)."""
    for seed in range(80):
        rnd = random.Random(seed)
        g = torch.Generator().manual_seed(seed)
        ndim = rnd.choice([2, 3])
        size = [rnd.randint(1, 20) for _ in range(ndim - 1)] + [4 * rnd.randint(1, 9) if rnd.random() < 0.8 else rnd.randint(1, 30)]
        channels, batch = rnd.choice([1, 3, 4, 8, 17, 64, 130]), rnd.randint(1, 3)
        feat = torch.randn(batch, channels, *size, generator=g).half()
        out = [rnd.randint(1, 8) for _ in range(ndim)]
        cells, voxels = 1, batch
        for o in out:
            cells *= o
        for n in size:
            voxels *= n
        count = max(1, min(3000, int(voxels / cells * rnd.choice([0.5, 1.0, 1.5, 3.0])) + 1))
        scale, sr = rnd.choice([0.5, 1.0, 1.0, 2.0]), rnd.choice([0, 1, 2, 2, 3])
        ext = torch.tensor(size[::-1], dtype=torch.float32) / scale
        lo = (torch.rand(count, ndim, generator=g) * 1.4 - 0.3) * ext
        hi = lo + torch.rand(count, ndim, generator=g) * ext * rnd.choice([0.1, 0.3, 0.8, 1.6])
        rois = torch.cat([torch.randint(0, batch, (count, 1), generator=g).float(), lo, hi], 1)
        got = ops.RoIAlign(tuple(out), scale, sr)(feat.to(DEV), rois.to(DEV))
        want = oracle.roi_align_forward(feat, rois, tuple(out), scale, sr)
        what = f"seed {seed}: {ndim}-D {tuple(feat.shape)} -> {out} x {count} rois, scale {scale}, sr {sr}"
        assert rel_err(got, want) <= FWD_TOL[torch.float16], what


def test_rotated_backward_sweep(ops, oracle):
    """Backward of resampling-sized rotated rois (tiles of the source boxes; fp64 tensors and narrow
    outputs: the gather over input voxels): volumes and images,
    orders 0 and 1, several rois per image, mirrored rois, rotations up to 180 degrees.  Among the
    seeds are cases in which a sample lies within 1e-5 of the edge of [-1, size], where it turns
    void, or of a nearest-neighbour tie: decided in fp32, each of them misses the tolerance."""
    seeds = [3024, 3061, 3080, 3091, 3097, 3100, 3106, 3108, 3109, 3114] + list(range(3000, 3016))
    for seed in seeds:
        rnd = random.Random(seed)
        g = torch.Generator().manual_seed(seed)
        ndim = rnd.choice([3, 3, 2])
        dtype = rnd.choice([torch.float32, torch.float16])
        hi = 72 if ndim == 3 else 200
        size = [rnd.randint(17, hi) for _ in range(ndim)]           # D, H, W
        batch = rnd.randint(1, 3)
        out = [max(16, int(s * rnd.choice([0.7, 1.0, 1.0, 1.3]))) for s in size]
        vol = torch.randn(batch, 1, *size, generator=g).to(dtype)
        xyz = torch.tensor(size[::-1], dtype=torch.float32)
        n = batch if rnd.random() < 0.7 else min(2 * batch, batch + 1)
        idx = torch.tensor([i % batch for i in range(n)], dtype=torch.float32)[:, None]
        ctr = xyz / 2 + (torch.rand(n, ndim, generator=g) * 2 - 1) * xyz * rnd.choice([0.05, 0.2, 0.5])
        ext = xyz * (0.5 + torch.rand(n, ndim, generator=g) * 1.2)
        if rnd.random() < 0.1:
            ext[0, 0] = -ext[0, 0]                                  # mirrored
        ang = (torch.rand(n, 3 if ndim == 3 else 1, generator=g) * 2 - 1) * math.radians(rnd.choice([5, 30, 90, 180]))
        rois = torch.cat([idx, ctr, ext, ang], 1)
        order = rnd.choice([1, 1, 0])
        x = vol.to(DEV).requires_grad_(True)
        y = ops.RoIAlignRotated(tuple(out), 1.0, 1, True)(x, rois.to(DEV), order=order)
        gy = torch.randn(y.shape, generator=g).to(dtype)
        y.backward(gy.to(DEV))
        want = oracle.roi_align_backward(gy, rois, vol.shape, 1.0, 1, True, order, True)
        what = f"seed {seed}: {ndim}-D {tuple(vol.shape)} -> {out}, {n} rois, order {order}, {dtype}"
        assert rel_err(x.grad, want) <= BWD_TOL[dtype], what


def test_resampling_backward_mixed_sweep(ops, oracle):
    """Backward of resampling-sized outputs through tiles of the source boxes: plain and rotated rois,
    1 - 3 channels, up to four rois that share images, spatial scales, reductions whose boxes exceed
    the tile, enlargements with many terms per voxel, bf16.  Order 0: cells whose sample sits within
    1e-9 voxel of a tie or of the void's edge carry no gradient (the rounding of the coordinate
    arithmetic decides them)."""
    for seed in range(5000, 5060):
        rnd = random.Random(seed)
        g = torch.Generator().manual_seed(seed)
        ndim = rnd.choice([3, 3, 2])
        dtype = rnd.choice([torch.float32, torch.float16, torch.bfloat16])
        rotated = rnd.random() < 0.6
        hi = 56 if ndim == 3 else 160
        size = [rnd.randint(5, hi) for _ in range(ndim)]           # D, H, W
        batch, channels = rnd.randint(1, 2), rnd.choice([1, 1, 2, 3])
        out = [max(16 if i == ndim - 1 else 4, int(s * rnd.choice([0.4, 0.7, 1.0, 1.0, 1.5]))) for i, s in enumerate(size)]
        while math.prod(out) < 4096:
            out = [o + 4 for o in out]
        xyz = torch.tensor(size[::-1], dtype=torch.float32)
        n = rnd.randint(1, 4)
        idx = torch.tensor([rnd.randint(0, batch - 1) for _ in range(n)], dtype=torch.float32)[:, None]
        ctr = xyz / 2 + (torch.rand(n, ndim, generator=g) * 2 - 1) * xyz * rnd.choice([0.05, 0.2, 0.6])
        ext = xyz * (0.3 + torch.rand(n, ndim, generator=g) * rnd.choice([0.5, 1.2, 3.0]))
        if rotated:
            if rnd.random() < 0.1:
                ext[0, 0] = -ext[0, 0]
            ang = (torch.rand(n, 3 if ndim == 3 else 1, generator=g) * 2 - 1) * math.radians(rnd.choice([0, 5, 30, 90, 180]))
            rois = torch.cat([idx, ctr, ext, ang], 1)
        else:
            rois = torch.cat([idx, ctr - ext / 2, ctr + ext / 2], 1)
        order = rnd.choice([1, 1, 0])
        scale = rnd.choice([1.0, 1.0, 0.5])
        rois[:, 1:1 + 2 * ndim] /= scale
        shape = (batch, channels, *size)
        gy = torch.randn(n, channels, *out, generator=g).to(dtype)
        if order == 0:
            margin = oracle.roi_decision_margin(shape, rois, tuple(out), scale, 1, True, rotated)
            gy = gy * (margin > NEAREST_EPS[torch.float32])[:, None].to(dtype)
        x = torch.zeros(shape, dtype=dtype, device=DEV, requires_grad=True)
        mod = (ops.RoIAlignRotated if rotated else ops.RoIAlign)(tuple(out), scale, 1)
        mod(x, rois.to(DEV), order=order).backward(gy.to(DEV))
        want = oracle.roi_align_backward(gy, rois, shape, scale, 1, True, order, rotated)
        what = f"seed {seed}: {ndim}-D {shape} -> {out}, {n} rois, rotated {rotated}, order {order}, scale {scale}, {dtype}"
        if float(want.abs().max()) > 0:
            assert rel_err(x.grad, want) <= BWD_TOL[dtype], what
        else:
            assert float(x.grad.abs().max()) == 0, what


def test_affine_and_warp_sweep(ops, oracle):
    """Larger outputs, so that the LDS-tiled resampler (orders 0 / 1 and 3) takes most cases."""
    for seed in range(8000, 8120):
        rnd = random.Random(seed)
        g = torch.Generator().manual_seed(seed)
        ndim = rnd.choice([2, 3])
        hi = 64 if ndim == 3 else 150
        size = [rnd.randint(1, hi) for _ in range(ndim)]
        if rnd.random() < 0.3:
            size[-1] = rnd.choice([8, 16, 24, 32, 40, 64])   # rows of whole 16-byte groups
        batch, channels = rnd.randint(1, 2), rnd.choice([1, 1, 1, 2, 3])
        dtype = rnd.choice(DTYPES)
        out = tuple(rnd.randint(1, hi) for _ in range(ndim))
        order = rnd.choice([0, 1, 1, 3, 3])
        sr = 1 if order == 0 else rnd.choice([1, 1, 1, 2, 0])
        scale = rnd.choice([0.5, 1.0, 1.0, 2.0])
        aligned = rnd.random() < 0.7
        feat = torch.randn(batch, channels, *size, generator=g).to(dtype)
        ext = torch.tensor(size[::-1], dtype=torch.float32) / scale
        n = rnd.randint(1, 3)
        cols = 6 if ndim == 2 else 10
        rois = torch.zeros(n, cols)
        rois[:, 0] = torch.randint(0, batch, (n,), generator=g)
        spread = rnd.choice([0.05, 0.2, 1.0])   # never exactly centred: no systematic .5 ties at order 0
        rois[:, 1:1 + ndim] = ext / 2 + (torch.rand(n, ndim, generator=g) - 0.5) * ext * spread
        rois[:, 1 + ndim:1 + 2 * ndim] = ext * (0.3 + torch.rand(n, ndim, generator=g) * rnd.choice([0.7, 1.0, 1.5]))
        rois[:, 1 + 2 * ndim:] = (torch.rand(n, cols - 1 - 2 * ndim, generator=g) - 0.5) * rnd.choice([0.0, 0.3, 1.0, 3.0])
        if aligned and sr == 1 and seed % 5 == 2:   # a mirrored roi (negative extent, bins run backwards)
            rois[-1, 1 + ndim + seed % ndim] *= -1.0
        what = f"seed {seed}: {ndim}-D {tuple(feat.shape)} -> {out} sr={sr} order={order} {dtype}"
        fn = ops.affine_3d if ndim == 3 else ops.affine_2d
        got = fn(feat.to(DEV), rois.to(DEV), out, scale, sr, aligned, order)
        want = oracle.roi_align_forward(feat, rois, out, scale, sr, aligned, order, True)
        if order == 0:
            margin = oracle.roi_decision_margin(feat.shape, rois, out, scale, sr, aligned, True)
            assert_nearest(got, want, margin, dtype, what)
        else:
            assert rel_err(got, want) <= FWD_TOL[dtype], what
        worder = rnd.choice([0, 1, 3])
        off = (torch.randn(batch, ndim, *size, generator=g) * rnd.choice([0.0, 0.7, 3.0])).to(dtype)
        warp = ops.apply_offset_3d if ndim == 3 else ops.apply_offset_2d
        gotw = warp(feat.to(DEV), off.to(DEV), worder)
        wantw = oracle.deform_warp(feat, off, worder)
        if worder == 0:
            assert_nearest(gotw, wantw, _warp_margin(feat.shape, off), dtype, what + " (warp order 0)")
        else:
            assert rel_err(gotw, wantw) <= FWD_TOL[dtype], what + f" (warp order {worder})"


def test_dcn_sweep(ops, oracle):
    assert _dcn_sweep(oracle, range(9000, 9260), tiles=False) > 200


def test_dcn_sweep_of_the_lds_scatter_path(ops, oracle):
    """Unit-stride layers with 32 or 64 channels per group and up to 160 output channels per group,
    volumes larger and smaller than a brick of positions, 1 to 125 taps: the layers whose input
    gradient goes through the LDS tiles (and their neighbours that just miss the conditions)."""
    assert _dcn_sweep(oracle, range(9500, 9580), tiles=True) > 60


def _dcn_sweep(oracle, seeds, tiles):
    from medvision_amd.ops.deform_conv_2d import deform_conv as dc2
    from medvision_amd.ops.deform_conv_3d import deform_conv as dc3
    from medvision_amd.ops.modulated_deform_conv_2d import modulated_deform_conv as mdc2
    from medvision_amd.ops.modulated_deform_conv_3d import modulated_deform_conv as mdc3
    ran = 0
    for seed in seeds:
        rnd = random.Random(seed)
        g = torch.Generator().manual_seed(seed)
        nd = rnd.choice([2, 3])
        modulated = rnd.random() < 0.5
        groups, dg = rnd.choice([1, 1, 2, 4]), rnd.choice([1, 1, 2])
        matrix = rnd.random() < 0.5   # channel counts the matrix-core kernels accept
        if tiles:
            groups = rnd.choice([1, 1, 2])
            cin, cout = rnd.choice([32, 32, 64]) * groups, rnd.choice([32, 64, 96, 128, 160]) * groups
            if cin % dg or (cin // dg) % 32:
                dg = 1
        elif matrix:
            cin, cout = rnd.choice([16, 32, 48]) * groups, rnd.choice([32, 64, 96]) * groups
            if cin % dg or (cin // dg) % 16:
                dg = 1
        else:
            cin, cout = groups * dg * rnd.randint(1, 3), groups * rnd.randint(1, 5)
        batch = rnd.randint(1, 3)
        size = [rnd.randint(2, 9 if matrix else 11) for _ in range(nd)]
        dtype = rnd.choice(DTYPES)
        if tiles:
            batch = rnd.randint(1, 2)
            size = [rnd.randint(3, 13) for _ in range(nd)] if nd == 3 else [rnd.randint(5, 40) for _ in range(nd)]
            dtype = rnd.choice([torch.float32, torch.float16, torch.bfloat16])
            kk = rnd.choice([1, 2, 3, 3, 3, 5]) if nd == 3 else rnd.choice([1, 3, 3, 5])
            k = [kk] * nd if rnd.random() < 0.7 else [rnd.randint(1, 3) for _ in range(nd)]
            st, pa, di = [1] * nd, [rnd.randint(0, 2)] * nd, [rnd.choice([1, 1, 2])] * nd
        elif modulated:   # one stride / padding / dilation for all axes, as the reference's layer
            k = [rnd.randint(1, 3)] * nd if rnd.random() < 0.5 else [rnd.randint(1, 3) for _ in range(nd)]
            st, pa, di = [rnd.randint(1, 2)] * nd, [rnd.randint(0, 2)] * nd, [rnd.randint(1, 2)] * nd
        else:
            k = [rnd.randint(1, 3) for _ in range(nd)]
            st = [rnd.randint(1, 2) for _ in range(nd)]
            pa = [rnd.randint(0, 2) for _ in range(nd)]
            di = [rnd.randint(1, 2) for _ in range(nd)]
        out = [(s + 2 * p - (d * (kk - 1) + 1)) // t + 1 for s, p, d, kk, t in zip(size, pa, di, k, st)]
        if min(out) < 1:
            continue
        ran += 1
        taps = math.prod(k)
        x = torch.randn(batch, cin, *size, generator=g)
        w = (torch.rand(cout, cin // groups, *k, generator=g) * 2 - 1) / math.sqrt(cin // groups * taps)
        b = torch.rand(cout, generator=g) * 2 - 1
        off = torch.randn(batch, dg * nd * taps, *out, generator=g) * rnd.choice([0.0, 0.5, 2.0, 6.0])
        if rnd.random() < 0.3:
            off = off.round()   # lattice points: the offset gradient is one-sided there, not compared
        mask = torch.sigmoid(torch.randn(batch, dg * taps, *out, generator=g)) if modulated else None
        x, w, b, off = [t.to(dtype) for t in (x, w, b, off)]
        mask = None if mask is None else mask.to(dtype)
        what = (f"seed {seed}: {nd}-D v{2 if modulated else 1} groups={groups} dg={dg} {cin}->{cout} "
                f"{size} k={k} stride={st} pad={pa} dil={di} {dtype}")
        xs, offs, ws, bs = [t.to(DEV).requires_grad_(True) for t in (x, off, w, b)]
        ms = None if mask is None else mask.to(DEV).requires_grad_(True)
        if modulated:
            y = (mdc3 if nd == 3 else mdc2)(xs, offs, ms, ws, bs, st[0], pa[0], di[0], groups, dg)
        else:
            y = (dc3 if nd == 3 else dc2)(xs, offs, ws, bs, tuple(st), tuple(pa), tuple(di), groups, dg, 64)
        want = oracle.dcn3d_forward(x, off, mask, w, b, tuple(st), tuple(pa), tuple(di), groups, dg)
        # bf16 matrix-core path: the blended columns are rounded to bf16 as well as the output
        ftol = FWD_TOL[dtype] * (1.5 if dtype == torch.bfloat16 else 1.0)
        assert rel_err(y, want) <= ftol, what
        gy = torch.randn(y.shape, generator=g).to(dtype)
        y.backward(gy.to(DEV))
        gx, goff, gm, gw, gb = oracle.dcn3d_backward(x, off, mask, w, gy, True, tuple(st), tuple(pa), tuple(di), groups, dg)
        tol = BWD_TOL[dtype]
        assert rel_err(xs.grad, gx) <= tol, what + " (grad input)"
        assert rel_err(ws.grad, gw) <= tol, what + " (grad weight)"
        assert rel_err(bs.grad, gb) <= tol, what + " (grad bias)"
        on_lattice = bool((off == off.round()).all()) and float(off.abs().max()) > 0
        if not on_lattice:
            assert rel_err(offs.grad, goff) <= tol, what + " (grad offset)"
        if modulated:
            assert rel_err(ms.grad, gm) <= tol, what + " (grad mask)"
    return ran


def test_resampling_backward_sweep(ops, oracle):
    """Backward of resampling-sized problems (one sample per cell, outputs about as large as the
    image, a roi or two per image): these take the atomic-free gather kernel.  Plain and rotated
    rois that reach beyond every border, up- and down-sampling, zero extents, orders 0 and 1."""
    for seed in range(9500, 9580):
        rnd = random.Random(seed)
        g = torch.Generator().manual_seed(seed)
        ndim = rnd.choice([2, 3])
        rotated = rnd.random() < 0.7
        hi = 40 if ndim == 3 else 120
        lo = 12 if ndim == 3 else 50
        size = [rnd.randint(lo, hi) for _ in range(ndim)]
        out = tuple(rnd.randint(max(lo, s // 2), hi) for s in size)   # >= 4096 cells, >= plane / 8
        batch, channels = rnd.randint(1, 3), rnd.choice([1, 1, 2])
        n = rnd.randint(1, 2 * batch)
        dtype = rnd.choice(DTYPES)
        order = rnd.choice([0, 1, 1, 1])
        scale = rnd.choice([0.5, 1.0, 1.0, 2.0])
        aligned = rnd.random() < 0.7
        feat = torch.randn(batch, channels, *size, generator=g).to(dtype)
        ext = torch.tensor(size[::-1], dtype=torch.float32) / scale
        cols = {(2, False): 5, (3, False): 7, (2, True): 6, (3, True): 10}[(ndim, rotated)]
        rois = torch.zeros(n, cols)
        rois[:, 0] = torch.randint(0, batch, (n,), generator=g)
        if rotated:
            rois[:, 1:1 + ndim] = ext / 2 + (torch.rand(n, ndim, generator=g) - 0.5) * ext * rnd.choice([0.1, 0.5, 1.2])
            rois[:, 1 + ndim:1 + 2 * ndim] = ext * (0.2 + torch.rand(n, ndim, generator=g) * rnd.choice([0.8, 1.3, 2.5]))
            rois[:, 1 + 2 * ndim:] = (torch.rand(n, cols - 1 - 2 * ndim, generator=g) - 0.5) * rnd.choice([0.0, 0.4, 1.2, 6.3])
        else:
            start = (torch.rand(n, ndim, generator=g) * 0.8 - 0.3) * ext
            rois[:, 1:1 + ndim] = start
            rois[:, 1 + ndim:] = start + ext * (0.2 + torch.rand(n, ndim, generator=g) * rnd.choice([0.8, 1.5]))
        if rnd.random() < 0.15:
            rois[0, 1 + ndim:1 + 2 * ndim] = 0.0 if rotated else rois[0, 1:1 + ndim]   # zero extent
        if rotated and aligned and seed % 4 == 1:
            # a mirrored roi: aligned rotated rois keep a negative extent (the bins run backwards)
            rois[-1, 1 + ndim + seed % ndim] *= -1.0
        mod = ops.RoIAlignRotated(out, scale, 1, aligned) if rotated else ops.RoIAlign(out, scale, 1)
        fg = feat.to(DEV).requires_grad_(True)
        got = mod(fg, rois.to(DEV), order=order)
        gy = torch.randn(got.shape, generator=g).to(dtype)
        if order == 0:
            # a sample within the kernel's coordinate rounding of a .5 tie may send its gradient to
            # the other neighbour: such cells carry no gradient in this test, all others must land
            # on the oracle's voxel
            margin = oracle.roi_decision_margin(feat.shape, rois, out, scale, 1, aligned, rotated)
            gy = gy * (margin > NEAREST_EPS[dtype])[:, None].to(dtype)
        got.backward(gy.to(DEV))
        want = oracle.roi_align_backward(gy, rois, feat.shape, scale, 1, aligned, order, rotated)
        what = f"seed {seed}: {ndim}-D rotated={rotated} {tuple(feat.shape)} -> {out} rois={n} order={order} {dtype}"
        # no atomics, fp32 sums, one rounding per voxel: 16-bit results carry half an ulp
        tol = BWD_TOL[dtype] if dtype in (torch.float32, torch.float64) else FWD_TOL[dtype]
        assert rel_err(fg.grad, want) <= tol, what


def test_pooled_sweep(ops, oracle):
    """Plain boxes with at most 16 cells per axis (the pooled kernels): boxes from a fraction of a
    voxel to more than a hundred voxels wide, elongated volumes, fixed and adaptive sampling grids."""
    for seed in range(9600, 9750):
        rnd = random.Random(seed)
        g = torch.Generator().manual_seed(seed)
        ndim = rnd.choice([2, 3])
        size = [rnd.randint(1, 130) for _ in range(2)] if ndim == 2 else \
            [rnd.randint(1, 20), rnd.randint(1, 40), rnd.randint(1, 110)]
        batch, channels = rnd.randint(1, 2), rnd.choice([1, 2, 3, 7, 40])
        dtype = rnd.choice([torch.float32, torch.float16, torch.bfloat16])
        out = tuple(rnd.randint(1, 16) for _ in range(ndim))
        n = rnd.randint(1, 6)
        scale = rnd.choice([0.25, 0.5, 1.0, 1.0])
        sr = rnd.choice([-1, 0, 1, 2, 2, 3, 4])
        feat = torch.randn(batch, channels, *size, generator=g).to(dtype)
        ext = torch.tensor(size[::-1], dtype=torch.float32) / scale
        rois = torch.zeros(n, 1 + 2 * ndim)
        rois[:, 0] = torch.randint(0, batch, (n,), generator=g)
        lo = (torch.rand(n, ndim, generator=g) * 1.3 - 0.2) * ext
        rois[:, 1:1 + ndim] = lo
        rois[:, 1 + ndim:] = lo + torch.rand(n, ndim, generator=g) * ext * rnd.choice([0.1, 0.5, 1.0, 1.5])
        what = f"seed {seed}: {ndim}-D {tuple(feat.shape)} -> {out} rois={n} scale={scale} sr={sr} {dtype}"
        fg = feat.to(DEV).requires_grad_(True)
        got = ops.RoIAlign(out, scale, sr)(fg, rois.to(DEV))
        want = oracle.roi_align_forward(feat, rois, out, scale, sr, True, 1, False)
        assert rel_err(got, want) <= FWD_TOL[dtype], what
        gy = torch.randn(got.shape, generator=g).to(dtype)
        got.backward(gy.to(DEV))
        gwant = oracle.roi_align_backward(gy, rois, feat.shape, scale, sr, True, 1, False)
        assert rel_err(fg.grad, gwant) <= BWD_TOL[dtype], what + " (backward)"
