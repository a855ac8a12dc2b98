"""Pins the oracle's samplers (semantics S) without retyping its formula.

* order 1: torch's grid_sample(border, align_corners=True) times the closed-interval mask
* order 1 edges: values that follow from the definition (replicate within one voxel of the
  border, zero beyond it, CLOSED interval at exactly -1 and S)
* order 0: a hand-written answer table on a 3^3 volume including the 0.5 ties (low index wins)
"""
import itertools

import torch

from torch_ref import sample_border


def test_linear_matches_grid_sample(oracle):
    g = torch.Generator().manual_seed(0)
    vol = torch.randn(5, 6, 7, generator=g, dtype=torch.float64)
    pts = torch.rand(400, 3, generator=g, dtype=torch.float64) * torch.tensor([8., 9., 10.]) - 1.5
    ref = sample_border(vol[None], pts[:, 0], pts[:, 1], pts[:, 2])[0]
    for p, r in zip(pts, ref):
        got = oracle.sample_clamped(vol, p[0], p[1], p[2], order=1)
        assert abs(got - float(r)) < 1e-12


def test_linear_edge_table(oracle):
    # 1-D ramp along x embedded in a 1x1x4 volume: v = [10, 20, 40, 80]
    vol = torch.tensor([10., 20., 40., 80.], dtype=torch.float64).reshape(1, 1, 4)
    cases = {
        -1.0000001: 0.0,   # outside the closed interval
        -1.0: 10.0,        # exactly -1 is INSIDE and snaps to voxel 0
        -0.5: 10.0, 0.0: 10.0,
        0.25: 12.5, 1.5: 30.0, 2.75: 70.0,
        3.0: 80.0, 3.5: 80.0,   # replicate beyond the last voxel
        4.0: 80.0,         # exactly S is INSIDE
        4.0000001: 0.0,
    }
    for x, want in cases.items():
        assert abs(oracle.sample_clamped(vol, 0.0, 0.0, x, order=1) - want) < 1e-9, x
    # the same rule on the other two axes
    assert oracle.sample_clamped(vol.reshape(1, 4, 1), 0.0, 4.0, 0.0) == 80.0
    assert oracle.sample_clamped(vol.reshape(4, 1, 1), 4.0000001, 0.0, 0.0) == 0.0
    assert oracle.sample_clamped(vol.reshape(4, 1, 1), -1.0, 0.0, 0.0) == 10.0


def test_linear_is_exact_at_voxels_and_trilinear_inside(oracle):
    g = torch.Generator().manual_seed(1)
    vol = torch.randn(3, 4, 5, generator=g, dtype=torch.float64)
    for z, y, x in itertools.product(range(3), range(4), range(5)):
        assert oracle.sample_clamped(vol, z, y, x) == float(vol[z, y, x])
    # centre of a cell = mean of its 8 corners
    got = oracle.sample_clamped(vol, 0.5, 1.5, 2.5)
    assert abs(got - float(vol[0:2, 1:3, 2:4].mean())) < 1e-12


def test_nearest_table(oracle):
    vol = torch.arange(27, dtype=torch.float64).reshape(3, 3, 3)
    # per-axis rule written out by hand: coordinate -> picked index (size 3)
    axis = {-1.5: None, -1.0: 0, -0.2: 0, 0.0: 0, 0.49: 0, 0.5: 0, 0.51: 1, 1.0: 1, 1.5: 1,
            1.500001: 2, 2.0: 2, 2.4: 2, 2.9: 2, 3.0: 2, 3.01: None}
    for (z, iz), (y, iy), (x, ix) in itertools.product(axis.items(), repeat=3):
        want = 0.0 if None in (iz, iy, ix) else float(vol[iz, iy, ix])
        assert oracle.sample_clamped(vol, z, y, x, order=0) == want, (z, y, x)


# ---- order 3 -----------------------------------------------------------------------------------
def _hermite_axis(arr, v, axis):
    """Textbook cubic Hermite spline through the samples of `arr` along `axis`, tangents = central
    differences, evaluated at coordinate v >= 0 of an array whose borders were edge-padded by 3."""
    import numpy as np
    base = int(np.floor(v))
    u = v - base
    take = lambda i: np.take(arr, base + 3 + i, axis=axis)
    p0, p1, p2, p3 = take(-1), take(0), take(1), take(2)
    m1, m2 = (p2 - p0) / 2, (p3 - p1) / 2
    h00, h10 = 2 * u ** 3 - 3 * u ** 2 + 1, u ** 3 - 2 * u ** 2 + u
    h01, h11 = -2 * u ** 3 + 3 * u ** 2, u ** 3 - u ** 2
    return h00 * p1 + h10 * m1 + h01 * p2 + h11 * m2


def test_cubic_matches_hermite_spline_on_edge_padded_copy(oracle):
    import numpy as np
    g = torch.Generator().manual_seed(2)
    vol = torch.randn(5, 6, 7, generator=g, dtype=torch.float64)
    padded = np.pad(vol.numpy(), 3, mode="edge")
    # coordinates over the whole live range [0, S] (above S-1 the spline runs on repeated voxels)
    pts = torch.rand(300, 3, generator=g, dtype=torch.float64) * torch.tensor([5., 6., 7.])
    for z, y, x in pts.tolist():
        want = _hermite_axis(_hermite_axis(_hermite_axis(padded, x, 2), y, 1), z, 0)
        assert abs(oracle.sample_cubic(vol, z, y, x) - float(want)) < 1e-12
    # 2-D images: same spline without the z axis
    img = vol[0]
    for _, y, x in pts[:100].tolist():
        want = _hermite_axis(_hermite_axis(padded[3], x, 1), y, 0)
        assert abs(oracle.sample_cubic(img, 0.0, y, x) - float(want)) < 1e-12


def test_cubic_reproduces_quadratics_and_voxels(oracle):
    z, y, x = torch.meshgrid(torch.arange(6.), torch.arange(7.), torch.arange(8.), indexing="ij")
    f = lambda z, y, x: (1 + 0.5 * z - 0.25 * z * z) * (2 - y + 0.125 * y * y) * (x * x - 3 * x + 0.5)
    vol = f(z, y, x).double()
    g = torch.Generator().manual_seed(3)
    # away from the border (all four taps are real voxels) the spline is exact for quadratics
    pts = 1 + torch.rand(200, 3, generator=g, dtype=torch.float64) * torch.tensor([3., 4., 5.])
    for pz, py, px in pts.tolist():
        assert abs(oracle.sample_cubic(vol, pz, py, px) - f(pz, py, px)) < 1e-9
    rnd = torch.randn(3, 4, 5, generator=g, dtype=torch.float64)
    for iz, iy, ix in itertools.product(range(3), range(4), range(5)):
        assert oracle.sample_cubic(rnd, iz, iy, ix) == float(rnd[iz, iy, ix])
    # weights sum to one: a constant volume stays constant everywhere inside [-1, S]
    const = torch.full((3, 4, 5), 7.0, dtype=torch.float64)
    for pz, py, px in [(-1, -1, -1), (0.3, 3.7, 4.9), (3, 4, 5), (2.5, 0.1, 4.01)]:
        assert abs(oracle.sample_cubic(const, pz, py, px) - 7.0) < 1e-12


def test_cubic_edge_table(oracle):
    # answers worked out by hand from "taps base-1..base+2 clamped into the image"
    vol = torch.tensor([10., 20., 40., 80.], dtype=torch.float64).reshape(1, 1, 4)
    cases = {
        -1.0000001: 0.0, -1.0: 10.0, -0.5: 10.0, 0.0: 10.0,
        0.5: 13.75,        # taps 10,10,20,40 with weights (-1, 9, 9, -1)/16
        1.5: 28.125,       # taps 10,20,40,80: (-10 + 180 + 360 - 80) / 16
        3.0: 80.0,
        3.5: 82.5,         # taps 40,80,80,80: overshoots past the last voxel (no fold at S-1)
        4.0: 80.0,         # exactly S: base = S, fraction 0, all taps clamp to the last voxel
        4.0000001: 0.0,
    }
    for x, want in cases.items():
        assert abs(oracle.sample_cubic(vol, 0.0, 0.0, x) - want) < 1e-9, x
    assert abs(oracle.sample_cubic(vol.reshape(1, 4, 1), 0.0, 3.5, 0.0) - 82.5) < 1e-9
    assert abs(oracle.sample_cubic(vol.reshape(4, 1, 1), 3.5, 0.0, 0.0) - 82.5) < 1e-9
    assert oracle.sample_cubic(vol.reshape(4, 1, 1), 4.0000001, 0.0, 0.0) == 0.0
    assert abs(oracle.sample_cubic(vol.reshape(4, 1)[:, :], 0.0, 3.5, 0.0) - 82.5) < 1e-9  # 2-D


def test_decision_margin_hand_values(oracle):
    """Distance of nearest-neighbour samples from a tie / the edge of the void, by hand: an
    identity roi samples voxel centres (0.5 from every tie, the last voxel 1 from the edge S); a
    quarter-voxel shift puts samples at -0.25 (clamped to 0: no tie), 0.75 and 1.75; a half-voxel
    shift puts them exactly on ties; far outside the distance to the volume counts."""
    shape = (1, 1, 3, 3, 3)
    roi = lambda cx: torch.tensor([[0, cx, 1.5, 1.5, 3, 3, 3, 0, 0, 0.]])
    m = oracle.roi_decision_margin(shape, roi(1.5), (3, 3, 3), 1.0, 1, True, True)
    assert m.shape == (1, 3, 3, 3) and float(m[0, 0, 0, 0]) == 0.5 and float(m[0, 2, 2, 2]) == 1.0
    m = oracle.roi_decision_margin(shape, roi(1.25), (3, 3, 3), 1.0, 1, True, True)
    assert m[0, 0, 0].tolist() == [0.5, 0.25, 0.25]
    m = oracle.roi_decision_margin(shape, roi(2.0), (3, 3, 3), 1.0, 1, True, True)
    assert m[0, 0, 0].tolist() == [0.0, 0.0, 0.5]          # 0.5, 1.5 are ties; 2.5 clamps to 2
    m = oracle.roi_decision_margin(shape, roi(7.0), (3, 3, 3), 1.0, 1, True, True)
    assert m[0, 1, 1].tolist() == [2.5, 3.5, 4.5]          # samples at 5.5, 6.5, 7.5; S = 3
    # plain boxes, 2-D, two samples per cell: the smaller of the two distances
    m = oracle.roi_decision_margin((1, 1, 4, 4), torch.tensor([[0, 0.0, 0.0, 4.0, 4.0]]), (2, 2), 1.0, 2, True, False)
    assert m.shape == (1, 2, 2) and float(m[0, 0, 0]) == 0.0   # samples at 0.5 and 1.5
