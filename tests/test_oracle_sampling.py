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
