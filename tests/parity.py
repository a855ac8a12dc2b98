"""Error measures shared by the GPU parity tests.

``rel_err(got, want)`` = max|got - want| / max(1e-30, max|want|): the largest deviation relative to
the scale of the reference result.  Tolerances (stated by the benchmark contract):
forward 1e-5 for fp32 tensors, 2e-3 for fp16 (fp32 arithmetic, fp16 storage; 4e-3 = one bf16 ulp
for bf16 whose 8-bit mantissa alone rounds by up to 2e-3), backward 1e-4 for fp32 (atomic
summation order), fp64 tensors 1e-11.
"""
import torch

FWD_TOL = {torch.float32: 1e-5, torch.float16: 2e-3, torch.bfloat16: 4e-3, torch.float64: 1e-11}
BWD_TOL = {torch.float32: 1e-4, torch.float16: 4e-3, torch.bfloat16: 8e-3, torch.float64: 1e-10}


def rel_err(got, want):
    got = got.detach().to("cpu", torch.float64)
    want = want.detach().to("cpu", torch.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    if want.numel() == 0:
        return 0.0
    return float((got - want).abs().max() / max(1e-30, float(want.abs().max())))


def assert_close(got, want, tol, what=""):
    e = rel_err(got, want)
    assert e <= tol, f"{what}: rel err {e:.3e} > {tol:.1e}"
    return e


# Coordinate rounding of the kernels, in voxels: 16-bit tensors go through fp32 box-relative
# coordinates in the tiled resampler (ulp of a ~100-voxel box coordinate, three rounded FMAs);
# fp32 / fp64 tensors through fp64 coordinates whose operation order differs from the oracle's.
NEAREST_EPS = {torch.float16: 2e-5, torch.bfloat16: 2e-5, torch.float32: 1e-9, torch.float64: 1e-9}


def assert_nearest(got, want, margin, dtype, what=""):
    """Order 0 picks voxels: outputs [R, C, ...] must EQUAL the oracle's (to the rounding of the
    storage type where several samples are averaged) except in cells whose sample lies within the
    kernel's coordinate rounding of a decision of the sampler (``margin`` [R, ...] from
    ``oracle.roi_decision_margin``): there the other neighbour is as legitimate as the oracle's.
    Returns the fraction of cells that differ."""
    got = got.detach().to("cpu", torch.float64)
    want = want.detach().to("cpu", torch.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    if want.numel() == 0:
        return 0.0
    den = max(1e-30, float(want.abs().max()))
    cells = ((got - want).abs() > FWD_TOL[dtype] * den).any(dim=1)
    unexplained = cells & (margin > NEAREST_EPS[dtype])
    n = int(unexplained.sum())
    assert n == 0, (f"{what}: {n} differing cells are not within {NEAREST_EPS[dtype]:g} voxel of a tie "
                    f"(smallest margin among them {float(margin[unexplained].min()):.3e})")
    return float(cells.double().mean())
