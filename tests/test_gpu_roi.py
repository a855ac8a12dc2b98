"""GPU parity of RoIAlign / RoIAlignRotated / affine (through medvision_amd.ops -> _C -> C ABI)
against the fp64 oracle on the same seeded inputs, plus the reference test-script's crop
identities and size-independent properties at the benchmark's full sizes."""
import math

import pytest
import torch

from parity import BWD_TOL, FWD_TOL, NEAREST_EPS, assert_close, assert_nearest, rel_err
import workloads as wl

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.float16, torch.bfloat16, torch.float64]


@pytest.fixture(scope="module")
def ops():
    import medvision_amd.ops as ops_
    from medvision_amd import _lib
    _lib.load()
    return ops_


def _random_case(ndim, rotated, seed, R=12):
    g = wl.gen(seed)
    size = (9, 12, 14)[3 - ndim:]
    feat = torch.randn(2, 5, *size, generator=g)
    ext = torch.tensor(size[::-1], dtype=torch.float32)
    cols = {(2, False): 5, (3, False): 7, (2, True): 6, (3, True): 10}[(ndim, rotated)]
    rois = torch.zeros(R, cols)
    rois[:, 0] = torch.randint(0, 2, (R,), generator=g)
    if rotated:
        rois[:, 1:1 + ndim] = torch.rand(R, ndim, generator=g) * ext * 2.0
        rois[:, 1 + ndim:1 + 2 * ndim] = (torch.rand(R, ndim, generator=g) * 0.9 + 0.05) * ext * 2.4
        rois[:, 1 + 2 * ndim:] = (torch.rand(R, cols - 1 - 2 * ndim, generator=g) - 0.5) * 2.0
        rois[0, 1 + ndim:1 + 2 * ndim] = 0.3
    else:
        lo = (torch.rand(R, ndim, generator=g) * 1.2 - 0.2) * ext * 2.0
        rois[:, 1:1 + ndim] = lo
        rois[:, 1 + ndim:] = lo + torch.rand(R, ndim, generator=g) * ext * 1.6
        rois[0, 1 + ndim:] = rois[0, 1:1 + ndim] + 0.4
    return feat, rois


def _module(ops, ndim, rotated, out_size, scale, sr, aligned):
    if rotated:
        return ops.RoIAlignRotated(out_size, scale, sr, aligned)
    return ops.RoIAlign(out_size, scale, sr)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("ndim,rotated", [(2, False), (3, False), (2, True), (3, True)])
@pytest.mark.parametrize("sr,aligned,order", [(2, True, 1), (0, False, 1), (1, True, 0), (-1, True, 1)])
def test_forward_backward_vs_oracle(ops, oracle, dtype, ndim, rotated, sr, aligned, order):
    feat, rois = _random_case(ndim, rotated, seed=100 * ndim + 10 * rotated + sr + 3)
    feat = feat.to(dtype)
    out_size = (3, 4, 5)[3 - ndim:]
    mod = _module(ops, ndim, rotated, out_size, 0.5, sr, aligned)
    fg = feat.to(DEV).requires_grad_(True)
    out = mod(fg, rois.to(DEV), order=order)
    eff_sr = 1 if order == 0 else sr
    want = oracle.roi_align_forward(feat, rois, out_size, 0.5, eff_sr, aligned, order, rotated)
    assert out.dtype == dtype and out.shape == want.shape
    assert_close(out, want, FWD_TOL[dtype], "forward")
    gy = torch.randn(out.shape, generator=wl.gen(7)).to(dtype)
    out.backward(gy.to(DEV))
    gwant = oracle.roi_align_backward(gy, rois, feat.shape, 0.5, eff_sr, aligned, order, rotated)
    assert fg.grad.dtype == dtype
    assert_close(fg.grad, gwant, BWD_TOL[dtype], "backward")


def test_reference_crop_identities(ops):
    """Known answers of the reference's own script (test/ops_test_RoIAlign.py:68,86,121,124,131)."""
    g = wl.gen(0)
    img = torch.randn(2, 1, 400, 440, generator=g).to(DEV)
    rois = torch.tensor([[0, 161.5, 111.5, 417.5, 367.5]] * 3).to(DEV)
    out = ops.RoIAlign((256, 256), 1.0, 1)(img, rois)
    assert torch.equal(out[2, 0], img[0, 0, 112:368, 162:418])
    out = ops.RoIAlign((256, 256), 1.0, 1)(img.half(), rois.half())   # the script runs in fp16
    assert torch.equal(out[0, 0], img.half()[0, 0, 112:368, 162:418])
    rr = torch.tensor([[0, 290., 240., 256., 256., 0.0]]).to(DEV)
    out = ops.RoIAlignRotated((256, 256), 1.0, 1)(img, rr)
    assert torch.equal(out[0, 0], img[0, 0, 112:368, 162:418])
    vol = torch.randn(1, 1, 95, 192, 190, generator=g).to(DEV)
    r3 = torch.tensor([[0, 9.5, 9.5, 59.5, 187.5, 187.5, 89.5]]).to(DEV)
    out = ops.RoIAlign((30, 178, 178), 1.0, 1)(vol, r3)
    assert torch.equal(out[0, 0], vol[0, 0, 60:90, 10:188, 10:188])
    rr3 = torch.tensor([[0, 99., 99., 75., 178, 178, 30, 0, 0, 0]]).to(DEV)
    for order in (0, 1):
        out = ops.RoIAlignRotated((30, 178, 178), 1.0, 1)(vol, rr3, order=order)
        assert torch.equal(out[0, 0], vol[0, 0, 60:90, 10:188, 10:188])


def test_edge_cases_and_errors(ops):
    feat = torch.randn(2, 3, 6, 7, 8, device=DEV)
    empty = ops.RoIAlignRotated((2, 2, 2), 1.0, 2)(feat, torch.zeros(0, 10, device=DEV))
    assert empty.shape == (0, 3, 2, 2, 2)
    # batch index outside [0, N): zeros instead of an out-of-bounds read
    bad = torch.tensor([[5, 4., 3., 3., 4., 4., 4., 0, 0, 0], [-1, 4., 3., 3., 4., 4., 4., 0, 0, 0]], device=DEV)
    assert float(ops.RoIAlignRotated((2, 2, 2), 1.0, 2)(feat, bad).abs().max()) == 0.0
    with pytest.raises(RuntimeError, match="size_rois should be 10"):
        ops.RoIAlignRotated((2, 2, 2), 1.0, 2)(feat, torch.zeros(1, 7, device=DEV))
    with pytest.raises(RuntimeError, match="size_rois should be 7"):
        ops.RoIAlign((2, 2, 2), 1.0, 2)(feat, torch.zeros(1, 10, device=DEV))
    with pytest.raises(RuntimeError, match="size_rois should be 5"):
        ops.RoIAlign((2, 2), 1.0, 2)(feat[:, :, 0], torch.zeros(1, 7, device=DEV))
    with pytest.raises(RuntimeError, match="not implemented on CPU"):
        ops.RoIAlign((2, 2, 2), 1.0, 2)(feat.cpu(), torch.zeros(1, 7))
    with pytest.raises(AssertionError):
        ops.RoIAlign((2, 2, 2), 1.0, 2)(feat, torch.zeros(1, 7, device=DEV), order=3)
    # order 3 exists for the affine engine only; the RoIAlign bindings reject it like the reference
    from medvision_amd import _C
    with pytest.raises(RuntimeError, match="only support order = 0"):
        _C.roi_align_rotated_3d_forward(feat, torch.zeros(1, 10, device=DEV),
                                        torch.zeros(1, 3, 2, 2, 2, device=DEV), 2, 2, 2, 1.0, 2, True, 3)
    with pytest.raises(RuntimeError, match="order 2 is not supported"):
        _C.affine_3d(feat, torch.zeros(1, 10, device=DEV), torch.zeros(1, 3, 2, 2, 2, device=DEV),
                     2, 2, 2, 1.0, 2, True, 2)
    # non-contiguous features are accepted (made contiguous), result unchanged
    r = torch.tensor([[1, 1., 1., 1., 6., 5., 4.]], device=DEV)
    a = ops.RoIAlign((2, 2, 2), 1.0, 2)(feat, r)
    b = ops.RoIAlign((2, 2, 2), 1.0, 2)(feat.transpose(3, 4).contiguous().transpose(3, 4), r)
    assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_config2_affine_resampling_full_size(ops, oracle, dtype):
    """Benchmark configuration 2: [4,1,128^3] -> 128^3, one rotated full-volume roi per sample, sr=1."""
    g = wl.gen(1)
    vol = torch.randn(4, 1, 128, 128, 128, generator=g).to(dtype)
    rois = wl.affine_rois(g, 4, (128, 128, 128))
    got = ops.affine_3d(vol.to(DEV), rois.to(DEV), (128, 128, 128), 1.0, 1, True, 1)
    want = oracle.roi_align_forward(vol, rois, (128, 128, 128), 1.0, 1, True, 1, True)
    assert_close(got, want, FWD_TOL[dtype], "config 2 forward")
    same = ops.RoIAlignRotated((128, 128, 128), 1.0, 1, True)(vol.to(DEV), rois.to(DEV))
    assert torch.equal(same, got)
    # identity roi -> exact copy; nearest on the identity roi too
    ident = torch.tensor([[b, 64, 64, 64, 128, 128, 128, 0, 0, 0] for b in range(4)], dtype=torch.float32)
    for order in (0, 1):
        out = ops.affine_3d(vol.to(DEV), ident.to(DEV), (128, 128, 128), 1.0, 1, True, order)
        assert torch.equal(out.cpu(), vol)
    # nearest under rotation: every output is one of the input values of its sample or 0
    out0 = ops.affine_3d(vol.to(DEV), rois.to(DEV), (128, 128, 128), 1.0, 1, True, 0)
    want0 = oracle.roi_align_forward(vol, rois, (128, 128, 128), 1.0, 1, True, 0, True)
    # the tiled kernel rounds box-relative coordinates to fp32, so a sample within that distance
    # of a 0.5 tie may pick the other neighbour than the fp64 oracle: such cells, and only such
    # cells, may differ
    margin = oracle.roi_decision_margin(vol.shape, rois, (128, 128, 128), 1.0, 1, True, True)
    frac = assert_nearest(out0, want0, margin, dtype, "config 2 nearest")
    assert frac < 5e-5, f"nearest mismatches: {frac:.2e}"


def test_config2_backward_adjoint_full_size(ops, oracle):
    g = wl.gen(11)
    vol = torch.randn(4, 1, 128, 128, 128, generator=g)
    rois = wl.affine_rois(g, 4, (128, 128, 128))
    x = vol.to(DEV).requires_grad_(True)
    y = ops.RoIAlignRotated((128, 128, 128), 1.0, 1, True)(x, rois.to(DEV))
    gy = torch.randn(y.shape, generator=g)
    y.backward(gy.to(DEV))
    lhs = float((y.detach().double() * gy.to(DEV).double()).sum())
    rhs = float((x.detach().double() * x.grad.double()).sum())
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), 1.0)
    gwant = oracle.roi_align_backward(gy, rois, vol.shape, 1.0, 1, True, 1, True)
    assert_close(x.grad, gwant, BWD_TOL[torch.float32], "config 2 backward")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("order", [1, 0])
def test_backward_through_source_box_tiles(ops, oracle, dtype, order):
    """Backward of resampling-sized outputs (grid 1): output tiles add into an LDS tile of their source
    box.  Several channels, rois that overlap on one image, rotated and plain rois, images, and a
    strong reduction whose boxes exceed the LDS tile (every term then goes out as a single atomic)."""
    g = wl.gen(800 + order)

    def check(feat_shape, rois, out, rotated, what):
        gy = torch.randn(rois.shape[0], feat_shape[1], *out, generator=g).to(dtype)
        if order == 0:
            # plain boxes with rational bins put samples exactly on 0.5 ties, where the rounding of the
            # coordinate arithmetic decides: as in the forward tests those cells prove nothing
            margin = oracle.roi_decision_margin(feat_shape, rois, out, 1.0, 1, True, rotated)
            gy = gy * (margin > NEAREST_EPS[torch.float32])[:, None].to(dtype)
        x = torch.zeros(feat_shape, dtype=dtype, device=DEV, requires_grad=True)
        mod = (ops.RoIAlignRotated if rotated else ops.RoIAlign)(out, 1.0, 1)
        mod(x, rois.to(DEV), order=order).backward(gy.to(DEV))
        want = oracle.roi_align_backward(gy, rois, feat_shape, 1.0, 1, True, order, rotated)
        assert float(want.abs().max()) > 0
        assert_close(x.grad, want, BWD_TOL[dtype], what)

    rois = torch.cat([wl.affine_rois(g, 2, (48, 40, 24)), wl.affine_rois(g, 2, (48, 40, 24))[:1]])
    check((2, 3, 24, 40, 48), rois, (20, 24, 40), True, "rotated volumes")
    boxes = torch.tensor([[0, 2.3, 1.2, 0.5, 40.1, 33.3, 20.7], [1, -3.0, 5.0, 2.0, 30.0, 45.0, 30.0],
                          [1, 10.0, 3.0, 4.0, 52.0, 30.0, 18.0]])
    check((2, 2, 24, 40, 48), boxes, (18, 24, 32), False, "plain volumes")
    r2 = torch.tensor([[0, 45.0, 35.0, 80.0, 60.0, 0.4], [1, 40.0, 30.0, 100.0, 50.0, -1.2], [0, 30.0, 40.0, 50.0, 70.0, 2.0]])
    check((2, 3, 70, 90), r2, (72, 80), True, "rotated images")
    big = torch.tensor([[0, 64.0, 48.0, 24.0, 150.0, 110.0, 60.0, 0.2, -0.3, 0.5]])
    check((1, 2, 48, 96, 128), big, (16, 20, 24), True, "boxes beyond the tile")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("sr", [2, 3, 0, 6])
def test_backward_tiles_with_sampling_grids(ops, oracle, dtype, sr):
    """Backward of resampling-sized outputs with a sampling grid: fixed ratios, the adaptive grid
    ceil(roi extent / cells) per roi (rois of different extents on one call), and a ratio whose many
    samples over small bins leave too few bits per term for fp32 tensors (those tiles add term by term).
    Rotated and plain rois, volumes and images, forward checked along the way."""
    g = wl.gen(830 + max(sr, 0))

    def check(feat_shape, rois, out, rotated, what):
        feat = torch.randn(feat_shape, generator=g).to(dtype)
        x = feat.to(DEV).requires_grad_(True)
        mod = (ops.RoIAlignRotated if rotated else ops.RoIAlign)(out, 1.0, sr)
        y = mod(x, rois.to(DEV))
        # cells with a sample within coordinate rounding of the edge of [-1, size] prove nothing
        margin = oracle.roi_decision_margin(feat_shape, rois, out, 1.0, sr, True, rotated)
        keep = (margin > NEAREST_EPS[dtype])[:, None]
        want = oracle.roi_align_forward(feat, rois, out, 1.0, sr, True, 1, rotated)
        assert_close(y.detach().cpu() * keep, want * keep, FWD_TOL[dtype], what + ", forward")
        gy = (torch.randn(y.shape, generator=g) * keep).to(dtype)
        y.backward(gy.to(DEV))
        gwant = oracle.roi_align_backward(gy, rois, feat_shape, 1.0, sr, True, 1, rotated)
        assert float(gwant.abs().max()) > 0
        assert_close(x.grad, gwant, BWD_TOL[dtype], what + ", backward")

    rois = wl.affine_rois(g, 2, (48, 40, 24))
    rois[1, 4:7] *= 2.2                               # a roi that wants more samples per bin than the other
    check((2, 2, 24, 40, 48), rois, (18, 22, 36), True, "rotated volumes")
    boxes = torch.tensor([[0, 2.3, 1.2, 0.5, 40.1, 33.3, 20.7], [1, -3.0, 5.0, 2.0, 30.0, 45.0, 30.0],
                          [1, 10.0, 3.0, 4.0, 14.0, 9.0, 8.0]])       # the last one: bins far below a voxel
    check((2, 2, 24, 40, 48), boxes, (18, 24, 32), False, "plain volumes")
    r2 = torch.tensor([[0, 45.0, 35.0, 80.0, 60.0, 0.4], [1, 40.0, 30.0, 160.0, 110.0, -1.2]])
    check((2, 3, 70, 90), r2, (72, 80), True, "rotated images")


def test_backward_tiles_precision_over_a_wide_range_of_gradients(ops, oracle):
    """fp32 tensors: a tile's terms are rounded to 2^-(t+1) of the tile's largest gradient, t >= 19 at one
    sample per bin (32-bit fixed-point sums in LDS), so a gradient a million times smaller than its
    neighbours keeps three digits, not seven: the error is bounded per element against the largest
    gradient of the volume, and stated here."""
    g = wl.gen(840)
    rois = wl.affine_rois(g, 2, (48, 40, 24))
    shape, out = (2, 1, 24, 40, 48), (20, 24, 40)
    gy = torch.randn(2, 1, *out, generator=g) * torch.pow(10.0, -6.0 * torch.rand(2, 1, *out, generator=g))
    x = torch.zeros(shape, device=DEV, requires_grad=True)
    ops.RoIAlignRotated(out, 1.0, 1)(x, rois.to(DEV)).backward(gy.to(DEV))
    want = oracle.roi_align_backward(gy, rois, shape, 1.0, 1, True, 1, True)
    err = (x.grad.cpu().double() - want).abs()
    bound = 8 * 2.0 ** -20 * float(gy.abs().max())      # eight terms reach a voxel from one output voxel's sample
    assert float(err.max()) <= bound, f"largest error {float(err.max()):.3e} > {bound:.3e}"
    small = want.abs() < 1e-3 * float(want.abs().max())
    assert bool(small.any()) and float(err[small].max()) <= bound


def test_backward_tiles_with_zero_and_infinite_gradients(ops, oracle):
    """A grad_output of zeros leaves the gradient untouched; an infinity reaches the voxels the oracle
    sends it to (the tile that holds it adds its terms one by one, the others stay in fixed point)."""
    g = wl.gen(820)
    rois = wl.affine_rois(g, 2, (48, 40, 24))
    shape, out = (2, 1, 24, 40, 48), (20, 24, 40)
    for dtype in (torch.float32, torch.float16):
        x = torch.zeros(shape, dtype=dtype, device=DEV, requires_grad=True)
        y = ops.RoIAlignRotated(out, 1.0, 1)(x, rois.to(DEV))
        y.backward(torch.zeros_like(y))
        assert float(x.grad.abs().max()) == 0.0
        gy = torch.randn(2, 1, *out, generator=g).to(dtype)
        gy[1, 0, 9, 11, 17] = float("inf")
        x = torch.zeros(shape, dtype=dtype, device=DEV, requires_grad=True)
        ops.RoIAlignRotated(out, 1.0, 1)(x, rois.to(DEV)).backward(gy.to(DEV))
        want = oracle.roi_align_backward(gy, rois, shape, 1.0, 1, True, 1, True)
        got = x.grad.cpu().double()
        assert torch.equal(torch.isfinite(got), torch.isfinite(want)) and int((~torch.isfinite(want)).sum()) == 8
        assert torch.equal(got[~torch.isfinite(want)], want[~torch.isfinite(want)])
        fin = torch.isfinite(want)
        assert_close(torch.where(fin, got, torch.zeros_like(got)), torch.where(fin, want, torch.zeros_like(want)),
                     BWD_TOL[dtype], "finite part")


@pytest.mark.parametrize("shape,out,sr,extent,dtype", [
    ((2, 20, 30, 40, 48), (7, 7, 7), 2, (18, 30), torch.float16),     # dense matrices, channels-last sums
    ((2, 20, 30, 40, 48), (7, 7, 7), 2, (18, 30), torch.float32),     # dense matrices, planar sums
    ((2, 20, 30, 40, 48), (7, 7, 7), 2, (18, 30), torch.bfloat16),
    ((1, 8, 40, 44, 60), (6, 5, 7), 3, (28, 44), torch.float16),      # boxes beyond the dense matrices: tap tables
    ((1, 8, 40, 44, 60), (6, 5, 7), 3, (28, 44), torch.float32),
    ((2, 6, 24, 36, 40), (12, 10, 14), 1, (20, 34), torch.float16),   # more than 8 cells per axis
    ((2, 70, 90, 120), (14, 14), 2, (40, 64), torch.float32),         # images
])
def test_pooled_kernels_with_large_boxes(ops, oracle, shape, out, sr, extent, dtype):
    """Boxes of 18 - 64 voxels per axis with many channels: the pooled backward works through such a
    box in slabs of planes, so that a pass still takes enough channels for whole-sector atomics (it
    used to fall back to one atomic per corner of every sample: 240 ms instead of 19 ms for 1000 rois
    of 24^3 voxels x 256 channels)."""
    g = wl.gen(77)
    nd = len(shape) - 2
    size = torch.tensor(shape[2:][::-1], dtype=torch.float32)
    n = 6
    e = torch.minimum(extent[0] + torch.rand(n, nd, generator=g) * (extent[1] - extent[0]), size + 4)
    lo = torch.rand(n, nd, generator=g) * (size - e + 6) - 3
    rois = torch.cat([torch.randint(0, shape[0], (n, 1), generator=g).float(), lo, lo + e], 1)
    for order in (1, 0):
        feat = torch.randn(shape, generator=g).to(dtype)
        x = feat.to(DEV).requires_grad_(True)
        y = ops.RoIAlign(out, 1.0, sr)(x, rois.to(DEV), order=order)
        eff = 1 if order == 0 else sr
        assert_close(y, oracle.roi_align_forward(feat, rois, out, 1.0, eff, True, order, False), FWD_TOL[dtype], "forward")
        gy = torch.randn(y.shape, generator=g).to(dtype)
        y.backward(gy.to(DEV))
        assert_close(x.grad, oracle.roi_align_backward(gy, rois, shape, 1.0, eff, True, order, False), BWD_TOL[dtype],
                     "backward")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("ndim", [2, 3])
def test_pooled_forward_with_dense_and_sparse_rois_in_one_call(ops, oracle, dtype, ndim):
    """Plain boxes from a fraction of a voxel to most of the feature map, grids of 1 and 2: a roi whose box
    holds more than half as many voxels as its samples have taps is read sparsely and takes its taps one
    by one (on images four per sample, the absent slice left out), the others stage their box in LDS;
    both kinds in one launch, 40 channels (matrix-core blocks and the remainder)."""
    g = wl.gen(420 + ndim)
    size = (20, 72, 88)[3 - ndim:]
    out = (7,) * ndim
    feat = torch.randn(2, 40, *size, generator=g).to(dtype)
    xyz = torch.tensor(size[::-1], dtype=torch.float32)
    n = 48
    ext = torch.exp(torch.rand(n, ndim, generator=g) * math.log(150.0)) * 0.5          # 0.5 .. 75 voxels
    ext = torch.minimum(ext, xyz * 1.1)
    lo = torch.rand(n, ndim, generator=g) * (xyz - ext + 6) - 3
    rois = torch.cat([torch.randint(0, 2, (n, 1), generator=g).float(), lo, lo + ext], 1)
    for sr in (1, 2):
        y = ops.RoIAlign(out, 1.0, sr)(feat.to(DEV), rois.to(DEV))
        assert_close(y, oracle.roi_align_forward(feat, rois, out, 1.0, sr, True, 1, False), FWD_TOL[dtype], f"forward sr={sr}")


@pytest.mark.parametrize("out", [(1, 1, 1), (1, 2, 3), (2, 3, 3)])
def test_pooled_backward_reads_only_its_own_gradients(ops, oracle, out):
    """fp16 heads with a few cells per roi: the matrix-core backward loads a plane of cells as 16-byte
    pieces that reach into the next plane, channel or roi and, for the last rois, past the tensor.
    What lies there must not matter: grad_output is the front of a buffer that holds NaN behind it, and
    one roi's gradient is infinite (it reaches that roi's box alone, as in the oracle)."""
    g = wl.gen(311)
    n, channels, size = 60, 5, (13, 39, 39)
    cells = out[0] * out[1] * out[2]
    feat = torch.randn(3, channels, *size, generator=g).half()
    lo = torch.rand(n, 3, generator=g) * torch.tensor([30.0, 30.0, 8.0])
    rois = torch.cat([torch.randint(0, 3, (n, 1), generator=g).float(), lo, lo + 1 + torch.rand(n, 3, generator=g) * 6], 1)
    rois[7] = torch.tensor([1, 33.0, 33.0, 9.0, 38.0, 38.0, 12.0])      # a corner of its own
    keep = ~((rois[:, 0] == 1) & (rois[:, 4] > 32) & (rois[:, 5] > 32) & (rois[:, 6] > 8))
    keep[7] = True
    rois = rois[keep]
    n = rois.size(0)
    buf = torch.full((n * channels * cells + 64,), float("nan"), dtype=torch.float16)
    gy = buf[:n * channels * cells].view(n, channels, *out)
    gy.copy_(torch.randn(gy.shape, generator=g))
    gy[7, 2] = float("inf")
    x = feat.to(DEV).requires_grad_(True)
    y = ops.RoIAlign(out, 1.0, 2)(x, rois.to(DEV))
    y.backward(buf.to(DEV)[:n * channels * cells].view(n, channels, *out))
    want = oracle.roi_align_backward(gy, rois, feat.shape, 1.0, 2)
    got = x.grad.cpu().double()
    assert torch.isinf(want).any() and torch.equal(torch.isfinite(got), torch.isfinite(want))
    ok = torch.isfinite(want)
    assert_close(torch.where(ok, got, 0.0), torch.where(ok, want, 0.0), BWD_TOL[torch.float16], "backward")


def test_config3_resize_and_crops(ops, oracle):
    """Benchmark configuration 3 at reduced size: CT-like fp16 volume, resize then rotated 3-D crops."""
    g = wl.gen(2)
    vol = wl.ct_like(g, (2, 1, 64, 128, 128))
    full = torch.tensor([[b, 64, 64, 32, 128, 128, 64, 0, 0, 0] for b in range(2)], dtype=torch.float32)
    small = ops.affine_3d(vol.to(DEV), full.to(DEV), (40, 64, 64), 1.0, 1, True, 1)
    want = oracle.roi_align_forward(vol, full, (40, 64, 64), 1.0, 1, True, 1, True)
    assert_close(small, want, FWD_TOL[torch.float16], "resize")
    crops = []
    for b in range(2):
        for _ in range(8):
            c = torch.rand(3, generator=g) * torch.tensor([64 - 24., 64 - 24., 40 - 24.]) + 12
            ang = (float(torch.rand(1, generator=g)) * 2 - 1) * math.radians(15)
            crops.append([b, *c.tolist(), 24, 24, 24, 0, 0, ang])
    crops = torch.tensor(crops)
    got = ops.affine_3d(small, crops.to(DEV), (24, 24, 24), 1.0, 1, True, 1)
    want = oracle.roi_align_forward(small, crops, (24, 24, 24), 1.0, 1, True, 1, True)
    assert_close(got, want, FWD_TOL[torch.float16], "crops")
    # segmentation-style call: nearest, values stay in the input's value set
    seg = (vol > 0).to(torch.float16)
    got = ops.affine_3d(seg.to(DEV), crops.to(DEV), (24, 24, 24), 1.0, 1, True, 0)
    assert set(got.unique().tolist()) <= {0.0, 1.0}
    want = oracle.roi_align_forward(seg, crops, (24, 24, 24), 1.0, 1, True, 0, True)
    margin = oracle.roi_decision_margin(seg.shape, crops, (24, 24, 24), 1.0, 1, True, True)
    frac = assert_nearest(got, want, margin, torch.float16, "nearest crops of the label map")
    assert frac < 1e-3, f"nearest mismatches: {frac:.2e}"


@pytest.mark.parametrize("dtype,channels,rois_n,size,out,order", [
    (torch.float16, 3, 5, (20, 40, 48), (24, 40, 40), 1),    # ragged tiles, several channels and rois
    (torch.bfloat16, 2, 3, (16, 24, 40), (16, 24, 32), 1),
    (torch.float32, 3, 4, (20, 40, 44), (24, 40, 40), 1),    # rows of 44 fp32: 16-byte groups
    (torch.float16, 2, 3, (20, 40, 46), (24, 40, 40), 1),    # rows of 46 fp16: unaligned, element-wise staging
    (torch.float32, 2, 3, (18, 30, 37), (16, 32, 32), 0),    # unaligned fp32, nearest
    (torch.float16, 64, 2, (24, 24, 24), (64, 64, 64), 1),   # more items than resident workgroups x 16
    (torch.float16, 2, 3, (20, 40, 48), (24, 40, 40), 3),    # order 3: halo boxes, clamped and interior tiles
    (torch.float32, 1, 3, (18, 30, 37), (16, 32, 32), 3),    # order 3, fp32, rows that are not 16-byte multiples
    (torch.bfloat16, 2, 2, (6, 7, 8), (48, 56, 64), 3),      # order 3 up-sampling of a tiny volume (every tile clamped)
])
def test_tiled_resampler_shapes(ops, oracle, dtype, channels, rois_n, size, out, order):
    """The persistent tiled kernel (outputs >= 4096 voxels per roi and channel, sampling_ratio 1) on
    rotated, scaled, partly outside rois: several channels and rois, output sizes that are not
    multiples of the tile, feature rows that are / are not multiples of 16 bytes, both orders."""
    g = wl.gen(31 + channels + rois_n)
    D, H, W = size
    feat = torch.randn(2, channels, D, H, W, generator=g).to(dtype)
    rows = []
    for r in range(rois_n):
        c = (torch.rand(3, generator=g) * 0.6 + 0.2) * torch.tensor([W, H, D], dtype=torch.float32)
        ext = (torch.rand(3, generator=g) * 0.9 + 0.5) * torch.tensor([W, H, D], dtype=torch.float32)
        ang = (torch.rand(3, generator=g) * 2 - 1) * math.radians(40)
        rows.append([r % 2, *c.tolist(), *ext.tolist(), *ang.tolist()])
    rois = torch.tensor(rows, dtype=torch.float32)
    got = ops.affine_3d(feat.to(DEV), rois.to(DEV), out, 1.0, 1, True, order)
    want = oracle.roi_align_forward(feat, rois, out, 1.0, 1, True, order, True)
    if order != 0:
        assert_close(got, want, FWD_TOL[dtype], "tiled forward")
    else:
        margin = oracle.roi_decision_margin(feat.shape, rois, out, 1.0, 1, True, True)
        frac = assert_nearest(got, want, margin, dtype, "tiled nearest")
        assert frac < 1e-4, f"nearest mismatches: {frac:.2e}"


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [120, 123])
def test_tiled_resampler_2d(ops, oracle, dtype, width):
    """Images of resampling size run the tiled kernel as volumes whose slices are the image rows (the
    rois are rewritten on the device: one cell on the middle axis that samples row 0, the rotation about
    that axis): rotated rois beyond every border, both `aligned` settings, a spatial scale that is no
    power of two, orders 0, 1 and 3 (order 3: the four taps of the middle axis are its one row and are
    left out), rows of whole 16-byte groups and ragged ones, plain boxes, several channels."""
    g = wl.gen(37 + width)
    img = torch.randn(2, 3, 96, width, generator=g).to(dtype)
    rois = torch.tensor([[0, 60.3, 47.1, 130.0, 90.0, 0.4], [1, 50.0, 40.0, 70.0, 110.0, -0.7],
                         [0, 10.0, 90.0, 60.0, 60.0, 1.3], [1, 61.3, 48.2, 121.0, 97.0, 0.0]], dtype=torch.float32)
    x, r = img.to(DEV), rois.to(DEV)
    out = (80, 96)
    for aligned in (True, False):
        for scale in (1.0, 0.3):
            rs = rois.clone()
            rs[:, 1:5] /= scale
            got = ops.RoIAlignRotated(out, scale, 1, aligned)(x, rs.to(DEV))
            want = oracle.roi_align_forward(img, rs, out, scale, 1, aligned, 1, True)
            assert float(want.abs().max()) > 0.5
            assert_close(got, want, FWD_TOL[dtype], f"image tiles, aligned {aligned}, scale {scale}")
    for order in (1, 3):
        got = ops.affine_2d(x, r, out, 1.0, 1, True, order)
        want = oracle.roi_align_forward(img, rois, out, 1.0, 1, True, order, True)
        assert_close(got, want, FWD_TOL[dtype], f"affine_2d, order {order}")
    got = ops.affine_2d(x, r, out, 1.0, 1, True, 0)
    want = oracle.roi_align_forward(img, rois, out, 1.0, 1, True, 0, True)
    margin = oracle.roi_decision_margin(img.shape, rois, out, 1.0, 1, True, True)
    frac = assert_nearest(got, want, margin, dtype, "image tiles, nearest")
    assert frac < 2e-4, f"nearest mismatches: {frac:.2e}"
    # an identity roi copies the image (rows as slices: the output's rows are the volume's slices)
    ident = torch.tensor([[b, width / 2, 48, width, 96, 0] for b in range(2)], dtype=torch.float32)
    same = ops.affine_2d(x, ident.to(DEV), (96, width), 1.0, 1, True, 1)
    assert torch.equal(same.cpu(), img)
    assert torch.equal(ops.affine_2d(x, ident.to(DEV), (96, width), 1.0, 1, True, 3).cpu(), img)
    # order 3 without rotation (a resize): windows that reach beyond every border
    got = ops.affine_2d(x, ident.to(DEV), (130, 77), 1.0, 1, True, 3)
    want = oracle.roi_align_forward(img, ident, (130, 77), 1.0, 1, True, 3, True)
    assert_close(got, want, FWD_TOL[dtype], "order 3 resize of images")
    # plain boxes with one sample per cell
    boxes = torch.tensor([[0, 3.2, 1.7, 100.4, 80.9], [1, -10.0, 20.0, 60.0, 120.0]], dtype=torch.float32)
    got = ops.RoIAlign(out, 1.0, 1)(x, boxes.to(DEV))
    want = oracle.roi_align_forward(img, boxes, out, 1.0, 1, True, 1, False)
    assert_close(got, want, FWD_TOL[dtype], "plain boxes")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("ndim,sr", [(3, 1), (3, 2), (2, 1), (2, 0)])
def test_cubic_affine_vs_oracle(ops, oracle, dtype, ndim, sr):
    """Order 3 of the affine engine (Catmull-Rom over 4^ndim clamped taps): rotated rois that
    reach beyond every border, so the clamped taps, the overshoot between S-1 and S and the void
    beyond [-1, S] are all sampled."""
    feat, rois = _random_case(ndim, True, 90 + ndim + sr)
    feat = feat.to(dtype)
    out = (5, 6, 7)[3 - ndim:]
    fn = ops.affine_3d if ndim == 3 else ops.affine_2d
    got = fn(feat.to(DEV), rois.to(DEV), out, 0.5, sr, True, 3)
    want = oracle.roi_align_forward(feat, rois, out, 0.5, sr, True, 3, True)
    assert float(want.abs().max()) > 0.5
    assert_close(got, want, FWD_TOL[dtype], "cubic affine")
    # identity roi at order 3 returns the volume itself (weights 0,1,0,0 at integer coordinates)
    size = feat.shape[2:]
    ident = torch.tensor([[0, *[s / 2 for s in size[::-1]], *size[::-1], *([0.0] * (2 * ndim - 3))]])
    same = fn(feat.to(DEV), ident.to(DEV), tuple(size), 1.0, 1, True, 3)
    assert torch.equal(same[0].cpu(), feat[0])


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sr", [2, 3, 4])
def test_large_outputs_with_a_sampling_grid(ops, oracle, dtype, sr):
    """sampling_ratio 2..4 on outputs of resampling size.  Volumes at orders 0 / 1: the tiled kernel walks
    the samples of a bin in a loop (any of the three types).  Images at order 1 with a grid of 2 or 4: the
    kernel works on the sr times finer grid of the bins' samples and takes the means inside; a grid of 3
    and order 3 write the finer volume and a second pass takes the means (fp16 / fp32).  Rotated and
    plain rois in 3-D and 2-D, order 1, and order 3 through the affine engine; a second output shape
    whose tiles are cut on every axis."""
    g = wl.gen(700 + sr)
    feat = torch.randn(2, 2, 24, 40, 48, generator=g).to(dtype)
    out = (20, 24, 32) if sr < 4 else (10, 24, 32)
    rois = wl.affine_rois(g, 2, (48, 40, 24))
    got = ops.RoIAlignRotated(out, 1.0, sr)(feat.to(DEV), rois.to(DEV))
    want = oracle.roi_align_forward(feat, rois, out, 1.0, sr, True, 1, True)
    assert float((want == 0).double().mean()) > 0.01       # bins with samples in the void
    assert_close(got, want, FWD_TOL[dtype], "rotated 3-D")
    boxes = torch.tensor([[0, 2.3, 1.2, 0.5, 40.1, 33.3, 20.7], [1, -3.0, 5.0, 2.0, 30.0, 45.0, 30.0]])
    got = ops.RoIAlign(out, 0.5, sr)(feat.to(DEV), (boxes * torch.tensor([1.] + [2.] * 6)).to(DEV))
    want = oracle.roi_align_forward(feat, boxes * torch.tensor([1.] + [2.] * 6), out, 0.5, sr, True, 1, False)
    assert_close(got, want, FWD_TOL[dtype], "plain 3-D")
    ragged = (17, 21, 27) if sr < 4 else (9, 21, 27)
    got = ops.RoIAlignRotated(ragged, 1.0, sr)(feat.to(DEV), rois.to(DEV))
    want = oracle.roi_align_forward(feat, rois, ragged, 1.0, sr, True, 1, True)
    assert_close(got, want, FWD_TOL[dtype], "rotated 3-D, tiles cut on every axis")
    img = torch.randn(2, 3, 70, 90, generator=g).to(dtype)
    r2 = torch.tensor([[0, 45.0, 35.0, 80.0, 60.0, 0.4], [1, 40.0, 30.0, 100.0, 50.0, -1.2]])
    got = ops.RoIAlignRotated((64, 80), 1.0, sr)(img.to(DEV), r2.to(DEV))
    want = oracle.roi_align_forward(img, r2, (64, 80), 1.0, sr, True, 1, True)
    assert_close(got, want, FWD_TOL[dtype], "rotated 2-D")
    if dtype != torch.bfloat16:
        got = ops.affine_3d(feat.to(DEV), rois.to(DEV), out, 1.0, sr, True, 3)
        want = oracle.roi_align_forward(feat, rois, out, 1.0, sr, True, 3, True)
        assert_close(got, want, FWD_TOL[dtype], "order 3")
        got = ops.affine_2d(img.to(DEV), r2.to(DEV), (64, 80), 1.0, sr, False, 3)
        want = oracle.roi_align_forward(img, r2, (64, 80), 1.0, sr, False, 3, True)
        assert_close(got, want, FWD_TOL[dtype], "order 3, images")


def test_cubic_resize_larger_volume(ops, oracle):
    """Resize of a 40x48x56 volume to 64x80x96 at order 3, as CudaResize(order=3) issues it."""
    g = wl.gen(97)
    vol = torch.randn(2, 2, 40, 48, 56, generator=g).half()
    rois = torch.tensor([[b, 28, 24, 20, 56, 48, 40, 0, 0, 0] for b in range(2)], dtype=torch.float32)
    got = ops.affine_3d(vol.to(DEV), rois.to(DEV), (64, 80, 96), 1.0, 1, True, 3)
    want = oracle.roi_align_forward(vol, rois, (64, 80, 96), 1.0, 1, True, 3, True)
    assert_close(got, want, FWD_TOL[torch.float16], "cubic resize")


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("ndim", [3, 2])
def test_cubic_unrotated_windows(ops, oracle, dtype, ndim):
    """Order 3 without rotation (the separable form of the tiled kernel): windows that reach beyond
    the volume on either side (clamped taps, the overshoot up to S and the void beyond), an
    up-sampling of a tiny control grid as the elastic deformation issues it, and a down-sampling
    whose boxes leave no room for the intermediates (general form)."""
    g = wl.gen(61 + ndim)
    size = (20, 24, 28)[3 - ndim:]
    vol = torch.randn(2, 3, *size, generator=g).to(dtype)
    xyz = list(size[::-1])
    zeros = [0.0] * (2 * ndim - 3)
    rois = torch.tensor([[0, *[0.3 * s for s in xyz], *[1.2 * s for s in xyz], *zeros],
                         [1, *[0.8 * s for s in xyz], *[0.9 * s for s in xyz], *zeros],
                         [1, *[0.5 * s for s in xyz], *[0.25 * s for s in xyz], *zeros]], dtype=torch.float32)
    out = (32, 40, 48)[3 - ndim:]
    fn = ops.affine_3d if ndim == 3 else ops.affine_2d
    got = fn(vol.to(DEV), rois.to(DEV), out, 1.0, 1, True, 3)
    want = oracle.roi_align_forward(vol, rois, out, 1.0, 1, True, 3, True)
    assert float((want == 0).float().mean()) > 0.05            # the void is sampled
    assert_close(got, want, FWD_TOL[dtype], "cubic windows")
    grid = torch.randn(1, 3, *([8] * ndim), generator=g).to(dtype)
    groi = torch.tensor([[0, *([4.0] * ndim), *([5.0] * ndim), *zeros]], dtype=torch.float32)
    big = (64, 64, 80)[3 - ndim:]
    got = fn(grid.to(DEV), groi.to(DEV), big, 1.0, 1, True, 3)
    want = oracle.roi_align_forward(grid, groi, big, 1.0, 1, True, 3, True)
    assert_close(got, want, FWD_TOL[dtype], "control-grid upsampling")
    if ndim == 3:
        wide = torch.randn(1, 1, 40, 72, 80, generator=g).to(dtype)
        wroi = torch.tensor([[0, 40.0, 36.0, 20.0, 80.0, 72.0, 40.0, 0, 0, 0]], dtype=torch.float32)
        got = fn(wide.to(DEV), wroi.to(DEV), (16, 24, 32), 1.0, 1, True, 3)
        want = oracle.roi_align_forward(wide, wroi, (16, 24, 32), 1.0, 1, True, 3, True)
        assert_close(got, want, FWD_TOL[dtype], "cubic down-sampling")


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_config5_detection_head_reduced(ops, oracle, dtype):
    """Benchmark configuration 5 shape family (log-uniform extents, scale 0.25, 7^3, sr=2), reduced."""
    g = wl.gen(4)
    feat = torch.randn(2, 16, 12, 48, 48, generator=g).to(dtype)
    rois = wl.roi3d_detection(g, 200, 2, (192, 192, 48), (2.0, 48.0), log_uniform=True)
    x = feat.to(DEV).requires_grad_(True)
    out = ops.RoIAlign((7, 7, 7), 0.25, 2)(x, rois.to(DEV))
    want = oracle.roi_align_forward(feat, rois, (7, 7, 7), 0.25, 2)
    assert_close(out, want, FWD_TOL[dtype], "forward")
    gy = torch.randn(out.shape, generator=g).to(dtype)
    out.backward(gy.to(DEV))
    gwant = oracle.roi_align_backward(gy, rois, feat.shape, 0.25, 2)
    assert_close(x.grad, gwant, BWD_TOL[dtype], "backward")


@pytest.mark.parametrize("ndim", [3, 2])
def test_pooled_forward_from_blocked_copy(ops, oracle, ndim):
    """fp16 detection heads with about as many pooled outputs as input voxels read a re-ordered copy
    of the features (units of four columns, channels innermost): boxes starting at every column
    phase, sticking out of the volume on every side, of one voxel, larger than the matrix-core form
    takes (plain form from the same launch); channel counts that are no multiple of the tile or of the
    copy's chunk; a width whose units do not fill the copy's last chunk."""
    from medvision_amd import _lib
    g = wl.gen(77 + ndim)
    size = (10, 24, 40)[3 - ndim:]
    channels = 70
    feat = torch.randn(2, channels, *size, generator=g).half()
    xyz = torch.tensor(size[::-1], dtype=torch.float32)
    n = 900 if ndim == 3 else 120
    lo = (torch.rand(n, ndim, generator=g) * 1.3 - 0.15) * xyz
    ext = torch.exp(torch.rand(n, ndim, generator=g) * math.log(30.0)) * 0.6      # 0.6 .. 18 voxels
    ext[:8] = xyz * 1.2                                                            # whole-volume boxes
    rois = torch.cat([torch.randint(0, 2, (n, 1), generator=g).float(), lo, lo + ext], 1)
    out = (7, 7, 7)[3 - ndim:]
    out3 = out if ndim == 3 else (1, *out)
    in3 = size if ndim == 3 else (1, *size)
    need = _lib.load().mv_roi_align_forward_workspace_bytes_for_input(_lib.MV_F16, ndim, 2, channels, *in3, n, *out3, 2)
    assert need == feat.numel() * 2 + 4 * n     # the copy (and the launch order of the rois) is in use
    got = ops.RoIAlign(out, 1.0, 2)(feat.to(DEV), rois.to(DEV))
    want = oracle.roi_align_forward(feat, rois, out, 1.0, 2)
    assert_close(got, want, FWD_TOL[torch.float16], "pooled forward from the blocked copy")
    # the copy made once and handed in (heads that pool one feature map several times): the same
    # outputs bit for bit, also for a second, smaller batch of rois and with few rois (no copy would be
    # made for them inside a call); gradients reach the features
    x = feat.to(DEV).requires_grad_(True)
    kept = ops.PreparedFeatures(x)
    assert kept.copy is not None and kept.copy.numel() == feat.numel() * 2
    again = ops.RoIAlign(out, 1.0, 2)(kept, rois.to(DEV))
    assert torch.equal(again, got)
    few = ops.RoIAlign(out, 1.0, 2)(kept, rois[:5].to(DEV))
    assert torch.equal(few, got[:5])
    nearest = ops.RoIAlign(out, 1.0, 2)(kept, rois[:40].to(DEV), order=0)
    assert torch.equal(nearest, ops.RoIAlign(out, 1.0, 2)(feat.to(DEV), rois[:40].to(DEV), order=0))
    gy = torch.randn(again.shape, generator=g).half()
    again.backward(gy.to(DEV))
    gwant = oracle.roi_align_backward(gy, rois, feat.shape, 1.0, 2)
    assert_close(x.grad, gwant, BWD_TOL[torch.float16], "backward behind the prepared copy")
    # heads the copy does not serve run as without it
    big = tuple(12 for _ in out)
    assert torch.equal(ops.RoIAlign(big, 1.0, 2)(kept, rois[:50].to(DEV)),
                       ops.RoIAlign(big, 1.0, 2)(feat.to(DEV), rois[:50].to(DEV)))
    with torch.no_grad():
        x.mul_(2.0)
    with pytest.raises(RuntimeError, match="changed in place"):
        ops.RoIAlign(out, 1.0, 2)(kept, rois.to(DEV))
    assert ops.PreparedFeatures(feat.float().to(DEV)).copy is None      # fp16 only
    # few rois: no copy, same kernels from the input itself
    few = rois[:15]
    assert _lib.load().mv_roi_align_forward_workspace_bytes_for_input(_lib.MV_F16, ndim, 2, channels, *in3, 15, *out3, 2) == 0
    got = ops.RoIAlign(out, 1.0, 2)(feat.to(DEV), few.to(DEV))
    assert_close(got, want[:15], FWD_TOL[torch.float16], "pooled forward from the input")
    # straight through the C ABI with a workspace that is too small for the copy (a caller that sized
    # its arena with the query that does not know the input): the entry point must not use it
    import ctypes
    lib = _lib.load()
    x, r = feat.to(DEV), rois.to(DEV)
    raw = torch.full((n, channels, *out), float("nan"), dtype=torch.float16, device=DEV)
    small = torch.full((4096,), 7, dtype=torch.uint8, device=DEV)
    fn = lib.mv_roi_align_3d_forward if ndim == 3 else lib.mv_roi_align_2d_forward
    _lib.check(fn(_lib.ptr(x), _lib.ptr(r), _lib.ptr(raw), _lib.MV_F16, *x.shape, n, *out, 1.0, 2, 1,
                  _lib.ptr(small), 4096, _lib.stream_of(x)))
    torch.cuda.synchronize()
    assert bool((small == 7).all()), "the undersized workspace was written"
    assert_close(raw, want, FWD_TOL[torch.float16], "pooled forward, workspace too small for the copy")


@pytest.mark.parametrize("out", [(8, 8, 8), (3, 6, 6), (2, 5, 7), (7, 4, 8), (5, 5, 5), (6, 6), (4, 8), (5, 5)])
@pytest.mark.parametrize("channels", [8, 12, 10])
def test_pooled_forward_output_layouts(ops, oracle, out, channels):
    """The matrix-core pooled forward writes a finished tile of four channels through LDS when a row
    of cells (oh * ow) has at least 32 of them and the channel block is a whole number of tiles:
    rows of exactly 32 and 64 cells, rows whose last run of eight is cut, rows too short for that
    form, a channel count that is no multiple of four, outputs of odd rois (whose address is no
    multiple of 8 bytes when channels * cells is odd), images and volumes."""
    ndim = len(out)
    g = wl.gen(400 + 10 * ndim + channels + sum(out))
    size = (6, 12, 16)[3 - ndim:]
    feat = torch.randn(2, channels, *size, generator=g).half()
    xyz = torch.tensor(size[::-1], dtype=torch.float32)
    cells = 1
    for o in out:
        cells *= o
    n = max(40, 3 * feat[:, 0].numel() // cells)        # enough rois for the re-ordered copy of the features
    lo = (torch.rand(n, ndim, generator=g) * 1.2 - 0.1) * xyz
    ext = torch.exp(torch.rand(n, ndim, generator=g) * math.log(12.0)) * 0.8
    rois = torch.cat([torch.randint(0, 2, (n, 1), generator=g).float(), lo, lo + ext], 1)
    got = ops.RoIAlign(out, 1.0, 2)(feat.to(DEV), rois.to(DEV))
    want = oracle.roi_align_forward(feat, rois, out, 1.0, 2)
    assert_close(got, want, FWD_TOL[torch.float16], f"pooled forward {out} x {channels} channels")
    got = ops.RoIAlign(out, 1.0, 2)(feat.to(DEV), rois[:7].to(DEV))      # few rois: from the input itself
    assert_close(got, want[:7], FWD_TOL[torch.float16], f"pooled forward {out} x {channels} channels, few rois")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("sr,order", [(2, 1), (-1, 1), (3, 1), (1, 0)])
def test_pooled_kernel_paths(ops, oracle, dtype, sr, order):
    """Plain boxes with small outputs run through the separable LDS kernels; this covers their
    special cases: boxes larger than the LDS budget, adaptive grids whose tap tables overflow,
    boxes (partly) outside the volume, degenerate and single-voxel boxes, several channel chunks."""
    g = wl.gen(21)
    feat = torch.randn(2, 40, 20, 40, 44, generator=g).to(dtype)
    rois = torch.tensor([
        [0, 0.0, 0.0, 0.0, 44.0, 40.0, 20.0],        # whole volume: 44*40*20 voxels per channel
        [1, -30.0, -30.0, -30.0, 80.0, 90.0, 60.0],   # far larger than the volume
        [1, 50.0, 45.0, 25.0, 60.0, 55.0, 30.0],      # completely outside: all samples void
        [0, -5.1, -3.2, -2.3, 6.05, 4.1, 3.2],        # partly outside (no sample on an exact .5 tie)
        [0, 10.2, 11.7, 5.1, 10.3, 11.8, 5.2],        # degenerate (extent clamped to 1)
        [1, 43.0, 39.0, 19.0, 44.0, 40.0, 20.0],      # last voxel, taps clamp at the border
        [1, 3.3, 2.2, 1.1, 17.9, 21.4, 9.6],
    ])
    x = feat.to(DEV).requires_grad_(True)
    out = ops.RoIAlign((5, 6, 7), 1.0, sr)(x, rois.to(DEV), order=order)
    eff = 1 if order == 0 else sr
    want = oracle.roi_align_forward(feat, rois, (5, 6, 7), 1.0, eff, True, order)
    assert_close(out, want, FWD_TOL[dtype], "pooled forward")
    gy = torch.randn(out.shape, generator=g).to(dtype)
    out.backward(gy.to(DEV))
    gwant = oracle.roi_align_backward(gy, rois, feat.shape, 1.0, eff, True, order)
    assert_close(x.grad, gwant, BWD_TOL[dtype], "pooled backward")
    # 2-D twin
    f2 = torch.randn(2, 5, 30, 34, generator=g).to(dtype)
    r2 = torch.tensor([[0, 0.0, 0.0, 34.0, 30.0], [1, -4.0, 3.0, 9.5, 40.0], [1, 7.7, 8.8, 7.9, 8.9]])
    x2 = f2.to(DEV).requires_grad_(True)
    o2 = ops.RoIAlign((6, 7), 1.0, sr)(x2, r2.to(DEV), order=order)
    assert_close(o2, oracle.roi_align_forward(f2, r2, (6, 7), 1.0, eff, True, order), FWD_TOL[dtype], "2-d")
    gy2 = torch.randn(o2.shape, generator=g).to(dtype)
    o2.backward(gy2.to(DEV))
    assert_close(x2.grad, oracle.roi_align_backward(gy2, r2, f2.shape, 1.0, eff, True, order),
                 BWD_TOL[dtype], "2-d backward")


def test_config1_rois_on_gpu(ops, oracle):
    """Benchmark configuration 1 inputs (fp32 [2,16,32,64,64], 128 rois, 7^3, sr=2) through RoIAlign3D."""
    g = wl.gen(0)
    feat = torch.randn(2, 16, 32, 64, 64, generator=g)
    rois = wl.roi3d_detection(g, 128, 2, (64, 64, 32), (4.0, 24.0))
    out = ops.RoIAlign((7, 7, 7), 1.0, 2)(feat.to(DEV), rois.to(DEV))
    want = oracle.roi_align_forward(feat, rois, (7, 7, 7), 1.0, 2)
    assert_close(out, want, FWD_TOL[torch.float32], "config 1")


def test_non_default_stream_and_determinism(ops):
    g = wl.gen(3)
    vol = torch.randn(1, 2, 32, 32, 32, generator=g).to(DEV)
    rois = wl.affine_rois(g, 1, (32, 32, 32)).to(DEV)
    ref = ops.affine_3d(vol, rois, (32, 32, 32), 1.0, 2, True, 1)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        again = ops.affine_3d(vol, rois, (32, 32, 32), 1.0, 2, True, 1)
    s.synchronize()
    assert torch.equal(ref, again)


def test_volume_beyond_2_31_elements(ops):
    """A 1300^3 fp16 volume (2.2e9 elements): crops at its far corner come back exactly, and the
    backward pass puts the gradient there (the reference's `int` index arithmetic overflows at this
    size, roi_align_3d_cuda_kernel.cuh:28-50; offsets here are 64-bit)."""
    S, n = 1300, 64
    vol = torch.empty(1, 1, S, S, S, dtype=torch.float16, device=DEV)
    ar = torch.arange(S, device=DEV, dtype=torch.float32)
    for z in range(S):
        vol[0, 0, z] = (((ar[:, None] * 7 + ar[None, :] * 3 + z * 11) % 251) - 125).half()
    lo = S - n - 3
    c = lo + n / 2
    rois = torch.tensor([[0, c, c, c, n, n, n, 0, 0, 0]], dtype=torch.float32, device=DEV)
    want = vol[0, 0, lo:lo + n, lo:lo + n, lo:lo + n]
    assert torch.equal(ops.RoIAlignRotated((n, n, n), 1.0, 1, True)(vol, rois)[0, 0], want)
    assert torch.equal(ops.affine_3d(vol, rois, (n, n, n), 1.0, 1, True, 1)[0, 0], want)
    box = torch.tensor([[0, lo, lo, lo, lo + n, lo + n, lo + n]], dtype=torch.float32, device=DEV)
    got = ops.RoIAlign((n, n, n), 1.0, 1)(vol, box)[0, 0].float()   # samples at cell centres: mean of 8
    w = vol[0, 0, lo:lo + n + 1, lo:lo + n + 1, lo:lo + n + 1].float()
    mean8 = sum(w[a:a + n, b:b + n, e:e + n] for a in (0, 1) for b in (0, 1) for e in (0, 1)) / 8
    assert float((got - mean8).abs().max()) <= 0.13   # fp16 rounding of values up to 125
    vol.requires_grad_(True)
    out = ops.RoIAlignRotated((n, n, n), 1.0, 1, True)(vol, rois)
    out.backward(torch.ones_like(out))
    assert float(vol.grad[0, 0, lo:lo + n, lo:lo + n, lo:lo + n].float().sum()) == n ** 3
    assert float(vol.grad[0, 0, lo, lo, lo]) == 1.0 and float(vol.grad[0, 0, 0, 0, 0]) == 0.0


@pytest.mark.parametrize("order", [0, 1, 3])
@pytest.mark.parametrize("out", [(6, 7, 8), (24, 40, 48)])   # general / pooled kernels, tiled kernels
def test_every_output_element_is_written(ops, oracle, order, out):
    """The operators allocate their outputs uninitialised: every element has to be stored by the
    kernels, zeros included (rois wholly outside the volume, rois of an image that does not exist,
    void samples at the borders).  The buffers handed to the shim here are full of NaN."""
    from medvision_amd import _C
    g = wl.gen(31 + order)
    feat = torch.randn(2, 3, 10, 12, 16, generator=g).half()
    rot = torch.tensor([[0, 8.0, 6.0, 5.0, 20.0, 14.0, 12.0, 0.3, -0.2, 0.5],        # reaches beyond every border
                        [1, 200.0, 6.0, 5.0, 10.0, 10.0, 10.0, 0.0, 0.0, 0.4],      # wholly outside
                        [1, -50.0, -60.0, -70.0, 8.0, 8.0, 8.0, 0.1, 0.0, 0.0],     # wholly outside
                        [5, 8.0, 6.0, 5.0, 8.0, 8.0, 8.0, 0.0, 0.0, 0.0]])          # no such image
    output = torch.full((4, 3, *out), float("nan"), dtype=torch.float16, device=DEV)
    _C.affine_3d(feat.to(DEV), rot.to(DEV), output, *out, 1.0, 1, True, order)
    assert not bool(torch.isnan(output).any())
    assert float(output[1:].abs().max()) == 0.0
    assert_close(output[:1], oracle.roi_align_forward(feat, rot[:1], out, 1.0, 1, True, order, True),
                 FWD_TOL[torch.float16], "affine")
    if order == 3:
        return
    output.fill_(float("nan"))
    sr = 1 if order == 0 else 2   # the operator classes never average nearest-neighbour samples
    _C.roi_align_rotated_3d_forward(feat.to(DEV), rot.to(DEV), output, *out, 1.0, sr, True, order)
    assert not bool(torch.isnan(output).any()) and float(output[1:].abs().max()) == 0.0
    # (extents that put no sample on a .5 tie: at order 0 rounding would decide those)
    box = torch.tensor([[0, -3.1, 2.2, 1.3, 12.4, 15.1, 9.2], [1, 300.0, 2.0, 1.0, 312.0, 9.0, 8.0],
                        [7, 1.0, 2.0, 1.0, 9.0, 9.0, 8.0]])
    output = torch.full((3, 3, *out), float("nan"), dtype=torch.float16, device=DEV)
    _C.roi_align_3d_forward(feat.to(DEV), box.to(DEV), output, *out, 1.0, sr, order)
    assert not bool(torch.isnan(output).any()) and float(output[1:].abs().max()) == 0.0
    assert_close(output[:1], oracle.roi_align_forward(feat, box[:1], out, 1.0, sr, True, order, False),
                 FWD_TOL[torch.float16], "plain boxes")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_pooled_boxes_wider_than_the_tap_tables(ops, oracle, dtype):
    """Few cells spread over many voxels: boxes of 70-100 voxels on one axis with 7 cells of 2
    samples, and of more than 258.  The separable backward kernel indexes its tap ranges by source
    voxel through a table of 260 entries and has to hand wider boxes to the per-output scatter (with
    68 entries and no such hand-over it once ran off the table and never finished)."""
    g = wl.gen(77)
    img = torch.randn(2, 6, 110, 120, generator=g).to(dtype)
    rois2 = torch.tensor([[0, 3.0, 5.0, 98.0, 60.0], [1, 10.5, 2.0, 105.0, 101.0], [0, 40.0, 40.0, 47.0, 46.0],
                          [1, -20.0, 30.0, 70.0, 90.0]])
    vol = torch.randn(1, 5, 9, 10, 96, generator=g).to(dtype)
    rois3 = torch.tensor([[0, 2.0, 1.0, 1.0, 88.0, 7.5, 7.0], [0, 10.0, 2.0, 0.5, 93.0, 8.0, 8.5]])
    wide = torch.randn(1, 3, 12, 300, generator=g).to(dtype)
    rois4 = torch.tensor([[0, 4.0, 1.0, 292.5, 10.0], [0, 20.0, 2.0, 278.0, 11.0], [0, -5.0, 0.0, 310.0, 12.0]])
    for feat, rois, out in ((img, rois2, (7, 7)), (vol, rois3, (7, 7, 7)), (wide, rois4, (7, 7))):
        mod = ops.RoIAlign(out, 1.0, 2)
        x = feat.to(DEV).requires_grad_(True)
        y = mod(x, rois.to(DEV))
        assert_close(y, oracle.roi_align_forward(feat, rois, out, 1.0, 2, True, 1, False), FWD_TOL[dtype], "forward")
        gy = torch.randn(y.shape, generator=g).to(dtype)
        y.backward(gy.to(DEV))
        want = oracle.roi_align_backward(gy, rois, feat.shape, 1.0, 2, True, 1, False)
        assert_close(x.grad, want, BWD_TOL[dtype], "backward")


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_pooled_kernels_with_adaptive_grids_on_large_boxes(ops, oracle, dtype):
    """sampling_ratio 0 (the reference's default): ceil(box / cells) samples per bin, so boxes of 64 -
    126 voxels need 65 - 128 tap entries per axis (two per lane of the wavefront that builds a table);
    beyond that the per-sample kernels take over."""
    g = wl.gen(79)
    img = torch.randn(2, 5, 140, 150, generator=g).to(dtype)
    rois2 = torch.tensor([[0, 3.0, 5.0, 98.0, 80.0], [1, 10.5, 2.0, 135.0, 121.0], [0, 40.0, 40.0, 47.0, 46.0],
                          [1, -20.0, 30.0, 70.0, 150.0], [0, 1.0, 1.0, 149.0, 139.0]])
    vol = torch.randn(1, 3, 9, 10, 120, generator=g).to(dtype)
    rois3 = torch.tensor([[0, 2.0, 1.0, 1.0, 88.0, 7.5, 7.0], [0, 10.0, 2.0, 0.5, 118.0, 8.0, 8.5]])
    # boxes of 26 - 36 voxels on every axis: too large for LDS with all their planes, four or five samples
    # per bin and axis (the forward pass then goes through slabs of planes as well)
    cube = torch.randn(2, 10, 30, 34, 40, generator=g).to(dtype)
    rois5 = torch.tensor([[0, 2.0, 1.0, 1.0, 30.0, 29.5, 27.0], [1, 5.0, 2.0, 0.5, 39.0, 33.0, 29.5],
                          [1, -4.0, -3.0, -2.0, 32.0, 31.0, 28.0]])
    for feat, rois, out in ((img, rois2, (7, 7)), (img, rois2, (14, 14)), (vol, rois3, (7, 7, 7)), (cube, rois5, (7, 7, 7))):
        x = feat.to(DEV).requires_grad_(True)
        y = ops.RoIAlign(out, 1.0, 0)(x, rois.to(DEV))
        assert_close(y, oracle.roi_align_forward(feat, rois, out, 1.0, 0, True, 1, False), FWD_TOL[dtype], "forward")
        gy = torch.randn(y.shape, generator=g).to(dtype)
        y.backward(gy.to(DEV))
        want = oracle.roi_align_backward(gy, rois, feat.shape, 1.0, 0, True, 1, False)
        assert_close(x.grad, want, BWD_TOL[dtype], "backward")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_pooled_heads_with_9_to_16_cells(ops, oracle, dtype):
    """14 x 14 mask heads and a 10 x 12 x 14 volume head: the pooled kernels' 16-cell instance
    (dense per-axis matrices in the backward pass, tap registers in the forward pass)."""
    g = wl.gen(78)
    img = torch.randn(2, 9, 40, 52, generator=g).to(dtype)
    rois2 = wl.roi3d_detection(g, 12, 2, (52, 40, 1), (5.0, 28.0))[:, [0, 1, 2, 4, 5]]
    vol = torch.randn(2, 5, 14, 20, 24, generator=g).to(dtype)
    rois3 = wl.roi3d_detection(g, 8, 2, (24, 20, 14), (4.0, 14.0))
    for feat, rois, out, sr in ((img, rois2, (14, 14), 2), (vol, rois3, (10, 12, 14), 2), (img, rois2, (14, 9), 0)):
        mod = ops.RoIAlign(out, 1.0, sr)
        x = feat.to(DEV).requires_grad_(True)
        y = mod(x, rois.to(DEV))
        assert_close(y, oracle.roi_align_forward(feat, rois, out, 1.0, sr, True, 1, False), FWD_TOL[dtype], "forward")
        gy = torch.randn(y.shape, generator=g).to(dtype)
        y.backward(gy.to(DEV))
        want = oracle.roi_align_backward(gy, rois, feat.shape, 1.0, sr, True, 1, False)
        assert_close(x.grad, want, BWD_TOL[dtype], "backward")


def test_config3_full_size_properties(ops):
    """Benchmark configuration 3 at its full size (fp16 [2,1,256,512,512] -> 160x256x256, then 16
    crops of 96^3): properties that need no oracle run.  A constant volume stays constant under
    resize and rotated crops (weights sum to one wherever no sample is void); crops with zero
    angles on whole-voxel centres are slices of the resized volume; resizing is linear."""
    g = wl.gen(2)
    vol = wl.ct_like(g, (2, 1, 256, 512, 512)).to(DEV)
    full = torch.tensor([[b, 256, 256, 128, 512, 512, 256, 0, 0, 0] for b in range(2)], dtype=torch.float32, device=DEV)
    small = ops.affine_3d(vol, full, (160, 256, 256), 1.0, 1, True, 1)
    const = torch.full_like(vol, 3.25)
    assert torch.equal(ops.affine_3d(const, full, (160, 256, 256), 1.0, 1, True, 1), torch.full_like(small, 3.25))
    # scaling by a power of two commutes with every rounding except into fp16's subnormal range
    # (below 2^-14 the spacing no longer scales): exact above it, one subnormal step below
    twice = ops.affine_3d(vol * 2, full, (160, 256, 256), 1.0, 1, True, 1)
    normal = small.abs() >= 2.0 ** -14
    assert torch.equal(twice[normal], (small * 2)[normal])
    assert float((twice.float() - small.float() * 2)[~normal].abs().max()) <= 2.0 ** -24
    lo = torch.tensor([[30, 40, 20], [100, 17, 60]])
    crops = torch.tensor([[b, lo[b, 0] + 48, lo[b, 1] + 48, lo[b, 2] + 48, 96, 96, 96, 0, 0, 0] for b in range(2)],
                         dtype=torch.float32, device=DEV)
    got = ops.affine_3d(small, crops, (96, 96, 96), 1.0, 1, True, 1)
    for b in range(2):
        x, y, z = lo[b].tolist()
        assert torch.equal(got[b, 0], small[b, 0, z:z + 96, y:y + 96, x:x + 96])
    rot = crops.clone()
    rot[:, 9] = torch.tensor([0.2, -0.25])
    csmall = torch.full_like(small, -7.5)
    assert torch.equal(ops.affine_3d(csmall, rot, (96, 96, 96), 1.0, 1, True, 1),
                       torch.full((2, 1, 96, 96, 96), -7.5, dtype=torch.float16, device=DEV))


def test_config5_full_size_properties(ops):
    """Benchmark configuration 5 at its full size (fp16 [2,256,24,96,96], 4000 rois, 7^3, sr 2,
    scale 0.25): a constant feature map pools to the constant (all boxes lie inside the volume),
    pooling is linear, and the backward pass conserves the gradient mass per image and channel."""
    g = wl.gen(4)
    rois = wl.roi3d_detection(g, 4000, 2, (384, 384, 96), (2.0, 48.0), log_uniform=True)
    feat = torch.randn(2, 256, 24, 96, 96, generator=g).half().to(DEV)
    mod = ops.RoIAlign((7, 7, 7), 0.25, 2)
    r = rois.to(DEV)
    # boxes narrower than one voxel are widened to one and may then reach beyond the volume, where
    # samples are void: 16 of the 4000; the properties below hold for the others
    lo, hi = rois[:, 1:4] * 0.25, rois[:, 4:7] * 0.25
    inside = ((lo + (hi - lo).clamp(min=1.0)) <= torch.tensor([96.0, 96.0, 24.0])).all(dim=1)
    assert int(inside.sum()) >= 3950
    const = mod(torch.full_like(feat, 1.5), r)
    assert float((const[inside.to(DEV)].float() - 1.5).abs().max()) <= 1.5 * 2 ** -10   # one fp16 rounding of the sum
    x = feat.clone().requires_grad_(True)
    y = mod(x, r)
    # doubling the features doubles every intermediate exactly, except where an fp16 intermediate of
    # the matrix-core path is subnormal (fixed spacing 2^-24): that may move a result by one rounding
    # step, in a tiny share of the outputs
    twice, dbl = mod(feat * 2, r).float(), y.detach().float() * 2
    dev = (twice - dbl).abs()
    assert bool((dev <= 2.0 ** -10 * dbl.abs() + 2.0 ** -23).all())
    assert float((dev > 0).float().mean()) <= 1e-4
    del twice, dbl, dev
    gy = torch.randn(y.shape, generator=g).half()
    gy[~inside] = 0
    gy = gy.to(DEV)
    y.backward(gy)
    # every sample lies inside the volume: each output's gradient is spread with weights summing to 1
    for b in range(2):
        pick = (rois[:, 0] == b).to(DEV)
        want = gy[pick].double().sum(dim=(0, 2, 3, 4))
        got = x.grad[b].double().sum(dim=(1, 2, 3))
        scale = float(gy[pick].double().abs().sum(dim=(0, 2, 3, 4)).max())
        assert float((got - want).abs().max()) <= 2e-3 * scale   # fp16 rounding of 1.8 M accumulated cells


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("ndim", [3, 2])
def test_rotated_heads_backward_through_box_tiles(ops, oracle, dtype, ndim):
    """Rotated rois with detection-head outputs (7^3 / 14^2 cells): the backward pass sums each block of
    cells in an LDS tile of the source box.  Rois from a fraction of a voxel (thousands of samples in one
    voxel: per-sample path) to half the volume (several blocks per roi), sticking out of the volume,
    fixed and adaptive grids, more channels than a workgroup's tile holds, a NaN in one gradient."""
    g = wl.gen(610 + ndim)
    size = (20, 44, 52)[3 - ndim:]
    out = (7, 7, 7) if ndim == 3 else (14, 14)
    C = 21
    feat = torch.randn(2, C, *size, generator=g).to(dtype)
    xyz = torch.tensor(size[::-1], dtype=torch.float32)
    n = 40
    ctr = (torch.rand(n, ndim, generator=g) * 1.2 - 0.1) * xyz
    ext = torch.exp(torch.rand(n, ndim, generator=g) * math.log(100.0)) * 0.3      # 0.3 .. 30 voxels
    ext[:3] = xyz * 0.6
    ang = (torch.rand(n, 3 if ndim == 3 else 1, generator=g) * 2 - 1) * math.radians(40)
    rois = torch.cat([torch.randint(0, 2, (n, 1), generator=g).float(), ctr, ext, ang], 1)
    for sr in (2, 0, 3):
        x = feat.to(DEV).requires_grad_(True)
        y = ops.RoIAlignRotated(out, 1.0, sr, True)(x, rois.to(DEV))
        assert_close(y, oracle.roi_align_forward(feat, rois, out, 1.0, sr, True, 1, True), FWD_TOL[dtype], f"forward sr={sr}")
        gy = torch.randn(y.shape, generator=g).to(dtype)
        y.backward(gy.to(DEV))
        want = oracle.roi_align_backward(gy, rois, feat.shape, 1.0, sr, True, 1, True)
        assert_close(x.grad, want, BWD_TOL[dtype], f"backward sr={sr}")
    # order 0 (a grid of one)
    x = feat.to(DEV).requires_grad_(True)
    y = ops.RoIAlignRotated(out, 1.0, 2, True)(x, rois.to(DEV), order=0)
    gy = torch.randn(y.shape, generator=g).to(dtype)
    y.backward(gy.to(DEV))
    assert_close(x.grad, oracle.roi_align_backward(gy, rois, feat.shape, 1.0, 1, True, 0, True), BWD_TOL[dtype], "order 0")
    # a NaN in one channel of one roi's gradient: that channel adds per sample, and the voxels its samples
    # touch are NaN as in the oracle (roi 0 covers most of the volume: interior samples, no zero weights)
    x = feat.to(DEV).requires_grad_(True)
    y = ops.RoIAlignRotated(out, 1.0, 2, True)(x, rois.to(DEV))
    gy = torch.randn(y.shape, generator=g).to(dtype)
    gy[0, 3].view(-1)[gy[0, 3].numel() // 2] = float("nan")
    y.backward(gy.to(DEV))
    want = oracle.roi_align_backward(gy, rois, feat.shape, 1.0, 2, True, 1, True)
    got = x.grad.cpu()
    assert torch.isnan(want).any() and torch.equal(torch.isnan(got), torch.isnan(want))
    ok = ~torch.isnan(want)
    assert_close(got[ok], want[ok], BWD_TOL[dtype], "a NaN gradient")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("rotated", [False, True])
@pytest.mark.parametrize("out", [(14, 14, 14), (20, 20, 20)])
def test_backward_of_finely_sampled_rois_with_gradients_of_one_sign(ops, oracle, dtype, rotated, out):
    """Grids far finer than the voxels (bins of 0.15 - 0.6 voxels with 2 or 3 samples each): thousands of
    samples reach a voxel, and the 32-bit fixed-point sums of the box and tile kernels are scaled by a bound
    on the sum of their weights, not by their number.  Gradients that are all +1 add up without cancelling:
    a bound that were too small would overflow the sums, and the result would be far off."""
    g = wl.gen(900 + len(out) + out[0])
    size = (16, 20, 24)
    n, C = 10, 3
    xyz = torch.tensor(size[::-1], dtype=torch.float32)
    ext = 2.0 + torch.rand(n, 3, generator=g) * 6.0
    ctr = torch.rand(n, 3, generator=g) * xyz
    # rois that start one voxel before the volume or end one voxel behind it: every sample out there is moved onto
    # the first / last voxel with its full weight, the most that one voxel can collect
    ctr[0] = ext[0] / 2 - 1.0
    ctr[1] = xyz - ext[1] / 2 + 1.0
    ctr[2, 0] = ext[2, 0] / 2 - 1.0
    b = torch.randint(0, 2, (n, 1), generator=g).float()
    if rotated:
        ext[:3] = ext[:3].clamp(max=4.0)
        ang = (torch.rand(n, 3, generator=g) * 2 - 1) * 0.7
        ang[:3] = 0
        rois = torch.cat([b, ctr + 0.5, ext, ang], 1)    # (aligned: the centre is taken half a voxel lower)
        mod = lambda sr: ops.RoIAlignRotated(out, 1.0, sr, True)
    else:
        rois = torch.cat([b, ctr - ext / 2, ctr + ext / 2], 1)
        mod = lambda sr: ops.RoIAlign(out, 1.0, sr)
    shape = (2, C, *size)
    for sr in (2, 3):
        x = torch.zeros(shape, dtype=dtype, device=DEV, requires_grad=True)
        y = mod(sr)(x, rois.to(DEV))
        gy = torch.ones(y.shape, dtype=dtype)
        y.backward(gy.to(DEV))
        want = oracle.roi_align_backward(gy, rois, shape, 1.0, sr, True, 1, rotated)
        assert_close(x.grad, want, BWD_TOL[dtype], f"backward sr={sr}")
        # every sample lies in the volume or is void: the mass that arrives is the mass of the valid samples
        assert abs(float(x.grad.double().sum()) - float(want.sum())) <= 2e-3 * float(want.abs().sum())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("ndim", [3, 2])
def test_rotated_heads_backward_with_many_rois_and_channels(ops, oracle, dtype, ndim):
    """Enough rois x channels for a workgroup to own several channels: a block's samples are worked out
    once and their taps kept in registers while the channels pass through the LDS tile.  Boxes from one
    channel per pass (large rois) to all of a workgroup's channels side by side (small ones), more samples
    per thread than are kept (grid 3, 14^2 cells), a NaN and an infinity in single channels (those
    channels' terms go out one by one, the others' through the tile), zero gradients."""
    g = wl.gen(650 + ndim)
    size = (18, 26, 30)[3 - ndim:]
    out = (7, 7, 7) if ndim == 3 else (14, 14)
    C, n = 32, 300
    feat = torch.randn(2, C, *size, generator=g).to(dtype)
    xyz = torch.tensor(size[::-1], dtype=torch.float32)
    ctr = (torch.rand(n, ndim, generator=g) * 1.2 - 0.1) * xyz
    ext = torch.exp(torch.rand(n, ndim, generator=g) * math.log(40.0)) * 0.6      # 0.6 .. 24 voxels
    ang = (torch.rand(n, 3 if ndim == 3 else 1, generator=g) * 2 - 1) * math.radians(40)
    rois = torch.cat([torch.randint(0, 2, (n, 1), generator=g).float(), ctr, ext, ang], 1)
    for sr in (2, 3, 0):
        x = feat.to(DEV).requires_grad_(True)
        y = ops.RoIAlignRotated(out, 1.0, sr, True)(x, rois.to(DEV))
        gy = torch.randn(y.shape, generator=g).to(dtype)
        gy[torch.rand(y.shape, generator=g) < 0.05] = 0
        y.backward(gy.to(DEV))
        want = oracle.roi_align_backward(gy, rois, feat.shape, 1.0, sr, True, 1, True)
        assert_close(x.grad, want, BWD_TOL[dtype], f"backward sr={sr}")
    x = feat.to(DEV).requires_grad_(True)
    y = ops.RoIAlignRotated(out, 1.0, 2, True)(x, rois.to(DEV))
    gy = torch.randn(y.shape, generator=g).to(dtype)
    big = int(torch.argmax(ext.prod(dim=1)))
    gy[big, 3].view(-1)[gy[big, 3].numel() // 2] = float("nan")
    gy[(big + 1) % n, 17].view(-1)[5] = float("inf")
    y.backward(gy.to(DEV))
    want = oracle.roi_align_backward(gy, rois, feat.shape, 1.0, 2, True, 1, True)
    got = x.grad.cpu()
    assert torch.isnan(want).any() and torch.equal(torch.isnan(got), torch.isnan(want))
    assert torch.equal(torch.isinf(got), torch.isinf(want))
    ok = torch.isfinite(want)
    assert_close(got[ok], want[ok], BWD_TOL[dtype], "NaN and infinite gradients")
    # Workgroups take the rois in descending order of size (every workgroup finds the roi of its rank by
    # itself), up to 4096 rois; beyond, in index order.  Either way every roi must be taken exactly once:
    # rois of equal size (one size class, ranks told apart by index), sizes over many octaves.
    for n in (4096, 4099):
        small = (2,) * ndim
        ctr = torch.rand(n, ndim, generator=g) * xyz
        ext = torch.exp(torch.rand(n, ndim, generator=g) * math.log(3000.0)) * 0.01
        ext[: n // 4] = 3.0
        ang = (torch.rand(n, 3 if ndim == 3 else 1, generator=g) * 2 - 1) * math.radians(40)
        rois = torch.cat([torch.randint(0, 2, (n, 1), generator=g).float(), ctr, ext, ang], 1)
        x = feat[:, :3].to(DEV).requires_grad_(True)
        y = ops.RoIAlignRotated(small, 1.0, 2, True)(x, rois.to(DEV))
        gy = torch.randn(y.shape, generator=g).to(dtype)
        y.backward(gy.to(DEV))
        want = oracle.roi_align_backward(gy, rois, x.shape, 1.0, 2, True, 1, True)
        assert_close(x.grad, want, BWD_TOL[dtype], f"{n} rois")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("ndim,rotated,C,out", [(3, True, 24, (7, 7, 7)), (3, True, 72, (7, 7, 7)),
                                                (2, True, 520, (14, 14)), (2, False, 32, (20, 20))])
def test_heads_forward_from_channels_last_copy(ops, oracle, dtype, ndim, rotated, C, out):
    """Detection heads that the separable pooled kernels do not take (rotated boxes, more than 16 cells per
    axis) read a channels-last copy of the features, a lane per (cell, 16 bytes of channels): channel
    counts that fill part of a wavefront, leave lanes idle (72 -> 9 lanes per cell) or need two passes
    (520), fixed and adaptive grids, order 0, rois sticking out of the image, a NaN feature; and the
    same call with a workspace too small for the copy (general kernel) gives the same numbers."""
    import ctypes
    from medvision_amd import _lib
    g = wl.gen(640 + ndim + C)
    size = (12, 20, 24)[3 - ndim:] if ndim == 3 else (40, 48)
    feat = torch.randn(2, C, *size, generator=g).to(dtype)
    xyz = torch.tensor(size[::-1], dtype=torch.float32)
    n = 30
    ctr = (torch.rand(n, ndim, generator=g) * 1.2 - 0.1) * xyz
    ext = torch.exp(torch.rand(n, ndim, generator=g) * math.log(40.0)) * 0.5      # 0.5 .. 20 voxels
    idx = torch.randint(0, 2, (n, 1), generator=g).float()
    ctr[:3], ext[:3], idx[0] = xyz * 0.5, xyz * 0.6, 0.0      # three rois over the middle of the image, one of them in image 0
    if rotated:
        ang = (torch.rand(n, 3 if ndim == 3 else 1, generator=g) * 2 - 1) * math.radians(40)
        rois = torch.cat([idx, ctr, ext, ang], 1)
        op = lambda sr: ops.RoIAlignRotated(out, 1.0, sr, True)
    else:
        rois = torch.cat([idx, ctr - ext / 2, ctr + ext / 2], 1)
        op = lambda sr: ops.RoIAlign(out, 1.0, sr)
    lib = _lib.load()
    in3, out3 = ([1, *size] if ndim == 2 else list(size)), ([1, *out] if ndim == 2 else list(out))
    need = lib.mv_roi_align_forward_workspace_bytes_for_input(_lib.dtype_code(feat), ndim, 2, C, *in3, n, *out3, 2)
    assert need == feat.numel() * feat.element_size(), "the channels-last path does not take this problem"
    x, r = feat.to(DEV), rois.to(DEV)
    for sr in (2, 0, 3):
        assert_close(op(sr)(x, r), oracle.roi_align_forward(feat, rois, out, 1.0, sr, True, 1, rotated),
                     FWD_TOL[dtype], f"forward sr={sr}")
    # without room for the copy the general kernel runs: same sample positions and tap decisions (the
    # same fp64 expressions), the same order of the sums -- order 0, which only picks voxels, must agree
    # exactly
    fn = {(3, True): lib.mv_roi_align_rotated_3d_forward, (2, True): lib.mv_roi_align_rotated_2d_forward,
          (2, False): lib.mv_roi_align_2d_forward}[(ndim, rotated)]
    # (through the C entry point: the module turns order 0 into a grid of one sample, too few for this path)
    small, room = torch.empty(1024, dtype=torch.uint8, device=DEV), torch.empty(need, dtype=torch.uint8, device=DEV)

    def raw(order, ws):
        y = torch.empty(n, C, *out, dtype=dtype, device=DEV)
        extra = (1, order) if rotated else (order,)
        _lib.check(fn(_lib.ptr(x), _lib.ptr(r), _lib.ptr(y), _lib.dtype_code(feat), 2, C, *size, n, *out,
                      ctypes.c_float(1.0), 2, *extra, _lib.ptr(ws), ctypes.c_size_t(ws.numel()), _lib.stream_of(x)))
        torch.cuda.synchronize()
        return y

    assert torch.equal(raw(1, room), op(2)(x, r))
    assert_close(raw(1, small), raw(1, room).cpu(), {torch.float32: 2e-6, torch.float16: 1.1e-3, torch.bfloat16: 8.5e-3}[dtype],
                 "general kernel")
    assert torch.equal(raw(0, small), raw(0, room)), "order 0 against the general kernel"
    # a NaN feature reaches exactly the outputs it reaches in the oracle
    bad = feat.clone()
    bad[(0, 1) + tuple(v // 2 for v in size)] = float("nan")
    got = op(2)(bad.to(DEV), r).cpu()
    want = oracle.roi_align_forward(bad, rois, out, 1.0, 2, True, 1, rotated)
    assert torch.isnan(want).any() and torch.equal(torch.isnan(got), torch.isnan(want))
