"""Pins the oracle's deformable-convolution and warp routines.

* zero offsets, mask == 1  ->  torch F.conv3d (textbook convolution), incl. groups/stride/dilation
* integer offsets          ->  convolution of a shifted input
* general                  ->  grid_sample(zeros, align_corners=True) + einsum (torch_ref.dcn3d)
* gradients                ->  torch autograd through that formulation (all five inputs)
* 2-D layers               ->  F.conv2d at zero offsets, a hand-shifted image for the channel order
                              (2k = rows, 2k+1 = columns), 2-D grid_sample + autograd in general
* warp                     ->  grid_sample(border) on the open interval, identity at zero offset
* augmentation DCN         ->  F.conv3d / F.conv2d at zero offsets for orders 0, 1 and 3; a pointwise
                              convolution of the (pinned) warp; grid_sample(border) per tap on the
                              open interval for kernels, strides, paddings, dilations and groups
"""
import pytest
import torch
import torch.nn.functional as F

import torch_ref


def _g(seed):
    return torch.Generator().manual_seed(seed)


@pytest.mark.parametrize("groups,stride,pad,dil", [(1, 1, 1, 1), (2, 2, 1, 1), (1, 1, 2, 2), (2, (1, 2, 1), (0, 1, 2), (1, 1, 2))])
def test_zero_offset_is_conv3d(oracle, groups, stride, pad, dil):
    g = _g(0)
    x = torch.randn(2, 4, 6, 7, 8, generator=g, dtype=torch.float64)
    w = torch.randn(6, 4 // groups, 3, 2, 3, generator=g, dtype=torch.float64)
    b = torch.randn(6, generator=g, dtype=torch.float64)
    want = F.conv3d(x, w, b, stride, pad, dil, groups)
    K = 18
    off = torch.zeros(2, 3 * K, *want.shape[2:], dtype=torch.float64)
    got = oracle.dcn3d_forward(x, off, None, w, b, stride, pad, dil, groups, 1)
    assert got.shape == want.shape
    assert torch.allclose(got, want, atol=1e-11)
    m = torch.full((2, K, *want.shape[2:]), 0.5, dtype=torch.float64)
    got = oracle.dcn3d_forward(x, off, m, w, None, stride, pad, dil, groups, 1)
    assert torch.allclose(got, 0.5 * (want - b.view(1, -1, 1, 1, 1)), atol=1e-11)


def test_integer_offset_is_shifted_conv(oracle):
    g = _g(1)
    x = torch.randn(1, 2, 6, 6, 6, generator=g, dtype=torch.float64)
    w = torch.randn(3, 2, 3, 3, 3, generator=g, dtype=torch.float64)
    off = torch.zeros(1, 81, 6, 6, 6, dtype=torch.float64)
    off[:, 0::3] = 1.0    # every tap moves +1 in depth
    off[:, 2::3] = -2.0   # and -2 in width
    got = oracle.dcn3d_forward(x, off, None, w, None, 1, 1, 1, 1, 1)
    # shifted input, zero fill: xs[d,h,w] = x[d+1,h,w-2]
    xs = torch.zeros(1, 2, 8, 8, 8, dtype=torch.float64)   # padded by 1 for the conv
    xp = F.pad(x, (3, 3, 3, 3, 3, 3))
    xs = xp[:, :, 2 + 1:2 + 1 + 8, 2:2 + 8, 2 - 2:2 - 2 + 8]
    want = F.conv3d(xs, w)
    assert torch.allclose(got, want, atol=1e-11)


@pytest.mark.parametrize("v2,groups,dg", [(True, 1, 1), (True, 2, 2), (False, 1, 2), (False, 2, 1)])
def test_general_and_gradients_vs_autograd(oracle, v2, groups, dg):
    g = _g(2 + groups + 2 * dg)
    B, Cin, Cout, D, H, W = 2, 4, 4, 4, 5, 6
    k, stride, pad, dil = (2, 3, 2), (1, 2, 1), (1, 1, 0), (1, 1, 2)
    K = 12
    x = torch.randn(B, Cin, D, H, W, generator=g, dtype=torch.float64, requires_grad=True)
    w = torch.randn(Cout, Cin // groups, *k, generator=g, dtype=torch.float64, requires_grad=True)
    b = torch.randn(Cout, generator=g, dtype=torch.float64, requires_grad=True)
    Do, Ho, Wo = [(S + 2 * p_ - (d_ * (k_ - 1) + 1)) // s_ + 1
                  for S, p_, d_, k_, s_ in zip((D, H, W), pad, dil, k, stride)]
    # offsets away from the integer lattice (bilinear kinks) but reaching outside the volume
    off = (torch.randn(B, dg * 3 * K, Do, Ho, Wo, generator=g, dtype=torch.float64) * 2.0)
    frac = off - off.floor()
    off = (off.floor() + frac.clamp(0.05, 0.95)).requires_grad_(True)
    m = torch.rand(B, dg * K, Do, Ho, Wo, generator=g, dtype=torch.float64).requires_grad_(True) if v2 else None
    want = torch_ref.dcn3d(x, off, m, w, b, stride, pad, dil, groups, dg)
    got = oracle.dcn3d_forward(x, off, m, w, b, stride, pad, dil, groups, dg)
    assert torch.allclose(got, want.detach(), atol=1e-11)
    gy = torch.randn(want.shape, generator=g, dtype=torch.float64)
    ins = [x, off, w, b] + ([m] if v2 else [])
    grads = torch.autograd.grad(want, ins, gy)
    gx, goff, gm, gw, gb = oracle.dcn3d_backward(x, off, m, w, gy, True, stride, pad, dil, groups, dg)
    assert torch.allclose(gx, grads[0], atol=1e-10)
    assert torch.allclose(goff, grads[1], atol=1e-10)
    assert torch.allclose(gw, grads[2], atol=1e-10)
    assert torch.allclose(gb, grads[3], atol=1e-10)
    if v2:
        assert torch.allclose(gm, grads[4], atol=1e-10)
    else:
        assert gm is None


@pytest.mark.parametrize("groups,stride,pad,dil", [(1, 1, 1, 1), (2, 2, 1, 1), (1, (1, 2), (2, 0), (2, 1))])
def test_2d_zero_offset_is_conv2d(oracle, groups, stride, pad, dil):
    g = _g(20)
    x = torch.randn(2, 4, 9, 10, generator=g, dtype=torch.float64)
    w = torch.randn(6, 4 // groups, 3, 2, generator=g, dtype=torch.float64)
    b = torch.randn(6, generator=g, dtype=torch.float64)
    want = F.conv2d(x, w, b, stride, pad, dil, groups)
    off = torch.zeros(2, 2 * 6, *want.shape[2:], dtype=torch.float64)
    got = oracle.dcn2d_forward(x, off, None, w, b, stride, pad, dil, groups, 1)
    assert got.shape == want.shape and torch.allclose(got, want, atol=1e-11)


def test_2d_offset_channel_order(oracle):
    """Channel 2k moves tap k along the rows (h), 2k+1 along the columns (w)."""
    g = _g(21)
    x = torch.randn(1, 1, 6, 7, generator=g, dtype=torch.float64)
    w = torch.ones(1, 1, 1, 1, dtype=torch.float64)
    off = torch.zeros(1, 2, 6, 7, dtype=torch.float64)
    off[:, 0] = 2.0   # rows
    off[:, 1] = -1.0  # columns
    got = oracle.dcn2d_forward(x, off, None, w, None)
    want = torch.zeros_like(x)
    want[0, 0, :4, 1:] = x[0, 0, 2:, :6]
    assert torch.allclose(got, want)


@pytest.mark.parametrize("v2,groups,dg", [(True, 1, 1), (True, 2, 2), (False, 1, 2), (False, 2, 1)])
def test_2d_general_and_gradients_vs_autograd(oracle, v2, groups, dg):
    g = _g(22 + groups + 2 * dg)
    B, Cin, Cout, H, W = 2, 4, 6, 7, 8
    k, stride, pad, dil = (3, 2), (2, 1), (1, 0), (1, 2)
    K = 6
    x = torch.randn(B, Cin, H, W, generator=g, dtype=torch.float64, requires_grad=True)
    w = torch.randn(Cout, Cin // groups, *k, generator=g, dtype=torch.float64, requires_grad=True)
    b = torch.randn(Cout, generator=g, dtype=torch.float64, requires_grad=True)
    Ho, Wo = [(S + 2 * p_ - (d_ * (k_ - 1) + 1)) // s_ + 1
              for S, p_, d_, k_, s_ in zip((H, W), pad, dil, k, stride)]
    off = torch.randn(B, dg * 2 * K, Ho, Wo, generator=g, dtype=torch.float64) * 2.0
    frac = off - off.floor()
    off = (off.floor() + frac.clamp(0.05, 0.95)).requires_grad_(True)
    m = torch.rand(B, dg * K, Ho, Wo, generator=g, dtype=torch.float64).requires_grad_(True) if v2 else None
    want = torch_ref.dcn2d(x, off, m, w, b, stride, pad, dil, groups, dg)
    got = oracle.dcn2d_forward(x, off, m, w, b, stride, pad, dil, groups, dg)
    assert torch.allclose(got, want.detach(), atol=1e-11)
    gy = torch.randn(want.shape, generator=g, dtype=torch.float64)
    ins = [x, off, w, b] + ([m] if v2 else [])
    grads = torch.autograd.grad(want, ins, gy)
    gx, goff, gm, gw, gb = oracle.dcn2d_backward(x, off, m, w, gy, True, stride, pad, dil, groups, dg)
    for got_, want_ in zip((gx, goff, gw, gb), grads[:4]):
        assert torch.allclose(got_, want_, atol=1e-10)
    if v2:
        assert torch.allclose(gm, grads[4], atol=1e-10)


def test_warp(oracle):
    g = _g(9)
    img = torch.randn(2, 3, 5, 6, 7, generator=g, dtype=torch.float64)
    zero = torch.zeros(2, 3, 5, 6, 7, dtype=torch.float64)
    assert torch.equal(oracle.deform_warp(img, zero), img)
    assert torch.equal(oracle.deform_warp(img, zero, order=0), img)
    off = torch.randn(2, 3, 5, 6, 7, generator=g, dtype=torch.float64) * 2
    dd, hh, ww = torch.meshgrid(torch.arange(5.), torch.arange(6.), torch.arange(7.), indexing="ij")
    for b in range(2):
        z, y, x = dd + off[b, 0], hh + off[b, 1], ww + off[b, 2]
        inside = (z > -1) & (z < 5) & (y > -1) & (y < 6) & (x > -1) & (x < 7)
        want = torch_ref.sample_border(img[b], z.double(), y.double(), x.double()) * inside
        assert torch.allclose(oracle.deform_warp(img, off)[b], want, atol=1e-12)
    # 2-D: channel 0 = h, channel 1 = w (integer shift check)
    im2 = torch.randn(1, 1, 6, 8, generator=g, dtype=torch.float64)
    o2 = torch.zeros(1, 2, 6, 8, dtype=torch.float64)
    o2[:, 0] = 1.0
    o2[:, 1] = -2.0
    got = oracle.deform_warp(im2, o2)
    want = torch.zeros_like(im2)
    for h in range(6):
        for w_ in range(8):
            sh, sw = h + 1, w_ - 2
            if -1 < sh < 6 and -1 < sw < 8:
                want[0, 0, h, w_] = im2[0, 0, min(max(sh, 0), 5), min(max(sw, 0), 7)]
    assert torch.allclose(got, want)


@pytest.mark.parametrize("order", [0, 1, 3])
def test_deform_conv_zero_offset_is_conv(oracle, order):
    g = _g(20 + order)
    x = torch.randn(2, 4, 6, 7, 8, generator=g, dtype=torch.float64)
    w = torch.randn(6, 2, 3, 2, 3, generator=g, dtype=torch.float64)
    b = torch.randn(6, generator=g, dtype=torch.float64)
    stride, pad, dil = (1, 2, 1), (2, 1, 3), (1, 1, 2)
    want = F.conv3d(x, w, b, stride, pad, dil, 2)
    off = torch.zeros(2, 2 * 3 * 18, *want.shape[2:], dtype=torch.float64)
    got = oracle.deform_conv(x, off, w, b, stride, pad, dil, 2, 2, order)
    assert got.shape == want.shape and torch.allclose(got, want, atol=1e-11)
    x2 = torch.randn(2, 4, 9, 8, generator=g, dtype=torch.float64)
    w2 = torch.randn(2, 4, 3, 2, generator=g, dtype=torch.float64)
    want = F.conv2d(x2, w2, None, (2, 1), (1, 2), (2, 1))
    off = torch.zeros(2, 2 * 6, *want.shape[2:], dtype=torch.float64)
    got = oracle.deform_conv(x2, off, w2, None, (2, 1), (1, 2), (2, 1), 1, 1, order)
    assert got.shape == want.shape and torch.allclose(got, want, atol=1e-11)


@pytest.mark.parametrize("order", [0, 1, 3])
def test_deform_conv_pointwise_is_conv_of_warp(oracle, order):
    g = _g(30 + order)
    x = torch.randn(2, 4, 5, 6, 7, generator=g, dtype=torch.float64)
    w = torch.randn(6, 2, 1, 1, 1, generator=g, dtype=torch.float64)
    b = torch.randn(6, generator=g, dtype=torch.float64)
    off = torch.randn(2, 2 * 3, 5, 6, 7, generator=g, dtype=torch.float64) * 2   # two offset groups
    warped = torch.cat([oracle.deform_warp(x[:, :2], off[:, :3], order),
                        oracle.deform_warp(x[:, 2:], off[:, 3:], order)], 1)
    want = F.conv3d(warped, w, b, groups=2)
    got = oracle.deform_conv(x, off, w, b, 1, 0, 1, 2, 2, order)
    assert torch.allclose(got, want, atol=1e-11)
    x2, off2 = x[:, :, 0].contiguous(), off[:, [1, 2, 4, 5], 0].contiguous()
    warped = torch.cat([oracle.deform_warp(x2[:, :2], off2[:, :2], order),
                        oracle.deform_warp(x2[:, 2:], off2[:, 2:], order)], 1)
    want = F.conv2d(warped, w[:, :, 0], b, groups=2)
    got = oracle.deform_conv(x2, off2, w[:, :, 0].contiguous(), b, 1, 0, 1, 2, 2, order)
    assert torch.allclose(got, want, atol=1e-11)


@pytest.mark.parametrize("groups,dg", [(1, 1), (2, 2), (2, 1)])
def test_deform_conv_linear_vs_grid_sample(oracle, groups, dg):
    g = _g(40 + groups + 2 * dg)
    B, Cin, Cout, D, H, W = 2, 4, 4, 4, 5, 6
    k, stride, pad, dil = (2, 3, 2), (1, 2, 1), (1, 1, 0), (1, 1, 2)
    K = 12
    x = torch.randn(B, Cin, D, H, W, generator=g, dtype=torch.float64)
    w = torch.randn(Cout, Cin // groups, *k, generator=g, dtype=torch.float64)
    b = torch.randn(Cout, generator=g, dtype=torch.float64)
    Do, Ho, Wo = [(S + 2 * p_ - (d_ * (k_ - 1) + 1)) // s_ + 1
                  for S, p_, d_, k_, s_ in zip((D, H, W), pad, dil, k, stride)]
    off = torch.randn(B, dg * 3 * K, Do, Ho, Wo, generator=g, dtype=torch.float64) * 2.0
    want = torch_ref.dcn3d(x, off, None, w, b, stride, pad, dil, groups, dg,
                           sampler=torch_ref.sample_border_open)
    got = oracle.deform_conv(x, off, w, b, stride, pad, dil, groups, dg, 1)
    assert torch.allclose(got, want, atol=1e-11)
    # image layer = the depth-1 volume with offset channels (2k, 2k+1) = (rows, columns)
    x2 = torch.randn(B, Cin, 7, 6, generator=g, dtype=torch.float64)
    w2 = torch.randn(Cout, Cin // groups, 3, 2, generator=g, dtype=torch.float64)
    Ho, Wo = (7 + 2 - 3) // 2 + 1, (6 + 0 - 3) // 1 + 1
    off2 = torch.randn(B, dg * 2 * 6, Ho, Wo, generator=g, dtype=torch.float64) * 2.0
    off3 = torch.zeros(B, dg * 6, 3, 1, Ho, Wo, dtype=torch.float64)
    off3[:, :, 1:, 0] = off2.reshape(B, dg * 6, 2, Ho, Wo)
    want = torch_ref.dcn3d(x2[:, :, None], off3.reshape(B, dg * 18, 1, Ho, Wo), None, w2[:, :, None],
                           b, (1, 2, 1), (0, 1, 0), (1, 1, 2), groups, dg,
                           sampler=torch_ref.sample_border_open)[:, :, 0]
    got = oracle.deform_conv(x2, off2, w2, b, (2, 1), (1, 0), (1, 2), groups, dg, 1)
    assert torch.allclose(got, want, atol=1e-11)
