"""Random deformable convolutions against the fp64 oracle: v1 / v2, 2-D / 3-D, per-axis kernel sizes,
strides, paddings and dilations, weight groups, deformable groups, channel counts on and off the
matrix-core paths, with and without bias - forward and all gradients through the functions of the
binding (`_C.*deform_conv_*`).  A longer run of the same generator (90 000 cases) found no mismatch
beyond the two effects the generator now avoids or allows for: the offset gradient is one-sided at
integer sample positions (fp32 position arithmetic rounds a position within 1e-7 of an integer onto it,
the fp64 oracle does not), and bf16 outputs of small layers reach 5e-3 of the largest output."""
import math
import random

import pytest
import torch

from parity import BWD_TOL, FWD_TOL, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    import medvision_amd.ops as ops_
    from medvision_amd import _lib
    _lib.load()
    return ops_


def make_case(seed):
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    nd = rng.choice([2, 3, 3])
    modulated = rng.random() < 0.6
    dtype = rng.choice([torch.float32, torch.float16, torch.bfloat16, torch.float16])
    groups, dg = rng.choice([1, 1, 1, 2, 4]), rng.choice([1, 1, 2, 4])
    both = groups * dg // math.gcd(groups, dg)
    cin = both * (rng.choice([5, 6, 10, 12, 20]) if rng.random() < 0.3 else rng.choice([1, 2, 3, 4, 8, 8, 16, 16, 32]))
    cout = groups * rng.choice([1, 2, 3, 8, 16, 16, 32, 32, 40, 64])
    k = [rng.choice([1, 2, 3, 3, 3, 5]) for _ in range(nd)]
    if math.prod(k) > 45:
        k = [3] * nd
    stride = [rng.choice([1, 1, 1, 2]) for _ in range(nd)]
    pad = [rng.choice([0, 1, 1, 2]) for _ in range(nd)]
    dil = [rng.choice([1, 1, 1, 2]) for _ in range(nd)]
    B = rng.choice([1, 2, 3])
    lo, hi = (3, 14) if nd == 3 else (5, 34)
    size = [rng.randint(lo, hi) for _ in range(nd)]
    out = [(s + 2 * p - (d * (kk - 1) + 1)) // st + 1 for s, p, d, kk, st in zip(size, pad, dil, k, stride)]
    if min(out) < 1:
        return None
    K, Q = math.prod(k), math.prod(out)
    while B * cout * (cin // groups) * K * Q > 4e7 and cout > groups:
        cout = max(groups, cout // 2 // groups * groups)
    while B * cout * (cin // groups) * K * Q > 4e7 and cin > both:
        cin = max(both, cin // 2 // both * both)
    if B * cout * (cin // groups) * K * Q > 4e7:
        return None
    std = rng.choice([0.5, 2.0, 2.0, 5.0])
    x = torch.randn(B, cin, *size, generator=g)
    bound = 1.0 / math.sqrt(cin // groups * K)
    w = (torch.rand(cout, cin // groups, *k, generator=g) * 2 - 1) * bound
    bias = (torch.rand(cout, generator=g) * 2 - 1) * bound
    with_bias = rng.random() < 0.8 or not modulated
    off = (torch.randn(B, dg * nd * K, *out, generator=g) * std).to(dtype).float()
    # sample positions are integers plus the offset: keep them away from the integers
    off = torch.where((off - off.round()).abs() < 2e-3, off + 0.25, off)
    mask = torch.sigmoid(torch.randn(B, dg * K, *out, generator=g)) if modulated else None
    gy = torch.randn(B, cout, *out, generator=g)
    cast = lambda t: None if t is None else t.to(dtype)
    what = (f"seed={seed} nd={nd} v{2 if modulated else 1} {dtype} groups={groups} dg={dg} cin={cin} cout={cout} k={k} "
            f"stride={stride} pad={pad} dil={dil} B={B} size={size} std={std} bias={with_bias}")
    return dict(nd=nd, modulated=modulated, dtype=dtype, geometry=(*k, *stride, *pad, *dil, groups, dg),
                stride=tuple(stride), pad=tuple(pad), dil=tuple(dil), groups=groups, dg=dg, out=out,
                x=cast(x), w=cast(w), bias=cast(bias), off=cast(off), mask=cast(mask), gy=cast(gy),
                with_bias=with_bias, what=what)


@pytest.mark.parametrize("block", range(4))
def test_random_layers_vs_oracle(ops, oracle, block):
    from medvision_amd import _C
    for seed in range(800000 + block * 120, 800000 + (block + 1) * 120):
        c = make_case(seed)
        if c is None:
            continue
        dtype, what = c["dtype"], c["what"]
        x, w, bias, off, mask, gy = [None if c[n] is None else c[n].to(DEV) for n in ("x", "w", "bias", "off", "mask", "gy")]
        family = "3d" if c["nd"] == 3 else "2d"
        has_bias = c["with_bias"] or not c["modulated"]
        if c["modulated"]:
            y = torch.empty(x.size(0), w.size(0), *c["out"], dtype=dtype, device=DEV)
            getattr(_C, f"modulated_deform_conv_{family}_forward")(x, w, bias, None, off, mask, y, None, *c["geometry"],
                                                                    c["with_bias"])
        else:
            y = getattr(_C, f"deform_conv_{family}_forward")(x, w, bias, off, *c["geometry"], 64)
        geo = (c["stride"], c["pad"], c["dil"], c["groups"], c["dg"])
        want = oracle.dcn3d_forward(c["x"], c["off"], c["mask"], c["w"], c["bias"] if has_bias else None, *geo)
        e = rel_err(y, want)
        assert e <= (6e-3 if dtype == torch.bfloat16 else FWD_TOL[dtype]), f"{what}: forward rel err {e:.3e}"
        if c["modulated"]:
            gi, gw, gb, goff, gm = [torch.zeros_like(t) for t in (x, w, bias, off, mask)]
            getattr(_C, f"modulated_deform_conv_{family}_backward")(x, w, bias, None, off, mask, None, gi, gw, gb, goff, gm,
                                                                     gy, *c["geometry"], c["with_bias"])
        else:
            gi, goff, gw, gb = getattr(_C, f"deform_conv_{family}_backward")(x, w, bias, off, gy, *c["geometry"], 64)
            gm = None
        ox, ooff, om, ow, ob = oracle.dcn3d_backward(c["x"], c["off"], c["mask"], c["w"], c["gy"], has_bias, *geo)
        tol = BWD_TOL[dtype]
        for name, got, ref in (("input", gi, ox), ("offset", goff, ooff), ("weight", gw, ow), ("mask", gm, om)):
            if ref is not None:
                e = rel_err(got, ref)
                assert e <= tol, f"{what}: grad {name} rel err {e:.3e}"
        if has_bias:
            # a sum of B * Q gradients: measured against the size such a sum has when it does not cancel
            terms = c["gy"].numel() // c["gy"].size(1)
            e = float((gb.cpu().double() - ob).abs().max()) / max(float(ob.abs().max()), math.sqrt(terms))
            assert e <= tol, f"{what}: grad bias err {e:.3e}"
