"""TEST INFRASTRUCTURE ONLY: Python binding of the fp64 CPU oracle (``sampling_oracle.c``).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package.  The shipped package ``medvision_amd`` never does; its operators raise when
the HIP library is missing instead of falling back to anything here.

All functions take torch tensors (any float dtype, any device), convert them *exactly* to fp64 on
the CPU and return fp64 CPU tensors, i.e. they evaluate the reference operator
(``/root/reference/medvision/csrc/cuda/*.cuh`` with ``scalar_t = double``) on the very values the
device kernels see.  ``spatial_scale`` is rounded to fp32 first because the reference's binding
takes a C ``float`` (csrc/roi_align_3d.h:71).
"""
import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

_dp = ctypes.POINTER(ctypes.c_double)
_ip = ctypes.POINTER(ctypes.c_int)


def build(force=False):
    """Compile ``liboracle.so`` with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH) or (
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "sampling_oracle.c"))):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_sample_clamped.restype = ctypes.c_double
        _lib.orc_sample_clamped.argtypes = [_dp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                            ctypes.c_double, ctypes.c_double, ctypes.c_double,
                                            ctypes.c_int]
        _lib.orc_sample_cubic.restype = ctypes.c_double
        _lib.orc_sample_cubic.argtypes = [_dp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                          ctypes.c_int, ctypes.c_double, ctypes.c_double,
                                          ctypes.c_double]
    return _lib


def _f64(t):
    return t.detach().to("cpu", torch.float64).contiguous()


def _ptr(t):
    return ctypes.cast(t.data_ptr(), _dp) if t is not None else None


def _f32(v):
    return float(np.float32(v))


def sample_clamped(volume, z, y, x, order=1):
    """One sample of semantics S on a [D,H,W] volume (interpolation_helpers_3d.h:5-68,129-199)."""
    v = _f64(volume)
    D, H, W = v.shape
    return lib().orc_sample_clamped(_ptr(v), D, H, W, float(z), float(y), float(x), int(order))


def sample_cubic(volume, z, y, x):
    """One order-3 sample on a [D,H,W] volume or, for a 2-D tensor, an [H,W] image
    (cuda_aug/interpolation_helpers_3d.h:571-792, interpolation_helpers_2d.h:335-423)."""
    v = _f64(volume)
    ndim = v.dim()
    D, H, W = v.shape if ndim == 3 else (1,) + tuple(v.shape)
    return lib().orc_sample_cubic(_ptr(v), ndim, D, H, W, float(z), float(y), float(x))


def _roi_common(features_shape, rois, rotated):
    ndim = len(features_shape) - 2
    cols = {(2, False): 5, (3, False): 7, (2, True): 6, (3, True): 10}[(ndim, bool(rotated))]
    if rois.dim() != 2 or rois.shape[1] != cols:
        raise RuntimeError(f"wrong roi size! size_rois should be {cols}")
    if ndim == 2:
        N, C, H, W = features_shape
        D = 1
    else:
        N, C, D, H, W = features_shape
    return ndim, N, C, D, H, W


def _out_dims(ndim, output_size):
    if isinstance(output_size, int):
        output_size = (output_size,) * ndim
    assert len(output_size) == ndim
    return ((1,) + tuple(output_size)) if ndim == 2 else tuple(output_size)


def roi_align_forward(features, rois, output_size, spatial_scale=1.0, sampling_ratio=0,
                      aligned=True, order=1, rotated=False):
    """RoIAlign / RoIAlignRotated forward, 2-D or 3-D by the rank of ``features``.

    cuda/roi_align_{2,3}d_cuda_kernel.cuh (forward), cuda/roi_align_rotated_{2,3}d_cuda_kernel.cuh
    (forward).  ``aligned`` is ignored for the plain flavour, like in the reference.
    """
    ndim, N, C, D, H, W = _roi_common(features.shape, rois, rotated)
    od, oh, ow = _out_dims(ndim, output_size)
    f, r = _f64(features), _f64(rois)
    R = r.shape[0]
    out = torch.zeros((R, C, od, oh, ow), dtype=torch.float64)
    if R:
        lib().orc_roi_align_forward(_ptr(f), _ptr(r), _ptr(out), ndim, int(bool(rotated)),
                                    N, C, D, H, W, R, od, oh, ow,
                                    ctypes.c_double(_f32(spatial_scale)), int(sampling_ratio),
                                    int(bool(aligned)), int(order))
    return out[:, :, 0] if ndim == 2 else out


def roi_decision_margin(features_shape, rois, output_size, spatial_scale=1.0, sampling_ratio=0,
                        aligned=True, rotated=False):
    """[R, (od,) oh, ow]: distance (voxels) of each output cell's samples from a decision of the
    nearest-neighbour sampler (a 0.5 tie between two voxels, or the -1 / S edge of the void).
    A test may accept a differing order-0 output only where this is within the coordinate
    rounding of the kernel under test."""
    ndim, N, C, D, H, W = _roi_common(tuple(features_shape), rois, rotated)
    od, oh, ow = _out_dims(ndim, output_size)
    r = _f64(rois)
    R = r.shape[0]
    out = torch.zeros((R, od, oh, ow), dtype=torch.float64)
    if R:
        lib().orc_roi_decision_margin(_ptr(r), _ptr(out), ndim, int(bool(rotated)), D, H, W, R,
                                      od, oh, ow, ctypes.c_double(_f32(spatial_scale)),
                                      int(sampling_ratio), int(bool(aligned)))
    return out[:, 0] if ndim == 2 else out


def roi_align_backward(grad_output, rois, features_shape, spatial_scale=1.0, sampling_ratio=0,
                       aligned=True, order=1, rotated=False):
    """Adjoint of :func:`roi_align_forward`; returns grad wrt features (fp64, zero-initialised)."""
    ndim, N, C, D, H, W = _roi_common(tuple(features_shape), rois, rotated)
    g, r = _f64(grad_output), _f64(rois)
    if ndim == 2:
        oh, ow = g.shape[2:]
        od = 1
    else:
        od, oh, ow = g.shape[2:]
    R = r.shape[0]
    gin = torch.zeros((N, C, D, H, W), dtype=torch.float64)
    if R:
        lib().orc_roi_align_backward(_ptr(g), _ptr(r), _ptr(gin), ndim, int(bool(rotated)),
                                     N, C, D, H, W, R, od, oh, ow,
                                     ctypes.c_double(_f32(spatial_scale)), int(sampling_ratio),
                                     int(bool(aligned)), int(order))
    return gin[:, :, 0] if ndim == 2 else gin


def _triple(v):
    return tuple(v) if isinstance(v, (tuple, list)) else (v, v, v)


def _dcn_params(x, weight, stride, padding, dilation, groups, deformable_groups):
    """Shape record of the C oracle.  4-D ``x`` = image layer: a depth-1 volume with a 1 x kh x kw
    kernel and two offset components per tap (returns the 2-D output size)."""
    if x.dim() == 4:
        B, Cin, H, W = x.shape
        Cout, _, kh, kw = weight.shape
        pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
        (sh, sw), (ph, pw), (dh, dw) = pair(stride), pair(padding), pair(dilation)
        arr = (ctypes.c_int * 21)(B, Cin, 1, H, W, Cout, 1, kh, kw, 1, sh, sw, 0, ph, pw, 1, dh, dw,
                                  groups, deformable_groups, 2)
    else:
        B, Cin, D, H, W = x.shape
        Cout, _, kd, kh, kw = weight.shape
        s, p, d = _triple(stride), _triple(padding), _triple(dilation)
        arr = (ctypes.c_int * 21)(B, Cin, D, H, W, Cout, kd, kh, kw, *s, *p, *d, groups,
                                  deformable_groups, 3)
    dims = (ctypes.c_int * 3)()
    lib().orc_dcn3d_out_dims(arr, dims)
    return arr, (tuple(dims)[1:] if x.dim() == 4 else tuple(dims))


def dcn3d_forward(x, offset, mask, weight, bias=None, stride=1, padding=0, dilation=1, groups=1,
                  deformable_groups=1):
    """DCN 3-D forward; ``mask=None`` gives v1 (cuda/deform_conv_3d_cuda_kernel.cuh:178-254),
    otherwise v2 (cuda/modulated_deform_conv_3d_cuda_kernel.cuh:178-257).  4-D tensors give the
    2-D layers (cuda/deform_conv_2d_cuda_kernel.cuh, cuda/modulated_deform_conv_2d_cuda_kernel.cuh
    :118-190: offset channels 2k = h, 2k+1 = w)."""
    xs, offs, ws = _f64(x), _f64(offset), _f64(weight)
    ms = _f64(mask) if mask is not None else None
    bs = _f64(bias) if bias is not None else None
    arr, out = _dcn_params(xs, ws, stride, padding, dilation, groups, deformable_groups)
    y = torch.zeros((xs.shape[0], ws.shape[0], *out), dtype=torch.float64)
    lib().orc_dcn3d_forward(_ptr(xs), _ptr(offs), _ptr(ms), _ptr(ws), _ptr(bs), _ptr(y), arr)
    return y


def dcn3d_backward(x, offset, mask, weight, grad_output, with_bias=True, stride=1, padding=0,
                   dilation=1, groups=1, deformable_groups=1):
    """Analytic DCN 3-D gradients -> (gx, goffset, gmask|None, gweight, gbias|None)."""
    xs, offs, ws, gy = _f64(x), _f64(offset), _f64(weight), _f64(grad_output)
    ms = _f64(mask) if mask is not None else None
    arr, _ = _dcn_params(xs, ws, stride, padding, dilation, groups, deformable_groups)
    gx, goff, gw = torch.zeros_like(xs), torch.zeros_like(offs), torch.zeros_like(ws)
    gm = torch.zeros_like(ms) if ms is not None else None
    gb = torch.zeros(ws.shape[0], dtype=torch.float64) if with_bias else None
    lib().orc_dcn3d_backward(_ptr(xs), _ptr(offs), _ptr(ms), _ptr(ws), _ptr(gy), _ptr(gx),
                             _ptr(goff), _ptr(gm), _ptr(gw), _ptr(gb), arr)
    return gx, goff, gm, gw, gb


dcn2d_forward = dcn3d_forward     # the rank of ``x`` selects the layer family
dcn2d_backward = dcn3d_backward


def deform_warp(img, offset, order=1):
    """Displacement-field warp (ops/cuda_fun_tools.py:94-167, cuda_aug/deform_3d_cuda_kernel.cuh)."""
    ndim = img.dim() - 2
    im, of = _f64(img), _f64(offset)
    assert of.shape[1] == ndim and of.shape[2:] == im.shape[2:]
    B, C = im.shape[:2]
    D, H, W = ((1,) + tuple(im.shape[2:])) if ndim == 2 else tuple(im.shape[2:])
    out = torch.zeros_like(im)
    lib().orc_deform_warp(_ptr(im), _ptr(of), _ptr(out), ndim, B, C, D, H, W, int(order))
    return out


def deform_conv(x, offset, weight, bias=None, stride=1, padding=0, dilation=1, groups=1,
                deformable_groups=1, order=1):
    """The augmentation DCN in general: v1 forward with the clamped samplers, any kernel and weight
    (cuda_aug/deform_3d_cuda.cu:43-152, cuda_aug/deform_3d_cuda_kernel.cuh:8-89; 4-D tensors: the
    2-D twin, cuda_aug/deform_2d_cuda_kernel.cuh)."""
    xs, offs, ws = _f64(x), _f64(offset), _f64(weight)
    bs = _f64(bias) if bias is not None else None
    arr, out = _dcn_params(xs, ws, stride, padding, dilation, groups, deformable_groups)
    y = torch.zeros((xs.shape[0], ws.shape[0], *out), dtype=torch.float64)
    lib().orc_deform_conv(_ptr(xs), _ptr(offs), _ptr(ws), _ptr(bs), _ptr(y), arr, int(order))
    return y


def set_threads(n):
    """Number of OpenMP threads the oracle uses (for the CPU baseline timing)."""
    omp = ctypes.CDLL("libgomp.so.1")
    omp.omp_set_num_threads(int(n))
