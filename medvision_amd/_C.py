"""Drop-in for the reference's pybind11 module ``medvision._C`` on the sampling path.

Function names, argument order and error behaviour follow ``medvision/csrc/vision.cpp:26-77`` and
the dispatch headers it includes; the work is done by ``libmedvision_hip.so`` through its C ABI.
Deliberate differences from the reference binding:

* rois may have any float dtype; they are cast once to fp32 (fp64 for double features) instead of
  having to match the feature dtype (reference reads ``rois.data<scalar_t>()``,
  csrc/cuda/roi_align_3d_cuda.cu:17);
* kernels run on the current torch stream of the feature tensor's device (the reference RoI
  launchers use the legacy default stream, csrc/cuda/roi_align_3d_cuda.cu:20-21);
* output / gradient buffers must be contiguous (the reference silently writes into a temporary
  when they are not, csrc/cuda/roi_align_3d_cuda.cu:18);
* bfloat16 is accepted in addition to double / float / half.
"""
import ctypes

import torch

from . import _lib


def _require_cuda(t, what):
    if not t.is_cuda:
        raise RuntimeError(f"{what} is not implemented on CPU")


def _same_device(ref, **tensors):
    """Every tensor whose address goes to a kernel must live on the device the kernel runs on (a
    host or foreign pointer would fault on the GPU instead of raising)."""
    for name, t in tensors.items():
        if t is not None and t.device != ref.device:
            raise RuntimeError(f"{name} is on {t.device}, expected {ref.device} like the input tensor")


class _on_device:
    """``torch.cuda.device`` only when the tensor's device is not already current."""
    __slots__ = ("guard",)

    def __init__(self, t):
        idx = t.device.index
        self.guard = None if idx is None or idx == torch.cuda.current_device() else torch.cuda.device(idx)

    def __enter__(self):
        if self.guard is not None:
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)
        return False


_ws_bytes_cache = {}


def _cached_bytes(fn, *key):
    """Workspace sizes depend on the shape key alone: ask the library once per key."""
    k = (fn, key)
    n = _ws_bytes_cache.get(k)
    if n is None:
        n = _ws_bytes_cache[k] = getattr(_lib.load(), fn)(*key)
    return n


def _prep_rois(rois, features, cols):
    if rois.dim() != 2 or rois.size(1) != cols:
        raise RuntimeError(f"wrong roi size! size_rois should be {cols}")
    want = torch.float64 if features.dtype == torch.float64 else torch.float32
    return rois.to(device=features.device, dtype=want).contiguous()


def _require_contiguous(t, name):
    if not t.is_contiguous():
        raise RuntimeError(f"{name} tensor has to be contiguous")


def _roi_forward(fn_name, what, ndim, cols, input, rois, output, out_sizes, spatial_scale,
                 sampling_ratio, extra):
    _require_cuda(input, what)
    lib = _lib.load()
    _same_device(input, output=output)
    _require_contiguous(output, "output")
    if output.dtype != input.dtype:
        raise RuntimeError("output dtype must match input dtype")
    feats = input.contiguous()
    r = _prep_rois(rois, feats, cols)
    dims = list(feats.shape)
    if len(dims) != ndim + 2:
        raise RuntimeError(f"expected a {ndim + 2}-d feature tensor, got {len(dims)}-d")
    want_shape = (r.size(0), dims[1], *out_sizes)
    if tuple(output.shape) != want_shape:
        raise RuntimeError(f"output has shape {tuple(output.shape)}, expected {want_shape}")
    # (int32: label maps through the affine engines at order 0, which the library samples as they are)
    code = _lib.MV_I32 if feats.dtype == torch.int32 and what == "affine" else _lib.dtype_code(feats)
    out3 = out_sizes if ndim == 3 else (1, *out_sizes)
    # the tiled resampler's plans, a re-ordered copy of the features for detection heads with plain
    # boxes, a channels-last copy for heads the separable kernels do not take
    in3 = dims[2:] if ndim == 3 else [1, *dims[2:]]
    ws_bytes = _cached_bytes("mv_roi_align_forward_workspace_bytes_for_input", code, ndim, dims[0], dims[1],
                             *in3, r.size(0), *out3, int(sampling_ratio))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=feats.device) if ws_bytes else None
    with _on_device(feats):
        _lib.check(getattr(lib, fn_name)(
            _lib.ptr(feats), _lib.ptr(r), _lib.ptr(output), code, *dims,
            r.size(0), *out_sizes, float(spatial_scale), int(sampling_ratio), *extra,
            _lib.ptr(ws), ws_bytes, _lib.stream_of(feats)))


def roi_align_prepare(features):
    """The re-ordered copy of ``features`` that the RoIAlign forward of detection heads reads (made by
    every call in its workspace otherwise), for callers that pool one feature map several times; None
    when the forward pass has no use for one (other than fp16, width no multiple of four).  No
    counterpart in the reference.  Pass it as ``prepared`` to ``roi_align_{2,3}d_forward`` together with
    the same, unchanged features."""
    _require_cuda(features, "RoIAlign")
    _require_contiguous(features, "features")
    ndim = features.dim() - 2
    if ndim not in (2, 3):
        raise RuntimeError(f"expected a 4-d or 5-d feature tensor, got {features.dim()}-d")
    lib = _lib.load()
    code = _lib.dtype_code(features)
    dims = list(features.shape)
    d5 = dims if ndim == 3 else [dims[0], dims[1], 1, dims[2], dims[3]]
    nbytes = _cached_bytes("mv_roi_align_prepared_bytes", code, ndim, *d5)
    if nbytes == 0:
        return None
    copy = torch.empty(nbytes, dtype=torch.uint8, device=features.device)
    with _on_device(features):
        _lib.check(lib.mv_roi_align_prepare_features(_lib.ptr(features), code, ndim, *d5, _lib.ptr(copy), nbytes,
                                                     _lib.stream_of(features)))
    return copy


def _roi_forward_prepared(ndim, input, prepared, rois, output, out_sizes, spatial_scale, sampling_ratio, order):
    _require_cuda(input, "RoIAlign")
    lib = _lib.load()
    _same_device(input, output=output, prepared=prepared)
    _require_contiguous(output, "output")
    _require_contiguous(input, "input")
    if output.dtype != input.dtype:
        raise RuntimeError("output dtype must match input dtype")
    r = _prep_rois(rois, input, 1 + 2 * ndim)
    dims = list(input.shape)
    if len(dims) != ndim + 2:
        raise RuntimeError(f"expected a {ndim + 2}-d feature tensor, got {len(dims)}-d")
    want_shape = (r.size(0), dims[1], *out_sizes)
    if tuple(output.shape) != want_shape:
        raise RuntimeError(f"output has shape {tuple(output.shape)}, expected {want_shape}")
    code = _lib.dtype_code(input)
    d5 = dims if ndim == 3 else [dims[0], dims[1], 1, dims[2], dims[3]]
    out3 = out_sizes if ndim == 3 else (1, *out_sizes)
    if prepared.numel() != _cached_bytes("mv_roi_align_prepared_bytes", code, ndim, *d5):
        raise RuntimeError("prepared copy does not belong to features of this shape")
    # four bytes per roi for the order the rois are worked in; what heads the copy does not serve need
    ws_bytes = max(4 * r.size(0), _cached_bytes("mv_roi_align_forward_workspace_bytes", code, ndim, dims[1], r.size(0),
                                                *out3, int(sampling_ratio)))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=input.device) if ws_bytes else None
    with _on_device(input):
        _lib.check(lib.mv_roi_align_forward_prepared(
            _lib.ptr(input), _lib.ptr(prepared), _lib.ptr(r), _lib.ptr(output), code, ndim, *d5, r.size(0), *out3,
            float(spatial_scale), int(sampling_ratio), int(order), _lib.ptr(ws), ws_bytes, _lib.stream_of(input)))


def _roi_backward(fn_name, what, ndim, cols, top_grad, rois, bottom_grad, out_sizes,
                  spatial_scale, sampling_ratio, extra):
    _require_cuda(top_grad, what)
    lib = _lib.load()
    _same_device(top_grad, bottom_grad=bottom_grad)
    _require_contiguous(bottom_grad, "bottom_grad")
    if bottom_grad.dtype != top_grad.dtype:
        raise RuntimeError("bottom_grad dtype must match top_grad dtype")
    g = top_grad.contiguous()
    r = _prep_rois(rois, g, cols)
    dims = list(bottom_grad.shape)
    if len(dims) != ndim + 2:
        raise RuntimeError(f"expected a {ndim + 2}-d gradient buffer, got {len(dims)}-d")
    want_shape = (r.size(0), dims[1], *out_sizes)
    if tuple(g.shape) != want_shape:
        raise RuntimeError(f"top_grad has shape {tuple(g.shape)}, expected {want_shape}")
    code = _lib.dtype_code(g)
    d5 = dims if ndim == 3 else [dims[0], dims[1], 1, dims[2], dims[3]]
    ws_bytes = _cached_bytes("mv_roi_align_backward_workspace_bytes", code, *d5)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=g.device) if ws_bytes else None
    with _on_device(g):
        _lib.check(getattr(lib, fn_name)(
            _lib.ptr(g), _lib.ptr(r), _lib.ptr(bottom_grad), code, *dims, r.size(0), *out_sizes,
            float(spatial_scale), int(sampling_ratio), *extra, _lib.ptr(ws), _lib.stream_of(g)))


# ---- csrc/roi_align_2d.h, csrc/roi_align_3d.h:71-117 ------------------------------------
def roi_align_2d_forward(input, rois, output, out_h, out_w, spatial_scale, sampling_ratio, order, prepared=None):
    if prepared is not None:
        return _roi_forward_prepared(2, input, prepared, rois, output, (out_h, out_w), spatial_scale, sampling_ratio, order)
    _roi_forward("mv_roi_align_2d_forward", "RoIAlign", 2, 5, input, rois, output,
                 (out_h, out_w), spatial_scale, sampling_ratio, (int(order),))


def roi_align_2d_backward(top_grad, rois, bottom_grad, out_h, out_w, spatial_scale,
                          sampling_ratio, order):
    _roi_backward("mv_roi_align_2d_backward", "RoIAlign", 2, 5, top_grad, rois, bottom_grad,
                  (out_h, out_w), spatial_scale, sampling_ratio, (int(order),))


def roi_align_3d_forward(input, rois, output, out_d, out_h, out_w, spatial_scale, sampling_ratio,
                         order, prepared=None):
    if prepared is not None:
        return _roi_forward_prepared(3, input, prepared, rois, output, (out_d, out_h, out_w), spatial_scale,
                                     sampling_ratio, order)
    _roi_forward("mv_roi_align_3d_forward", "RoIAlign", 3, 7, input, rois, output,
                 (out_d, out_h, out_w), spatial_scale, sampling_ratio, (int(order),))


def roi_align_3d_backward(top_grad, rois, bottom_grad, out_d, out_h, out_w, spatial_scale,
                          sampling_ratio, order):
    _roi_backward("mv_roi_align_3d_backward", "RoIAlign", 3, 7, top_grad, rois, bottom_grad,
                  (out_d, out_h, out_w), spatial_scale, sampling_ratio, (int(order),))


# ---- csrc/roi_align_rotated_2d.h, csrc/roi_align_rotated_3d.h:71-117 ----------------------
def roi_align_rotated_2d_forward(input, rois, output, out_h, out_w, spatial_scale,
                                 sampling_ratio, aligned, order):
    _roi_forward("mv_roi_align_rotated_2d_forward", "RoIAlignRotated", 2, 6, input, rois, output,
                 (out_h, out_w), spatial_scale, sampling_ratio, (int(bool(aligned)), int(order)))


def roi_align_rotated_2d_backward(top_grad, rois, bottom_grad, out_h, out_w, spatial_scale,
                                  sampling_ratio, aligned, order):
    _roi_backward("mv_roi_align_rotated_2d_backward", "RoIAlignRotated", 2, 6, top_grad, rois,
                  bottom_grad, (out_h, out_w), spatial_scale, sampling_ratio,
                  (int(bool(aligned)), int(order)))


def roi_align_rotated_3d_forward(input, rois, output, out_d, out_h, out_w, spatial_scale,
                                 sampling_ratio, aligned, order):
    _roi_forward("mv_roi_align_rotated_3d_forward", "RoIAlignRotated", 3, 10, input, rois, output,
                 (out_d, out_h, out_w), spatial_scale, sampling_ratio,
                 (int(bool(aligned)), int(order)))


def roi_align_rotated_3d_backward(top_grad, rois, bottom_grad, out_d, out_h, out_w, spatial_scale,
                                  sampling_ratio, aligned, order):
    _roi_backward("mv_roi_align_rotated_3d_backward", "RoIAlignRotated", 3, 10, top_grad, rois,
                  bottom_grad, (out_d, out_h, out_w), spatial_scale, sampling_ratio,
                  (int(bool(aligned)), int(order)))


# ---- csrc/affine_2d.h, csrc/affine_3d.h:40-65 ---------------------------------------------
def affine_2d(input, rois, output, out_h, out_w, spatial_scale, sampling_ratio, aligned, order):
    _roi_forward("mv_affine_2d", "affine", 2, 6, input, rois, output, (out_h, out_w),
                 spatial_scale, sampling_ratio, (int(bool(aligned)), int(order)))


def affine_3d(input, rois, output, out_d, out_h, out_w, spatial_scale, sampling_ratio, aligned,
              order):
    _roi_forward("mv_affine_3d", "affine", 3, 10, input, rois, output, (out_d, out_h, out_w),
                 spatial_scale, sampling_ratio, (int(bool(aligned)), int(order)))


# ---- deformable convolution (3-D volumes, 2-D images) ----------------------------------------
def _dcn_shape(input, weight, kernel, stride, pad, dil, group, deformable_group):
    """Checked shape record; the rank of ``input`` (5 or 4) selects volumes or images."""
    _require_contiguous(input, "input")
    _require_contiguous(weight, "weight")
    nd = len(kernel)
    if input.dim() != nd + 2 or weight.dim() != nd + 2:
        raise RuntimeError(f"expected {nd + 2}-d input and weight tensors")
    B, C = input.shape[:2]
    Cout, ck = weight.shape[:2]
    if tuple(weight.shape[2:]) != tuple(kernel):
        if nd == 3:
            raise RuntimeError("Input shape and kernel shape wont match: (%d x %d x %d vs %d x %d x %d)."
                               % (kernel[1], kernel[2], kernel[0], weight.shape[3], weight.shape[4],
                                  weight.shape[2]))
        raise RuntimeError("Input shape and kernel shape wont match: (%d x %d vs %d x %d)."
                           % (*kernel, *weight.shape[2:]))
    if C != ck * group:
        raise RuntimeError("Input shape and kernel channels wont match: (%d vs %d)." % (C, ck * group))
    if C % group or Cout % group:
        raise RuntimeError("channels(%d) and channels_out(%d) must divide group(%d)" % (C, Cout, group))
    if C % deformable_group:
        raise RuntimeError("channels(%d) must divide deformable_group(%d)" % (C, deformable_group))
    cls = _lib.DcnShape if nd == 3 else _lib.Dcn2dShape
    return cls(B, C, *input.shape[2:], Cout, *kernel, *stride, *pad, *dil, group, deformable_group)


def _dcn_family(shape):
    return "mv_dcn3d" if isinstance(shape, _lib.DcnShape) else "mv_dcn2d"


def _dcn_out_dims(lib, shape):
    nd = 3 if isinstance(shape, _lib.DcnShape) else 2
    dims = [ctypes.c_int() for _ in range(nd)]
    _lib.check(getattr(lib, _dcn_family(shape) + "_output_dims")(
        ctypes.byref(shape), *[ctypes.byref(d) for d in dims]))
    return tuple(d.value for d in dims)


def _dcn_taps(shape):
    return (shape.kernel_d if isinstance(shape, _lib.DcnShape) else 1) * shape.kernel_h * shape.kernel_w


def _dcn_check_aux(shape, dims, offset, mask, K):
    B, dg, nd = shape.batch, shape.deformable_groups, len(dims)
    if tuple(offset.shape) != (B, dg * nd * K, *dims):
        raise RuntimeError(f"offset has shape {tuple(offset.shape)}, expected {(B, dg * nd * K, *dims)}")
    if mask is not None and tuple(mask.shape) != (B, dg * K, *dims):
        raise RuntimeError(f"mask has shape {tuple(mask.shape)}, expected {(B, dg * K, *dims)}")


def _dcn_bytes(fn, shape, code):
    k = (fn, code, bytes(shape))
    n = _ws_bytes_cache.get(k)
    if n is None:
        n = _ws_bytes_cache[k] = getattr(_lib.load(), fn)(ctypes.byref(shape), code)
    return n


def _dcn_forward(input, offset, mask, weight, bias, output, shape):
    lib = _lib.load()
    _same_device(input, offset=offset, mask=mask, weight=weight, bias=bias, output=output)
    fam = _dcn_family(shape)
    dims = _dcn_out_dims(lib, shape)
    K = _dcn_taps(shape)
    offset = offset.to(input.dtype).contiguous()
    mask = mask.to(input.dtype).contiguous() if mask is not None else None
    _dcn_check_aux(shape, dims, offset, mask, K)
    if weight.dtype != input.dtype or (bias is not None and bias.dtype != input.dtype):
        raise RuntimeError("input, weight and bias must share one dtype")
    code = _lib.dtype_code(input)
    nbytes = _dcn_bytes(fam + "_forward_workspace_bytes", shape, code)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=input.device) if nbytes else None
    with _on_device(input):
        _lib.check(getattr(lib, fam + "_forward")(
            _lib.ptr(input), _lib.ptr(offset), _lib.ptr(mask), _lib.ptr(weight), _lib.ptr(bias),
            _lib.ptr(output), ctypes.byref(shape), code, _lib.ptr(ws), _lib.stream_of(input)))


def _dcn_backward(input, offset, mask, weight, grad_output, gi, goff, gmask, gw, gb, shape):
    lib = _lib.load()
    _same_device(input, offset=offset, mask=mask, weight=weight, grad_output=grad_output,
                 grad_input=gi, grad_offset=goff, grad_mask=gmask, grad_weight=gw, grad_bias=gb)
    fam = _dcn_family(shape)
    dims = _dcn_out_dims(lib, shape)
    K = _dcn_taps(shape)
    offset = offset.to(input.dtype).contiguous()
    mask = mask.to(input.dtype).contiguous() if mask is not None else None
    _dcn_check_aux(shape, dims, offset, mask, K)
    grad_output = grad_output.to(input.dtype).contiguous()
    if tuple(grad_output.shape) != (shape.batch, shape.out_channels, *dims):
        raise RuntimeError("Input shape and grad_out shape wont match: (%s vs %s)."
                           % ((shape.batch, shape.out_channels, *dims), tuple(grad_output.shape)))
    for t, n in ((gi, "grad_input"), (goff, "grad_offset"), (gw, "grad_weight")):
        _require_contiguous(t, n)
    code = _lib.dtype_code(input)
    nbytes = _dcn_bytes(fam + "_backward_workspace_bytes", shape, code)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=input.device) if nbytes else None
    with _on_device(input):
        _lib.check(getattr(lib, fam + "_backward")(
            _lib.ptr(input), _lib.ptr(offset), _lib.ptr(mask), _lib.ptr(weight),
            _lib.ptr(grad_output), _lib.ptr(gi), _lib.ptr(goff), _lib.ptr(gmask), _lib.ptr(gw),
            _lib.ptr(gb), ctypes.byref(shape), code, _lib.ptr(ws), _lib.stream_of(input)))


def set_dcn_column_budget(nbytes):
    """Budget (bytes) of the column buffer the DCN backward keeps for its weight kernel; layers
    beyond it gather the input a second time.  Returns the previous budget."""
    lib = _lib.load()
    old = lib.mv_dcn_column_budget()
    lib.mv_dcn_set_column_budget(int(nbytes))
    _ws_bytes_cache.clear()   # workspace sizes depend on it
    return old


def _im2col_step_check(batch, im2col_step):
    step = min(batch, im2col_step)
    if batch % step != 0:
        raise RuntimeError("batch(%d) must divide im2col_step(%d)" % (batch, step))


def _dcn_v1_forward(input, weight, bias, offset, kernel, stride, pad, dil, group, deformable_group,
                    im2col_step):
    if not input.is_cuda:
        raise RuntimeError("Not implemented on the CPU")
    _im2col_step_check(input.size(0), im2col_step)
    shape = _dcn_shape(input, weight, kernel, stride, pad, dil, group, deformable_group)
    dims = _dcn_out_dims(_lib.load(), shape)
    output = torch.empty((input.size(0), weight.size(0), *dims), dtype=input.dtype, device=input.device)
    _dcn_forward(input, offset, None, weight, bias.contiguous(), output, shape)
    return output


def _dcn_v1_backward(input, weight, bias, offset, grad_output, kernel, stride, pad, dil, group,
                     deformable_group, im2col_step):
    if not input.is_cuda:
        raise RuntimeError("Not implemented on the CPU")
    _im2col_step_check(input.size(0), im2col_step)
    shape = _dcn_shape(input, weight, kernel, stride, pad, dil, group, deformable_group)
    gi, goff = torch.zeros_like(input), torch.zeros_like(offset, dtype=input.dtype)
    gw, gb = torch.zeros_like(weight), torch.zeros_like(bias)
    _dcn_backward(input, offset, None, weight, grad_output, gi, goff, None, gw, gb, shape)
    return [gi, goff, gw, gb]


def _dcn_v2_forward(input, weight, bias, offset, mask, output, kernel, stride, pad, dil, group,
                    deformable_group, with_bias):
    if not input.is_cuda:
        raise RuntimeError("Not implemented on the CPU")
    shape = _dcn_shape(input, weight, kernel, stride, pad, dil, group, deformable_group)
    dims = _dcn_out_dims(_lib.load(), shape)
    want = (input.size(0), weight.size(0), *dims)
    if output.numel() != torch.Size(want).numel() or not output.is_contiguous():
        raise RuntimeError(f"output must be a contiguous tensor of shape {want}")
    if output.dtype != input.dtype:
        raise RuntimeError("output dtype must match input dtype")
    _dcn_forward(input, offset, mask, weight, bias.contiguous() if with_bias else None, output, shape)


def _dcn_v2_backward(input, weight, offset, mask, grad_input, grad_weight, grad_bias, grad_offset,
                     grad_mask, grad_output, kernel, stride, pad, dil, group, deformable_group,
                     with_bias):
    if not input.is_cuda:
        raise RuntimeError("Not implemented on the CPU")
    shape = _dcn_shape(input, weight, kernel, stride, pad, dil, group, deformable_group)
    for t in (grad_input, grad_weight, grad_offset, grad_mask):
        if t.dtype != input.dtype:
            raise RuntimeError("gradient buffers must have the dtype of input")
    _require_contiguous(grad_mask, "grad_mask")
    _dcn_backward(input, offset, mask, weight, grad_output, grad_input, grad_offset, grad_mask,
                  grad_weight, grad_bias if with_bias else None, shape)


# csrc/deform_conv_3d.h:48-129 (host: csrc/cuda/deform_conv_3d_cuda.cu:110-376)
def deform_conv_3d_forward(input, weight, bias, offset, kernel_d, kernel_h, kernel_w, stride_d,
                           stride_h, stride_w, pad_d, pad_h, pad_w, dilation_d, dilation_h,
                           dilation_w, group, deformable_group, im2col_step):
    return _dcn_v1_forward(input, weight, bias, offset, (kernel_d, kernel_h, kernel_w),
                           (stride_d, stride_h, stride_w), (pad_d, pad_h, pad_w),
                           (dilation_d, dilation_h, dilation_w), group, deformable_group, im2col_step)


def deform_conv_3d_backward(input, weight, bias, offset, grad_output, kernel_d, kernel_h, kernel_w,
                            stride_d, stride_h, stride_w, pad_d, pad_h, pad_w, dilation_d,
                            dilation_h, dilation_w, group, deformable_group, im2col_step):
    return _dcn_v1_backward(input, weight, bias, offset, grad_output, (kernel_d, kernel_h, kernel_w),
                            (stride_d, stride_h, stride_w), (pad_d, pad_h, pad_w),
                            (dilation_d, dilation_h, dilation_w), group, deformable_group, im2col_step)


# csrc/deform_conv_2d.h:41-109 (host: csrc/cuda/deform_conv_2d_cuda.cu:110-330)
def deform_conv_2d_forward(input, weight, bias, offset, kernel_h, kernel_w, stride_h, stride_w,
                           pad_h, pad_w, dilation_h, dilation_w, group, deformable_group,
                           im2col_step):
    return _dcn_v1_forward(input, weight, bias, offset, (kernel_h, kernel_w), (stride_h, stride_w),
                           (pad_h, pad_w), (dilation_h, dilation_w), group, deformable_group,
                           im2col_step)


def deform_conv_2d_backward(input, weight, bias, offset, grad_output, kernel_h, kernel_w, stride_h,
                            stride_w, pad_h, pad_w, dilation_h, dilation_w, group, deformable_group,
                            im2col_step):
    return _dcn_v1_backward(input, weight, bias, offset, grad_output, (kernel_h, kernel_w),
                            (stride_h, stride_w), (pad_h, pad_w), (dilation_h, dilation_w), group,
                            deformable_group, im2col_step)


# csrc/modulated_deform_conv_3d.h:61-117 (host: csrc/cuda/modulated_deform_conv_3d_cuda.cu:137-396)
def modulated_deform_conv_3d_forward(input, weight, bias, ones, offset, mask, output, columns,
                                     kernel_d, kernel_h, kernel_w, stride_d, stride_h, stride_w,
                                     pad_d, pad_h, pad_w, dilation_d, dilation_h, dilation_w,
                                     group, deformable_group, with_bias):
    """``ones`` and ``columns`` are scratch handles of the reference and are ignored."""
    _dcn_v2_forward(input, weight, bias, offset, mask, output, (kernel_d, kernel_h, kernel_w),
                    (stride_d, stride_h, stride_w), (pad_d, pad_h, pad_w),
                    (dilation_d, dilation_h, dilation_w), group, deformable_group, with_bias)


def modulated_deform_conv_3d_backward(input, weight, bias, ones, offset, mask, columns, grad_input,
                                      grad_weight, grad_bias, grad_offset, grad_mask, grad_output,
                                      kernel_d, kernel_h, kernel_w, stride_d, stride_h, stride_w,
                                      pad_d, pad_h, pad_w, dilation_d, dilation_h, dilation_w,
                                      group, deformable_group, with_bias):
    """Writes the analytic gradients of the forward.  The reference's 3-D v2 backward launches its
    col2im over a truncated index range and writes the mask gradient with a 2-D channel index
    (csrc/cuda/modulated_deform_conv_3d_cuda.cu:64, ..._kernel.cuh:410-411); those two defects
    are not reproduced."""
    _dcn_v2_backward(input, weight, offset, mask, grad_input, grad_weight, grad_bias, grad_offset,
                     grad_mask, grad_output, (kernel_d, kernel_h, kernel_w),
                     (stride_d, stride_h, stride_w), (pad_d, pad_h, pad_w),
                     (dilation_d, dilation_h, dilation_w), group, deformable_group, with_bias)


# csrc/modulated_deform_conv_2d.h:23-70 (host: csrc/cuda/modulated_deform_conv_2d_cuda.cu)
def modulated_deform_conv_2d_forward(input, weight, bias, ones, offset, mask, output, columns,
                                     kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w,
                                     dilation_h, dilation_w, group, deformable_group, with_bias):
    """``ones`` and ``columns`` are scratch handles of the reference and are ignored."""
    _dcn_v2_forward(input, weight, bias, offset, mask, output, (kernel_h, kernel_w),
                    (stride_h, stride_w), (pad_h, pad_w), (dilation_h, dilation_w), group,
                    deformable_group, with_bias)


def modulated_deform_conv_2d_backward(input, weight, bias, ones, offset, mask, columns, grad_input,
                                      grad_weight, grad_bias, grad_offset, grad_mask, grad_output,
                                      kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w,
                                      dilation_h, dilation_w, group, deformable_group, with_bias):
    _dcn_v2_backward(input, weight, offset, mask, grad_input, grad_weight, grad_bias, grad_offset,
                     grad_mask, grad_output, (kernel_h, kernel_w), (stride_h, stride_w),
                     (pad_h, pad_w), (dilation_h, dilation_w), group, deformable_group, with_bias)


# csrc/deform_2d.h, csrc/deform_3d.h:27-65 as used by ops/cuda_fun_tools.py:94-167
def _is_identity_warp(weight, bias, C, ndim):
    """True when ``weight`` is the C x C identity over a 1x1(x1) kernel and ``bias`` is zero.
    Checked on every call (one read-back): a tensor's address and version do not identify its
    contents (the allocator reuses addresses, writes through ``.data`` leave the version alone), so
    a remembered verdict could send a real 1x1x1 convolution down the warp path."""
    if tuple(weight.shape) != (C, C, *([1] * ndim)) or tuple(bias.shape) != (C,):
        return False
    eye = torch.eye(C, dtype=weight.dtype, device=weight.device)
    return bool(((weight.reshape(C, C) == eye).all() & (bias == 0).all()).item())


def _deform(fn_name, ndim, input, weight, bias, offset, kernel, stride, pad, dil, group,
            deformable_group, im2col_step, order):
    """csrc/deform_3d.h:27 -> csrc/cuda_aug/deform_3d_cuda.cu:43-152.  The way the reference calls
    it (1x1x1 kernel, identity weight, zero bias: ops/cuda_fun_tools.py:134-167) is a displacement-
    field warp and runs as one; anything else is the DCNv1 forward with the clamped samplers."""
    if not input.is_cuda:
        raise RuntimeError("Not implemented on the CPU")
    _same_device(input, weight=weight, bias=bias)
    if order not in (0, 1, 3):
        raise RuntimeError(f"order {order} is not supported (0 nearest, 1 linear, 3 cubic)")
    _require_contiguous(input, "input")
    offset = offset.to(device=input.device, dtype=input.dtype).contiguous()
    if (all(k == 1 for k in kernel) and all(s == 1 for s in stride) and all(p == 0 for p in pad)
            and group == 1 and deformable_group == 1
            and _is_identity_warp(weight, bias, input.size(1), ndim)):
        if tuple(offset.shape) != (input.size(0), ndim, *input.shape[2:]):
            raise RuntimeError("offset must have shape [B, %d, *spatial]" % ndim)
        out = torch.empty_like(input)
        with _on_device(input):
            _lib.check(getattr(_lib.load(), fn_name)(
                _lib.ptr(input), _lib.ptr(offset), _lib.ptr(out), _lib.dtype_code(input),
                *input.shape, int(order), _lib.stream_of(input)))
        return out
    _im2col_step_check(input.size(0), im2col_step)
    shape = _dcn_shape(input, weight, kernel, stride, pad, dil, group, deformable_group)
    lib = _lib.load()
    dims = _dcn_out_dims(lib, shape)
    _dcn_check_aux(shape, dims, offset, None, _dcn_taps(shape))
    bias = bias.contiguous()
    if weight.dtype != input.dtype or bias.dtype != input.dtype:
        raise RuntimeError("input, weight and bias must share one dtype")
    if tuple(bias.shape) != (weight.size(0),):
        raise RuntimeError("bias must have one entry per output channel")
    out = torch.empty((input.size(0), weight.size(0), *dims), dtype=input.dtype, device=input.device)
    with _on_device(input):
        _lib.check(getattr(lib, "mv_deform_conv_%dd" % ndim)(
            _lib.ptr(input), _lib.ptr(offset), _lib.ptr(weight), _lib.ptr(bias), _lib.ptr(out),
            ctypes.byref(shape), _lib.dtype_code(input), int(order), _lib.stream_of(input)))
    return out


def deform_2d(input, weight, bias, offset, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w,
              dilation_h, dilation_w, group, deformable_group, im2col_step, order):
    return _deform("mv_deform_warp_2d", 2, input, weight, bias, offset, (kernel_h, kernel_w),
                   (stride_h, stride_w), (pad_h, pad_w), (dilation_h, dilation_w), group,
                   deformable_group, im2col_step, order)


def deform_3d(input, weight, bias, offset, kernel_d, kernel_h, kernel_w, stride_d, stride_h,
              stride_w, pad_d, pad_h, pad_w, dilation_d, dilation_h, dilation_w, group,
              deformable_group, im2col_step, order):
    return _deform("mv_deform_warp_3d", 3, input, weight, bias, offset,
                   (kernel_d, kernel_h, kernel_w), (stride_d, stride_h, stride_w),
                   (pad_d, pad_h, pad_w), (dilation_d, dilation_h, dilation_w), group,
                   deformable_group, im2col_step, order)


def deform_warp(img, offset, order=1):
    """Direct entry to the warp kernel (no identity weight to build or verify)."""
    ndim = img.dim() - 2
    if not img.is_cuda:
        raise RuntimeError("Not implemented on the CPU")
    img = img.contiguous()
    labels = img.dtype == torch.int32   # label maps: order 0 picks voxels, so they are warped as they are
    if labels and order != 0:
        raise RuntimeError("int32 label maps are warped at order 0 only")
    offset = offset.to(device=img.device, dtype=torch.float32 if labels else img.dtype).contiguous()
    if tuple(offset.shape) != (img.size(0), ndim, *img.shape[2:]):
        raise RuntimeError("offset must have shape [B, %d, *spatial]" % ndim)
    if order not in (0, 1, 3):
        raise RuntimeError(f"order {order} is not supported (0 nearest, 1 linear, 3 cubic)")
    out = torch.empty_like(img)
    fn = "mv_deform_warp_2d" if ndim == 2 else "mv_deform_warp_3d"
    with _on_device(img):
        _lib.check(getattr(_lib.load(), fn)(
            _lib.ptr(img), _lib.ptr(offset), _lib.ptr(out), _lib.MV_I32 if labels else _lib.dtype_code(img),
            *img.shape, int(order), _lib.stream_of(img)))
    return out
