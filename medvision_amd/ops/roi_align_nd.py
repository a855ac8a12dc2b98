"""``RoIAlign`` for plain (axis-aligned) boxes, 2-D and 3-D.

Interface of the reference's ``medvision/ops/roi_align_nd.py`` (module :158-198, autograd
functions :7-155): ``RoIAlign(output_size, spatial_scale, sampling_ratio=-1)(features, rois,
order=1)`` with rois ``(n, 5) = (batch_index, x1, y1, x2, y2)`` or ``(n, 7) = (batch_index, x1, y1,
z1, x2, y2, z2)``.
"""
import torch.nn as nn
from torch.autograd import Function

from .. import _C


def _parse_output_size(output_size, ndim):
    if isinstance(output_size, int):
        return (output_size,) * ndim
    if isinstance(output_size, tuple):
        assert len(output_size) == ndim
        assert all(isinstance(v, int) for v in output_size)
        return output_size
    raise TypeError('"output_size" must be an integer or tuple of integers')


def _kernels(ndim):
    if ndim == 2:
        return _C.roi_align_2d_forward, _C.roi_align_2d_backward
    return _C.roi_align_3d_forward, _C.roi_align_3d_backward


class PreparedFeatures:
    """Features of a detection head together with the re-ordered copy that the forward pass of
    ``RoIAlign`` reads (it is made anew by every call otherwise): for heads that pool ONE feature map
    several times (cascade stages, several batches of rois).  Pass the object to ``RoIAlign`` in place of
    the features; gradients flow to ``features`` as usual.  The copy follows the contents the features
    had when the object was made: an in-place change that autograd sees raises, one that it does not see
    (writes through ``.data``) is the caller's to avoid.  No counterpart in the reference."""

    def __init__(self, features):
        self.features = features.contiguous()
        self.copy = _C.roi_align_prepare(self.features.detach())   # None: the forward pass has no use for one
        self._version = self.features._version

    def check(self):
        if self.features._version != self._version:
            raise RuntimeError("the features were changed in place after PreparedFeatures was made")


def _forward(ndim, ctx, features, rois, output_size, spatial_scale, sampling_ratio, order, prepared=None):
    out = _parse_output_size(output_size, ndim)
    ctx.spatial_scale, ctx.sampling_ratio, ctx.order = spatial_scale, sampling_ratio, order
    ctx.save_for_backward(rois)
    ctx.feature_size = features.size()
    # every output element is written by the kernel (zeros where a sample is void): no zero fill
    output = features.new_empty(rois.size(0), features.size(1), *out)
    if prepared is not None:
        _kernels(ndim)[0](features.contiguous(), rois, output, *out, spatial_scale, sampling_ratio, order, prepared)
    else:
        _kernels(ndim)[0](features, rois, output, *out, spatial_scale, sampling_ratio, order)
    return output


def _backward(ndim, ctx, grad_output):
    (rois,) = ctx.saved_tensors
    grad_input = None
    if ctx.needs_input_grad[0]:
        # the reference allocates this with the rois' dtype (roi_align_nd.py:64,139); the
        # gradient's dtype is used here, which is the same whenever the reference runs at all
        grad_input = grad_output.new_zeros(ctx.feature_size)
        _kernels(ndim)[1](grad_output.contiguous(), rois, grad_input, *grad_output.shape[2:],
                          ctx.spatial_scale, ctx.sampling_ratio, ctx.order)
    return grad_input, None, None, None, None, None, None


class RoIAlign2DFunction(Function):
    @staticmethod
    def forward(ctx, features, rois, output_size, spatial_scale, sampling_ratio=0, order=1, prepared=None):
        return _forward(2, ctx, features, rois, output_size, spatial_scale, sampling_ratio, order, prepared)

    @staticmethod
    def backward(ctx, grad_output):
        return _backward(2, ctx, grad_output)


class RoIAlign3DFunction(Function):
    @staticmethod
    def forward(ctx, features, rois, output_size, spatial_scale, sampling_ratio=0, order=1, prepared=None):
        return _forward(3, ctx, features, rois, output_size, spatial_scale, sampling_ratio, order, prepared)

    @staticmethod
    def backward(ctx, grad_output):
        return _backward(3, ctx, grad_output)


roi_align_2d = RoIAlign2DFunction.apply
roi_align_3d = RoIAlign3DFunction.apply


class RoIAlign(nn.Module):
    """RoI align pooling layer.

    Args:
        output_size (tuple): (h, w) or (d, h, w)
        spatial_scale (float): multiplies the box coordinates
        sampling_ratio (int): samples per bin and axis; <= 0 takes ceil(roi_size / output_size)
    """

    def __init__(self, output_size, spatial_scale, sampling_ratio=-1):
        super().__init__()
        assert iter(output_size)
        self.output_size = output_size
        self.spatial_scale = float(spatial_scale)
        self.sampling_ratio = int(sampling_ratio)
        self.dim = len(self.output_size)
        if self.dim == 2:
            self.roi_align = roi_align_2d
        elif self.dim == 3:
            self.roi_align = roi_align_3d
        else:
            raise Exception(
                "Tried to init RoIAlign module with incorrect output size: {}".format(self.output_size))

    def forward(self, features, rois, order=1):
        assert order in [0, 1], "only support order = 0 (nearest) or 1 (linear)"
        # nearest sampling must not average several samples (reference roi_align_nd.py:195)
        sampling_ratio = 1 if order == 0 else self.sampling_ratio
        if isinstance(features, PreparedFeatures):
            features.check()
            return self.roi_align(features.features, rois, self.output_size, self.spatial_scale, sampling_ratio,
                                  order, features.copy)
        return self.roi_align(features, rois, self.output_size, self.spatial_scale, sampling_ratio,
                              order)

    def __repr__(self):
        return (f"{self.__class__.__name__}(output_size={self.output_size}, "
                f"spatial_scale={self.spatial_scale}, sampling_ratio={self.sampling_ratio})")
