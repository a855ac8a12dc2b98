"""``RoIAlignRotated`` for rotated boxes, 2-D and 3-D.

Interface of the reference's ``medvision/ops/roi_align_rotated_nd.py`` (module :168-239, autograd
functions :7-165): ``RoIAlignRotated(output_size, spatial_scale, sampling_ratio=-1,
aligned=True)(features, rois, order=1)`` with rois ``(n, 6) = (batch_index, center_x, center_y, w,
h, angle)`` or ``(n, 10) = (batch_index, center_x, center_y, center_z, w, h, d, angleX, angleY,
angleZ)``; angles in radian, counter-clockwise, applied as Rz * Ry * Rx.

``aligned=True`` shifts the scaled box by -0.5 so that continuous coordinate c has the pixel
neighbours floor(c - 0.5) and ceil(c - 0.5); ``aligned=False`` keeps the legacy behaviour and
forces degenerate boxes to be at least 1 x 1.
"""
import torch.nn as nn
from torch.autograd import Function

from .. import _C
from .roi_align_nd import _parse_output_size


def _kernels(ndim):
    if ndim == 2:
        return _C.roi_align_rotated_2d_forward, _C.roi_align_rotated_2d_backward
    return _C.roi_align_rotated_3d_forward, _C.roi_align_rotated_3d_backward


def _forward(ndim, ctx, features, rois, output_size, spatial_scale, sampling_ratio, aligned, order):
    out = _parse_output_size(output_size, ndim)
    ctx.spatial_scale, ctx.sampling_ratio = spatial_scale, sampling_ratio
    ctx.aligned, ctx.order = aligned, order
    ctx.save_for_backward(rois)
    ctx.feature_size = features.size()
    # every output element is written by the kernel (zeros where a sample is void): no zero fill
    output = features.new_empty(rois.size(0), features.size(1), *out)
    _kernels(ndim)[0](features, rois, output, *out, spatial_scale, sampling_ratio, aligned, order)
    return output


def _backward(ndim, ctx, grad_output):
    (rois,) = ctx.saved_tensors
    grad_input = None
    if ctx.needs_input_grad[0]:
        grad_input = grad_output.new_zeros(ctx.feature_size)
        _kernels(ndim)[1](grad_output.contiguous(), rois, grad_input, *grad_output.shape[2:],
                          ctx.spatial_scale, ctx.sampling_ratio, ctx.aligned, ctx.order)
    return grad_input, None, None, None, None, None, None


class RoIAlignRotated2DFunction(Function):
    @staticmethod
    def forward(ctx, features, rois, output_size, spatial_scale, sampling_ratio=0, aligned=True,
                order=1):
        return _forward(2, ctx, features, rois, output_size, spatial_scale, sampling_ratio, aligned,
                        order)

    @staticmethod
    def backward(ctx, grad_output):
        return _backward(2, ctx, grad_output)


class RoIAlignRotated3DFunction(Function):
    @staticmethod
    def forward(ctx, features, rois, output_size, spatial_scale, sampling_ratio=0, aligned=True,
                order=1):
        return _forward(3, ctx, features, rois, output_size, spatial_scale, sampling_ratio, aligned,
                        order)

    @staticmethod
    def backward(ctx, grad_output):
        return _backward(3, ctx, grad_output)


roi_align_rotated_2d = RoIAlignRotated2DFunction.apply
roi_align_rotated_3d = RoIAlignRotated3DFunction.apply


class RoIAlignRotated(nn.Module):
    """RoI align pooling layer for rotated proposals.

    Args:
        output_size (tuple): (h, w) or (d, h, w)
        spatial_scale (float): multiplies the box centre and size
        sampling_ratio (int): samples per bin and axis; <= 0 takes ceil(roi_size / output_size)
        aligned (bool): pixel-centre alignment (see module docstring). Default: True.
    """

    def __init__(self, output_size, spatial_scale, sampling_ratio=-1, aligned=True):
        super().__init__()
        assert iter(output_size)
        self.output_size = output_size
        self.spatial_scale = float(spatial_scale)
        self.sampling_ratio = int(sampling_ratio)
        self.aligned = aligned
        self.dim = len(self.output_size)
        if self.dim == 2:
            self.roi_align = roi_align_rotated_2d
        elif self.dim == 3:
            self.roi_align = roi_align_rotated_3d
        else:
            raise Exception(
                "Tried to init RoIAlign module with incorrect output size: {}".format(self.output_size))

    def forward(self, features, rois, order=1):
        assert order in [0, 1], "only support order = 0 (nearest) or 1 (linear)"
        sampling_ratio = 1 if order == 0 else self.sampling_ratio
        return self.roi_align(features, rois, self.output_size, self.spatial_scale, sampling_ratio,
                              self.aligned, order)

    def __repr__(self):
        return (f"{self.__class__.__name__}(output_size={self.output_size}, "
                f"spatial_scale={self.spatial_scale}, sampling_ratio={self.sampling_ratio}, "
                f"aligned={self.aligned})")
