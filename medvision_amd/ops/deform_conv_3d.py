"""DCNv1 in 3-D: ``DeformConv3dFunction``, ``DeformConv3d``, ``DeformConv3dPack``.

Interface and parameter names of the reference's ``medvision/ops/deform_conv_3d.py`` (function
:17-74, module :77-146, pack :149-191), so state dicts are interchangeable.  As there, the
``bias`` parameter always exists and is always added; ``bias=False`` only freezes it.
"""
import math

import torch
from torch import nn
from torch.autograd import Function
from torch.autograd.function import once_differentiable
from torch.nn import init
from torch.nn.modules.utils import _triple

from .. import _C


class DeformConv3dFunction(Function):
    @staticmethod
    def forward(ctx, input, offset, weight, bias, stride, padding, dilation, group,
                deformable_groups, im2col_step):
        ctx.stride, ctx.padding, ctx.dilation = _triple(stride), _triple(padding), _triple(dilation)
        ctx.kernel_size = tuple(weight.shape[2:5])
        ctx.group, ctx.deformable_groups, ctx.im2col_step = group, deformable_groups, im2col_step
        if offset.dtype in (torch.float16, torch.bfloat16):   # autocast: follow the offset branch
            input, bias, weight = input.to(offset.dtype), bias.to(offset.dtype), weight.to(offset.dtype)
        output = _C.deform_conv_3d_forward(input, weight, bias, offset, *ctx.kernel_size,
                                           *ctx.stride, *ctx.padding, *ctx.dilation, group,
                                           deformable_groups, im2col_step)
        ctx.save_for_backward(input, offset, weight, bias)
        return output

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        input, offset, weight, bias = ctx.saved_tensors
        grad_input, grad_offset, grad_weight, grad_bias = _C.deform_conv_3d_backward(
            input, weight, bias, offset, grad_output, *ctx.kernel_size, *ctx.stride, *ctx.padding,
            *ctx.dilation, ctx.group, ctx.deformable_groups, ctx.im2col_step)
        return grad_input, grad_offset, grad_weight, grad_bias, None, None, None, None, None, None


deform_conv = DeformConv3dFunction.apply


class DeformConv3d(nn.Module):

    def __init__(self, in_channels, out_channels, kernel_size, stride, padding, dilation=1,
                 groups=1, deformable_groups=1, im2col_step=64, bias=True):
        super().__init__()
        if in_channels % groups != 0:
            raise ValueError('in_channels {} must be divisible by groups {}'.format(in_channels, groups))
        if out_channels % groups != 0:
            raise ValueError('out_channels {} must be divisible by groups {}'.format(out_channels, groups))
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size = _triple(kernel_size)
        self.stride, self.padding, self.dilation = _triple(stride), _triple(padding), _triple(dilation)
        self.groups, self.deformable_groups = groups, deformable_groups
        self.im2col_step = im2col_step
        self.use_bias = bias
        self.weight = nn.Parameter(torch.Tensor(out_channels, in_channels // groups, *self.kernel_size))
        self.bias = nn.Parameter(torch.Tensor(out_channels))
        self.reset_parameters()
        if not self.use_bias:
            self.bias.requires_grad = False

    def reset_parameters(self):
        init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        fan_in, _ = init._calculate_fan_in_and_fan_out(self.weight)
        bound = 1 / math.sqrt(fan_in)
        init.uniform_(self.bias, -bound, bound)

    def forward(self, input, offset):
        k = self.kernel_size
        assert 3 * self.deformable_groups * k[0] * k[1] * k[2] == offset.shape[1]
        return deform_conv(input, offset, self.weight, self.bias, self.stride, self.padding,
                           self.dilation, self.groups, self.deformable_groups, self.im2col_step)

    def __repr__(self):
        return (f'{self.__class__.__name__}(in_channels={self.in_channels}, '
                f'out_channels={self.out_channels}, kernel_size={self.kernel_size}, '
                f'stride={self.stride}, padding={self.padding}, dilation={self.dilation}, '
                f'groups={self.groups}, deformable_groups={self.deformable_groups})')


class DeformConv3dPack(DeformConv3d):
    """DeformConv3d that predicts its own offsets with a zero-initialised ``conv_offset``."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, deformable_groups=1, im2col_step=64, bias=True, lr_mult=0.1):
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, groups,
                         deformable_groups, im2col_step, bias)
        k = self.kernel_size
        self.conv_offset = nn.Conv3d(self.in_channels, self.deformable_groups * 3 * k[0] * k[1] * k[2],
                                     kernel_size=self.kernel_size, stride=self.stride,
                                     padding=self.padding, bias=True)
        self.conv_offset.lr_mult = lr_mult
        self.init_offset()

    def init_offset(self):
        self.conv_offset.weight.data.zero_()
        self.conv_offset.bias.data.zero_()

    def forward(self, input):
        offset = self.conv_offset(input)
        return deform_conv(input, offset, self.weight, self.bias, self.stride, self.padding,
                           self.dilation, self.groups, self.deformable_groups, self.im2col_step)
