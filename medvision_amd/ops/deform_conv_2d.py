"""DCNv1 in 2-D: ``DeformConv2dFunction``, ``DeformConv2d``, ``DeformConv2dPack``.

Interface and parameter names of the reference's ``medvision/ops/deform_conv_2d.py`` (function
:13-70, module :73-142, pack :145-186), so state dicts are interchangeable.  The ``bias``
parameter always exists and is always added; ``bias=False`` only freezes it.  Offsets carry two
channels per kernel tap: 2k = row, 2k+1 = column displacement.
"""
import math

import torch
from torch import nn
from torch.autograd import Function
from torch.autograd.function import once_differentiable
from torch.nn import init
from torch.nn.modules.utils import _pair

from .. import _C


class DeformConv2dFunction(Function):
    @staticmethod
    def forward(ctx, input, offset, weight, bias, stride, padding, dilation, group,
                deformable_groups, im2col_step):
        ctx.geometry = (*weight.shape[2:4], *_pair(stride), *_pair(padding), *_pair(dilation),
                        group, deformable_groups, im2col_step)
        if offset.dtype in (torch.float16, torch.bfloat16):   # autocast: follow the offset branch
            input, bias, weight = input.to(offset.dtype), bias.to(offset.dtype), weight.to(offset.dtype)
        output = _C.deform_conv_2d_forward(input, weight, bias, offset, *ctx.geometry)
        ctx.save_for_backward(input, offset, weight, bias)
        return output

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        input, offset, weight, bias = ctx.saved_tensors
        grads = _C.deform_conv_2d_backward(input, weight, bias, offset, grad_output, *ctx.geometry)
        return (*grads, None, None, None, None, None, None)


deform_conv = DeformConv2dFunction.apply


class DeformConv2d(nn.Module):

    def __init__(self, in_channels, out_channels, kernel_size, stride, padding, dilation=1,
                 groups=1, deformable_groups=1, im2col_step=64, bias=True):
        super().__init__()
        if in_channels % groups != 0:
            raise ValueError('in_channels {} must be divisible by groups {}'.format(in_channels, groups))
        if out_channels % groups != 0:
            raise ValueError('out_channels {} must be divisible by groups {}'.format(out_channels, groups))
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size = _pair(kernel_size)
        self.stride, self.padding, self.dilation = _pair(stride), _pair(padding), _pair(dilation)
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
        init.uniform_(self.bias, -1 / math.sqrt(fan_in), 1 / math.sqrt(fan_in))

    def forward(self, input, offset):
        assert 2 * self.deformable_groups * self.kernel_size[0] * self.kernel_size[1] == offset.shape[1]
        return deform_conv(input, offset, self.weight, self.bias, self.stride, self.padding,
                           self.dilation, self.groups, self.deformable_groups, self.im2col_step)

    def __repr__(self):
        return (f'{self.__class__.__name__}(in_channels={self.in_channels}, '
                f'out_channels={self.out_channels}, kernel_size={self.kernel_size}, '
                f'stride={self.stride}, padding={self.padding}, dilation={self.dilation}, '
                f'groups={self.groups}, deformable_groups={self.deformable_groups})')


class DeformConv2dPack(DeformConv2d):
    """DeformConv2d that predicts its own offsets with a zero-initialised ``conv_offset``."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, deformable_groups=1, im2col_step=64, bias=True, lr_mult=0.1):
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, groups,
                         deformable_groups, im2col_step, bias)
        taps = self.kernel_size[0] * self.kernel_size[1]
        self.conv_offset = nn.Conv2d(self.in_channels, self.deformable_groups * 2 * taps,
                                     kernel_size=self.kernel_size, stride=self.stride,
                                     padding=self.padding, bias=True)
        self.conv_offset.lr_mult = lr_mult
        self.init_offset()

    def init_offset(self):
        self.conv_offset.weight.data.zero_()
        self.conv_offset.bias.data.zero_()

    def forward(self, input):
        return deform_conv(input, self.conv_offset(input), self.weight, self.bias, self.stride,
                           self.padding, self.dilation, self.groups, self.deformable_groups,
                           self.im2col_step)
