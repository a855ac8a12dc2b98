"""DCNv2 (modulated) in 2-D: ``ModulatedDeformConv2dFunction``, ``ModulatedDeformConv2d``,
``ModulatedDeformConv2dPack``.

Interface and parameter names of the reference's ``medvision/ops/modulated_deform_conv_2d.py``
(function :12-93, module :99-157, pack :160-186): scalar stride / padding / dilation applied to
both axes, optional bias, offsets + mask predicted by ``conv_offset_mask`` in the pack (two offset
thirds, then the mask logits).
"""
import math

import torch
from torch import nn
from torch.autograd import Function
from torch.autograd.function import once_differentiable
from torch.nn.modules.utils import _pair

from .. import _C


class ModulatedDeformConv2dFunction(Function):
    @staticmethod
    def forward(ctx, input, offset, mask, weight, bias=None, stride=1, padding=0, dilation=1,
                groups=1, deformable_groups=1):
        ctx.with_bias = bias is not None
        if not ctx.with_bias:
            bias = input.new_empty(1)  # placeholder so that five tensors are always saved
        if not input.is_cuda:
            raise NotImplementedError
        if offset.dtype in (torch.float16, torch.bfloat16):   # autocast: follow the offset branch
            input, bias, weight = input.to(offset.dtype), bias.to(offset.dtype), weight.to(offset.dtype)
        ctx.geometry = (*weight.shape[2:4], stride, stride, padding, padding, dilation, dilation,
                        groups, deformable_groups, ctx.with_bias)
        spatial = [(size + 2 * padding - (dilation * (k - 1) + 1)) // stride + 1
                   for size, k in zip(input.shape[2:4], weight.shape[2:4])]
        output = input.new_empty((input.size(0), weight.size(0), *spatial))
        _C.modulated_deform_conv_2d_forward(input, weight, bias, None, offset, mask, output, None,
                                            *ctx.geometry)
        ctx.save_for_backward(input, offset, mask, weight, bias)
        return output

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        if not grad_output.is_cuda:
            raise NotImplementedError
        input, offset, mask, weight, bias = ctx.saved_tensors
        grad_input = torch.zeros_like(input)
        grad_offset = torch.zeros_like(offset, dtype=input.dtype)
        grad_mask = torch.zeros_like(mask, dtype=input.dtype)
        grad_weight = torch.zeros_like(weight)
        grad_bias = torch.zeros_like(bias)
        _C.modulated_deform_conv_2d_backward(input, weight, bias, None, offset, mask, None,
                                             grad_input, grad_weight, grad_bias, grad_offset,
                                             grad_mask, grad_output, *ctx.geometry)
        return (grad_input, grad_offset.to(offset.dtype), grad_mask.to(mask.dtype), grad_weight,
                grad_bias if ctx.with_bias else None, None, None, None, None, None)


modulated_deform_conv = ModulatedDeformConv2dFunction.apply


class ModulatedDeformConv2d(nn.Module):

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, deformable_groups=1, bias=True):
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size = _pair(kernel_size)
        self.stride, self.padding, self.dilation = stride, padding, dilation
        self.groups, self.deformable_groups = groups, deformable_groups
        self.with_bias = bias
        self.weight = nn.Parameter(torch.Tensor(out_channels, in_channels // groups, *self.kernel_size))
        if bias:
            self.bias = nn.Parameter(torch.Tensor(out_channels))
        else:
            self.register_parameter('bias', None)
        self.reset_parameters()

    def reset_parameters(self):
        stdv = 1. / math.sqrt(self.in_channels * self.kernel_size[0] * self.kernel_size[1])
        self.weight.data.uniform_(-stdv, stdv)
        if self.bias is not None:
            self.bias.data.zero_()

    def forward(self, x, offset, mask):
        return modulated_deform_conv(x, offset, mask, self.weight, self.bias, self.stride,
                                     self.padding, self.dilation, self.groups, self.deformable_groups)

    def __repr__(self):
        return (f'{self.__class__.__name__}(in_channels={self.in_channels}, '
                f'out_channels={self.out_channels}, kernel_size={self.kernel_size}, '
                f'stride={_pair(self.stride)}, padding={_pair(self.padding)}, '
                f'dilation={_pair(self.dilation)}, groups={self.groups}, '
                f'deform_groups={self.deformable_groups})')


class ModulatedDeformConv2dPack(ModulatedDeformConv2d):
    """ModulatedDeformConv2d that predicts offsets and masks with a zero-initialised conv
    (``3 * K * deformable_groups`` channels)."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        taps = self.kernel_size[0] * self.kernel_size[1]
        self.conv_offset_mask = nn.Conv2d(self.in_channels, self.deformable_groups * 3 * taps,
                                          kernel_size=self.kernel_size, stride=_pair(self.stride),
                                          padding=_pair(self.padding), bias=True)
        self.init_offset()

    def init_offset(self):
        self.conv_offset_mask.weight.data.zero_()
        self.conv_offset_mask.bias.data.zero_()

    def forward(self, x):
        o1, o2, mask = torch.chunk(self.conv_offset_mask(x), 3, dim=1)
        return modulated_deform_conv(x, torch.cat((o1, o2), dim=1), torch.sigmoid(mask), self.weight,
                                     self.bias, self.stride, self.padding, self.dilation,
                                     self.groups, self.deformable_groups)
