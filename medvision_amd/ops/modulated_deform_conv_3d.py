"""DCNv2 (modulated) in 3-D: ``ModulatedDeformConv3dFunction``, ``ModulatedDeformConv3d``,
``ModulatedDeformConv3dPack``.

Interface and parameter names of the reference's ``medvision/ops/modulated_deform_conv_3d.py``
(function :17-97, module :104-160, pack :163-189): scalar stride / padding / dilation applied to
all three axes, optional bias, offsets+mask predicted by ``conv_offset_mask`` in the pack.
The backward returns the analytic gradients (the reference's 3-D v2 backward is defective, see
``medvision_amd/_C.py``).
"""
import math

import torch
from torch import nn
from torch.autograd import Function
from torch.autograd.function import once_differentiable
from torch.nn.modules.utils import _triple

from .. import _C


class ModulatedDeformConv3dFunction(Function):
    @staticmethod
    def forward(ctx, input, offset, mask, weight, bias=None, stride=1, padding=0, dilation=1,
                groups=1, deformable_groups=1):
        ctx.stride, ctx.padding, ctx.dilation = stride, padding, dilation
        ctx.groups, ctx.deformable_groups = groups, deformable_groups
        ctx.with_bias = bias is not None
        if not ctx.with_bias:
            bias = input.new_empty(1)  # placeholder so that five tensors are always saved
        if not input.is_cuda:
            raise NotImplementedError
        if offset.dtype in (torch.float16, torch.bfloat16):   # autocast: follow the offset branch
            input, bias, weight = input.to(offset.dtype), bias.to(offset.dtype), weight.to(offset.dtype)
        output = offset.new_empty(ModulatedDeformConv3dFunction._infer_shape(ctx, input, weight),
                                  dtype=input.dtype)
        k = weight.shape[2:5]
        _C.modulated_deform_conv_3d_forward(
            input, weight, bias, None, offset, mask, output, None, k[0], k[1], k[2],
            stride, stride, stride, padding, padding, padding, dilation, dilation, dilation,
            groups, deformable_groups, ctx.with_bias)
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
        k = weight.shape[2:5]
        s, p, d = ctx.stride, ctx.padding, ctx.dilation
        _C.modulated_deform_conv_3d_backward(
            input, weight, bias, None, offset, mask, None, grad_input, grad_weight, grad_bias,
            grad_offset, grad_mask, grad_output, k[0], k[1], k[2], s, s, s, p, p, p, d, d, d,
            ctx.groups, ctx.deformable_groups, ctx.with_bias)
        if not ctx.with_bias:
            grad_bias = None
        return (grad_input, grad_offset.to(offset.dtype), grad_mask.to(mask.dtype), grad_weight,
                grad_bias, None, None, None, None, None)

    @staticmethod
    def _infer_shape(ctx, input, weight):
        n, channels_out = input.size(0), weight.size(0)
        spatial = [(size + 2 * ctx.padding - (ctx.dilation * (k - 1) + 1)) // ctx.stride + 1
                   for size, k in zip(input.shape[2:5], weight.shape[2:5])]
        return (n, channels_out, *spatial)


modulated_deform_conv = ModulatedDeformConv3dFunction.apply


class ModulatedDeformConv3d(nn.Module):

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, deformable_groups=1, bias=True):
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size = _triple(kernel_size)
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
        n = self.in_channels * self.kernel_size[0] * self.kernel_size[1] * self.kernel_size[2]
        stdv = 1. / math.sqrt(n)
        self.weight.data.uniform_(-stdv, stdv)
        if self.bias is not None:
            self.bias.data.zero_()

    def forward(self, x, offset, mask):
        return modulated_deform_conv(x, offset, mask, self.weight, self.bias, self.stride,
                                     self.padding, self.dilation, self.groups, self.deformable_groups)

    def __repr__(self):
        return (f'{self.__class__.__name__}(in_channels={self.in_channels}, '
                f'out_channels={self.out_channels}, kernel_size={self.kernel_size}, '
                f'stride={_triple(self.stride)}, padding={_triple(self.padding)}, '
                f'dilation={_triple(self.dilation)}, groups={self.groups}, '
                f'deform_groups={self.deformable_groups})')


class ModulatedDeformConv3dPack(ModulatedDeformConv3d):
    """ModulatedDeformConv3d that predicts offsets and masks with a zero-initialised conv
    (``4 * K * deformable_groups`` channels: three offset thirds followed by the mask logits)."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        k = self.kernel_size
        self.conv_offset_mask = nn.Conv3d(self.in_channels,
                                          self.deformable_groups * 4 * k[0] * k[1] * k[2],
                                          kernel_size=self.kernel_size, stride=_triple(self.stride),
                                          padding=_triple(self.padding), bias=True)
        self.init_offset()

    def init_offset(self):
        self.conv_offset_mask.weight.data.zero_()
        self.conv_offset_mask.bias.data.zero_()

    def forward(self, x):
        out = self.conv_offset_mask(x)
        o1, o2, o3, mask = torch.chunk(out, 4, dim=1)
        offset = torch.cat((o1, o2, o3), dim=1)
        mask = torch.sigmoid(mask)
        return modulated_deform_conv(x, offset, mask, self.weight, self.bias, self.stride,
                                     self.padding, self.dilation, self.groups, self.deformable_groups)
