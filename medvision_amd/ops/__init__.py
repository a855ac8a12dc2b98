"""Operator classes with the names and signatures of the reference's ``medvision.ops``
(``medvision/ops/__init__.py:1-24``), restricted to the trilinear-sampling family."""
from .roi_align_nd import PreparedFeatures, RoIAlign
from .roi_align_rotated_nd import RoIAlignRotated
from .deform_conv_2d import DeformConv2d, DeformConv2dPack
from .modulated_deform_conv_2d import ModulatedDeformConv2d, ModulatedDeformConv2dPack
from .deform_conv_3d import DeformConv3d, DeformConv3dPack
from .modulated_deform_conv_3d import ModulatedDeformConv3d, ModulatedDeformConv3dPack
from .cuda_fun_tools import affine_2d, affine_3d, apply_offset_2d, apply_offset_3d

__all__ = [
    'RoIAlign',
    'PreparedFeatures',
    'RoIAlignRotated',
    'DeformConv2d',
    'DeformConv2dPack',
    'ModulatedDeformConv2d',
    'ModulatedDeformConv2dPack',
    'DeformConv3d',
    'DeformConv3dPack',
    'ModulatedDeformConv3d',
    'ModulatedDeformConv3dPack',
    'affine_2d', 'affine_3d', 'apply_offset_2d', 'apply_offset_3d',
]
