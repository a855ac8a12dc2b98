"""Functional resampling engines used by the augmentation layer.

Interface of the reference's ``medvision/ops/cuda_fun_tools.py``: ``affine_2d`` / ``affine_3d``
(:6-92) resample with rotated rois (Resize, RandomAffine, Crop); ``apply_offset_2d`` /
``apply_offset_3d`` (:94-167) warp an image by a dense displacement field
(RandomElasticDeformation).  Orders: 0 nearest, 1 linear, 3 cubic (Catmull-Rom).
"""
import torch

from .. import _C
from .roi_align_nd import _parse_output_size


def _affine(ndim, features, rois, out_size, spatial_scale, sampling_ratio, aligned, order):
    out = _parse_output_size(out_size, ndim)
    # (int32: label maps at order 0, sampled as they are -- the reference resamples a float copy of them)
    assert features.dtype in [torch.float32, torch.float16, torch.bfloat16, torch.float64] or \
        (features.dtype == torch.int32 and order == 0), f'input must be a floating tensor but got {features.dtype}'
    assert order in [0, 1, 3], f'order {order} is not supported!'
    if order == 0:
        sampling_ratio = 1  # never average nearest-neighbour samples (reference :72-74)
    # every output element is written by the kernel (zeros where a sample is void): no zero fill
    output = features.new_empty(rois.size(0), features.size(1), *out)
    fn = _C.affine_2d if ndim == 2 else _C.affine_3d
    fn(features, rois, output, *out, spatial_scale, sampling_ratio, aligned, order)
    return output


def affine_2d(features, rois, out_size, spatial_scale, sampling_ratio=0, aligned=True, order=1):
    """features [B,C,H,W], rois [n,6] = (b, cx, cy, w, h, angle) -> [n,C,*out_size]."""
    return _affine(2, features, rois, out_size, spatial_scale, sampling_ratio, aligned, order)


def affine_3d(features, rois, out_size, spatial_scale, sampling_ratio=0, aligned=True, order=1):
    """features [B,C,D,H,W], rois [n,10] = (b, cx, cy, cz, w, h, d, ax, ay, az) -> [n,C,*out_size]."""
    return _affine(3, features, rois, out_size, spatial_scale, sampling_ratio, aligned, order)


def apply_offset_2d(img, offset, order=1):
    """img [B,C,H,W], offset [B,2,H,W] (channel 0 = rows, 1 = columns): out(q) = img(q + offset(q))."""
    assert img.shape[2:] == offset.shape[2:]
    assert offset.shape[1] == 2
    output = _C.deform_warp(img, offset, order)
    assert img.shape == output.shape
    return output


def apply_offset_3d(img, offset, order=1):
    """img [B,C,D,H,W], offset [B,3,D,H,W] (channels depth, height, width)."""
    assert img.shape[2:] == offset.shape[2:]
    assert offset.shape[1] == 3
    output = _C.deform_warp(img, offset, order)
    assert img.shape == output.shape, f"input is {img.shape}, out is {output.shape}"
    return output
