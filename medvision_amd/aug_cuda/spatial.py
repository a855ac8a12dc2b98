"""Spatial GPU augmentations on top of the affine resampling engine and the displacement warp.

Classes, constructor arguments, result-dict keys and random draws follow the reference's
``medvision/aug_cuda/aug_spatial.py`` (Resize :20-152, RandomAffine :240-482, elastic :485-706,
CropRandomWithAffine :967-1228) and, for the ``Batch*`` classes, ``medvision/aug_cuda_batch/
aug_spatial.py`` (:69-202, :356-597, :600-850).  Every image stage boils down to ONE call of
``affine_2d`` / ``affine_3d`` with one rotated roi per sample (built in ``geometry.py``);
segmentations go through the same rois at order 0 as float and come back as int32.
"""
import itertools
import random
import math
import warnings

import numpy as np
import torch

from ..ops.cuda_fun_tools import affine_2d, affine_3d, apply_offset_2d, apply_offset_3d
from . import geometry
from .base import BatchCudaAugBase, CudaAugBase


class _Resampler:
    """Shared image / segmentation path: subclasses give the rois and the output size."""

    sampling_ratio = 1
    order = 1

    def _rois(self):
        raise NotImplementedError

    def _out_size(self):
        raise NotImplementedError

    def _skip(self):
        return False

    def _resample(self, tensor, order, sampling_ratio):
        assert tensor.is_cuda, 'image should be cuda'
        lead = 2 if self.batched else 1
        assert tensor.ndim == self.dim + lead, 'image should be [batch,] channel, **dim'
        fn = affine_2d if self.dim == 2 else affine_3d
        rois = getattr(self, '_device_rois', None)
        if rois is None or rois.device != tensor.device:
            rois = self._device_rois = torch.from_numpy(self._rois()).to(tensor.device)
        batch = tensor if self.batched else tensor.unsqueeze(0)
        out = fn(batch, rois, tuple(int(v) for v in self._out_size()), 1.0, sampling_ratio, True, order)
        return out if self.batched else out.squeeze(0)

    def _labels(self, seg, sampling_ratio):
        """Order 0 on a label map.  The reference resamples a float copy and converts back
        (aug_cuda/aug_spatial.py: ``.float()`` ... ``.int()``); int32 maps go to the library as they are,
        which picks the same voxels and saves the two conversion passes."""
        if seg.dtype == torch.int32:
            return self._resample(seg, 0, sampling_ratio)
        return self._resample(seg.float(), 0, sampling_ratio).int()

    def apply_to_img(self, result):
        for key in result.get('img_fields', []):
            if not self._skip():
                result[key] = self._resample(result[key], self.order, self.sampling_ratio)
            self._after_img(result, key)

    def apply_to_seg(self, result):
        for key in result.get('seg_fields', []):
            if not self._skip():
                result[key] = self._labels(result[key], self.sampling_ratio)

    def _after_img(self, result, key):
        if key == 'img' and not self.batched:
            result['img_shape'] = tuple(result[key].shape)


# ---- resize ------------------------------------------------------------------------------------
class CudaResize(_Resampler, CudaAugBase):
    """Resize to a spacing, a shape or by factors (exactly one of the three; -1 keeps an axis)."""

    def __init__(self, spacing=None, scale=None, factor=None, order=1):
        super().__init__()
        self.always = True
        self.spacing, self.scale, self.factor, self.order = spacing, scale, factor, order
        assert sum(v is not None for v in (spacing, scale, factor)) == 1

    def __repr__(self):
        return f'{self.__class__.__name__}(spacing={self.spacing}, scale={self.scale}, factor={self.factor})'

    @property
    def canBackward(self):
        return True

    def _forward_params(self, result):
        self._init_params(result)
        given = self.spacing if self.spacing is not None else self.scale if self.scale is not None else self.factor
        assert len(given) == self.dim, f"not match with a {result['img_dim']}D image"
        if self.spacing is not None:
            have = np.array(result['img_spacing'])
            want = np.array(self.spacing)
            factors = have / np.where(want == -1, have, want)
        elif self.scale is not None:
            want = np.array(self.scale)
            factors = np.where(want == -1, self.image_shape, want) / self.image_shape
        else:
            factors = self.factor
        self.params = tuple(factors)
        result[self.key_name] = self.params

    def _backward_params(self, result):
        self._init_params(result)
        params = result.pop(self.key_name, None)
        if params:
            self.params = tuple(1 / np.array(params))

    def _skip(self):
        return all(f == 1.0 for f in self.params)

    def _rois(self):
        return geometry.frame_rois(self.image_shape, self.batch)

    def _out_size(self):
        return [int(s * f) for s, f in zip(self.image_shape, self.params)]

    def _after_img(self, result, key):
        if key == 'img' and not self.batched:
            result['img_shape'] = tuple(result[key].shape)
            result['img_spacing'] = tuple(np.array(result['img_spacing']) / np.array(self.params))

    def apply_to_seg(self, result):   # always a sampling grid of one (nearest)
        for key in result.get('seg_fields', []):
            if not self._skip():
                result[key] = self._labels(result[key], 1)

    def apply_to_img(self, result):
        for key in result.get('img_fields', []):
            if not self._skip():
                result[key] = self._resample(result[key], self.order, 1)
            self._after_img(result, key)

    def apply_to_det(self, result):
        for key in result.get('det_fields', []):
            if self.batched:
                raise NotImplementedError
            if not self._skip():
                factors = torch.from_numpy(np.hstack(self.params[::-1] * 2)).to(result[key].device)
                result[key][:, :2 * self.dim] = result[key][:, :2 * self.dim] * factors


class BatchCudaResize(CudaResize, BatchCudaAugBase):
    pass


# ---- scale / shift / rotate ----------------------------------------------------------------------
class CudaRandomAffine(_Resampler, CudaAugBase):
    """One isotropic scale 1 + U(scale), per-axis shifts U(shift) (fractions of the image) and a
    rotation U(rotate) degrees in the xy plane (counter-clockwise for positive angles)."""

    def __init__(self, p, scale, shift, rotate, sampling_ratio=1, order=1):
        super().__init__()
        self.p, self.scale, self.shift, self.rotate = p, scale, shift, rotate
        self.sampling_ratio, self.order = sampling_ratio, order

    def __repr__(self):
        return (f'{self.__class__.__name__}(dim={self.dim}, scale={self.scale}, shift={self.shift}, '
                f'rotate={self.rotate})')

    def _draw(self):
        scales = [self.get_range(self.scale, 1)] * self.dim
        shifts = [self.get_range(self.shift, 0) for _ in range(self.dim)]
        rotate = [math.pi * self.get_range(self.rotate, 0) / 180]
        return scales, shifts, rotate

    def _forward_params(self, result):
        self._init_params(result)
        if self.batched:
            draws = [self._draw() for _ in range(self.batch)]
            self.params = {k: np.array([d[i] for d in draws]) for i, k in enumerate(("scales", "shifts", "rotate"))}
        else:
            scales, shifts, rotate = self._draw()
            self.params = {"_scales": scales, "_shifts": shifts, "_rotate": rotate}
        result[self.key_name] = self.params

    def _affine(self):
        p = self.params
        return (p["scales"], p["shifts"], p["rotate"]) if self.batched else (p["_scales"], p["_shifts"], p["_rotate"])

    def _window(self):
        """(start, end) of the resampled window in (x, y, z) order: the whole image."""
        return [0.0] * self.dim, [float(s) for s in self.image_shape[::-1]]

    def _rois(self):
        start, end = self._window()
        return geometry.window_rois(self.dim, start, end, *self._affine(), index=np.arange(self.batch))

    def _out_size(self):
        return self.image_shape

    def apply_to_det(self, result):
        for key in result.get('det_fields', []):
            if self.batched:
                raise NotImplementedError
            boxes = result[key].cpu().numpy()
            scales, shifts, rotate = self._affine()
            out_xyz = list(self._out_size())[::-1]
            start, _ = self._window()
            moved = geometry.map_boxes(self.dim, boxes, out_xyz, scales, shifts, rotate, start)
            kept = geometry.clip_boxes(moved, result['img'].shape[1:])
            result[key] = torch.from_numpy(kept).to(result[key].device)


class CudaRandomScale(CudaRandomAffine):
    def __init__(self, p, scale, sampling_ratio=1):
        super().__init__(p, scale=scale, shift=0, rotate=0, sampling_ratio=sampling_ratio)


class CudaRandomShift(CudaRandomAffine):
    def __init__(self, p, shift, sampling_ratio=1):
        super().__init__(p, scale=0, shift=shift, rotate=0, sampling_ratio=sampling_ratio)


class CudaRandomRotate(CudaRandomAffine):
    def __init__(self, p, rotate, sampling_ratio=1):
        super().__init__(p, scale=0, shift=0, rotate=rotate, sampling_ratio=sampling_ratio)


class BatchCudaRandomAffine(CudaRandomAffine, BatchCudaAugBase):
    pass


class BatchCudaRandomScale(CudaRandomScale, BatchCudaAugBase):
    pass


class BatchCudaRandomShift(CudaRandomShift, BatchCudaAugBase):
    pass


class BatchCudaRandomRotate(CudaRandomRotate, BatchCudaAugBase):
    pass


# ---- crop with affine ------------------------------------------------------------------------------
class CudaCropRandomWithAffine(CudaRandomAffine):
    """A random ``patch_size`` window, resampled with a random scale / shift / rotation in one
    pass; ``times`` patches per input when called on a list or with times > 1."""

    def __init__(self, patch_size, scale, shift, rotate, sampling_ratio=1, order=1, times=1):
        super().__init__(0., scale, shift, rotate, sampling_ratio, order)
        self.always = True
        self.dim = len(patch_size)
        self.patch_size = patch_size
        self.times = times

    def __repr__(self):
        return f'{self.__class__.__name__}(patch_size={self.patch_size})'

    @property
    def repeats(self):
        return self.times

    def _crop_start(self, result, sample):
        """First voxel of the window in (z, y, x) order."""
        return tuple(np.random.randint(0, size - patch + 1)
                     for size, patch in zip(self.image_shape, self.patch_size))

    def _forward_params(self, result):
        self._init_params(result)
        assert self.dim == len(self.patch_size)
        assert all(s >= p for s, p in zip(self.image_shape, self.patch_size)), self.image_shape
        if self.batched:
            starts = [self._crop_start(result, i) for i in range(self.batch)]
            draws = [self._draw() for _ in range(self.batch)]
            self.params = {"start": np.array([s[::-1] for s in starts]),
                           "end": np.array([tuple(a + b for a, b in zip(s, self.patch_size))[::-1] for s in starts]),
                           "scales": np.array([d[0] for d in draws]),
                           "shifts": np.array([d[1] for d in draws]),
                           "rotate": np.array([d[2] for d in draws])}
        else:
            start = self._crop_start(result, 0)
            end = tuple(a + b for a, b in zip(start, self.patch_size))
            scales, shifts, rotate = self._draw()
            self.params = {"start": start[::-1], "end": end[::-1],   # x, y, z
                           "_scales": scales, "_shifts": shifts, "_rotate": rotate}
        result[self.key_name] = self.params

    def _window(self):
        return self.params["start"], self.params["end"]

    def _out_size(self):
        return self.patch_size


class CudaCropCenterWithAffine(CudaCropRandomWithAffine):
    def _crop_start(self, result, sample):
        return tuple(size // 2 - patch // 2 for size, patch in zip(self.image_shape, self.patch_size))


class CudaCropFirstDetWithAffine(CudaCropRandomWithAffine):
    """Window placed so that the first ground-truth box (plus ``border``) lies inside it."""

    def __init__(self, border=12, *args, **kwargs):
        self.border = border
        super().__init__(*args, **kwargs)

    def _start_around(self, lo_zyx, hi_zyx):
        """A window start (z, y, x) drawn so that [lo, hi) widened by ``border`` lies inside the window
        where the patch and the volume allow it."""
        start = []
        for axis in range(self.dim):
            room = self.image_shape[axis] - self.patch_size[axis]
            first = min(max(hi_zyx[axis] + self.border - self.patch_size[axis], 0), room)
            last = min(max(lo_zyx[axis] - self.border, 0), room)
            start.append(np.random.randint(min(first, last), max(first, last) + 1))
        return tuple(start)

    def _start_around_box(self, box):
        """``box`` = (x1, y1[, z1], x2, y2[, z2], ...) as the detection fields store it."""
        box = box.cpu().numpy() if torch.is_tensor(box) else np.asarray(box)
        return self._start_around([box[self.dim - axis - 1] for axis in range(self.dim)],
                                  [box[2 * self.dim - axis - 1] for axis in range(self.dim)])

    def _crop_start(self, result, sample):
        assert 'gt_det' in result, "it only used for detection tasks"
        if len(result['gt_det']) == 0:
            return super()._crop_start(result, sample)
        return self._start_around_box(result['gt_det'][0])


class BatchCudaCropRandomWithAffine(CudaCropRandomWithAffine, BatchCudaAugBase):
    pass


class BatchCudaCropCenterWithAffine(CudaCropCenterWithAffine, BatchCudaAugBase):
    pass


class BatchCudaCropFirstDetWithAffine(CudaCropFirstDetWithAffine, BatchCudaAugBase):
    """aug_cuda_batch/aug_spatial.py:928-960: every sample's window is drawn around the first box."""

    def __init__(self, border=12, **kwargs):
        super().__init__(border, **kwargs)

    def _crop_start(self, result, sample):
        assert 'gt_det' in result, "it only used for detection tasks"
        return self._start_around_box(result['gt_det'][0])


class BatchCudaCropDetWithAffine(BatchCudaCropFirstDetWithAffine):
    """aug_cuda_batch/aug_spatial.py:893-925: the boxes take turns, one per drawn window."""

    def __init__(self, border=12, **kwargs):
        super().__init__(border, **kwargs)
        self.current_repeat_idx = 0

    def _crop_start(self, result, sample):
        assert 'gt_det' in result, "it only used for detection tasks"
        pick = min(self.current_repeat_idx % self.repeats, len(result['gt_det']) - 1)
        self.current_repeat_idx += 1
        return self._start_around_box(result['gt_det'][pick])


class BatchCudaCropForegroundWithAffine(BatchCudaCropFirstDetWithAffine):
    """aug_cuda_batch/aug_spatial.py:852-890: the window is drawn around one connected component of the
    sample's label map (``gt_seg``, else ``pseudo_mask``), anywhere when the map is empty."""

    def _crop_start(self, result, sample):
        from scipy import ndimage as ndi
        assert 'gt_seg' in result or 'pseudo_mask' in result
        mask = result['gt_seg' if 'gt_seg' in result else 'pseudo_mask'][sample, 0]
        objs = ndi.find_objects(ndi.label(mask.cpu().numpy())[0])
        if not objs:
            return CudaCropRandomWithAffine._crop_start(self, result, sample)
        obj = random.choice(objs)
        return self._start_around([o.start for o in obj], [o.stop for o in obj])


# ---- elastic deformation ---------------------------------------------------------------------------
class CudaRandomElasticDeformation(CudaAugBase):
    """Random displacements on a coarse control grid (two locked border layers), upsampled to a
    dense field with the order-3 affine engine and applied with the displacement-field warp."""

    def __init__(self, p, num_control_points=8, max_displacement=0.8, order=3):
        super().__init__()
        self.p = p
        self.num_control_points = num_control_points   # z, y, x
        self.max_displacement = max_displacement       # fraction of half a grid cell
        self.INTER_ORDER = order                       # of the control grid's upsampling
        self.num_locked_borders = 2
        assert max_displacement <= 1.0
        self.tmp_params = None

    def __repr__(self):
        return (f'{self.__class__.__name__}(p={self.p}, num_control_points={self.num_control_points}, '
                f'max_displacement={self.max_displacement})')

    @property
    def canBackward(self):
        return True

    def _forward_params(self, result):
        self.tmp_params = None
        self._init_params(result)
        grid = self.to_tuple(self.num_control_points, self.dim)
        cell = np.array(self.image_shape) / (np.array(grid) - 1)
        inner = tuple(slice(self.num_locked_borders, n - self.num_locked_borders) for n in grid)
        fields = []
        for _ in range(self.batch):      # one draw per sample, in sample order
            coarse = 2 * np.random.rand(*grid, self.dim).astype(np.float32) - 1
            coarse *= self.max_displacement * cell / 2          # per component (z, y, x)
            locked = np.zeros_like(coarse)
            locked[inner] = coarse[inner]
            fields.append(locked)
        # per-sample stage: [*grid, dim]; batch stage: [batch, *grid, dim]
        self.params = np.array(fields) if self.batched else fields[0]
        result[self.key_name] = self.params

    def _backward_params(self, result):
        self.tmp_params = None
        self._init_params(result)
        params = result.pop(self.key_name, None)
        if params is not None:
            self.params = -params

    def dense_field(self, device):
        """[dim, *image_shape] displacements (z, y, x components) -- the batch stage: [batch, dim,
        *image_shape] -- cached per draw."""
        if self.tmp_params is None:
            coarse = torch.from_numpy(self.params if self.batched else self.params[None])
            grid = coarse.permute(0, self.dim + 1, *range(1, self.dim + 1)) / 2
            shape_xyz = list(grid.shape[2:])[::-1]
            roi = geometry.window_rois(self.dim, [1.5] * self.dim, [s - 1.5 for s in shape_xyz],
                                       index=np.arange(grid.shape[0]))
            fn = affine_2d if self.dim == 2 else affine_3d
            dense = fn(grid.to(device).contiguous(), torch.from_numpy(roi).to(device),
                       tuple(self.image_shape), 1, 1, True, self.INTER_ORDER)
            self.tmp_params = dense if self.batched else dense.squeeze(0)
        return self.tmp_params

    def elastic_transform(self, image, order=1):
        field = self.dense_field(image.device)
        fn = apply_offset_2d if self.dim == 2 else apply_offset_3d
        if not self.batched:
            image, field = image.unsqueeze(0), field.unsqueeze(0)
        if order == 0 and image.dtype == torch.int32:
            # the reference converts labels to float, warps and converts back
            # (aug_cuda/aug_spatial.py:664-668); the warp takes int32 maps as they are
            out = fn(image, field, order=0)
        else:
            if order == 0:
                image = image.to(self.img_type)
            out = fn(image, field.to(image.dtype), order=order)
            out = out.int() if order == 0 else out
        return out if self.batched else out.squeeze(0)

    def apply_to_img(self, result):
        for key in result.get('img_fields', []):
            result[key] = self.elastic_transform(result[key])

    def apply_to_seg(self, result):
        for key in result.get('seg_fields', []):
            result[key] = self.elastic_transform(result[key], order=0).int()

    def apply_to_det(self, result):
        for key in result.get('det_fields', []):
            if self.batched:   # as in the reference (aug_cuda_batch/aug_spatial.py:318-320)
                raise NotImplementedError
            boxes = np.copy(result[key].cpu().numpy())
            field = self.dense_field(result[key].device).cpu().numpy()
            top = np.array(self.image_shape) - 1
            for box in boxes:
                corners = []
                for pick in itertools.product(*[(a, a + self.dim) for a in range(self.dim)]):
                    point = box[list(pick)]                                  # x, y[, z]
                    voxel = np.clip(np.int64(point)[::-1], 0, top)           # z, y, x index
                    corners.append(point - field[(slice(None), *voxel)][::-1])
                corners = np.stack(corners)
                box[:self.dim] = corners.min(0)
                box[self.dim:2 * self.dim] = corners.max(0)
            result[key] = torch.from_numpy(boxes).to(result[key].device)


class BatchCudaRandomElasticDeformation(CudaRandomElasticDeformation, BatchCudaAugBase):
    """aug_cuda_batch/aug_spatial.py:204-320: one control grid per sample of the batch (drawn in sample
    order), all upsampled by one call of the affine engine and applied by one warp."""
