"""Stage protocol of the GPU augmentation layer.

Same contract as the reference's ``CudaAugBase`` (medvision/aug_cuda/base.py:28-223) and
``BatchCudaAugBase`` (medvision/aug_cuda_batch/base.py:28-226): a stage is called with a result
dict (``img`` [C, *spatial] -- or [B, C, *spatial] for batch stages -- on the GPU, ``img_dim``,
the field lists ``img_fields`` / ``seg_fields`` / ``det_fields``, optional ``img_spacing``), runs
with probability ``p * latitude`` (or always), draws its parameters into ``result[<Name>_params]``
and applies them to images, segmentations and boxes; ``history`` / ``time`` / ``memory`` record
what ran; stages with ``canBackward`` undo themselves from the stored parameters when called with
``forward=False``.  Random draws use ``random`` for the gate and ``numpy.random`` for parameters,
in the reference's order, so seeded pipelines draw the same parameters.
"""
import copy
import random
import time
from datetime import datetime

import numpy as np
import torch


def _peak_mib():
    """Peak of allocated GPU memory in MiB, as ``torch.cuda.max_memory_allocated`` reports it; read
    from the nested statistics (that call flattens the whole tree first, tens of microseconds per
    stage)."""
    if not torch.cuda.is_available():
        return 0.0
    stats = torch.cuda.memory_stats_as_nested_dict()     # {} before the first GPU call
    return stats.get("allocated_bytes", {}).get("all", {}).get("peak", 0) / 2 ** 20


class CudaAugBase:
    batched = False     # True: tensors carry a leading batch axis

    def __init__(self):
        self.p = 0.
        self.latitude = 1.0
        self.always = False
        self.dim = None
        self.params = None
        self.isForwarding = None
        self.name = self.__class__.__name__
        self.key_name = self.name + '_params'

    def __repr__(self):
        return self.__class__.__name__ + '()'

    # ---- what a stage may override -----------------------------------------------------------
    @property
    def canBackward(self):
        return False

    @property
    def repeats(self):
        return 1

    def _forward_params(self, result):
        pass

    def _backward_params(self, result):
        pass

    def apply_to_img(self, result):
        pass

    def apply_to_cls(self, result):
        pass

    def apply_to_seg(self, result):
        pass

    def apply_to_det(self, result):
        pass

    # ---- helpers -----------------------------------------------------------------------------
    @staticmethod
    def get_range(val_range, bias=0, always_pos=False):
        """bias + U(lo, hi); a single number r means (-r, r), or (0, r) with ``always_pos``."""
        if isinstance(val_range, (list, tuple)):
            if len(val_range) != 2 or val_range[0] > val_range[1]:
                raise AssertionError(f"a range is (low, high) with low <= high, got {val_range}")
            low, high = val_range
        elif isinstance(val_range, (int, float)):
            low, high = (0, val_range) if always_pos else (-val_range, val_range)
        else:
            raise AssertionError(f"a range is a number or a (low, high) pair, got {val_range!r}")
        return bias + np.random.uniform(low, high)

    @staticmethod
    def to_tuple(value, length=1):
        """A scalar repeated ``length`` times; an iterable as a tuple, which must have ``length`` entries."""
        if np.ndim(value) == 0:
            return (value,) * length
        entries = tuple(value)
        assert len(entries) == length, f'Dimension not match. Required is {length}D but value is {len(entries)}D'
        return entries

    def setLatitude(self, val):
        self.latitude = val

    def getLatitude(self):
        return self.latitude

    def _init_params(self, result):
        lead = 2 if self.batched else 1
        self.dim = self.dim if self.dim else result['img_dim']
        self.img_type = result['img'].dtype
        self.array_shape = tuple(result['img'].shape) if 'img' in result else tuple(result['img_shape'])
        self.batch = self.array_shape[0] if self.batched else 1
        self.channels = self.array_shape[lead - 1]
        self.image_shape = self.array_shape[lead:]
        self.image_axes = tuple(range(lead, self.dim + lead))
        self.params = None

    # ---- driver ------------------------------------------------------------------------------
    def _apply_all(self, result):
        self._device_rois = None   # images and segmentations share one upload of the stage's rois
        self.apply_to_img(result)
        self.apply_to_cls(result)
        self.apply_to_seg(result)
        self.apply_to_det(result)

    def forward(self, result):
        assert isinstance(result, dict), f'A dict is required but got a {type(result)}!'
        tic = time.time()
        self.isForwarding = True
        assert self.always or self.p > 0., f'self.always={self.always} or self.p={self.p} is needed.'
        if self.always or random.random() <= self.p * self.latitude:
            self.params = None
            self._forward_params(result)
            self._apply_all(result)
        for key in ('history', 'time', 'memory'):
            result.setdefault(key, [])
        peak = _peak_mib()
        result['history'].append(self.name)
        result['memory'].append(f"{self.name}-{peak:.02f}MB")
        started = datetime.fromtimestamp(tic).strftime('%H:%M:%S.%f')
        result['time'].append(f"{self.name}-{started}-{time.time() - tic:.03f}s")
        return result

    def backward(self, result):
        assert isinstance(result, dict)
        stamp, last = result['time'].pop(), result['history'].pop()
        assert self.name in stamp, f'{self.name} {stamp}'
        assert last == self.name, f'require params to be {self.name}, but the last is {last}'
        self.isForwarding = False
        if self.canBackward:
            self.params = None
            self._backward_params(result)
            if self.params is not None:   # the stage may not have fired in the forward pass
                self._apply_all(result)
        return result

    def __call__(self, result, forward=True):
        if forward:
            if isinstance(result, dict) and self.repeats == 1:
                return self.forward(result)
            items = [result] if isinstance(result, dict) else result
            if self.repeats > 1:
                return [self.forward(copy.deepcopy(r)) for r in items for _ in range(self.repeats)]
            return [self.forward(r) for r in items]
        if isinstance(result, list):
            return [self.backward(r) for r in result]
        return self.backward(result)


class BatchCudaAugBase(CudaAugBase):
    batched = True
