"""GPU augmentation stages that build rois for the resampling engine (the callers of
``affine_2d`` / ``affine_3d`` / ``apply_offset_*`` in the reference's ``medvision.aug_cuda`` and
``medvision.aug_cuda_batch``)."""
from .base import BatchCudaAugBase, CudaAugBase
from .spatial import (BatchCudaCropCenterWithAffine, BatchCudaCropDetWithAffine,
                      BatchCudaCropFirstDetWithAffine, BatchCudaCropForegroundWithAffine,
                      BatchCudaCropRandomWithAffine,
                      BatchCudaRandomAffine, BatchCudaRandomElasticDeformation, BatchCudaRandomRotate, BatchCudaRandomScale,
                      BatchCudaRandomShift, BatchCudaResize, CudaCropCenterWithAffine,
                      CudaCropFirstDetWithAffine, CudaCropRandomWithAffine, CudaRandomAffine,
                      CudaRandomElasticDeformation, CudaRandomRotate, CudaRandomScale,
                      CudaRandomShift, CudaResize)

__all__ = [n for n in dir() if n.startswith(('Cuda', 'BatchCuda'))]
