"""ctypes loader for ``libmedvision_hip.so`` (the C ABI declared in ``include/medvision_hip.h``).

There is no CPU or pure-torch fallback: if the library has not been built, every operator raises.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmedvision_hip.so")

MV_F32, MV_F16, MV_BF16, MV_F64 = 0, 1, 2, 3
MV_I32 = 4   # int32 label maps: the displacement warp and the affine engines at order 0
DTYPES = {torch.float32: MV_F32, torch.float16: MV_F16, torch.bfloat16: MV_BF16,
          torch.float64: MV_F64}

_i, _f, _p, _sz = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t


class DcnShape(ctypes.Structure):
    """Mirror of ``mv_dcn3d_shape``."""
    _fields_ = [(n, _i) for n in (
        "batch", "in_channels", "depth", "height", "width", "out_channels", "kernel_d", "kernel_h",
        "kernel_w", "stride_d", "stride_h", "stride_w", "pad_d", "pad_h", "pad_w", "dil_d",
        "dil_h", "dil_w", "groups", "deformable_groups")]


class Dcn2dShape(ctypes.Structure):
    """Mirror of ``mv_dcn2d_shape``."""
    _fields_ = [(n, _i) for n in (
        "batch", "in_channels", "height", "width", "out_channels", "kernel_h", "kernel_w",
        "stride_h", "stride_w", "pad_h", "pad_w", "dil_h", "dil_w", "groups", "deformable_groups")]


_SHAPE_P = ctypes.POINTER(DcnShape)
_SHAPE2_P = ctypes.POINTER(Dcn2dShape)

# name -> (restype, argtypes); must list every symbol of include/medvision_hip.h
SIGNATURES = {
    "mv_last_error": (ctypes.c_char_p, []),
    "mv_version": (_i, []),
    "mv_roi_align_2d_forward": (_i, [_p, _p, _p, _i] + [_i] * 7 + [_f, _i, _i, _p, _sz, _p]),
    "mv_roi_align_2d_backward": (_i, [_p, _p, _p, _i] + [_i] * 7 + [_f, _i, _i, _p, _p]),
    "mv_roi_align_3d_forward": (_i, [_p, _p, _p, _i] + [_i] * 9 + [_f, _i, _i, _p, _sz, _p]),
    "mv_roi_align_3d_backward": (_i, [_p, _p, _p, _i] + [_i] * 9 + [_f, _i, _i, _p, _p]),
    "mv_roi_align_rotated_2d_forward": (_i, [_p, _p, _p, _i] + [_i] * 7 + [_f, _i, _i, _i, _p, _sz, _p]),
    "mv_roi_align_rotated_2d_backward": (_i, [_p, _p, _p, _i] + [_i] * 7 + [_f, _i, _i, _i, _p, _p]),
    "mv_roi_align_rotated_3d_forward": (_i, [_p, _p, _p, _i] + [_i] * 9 + [_f, _i, _i, _i, _p, _sz, _p]),
    "mv_roi_align_rotated_3d_backward": (_i, [_p, _p, _p, _i] + [_i] * 9 + [_f, _i, _i, _i, _p, _p]),
    "mv_roi_align_backward_workspace_bytes": (_sz, [_i] * 6),
    "mv_roi_align_forward_workspace_bytes": (_sz, [_i] * 8),
    "mv_roi_align_forward_workspace_bytes_for_input": (_sz, [_i] * 12),
    "mv_roi_align_prepared_bytes": (_sz, [_i] * 7),
    "mv_roi_align_prepare_features": (_i, [_p, _i] + [_i] * 6 + [_p, _sz, _p]),
    "mv_roi_align_forward_prepared": (_i, [_p, _p, _p, _p, _i] + [_i] * 10 + [_f, _i, _i, _p, _sz, _p]),
    "mv_affine_2d": (_i, [_p, _p, _p, _i] + [_i] * 7 + [_f, _i, _i, _i, _p, _sz, _p]),
    "mv_affine_3d": (_i, [_p, _p, _p, _i] + [_i] * 9 + [_f, _i, _i, _i, _p, _sz, _p]),
    "mv_dcn3d_output_dims": (_i, [_SHAPE_P, ctypes.POINTER(_i), ctypes.POINTER(_i), ctypes.POINTER(_i)]),
    "mv_dcn3d_forward_workspace_bytes": (_sz, [_SHAPE_P, _i]),
    "mv_dcn3d_backward_workspace_bytes": (_sz, [_SHAPE_P, _i]),
    "mv_dcn3d_forward": (_i, [_p] * 6 + [_SHAPE_P, _i, _p, _p]),
    "mv_dcn3d_backward": (_i, [_p] * 10 + [_SHAPE_P, _i, _p, _p]),
    "mv_dcn_set_column_budget": (None, [_sz]),
    "mv_dcn_column_budget": (_sz, []),
    "mv_dcn3d_forward_static": (_i, [_p] * 6 + [_SHAPE_P, _i, _p]),
    "mv_dcn2d_output_dims": (_i, [_SHAPE2_P, ctypes.POINTER(_i), ctypes.POINTER(_i)]),
    "mv_dcn2d_forward_workspace_bytes": (_sz, [_SHAPE2_P, _i]),
    "mv_dcn2d_backward_workspace_bytes": (_sz, [_SHAPE2_P, _i]),
    "mv_dcn2d_forward": (_i, [_p] * 6 + [_SHAPE2_P, _i, _p, _p]),
    "mv_dcn2d_backward": (_i, [_p] * 10 + [_SHAPE2_P, _i, _p, _p]),
    "mv_deform_warp_2d": (_i, [_p, _p, _p, _i] + [_i] * 4 + [_i, _p]),
    "mv_deform_warp_3d": (_i, [_p, _p, _p, _i] + [_i] * 5 + [_i, _p]),
    "mv_deform_conv_3d": (_i, [_p] * 6 + [_i, _i, _p]),
    "mv_deform_conv_2d": (_i, [_p] * 6 + [_i, _i, _p]),
}

_lib = None


def load():
    """Load the shared library and bind every entry point; raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m medvision_amd.build` "
                "(there is no CPU fallback)")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(status):
    if status != 0:
        raise RuntimeError(load().mv_last_error().decode())


def dtype_code(t):
    try:
        return DTYPES[t.dtype]
    except KeyError:
        raise RuntimeError(f"unsupported dtype {t.dtype}") from None


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def stream_of(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)
