"""CPU-side checks of the boundary: the shared library loads, exports every symbol the header
declares, and the host shim rejects bad arguments without touching a GPU."""
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_symbols():
    text = open(os.path.join(ROOT, "include", "medvision_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(mv_[a-z0-9_]+)\s*\(", text))


def test_library_exports_every_declared_symbol():
    from medvision_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from medvision_amd import build
        build.build()
    lib = _lib.load()
    declared = _header_symbols()
    assert declared, "no symbols parsed from the header"
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.mv_version() >= 1


def test_workspace_queries_and_dims_need_no_gpu():
    from medvision_amd import _lib
    import ctypes
    lib = _lib.load()
    assert lib.mv_roi_align_backward_workspace_bytes(_lib.MV_F32, 2, 3, 4, 5, 6) == 0
    assert lib.mv_roi_align_backward_workspace_bytes(_lib.MV_F16, 2, 3, 4, 5, 6) == 4 * 2 * 3 * 4 * 5 * 6
    s = _lib.DcnShape(2, 32, 48, 48, 48, 64, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1)
    d, h, w = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    assert lib.mv_dcn3d_output_dims(ctypes.byref(s), ctypes.byref(d), ctypes.byref(h), ctypes.byref(w)) == 0
    assert (d.value, h.value, w.value) == (48, 48, 48)
    s2 = _lib.DcnShape(2, 32, 9, 10, 11, 64, 3, 2, 3, 2, 1, 2, 0, 1, 2, 1, 2, 1, 1, 1)
    assert lib.mv_dcn3d_output_dims(ctypes.byref(s2), ctypes.byref(d), ctypes.byref(h), ctypes.byref(w)) == 0
    assert (d.value, h.value, w.value) == ((9 - 3) // 2 + 1, (10 + 2 - 3) // 1 + 1, (11 + 4 - 3) // 2 + 1)
    bad = _lib.DcnShape(2, 30, 8, 8, 8, 64, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 4, 1)
    assert lib.mv_dcn3d_output_dims(ctypes.byref(bad), ctypes.byref(d), ctypes.byref(h), ctypes.byref(w)) == 1
    assert b"must divide group" in lib.mv_last_error()


def test_host_shim_rejects_cpu_tensors_and_bad_rois():
    import medvision_amd.ops as ops
    feat = torch.randn(1, 2, 4, 5, 6)
    with pytest.raises(RuntimeError, match="RoIAlign is not implemented on CPU"):
        ops.RoIAlign((2, 2, 2), 1.0, 2)(feat, torch.zeros(1, 7))
    with pytest.raises(RuntimeError, match="RoIAlignRotated is not implemented on CPU"):
        ops.RoIAlignRotated((2, 2, 2), 1.0, 2)(feat, torch.zeros(1, 10))
    with pytest.raises(AssertionError):
        ops.RoIAlignRotated((2, 2, 2), 1.0, 2)(feat, torch.zeros(1, 10), order=2)
    with pytest.raises(TypeError):
        from medvision_amd.ops.roi_align_nd import roi_align_3d
        roi_align_3d(feat, torch.zeros(1, 7), [2, 2, 2], 1.0, 2, 1)
    with pytest.raises(NotImplementedError):
        ops.ModulatedDeformConv3dPack(2, 3, 3, padding=1)(feat)
    with pytest.raises(AssertionError, match="order 2 is not supported"):
        ops.affine_3d(feat, torch.zeros(1, 10), (2, 2, 2), 1.0, 1, True, 2)
    with pytest.raises(RuntimeError, match="affine is not implemented on CPU"):
        ops.affine_3d(feat, torch.zeros(1, 10), (2, 2, 2), 1.0, 1, True, 3)
    m = ops.DeformConv3dPack(2, 4, 3, padding=1, bias=False)
    assert set(m.state_dict()) == {"weight", "bias", "conv_offset.weight", "conv_offset.bias"}
    assert not m.bias.requires_grad and m.conv_offset.lr_mult == 0.1
    with pytest.raises(ValueError):
        ops.DeformConv3d(3, 4, 3, 1, 1, groups=2)


def test_product_does_not_import_the_oracle():
    import subprocess, sys
    code = ("import sys; sys.path.insert(0, %r); import medvision_amd.ops, medvision_amd._C; "
            "assert not any(m == 'oracle' or m.startswith('oracle.') for m in sys.modules)" % ROOT)
    subprocess.check_call([sys.executable, "-c", code])
    for dirpath, _, files in os.walk(os.path.join(ROOT, "medvision_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                assert "oracle" not in open(os.path.join(dirpath, f)).read().lower(), f


def test_foreign_device_tensors_are_refused():
    """Every tensor handed to a kernel must sit on the input's device; the check runs on the host."""
    from medvision_amd import _C
    here, there = torch.zeros(2), torch.zeros(2, device="meta")
    _C._same_device(here, weight=here, bias=None)
    with pytest.raises(RuntimeError, match="weight is on meta"):
        _C._same_device(here, weight=there)
    with pytest.raises(RuntimeError, match="grad_input is on meta"):
        _C._same_device(here, output=here, grad_input=there)


def test_host_shim_cost_per_call(monkeypatch):
    """Host time of one call through the Python shim with the library stubbed out (argument checks,
    roi cast, workspace query cache, pointer and stream marshalling): the part of a launch that the
    shim adds on top of the C entry point.  Printed for the record; the bound is loose because the
    machine running the CPU suite is shared."""
    import ctypes
    import time
    import torch
    from medvision_amd import _C, _lib

    class Stub:
        def __getattr__(self, name):
            return lambda *a: 0

    class NoGuard:
        def __init__(self, t): pass
        def __enter__(self): pass
        def __exit__(self, *e): return False

    monkeypatch.setattr(_lib, "load", lambda: Stub())
    monkeypatch.setattr(_lib, "stream_of", lambda t: ctypes.c_void_p(0))
    monkeypatch.setattr(_C, "_require_cuda", lambda t, what: None)
    monkeypatch.setattr(_C, "_on_device", NoGuard)
    monkeypatch.setattr(_C, "_ws_bytes_cache", {})
    vol = torch.zeros(1, 1, 16, 16, 16, dtype=torch.float16)
    roi = torch.tensor([[0, 8, 8, 8, 16, 16, 16, 0, 0, 0]], dtype=torch.float32)
    out = torch.empty(1, 1, 16, 16, 16, dtype=torch.float16)
    call = lambda: _C.roi_align_rotated_3d_forward(vol, roi, out, 16, 16, 16, 1.0, 1, True, 1)
    for _ in range(200):
        call()
    best = 1e9
    for _ in range(5):
        t = time.perf_counter()
        for _ in range(2000):
            call()
        best = min(best, (time.perf_counter() - t) / 2000 * 1e6)
    print(f"roi_align_rotated_3d_forward shim: {best:.1f} us per call")
    assert best < 2000.0   # (a sanity bound only: ~8 us on an idle core)
