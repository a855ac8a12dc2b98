"""``mv_dcn3d_forward_static`` -- the forward pass for callers that cannot allocate -- against
``mv_dcn3d_forward`` with a caller-provided workspace, through the C ABI.  Both run the same
kernels, so the results must be bit-identical.  Two calls in a row share the library's static
scratch array, the second on a smaller layer."""
import ctypes

import pytest
import torch

import workloads as wl

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
_warm = []


def _call_pair(lib, _lib, B, Cin, Cout, size, dtype, seed):
    g = wl.gen(seed)
    x, off, mask, w, b = [t.to(DEV) for t in wl.dcn_inputs(g, B, Cin, Cout, size, 3, 1, 1, dtype)]
    shape = _lib.DcnShape(B, Cin, *size, Cout, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1)
    code = _lib.dtype_code(x)
    need = lib.mv_dcn3d_forward_workspace_bytes(ctypes.byref(shape), code)
    assert 0 < need <= 32 << 20
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    want = torch.full((B, Cout, *size), float("nan"), dtype=dtype, device=DEV)
    got = torch.full_like(want, float("nan"))
    stream = _lib.stream_of(x)
    _lib.check(lib.mv_dcn3d_forward(_lib.ptr(x), _lib.ptr(off), _lib.ptr(mask), _lib.ptr(w), _lib.ptr(b),
                                    _lib.ptr(want), ctypes.byref(shape), code, _lib.ptr(ws), stream))
    torch.cuda.synchronize()
    if not _warm:
        # the first call on a device looks the scratch array's address up (and may load the code
        # object); the allocation check below is about the calls after it
        _lib.check(lib.mv_dcn3d_forward_static(_lib.ptr(x), _lib.ptr(off), _lib.ptr(mask), _lib.ptr(w),
                                               _lib.ptr(b), _lib.ptr(got), ctypes.byref(shape), code, stream))
        torch.cuda.synchronize()
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        _warm.append(True)
    # free device memory as the driver reports it (hipMemGetInfo): sees a hipMalloc / hipFree made
    # inside the library, which torch's allocator statistics would not
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    _lib.check(lib.mv_dcn3d_forward_static(_lib.ptr(x), _lib.ptr(off), _lib.ptr(mask), _lib.ptr(w),
                                           _lib.ptr(b), _lib.ptr(got), ctypes.byref(shape), code, stream))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before, "device memory changed hands during the call"
    assert torch.isfinite(want).all()
    assert torch.equal(got, want), float((got.float() - want.float()).abs().max())


def test_static_scratch_forward_matches_workspace_forward():
    from medvision_amd import _lib
    lib = _lib.load()
    print("case: fp16 [2,32,24,24,32] -> 64, then [1,32,9,10,11] -> 32, then bf16, fp32", flush=True)
    _call_pair(lib, _lib, 2, 32, 64, (24, 24, 32), torch.float16, 11)
    _call_pair(lib, _lib, 1, 32, 32, (9, 10, 11), torch.float16, 12)     # smaller: stale scratch beyond it
    _call_pair(lib, _lib, 1, 32, 64, (8, 12, 16), torch.bfloat16, 13)
    _call_pair(lib, _lib, 2, 16, 32, (10, 9, 8), torch.float32, 14)


def test_static_scratch_rejects_layers_beyond_its_size():
    from medvision_amd import _lib
    lib = _lib.load()
    shape = _lib.DcnShape(4, 64, 64, 64, 64, 64, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1)   # 134 MB of layout buffers
    assert lib.mv_dcn3d_forward_workspace_bytes(ctypes.byref(shape), _lib.MV_F16) > 32 << 20
    t = torch.zeros(1, device=DEV)
    status = lib.mv_dcn3d_forward_static(_lib.ptr(t), _lib.ptr(t), _lib.ptr(t), _lib.ptr(t), None,
                                         _lib.ptr(t), ctypes.byref(shape), _lib.MV_F16, None)
    assert status == 1
    assert b"static scratch holds 33554432" in lib.mv_last_error()
