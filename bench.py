#!/usr/bin/env python
"""Benchmark of the trilinear-sampling hot path on one MI355X.

A "step" is one RoIAlignRotated3D forward over one batch of benchmark configuration 2 (fp16 volume
[4,1,128^3] -> 128^3, one rotated full-volume roi per sample, sampling_ratio 1), inputs resident in
HBM.  ``value`` is output Gvox/s.  Inputs/outputs rotate over ``--copies`` buffer sets (default 16,
~540 MB) so that consecutive steps are not served from the 256 MB Infinity Cache.  The same JSON
line carries the roofline of that kernel, the DCNv2-3D forward figure of config 4 (``dcn``) and the
CPU baseline (the reference's torch-function RoIAlign on the same shape, timed on the host cores on a
bounded sample; the fp64 oracle beside it).
"""
import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0   # MI355X dense fp16/bf16
# Measured on this part (microbenchmark, 4 wavefronts per SIMD): a three-operand vector instruction
# of one wavefront (v_fma_f32, v_fma_mix_f32, conversions) takes 2.03 ns of its SIMD; the vector L1
# returns 64 bytes per clock and compute unit at the ~1.97 GHz these kernels run at.
VALU_NS_PER_WAVE_INSTR = 2.03
SIMDS, CUS, L1_BYTES_PER_CLK, SHADER_GHZ = 1024, 256, 64, 1.97
DCN_L1_MISS_REQUESTS = 2.74e7   # config 4 forward, 64-byte requests from the L1s to the L2s per launch
L2_GATHER_TBPS = 15.0           # measured line rate of the L2s for scattered 16-byte gathers


PREHEAT_S = 0.3   # untimed launches of the same step before every timed leg, whatever --steps / --warmup say
_preheat_log = []


def _events_ms(fn, steps, warmup, preheat_s=None):
    # A short run reads the clocks of an idle GPU (20 steps of 25 us end long before the power
    # management has settled): keep the GPU busy with the same launches for a fixed time first.
    preheat_s = PREHEAT_S if preheat_s is None else preheat_s
    t_heat, n = time.perf_counter(), 0
    while preheat_s > 0 and time.perf_counter() - t_heat < preheat_s:
        for i in range(50):
            fn(n + i)
        n += 50
        torch.cuda.synchronize()
    _preheat_log.append(round((time.perf_counter() - t_heat) * 1e3, 1))
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        fn(i)
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return start.elapsed_time(stop) / steps, wall_ms / steps


def bench_affine(args, dtype=torch.float16):
    import medvision_amd.ops as ops
    import workloads as wl
    dev = "cuda:0"
    g = wl.gen(1)
    B, S = 4, 128
    vols = [torch.randn(B, 1, S, S, S, generator=g).to(dtype).to(dev) for _ in range(args.copies)]
    rois = [wl.affine_rois(g, B, (S, S, S)).to(dev) for _ in range(args.copies)]
    outs = [torch.empty(B, 1, S, S, S, dtype=dtype, device=dev) for _ in range(args.copies)]
    from medvision_amd import _C

    def step(i):
        j = i % args.copies
        _C.roi_align_rotated_3d_forward(vols[j], rois[j], outs[j], S, S, S, 1.0, 1, True, 1)

    ms, wall_ms = _events_ms(step, args.steps, args.warmup)
    preheat_ms = _preheat_log[-1]
    # practical ceiling of a launch of this size: a plain device copy of the same bytes
    copy_ms, _ = _events_ms(lambda i: outs[i % args.copies].copy_(vols[(i + 1) % args.copies]), args.steps, args.warmup)
    vox = B * S ** 3
    esz = torch.finfo(dtype).bits // 8
    alg_bytes = 2 * vox * esz            # read every input voxel once + write every output voxel
    return {"ms": ms, "wall_ms": wall_ms, "gvox_s": vox / ms / 1e6, "gbps": alg_bytes / ms / 1e6,
            "alg_bytes": alg_bytes, "vox": vox, "copy_ms": copy_ms, "preheat_ms": preheat_ms}


def bench_dcn(args, dtype=torch.float16):
    import workloads as wl
    from medvision_amd.ops.modulated_deform_conv_3d import modulated_deform_conv
    dev = "cuda:0"
    g = wl.gen(3)
    x, off, mask, w, b = [t.to(dev) for t in wl.dcn_inputs(g, 2, 32, 64, (48, 48, 48), 3, 1, 1, dtype)]

    def step(i):
        with torch.no_grad():
            modulated_deform_conv(x, off, mask, w, b, 1, 1, 1, 1, 1)

    ms, wall_ms = _events_ms(step, max(3, min(args.steps, 400)), max(1, min(args.warmup, 40)))
    flops = 2 * 2 * 64 * 32 * 27 * 48 ** 3
    # floors of the fused gather + blend: per (tap, position) 8 corners x 32 channels are blended in
    # fp32 (one fma per wavefront instruction and 64 lanes), and 8 x 64 bytes pass through the L1
    taps_pos = 2 * 48 ** 3 * 27
    blend_floor_us = taps_pos * 8 * 32 / 64 / SIMDS * VALU_NS_PER_WAVE_INSTR / 1e3
    gather_floor_us = taps_pos * 8 * 64 / (CUS * L1_BYTES_PER_CLK * SHADER_GHZ * 1e9) * 1e6
    # second floor, the L2 side of the gather: the kernel's corner reads miss the vector L1 for
    # DCN_L1_MISS_REQUESTS 64-byte requests per launch (TCP_TCC_READ_REQ_sum of the rocprofv3 counter
    # profile of this layer), and a microbenchmark of 16-byte gathers at random places of an 8 MB buffer
    # puts the L2s' line rate at L2_GATHER_TBPS over the chip
    l2_floor_us = DCN_L1_MISS_REQUESTS * 64 / (L2_GATHER_TBPS * 1e12) * 1e6

    # training step (forward + all five gradients), reported beside the forward figure
    ins = [t.clone().requires_grad_(True) for t in (x, off, mask, w, b)]
    gy = torch.randn(2, 64, 48, 48, 48, generator=g).to(dtype).to(dev)

    def train_step(i):
        for t in ins:
            t.grad = None
        modulated_deform_conv(*ins, 1, 1, 1, 1, 1).backward(gy)

    train_ms, _ = _events_ms(train_step, max(3, min(args.steps // 4, 50)), 3)
    return {"ms": ms, "wall_ms": wall_ms, "tflops": flops / ms / 1e9, "flops": flops, "train_ms": train_ms,
            "blend_floor_us": blend_floor_us, "gather_floor_us": gather_floor_us, "l2_floor_us": l2_floor_us}


def bench_other_configs(args):
    """The remaining measurement configurations of the path on the GPU (HIP events, 10 to 200 steps
    each): config 1 rois through the HIP RoIAlign3D, config 2 backward, config 3 (CT resize + 16
    rotated crops), config 5 (detection head: 4000 rois x 256 channels x 7^3) forward / backward.
    GB/s are algorithmic bytes (inputs read once + outputs written once) over the measured time."""
    import medvision_amd.ops as ops
    from medvision_amd import _C
    import workloads as wl
    dev = "cuda:0"
    res = {}
    g = wl.gen(0)
    feat = torch.randn(2, 16, 32, 64, 64, generator=g).to(dev)
    rois = wl.roi3d_detection(g, 128, 2, (64, 64, 32), (4.0, 24.0)).to(dev)
    out = torch.empty(128, 16, 7, 7, 7, device=dev)
    ms, _ = _events_ms(lambda i: _C.roi_align_3d_forward(feat, rois, out, 7, 7, 7, 1.0, 2, 1), 200, 20)
    res["config1_roialign3d_fp32"] = {"ms": round(ms, 4), "outputs_per_s": round(out.numel() / ms * 1e3, 1)}
    g = wl.gen(1)
    for dt, name in ((torch.float32, "fp32"), (torch.float16, "fp16")):
        vol = torch.randn(4, 1, 128, 128, 128, generator=g).to(dt).to(dev)
        r = wl.affine_rois(g, 4, (128, 128, 128)).to(dev)
        gy = torch.randn(4, 1, 128, 128, 128, generator=g).to(dt).to(dev)
        gi = torch.zeros_like(vol)
        ms, _ = _events_ms(lambda i: _C.roi_align_rotated_3d_backward(gy, r, gi, 128, 128, 128, 1.0, 1, True, 1), 50, 5)
        # algorithmic bytes: grad_output read once, grad_input read and written once (it accumulates)
        nbytes = 3 * vol.numel() * vol.element_size()
        res["config2_backward_" + name] = {"ms": round(ms, 4), "gbps": round(nbytes / ms / 1e6, 1),
                                           "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    # config 2 with a sampling grid of 2 per axis (8 samples per output voxel, summed inside the tiled kernel)
    g = wl.gen(1)
    r = wl.affine_rois(g, 4, (128, 128, 128)).to(dev)
    for dt, name in ((torch.float16, "fp16"), (torch.bfloat16, "bf16")):
        vol = torch.randn(4, 1, 128, 128, 128, generator=g).to(dt).to(dev)
        ms, _ = _events_ms(lambda i: ops.affine_3d(vol, r, (128, 128, 128), 1.0, 2, True, 1), 50, 5)
        res["config2_sampling_ratio_2_" + name] = {"ms": round(ms, 4), "gsamples_s": round(8 * vol.numel() / ms / 1e6, 1)}
        gy = torch.randn(4, 1, 128, 128, 128, generator=g).to(dt).to(dev)
        gi = torch.zeros_like(vol)
        bms, _ = _events_ms(lambda i: _C.roi_align_rotated_3d_backward(gy, r, gi, 128, 128, 128, 1.0, 2, True, 1), 30, 3)
        res["config2_sampling_ratio_2_" + name]["backward_ms"] = round(bms, 4)
    g = wl.gen(2)
    vol = wl.ct_like(g, (2, 1, 256, 512, 512)).to(dev)
    full = torch.tensor([[b, 256, 256, 128, 512, 512, 256, 0, 0, 0] for b in range(2)], dtype=torch.float32).to(dev)
    ms, _ = _events_ms(lambda i: ops.affine_3d(vol, full, (160, 256, 256), 1.0, 1, True, 1), 100, 10)
    nbytes = (vol.numel() + 2 * 160 * 256 * 256) * 2
    res["config3_resize_fp16"] = {"ms": round(ms, 4), "gbps": round(nbytes / ms / 1e6, 1)}
    small = ops.affine_3d(vol, full, (160, 256, 256), 1.0, 1, True, 1)
    crops = []
    for b in range(2):
        for _ in range(8):
            c = torch.rand(3, generator=g) * torch.tensor([256 - 96., 256 - 96., 160 - 96.]) + 48
            crops.append([b, *c.tolist(), 96, 96, 96, 0, 0, (float(torch.rand(1, generator=g)) * 2 - 1) * math.radians(15)])
    crops = torch.tensor(crops).to(dev)
    ms, _ = _events_ms(lambda i: ops.affine_3d(small, crops, (96, 96, 96), 1.0, 1, True, 1), 100, 10)
    res["config3_16_crops_96^3_fp16"] = {"ms": round(ms, 4), "gbps": round(2 * 16 * 96 ** 3 * 2 / ms / 1e6, 1)}
    del vol, small
    g = wl.gen(4)
    feat = torch.randn(2, 256, 24, 96, 96, generator=g).half().to(dev)
    rois = wl.roi3d_detection(g, 4000, 2, (384, 384, 96), (2.0, 48.0), log_uniform=True).to(dev)
    out = torch.empty(4000, 256, 7, 7, 7, dtype=torch.float16, device=dev)
    ms, _ = _events_ms(lambda i: _C.roi_align_3d_forward(feat, rois, out, 7, 7, 7, 0.25, 2, 1), 20, 3)
    nbytes = (feat.numel() + out.numel()) * 2
    res["config5_forward_fp16"] = {"ms": round(ms, 4), "goutputs_s": round(out.numel() / ms / 1e6, 2),
                                   "gbps": round(nbytes / ms / 1e6, 1)}
    # the same head when the re-ordered copy of the features is made once and kept (cascade stages, several
    # batches of rois on one feature map); the row above makes it in every call
    prepared = _C.roi_align_prepare(feat)
    ms, _ = _events_ms(lambda i: _C.roi_align_3d_forward(feat, rois, out, 7, 7, 7, 0.25, 2, 1, prepared), 20, 3)
    res["config5_forward_fp16_prepared_features"] = {"ms": round(ms, 4), "goutputs_s": round(out.numel() / ms / 1e6, 2),
                                                     "gbps": round(nbytes / ms / 1e6, 1)}
    del prepared
    gy = torch.randn_like(out)
    gi = torch.zeros_like(feat)
    ms, _ = _events_ms(lambda i: _C.roi_align_3d_backward(gy, rois, gi, 7, 7, 7, 0.25, 2, 1), 10, 2)
    res["config5_backward_fp16"] = {"ms": round(ms, 4), "gbps": round(nbytes / ms / 1e6, 1)}
    del feat, out, gy, gi
    # rotated detection head: 1000 rotated rois of 6 - 24 voxels x 64 channels x 7^3 cells, grid 2
    g = wl.gen(9)
    feat = torch.randn(2, 64, 48, 96, 96, generator=g).half().to(dev)
    ctr = torch.rand(1000, 3, generator=g) * torch.tensor([96., 96., 48.])
    ext = 6 + torch.rand(1000, 3, generator=g) * 18
    ang = (torch.rand(1000, 3, generator=g) * 2 - 1) * math.radians(30)
    rois = torch.cat([torch.randint(0, 2, (1000, 1), generator=g).float(), ctr, ext, ang], 1).to(dev)
    out = torch.empty(1000, 64, 7, 7, 7, dtype=torch.float16, device=dev)
    ms, _ = _events_ms(lambda i: _C.roi_align_rotated_3d_forward(feat, rois, out, 7, 7, 7, 1.0, 2, True, 1), 20, 3)
    gy = torch.randn_like(out)
    gi = torch.zeros_like(feat)
    bms, _ = _events_ms(lambda i: _C.roi_align_rotated_3d_backward(gy, rois, gi, 7, 7, 7, 1.0, 2, True, 1), 10, 2)
    res["rotated_head_1000x64x7^3_fp16"] = {"forward_ms": round(ms, 4), "backward_ms": round(bms, 4)}
    del feat, out, gy, gi
    # a 2-D head with large rois on a fine feature map (bins of 2 - 16 pixels, grid 2: the boxes are read sparsely)
    feat = torch.randn(2, 256, 200, 304, generator=g).half().to(dev)
    lo = torch.rand(1000, 2, generator=g) * torch.tensor([250., 160.])
    ext = 16 + torch.rand(1000, 2, generator=g) * 100
    rois = torch.cat([torch.randint(0, 2, (1000, 1), generator=g).float(), lo, lo + ext], 1).to(dev)
    out = torch.empty(1000, 256, 7, 7, dtype=torch.float16, device=dev)
    ms, _ = _events_ms(lambda i: _C.roi_align_2d_forward(feat, rois, out, 7, 7, 1.0, 2, 1), 20, 3)
    res["head_2d_1000x256x7^2_rois_16_116px_fp16"] = {"forward_ms": round(ms, 4)}
    del feat, out
    # RandomAffine on images: fp16 [8,3,512,512], one full-image rotated roi per sample (the tiled kernel with
    # the image rows as slices)
    g = wl.gen(10)
    img = torch.randn(8, 3, 512, 512, generator=g).half().to(dev)
    ang = (torch.rand(8, 1, generator=g) * 2 - 1) * math.radians(30)
    sc = 0.8 + torch.rand(8, 1, generator=g) * 0.4
    sh = (torch.rand(8, 2, generator=g) * 2 - 1) * 10
    rois = torch.cat([torch.arange(8, dtype=torch.float32)[:, None], 256 + sh, 512 / sc.expand(8, 2), ang], 1).to(dev)
    ms, _ = _events_ms(lambda i: ops.affine_2d(img, rois, (512, 512), 1.0, 1, True, 1), 100, 10)
    ms3, _ = _events_ms(lambda i: ops.affine_2d(img, rois, (512, 512), 1.0, 1, True, 3), 100, 10)
    res["affine_2d_8x3x512^2_fp16"] = {"ms": round(ms, 4), "gpix_s": round(img.numel() / ms / 1e6, 2),
                                       "gbps": round(2 * img.numel() * 2 / ms / 1e6, 1), "order3_ms": round(ms3, 4)}
    return res


def bench_next_rows(args):
    """Short timings of the operators either side of the headline path: order-3 resampling, the
    elastic pipeline (control-grid upsampling + displacement warp), a 2-D DCNv2 layer of FPN size
    and the augmentation stages that build the rois.  100 steps each (stages 50), HIP events."""
    import numpy as np
    import medvision_amd.ops as ops
    import medvision_amd.aug_cuda as aug
    from medvision_amd.ops.modulated_deform_conv_2d import modulated_deform_conv
    import workloads as wl
    dev, n = "cuda:0", 100
    g = wl.gen(7)
    res = {}
    vol = torch.randn(4, 1, 128, 128, 128, generator=g).half().to(dev)
    rois = wl.affine_rois(g, 4, (128, 128, 128)).to(dev)
    ms, _ = _events_ms(lambda i: ops.affine_3d(vol, rois, (128, 128, 128), 1.0, 1, True, 3), n, 10)
    res["affine_3d_order3_config2"] = {"ms": round(ms, 4), "gvox_s": round(4 * 128 ** 3 / ms / 1e6, 2)}
    grid = torch.randn(2, 3, 8, 8, 8, generator=g).to(dev)
    groi = torch.tensor([[b, 4, 4, 4, 5, 5, 5, 0, 0, 0] for b in range(2)], dtype=torch.float32, device=dev)
    ms, _ = _events_ms(lambda i: ops.affine_3d(grid, groi, (128, 128, 128), 1, 1, True, 3), n, 10)
    res["elastic_grid_upsample_8to128_order3"] = {"ms": round(ms, 4)}
    field = ops.affine_3d(grid, groi, (128, 128, 128), 1, 1, True, 3).half()
    img = vol[:2]
    ms, _ = _events_ms(lambda i: ops.apply_offset_3d(img, field, 1), n, 10)
    res["apply_offset_3d_2x128^3_fp16"] = {"ms": round(ms, 4), "gvox_s": round(2 * 128 ** 3 / ms / 1e6, 2)}
    img2 = torch.randn(8, 3, 512, 512, generator=g).half().to(dev)
    field2 = (torch.randn(8, 2, 512, 512, generator=g) * 3).half().to(dev)
    ms, _ = _events_ms(lambda i: ops.apply_offset_2d(img2, field2, 1), n, 10)
    res["apply_offset_2d_8x3x512^2_fp16"] = {"ms": round(ms, 4), "gpix_s": round(8 * 3 * 512 ** 2 / ms / 1e6, 2)}
    B, C, H, W = 8, 256, 100, 152
    x = torch.randn(B, C, H, W, generator=g).half().to(dev)
    w = (torch.randn(C, C, 3, 3, generator=g) * 0.02).half().to(dev)
    bias = torch.zeros(C, dtype=torch.float16, device=dev)
    off = (torch.randn(B, 18, H, W, generator=g) * 2).half().to(dev)
    msk = torch.sigmoid(torch.randn(B, 9, H, W, generator=g)).half().to(dev)
    ms, _ = _events_ms(lambda i: modulated_deform_conv(x, off, msk, w, bias, 1, 1, 1, 1, 1), n, 10)
    flops = 2 * B * C * C * 9 * H * W
    xs, ws, offs, ms_ = [t.clone().requires_grad_(True) for t in (x, w, off, msk)]

    def train(i):
        y = modulated_deform_conv(xs, offs, ms_, ws, bias, 1, 1, 1, 1, 1)
        y.backward(y)

    tms, _ = _events_ms(train, 20, 3)
    res["dcnv2_2d_fp16_[8,256,100,152]_3x3"] = {"ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 2),
                                                "forward_backward_ms": round(tms, 3)}
    # augmentation stages on one fp16 CT-sized sample [1, 128, 256, 256] with a label map
    np.random.seed(0)
    sample = {"img": torch.randn(1, 128, 256, 256, generator=g).half().to(dev),
              "gt_seg": torch.randint(0, 3, (1, 128, 256, 256), generator=g, dtype=torch.int32).to(dev),
              "img_dim": 3, "img_spacing": (1.0, 1.0, 1.0), "img_fields": ["img"], "seg_fields": ["gt_seg"],
              "det_fields": []}
    stages = {"CudaResize(0.75)": aug.CudaResize(factor=(0.75, 0.75, 0.75)),
              "CudaRandomAffine": aug.CudaRandomAffine(1.0, 0.2, 0.1, 30),
              "CudaCropRandomWithAffine(96^3)": aug.CudaCropRandomWithAffine((96, 96, 96), 0.2, 0.1, 30),
              "CudaRandomElasticDeformation": aug.CudaRandomElasticDeformation(1.0, 8, 0.8)}
    for name, stage in stages.items():
        ms, wall = _events_ms(lambda i: stage(dict(sample)), 50, 10)
        res["aug:" + name] = {"ms_gpu": round(ms, 3), "ms_wall": round(wall, 3)}
    return res


def cpu_baseline(args):
    """The reference's own CPU path on the shape of config 2: its torch-function RoIAlign (affine_grid +
    grid_sample per roi, fp32, medvision/ops/pytorch_ops/roi_align.py:22-105, restated in
    oracle/torchfun_roi_align.py) on a [4,1,128^3] volume with one full-volume box per sample and a
    128^3 output -- the class takes plain boxes only, so the rois carry no rotation; the work per output
    voxel (one trilinear sample) is that of the GPU step.  Passes are repeated for about half of
    --cpu-seconds with all torch threads, then a few passes with one thread; medians are reported.
    The fp64 C oracle (the checker of the parity tests) is timed on the rotated rois of the GPU step
    for the other half and reported under ``oracle_port``."""
    import oracle
    import workloads as wl
    from oracle.torchfun_roi_align import torchfun_roi_align
    g = wl.gen(1)
    B, S = 4, 128
    vol = torch.randn(B, 1, S, S, S, generator=g)
    boxes = torch.tensor([[b, 0, 0, 0, S, S, S] for b in range(B)], dtype=torch.float32)
    threads = torch.get_num_threads()

    def passes(budget_s, fn, at_most=200):
        fn()   # warm-up
        times, t_start = [], time.perf_counter()
        while time.perf_counter() - t_start < budget_s and len(times) < at_most:
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        return sorted(times)[len(times) // 2], len(times)

    t_all, n_all = passes(args.cpu_seconds * 0.35, lambda: torchfun_roi_align(vol, boxes, (S, S, S), 1.0))
    torch.set_num_threads(1)
    t_one, n_one = passes(args.cpu_seconds * 0.15, lambda: torchfun_roi_align(vol[:1], boxes[:1], (S, S, S), 1.0), 5)
    torch.set_num_threads(threads)

    # the fp64 oracle on the benchmark's own (rotated) rois
    oracle.build()
    cores = min(os.cpu_count() or 1, 16)
    oracle.set_threads(cores)
    half = vol.half()
    rois = wl.affine_rois(g, B, (S, S, S))
    t_orc, n_orc = passes(args.cpu_seconds * 0.4, lambda: oracle.roi_align_forward(half, rois, (S, S, S), 1.0, 1, True, 1, True))
    oracle.set_threads(1)
    t0 = time.perf_counter()
    oracle.roi_align_forward(half[:1], rois[:1], (S, S, S), 1.0, 1, True, 1, True)
    t_orc1 = time.perf_counter() - t0
    oracle.set_threads(cores)
    return {"value": round(B * S ** 3 / t_all / 1e9, 4), "unit": "Gvox/s", "cores": threads, "kind": "port",
            "reference_path": "medvision/ops/pytorch_ops/roi_align.py:22-105 (torch-function RoIAlign: affine_grid + "
                              "grid_sample per roi, fp32), restated line by line in oracle/torchfun_roi_align.py",
            "sample": f"config 2 shape: fp32 [4,1,128^3] -> 128^3, one full-volume box per sample (the class has no "
                      f"rotation), median of {n_all} passes after 1 warm-up ({t_all * 1e3:.0f} ms per pass), "
                      f"{threads} torch threads",
            "one_thread": {"value": round(S ** 3 / t_one / 1e9, 4), "unit": "Gvox/s", "cores": 1,
                           "sample": f"one sample of the same, median of {n_one} passes ({t_one * 1e3:.0f} ms per pass)"},
            "cpu_count": os.cpu_count(),
            "oracle_port": {"value": round(B * S ** 3 / t_orc / 1e9, 4), "unit": "Gvox/s", "cores": cores,
                            "sample": f"config 2 with its rotated rois (fp16 [4,1,128^3] -> 128^3) through the fp64 C "
                                      f"oracle, OpenMP x{cores}, median of {n_orc} passes ({t_orc * 1e3:.0f} ms per pass)",
                            "one_thread": {"value": round(S ** 3 / t_orc1 / 1e9, 4), "unit": "Gvox/s",
                                           "sample": f"one sample, one pass ({t_orc1 * 1e3:.0f} ms)"}}}


def cpu_reference_paths(args):
    """The reference's own CPU paths, restated (baseline only, no parity claim): the torch-function
    RoIAlign on config 1 (aligned as the configuration says, and with the class's default), the
    aug_cpu affine steps (scipy.ndimage) and its elastic step on one 128^3 volume, each with all
    threads and with one."""
    import numpy as np
    import workloads as wl
    from oracle.torchfun_roi_align import torchfun_roi_align
    res = {"cpu_count": os.cpu_count(), "torch_threads": torch.get_num_threads()}
    g = wl.gen(0)
    feat = torch.randn(2, 16, 32, 64, 64, generator=g)
    rois = wl.roi3d_detection(g, 128, 2, (64, 64, 32), (4.0, 24.0))
    torchfun_roi_align(feat, rois[:8], (7, 7, 7), 1.0)

    def timed(fn, reps=3):
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            out = fn()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[len(ts) // 2], out

    all_threads = torch.get_num_threads()
    for aligned in (True, False):
        entry = {}
        for threads in (all_threads, 1):
            torch.set_num_threads(threads)
            t, out = timed(lambda: torchfun_roi_align(feat, rois, (7, 7, 7), 1.0, aligned=aligned))
            entry["threads_%d" % threads] = {"ms": round(t * 1e3, 2), "outputs_per_s": round(out.numel() / t, 1)}
        torch.set_num_threads(all_threads)
        res["torchfun_roialign_config1_aligned_%s" % aligned] = entry
    try:
        from scipy import ndimage as ndi
        rng = np.random.default_rng(0)
        vol = rng.standard_normal((1, 128, 128, 128)).astype(np.float32)
        steps = {
            "rotate_order1": lambda: ndi.rotate(vol, 20.0, axes=(3, 2), reshape=False, order=1),
            "shift_order1": lambda: ndi.shift(vol, (0, 5.5, -3.2, 7.1), order=1),
            "zoom_order1": lambda: ndi.zoom(vol, (1, 1.1, 1.1, 1.1), order=1),
            "resize_zoom_order2": lambda: ndi.zoom(vol, (1, 0.625, 0.5, 0.5), order=2),
        }
        # Elastic step (aug_cpu/aug_spatial.py:604-638 goes through SimpleITK, which is not installed:
        # the same two stages with scipy): a coarse 8^3 field of three components is upsampled to the
        # volume with cubic splines, then the volume is sampled at identity + field, order 1.
        coarse = (rng.random((3, 8, 8, 8)).astype(np.float32) * 2 - 1) * 6.0
        ident = np.meshgrid(*[np.arange(128, dtype=np.float32)] * 3, indexing="ij")

        def elastic():
            field = [ndi.zoom(c, 16.0, order=3) for c in coarse]
            coords = [ident[a] + field[a] for a in range(3)]
            return ndi.map_coordinates(vol[0], coords, order=1, mode="nearest")

        steps["elastic_zoom3_plus_map_coordinates1"] = elastic
        for name, fn in steps.items():   # scipy.ndimage runs on one thread
            dt, o = timed(fn, 1)
            res["scipy_" + name] = {"ms": round(dt * 1e3, 1), "gvox_s": round(o.size / dt / 1e9, 5), "threads": 1}
    except Exception as e:  # scipy missing on the box
        res["scipy"] = f"unavailable: {e}"
    return res


def copy_calibration(args):
    """Plain device copy of known size, for scaling the FETCH_SIZE / WRITE_SIZE counters."""
    n = 4 * 128 ** 3
    src = [torch.randn(n, device="cuda:0").half() for _ in range(args.copies)]
    dst = [torch.empty(n, dtype=torch.float16, device="cuda:0") for _ in range(args.copies)]
    ms, _ = _events_ms(lambda i: dst[i % args.copies].copy_(src[i % args.copies]), args.steps, args.warmup)
    print(json.dumps({"copy_bytes_read": 2 * n, "copy_bytes_written": 2 * n, "ms": ms,
                      "gbps": 4 * n / ms / 1e6}))


def resample_timeline(args):
    """In-kernel phase times of the tiled resampler on config 2 (fp16): runs the instrumented twin of the
    library (time stamps of thread 0 of every workgroup, 100 MHz wall clock, see MV_TL in
    csrc/roi_resample.hip) and prints, per marked point, the minimum / median / maximum over the
    workgroups of the last launch in microseconds since the first workgroup entered the kernel."""
    import ctypes
    import numpy as np
    from medvision_amd import _lib, build
    import workloads as wl
    _lib.LIB_PATH = build.TIMELINE_LIB_PATH
    _lib.load()
    from medvision_amd import _C
    dev, B, S = "cuda:0", 4, 128
    g = wl.gen(1)
    vols = [torch.randn(B, 1, S, S, S, generator=g).half().to(dev) for _ in range(args.copies)]
    rois = [wl.affine_rois(g, B, (S, S, S)).to(dev) for _ in range(args.copies)]
    outs = [torch.empty(B, 1, S, S, S, dtype=torch.float16, device=dev) for _ in range(args.copies)]
    ms, _ = _events_ms(lambda i: _C.roi_align_rotated_3d_forward(vols[i % args.copies], rois[i % args.copies],
                                                                  outs[i % args.copies], S, S, S, 1.0, 1, True, 1),
                       args.steps, args.warmup)
    raw = ctypes.CDLL(_lib.LIB_PATH)
    buf = np.zeros(4096 * 16, dtype=np.uint64)
    rc = raw.mv_debug_resample_timeline(ctypes.c_void_p(buf.ctypes.data), ctypes.c_size_t(buf.nbytes))
    if rc != 0:
        sys.exit("mv_debug_resample_timeline failed: %d" % rc)
    t = buf.reshape(4096, 16).astype(np.int64)
    t = t[t[:, 0] > 0]
    t0 = t[:, 0].min()
    names = ["kernel entered", "first wavefront starts planning", "plans written", "past the barrier behind the plans",
             "first box arrived in registers", "box of item 0 in LDS", "box of item 1 in LDS", "box of item 2 in LDS",
             "box of item 3 in LDS", "last item interpolated", "stores drained"]
    rows = []
    for k, name in enumerate(names):
        v = (t[:, k] - t0)[t[:, k] > 0] / 100.0
        rows.append({"point": name, "min_us": round(float(v.min()), 2), "median_us": round(float(np.median(v)), 2),
                     "max_us": round(float(v.max()), 2)})
    # the two workgroups of a compute unit: blocks i and i + half the grid of an XCD share one (the older is served first)
    done = (t[:, 10] - t0) / 100.0
    print(json.dumps({"workgroups": int(len(t)), "instrumented_kernel_us": round(ms * 1e3, 2), "points": rows,
                      "finish_us_by_launch_order": {"first_half_of_each_xcd": round(float(np.median(done[: len(done) // 2])), 2),
                                                    "second_half_of_each_xcd": round(float(np.median(done[len(done) // 2:])), 2)}}))


def lds_tap_reads(args):
    """The tap reads of the tiled resampler on their own, in four forms (`mv_debug_lds_tap_reads` of the
    instrumented twin of the library, csrc/roi_resample.hip): clocks of a compute unit per voxel-wavefront."""
    import ctypes
    from medvision_amd import build
    raw = ctypes.CDLL(build.TIMELINE_LIB_PATH)
    fn = raw.mv_debug_lds_tap_reads
    fn.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.POINTER(ctypes.c_float), ctypes.c_void_p]
    props = torch.cuda.get_device_properties(0)
    cus, mhz = props.multi_processor_count, 1970.0   # (clocks at the shader clock that the profiles' counters showed: 1.97 GHz)
    out = torch.zeros(1024 * cus, dtype=torch.int32, device="cuda:0")
    torch.cuda.synchronize()
    names = ["eight 2-byte reads", "four ds_read2_b32", "four ds_read_b64 at 4-byte alignment",
             "four aligned dword reads (as from a shifted second copy)"]
    iters, rows = 400, []
    for form, name in enumerate(names):
        best = None
        for rep in range(4):
            ms = ctypes.c_float(0)
            rc = fn(form, iters, 20.0, ctypes.c_void_p(out.data_ptr()), ctypes.byref(ms), None)
            if rc != 0:
                sys.exit("mv_debug_lds_tap_reads failed: %d" % rc)
            best = ms.value if best is None or ms.value < best else best
        # a compute unit runs two workgroups of eight wavefronts, each wavefront iters x 8 voxels
        per = best * 1e-3 / (iters * 8 * 8 * 2)
        rows.append({"form": name, "ms": round(best, 4), "ns_per_voxel_wavefront": round(per * 1e9, 2),
                     "clocks_per_voxel_wavefront": round(per * mhz * 1e6, 1)})
    print(json.dumps({"lds_tap_reads": rows, "clock_mhz": mhz, "compute_units": cus}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--copies", type=int, default=16)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-dcn", action="store_true", help="skip the DCN leg")
    ap.add_argument("--no-next", action="store_true", help="skip the timings of the neighbouring operators")
    ap.add_argument("--no-configs", action="store_true", help="skip configs 1, 2-backward, 3 and 5")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="wall time spent on the CPU oracle")
    ap.add_argument("--timeline", action="store_true",
                    help="only print the in-kernel phase times of the tiled resampler (instrumented library)")
    ap.add_argument("--lds-taps", action="store_true",
                    help="only time the resampler's LDS tap reads on their own, in four forms (instrumented library)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a device copy of 4*128^3 fp16 elements (counter calibration)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    from medvision_amd import _lib
    if args.timeline:
        resample_timeline(args)
        return
    if args.lds_taps:
        lds_tap_reads(args)
        return
    _lib.load()
    if args.copy_calibration:
        copy_calibration(args)
        return

    a16 = bench_affine(args, torch.float16)
    a32 = bench_affine(args, torch.float32)
    line = {
        "metric": "RoIAlignRotated3D output throughput (fp16 [4,1,128^3] -> 128^3, sr=1)",
        "value": round(a16["gvox_s"], 3), "unit": "Gvox/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(a16["ms"], 6), "wall_ms_per_step": round(a16["wall_ms"], 6),
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "BASELINE config 2: RoIAlignRotated3D as RandomAffine resampling, "
                               "volume fp16 [4,1,128,128,128] N(0,1), one full-volume roi per sample, "
                               "angles U(+-30deg), scale U(0.8,1.2), shift +-10 vox, out 128^3, "
                               "sampling_ratio 1, aligned, order 1",
                   "buffer_sets": args.copies, "storage": "f16",
                   "arithmetic": "f32 interpolation and per-voxel coordinates, f64 roi geometry"},
        "roofline": {"bound": "hbm", "achieved": round(a16["gbps"], 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(a16["gbps"] / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "roi_resample_kernel", "algorithmic_bytes_per_launch": a16["alg_bytes"],
                     "avg_launch_us": round(a16["ms"] * 1e3, 3), "preheat_ms": a16["preheat_ms"],
                     "copy_ceiling_us": round(a16["copy_ms"] * 1e3, 3),
                     "frac_of_copy_ceiling": round(a16["copy_ms"] / a16["ms"], 4)},
        "fp32": {"gvox_s": round(a32["gvox_s"], 3), "gbps": round(a32["gbps"], 1),
                 "ms_per_step": round(a32["ms"], 6),
                 "frac": round(a32["gbps"] / HBM_PEAK_GBPS, 4)},
    }
    if not args.no_dcn:
        d = bench_dcn(args)
        line["dcn"] = {"metric": "DCNv2-3D forward (fp16 [2,32,48^3], 3^3, Cout 64)",
                       "value": round(d["tflops"], 3), "unit": "TFLOP/s",
                       "ms_per_step": round(d["ms"], 6), "wall_ms_per_step": round(d["wall_ms"], 6),
                       "forward_backward_ms": round(d["train_ms"], 4),
                       "roofline": {"bound": "mfma", "achieved": round(d["tflops"], 3),
                                    "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                    "frac": round(d["tflops"] / MFMA_F16_PEAK_TFLOPS, 5),
                                    "traffic": None, "flops_per_launch": d["flops"],
                                    "vector_blend_floor_us": round(d["blend_floor_us"], 1),
                                    "l1_gather_floor_us": round(d["gather_floor_us"], 1),
                                    "frac_of_gather_floor": round(d["gather_floor_us"] / (d["ms"] * 1e3), 4),
                                    "l2_gather_floor_us": round(d["l2_floor_us"], 1),
                                    "frac_of_l2_floor": round(d["l2_floor_us"] / (d["ms"] * 1e3), 4)}}
    if not args.no_configs:
        line["other_configs"] = bench_other_configs(args)
    if not args.no_next:
        line["next_rows"] = bench_next_rows(args)
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(args)
        line["cpu_reference_paths"] = cpu_reference_paths(args)
    traffic = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(traffic):   # HBM bytes per launch measured with rocprofv3 --pmc (see profiles/)
        measured = json.load(open(traffic))
        line["roofline"]["traffic"] = measured.get("roi_resample_fp16_config2")
        if "dcn" in line:
            line["dcn"]["roofline"]["traffic"] = measured.get("dcn_forward_fp16_config4")
    print(json.dumps(line))


if __name__ == "__main__":
    main()
