"""The forward entry points inside a captured graph: no entry point allocates, synchronises or clears
memory with a memset, so a serving loop can record them once and replay.  Every replay is checked
against the eager result, with eager work and synchronisations between the replays."""
import pytest
import torch

import workloads as wl

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    import medvision_amd.ops as ops_
    from medvision_amd import _lib
    _lib.load()
    return ops_


def _replay_against_eager(make_inputs, run, replays=3):
    """`run(*inputs)` -> output; recorded once on static inputs, replayed with fresh contents."""
    static = [t.to(DEV) for t in make_inputs(0)]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):          # (the first call of an op may load code: outside the capture)
        run(*static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = run(*static)
    for r in range(1, replays + 1):
        fresh = [t.to(DEV) for t in make_inputs(r)]
        want = run(*fresh)                 # eager, between the replays
        torch.cuda.synchronize()
        for s, f in zip(static, fresh):
            s.copy_(f)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {r} differs from the eager call"


def test_resampler_in_a_graph(ops):
    def inputs(r):
        g = wl.gen(500 + r)
        return torch.randn(2, 1, 48, 48, 48, generator=g).half(), wl.affine_rois(g, 2, (48, 48, 48))
    _replay_against_eager(inputs, lambda vol, rois: ops.RoIAlignRotated((48, 48, 48), 1.0, 1)(vol, rois))
    _replay_against_eager(inputs, lambda vol, rois: ops.RoIAlignRotated((24, 24, 24), 1.0, 2)(vol, rois))


def test_detection_head_in_a_graph(ops):
    def inputs(r):
        g = wl.gen(510 + r)
        feat = torch.randn(2, 64, 12, 48, 48, generator=g).half()
        rois = wl.roi3d_detection(g, 600, 2, (192, 192, 48), (2.0, 48.0), log_uniform=True)
        return feat, rois
    _replay_against_eager(inputs, lambda feat, rois: ops.RoIAlign((7, 7, 7), 0.25, 2)(feat, rois))


def test_deformable_convolution_in_a_graph(ops):
    from medvision_amd.ops.modulated_deform_conv_3d import modulated_deform_conv

    def inputs(r):
        return [t for t in wl.dcn_inputs(wl.gen(520 + r), 2, 32, 64, (12, 12, 16), 3, 1, 1, torch.float16)]
    _replay_against_eager(inputs, lambda x, off, mask, w, b: modulated_deform_conv(x, off, mask, w, b, 1, 1, 1, 1, 1))
