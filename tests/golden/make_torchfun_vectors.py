"""Writes tests/golden/torchfun_roi_align.npz: input / output vectors of the reference's pure-torch
RoIAlign (``medvision/ops/pytorch_ops/roi_align.py:9-105``) for the branches that no closed form in
tests/test_oracle_torchfun.py pins: ``aligned`` in {False, True} x ``order`` in {0, 1} x 2-D / 3-D.

Runs in the build container only: the reference file is loaded BY PATH (it depends on ``typing`` and
``torch`` alone; importing the package would pull in the CUDA extension).  The vectors travel, the
reference does not.  Usage:  python tests/golden/make_torchfun_vectors.py [/root/reference]
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def load_reference(root):
    path = os.path.join(root, "medvision", "ops", "pytorch_ops", "roi_align.py")
    spec = importlib.util.spec_from_file_location("reference_torchfun_roi_align", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.RoIAlign


def cases():
    g = torch.Generator().manual_seed(17)
    feat3 = torch.randn(2, 3, 6, 9, 11, generator=g)
    rois3 = torch.tensor([[1, 2.0, 1.0, 1.5, 9.0, 7.5, 5.0],
                          [0, 0.5, 3.0, 0.0, 10.0, 8.0, 4.5],
                          [1, -1.5, 2.0, 1.0, 6.0, 10.5, 7.0]])      # leaves the volume: zero padding
    feat2 = torch.randn(2, 4, 13, 10, generator=g)
    rois2 = torch.tensor([[0, 1.0, 2.0, 8.5, 11.0], [1, 0.0, 0.0, 9.0, 12.0], [1, 4.2, -2.0, 12.5, 6.3]])
    yield "3d", feat3, rois3, (3, 4, 5), 0.5
    yield "2d", feat2, rois2, (5, 4), 1.0


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    RoIAlign = load_reference(root)
    out = {}
    for name, feat, rois, size, scale in cases():
        out[name + "_feat"] = feat.numpy()
        out[name + "_rois"] = rois.numpy()
        out[name + "_size"] = np.array(size)
        out[name + "_scale"] = np.array(scale)
        for aligned in (False, True):
            for order in (0, 1):
                layer = RoIAlign(size, spatial_scale=scale)
                layer.aligned = aligned      # the attribute the class reads (no constructor argument)
                y = layer(feat, rois, order=order)
                out["%s_aligned%d_order%d" % (name, int(aligned), order)] = y.numpy()
    np.savez_compressed(os.path.join(HERE, "torchfun_roi_align.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
