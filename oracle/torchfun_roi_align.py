"""TEST AND CPU-BASELINE INFRASTRUCTURE ONLY: restatement of the reference's pure-torch RoIAlign.

Follows ``medvision/ops/pytorch_ops/roi_align.py:22-105`` (class ``RoIAlign``): fp32 only, one
sample per output cell (``sampling_ratio`` is ignored), boxes DIVIDED by ``spatial_scale``, a Python
loop over the rois, ``affine_grid`` + ``grid_sample`` with ``align_corners = aligned`` (False unless
the attribute is changed after construction), zero padding, chunks of 16 grids.  It is not the same
operator as the CUDA RoIAlign; it serves as the CPU timing baseline of benchmark config 1.

Per axis with input size S, n cells and box [x1, x2] (after the division) the sample of cell j is at
pixel  (x1+x2)/2 + ((2j+1)/n - 1) * (x2-x1)/2 * S/(S-1)          (aligned=False)
       (S-1)/S * [(x1+x2)/2 + (-1 + 2j/(n-1)) * (x2-x1)/2]        (aligned=True)
(tests/test_oracle_torchfun.py checks the first closed form).
"""
import torch
import torch.nn.functional as F


def torchfun_roi_align(feat_map, rois, output_size, spatial_scale=1.0, aligned=False, order=1,
                       max_parallel=16):
    """feat_map [N,C,(D,)H,W]; rois [R, 1 + 2*dim] = (batch, x1, y1, (z1,) x2, y2, (z2))."""
    dim = len(output_size)
    feat_map = feat_map.float()
    rois = rois.float()
    mode = {1: "bilinear", 0: "nearest"}[order]
    outs = []
    for roi in rois:
        b, box = int(roi[0]), roi[1:]
        feat = feat_map[b].unsqueeze(0)
        size = torch.tensor(feat.shape[2:][::-1], dtype=torch.float32)   # (W, H, D)
        lo, hi = box[:dim] / spatial_scale, box[dim:] / spatial_scale
        if aligned:
            scaling, shift = (hi - lo) / size, (hi + lo) / size - 1
        else:
            scaling, shift = (hi - lo) / (size - 1), (hi + lo + 1) / size - 1
        theta = torch.cat([torch.diag_embed(scaling), shift[:, None]], dim=-1)[None]
        grids = F.affine_grid(theta, [1, feat.shape[1], *output_size], align_corners=aligned)
        outs.append(torch.cat([F.grid_sample(feat, g, mode=mode, align_corners=aligned)
                               for g in torch.split(grids, max_parallel)]))
    return torch.cat(outs, dim=0)
