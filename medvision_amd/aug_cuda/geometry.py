"""RoI rows and box transforms of the GPU augmentation layer (numpy only, no device code).

All spatial augmentations of the reference's ``medvision/aug_cuda`` resample with ONE rotated roi
per sample: a window (start, end) of the image in (x, y[, z]) order, shrunk / grown by ``scales``,
moved by ``shifts`` (fractions of the window) and turned by ``rotate`` radians in the xy plane.
``window_rois`` builds those rows with the float32 arithmetic of the reference
(aug_spatial.py:304-318 RandomAffine, :1035-1050 CropRandomWithAffine, :82-92 Resize;
aug_cuda_batch/aug_spatial.py:423-434 for whole batches), ``map_boxes`` moves detection boxes
the same way (aug_spatial.py:381-455, :1103-1183) and ``clip_boxes`` is utils.py:117-139.
"""
import numpy as np


def _table(v, cols):
    """v as a float32 [rows, cols] table: scalars fill a row, vectors are one row."""
    a = np.asarray(v, dtype=np.float32)
    if a.ndim == 0:
        return np.full((1, cols), a, dtype=np.float32)
    return a.reshape(-1, cols)


def window_rois(dim, start_xyz, end_xyz, scales=1.0, shifts=0.0, rotate=0.0, index=None):
    """[n, 6] (2-D: b, cx, cy, w, h, angle) or [n, 10] (3-D: b, cx, cy, cz, w, h, d, 0, 0, angle)
    float32 rows.  Every argument is one value, one row, or n rows; ``index`` defaults to 0..n-1."""
    cols = {"start": dim, "end": dim, "scales": dim, "shifts": dim, "rotate": 1}
    tab = {k: _table(v, cols[k]) for k, v in (("start", start_xyz), ("end", end_xyz),
                                              ("scales", scales), ("shifts", shifts), ("rotate", rotate))}
    n = max([t.shape[0] for t in tab.values()] + ([len(index)] if index is not None else []))
    start, end, scales, shifts, rotate = [np.broadcast_to(tab[k], (n, cols[k])) for k in cols]
    centre = (start + end) / np.float32(2)
    extent = end - start
    rois = np.zeros((n, 2 * dim + (2 if dim == 2 else 4)), dtype=np.float32)
    rois[:, 0] = np.arange(n, dtype=np.float32) if index is None else np.asarray(index, dtype=np.float32)
    rois[:, 1:1 + dim] = centre - extent * shifts / scales
    rois[:, 1 + dim:1 + 2 * dim] = extent / scales
    rois[:, -1:] = rotate          # 3-D: the two leading angles (about x and y) stay 0
    return rois


def frame_rois(image_shape_zyx, n=1):
    """Rois that cover whole images of the given (d, h, w) / (h, w) shape, unrotated."""
    dim = len(image_shape_zyx)
    return window_rois(dim, [0.0] * dim, [float(s) for s in image_shape_zyx[::-1]], index=np.arange(n))


def clip_boxes(boxes, image_shape_zyx):
    """Clamp box corners into [0, size-1] and drop boxes that became empty on any axis.
    boxes [N, >= 2*dim] = (x1, y1[, z1], x2, y2[, z2], ...)."""
    boxes = np.array(boxes, dtype=np.float64, copy=True)
    if boxes.size == 0:
        return boxes
    dim = len(image_shape_zyx)
    top = np.array(list(image_shape_zyx[::-1]) * 2, dtype=np.float64) - 1
    boxes[:, :2 * dim] = np.clip(boxes[:, :2 * dim], 0, top)
    return boxes[np.all(boxes[:, dim:2 * dim] > boxes[:, :dim], axis=1)]


def map_boxes(dim, boxes, frame_xyz, scales, shifts, rotate, start_xyz=None):
    """Boxes of the source image expressed in the resampled output.

    A point p of the source lands at  s * (p + frame * shift / s - start) - frame / 2 * (s - 1);
    the rectangle spanned in the xy plane is then turned by -rotate about the output centre and
    replaced by its axis-aligned hull (z is untouched).  ``frame_xyz`` is the output size.
    """
    boxes = np.array(boxes, dtype=np.float64, copy=True)
    if boxes.size == 0:
        return boxes
    frame = np.asarray(frame_xyz, dtype=np.float64)
    s = np.broadcast_to(np.asarray(scales, dtype=np.float64), (dim,))
    t = np.broadcast_to(np.asarray(shifts, dtype=np.float64), (dim,))
    start = np.zeros(dim) if start_xyz is None else np.asarray(start_xyz, dtype=np.float64)
    for lo in (0, dim):
        boxes[:, lo:lo + dim] = s * (boxes[:, lo:lo + dim] + frame * t / s - start) - frame / 2 * (s - 1)
    angle = -float(np.asarray(rotate).reshape(-1)[0])
    cx, cy = 0.5 * frame[0], 0.5 * frame[1]
    xs = boxes[:, [0, dim, dim, 0]] - cx          # corners (x1,y1) (x2,y1) (x2,y2) (x1,y2)
    ys = boxes[:, [1, 1, dim + 1, dim + 1]] - cy
    xt = np.cos(angle) * xs - np.sin(angle) * ys + cx
    yt = np.sin(angle) * xs + np.cos(angle) * ys + cy
    boxes[:, 0], boxes[:, dim] = xt.min(1), xt.max(1)
    boxes[:, 1], boxes[:, dim + 1] = yt.min(1), yt.max(1)
    return boxes
