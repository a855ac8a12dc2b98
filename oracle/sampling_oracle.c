/*
 * TEST INFRASTRUCTURE ONLY -- fp64 CPU restatement of the reference's trilinear-sampling
 * operators.  Nothing in the shipped package may import, link or call this file; it exists so
 * that tests, the smoke check and the CPU-baseline leg of the benchmark have an independent
 * checker for the HIP kernels.
 *
 * Every routine follows one reference CUDA routine (cited as path:line under
 * /root/reference/medvision/csrc) evaluated with scalar_t = double.  The code is organised
 * differently from the reference (one axis-tap helper, one geometry record shared by the four
 * RoI flavours, a direct DCN contraction without a column matrix) but computes the same values
 * with the same operation order where the order matters for rounding.
 *
 * What pins each routine (see tests/test_oracle_*.py):
 *   sample_clamped (linear)   torch grid_sample(border, align_corners=True) x in-range mask,
 *                             brute-force edge table around -1, 0, S-1, S
 *   sample_clamped (nearest)  hand-enumerated 3^3 table incl. 0.5 ties (low index wins)
 *   roi_align_*               crop identities of the reference's own test script
 *                             (test/ops_test_RoIAlign.py:68,86,121,124,131), identity/shift/
 *                             quarter-turn identities, sr=g == mean of sub-bins, 2-D == textbook
 *                             Detectron RoIAlign restated with torch
 *   roi_align_*_backward      adjoint of the forward: <A x, y> == <x, A^T y>, torch autograd
 *   dcn3d_forward             F.conv3d at zero offsets, grid_sample(zeros, align_corners=True)
 *   dcn3d_backward            torch autograd through the grid_sample formulation
 *   deform3d_warp             grid_sample(border) on the open interval (-1, S)
 *   deform_conv               F.conv3d / F.conv2d at zero offsets (orders 0, 1, 3), a 1x1x1 conv
 *                             of the warp above, grid_sample(border) per tap x open-interval mask
 *   sample_cubic              textbook cubic Hermite spline with central-difference tangents on an
 *                             edge-padded copy (numpy), exact reproduction of quadratics in the
 *                             interior, node interpolation, partition of unity, brute-force
 *                             table around -1, 0, S-1, S
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------
 * Semantics "S": border-replicating tap on one axis.
 * cuda/interpolation_helpers_3d.h:12-48 (and :136-175 for nearest, 2-D twin
 * cuda/interpolation_helpers_2d.h:12-39): coordinates outside the CLOSED interval [-1, S]
 * give a zero sample; negatives snap to 0; a base index at or beyond S-1 collapses both taps
 * onto S-1 with zero fraction.
 * ---------------------------------------------------------------------------------------- */
typedef struct { int lo, hi; double frac; } tap1;

static int axis_tap(double v, int size, tap1 *t) {
  if (v < -1.0 || v > (double)size) return 0;
  if (v <= 0) v = 0;
  int base = (int)v;
  if (base >= size - 1) {
    t->lo = t->hi = size - 1;
    t->frac = 0.0;
  } else {
    t->lo = base;
    t->hi = base + 1;
    t->frac = v - base;
  }
  return 1;
}

/* nearest pick on one axis: the reference walks the 8 corners low-first and accepts the first
 * one whose three factors are all >= 0.5 (interpolation_helpers_3d.h:186-194), which per axis
 * means "low index when 1-frac >= 0.5, else high". */
static int nearest_pick(const tap1 *t) { return (1.0 - t->frac >= 0.5) ? t->lo : t->hi; }

/* Eight corner weights/indices of one sample; w[] ordered z-major (z0y0x0, z0y0x1, z0y1x0, ...)
 * like w1..w8 of interpolation_helpers_3d.h:62-63 / :123-124 / :254-262. Returns 0 when the
 * sample is outside [-1,S] on any axis (all weights zero, :80-85). */
static int corner_weights(int D, int H, int W, double z, double y, double x, int order,
                          long idx[8], double w[8]) {
  tap1 tz, ty, tx;
  /* the reference tests y, x, z in one expression; order is irrelevant for the result */
  if (!axis_tap(z, D, &tz) || !axis_tap(y, H, &ty) || !axis_tap(x, W, &tx)) return 0;
  const int zi[2] = {tz.lo, tz.hi}, yi[2] = {ty.lo, ty.hi}, xi[2] = {tx.lo, tx.hi};
  double wz[2], wy[2], wx[2];
  if (order == 0) {
    int pz = nearest_pick(&tz) == tz.lo ? 0 : 1;
    int py = nearest_pick(&ty) == ty.lo ? 0 : 1;
    int px = nearest_pick(&tx) == tx.lo ? 0 : 1;
    /* when lo == hi the pick is "lo" (frac = 0), matching the first-match rule */
    wz[0] = pz == 0; wz[1] = pz == 1;
    wy[0] = py == 0; wy[1] = py == 1;
    wx[0] = px == 0; wx[1] = px == 1;
  } else {
    wz[1] = tz.frac; wz[0] = 1. - tz.frac;
    wy[1] = ty.frac; wy[0] = 1. - ty.frac;
    wx[1] = tx.frac; wx[0] = 1. - tx.frac;
  }
  int n = 0;
  for (int a = 0; a < 2; a++)
    for (int b = 0; b < 2; b++)
      for (int c = 0; c < 2; c++, n++) {
        idx[n] = ((long)zi[a] * H + yi[b]) * W + xi[c];
        w[n] = wz[a] * wy[b] * wx[c];
      }
  return 1;
}

static double sample_clamped(const double *plane, int D, int H, int W, double z, double y,
                             double x, int order) {
  long idx[8];
  double w[8];
  if (!corner_weights(D, H, W, z, y, x, order, idx, w)) return 0.0;
  double v = 0.0;
  for (int n = 0; n < 8; n++) v += w[n] * plane[idx[n]];
  return v;
}

/* Order 3, one axis: cuda_aug/interpolation_helpers_3d.h:578-621 (2-D: interpolation_helpers_2d.h
 * :341-370).  Same void test and snap of negatives as above; base = (int)v WITHOUT the fold at the
 * upper border; the four indices base-1 .. base+2 are walked back into [0, size-1] one by one
 * (the while loops), i.e. clamped.  The 64 weights the reference spells out as polynomials
 * (:700-763) are the products of these per-axis Catmull-Rom weights: e.g. w000 starts with
 * -0.125 u^3 v^3 w^3 = (-0.5)^3, w111 ends with +1.  The reference rounds the fraction to float
 * (:589-591) even for double tensors; here it stays fp64 (difference <= 6e-8 relative). */
static int cubic_tap(double v, int size, int idx[4], double w[4]) {
  if (v < -1.0 || v > (double)size) return 0;
  if (v <= 0) v = 0;
  int base = (int)v;
  double u = v - base, u2 = u * u, u3 = u2 * u;
  w[0] = -0.5 * u3 + u2 - 0.5 * u;
  w[1] = 1.5 * u3 - 2.5 * u2 + 1.0;
  w[2] = -1.5 * u3 + 2.0 * u2 + 0.5 * u;
  w[3] = 0.5 * u3 - 0.5 * u2;
  for (int k = 0; k < 4; k++) {
    int i = base - 1 + k;
    idx[k] = i < 0 ? 0 : (i > size - 1 ? size - 1 : i);
  }
  return 1;
}

/* ndim 2: plane [H][W], z ignored (hermite_2d_interpolate); ndim 3: hermite_3d_interpolate. */
static double sample_cubic(const double *plane, int ndim, int D, int H, int W, double z, double y,
                           double x) {
  int zi[4] = {0, 0, 0, 0}, yi[4], xi[4];
  double wz[4] = {1, 0, 0, 0}, wy[4], wx[4];
  if (ndim == 3 && !cubic_tap(z, D, zi, wz)) return 0.0;
  if (!cubic_tap(y, H, yi, wy) || !cubic_tap(x, W, xi, wx)) return 0.0;
  double v = 0.0;
  for (int a = 0; a < (ndim == 3 ? 4 : 1); a++)
    for (int b = 0; b < 4; b++)
      for (int c = 0; c < 4; c++)
        v += wz[a] * wy[b] * wx[c] * plane[((long)zi[a] * H + yi[b]) * W + xi[c]];
  return v;
}

static double sample_any(const double *plane, int ndim, int D, int H, int W, double z, double y,
                         double x, int order) {
  return order == 3 ? sample_cubic(plane, ndim, D, H, W, z, y, x)
                    : sample_clamped(plane, D, H, W, z, y, x, order);
}

double orc_sample_cubic(const double *plane, int ndim, int D, int H, int W, double z, double y,
                        double x) {
  return sample_cubic(plane, ndim, D, H, W, z, y, x);
}

/* exported for the unit tests of S */
double orc_sample_clamped(const double *plane, int D, int H, int W, double z, double y, double x,
                          int order) {
  return sample_clamped(plane, D, H, W, z, y, x, order);
}

/* ------------------------------------------------------------------------------------------
 * RoI geometry "G".
 *   plain   3-D cuda/roi_align_3d_cuda_kernel.cuh:28-58, 2-D cuda/roi_align_2d_cuda_kernel.cuh:26-50
 *   rotated 3-D cuda/roi_align_rotated_3d_cuda_kernel.cuh:32-76,
 *           2-D cuda/roi_align_rotated_2d_cuda_kernel.cuh:40-64
 * A sample of output cell (pd,ph,pw), sub-sample (iz,iy,ix) sits at
 *   local  p_a = start_a + idx_a * bin_a + (i_a + .5) * bin_a / grid_a
 *   global r   = Rot * p + centre          (Rot = identity, centre = 0 for the plain flavour)
 * 2-D inputs are handled as depth-1 volumes with the z coordinate pinned to 0, which makes the
 * z taps collapse (lo = hi = 0, frac = 0) so that the 3-D formulas reduce to the 2-D ones.
 * ---------------------------------------------------------------------------------------- */
typedef struct {
  int batch;
  double rot[9];      /* row-major, acts on (x, y, z) */
  double centre[3];   /* x, y, z */
  double start[3];    /* x, y, z */
  double bin[3];      /* x, y, z */
  int grid[3];        /* x, y, z */
  double count;
} roi_geom;

static void geom_init(roi_geom *g) {
  memset(g, 0, sizeof *g);
  g->rot[0] = g->rot[4] = g->rot[8] = 1.0;
  g->grid[2] = 1;
}

static int grid_of(int sampling_ratio, double extent, int cells) {
  return sampling_ratio > 0 ? sampling_ratio : (int)ceil(extent / cells);
}

static void geom_plain(roi_geom *g, const double *roi, int ndim, double scale, int sr,
                       const int out[3] /* x,y,z cells */) {
  geom_init(g);
  g->batch = (int)roi[0];
  for (int a = 0; a < ndim; a++) {
    double lo = roi[1 + a] * scale, hi = roi[1 + ndim + a] * scale;
    double ext = fmax(hi - lo, 1.0);
    g->start[a] = lo;
    g->bin[a] = ext / out[a];
    g->grid[a] = grid_of(sr, ext, out[a]);
  }
  int cnt = g->grid[0] * g->grid[1] * (ndim == 3 ? g->grid[2] : 1);
  g->count = cnt > 1 ? cnt : 1;
}

static void geom_rotated(roi_geom *g, const double *roi, int ndim, double scale, int sr,
                         int aligned, const int out[3]) {
  geom_init(g);
  g->batch = (int)roi[0];
  double shift = aligned ? 0.5 : 0.0;
  for (int a = 0; a < ndim; a++) {
    double ext = roi[1 + ndim + a] * scale;
    if (!aligned) ext = fmax(ext, 1.0);
    g->centre[a] = roi[1 + a] * scale - shift;
    g->bin[a] = ext / out[a];
    g->grid[a] = grid_of(sr, ext, out[a]);
    g->start[a] = -ext / 2.0;
  }
  if (ndim == 3) {
    /* roi_align_rotated_3d_cuda_kernel.cuh:43-45,68-73,91-99: Rz(alpha) * Ry(beta) * Rx(gamma) */
    double cg = cos(roi[7]), sg = sin(roi[7]);
    double cb = cos(roi[8]), sb = sin(roi[8]);
    double ca = cos(roi[9]), sa = sin(roi[9]);
    g->rot[0] = ca * cb; g->rot[1] = ca * sb * sg - sa * cg; g->rot[2] = ca * sb * cg + sa * sg;
    g->rot[3] = sa * cb; g->rot[4] = sa * sb * sg + ca * cg; g->rot[5] = sa * sb * cg - ca * sg;
    g->rot[6] = -sb;     g->rot[7] = cb * sg;                g->rot[8] = cb * cg;
  } else {
    /* roi_align_rotated_2d_cuda_kernel.cuh:59-60,73-74 */
    double c = cos(roi[5]), s = sin(roi[5]);
    g->rot[0] = c; g->rot[1] = -s;
    g->rot[3] = s; g->rot[4] = c;
  }
  int cnt = g->grid[0] * g->grid[1] * (ndim == 3 ? g->grid[2] : 1);
  g->count = cnt > 1 ? cnt : 1;
}

static double local_coord(const roi_geom *g, int axis, int cell, int sub) {
  /* "start + p*bin + (i + .5f) * bin / grid", left to right as in the reference */
  return g->start[axis] + cell * g->bin[axis] +
         (double)((float)sub + .5f) * g->bin[axis] / (double)g->grid[axis];
}

static void to_global(const roi_geom *g, int ndim, double x, double y, double z, double r[3]) {
  const double *m = g->rot;
  if (ndim == 3) {
    r[0] = m[0] * x + m[1] * y + m[2] * z + g->centre[0];
    r[1] = m[3] * x + m[4] * y + m[5] * z + g->centre[1];
    r[2] = m[6] * x + m[7] * y + m[8] * z + g->centre[2];
  } else {
    r[0] = x * m[0] + y * m[1] + g->centre[0];
    r[1] = x * m[3] + y * m[4] + g->centre[1];
    r[2] = 0.0;
  }
}

static int roi_cols(int ndim, int rotated) {
  return ndim == 2 ? (rotated ? 6 : 5) : (rotated ? 10 : 7);
}

/* Forward of all four RoI flavours (order 0 / 1) and of the affine engine (also order 3:
 * cuda_aug/affine_3d_cuda_kernel.cuh:104-112, whose geometry is the rotated one).
 * feat [N,C,D,H,W] (D = 1 for 2-D), rois [R, 5|7|6|10], out [R,C,od,oh,ow].
 * roi_align_{2,3}d_forward_cuda_kernel, roi_align_rotated_{2,3}d_forward_cuda_kernel. */
void orc_roi_align_forward(const double *feat, const double *rois, double *out, int ndim,
                           int rotated, int N, int C, int D, int H, int W, int R, int od, int oh,
                           int ow, double scale, int sr, int aligned, int order) {
  (void)N;
  const int cols = roi_cols(ndim, rotated);
  const int cells[3] = {ow, oh, od};
  const long plane = (long)D * H * W, oplane = (long)od * oh * ow;
#pragma omp parallel for collapse(2) schedule(dynamic)
  for (int n = 0; n < R; n++)
    for (int c = 0; c < C; c++) {
      roi_geom g;
      if (rotated) geom_rotated(&g, rois + (long)n * cols, ndim, scale, sr, aligned, cells);
      else geom_plain(&g, rois + (long)n * cols, ndim, scale, sr, cells);
      const double *src = feat + ((long)g.batch * C + c) * plane;
      double *dst = out + ((long)n * C + c) * oplane;
      const int gz = ndim == 3 ? g.grid[2] : 1;
      for (int pd = 0; pd < od; pd++)
        for (int ph = 0; ph < oh; ph++)
          for (int pw = 0; pw < ow; pw++) {
            double acc = 0.0;
            for (int iz = 0; iz < gz; iz++) {
              double z = ndim == 3 ? local_coord(&g, 2, pd, iz) : 0.0;
              for (int iy = 0; iy < g.grid[1]; iy++) {
                double y = local_coord(&g, 1, ph, iy);
                for (int ix = 0; ix < g.grid[0]; ix++) {
                  double x = local_coord(&g, 0, pw, ix);
                  double r[3];
                  to_global(&g, ndim, x, y, z, r);
                  acc += sample_any(src, ndim, D, H, W, r[2], r[1], r[0], order);
                }
              }
            }
            dst[((long)pd * oh + ph) * ow + pw] = acc / g.count;
          }
    }
}

/* How far the samples of each output cell are from a DECISION of the order-0 (nearest) sampler:
 * a coordinate at exactly -1 or S (value or void, interpolation_helpers_3d.h:136) or a fraction of
 * exactly 0.5 (low or high neighbour, :186-194).  out [R,od,oh,ow] receives the smallest such
 * distance over the cell's samples and axes, in voxels; a sample that is void by more than the
 * distance on one axis does not count on the others.  Tests use it to tell a legitimate
 * difference (arithmetic of different precision picks the other side of a tie) from a wrong
 * voxel.  Same geometry code as the forward above. */
static double axis_margin(double v, int size) {
  double m = fmin(fabs(v + 1.0), fabs(v - (double)size));
  if (v < -1.0 || v > (double)size) return -m;          /* outside: negative distance */
  if (v <= 0) v = 0;
  int base = (int)v;
  if (base < size - 1) m = fmin(m, fabs((v - base) - 0.5));
  return m;
}

void orc_roi_decision_margin(const double *rois, double *out, int ndim, int rotated, int D, int H,
                             int W, int R, int od, int oh, int ow, double scale, int sr,
                             int aligned) {
  const int cols = roi_cols(ndim, rotated);
  const int cells[3] = {ow, oh, od};
  const int size[3] = {W, H, D};
  const long oplane = (long)od * oh * ow;
#pragma omp parallel for schedule(dynamic)
  for (int n = 0; n < R; n++) {
    roi_geom g;
    if (rotated) geom_rotated(&g, rois + (long)n * cols, ndim, scale, sr, aligned, cells);
    else geom_plain(&g, rois + (long)n * cols, ndim, scale, sr, cells);
    const int gz = ndim == 3 ? g.grid[2] : 1;
    for (int pd = 0; pd < od; pd++)
      for (int ph = 0; ph < oh; ph++)
        for (int pw = 0; pw < ow; pw++) {
          double best = 1e300;
          for (int iz = 0; iz < gz; iz++) {
            double z = ndim == 3 ? local_coord(&g, 2, pd, iz) : 0.0;
            for (int iy = 0; iy < g.grid[1]; iy++) {
              double y = local_coord(&g, 1, ph, iy);
              for (int ix = 0; ix < g.grid[0]; ix++) {
                double x = local_coord(&g, 0, pw, ix);
                double r[3];
                to_global(&g, ndim, x, y, z, r);
                double inside = 1e300, outside = 0.0;
                for (int a = 0; a < ndim; a++) {
                  double m = axis_margin(r[a], size[a]);
                  if (m < 0) outside = fmax(outside, -m);
                  else inside = fmin(inside, m);
                }
                best = fmin(best, outside > 0 ? outside : inside);
              }
            }
          }
          out[(long)n * oplane + ((long)pd * oh + ph) * ow + pw] = best;
        }
  }
}

/* Backward (adjoint) of the above: grad_in [N,C,D,H,W] is ACCUMULATED into, as the reference
 * kernels do with atomicAdd on a caller-zeroed buffer.
 * roi_align_3d_backward_cuda_kernel (cuda/roi_align_3d_cuda_kernel.cuh:90-202) and twins. */
void orc_roi_align_backward(const double *grad_out, const double *rois, double *grad_in, int ndim,
                            int rotated, int N, int C, int D, int H, int W, int R, int od, int oh,
                            int ow, double scale, int sr, int aligned, int order) {
  (void)N;
  const int cols = roi_cols(ndim, rotated);
  const int cells[3] = {ow, oh, od};
  const long plane = (long)D * H * W, oplane = (long)od * oh * ow;
#pragma omp parallel for schedule(dynamic)
  for (int c = 0; c < C; c++)
    for (int n = 0; n < R; n++) {
      roi_geom g;
      if (rotated) geom_rotated(&g, rois + (long)n * cols, ndim, scale, sr, aligned, cells);
      else geom_plain(&g, rois + (long)n * cols, ndim, scale, sr, cells);
      double *dst = grad_in + ((long)g.batch * C + c) * plane;
      const double *src = grad_out + ((long)n * C + c) * oplane;
      const int gz = ndim == 3 ? g.grid[2] : 1;
      for (int pd = 0; pd < od; pd++)
        for (int ph = 0; ph < oh; ph++)
          for (int pw = 0; pw < ow; pw++) {
            const double top = src[((long)pd * oh + ph) * ow + pw];
            for (int iz = 0; iz < gz; iz++) {
              double z = ndim == 3 ? local_coord(&g, 2, pd, iz) : 0.0;
              for (int iy = 0; iy < g.grid[1]; iy++) {
                double y = local_coord(&g, 1, ph, iy);
                for (int ix = 0; ix < g.grid[0]; ix++) {
                  double x = local_coord(&g, 0, pw, ix);
                  double r[3], w[8];
                  long idx[8];
                  to_global(&g, ndim, x, y, z, r);
                  if (!corner_weights(D, H, W, r[2], r[1], r[0], order, idx, w)) continue;
                  for (int k = 0; k < 8; k++) dst[idx[k]] += top * w[k] / g.count;
                }
              }
            }
          }
    }
}

/* ------------------------------------------------------------------------------------------
 * Deformable convolution 3-D (v1 when mask == NULL, v2 otherwise).
 * Sampling "Z": zero-padded trilinear, cuda/modulated_deform_conv_3d_cuda_kernel.cuh:9-54, gated
 * by the OPEN interval -1 < p < S (:240).  Geometry and channel conventions :201-235:
 *   p = q*stride - pad + tap*dil + off[b, dgi*3K + 3k + {0:d,1:h,2:w}, q],  k = (i*kh + j)*kw + kk
 *   col[c*K + k, q] = mask[b, dgi*K + k, q] * Z(x[b,c], p),   dgi = c / (Cin/dg)
 *   y[b,o,q] = sum_{c in group(o), k} Wt[o, c_local, k] * col[c*K+k, q] + bias[o]
 * (host: cuda/modulated_deform_conv_3d_cuda.cu:184-239; v1 cuda/deform_conv_3d_cuda.cu:168-214).
 * ---------------------------------------------------------------------------------------- */
typedef struct { int ok; long idx[8]; double w[8]; int inb[8]; double fd, fh, fw; } ztap;

static void zero_pad_taps(int D, int H, int W, double d, double h, double w, ztap *t) {
  t->ok = (d > -1 && h > -1 && w > -1 && d < D && h < H && w < W);
  if (!t->ok) return;
  int d0 = (int)floor(d), h0 = (int)floor(h), w0 = (int)floor(w);
  double ld = d - d0, lh = h - h0, lw = w - w0;
  t->fd = ld; t->fh = lh; t->fw = lw;
  int n = 0;
  for (int a = 0; a < 2; a++)
    for (int b = 0; b < 2; b++)
      for (int c = 0; c < 2; c++, n++) {
        int zd = d0 + a, zh = h0 + b, zw = w0 + c;
        t->inb[n] = zd >= 0 && zd <= D - 1 && zh >= 0 && zh <= H - 1 && zw >= 0 && zw <= W - 1;
        t->idx[n] = t->inb[n] ? ((long)zd * H + zh) * W + zw : 0;
        t->w[n] = (a ? ld : 1 - ld) * (b ? lh : 1 - lh) * (c ? lw : 1 - lw);
      }
}

static double zsample(const double *plane, const ztap *t) {
  if (!t->ok) return 0.0;
  double v = 0.0;
  for (int n = 0; n < 8; n++)
    if (t->inb[n]) v += t->w[n] * plane[t->idx[n]];
  return v;
}

/* d Z / d p_axis (axis 0:d 1:h 2:w): get_coordinate_weight, :94-172 -- the factor of the
 * differentiated axis is replaced by -1 (low corner) / +1 (high corner). */
static double zsample_grad(const double *plane, const ztap *t, int axis) {
  if (!t->ok) return 0.0;
  double v = 0.0;
  int n = 0;
  for (int a = 0; a < 2; a++)
    for (int b = 0; b < 2; b++)
      for (int c = 0; c < 2; c++, n++) {
        if (!t->inb[n]) continue;
        double wd = a ? t->fd : 1 - t->fd, wh = b ? t->fh : 1 - t->fh, ww = c ? t->fw : 1 - t->fw;
        if (axis == 0) wd = a ? 1 : -1;
        if (axis == 1) wh = b ? 1 : -1;
        if (axis == 2) ww = c ? 1 : -1;
        v += wd * wh * ww * plane[t->idx[n]];
      }
  return v;
}

typedef struct {
  int B, Cin, D, H, W, Cout, kd, kh, kw, sd, sh, sw, pd, ph, pw, dd, dh, dw, groups, dg;
  int nd; /* offset components per tap: 3 = (d,h,w) volumes; 2 = (h,w) images, which are depth-1
           * volumes with kd = 1, pad_d = 0 and p_d = 0 (cuda/modulated_deform_conv_2d_cuda_kernel.cuh
           * :143-176: offset channel 2k = h, 2k+1 = w of tap k = i*kw + j; bilinear with zero
           * padding :9-40, evaluated when -1 < p < size :167) */
  int Do, Ho, Wo, K;
} dcn_shape;
#define DCN_INTS 21

static void dcn_out_dims(dcn_shape *s) {
  s->Do = (s->D + 2 * s->pd - (s->dd * (s->kd - 1) + 1)) / s->sd + 1;
  s->Ho = (s->H + 2 * s->ph - (s->dh * (s->kh - 1) + 1)) / s->sh + 1;
  s->Wo = (s->W + 2 * s->pw - (s->dw * (s->kw - 1) + 1)) / s->sw + 1;
  s->K = s->kd * s->kh * s->kw;
}

static void dcn_taps(const dcn_shape *s, const double *off, int b, int dgi, int k, int od, int oh,
                     int ow, ztap *t) {
  const long Q = (long)s->Do * s->Ho * s->Wo, q = ((long)od * s->Ho + oh) * s->Wo + ow;
  const int nd = s->nd;
  const double *o = off + ((long)b * s->dg + dgi) * nd * s->K * Q;
  int i = k / (s->kh * s->kw), j = (k / s->kw) % s->kh, kk = k % s->kw;
  double pd = od * s->sd - s->pd + i * s->dd + (nd == 3 ? o[((long)nd * k + 0) * Q + q] : 0.0);
  double ph = oh * s->sh - s->ph + j * s->dh + o[((long)nd * k + nd - 2) * Q + q];
  double pw = ow * s->sw - s->pw + kk * s->dw + o[((long)nd * k + nd - 1) * Q + q];
  zero_pad_taps(s->D, s->H, s->W, pd, ph, pw, t);
}

void orc_dcn3d_out_dims(const int *p, int *dims) {
  dcn_shape s;
  memcpy(&s, p, DCN_INTS * sizeof(int));
  dcn_out_dims(&s);
  dims[0] = s.Do; dims[1] = s.Ho; dims[2] = s.Wo;
}

/* p: the 21 ints of dcn_shape in declaration order.  mask, bias may be NULL. */
void orc_dcn3d_forward(const double *x, const double *off, const double *mask, const double *wt,
                       const double *bias, double *y, const int *p) {
  dcn_shape s;
  memcpy(&s, p, DCN_INTS * sizeof(int));
  dcn_out_dims(&s);
  const long Q = (long)s.Do * s.Ho * s.Wo, P = (long)s.D * s.H * s.W;
  const int cpg = s.Cin / s.groups, opg = s.Cout / s.groups, cpd = s.Cin / s.dg;
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < s.B; b++)
    for (long q = 0; q < Q; q++) {
      int ow = q % s.Wo, oh = (q / s.Wo) % s.Ho, od = q / ((long)s.Wo * s.Ho);
      double *acc = (double *)calloc(s.Cout, sizeof(double));
      for (int dgi = 0; dgi < s.dg; dgi++)
        for (int k = 0; k < s.K; k++) {
          ztap t;
          dcn_taps(&s, off, b, dgi, k, od, oh, ow, &t);
          double m = mask ? mask[(((long)b * s.dg + dgi) * s.K + k) * Q + q] : 1.0;
          for (int c = dgi * cpd; c < (dgi + 1) * cpd; c++) {
            double col = zsample(x + ((long)b * s.Cin + c) * P, &t) * m;
            int grp = c / cpg, cl = c % cpg;
            for (int o = grp * opg; o < (grp + 1) * opg; o++)
              acc[o] += wt[((long)o * cpg + cl) * s.K + k] * col;
          }
        }
      for (int o = 0; o < s.Cout; o++)
        y[((long)b * s.Cout + o) * Q + q] = acc[o] + (bias ? bias[o] : 0.0);
      free(acc);
    }
}

/* Analytic gradients of the forward above (what DCNv1-3D implements,
 * cuda/deform_conv_3d_cuda_kernel.cuh:256-410 + cuda/deform_conv_3d_cuda.cu:305-370, and what the
 * v2-3D code intends; its truncated col2im launch, cuda/modulated_deform_conv_3d_cuda.cu:64, and
 * the 2-D "%2, /2" mask index, cuda/modulated_deform_conv_3d_cuda_kernel.cuh:410-411, are
 * reference defects that are NOT restated).
 *   gcol[c,k,q] = sum_o Wt[o,c_l,k] * gy[b,o,q]
 *   gx  += gcol * m * corner weight          (get_gradient_weight, :57-91)
 *   goff[3k+a] = sum_c gcol * m * dZ/dp_a    (get_coordinate_weight, :94-172)
 *   gm[k]   = sum_c gcol * Z(x, p)           (:400)
 *   gW[o,c_l,k] = sum_{b,q} gy * col ; gbias[o] = sum_{b,q} gy
 * All outputs are accumulated into (callers pass zero-filled buffers). gmask/gbias may be NULL. */
void orc_dcn3d_backward(const double *x, const double *off, const double *mask, const double *wt,
                        const double *gy, double *gx, double *goff, double *gmask, double *gw,
                        double *gbias, const int *p) {
  dcn_shape s;
  memcpy(&s, p, DCN_INTS * sizeof(int));
  dcn_out_dims(&s);
  const long Q = (long)s.Do * s.Ho * s.Wo, P = (long)s.D * s.H * s.W;
  const int cpg = s.Cin / s.groups, opg = s.Cout / s.groups, cpd = s.Cin / s.dg;
  /* pass A: per input channel (no two threads share gx planes or gW columns) */
#pragma omp parallel for schedule(dynamic)
  for (int c = 0; c < s.Cin; c++) {
    int grp = c / cpg, cl = c % cpg, dgi = c / cpd;
    for (int b = 0; b < s.B; b++)
      for (long q = 0; q < Q; q++) {
        int ow = q % s.Wo, oh = (q / s.Wo) % s.Ho, od = q / ((long)s.Wo * s.Ho);
        for (int k = 0; k < s.K; k++) {
          ztap t;
          dcn_taps(&s, off, b, dgi, k, od, oh, ow, &t);
          if (!t.ok) continue;
          double m = mask ? mask[(((long)b * s.dg + dgi) * s.K + k) * Q + q] : 1.0;
          const double *plane = x + ((long)b * s.Cin + c) * P;
          double col = zsample(plane, &t) * m, gcol = 0.0;
          for (int o = grp * opg; o < (grp + 1) * opg; o++) {
            double g = gy[((long)b * s.Cout + o) * Q + q];
            gcol += wt[((long)o * cpg + cl) * s.K + k] * g;
            gw[((long)o * cpg + cl) * s.K + k] += g * col;
          }
          double *gplane = gx + ((long)b * s.Cin + c) * P;
          for (int n = 0; n < 8; n++)
            if (t.inb[n]) gplane[t.idx[n]] += t.w[n] * gcol * m;
        }
      }
  }
  /* pass B: per output position (offset / mask gradients sum over the channels of a
   * deformable group) */
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < s.B; b++)
    for (long q = 0; q < Q; q++) {
      int ow = q % s.Wo, oh = (q / s.Wo) % s.Ho, od = q / ((long)s.Wo * s.Ho);
      for (int dgi = 0; dgi < s.dg; dgi++)
        for (int k = 0; k < s.K; k++) {
          ztap t;
          dcn_taps(&s, off, b, dgi, k, od, oh, ow, &t);
          if (!t.ok) continue;
          double m = mask ? mask[(((long)b * s.dg + dgi) * s.K + k) * Q + q] : 1.0;
          double go[3] = {0, 0, 0}, gm = 0;
          for (int c = dgi * cpd; c < (dgi + 1) * cpd; c++) {
            int grp = c / cpg, cl = c % cpg;
            double gcol = 0.0;
            for (int o = grp * opg; o < (grp + 1) * opg; o++)
              gcol += wt[((long)o * cpg + cl) * s.K + k] * gy[((long)b * s.Cout + o) * Q + q];
            const double *plane = x + ((long)b * s.Cin + c) * P;
            for (int a = 0; a < 3; a++) go[a] += zsample_grad(plane, &t, a) * gcol * m;
            gm += gcol * zsample(plane, &t);
          }
          double *o = goff + ((long)b * s.dg + dgi) * s.nd * s.K * Q;
          for (int a = 3 - s.nd; a < 3; a++) o[((long)s.nd * k + a - (3 - s.nd)) * Q + q] += go[a];
          if (gmask) gmask[(((long)b * s.dg + dgi) * s.K + k) * Q + q] += gm;
        }
    }
  if (gbias)
    for (int b = 0; b < s.B; b++)
      for (int o = 0; o < s.Cout; o++) {
        double acc = 0;
        for (long q = 0; q < Q; q++) acc += gy[((long)b * s.Cout + o) * Q + q];
        gbias[o] += acc;
      }
}

/* ------------------------------------------------------------------------------------------
 * Displacement-field warp: the 1x1x1, identity-weight use of the augmentation DCN
 * (ops/cuda_fun_tools.py:134-167 -> cuda_aug/deform_3d_cuda_kernel.cuh:58-85):
 *   out[b,c,q] = S(img[b,c], q + off[b,{0:d,1:h,2:w},q])  if  -1 < p < size on all axes, else 0
 * with S the clamped sampler above (order 0 or 1) or the cubic one (order 3, :80-81).  2-D images are depth-1 volumes with a
 * 2-channel offset (0:h, 1:w), cuda_aug/deform_2d_cuda_kernel.cuh.
 * ---------------------------------------------------------------------------------------- */
void orc_deform_warp(const double *img, const double *off, double *out, int ndim, int B, int C,
                     int D, int H, int W, int order) {
  const long P = (long)D * H * W;
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < B; b++)
    for (long q = 0; q < P; q++) {
      int w = q % W, h = (q / W) % H, d = q / ((long)W * H);
      const double *o = off + (long)b * ndim * P;
      double pd = ndim == 3 ? d + o[q] : 0.0;
      double ph = h + o[(ndim - 2) * P + q];
      double pw = w + o[(ndim - 1) * P + q];
      int ok = ph > -1 && pw > -1 && ph < H && pw < W && (ndim == 2 || (pd > -1 && pd < D));
      for (int c = 0; c < C; c++)
        out[((long)b * C + c) * P + q] =
            ok ? sample_any(img + ((long)b * C + c) * P, ndim, D, H, W, pd, ph, pw, order) : 0.0;
    }
}

/* ------------------------------------------------------------------------------------------
 * General augmentation DCN: the v1 forward with the CLAMPED samplers, for any kernel, stride,
 * padding, dilation, groups and weight (cuda_aug/deform_3d_cuda_kernel.cuh:8-89: column value
 * = S(x[b,c], p) when -1 < p < size on every axis, else 0, S = nearest / linear / Hermite by
 * `order`, offset channel nd*k + axis of tap k as in the DCN; cuda_aug/deform_3d_cuda.cu:43-152:
 * y = bias + W . columns per group; images: cuda_aug/deform_2d_cuda_kernel.cuh, offset channels
 * 2k = h, 2k+1 = w).  p: the 21 ints of dcn_shape.  bias may be NULL.
 * ---------------------------------------------------------------------------------------- */
void orc_deform_conv(const double *x, const double *off, const double *wt, const double *bias,
                     double *y, const int *p, int order) {
  dcn_shape s;
  memcpy(&s, p, DCN_INTS * sizeof(int));
  dcn_out_dims(&s);
  const long Q = (long)s.Do * s.Ho * s.Wo, P = (long)s.D * s.H * s.W;
  const int cpg = s.Cin / s.groups, opg = s.Cout / s.groups, cpd = s.Cin / s.dg, nd = s.nd;
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < s.B; b++)
    for (long q = 0; q < Q; q++) {
      int ow = q % s.Wo, oh = (q / s.Wo) % s.Ho, od = q / ((long)s.Wo * s.Ho);
      double *acc = (double *)calloc(s.Cout, sizeof(double));
      for (int dgi = 0; dgi < s.dg; dgi++)
        for (int k = 0; k < s.K; k++) {
          const double *o = off + ((long)b * s.dg + dgi) * nd * s.K * Q;
          int i = k / (s.kh * s.kw), j = (k / s.kw) % s.kh, kk = k % s.kw;
          double pd = od * s.sd - s.pd + i * s.dd + (nd == 3 ? o[((long)nd * k + 0) * Q + q] : 0.0);
          double ph = oh * s.sh - s.ph + j * s.dh + o[((long)nd * k + nd - 2) * Q + q];
          double pw = ow * s.sw - s.pw + kk * s.dw + o[((long)nd * k + nd - 1) * Q + q];
          int ok = ph > -1 && pw > -1 && ph < s.H && pw < s.W && (nd == 2 || (pd > -1 && pd < s.D));
          if (!ok) continue;
          for (int c = dgi * cpd; c < (dgi + 1) * cpd; c++) {
            double col = sample_any(x + ((long)b * s.Cin + c) * P, nd, s.D, s.H, s.W, pd, ph, pw, order);
            int grp = c / cpg, cl = c % cpg;
            for (int o2 = grp * opg; o2 < (grp + 1) * opg; o2++)
              acc[o2] += wt[((long)o2 * cpg + cl) * s.K + k] * col;
          }
        }
      for (int o2 = 0; o2 < s.Cout; o2++)
        y[((long)b * s.Cout + o2) * Q + q] = acc[o2] + (bias ? bias[o2] : 0.0);
      free(acc);
    }
}
