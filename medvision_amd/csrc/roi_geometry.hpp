// RoI sample-grid geometry shared by the RoIAlign / RoIAlignRotated / affine kernels.
//
// A sample of output cell (pd,ph,pw), sub-sample (iz,iy,ix) sits at
//     local   p_a = start_a + cell_a * bin_a + (i_a + .5) * bin_a / grid_a
//     global  r   = Rot * p + centre
// with, for plain boxes (b, lo.., hi..)         start = lo*s, extent = max(hi*s - lo*s, 1),
//                                               Rot = I, centre = 0
//      for rotated boxes (b, c.., size.., ang)  start = -extent/2, centre = c*s - (aligned ? .5 : 0),
//                                               extent = size*s (clamped to >= 1 only if !aligned),
//                                               Rot = Rz(alpha) Ry(beta) Rx(gamma) (3-D) or R(theta)
// bin = extent / cells, grid = sampling_ratio > 0 ? sampling_ratio : ceil(extent / cells).
// Reference: csrc/cuda/roi_align_3d_cuda_kernel.cuh:28-69, roi_align_rotated_3d_cuda_kernel.cuh:32-103,
// roi_align_2d_cuda_kernel.cuh:26-58, roi_align_rotated_2d_cuda_kernel.cuh:40-74.
// 2-D problems run as depth-1 volumes with z pinned to 0 (both z taps collapse onto slice 0).
#pragma once
#include "common.hpp"

namespace mv {

struct RoiGeom {
  double rot[9];     // row-major, acts on (x, y, z)
  double centre[3];  // x, y, z
  double start[3];
  double bin[3];
  double sub[3];     // bin / grid: spacing of the sub-samples inside a cell
  int grid[3];
  int batch;         // -1 when the roi's batch index is outside [0, N)
  int count;         // max(gx*gy*gz, 1)
};

struct RoiProblem {
  int ndim, rotated;
  int N, C, D, H, W, R;
  int od, oh, ow;
  double scale;
  int sampling_ratio, aligned, order;
  unsigned per_roi;  // C*od*oh*ow
  unsigned chunks;   // blocks per roi
};

__host__ __device__ inline int roi_columns(int ndim, int rotated) {
  return ndim == 2 ? (rotated ? 6 : 5) : (rotated ? 10 : 7);
}

// sin and cos of a moderate angle (|x| up to ~1e5 rad) in fp64: two-constant Cody-Waite reduction
// to [-pi/4, pi/4] followed by the classic minimax polynomials (errors below 1 ulp).  Much less
// code and latency than the general library routine, which matters for the tiny set-up kernels.
__device__ inline void sincos_moderate(double x, double &s, double &c) {
  const double k = rint(x * 0.63661977236758134308);            // x * 2/pi
  double r = fma(-k, 1.57079632679489655800e+00, x);             // pi/2 high part
  r = fma(-k, 6.12323399573676603587e-17, r);                    // pi/2 low part
  const double z = r * r;
  double ps = fma(z, 1.58969099521155010221e-10, -2.50507602534068634195e-08);
  ps = fma(z, ps, 2.75573137070700676789e-06);
  ps = fma(z, ps, -1.98412698298579493134e-04);
  ps = fma(z, ps, 8.33333333332248946124e-03);
  ps = fma(z, ps, -1.66666666666666324348e-01);
  const double sr = fma(z * r, ps, r);
  double pc = fma(z, -1.13596475577881948265e-11, 2.08757232129817482790e-09);
  pc = fma(z, pc, -2.75573143513906633035e-07);
  pc = fma(z, pc, 2.48015872894767294178e-05);
  pc = fma(z, pc, -1.38888888888741095749e-03);
  pc = fma(z, pc, 4.16666666666666019037e-02);
  const double cr = fma(z * z, pc, fma(z, -0.5, 1.0));
  const int q = static_cast<int>(k) & 3;
  const double ss = (q & 1) ? cr : sr, cc = (q & 1) ? sr : cr;
  s = (q & 2) ? -ss : ss;
  c = ((q + 1) & 2) ? -cc : cc;
}

// Angles of a rotated roi (up to three); lanes 0..2 of a workgroup call this in parallel and
// publish sin / cos through LDS before one lane assembles the geometry.
template <typename RT>
__device__ inline void roi_trig(const RT *roi, const RoiProblem &p, int which, double &s, double &c) {
  s = 0.0; c = 1.0;
  if (!p.rotated) return;
  const int first = 1 + 2 * p.ndim, count = p.ndim == 3 ? 3 : 1;
  if (which < count) sincos_moderate(static_cast<double>(roi[first + which]), s, c);
}

// sn / cs: sines and cosines of (angle_x, angle_y, angle_z) in 3-D, (theta, -, -) in 2-D.
template <typename RT>
__device__ inline void build_geom(RoiGeom &g, const RT *roi, const RoiProblem &p,
                                  const double sn[3], const double cs[3]) {
  const int nd = p.ndim;
  const int cells[3] = {p.ow, p.oh, p.od};
  for (int i = 0; i < 9; i++) g.rot[i] = (i % 4 == 0) ? 1.0 : 0.0;
  for (int a = 0; a < 3; a++) {
    g.centre[a] = 0.0; g.start[a] = 0.0; g.bin[a] = 0.0; g.sub[a] = 0.0; g.grid[a] = 1;
  }
  const int b = static_cast<int>(roi[0]);
  g.batch = (b >= 0 && b < p.N) ? b : -1;
  const double s = p.scale;
#pragma unroll
  for (int a = 0; a < 3; a++) {
    if (a >= nd) continue;
    double ext;
    if (p.rotated) {
      ext = static_cast<double>(roi[1 + nd + a]) * s;
      if (!p.aligned) ext = fmax(ext, 1.0);
      g.centre[a] = static_cast<double>(roi[1 + a]) * s - (p.aligned ? 0.5 : 0.0);
      g.start[a] = -ext / 2.0;
    } else {
      const double lo = static_cast<double>(roi[1 + a]) * s;
      const double hi = static_cast<double>(roi[1 + nd + a]) * s;
      ext = fmax(hi - lo, 1.0);
      g.start[a] = lo;
    }
    g.bin[a] = ext / static_cast<double>(cells[a]);
    g.grid[a] = p.sampling_ratio > 0 ? p.sampling_ratio
                                     : static_cast<int>(ceil(ext / static_cast<double>(cells[a])));
    g.sub[a] = g.bin[a] / static_cast<double>(g.grid[a] > 0 ? g.grid[a] : 1);
  }
  if (p.rotated) {
    if (nd == 3) {
      const double sg = sn[0], cg = cs[0], sb = sn[1], cb = cs[1], sa = sn[2], ca = cs[2];
      g.rot[0] = ca * cb; g.rot[1] = ca * sb * sg - sa * cg; g.rot[2] = ca * sb * cg + sa * sg;
      g.rot[3] = sa * cb; g.rot[4] = sa * sb * sg + ca * cg; g.rot[5] = sa * sb * cg - ca * sg;
      g.rot[6] = -sb;     g.rot[7] = cb * sg;                g.rot[8] = cb * cg;
    } else {
      g.rot[0] = cs[0]; g.rot[1] = -sn[0];
      g.rot[3] = sn[0]; g.rot[4] = cs[0];
    }
  }
  const long cnt = static_cast<long>(g.grid[0]) * g.grid[1] * (nd == 3 ? g.grid[2] : 1);
  g.count = cnt > 1 ? static_cast<int>(cnt) : 1;
}

// Workgroup-wide geometry setup: lanes 0..2 evaluate the trigonometry in parallel, lane 0
// assembles.  Contains two barriers; every thread of the workgroup must call it.
template <typename RT>
__device__ inline void build_geom_block(RoiGeom &g, double *trig /* LDS, 6 doubles */,
                                        const RT *roi, const RoiProblem &p) {
  if (threadIdx.x < 3) roi_trig(roi, p, threadIdx.x, trig[threadIdx.x], trig[3 + threadIdx.x]);
  __syncthreads();
  if (threadIdx.x == 0) build_geom(g, roi, p, trig, trig + 3);
  __syncthreads();
}

// The reference evaluates (sub + .5) * bin / grid; here bin / grid is formed once per roi, which
// can differ from it in the last bit of an fp64 coordinate.
__device__ __forceinline__ double local_coord(const RoiGeom &g, int axis, int cell, int sub) {
  return g.start[axis] + cell * g.bin[axis] +
         static_cast<double>(static_cast<float>(sub) + .5f) * g.sub[axis];
}

}  // namespace mv
