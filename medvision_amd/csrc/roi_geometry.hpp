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

template <typename RT>
__device__ inline void build_geom(RoiGeom &g, const RT *roi, const RoiProblem &p) {
  const int nd = p.ndim;
  const int cells[3] = {p.ow, p.oh, p.od};
  for (int i = 0; i < 9; i++) g.rot[i] = (i % 4 == 0) ? 1.0 : 0.0;
  for (int a = 0; a < 3; a++) {
    g.centre[a] = 0.0; g.start[a] = 0.0; g.bin[a] = 0.0; g.grid[a] = 1;
  }
  const int b = static_cast<int>(roi[0]);
  g.batch = (b >= 0 && b < p.N) ? b : -1;
  const double s = p.scale;
  for (int a = 0; a < nd; a++) {
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
  }
  if (p.rotated) {
    if (nd == 3) {
      double sg, cg, sb, cb, sa, ca;
      sincos(static_cast<double>(roi[7]), &sg, &cg);
      sincos(static_cast<double>(roi[8]), &sb, &cb);
      sincos(static_cast<double>(roi[9]), &sa, &ca);
      g.rot[0] = ca * cb; g.rot[1] = ca * sb * sg - sa * cg; g.rot[2] = ca * sb * cg + sa * sg;
      g.rot[3] = sa * cb; g.rot[4] = sa * sb * sg + ca * cg; g.rot[5] = sa * sb * cg - ca * sg;
      g.rot[6] = -sb;     g.rot[7] = cb * sg;                g.rot[8] = cb * cg;
    } else {
      double st, ct;
      sincos(static_cast<double>(roi[5]), &st, &ct);
      g.rot[0] = ct; g.rot[1] = -st;
      g.rot[3] = st; g.rot[4] = ct;
    }
  }
  const long cnt = static_cast<long>(g.grid[0]) * g.grid[1] * (nd == 3 ? g.grid[2] : 1);
  g.count = cnt > 1 ? static_cast<int>(cnt) : 1;
}

__device__ __forceinline__ double local_coord(const RoiGeom &g, int axis, int cell, int sub) {
  return g.start[axis] + cell * g.bin[axis] +
         static_cast<double>(static_cast<float>(sub) + .5f) * g.bin[axis] /
             static_cast<double>(g.grid[axis]);
}

}  // namespace mv
