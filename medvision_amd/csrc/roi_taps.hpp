// Pieces shared by the RoIAlign kernels that keep a roi's geometry in scalar registers and work a
// sample's taps out per lane.
#pragma once
#include "common.hpp"
#include "roi_geometry.hpp"
#include "sampling.hpp"

namespace mv {

// The workgroup's geometry record as wave-uniform values: read once from LDS and moved to scalar
// registers, so that the sample loops below keep no per-lane copy of its ~30 doubles.
__device__ __forceinline__ double uniform_f64(double v) {
  return __hiloint2double(__builtin_amdgcn_readfirstlane(__double2hiint(v)), __builtin_amdgcn_readfirstlane(__double2loint(v)));
}
__device__ __forceinline__ RoiGeom uniform_geom(const RoiGeom &shared) {
  RoiGeom u;
#pragma unroll
  for (int i = 0; i < 9; i++) u.rot[i] = uniform_f64(shared.rot[i]);
#pragma unroll
  for (int a = 0; a < 3; a++) {
    u.centre[a] = uniform_f64(shared.centre[a]); u.start[a] = uniform_f64(shared.start[a]);
    u.bin[a] = uniform_f64(shared.bin[a]); u.sub[a] = uniform_f64(shared.sub[a]);
    u.grid[a] = __builtin_amdgcn_readfirstlane(shared.grid[a]);
  }
  u.batch = __builtin_amdgcn_readfirstlane(shared.batch);
  u.count = __builtin_amdgcn_readfirstlane(shared.count);
  return u;
}
// The taps of sub-sample `sub` (z, y, x order) of output cell `cell`.  Returns false for a void sample.
struct BoxTaps {
  int xi[2], yi[2], zi[2];
  float fx, fy, fz;
  int cell;
};
template <bool ROT>
__device__ __forceinline__ bool box_taps(const RoiGeom &g, const RoiProblem &p, unsigned cell, unsigned sub, BoxTaps &t) {
  const unsigned pw = cell % p.ow, t1 = cell / p.ow, ph = t1 % p.oh, pd = t1 / p.oh;
  const unsigned ix = sub % g.grid[0], t2 = sub / g.grid[0], iy = t2 % g.grid[1], iz = t2 / g.grid[1];
  const double x = local_coord(g, 0, pw, ix), y = local_coord(g, 1, ph, iy);
  const double z = p.ndim == 3 ? local_coord(g, 2, pd, iz) : 0.0;
  double rx = x, ry = y, rz = z;
  if (ROT) {
    rx = g.rot[0] * x + g.rot[1] * y + g.rot[2] * z + g.centre[0];
    ry = g.rot[3] * x + g.rot[4] * y + g.rot[5] * z + g.centre[1];
    rz = p.ndim == 3 ? g.rot[6] * x + g.rot[7] * y + g.rot[8] * z + g.centre[2] : 0.0;
  }
  t.cell = static_cast<int>(cell);
  return clamped_tap<float>(rz, p.D, t.zi[0], t.zi[1], t.fz, p.order) && clamped_tap<float>(ry, p.H, t.yi[0], t.yi[1], t.fy, p.order) &&
         clamped_tap<float>(rx, p.W, t.xi[0], t.xi[1], t.fx, p.order);
}

}  // namespace mv
