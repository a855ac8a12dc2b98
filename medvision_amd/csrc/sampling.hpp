// Device-side samplers shared by the RoI, warp and DCN kernels.
//
// Coordinates are carried in fp64 (full-rate on CDNA and accurate enough that the position of a
// sample relative to the floor / 0.5-tie / [-1,S] discontinuities agrees with an fp64 evaluation);
// interpolation weights and sums use the arithmetic type A (fp32, or fp64 for double tensors).
#pragma once
#include "common.hpp"

namespace mv {

// Border-replicating tap on one axis (reference: csrc/cuda/interpolation_helpers_3d.h:12-48):
// outside the closed interval [-1, size] the sample is void; negatives snap to 0; a base index
// at or beyond size-1 collapses both taps onto size-1.
__device__ __forceinline__ bool clamped_tap64(double v, int size, int &lo, int &hi, double &frac) {
  if (v < -1.0 || v > static_cast<double>(size)) return false;
  v = v <= 0.0 ? 0.0 : v;
  const int base = static_cast<int>(v);
  if (base >= size - 1) {
    lo = hi = size - 1;
    frac = 0.0;
  } else {
    lo = base;
    hi = base + 1;
    frac = v - static_cast<double>(base);
  }
  return true;
}

// order 1: fraction rounded once to the arithmetic type A.  order 0: the fraction becomes 0 or 1;
// the pick "low index when 1 - frac >= 0.5" (csrc/cuda/interpolation_helpers_3d.h:186-194) is
// decided on the fp64 fraction so that coordinates a few ulp from a tie fall on the same side as
// in an fp64 evaluation.
template <typename A>
__device__ __forceinline__ bool clamped_tap(double v, int size, int &lo, int &hi, A &frac,
                                            int order = 1) {
  double f;
  if (!clamped_tap64(v, size, lo, hi, f)) return false;
  frac = order == 0 ? ((1.0 - f >= 0.5) ? A(0) : A(1)) : static_cast<A>(f);
  return true;
}

// Eight-corner description of one sample; `w` follows the z-major corner order
// (z0y0x0, z0y0x1, z0y1x0, ...).  For order 0 exactly one weight is 1: per axis the low index
// wins when 1 - frac >= 0.5 (csrc/cuda/interpolation_helpers_3d.h:186-194).
template <typename A> struct Corners {
  long idx[8];
  A w[8];
};

template <typename A>
__device__ __forceinline__ bool clamped_corners(int D, int H, int W, double z, double y, double x,
                                                int order, Corners<A> &c) {
  int z0, z1, y0, y1, x0, x1;
  A lz, ly, lx;
  if (!clamped_tap(z, D, z0, z1, lz, order) || !clamped_tap(y, H, y0, y1, ly, order) ||
      !clamped_tap(x, W, x0, x1, lx, order))
    return false;
  const A hz = A(1) - lz, hy = A(1) - ly, hx = A(1) - lx;
  const long r00 = (static_cast<long>(z0) * H + y0) * W, r01 = (static_cast<long>(z0) * H + y1) * W;
  const long r10 = (static_cast<long>(z1) * H + y0) * W, r11 = (static_cast<long>(z1) * H + y1) * W;
  c.idx[0] = r00 + x0; c.idx[1] = r00 + x1; c.idx[2] = r01 + x0; c.idx[3] = r01 + x1;
  c.idx[4] = r10 + x0; c.idx[5] = r10 + x1; c.idx[6] = r11 + x0; c.idx[7] = r11 + x1;
  c.w[0] = hz * hy * hx; c.w[1] = hz * hy * lx; c.w[2] = hz * ly * hx; c.w[3] = hz * ly * lx;
  c.w[4] = lz * hy * hx; c.w[5] = lz * hy * lx; c.w[6] = lz * ly * hx; c.w[7] = lz * ly * lx;
  return true;
}

template <typename T>
__device__ __forceinline__ typename Acc<T>::type sample_clamped(const T *plane, int D, int H,
                                                                int W, double z, double y,
                                                                double x, int order) {
  using A = typename Acc<T>::type;
  int z0, z1, y0, y1, x0, x1;
  A lz, ly, lx;
  if (!clamped_tap(z, D, z0, z1, lz, order) || !clamped_tap(y, H, y0, y1, ly, order) ||
      !clamped_tap(x, W, x0, x1, lx, order))
    return A(0);
  if (order == 0) {
    const int zi = lz == A(0) ? z0 : z1, yi = ly == A(0) ? y0 : y1, xi = lx == A(0) ? x0 : x1;
    return load(plane + (static_cast<long>(zi) * H + yi) * W + xi);
  }
  const A hz = A(1) - lz, hy = A(1) - ly, hx = A(1) - lx;
  const T *r00 = plane + (static_cast<long>(z0) * H + y0) * W;
  const T *r01 = plane + (static_cast<long>(z0) * H + y1) * W;
  if (D == 1) {
    // an image: the upper slice is the lower one with weight 0 (its four taps are not loaded), as in the
    // reference's bilinear 2-D kernels (csrc/cuda/interpolation_helpers_2d.h)
    const A v1 = load(r00 + x0), v2 = load(r00 + x1), v3 = load(r01 + x0), v4 = load(r01 + x1);
    return hy * (hx * v1 + lx * v2) + ly * (hx * v3 + lx * v4);
  }
  const T *r10 = plane + (static_cast<long>(z1) * H + y0) * W;
  const T *r11 = plane + (static_cast<long>(z1) * H + y1) * W;
  const A v1 = load(r00 + x0), v2 = load(r00 + x1), v3 = load(r01 + x0), v4 = load(r01 + x1);
  const A v5 = load(r10 + x0), v6 = load(r10 + x1), v7 = load(r11 + x0), v8 = load(r11 + x1);
  return hz * (hy * (hx * v1 + lx * v2) + ly * (hx * v3 + lx * v4)) +
         lz * (hy * (hx * v5 + lx * v6) + ly * (hx * v7 + lx * v8));
}

// Order 3: separable Catmull-Rom (cubic Hermite with central-difference tangents) over the 4 x 4
// (x 4) neighbourhood base-1 .. base+2 with every index clamped into the image
// (csrc/cuda_aug/interpolation_helpers_3d.h:571-792, 2-D twin interpolation_helpers_2d.h:335-423;
// the reference spells the 64 weights out as polynomials, which factor into these per-axis
// weights).  Same void region as the other orders (outside the closed interval [-1, size]) and
// negatives snap to 0, but the base index is NOT folded back at the upper border: between size-1
// and size the fraction keeps growing while the taps beyond the border repeat the last voxel.
template <typename A>
__device__ __forceinline__ bool cubic_tap(double v, int size, int idx[4], A w[4]) {
  if (v < -1.0 || v > static_cast<double>(size)) return false;
  v = v <= 0.0 ? 0.0 : v;
  const int base = static_cast<int>(v);
  const A u = static_cast<A>(v - static_cast<double>(base));
  const A u2 = u * u, u3 = u2 * u;
  w[0] = A(-0.5) * u3 + u2 - A(0.5) * u;
  w[1] = A(1.5) * u3 - A(2.5) * u2 + A(1);
  w[2] = A(-1.5) * u3 + A(2) * u2 + A(0.5) * u;
  w[3] = A(0.5) * u3 - A(0.5) * u2;
#pragma unroll
  for (int k = 0; k < 4; k++) idx[k] = min(max(base - 1 + k, 0), size - 1);
  return true;
}

// ndim == 2: the plane is [H][W] and z is ignored (one z tap of weight 1).
template <typename T>
__device__ __forceinline__ typename Acc<T>::type sample_cubic(const T *plane, int ndim, int D,
                                                              int H, int W, double z, double y,
                                                              double x) {
  using A = typename Acc<T>::type;
  int zi[4] = {0, 0, 0, 0}, yi[4], xi[4];
  A wz[4] = {A(1), A(0), A(0), A(0)}, wy[4], wx[4];
  if (ndim == 3 && !cubic_tap(z, D, zi, wz)) return A(0);
  if (!cubic_tap(y, H, yi, wy) || !cubic_tap(x, W, xi, wx)) return A(0);
  const int nz = ndim == 3 ? 4 : 1;
  A acc = A(0);
  for (int a = 0; a < nz; a++) {
    A slab = A(0);
#pragma unroll
    for (int b = 0; b < 4; b++) {
      const T *row = plane + (static_cast<long>(zi[a]) * H + yi[b]) * W;
      slab += wy[b] * (wx[0] * load(row + xi[0]) + wx[1] * load(row + xi[1]) +
                       wx[2] * load(row + xi[2]) + wx[3] * load(row + xi[3]));
    }
    acc += wz[a] * slab;
  }
  return acc;
}

}  // namespace mv
