// Backward of RoIAlign / RoIAlignRotated for resampling-sized problems, as a gather.
//
// The adjoint of a resampling (one sample per output voxel, an output about as large as the input,
// a roi or two per image: RandomAffine, Resize) is usually written as a scatter, eight atomic adds
// per output voxel.  Here every INPUT voxel collects its own gradient instead: the output voxels
// whose sample lies within one voxel of it form a small parallelepiped in output space, which is
// enumerated row by row (the extent along the fastest output axis is solved for exactly, the other
// two axes come from a bounding box), each candidate is evaluated with the very sampler of the
// forward pass (`clamped_tap`: closed interval [-1, size], border replicate, nearest ties low) and
// contributes grad_output * weight when the voxel is one of its taps.  No atomics, no fp32
// workspace for 16-bit tensors, one rounding per voxel, and a result that does not depend on the
// order in which workgroups run.
#include "common.hpp"
#include "roi_geometry.hpp"
#include "sampling.hpp"

namespace mv {

constexpr int kGatherThreads = 256;
constexpr int kGatherPerThread = 4;   // input voxels per thread (one in the launch for the faces: few voxels, long chains)

struct GatherShared {
  RoiGeom g;
  double trig[6];
  double reach[3];   // per local axis j: sum_a |rot[a][j]| + margin = how far (in local
                     // coordinates) a sample may be from the voxel and still touch it
  double inv_bin[3]; // 1 / bin (0 for a degenerate axis)
  // fp32 copies for the row test (it only has to be conservative: `slack` covers its rounding)
  float r1[3], r2[3];  // rot[a][1], rot[a][2]
  float inv_m[3];      // 1 / rot[a][0] (0 when source axis a does not move along an output row)
  float half[3];       // (1 + slack) * |inv_m|
  float inv_bin0, off0;  // cell along the row = x * inv_bin0 - off0
  float slack, slack_u;
};

// a wave-uniform value moved to scalar registers (LDS reads land in vector registers)
__device__ __forceinline__ float scalar(float v) { return __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(v))); }
__device__ __forceinline__ double scalar(double v) {
  return __hiloint2double(__builtin_amdgcn_readfirstlane(__double2hiint(v)), __builtin_amdgcn_readfirstlane(__double2loint(v)));
}

// weight with which tap (lo, hi, frac) of one axis falls on index v
template <typename A>
__device__ __forceinline__ A axis_weight(int v, int lo, int hi, A frac) {
  return (v == lo ? A(1) - frac : A(0)) + (v == hi ? frac : A(0));
}

// `clamped_tap` (sampling.hpp) in the coordinate type C
template <typename C, typename A>
__device__ __forceinline__ bool clamped_tap_in(C v, int size, int &lo, int &hi, A &frac, int order) {
  if (v < C(-1) || v > static_cast<C>(size)) return false;
  v = v <= C(0) ? C(0) : v;
  const int base = static_cast<int>(v);
  C f = C(0);
  if (base >= size - 1) {
    lo = hi = size - 1;
  } else {
    lo = base;
    hi = base + 1;
    f = v - static_cast<C>(base);
  }
  frac = order == 0 ? ((C(1) - f >= C(0.5)) ? A(0) : A(1)) : static_cast<A>(f);
  return true;
}

// Order in which a launch walks the voxels of a volume: those on no face first (x fastest), then the
// faces — z = 0, z = D - 1, y = 0, y = H - 1, x = 0, x = W - 1, each without what came before — so that
// all but one workgroup hold voxels of one kind.  An image (ndim 2) has no z faces.
struct ShellOrder {
  unsigned W, H, D, wi, hi, dz, z0;          // inner extents, first inner slice
  unsigned inner, a, b, c, d, e;             // cumulative ends of the inner block and of the first five faces
  __host__ __device__ ShellOrder(int ndim, int w, int h, int dd) {
    W = w; H = h; D = dd;
    wi = w > 2 ? w - 2 : 0; hi = h > 2 ? h - 2 : 0;
    dz = ndim == 3 ? (dd > 2 ? dd - 2 : 0) : 1; z0 = ndim == 3 ? 1 : 0;
    inner = wi * hi * dz;
    a = inner + (ndim == 3 ? W * H : 0);
    b = a + (ndim == 3 && dd > 1 ? W * H : 0);
    c = b + W * dz;
    d = c + (h > 1 ? W * dz : 0);
    e = d + hi * dz;
  }
  // voxel number i of the walk; true for one on no face
  __device__ __forceinline__ bool voxel(unsigned i, int (&v)[3]) const {
    if (i < inner) {
      const unsigned r = i / wi, x = i - r * wi, z = r / hi, y = r - z * hi;
      v[0] = x + 1; v[1] = y + 1; v[2] = z + z0;
      return true;
    }
    if (i < b) {          // z = 0 and z = D - 1, whole slices
      const unsigned j = i - (i < a ? inner : a), y = j / W;
      v[0] = j - y * W; v[1] = y; v[2] = i < a ? 0 : D - 1;
    } else if (i < d) {   // y = 0 and y = H - 1, rows of the inner slices
      const unsigned j = i - (i < c ? b : c), z = j / W;
      v[0] = j - z * W; v[1] = i < c ? 0 : H - 1; v[2] = z + z0;
    } else {              // x = 0 and x = W - 1, what is left of the inner slices
      const unsigned j = i - (i < e ? d : e), z = j / hi;
      v[0] = i < e ? 0 : W - 1; v[1] = j - z * hi + 1; v[2] = z + z0;
    }
    return false;
  }
};

struct GatherGeo {   // a roi's constants as the voxel routine reads them
  RoiGeom g;
  double reach[3], inv_bin[3];
  float r1[3], r2[3], inv_m[3], half[3];
  float inv_bin0, off0, slack, slack_u;
};
struct GatherDims { int nd, D, H, W, od, oh, ow, order; };

// The gradient one roi leaves at voxel v, candidates in the coordinate type C.  The linear sampler is
// continuous in the sample position except at the edges of [-1, size], beyond which a sample is
// void.  A sample that touches voxel v lies within one voxel of it on every axis, so for a voxel
// that is on no face of the volume no candidate comes near such an edge, and fp32 positions (off by
// ~1e-5 of a voxel, weights by as much) decide nothing differently from fp64.  The voxels on the
// faces, and order 0, which jumps wherever a fraction passes 0.5, are worked out in fp64 with the
// expressions of the fp64 reference.
template <typename T, typename C>
__device__ __forceinline__ typename Acc<T>::type gather_voxel(const GatherGeo &q, const GatherDims &d, const T *go,
                                                              const int (&v)[3]) {
  using A = typename Acc<T>::type;
  constexpr double kSlack = 1e-6;
  const RoiGeom &g = q.g;
  const double(&reach)[3] = q.reach;
  const double(&inv_bin)[3] = q.inv_bin;
  const float(&r1)[3] = q.r1;
  const float(&r2)[3] = q.r2;
  const float(&inv_m)[3] = q.inv_m;
  const float(&half)[3] = q.half;
  const float inv_bin0 = q.inv_bin0, off0 = q.off0, slack = q.slack, slack_u = q.slack_u;
  const int nd = d.nd;
  const int cells[3] = {d.ow, d.oh, d.od};
  const GatherDims &p = d;
  const A inv_count = A(1) / static_cast<A>(g.count);
    const C m0 = static_cast<C>(g.rot[0]), m3 = static_cast<C>(g.rot[3]), m6 = static_cast<C>(g.rot[6]);
    const C m1 = static_cast<C>(g.rot[1]), m4 = static_cast<C>(g.rot[4]), m7 = static_cast<C>(g.rot[7]);
    const C m2 = static_cast<C>(g.rot[2]), m5 = static_cast<C>(g.rot[5]), m8 = static_cast<C>(g.rot[8]);
    const C c0x = static_cast<C>(g.centre[0]), c0y = static_cast<C>(g.centre[1]), c0z = static_cast<C>(g.centre[2]);
    const C xbin = static_cast<C>(g.bin[0]), xoff = static_cast<C>(g.start[0] + 0.5 * g.sub[0]);
    const C ybin = static_cast<C>(g.bin[1]), yoff = static_cast<C>(g.start[1] + 0.5 * g.sub[1]);
    const C zbin = static_cast<C>(g.bin[2]), zoff = static_cast<C>(g.start[2] + 0.5 * g.sub[2]);
    // the voxel in the roi's local frame: q = Rot^T (v - centre)
    // (in the coordinate type; in fp32 the ranges are widened by what its rounding can move them)
    const C dx = static_cast<C>(v[0] - g.centre[0]), dy = static_cast<C>(v[1] - g.centre[1]),
            dz = nd == 3 ? static_cast<C>(v[2] - g.centre[2]) : C(0);
    const C wide = sizeof(C) == 4 ? static_cast<C>(slack) : static_cast<C>(kSlack);
    int lo[3], hi[3];
    bool any = true;
  #pragma unroll
    for (int j = 0; j < 3; j++) {
      if (j >= nd) { lo[j] = 0; hi[j] = 0; continue; }
      const C q = static_cast<C>(g.rot[j]) * dx + static_cast<C>(g.rot[3 + j]) * dy + static_cast<C>(g.rot[6 + j]) * dz;
      // cells u with |start + (u + .5) * bin - q| <= reach
      const C rj = static_cast<C>(reach[j]) + wide, sj = static_cast<C>(g.start[j]), ib = static_cast<C>(inv_bin[j]);
      const C a0 = q - rj - sj, a1 = q + rj - sj;
      if (inv_bin[j] != 0.0) {
        // (a negative bin, i.e. a mirrored roi, swaps the two ends)
        const C e0 = a0 * ib - C(0.5), e1 = a1 * ib - C(0.5);
        const C extra = wide * (C(1) + fabs(ib));
        const C u0 = fmin(fmax(fmin(e0, e1) - extra, C(-1)), static_cast<C>(cells[j]));
        const C u1 = fmin(fmax(fmax(e0, e1) + extra, C(-1)), static_cast<C>(cells[j]));
        lo[j] = max(static_cast<int>(ceil(u0)), 0);
        hi[j] = min(static_cast<int>(floor(u1)), cells[j] - 1);
      } else {   // every cell samples the same coordinate
        lo[j] = 0;
        hi[j] = (a0 <= C(0) && a1 >= C(0)) ? cells[j] - 1 : -1;
      }
      any = any && lo[j] <= hi[j];
    }
    if (!any) return A(0);
    A sum = A(0);
    const float cv[3] = {static_cast<float>(-dx), static_cast<float>(-dy), static_cast<float>(-dz)};
    const float cells0 = static_cast<float>(cells[0]);
    for (int uz = lo[2]; uz <= hi[2]; uz++) {
      const C zc = nd == 3 ? static_cast<C>(uz) * zbin + zoff : C(0);   // local_coord(g, 2, uz, 0)
      const float zf = static_cast<float>(zc);
      const float bz[3] = {fmaf(r2[0], zf, cv[0]), fmaf(r2[1], zf, cv[1]), fmaf(r2[2], zf, cv[2])};
      // the slice's share of the sample positions
      const C zx = fma(m2, zc, c0x), zy = fma(m5, zc, c0y), zw = fma(m8, zc, c0z);
      for (int uy = lo[1]; uy <= hi[1]; uy++) {
        const C yc = static_cast<C>(uy) * ybin + yoff;   // local_coord(g, 1, uy, 0)
        const float yf = static_cast<float>(yc);
        // samples of this output row: r_a(x) - v_a = rot[a][0] * x + base_a; keep it within +-1
        float xl = -3e38f, xh = 3e38f;
  #pragma unroll
        for (int a = 0; a < 3; a++) {
          if (a >= nd) continue;
          const float base = fmaf(r1[a], yf, bz[a]);
          if (inv_m[a] != 0.f) {
            const float mid = -base * inv_m[a];
            xl = fmaxf(xl, mid - half[a]);
            xh = fminf(xh, mid + half[a]);
          } else if (fabsf(base) > 1.f + 2.f * slack) {
            xh = -3e38f;
          }
        }
        if (xl > xh) continue;
        int x0 = lo[0], x1 = hi[0];
        if (inv_bin0 != 0.f) {
          const float e0 = fmaf(xl, inv_bin0, -off0), e1 = fmaf(xh, inv_bin0, -off0);
          const float u0 = fminf(fmaxf(fminf(e0, e1) - slack_u, -1.f), cells0);
          const float u1 = fminf(fmaxf(fmaxf(e0, e1) + slack_u, -1.f), cells0);
          x0 = max(x0, static_cast<int>(ceilf(u0)));
          x1 = min(x1, static_cast<int>(floorf(u1)));
        }
        if (x0 > x1) continue;
        // sample positions of the row: rot[a][0] * x + row term
        const C bx = fma(m1, yc, zx), by = fma(m4, yc, zy), bw = fma(m7, yc, zw);
        for (int ux = x0; ux <= x1; ux++) {
          const C x = static_cast<C>(ux) * xbin + xoff;   // local_coord(g, 0, ux, 0)
          const C rx = fma(m0, x, bx), ry = fma(m3, x, by);
          const C rz = nd == 3 ? fma(m6, x, bw) : C(0);
          int z0, z1, y0, y1, c0, c1;
          A lz, ly, lx;
          if (!clamped_tap_in<C, A>(rz, p.D, z0, z1, lz, p.order) || !clamped_tap_in<C, A>(ry, p.H, y0, y1, ly, p.order) ||
              !clamped_tap_in<C, A>(rx, p.W, c0, c1, lx, p.order))
            continue;
          const A w = axis_weight(v[2], z0, z1, lz) * axis_weight(v[1], y0, y1, ly) * axis_weight(v[0], c0, c1, lx);
          if (w != A(0))
            sum += load(go + (static_cast<long>(uz) * p.oh + uy) * p.ow + ux) * inv_count * w;
        }
      }
    }
  return sum;
}

// A workgroup's share of the voxels [walk_begin, walk_begin + walk_count) of the walk above, candidates in
// fp64 (EXACT) or fp32.
template <typename T, typename RT, bool EXACT, int PER>
__device__ __forceinline__ void gather_block(const T *__restrict__ gout, const RT *__restrict__ rois, T *__restrict__ gin,
                                             const RoiProblem &p, const unsigned walk_begin, const unsigned walk_count,
                                             const unsigned block_x) {
  using A = typename Acc<T>::type;
  using C = typename std::conditional<EXACT, double, float>::type;
  __shared__ GatherShared sh;
  const int b = blockIdx.z, c = blockIdx.y;
  const long plane = static_cast<long>(p.D) * p.H * p.W;
  const long first = walk_begin + static_cast<long>(block_x) * (kGatherThreads * PER) + threadIdx.x;
  const long walk_end = static_cast<long>(walk_begin) + walk_count;
  const int cols = roi_columns(p.ndim, p.rotated);
  const int nd = p.ndim;
  const long ocells = static_cast<long>(p.od) * p.oh * p.ow;
  constexpr double kSlack = 1e-6;   // the per-axis candidate ranges are widened by this much

  T *dst = gin + (static_cast<long>(b) * p.C + c) * plane;
  // per-voxel sums over the rois of the image (a thread's own slots; LDS because the voxel loop is
  // not unrolled): the gradient is rounded to the tensor type once
  __shared__ A sums[PER * kGatherThreads];
  for (int k = 0; k < PER; k++) sums[k * kGatherThreads + threadIdx.x] = A(0);
  const ShellOrder shell(nd, p.W, p.H, p.D);   // plane < 2^31 (checked on the host)

  for (int r = 0; r < p.R; r++) {
    const RT *roi = rois + static_cast<long>(r) * cols;
    if (static_cast<int>(roi[0]) != b) continue;   // uniform over the workgroup
    __syncthreads();                                // the previous roi's geometry is no longer read
    build_geom_block(sh.g, sh.trig, roi, p);
    if (threadIdx.x < 3) {
      const int j = threadIdx.x;
      sh.reach[j] = fabs(sh.g.rot[j]) + fabs(sh.g.rot[3 + j]) + fabs(sh.g.rot[6 + j]) + kSlack;
      sh.inv_bin[j] = fabs(sh.g.bin[j]) > 1e-12 ? 1.0 / sh.g.bin[j] : 0.0;   // negative for a mirrored roi
      const float slack = 1e-3f + 1e-6f * static_cast<float>(p.W + p.H + p.D);
      sh.r1[j] = static_cast<float>(sh.g.rot[3 * j + 1]);
      sh.r2[j] = static_cast<float>(sh.g.rot[3 * j + 2]);
      sh.inv_m[j] = fabs(sh.g.rot[3 * j]) > 1e-6 ? static_cast<float>(1.0 / sh.g.rot[3 * j]) : 0.f;
      sh.half[j] = (1.f + slack) * fabsf(sh.inv_m[j]);
      if (j == 0) {
        sh.inv_bin0 = static_cast<float>(sh.inv_bin[0]);
        sh.off0 = static_cast<float>(sh.g.start[0] * sh.inv_bin[0] + 0.5);
        sh.slack = slack;
        sh.slack_u = 1e-3f + 1e-6f * static_cast<float>(p.ow) + slack * fabsf(sh.inv_bin0);
      }
    }
    __syncthreads();
    // the roi's constants, in scalar registers for the loops below
    GatherGeo q;
#pragma unroll
    for (int i = 0; i < 9; i++) q.g.rot[i] = scalar(sh.g.rot[i]);
#pragma unroll
    for (int i = 0; i < 3; i++) {
      q.g.centre[i] = scalar(sh.g.centre[i]); q.g.start[i] = scalar(sh.g.start[i]);
      q.g.bin[i] = scalar(sh.g.bin[i]); q.g.sub[i] = scalar(sh.g.sub[i]);
      q.reach[i] = scalar(sh.reach[i]); q.inv_bin[i] = scalar(sh.inv_bin[i]);
      q.r1[i] = scalar(sh.r1[i]); q.r2[i] = scalar(sh.r2[i]); q.inv_m[i] = scalar(sh.inv_m[i]); q.half[i] = scalar(sh.half[i]);
      q.g.grid[i] = 0;
    }
    q.g.batch = 0;
    q.g.count = sh.g.count;
    q.inv_bin0 = scalar(sh.inv_bin0); q.off0 = scalar(sh.off0); q.slack = scalar(sh.slack); q.slack_u = scalar(sh.slack_u);
    const GatherDims dims = {nd, p.D, p.H, p.W, p.od, p.oh, p.ow, p.order};
    const T *go = gout + (static_cast<long>(r) * p.C + c) * ocells;

#pragma unroll 1
    for (int k = 0; k < PER; k++) {
      const long vi = first + static_cast<long>(k) * kGatherThreads;
      if (vi >= walk_end) continue;
      int v[3];
      shell.voxel(static_cast<unsigned>(vi), v);
      const A sum = gather_voxel<T, C>(q, dims, go, v);
      if (sum != A(0)) sums[k * kGatherThreads + threadIdx.x] += sum;
    }
  }
  // this thread owns its voxels: plain read-modify-write
  for (int k = 0; k < PER; k++) {
    const long vi = first + static_cast<long>(k) * kGatherThreads;
    const A total = sums[k * kGatherThreads + threadIdx.x];
    if (vi < walk_end && total != A(0)) {
      int v[3];
      shell.voxel(static_cast<unsigned>(vi), v);
      T *at = dst + (static_cast<long>(v[2]) * p.H + v[1]) * p.W + v[0];
      *at = store_cast<T>(load(at) + total);
    }
  }
}

// One launch: the first `exact_blocks` workgroups take the voxels [inner, plane) of the walk in fp64, one
// voxel per thread (few voxels with long chains of dependent instructions: they start first and run
// beside the others), the rest the first `inner` voxels in fp32.
template <typename T, typename RT>
__global__ __launch_bounds__(kGatherThreads) __attribute__((amdgpu_waves_per_eu(5))) void roi_backward_gather_kernel(
    const T *__restrict__ gout, const RT *__restrict__ rois, T *__restrict__ gin, const RoiProblem p,
    const unsigned inner, const unsigned plane, const unsigned exact_blocks) {
  if (blockIdx.x < exact_blocks)
    gather_block<T, RT, true, 1>(gout, rois, gin, p, inner, plane - inner, blockIdx.x);
  else
    gather_block<T, RT, false, kGatherPerThread>(gout, rois, gin, p, 0u, inner, blockIdx.x - exact_blocks);
}

// Applies when the problem is a resampling: one sample per cell, outputs of at least 4096 voxels
// that are not much smaller than the image, at most two rois per image on average (every input
// voxel walks over all rois of its image).  Returns -1 otherwise.
int roi_backward_gather(const void *grad_output, const void *rois, void *grad_input, int dtype,
                        const RoiProblem &p, hipStream_t s) {
  const long plane = static_cast<long>(p.D) * p.H * p.W;
  const long ocells = static_cast<long>(p.od) * p.oh * p.ow;
  if (p.sampling_ratio != 1 || (p.order != 0 && p.order != 1)) return -1;
  if (ocells < 4096 || ocells * 8 < plane || p.R > 2 * p.N) return -1;
  if (p.C > 65535 || p.N > 65535 || plane >= (1L << 31)) return -1;
  constexpr long per_block = kGatherThreads * kGatherPerThread;
  // Linear taps of 16- and 32-bit tensors: fp32 candidates for the voxels on no face of the volume
  // (the first `inner` of the walk), fp64 for the faces; everything else in fp64.
  const ShellOrder walk(p.ndim, p.W, p.H, p.D);
  const bool split = p.order == 1 && dtype != MV_F64;
  const unsigned inner = split ? walk.inner : 0u, rest = static_cast<unsigned>(plane) - inner;
  const long exact_blocks = (rest + kGatherThreads - 1) / kGatherThreads, inner_blocks = (inner + per_block - 1) / per_block;
  if (exact_blocks + inner_blocks >= (1L << 31)) return -1;
  const dim3 grid(static_cast<unsigned>(exact_blocks + inner_blocks), p.C, p.N), block(kGatherThreads);
  MV_DISPATCH(dtype, {
    using RT = typename std::conditional<std::is_same<T, double>::value, double, float>::type;
    hipLaunchKernelGGL((roi_backward_gather_kernel<T, RT>), grid, block, 0, s,
                       static_cast<const T *>(grad_output), static_cast<const RT *>(rois),
                       static_cast<T *>(grad_input), p, inner, static_cast<unsigned>(plane),
                       static_cast<unsigned>(exact_blocks));
  });
  return check_launch("roi_backward_gather_kernel");
}

}  // namespace mv
