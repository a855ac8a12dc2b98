// Forward resampling for LARGE outputs per roi (Resize / RandomAffine / Crop: one roi produces a
// whole volume) with a sampling grid of 1x1x1.  Used by the rotated, plain and affine entry
// points whenever one (roi, channel) yields at least a few thousand voxels and the caller passes
// a workspace.
//
// Two launches:
//   plan kernel    one lane per output tile (TX x TY x TZ voxels of one roi): builds the roi's
//                  affine sample map r = Rot * p + centre in fp64 (three sincos), the interval
//                  each source axis covers for the tile (centre +- sum_j |Rot[a][j]| * halfspan_j)
//                  and from it the axis-aligned box of source voxels to stage, clipped to the
//                  volume.  Writes one 128-byte tile plan: box, mode and the affine map expressed
//                  relative to the box origin (position of the tile's first voxel + the three
//                  per-voxel increments).
//   resample kernel one workgroup per (tile, channel).  If the box fits in LDS the workgroup
//                  copies it with coalesced 8-byte row loads and every lane produces a column of
//                  the tile from LDS: lanes run along x, so LDS reads of neighbouring lanes touch
//                  neighbouring banks and output stores are coalesced.  Otherwise (strong
//                  down-scaling, extreme rotations) lanes gather from global memory.
// Coordinates: box-relative, one FMA per axis and voxel in the coordinate type CT (fp32 for 16-bit
// tensors, fp64 for fp32 tensors), then floor / fraction in CT.  Tiles whose box is not clipped
// skip the [-1,S] tests and the border clamps.  Workgroup ids are permuted so that the workgroups
// resident on one XCD (own L2) process neighbouring tiles and share their halos in that L2.
#include "common.hpp"
#include "roi_geometry.hpp"
#include "sampling.hpp"

namespace mv {

constexpr int kXcds = 8;

struct TilePlan {          // 128 bytes
  double org[3];           // box-relative source position (x,y,z) of the tile's first output voxel
  double inc[9];           // d(source a)/d(output j) at inc[a * 3 + j], j = (x, y, z)
  int lo[3];               // first staged source voxel (x, y, z)
  int n[3];                // staged extent
  int batch;               // feature-map index of the roi
  int mode;                // 0 = all zero, 1 = staged (clipped box), 2 = gather, 3 = staged interior
};
static_assert(sizeof(TilePlan) == 128, "plan record size");

struct PlanShape {
  int tiles_x, tiles_y, tiles_z;  // spatial tiles per roi
  int tx, ty, tz;                 // tile extent in output voxels
  int vec;                        // elements per aligned 8-byte group (0: rows are not aligned)
  int cap;                        // LDS capacity in elements
};

__device__ inline void plan_tile(const RoiGeom &g, const RoiProblem &p, const PlanShape &ps,
                                 unsigned tile, TilePlan *dst) {
  const int is3d = p.ndim == 3;
  const int t0[3] = {static_cast<int>(tile % ps.tiles_x) * ps.tx,
                     static_cast<int>((tile / ps.tiles_x) % ps.tiles_y) * ps.ty,
                     static_cast<int>(tile / (ps.tiles_x * ps.tiles_y)) * ps.tz};
  const int out[3] = {p.ow, p.oh, p.od}, size[3] = {p.W, p.H, p.D}, ext[3] = {ps.tx, ps.ty, ps.tz};
  double first[3], half[3];  // local coordinate of the tile's first voxel, half span per axis
  for (int j = 0; j < 3; j++) {
    const int cells = min(ext[j], out[j] - t0[j]);
    const bool live = j < p.ndim;
    first[j] = live ? local_coord(g, j, t0[j], 0) : 0.0;
    half[j] = live ? 0.5 * (cells - 1) * g.bin[j] : 0.0;
  }
  TilePlan plan;
  plan.batch = g.batch;
  bool empty = false, clipped = false;
  double vol = 1.0;
  for (int a = 0; a < 3; a++) {
    double mid = g.centre[a], reach = 0.0, pos = g.centre[a];
    for (int j = 0; j < 3; j++) {
      const double r = g.rot[a * 3 + j];
      mid += r * (first[j] + half[j]);
      reach += fabs(r * half[j]);
      pos += r * first[j];
      plan.inc[a * 3 + j] = (j < p.ndim) ? r * g.bin[j] : 0.0;
    }
    if (!is3d && a == 2) {
      plan.lo[a] = 0; plan.n[a] = 1; plan.org[a] = 0.0;
      continue;
    }
    // widen by more than the rounding of the per-voxel coordinate arithmetic
    const double eps = 4e-5, rmin = mid - reach - eps, rmax = mid + reach + eps;
    const int S = size[a];
    empty |= rmax < -1.0 || rmin > S;
    clipped |= rmin < 0.0 || rmax > S - 1;
    int l = static_cast<int>(fmin(floor(fmax(rmin, 0.0)), static_cast<double>(S - 1)));
    int h = static_cast<int>(fmin(floor(fmax(rmax, 0.0)) + 1.0, static_cast<double>(S - 1)));
    if (a == 0 && ps.vec > 0) {  // whole 8-byte groups
      l = l / ps.vec * ps.vec;
      h = min((h / ps.vec + 1) * ps.vec, S) - 1;
    }
    plan.lo[a] = l;
    plan.n[a] = h - l + 1;
    plan.org[a] = pos - static_cast<double>(l);
    vol *= (a == 0) ? static_cast<double>((plan.n[0] + 4) / 4 * 4) : static_cast<double>(plan.n[a]);
  }
  const bool grid_one = g.grid[0] == 1 && g.grid[1] == 1 && (!is3d || g.grid[2] == 1);
  if (g.batch < 0 || empty || !grid_one) plan.mode = 0;   // (grid != 1 cannot happen: ratio is 1)
  else if (vol > ps.cap) plan.mode = 2;
  else plan.mode = clipped ? 1 : 3;
  *dst = plan;
}

constexpr int kPlanThreads = 256;

// One workgroup per roi: lanes 0..2 evaluate the trigonometry in parallel, lane 0 assembles the
// geometry, then every lane plans a share of the roi's tiles.
template <typename RT>
__global__ __launch_bounds__(kPlanThreads) void roi_plan_kernel(const RT *__restrict__ rois,
                                                                 TilePlan *__restrict__ plans,
                                                                 const RoiProblem p,
                                                                 const PlanShape ps) {
  __shared__ RoiGeom g;
  __shared__ double trig[6];
  const unsigned n = blockIdx.x;
  build_geom_block(g, trig, rois + static_cast<long>(n) * roi_columns(p.ndim, p.rotated), p);
  const unsigned per_roi = static_cast<unsigned>(ps.tiles_x) * ps.tiles_y * ps.tiles_z;
  for (unsigned tile = threadIdx.x; tile < per_roi; tile += kPlanThreads)
    plan_tile(g, p, ps, tile, plans + static_cast<long>(n) * per_roi + tile);
}


// Two x-neighbouring elements from LDS using naturally aligned accesses only (unaligned LDS reads
// stall the LDS pipeline).  16-bit types: read the two aligned dwords that contain the pair and
// shift the pair out; rows start at even element offsets.
// x-lerp of the pair (tile[idx], tile[idx + 1]) with weight w: a + w * (b - a), written as two
// FMAs whose 16-bit operands the compiler folds into mixed-precision FMA instructions.
__device__ __forceinline__ float lerp_pair(const float *tile, int idx, float w) {
  const float a = tile[idx], b = tile[idx + 1];
  return fmaf(w, b, fmaf(-w, a, a));
}
template <typename H>
__device__ __forceinline__ unsigned read_pair16(const H *tile, int idx) {
  const unsigned *w = reinterpret_cast<const unsigned *>(tile) + (idx >> 1);
  return __builtin_amdgcn_alignbit(w[1], w[0], static_cast<unsigned>(idx & 1) * 16u);
}
__device__ __forceinline__ float lerp_pair(const __half *tile, int idx, float w) {
  const unsigned bits = read_pair16(tile, idx);
  const float a = __half2float(__ushort_as_half(static_cast<unsigned short>(bits & 0xffffu)));
  const float b = __half2float(__ushort_as_half(static_cast<unsigned short>(bits >> 16)));
  return fmaf(w, b, fmaf(-w, a, a));
}
__device__ __forceinline__ float lerp_pair(const __hip_bfloat16 *tile, int idx, float w) {
  const unsigned bits = read_pair16(tile, idx);
  const float a = __uint_as_float(bits << 16), b = __uint_as_float(bits & 0xffff0000u);
  return fmaf(w, b, fmaf(-w, a, a));
}

__device__ __forceinline__ float clamp_ct(float v, float lo, float hi) { return __builtin_amdgcn_fmed3f(v, lo, hi); }
__device__ __forceinline__ double clamp_ct(double v, double lo, double hi) { return fmin(fmax(v, lo), hi); }

template <typename CT> struct BoxLimits { CT vmin[3], vmax[3], cmin[3], cmax[3]; int n1[3]; };

// One voxel from the staged box; (rx, ry, rz) are box-relative coordinates.
template <typename T, typename CT, bool INTERIOR>
__device__ __forceinline__ float staged_sample(const T *__restrict__ tile, CT rx, CT ry, CT rz,
                                               const BoxLimits<CT> &b, int pitch, int slice,
                                               int order) {
  bool ok = true;
  if (!INTERIOR) {
    ok = rx >= b.vmin[0] && rx <= b.vmax[0] && ry >= b.vmin[1] && ry <= b.vmax[1] &&
         rz >= b.vmin[2] && rz <= b.vmax[2];
    rx = clamp_ct(rx, b.cmin[0], b.cmax[0]);
    ry = clamp_ct(ry, b.cmin[1], b.cmax[1]);
    rz = clamp_ct(rz, b.cmin[2], b.cmax[2]);
  }
  const CT flx = floor(rx), fly = floor(ry), flz = floor(rz);
  const CT dx_ = rx - flx, dy_ = ry - fly, dz_ = rz - flz;
  const float wx = static_cast<float>(dx_), wy = static_cast<float>(dy_), wz = static_cast<float>(dz_);
  int ix = static_cast<int>(flx), iy = static_cast<int>(fly), iz = static_cast<int>(flz);
  int dy = pitch, dz = slice;
  if (!INTERIOR) {  // void samples may lie anywhere: keep every access inside the box
    ix = min(max(ix, 0), b.n1[0]); iy = min(max(iy, 0), b.n1[1]); iz = min(max(iz, 0), b.n1[2]);
    dy = iy < b.n1[1] ? pitch : 0;
    dz = iz < b.n1[2] ? slice : 0;
  }
  const int i00 = __mul24(iz, slice) + __mul24(iy, pitch) + ix;
  float v;
  if (order == 0) {
    v = load(tile + (i00 + (dz_ <= CT(0.5) ? 0 : dz) + (dy_ <= CT(0.5) ? 0 : dy) + (dx_ <= CT(0.5) ? 0 : 1)));
  } else {
    const float x00 = lerp_pair(tile, i00, wx), x01 = lerp_pair(tile, i00 + dy, wx);
    const float x10 = lerp_pair(tile, i00 + dz, wx), x11 = lerp_pair(tile, i00 + dz + dy, wx);
    const float y0 = x00 + wy * (x01 - x00), y1 = x10 + wy * (x11 - x10);
    v = y0 + wz * (y1 - y0);
  }
  return ok ? v : 0.f;
}

// Gather path: one column of the tile straight from global memory (sampling grid 1).
template <typename T>
__device__ __noinline__ void gather_column(const T *__restrict__ src, T *__restrict__ drow,
                                           long zstride, int count, double rx, double ry, double rz,
                                           double sx, double sy, double sz, int D, int H, int W,
                                           int order) {
  for (int k = 0; k < count; k++)
    drow[k * zstride] = store_cast<T>(sample_clamped<T>(src, D, H, W, rz + k * sz, ry + k * sy,
                                                        rx + k * sx, order));
}

template <typename T, int TX, int TY, int TZ, int THREADS, int LDS_BYTES>
__global__ __launch_bounds__(THREADS) void roi_resample_kernel(
    const T *__restrict__ feat, const TilePlan *__restrict__ plans, T *__restrict__ out,
    const int C, const int D, const int H, const int W, const int od, const int oh, const int ow,
    const int tiles_x, const int tiles_y, const int tiles_z, const unsigned total, const int vec,
    const int order) {
  using CT = typename std::conditional<(sizeof(T) == 2), float, double>::type;
  constexpr int kCap = LDS_BYTES / sizeof(T);
  constexpr int RZ = THREADS / (TX * TY);  // lane layers along z
  static_assert(RZ >= 1 && RZ * TX * TY == THREADS && TZ % RZ == 0, "tile shape");
  constexpr int ZPL = TZ / RZ;             // consecutive output slices per lane
  __shared__ __attribute__((aligned(16))) T tile[kCap];

  // XCD-aware numbering: workgroup ids go round-robin over the XCDs; give each XCD a contiguous
  // range of tiles.
  unsigned id = blockIdx.x;
  {
    const unsigned per = total / kXcds;
    if (id < per * kXcds) id = (id % kXcds) * per + id / kXcds;
  }
  const TilePlan &plan = plans[id];  // wave-uniform address: scalar loads
  const int c = blockIdx.y;
  const unsigned per_roi = static_cast<unsigned>(tiles_x) * tiles_y * tiles_z;
  const unsigned n = id / per_roi, tile_id = id % per_roi;
  const int tx0 = (tile_id % tiles_x) * TX;
  const int ty0 = ((tile_id / tiles_x) % tiles_y) * TY;
  const int tz0 = (tile_id / (tiles_x * tiles_y)) * TZ;
  const int lx = threadIdx.x % TX, ly = (threadIdx.x / TX) % TY, lz = threadIdx.x / (TX * TY);
  const int ox = tx0 + lx, oy = ty0 + ly, zb = tz0 + lz * ZPL;
  const int count = (ox < ow && oy < oh) ? min(ZPL, od - zb) : 0;  // may be <= 0
  const long zstride = static_cast<long>(oh) * ow;
  T *drow = out + (static_cast<long>(n) * C + c) * od * zstride + (static_cast<long>(zb) * oh + oy) * ow + ox;
  const int mode = plan.mode;

  if (mode == 0) {
    for (int k = 0; k < count; k++) drow[k * zstride] = store_cast<T>(0.f);
    return;
  }
  const T *src = feat + (static_cast<long>(plan.batch) * C + c) * static_cast<long>(D) * H * W;
  // box-relative position of this lane's first voxel and the per-slice increment
  const double bxr = plan.org[0] + lx * plan.inc[0] + ly * plan.inc[1] + (lz * ZPL) * plan.inc[2];
  const double byr = plan.org[1] + lx * plan.inc[3] + ly * plan.inc[4] + (lz * ZPL) * plan.inc[5];
  const double bzr = plan.org[2] + lx * plan.inc[6] + ly * plan.inc[7] + (lz * ZPL) * plan.inc[8];
  if (mode == 2) {
    if (count > 0)
      gather_column<T>(src, drow, zstride, count, bxr + plan.lo[0], byr + plan.lo[1], bzr + plan.lo[2],
                       plan.inc[2], plan.inc[5], plan.inc[8], D, H, W, order);
    return;
  }

  // ---- stage the box ---------------------------------------------------------------------
  const int bx = plan.n[0], by = plan.n[1], bz = plan.n[2];
  const int pitch = (bx + 4) / 4 * 4;  // >= bx + 1 (a finite pad ends every row), even
  const int slice = by * pitch;
  const int rows = by * bz;
  {
    const T *corner = src + (static_cast<long>(plan.lo[2]) * H + plan.lo[1]) * W + plan.lo[0];
    const float inv_by = 1.0f / static_cast<float>(by);
    if (vec > 0) {
      // 8 bytes per lane and item; item i = (row, group).  Eight independent loads are issued
      // before the first LDS store so that the copy is not serialised on memory latency.
      constexpr int V = 8 / sizeof(T);
      constexpr int kBatch = 8;
      const int groups = bx / V + 1;  // + the pad group (zeros)
      const int items = rows * groups;
      const float inv_groups = 1.0f / static_cast<float>(groups);
      for (int first = threadIdx.x; first < items; first += THREADS * kBatch) {
        uint2 val[kBatch];
        int dst_off[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; u++) {
          const int i = first + u * THREADS;
          val[u] = make_uint2(0u, 0u);
          dst_off[u] = -1;
          if (i < items) {
            const int r = static_cast<int>((static_cast<float>(i) + 0.5f) * inv_groups), gi = i - r * groups;
            const int zz = static_cast<int>((static_cast<float>(r) + 0.5f) * inv_by), yy = r - zz * by;
            dst_off[u] = r * pitch + gi * V;
            if (gi * V < bx)
              val[u] = *reinterpret_cast<const uint2 *>(corner + (static_cast<long>(zz) * H + yy) * W + gi * V);
          }
        }
#pragma unroll
        for (int u = 0; u < kBatch; u++)
          if (dst_off[u] >= 0) *reinterpret_cast<uint2 *>(tile + dst_off[u]) = val[u];
      }
    } else {
      int lpr = 1;
      while (lpr < pitch && lpr < kWave) lpr *= 2;
      const int lane_e = threadIdx.x & (lpr - 1), lane_r = threadIdx.x / lpr;
      for (int r = lane_r; r < rows; r += THREADS / lpr) {
        const int zz = static_cast<int>((static_cast<float>(r) + 0.5f) * inv_by), yy = r - zz * by;
        const T *row = corner + (static_cast<long>(zz) * H + yy) * W;
        for (int e = lane_e; e < pitch; e += lpr) tile[r * pitch + e] = e < bx ? row[e] : store_cast<T>(0.f);
      }
    }
  }
  __syncthreads();
  if (count <= 0) return;
  const CT b0 = static_cast<CT>(bxr), b1 = static_cast<CT>(byr), b2 = static_cast<CT>(bzr);
  const CT s0 = static_cast<CT>(plan.inc[2]), s1 = static_cast<CT>(plan.inc[5]), s2 = static_cast<CT>(plan.inc[8]);
  const int zslice = bz > 1 ? slice : 0;  // a single staged slice has no upper z neighbour
  BoxLimits<CT> lim;
  const int size[3] = {W, H, D};
  for (int a = 0; a < 3; a++) {
    lim.vmin[a] = static_cast<CT>(-1 - plan.lo[a]); lim.vmax[a] = static_cast<CT>(size[a] - plan.lo[a]);
    lim.cmin[a] = static_cast<CT>(-plan.lo[a]); lim.cmax[a] = static_cast<CT>(size[a] - 1 - plan.lo[a]);
    lim.n1[a] = plan.n[a] - 1;
  }
  if (mode == 3) {
#pragma unroll
    for (int k = 0; k < ZPL; k++) {
      if (k < count) {
        const CT kk = static_cast<CT>(k);
        drow[k * zstride] = store_cast<T>(staged_sample<T, CT, true>(
            tile, b0 + kk * s0, b1 + kk * s1, b2 + kk * s2, lim, pitch, zslice, order));
      }
    }
  } else {
#pragma unroll 2
    for (int k = 0; k < count; k++) {
      const CT kk = static_cast<CT>(k);
      drow[k * zstride] = store_cast<T>(staged_sample<T, CT, false>(
          tile, b0 + kk * s0, b1 + kk * s1, b2 + kk * s2, lim, pitch, zslice, order));
    }
  }
}

template <typename T, int TX, int TY, int TZ, int THREADS, int LDS_BYTES>
static int launch_resample(const T *feat, const float *rois, T *out, const RoiProblem &p,
                           void *workspace, size_t *need, hipStream_t s) {
  const long tx = (p.ow + TX - 1) / TX, ty = (p.oh + TY - 1) / TY, tz = (p.od + TZ - 1) / TZ;
  const long total = tx * ty * tz * static_cast<long>(p.R);
  if (total >= (1L << 31) || p.C > 65535) return -1;
  if (need) { *need = static_cast<size_t>(total) * sizeof(TilePlan); return MV_OK; }
  constexpr int V = 8 / sizeof(T);
  PlanShape ps;
  ps.tiles_x = static_cast<int>(tx); ps.tiles_y = static_cast<int>(ty); ps.tiles_z = static_cast<int>(tz);
  ps.tx = TX; ps.ty = TY; ps.tz = TZ;
  ps.vec = ((p.W % V == 0) && (reinterpret_cast<uintptr_t>(feat) % 8 == 0)) ? V : 0;
  ps.cap = LDS_BYTES / sizeof(T);
  TilePlan *plans = static_cast<TilePlan *>(workspace);
  hipLaunchKernelGGL((roi_plan_kernel<float>), dim3(p.R), dim3(kPlanThreads), 0, s, rois, plans, p, ps);
  hipLaunchKernelGGL((roi_resample_kernel<T, TX, TY, TZ, THREADS, LDS_BYTES>),
                     dim3(static_cast<unsigned>(total), p.C), dim3(THREADS), 0, s, feat, plans, out, p.C,
                     p.D, p.H, p.W, p.od, p.oh, p.ow, ps.tiles_x, ps.tiles_y, ps.tiles_z,
                     static_cast<unsigned>(total), ps.vec, p.order);
  return check_launch("roi_resample_kernel");
}

// The tiled path pays when one (roi, channel) yields many voxels and the sampling grid is 1.
// With `need` set only the workspace size is computed.  Returns -1 when the path does not apply.
int roi_forward_tiled(const void *input, const void *rois, void *output, int dtype,
                      const RoiProblem &p, void *workspace, size_t *need, hipStream_t s) {
  const long vox = static_cast<long>(p.od) * p.oh * p.ow;
  if (p.sampling_ratio != 1 || vox < 4096 || p.ow < 16 || p.R == 0) return -1;
  if (!need && !workspace) return -1;
  const float *r = static_cast<const float *>(rois);
  switch (dtype) {
    case MV_F16:
      return launch_resample<__half, 16, 16, 16, 512, 64 * 1024>(
          static_cast<const __half *>(input), r, static_cast<__half *>(output), p, workspace, need, s);
    case MV_BF16:
      return launch_resample<__hip_bfloat16, 16, 16, 16, 512, 64 * 1024>(
          static_cast<const __hip_bfloat16 *>(input), r, static_cast<__hip_bfloat16 *>(output), p,
          workspace, need, s);
    case MV_F32:
      return launch_resample<float, 16, 16, 8, 512, 64 * 1024>(
          static_cast<const float *>(input), r, static_cast<float *>(output), p, workspace, need, s);
    default:
      return -1;
  }
}

}  // namespace mv
