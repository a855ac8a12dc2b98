// Forward resampling for LARGE outputs per roi (Resize / RandomAffine / Crop: one roi produces a
// whole volume) with a sampling grid of 1x1x1.  Used by the rotated, plain and affine entry
// points whenever one (roi, channel) yields at least a few thousand voxels.  Same results as the
// reference's one-thread-per-output kernels (csrc/cuda/roi_align_rotated_3d_cuda_kernel.cuh:15-120,
// csrc/cuda_aug/affine_3d_cuda_kernel.cuh:14-120 and their 2-D twins).
//
// One launch of persistent workgroups.  An item is (output tile of TX x TY x TZ voxels, channel):
//   planning   (prologue) the first wavefront, four lanes per item of the workgroup: the roi's
//              affine sample map r = Rot * p + centre in fp64, the interval each source axis covers
//              for the tile (centre +- sum_j |Rot[a][j]| * halfspan_j) and from it the axis-aligned
//              box of source voxels to stage, clipped to the volume; the map is re-expressed
//              relative to the box origin.  The records (TilePlan, every wave-uniform value an item
//              needs) stay in LDS.  Meanwhile the other wavefronts pull a small input through the
//              caches.
//   staging    the box is copied to LDS as 16-byte row groups; the loads of item i+1 are issued
//              into registers while item i is interpolated.
//   sampling   every lane produces a column of the tile from LDS: lanes run along x, so LDS reads
//              of neighbouring lanes touch neighbouring banks and output stores are coalesced.
//              Boxes larger than the LDS buffer (strong down-scaling) are sampled straight from
//              global memory by the same code.
// Coordinates: box-relative in the coordinate type CT (fp32 for 16-bit tensors, fp64 for fp32
// tensors), then floor / fraction in CT.  Tiles whose box is not clipped skip the [-1,S] tests and
// the border clamps.
#include <algorithm>

#include "common.hpp"
#include "roi_geometry.hpp"
#include "sampling.hpp"

namespace mv {

// In-kernel time stamps of the tiled forward kernel (instrumented build only, -DMV_RESAMPLE_TIMELINE:
// a second library beside the product, read back by mv_debug_resample_timeline): thread 0 of every
// workgroup notes the 100 MHz wall clock at the points MV_TL marks.  Slots: 0 kernel entered, 1 first
// wavefront starts planning, 2 plans written, 3 past the barrier behind the plans, 4 first box has
// arrived in registers, 5..8 box of item 0..3 is in LDS, 9 last item interpolated, 10 stores drained.
#ifdef MV_RESAMPLE_TIMELINE
constexpr int kTimelineSlots = 16, kTimelineGroups = 4096;
__device__ unsigned long long mv_timeline[kTimelineGroups * kTimelineSlots];
#define MV_TL(i)                                                                                          \
  do {                                                                                                    \
    if (threadIdx.x == 0 && blockIdx.x < kTimelineGroups) mv_timeline[blockIdx.x * kTimelineSlots + (i)] = wall_clock64(); \
  } while (0)
#else
#define MV_TL(i) do { } while (0)
#endif

constexpr int kXcds = 8;

// What the workgroup's first wavefront works out per item and every wavefront then reads from LDS.
// Values a wavefront needs in scalar registers sit in the first 64 dwords (lane l fetches dword l,
// fields are pulled out with v_readlane); values only the vector unit uses are read as broadcasts.
struct TilePlan {            // 352 bytes
  // per source axis a, at [4 * a .. 4 * a + 3]: the box-relative source position of the tile's
  // first output voxel, then d(source a)/d(output j) for j = (x, y, z)
  double map[12];            // dword 0
  float mapf[12];            // dword 24: the same rounded to fp32 (coordinate type of the 16-bit kernels)
  int mode;                  // dword 36: 0 = all zero, 1 = staged (clipped box), 2 = gather, 3 = staged interior, 4 = no item
  int passes;                // copy passes through registers (ceil(n[2] / span)), 0: the box is copied in place
  unsigned src_lo, src_hi;   // byte offset of the box's first voxel in the feature tensor
  int extent;                // bytes from there to the end of the box's last row
  int stride;                // bytes between the passes of a lane (span slices)
  unsigned out_lo, out_hi;   // byte offset of the item's (roi, channel) volume in the output tensor
  int zcount;                // output slices from the tile's first one to the end of the volume
  int grid[3];               // samples per bin along (x, y, z): the fixed ratio, or ceil(roi extent / cells)
  // dword 48: a lane splits its index into (slice, row, 16-byte group) with two multiplications
  float inv_groups, inv_rows;
  int groups, by;
  // dword 52
  int rp;                    // box rows per pass (span whole slices)
  int gap_b;                 // LDS bytes between the end of a slice's last row and the next slice (padding)
  int bz, span;
  // dword 56: LDS geometry in bytes (dy / dz: 0 when the box is one row / slice thick)
  int pitch_b, slice_b, dy_b, dz_b;
  // dword 60: the tile in the output volume
  int tile_off;              // byte offset of the tile's first voxel
  int xlim, ylim;            // columns / rows from the tile's first voxel to the end of the volume
  int hop_b;                 // LDS bytes per pass
  // dword 64
  int lo[3];                 // first staged source voxel (x, y, z)
  int n[3];                  // staged extent
  int t0[3];                 // first output voxel of the tile (x, y, z)
  int roi;                   // roi index
  int batch;                 // feature-map index of the roi
  unsigned vol_lo, vol_hi;   // byte offset of the item's (image, channel) volume in the feature tensor
  int pad2[3];
  // dword 80: box-relative limits of a clipped box as fp32: coordinates clamp to [0, cmax], the
  // low tap index is at most top = max(n - 2, 0)
  float cmaxf[4], topf[4];
};
static_assert(sizeof(TilePlan) == 352 && offsetof(TilePlan, inv_groups) == 192 && offsetof(TilePlan, lo) == 256, "plan record layout");

// Division of n < 2^31 by a divisor fixed at launch: one 64-bit product and a shift.
struct FastDiv {
  unsigned mul, shift;
  __host__ void set(unsigned d) {
    unsigned s = 0;
    while ((2u << s) <= d && s < 30) s++;          // s = floor(log2 d)
    if ((d & (d - 1)) == 0) { mul = 0x80000000u; shift = 31 + s; }
    else { mul = static_cast<unsigned>(((1ull << (32 + s)) + d - 1) / d); shift = 32 + s; }
  }
  __device__ __forceinline__ unsigned div(unsigned n) const {
    return static_cast<unsigned>((static_cast<unsigned long long>(n) * mul) >> shift);
  }
};

struct PlanShape {
  int tiles_x, tiles_y, tiles_z;  // spatial tiles per roi
  int tx, ty, tz;                 // tile extent in output voxels
  int vec;                        // elements per aligned 16-byte group (0: rows are not aligned)
  int cap;                        // LDS capacity in elements
  int threads, max_items;         // workgroup size, 16-byte groups one lane holds in registers
  int es;                         // bytes per element
  FastDiv by_per_roi, by_tiles_x, by_tiles_y, by_total, by_slots;
  int halo_lo, halo_hi;           // voxels needed below / above the cell of a sample: 0 / 1, order 3: 1 / 2
  int grids;                      // 1: the kernel takes every sample of a bin (else items with grids above 1 are void)
  int flat_axis;                  // 1: the middle axis has one cell sampled once whatever the ratio (images as volumes of rows)
  unsigned warm_groups;           // 16-byte groups of the input to pull into the caches during planning (0: none)
  int pad_slices;                 // 1: LDS slices of a box start 32 bytes past a multiple of 128
};

constexpr unsigned kDone = 0xffffffffu;  // "no item"
constexpr unsigned kWarmStride = 4;      // words between the loads of the cache warm-up

// Lane-parallel planning: four lanes per item, lane `a` = 0..2 owns source axis / roi angle `a`
// (lane 3 idles), so the three sin / cos pairs, the per-axis divisions and the three box
// intervals of an item are evaluated side by side; values of the other axes come in through
// wave shuffles.  Every lane of the wavefront must call this (`item` may be kDone: nothing is
// written).  Same formulas as build_geom / local_coord in roi_geometry.hpp.
__device__ __forceinline__ double lane_get(double v, int src_lane) {
  const int lo = __builtin_amdgcn_ds_bpermute(src_lane * 4, __double2loint(v));
  const int hi = __builtin_amdgcn_ds_bpermute(src_lane * 4, __double2hiint(v));
  return __hiloint2double(hi, lo);
}
__device__ __forceinline__ int lane_get(int v, int src_lane) {
  return __builtin_amdgcn_ds_bpermute(src_lane * 4, v);
}

__device__ inline void plan_item_lanes(const float *__restrict__ rois, const RoiProblem &p,
                                       const PlanShape &ps, unsigned item, unsigned total,
                                       unsigned per_roi, TilePlan *dst) {
  const int lane = threadIdx.x & (kWave - 1), a = lane & 3, base = lane & ~3;
  const bool write = item != kDone && a < 3;
  const unsigned it = item != kDone ? item : 0u;
  const unsigned chan = p.C > 1 ? ps.by_total.div(it) : 0u;
  const unsigned idx = it - chan * total, n = ps.by_per_roi.div(idx), tile = idx - n * per_roi;
  const int nd = p.ndim, is3d = nd == 3, ax = a < 3 ? a : 0;
  const float *roi = rois + static_cast<long>(n) * roi_columns(nd, p.rotated);

  // ---- angle `ax`, axis `ax` of the roi -------------------------------------------------------
  double sn, cs;
  roi_trig(roi, p, ax, sn, cs);
  const int cells_all[3] = {p.ow, p.oh, p.od}, size_all[3] = {p.W, p.H, p.D}, ext_all[3] = {ps.tx, ps.ty, ps.tz};
  const int out_cells = ax == 0 ? cells_all[0] : (ax == 1 ? cells_all[1] : cells_all[2]);
  const int S = ax == 0 ? size_all[0] : (ax == 1 ? size_all[1] : size_all[2]);
  const int tile_ext = ax == 0 ? ext_all[0] : (ax == 1 ? ext_all[1] : ext_all[2]);
  const bool live_axis = ax < nd;
  double centre = 0.0, start = 0.0, bin = 0.0, sub = 0.0;
  int grid = 1;
  if (live_axis) {
    const double sc = p.scale;
    double ext;
    if (p.rotated) {
      ext = static_cast<double>(roi[1 + nd + ax]) * sc;
      if (!p.aligned) ext = fmax(ext, 1.0);
      centre = static_cast<double>(roi[1 + ax]) * sc - (p.aligned ? 0.5 : 0.0);
      start = -ext / 2.0;
    } else {
      const double lo = static_cast<double>(roi[1 + ax]) * sc, hi = static_cast<double>(roi[1 + nd + ax]) * sc;
      ext = fmax(hi - lo, 1.0);
      start = lo;
    }
    bin = ext / static_cast<double>(out_cells);
    grid = p.sampling_ratio > 0 ? p.sampling_ratio : static_cast<int>(ceil(ext / static_cast<double>(out_cells)));
    if (ps.flat_axis && ax == 1) grid = 1;
    sub = bin / static_cast<double>(grid > 0 ? grid : 1);
  }
  const int b = static_cast<int>(roi[0]);
  const int batch = (b >= 0 && b < p.N) ? b : -1;

  // ---- row `ax` of the rotation ----------------------------------------------------------------
  double row[3] = {ax == 0 ? 1.0 : 0.0, ax == 1 ? 1.0 : 0.0, ax == 2 ? 1.0 : 0.0};
  if (p.rotated) {
    const double sg = lane_get(sn, base), cg = lane_get(cs, base);
    const double sb = lane_get(sn, base + 1), cb = lane_get(cs, base + 1);
    const double sa = lane_get(sn, base + 2), ca = lane_get(cs, base + 2);
    if (is3d) {
      if (ax == 0) { row[0] = ca * cb; row[1] = ca * sb * sg - sa * cg; row[2] = ca * sb * cg + sa * sg; }
      else if (ax == 1) { row[0] = sa * cb; row[1] = sa * sb * sg + ca * cg; row[2] = sa * sb * cg - ca * sg; }
      else { row[0] = -sb; row[1] = cb * sg; row[2] = cb * cg; }
    } else {   // one angle, held by lane 0 of the group
      if (ax == 0) { row[0] = cg; row[1] = -sg; }
      else if (ax == 1) { row[0] = sg; row[1] = cg; }
    }
  }

  // ---- the tile along axis `ax` -----------------------------------------------------------------
  const unsigned qx = ps.by_tiles_x.div(tile), qy = ps.by_tiles_y.div(qx);
  const int tpos = ax == 0 ? static_cast<int>(tile - qx * ps.tiles_x)
                           : (ax == 1 ? static_cast<int>(qx - qy * ps.tiles_y) : static_cast<int>(qy));
  const int t0 = tpos * tile_ext;
  const int cells = min(tile_ext, out_cells - t0);
  const double first = live_axis ? start + t0 * bin + static_cast<double>(.5f) * sub : 0.0;
  // (from the first sample of the tile's first cell to the last sample of its last cell)
  const double half = live_axis ? 0.5 * ((cells - 1) * bin + (grid - 1) * sub) : 0.0;
  double mid = centre, reach = 0.0, pos = centre, inc[3];
  int grids = 1;
#pragma unroll
  for (int j = 0; j < 3; j++) {
    const double fj = lane_get(first, base + j), hj = lane_get(half, base + j), bj = lane_get(bin, base + j);
    const int gj = lane_get(grid, base + j);
    mid += row[j] * (fj + hj);
    reach += fabs(row[j] * hj);
    pos += row[j] * fj;
    inc[j] = j < nd ? row[j] * bj : 0.0;
    if (j < nd && gj != 1) grids = 0;
  }
  int lo = 0, cnt = 1, empty = 0, clipped = 0;
  double org = 0.0;
  if (is3d || ax < 2) {
    // widen by more than the rounding of the per-voxel coordinate arithmetic
    const double eps = 4e-5, rmin = mid - reach - eps, rmax = mid + reach + eps;
    empty = rmax < -1.0 || rmin > S || grid <= 0;   // (an adaptive grid of a roi without extent: no samples, zeros)
    clipped = rmin < static_cast<double>(ps.halo_lo) || rmax > S - ps.halo_hi;
    int l = static_cast<int>(fmin(fmax(floor(fmax(rmin, 0.0)) - ps.halo_lo, 0.0), static_cast<double>(S - 1)));
    int h = static_cast<int>(fmin(floor(fmax(rmax, 0.0)) + ps.halo_hi, static_cast<double>(S - 1)));
    if (ax == 0 && ps.vec > 0) {  // whole 16-byte groups (vec is 4 or 8)
      const int sh = ps.vec == 8 ? 3 : 2;
      l = (l >> sh) << sh;
      h = min(((h >> sh) + 1) << sh, S) - 1;
    }
    lo = l;
    cnt = h - l + 1;
    org = pos - static_cast<double>(l);
  }
  const int n0 = lane_get(cnt, base), n1 = lane_get(cnt, base + 1), n2 = lane_get(cnt, base + 2);
  const int l0 = lane_get(lo, base), l1 = lane_get(lo, base + 1), l2 = lane_get(lo, base + 2);
  const int ty0 = lane_get(t0, base + 1), tz0 = lane_get(t0, base + 2);
  const int any_empty = lane_get(empty, base) | lane_get(empty, base + 1) | lane_get(empty, base + 2);
  const int any_clip = lane_get(clipped, base) | lane_get(clipped, base + 1) | lane_get(clipped, base + 2);
  // LDS row pitch: the row's 16-byte groups, or (unaligned rows) the row plus one finite pad
  const int groups = ps.vec > 0 ? n0 / ps.vec : 0;
  const int pitch = ps.vec > 0 ? n0 : n0 + 1;
  const int es = ps.es;
  // LDS elements from slice to slice.  The eight taps of a wavefront's 64 samples fall on rows and
  // slices all over the box; with slices 32 bytes past a multiple of 128 a model of the 32 banks
  // counts 3.6 clocks per 2-byte tap read instead of 4.2 and 4.5 instead of 5.1 per 4-byte one (rotations
  // of up to 30 degrees about three axes); other remainders and odd row pitches gave less.
  int slice_e = n1 * pitch;
  if (ps.pad_slices && n2 > 1) slice_e = (((slice_e * es - 32 + 127) & ~127) + 32) / es;
  const long hw = static_cast<long>(p.H) * p.W;
  const long vol = (static_cast<long>(batch < 0 ? 0 : batch) * p.C + chan) * (hw * p.D) * es;
  int span = 0;
  if (a == 0) {
    if (item == kDone) {
      dst->mode = 4;
    } else {
      // register staging: a pass copies `span` whole z-slices, one 16-byte group per lane
      int passes = 0;
      if (ps.vec > 0) {
        const int per_slice = n1 * groups;   // small integers: the float quotients below are exact
        const int sp = min(static_cast<int>(static_cast<float>(ps.threads) / static_cast<float>(per_slice)), n2);
        if (sp >= 1) {
          const int ps_ = static_cast<int>(static_cast<float>(n2 + sp - 1) / static_cast<float>(sp));
          if (ps_ <= ps.max_items) { span = sp; passes = ps_; }
        }
      }
      const bool fits = static_cast<long>(n2) * slice_e <= ps.cap;
      int mode;
      if (batch < 0 || any_empty || (!grids && !ps.grids)) mode = 0;   // (kernels without grids are launched at ratio 1)
      else if (!fits) mode = 2;
      else mode = any_clip ? 1 : 3;
      const int rp = span * n1;
      const long src = vol + ((static_cast<long>(l2) * p.H + l1) * p.W + l0) * es;
      dst->mode = mode;
      dst->passes = passes;
      dst->src_lo = static_cast<unsigned>(src); dst->src_hi = static_cast<unsigned>(src >> 32);
      dst->extent = static_cast<int>((((n2 - 1) * hw + static_cast<long>(n1 - 1) * p.W + n0) * es));
      dst->stride = static_cast<int>(span * hw * es);
      dst->inv_groups = 1.0f / static_cast<float>(max(groups, 1));
      dst->inv_rows = 1.0f / static_cast<float>(n1);
      dst->groups = groups; dst->by = n1;
      dst->rp = rp; dst->bz = n2; dst->span = span;
      dst->hop_b = span * slice_e * es;
      dst->gap_b = (slice_e - n1 * pitch) * es;
    }
  }
  if (!write) return;
  dst->map[a * 4] = org;
  dst->mapf[a * 4] = static_cast<float>(org);
#pragma unroll
  for (int j = 0; j < 3; j++) {
    dst->map[a * 4 + 1 + j] = inc[j];
    dst->mapf[a * 4 + 1 + j] = static_cast<float>(inc[j]);
  }
  dst->lo[a] = lo;
  dst->n[a] = cnt;
  dst->grid[a] = live_axis ? grid : 1;
  dst->t0[a] = t0;
  dst->cmaxf[a] = static_cast<float>(S - 1 - lo);
  dst->topf[a] = static_cast<float>(max(cnt - 2, 0));
  if (a != 0) return;
  const long outv = (static_cast<long>(n) * p.C + chan) * (static_cast<long>(p.od) * p.oh * p.ow) * es;
  dst->out_lo = static_cast<unsigned>(outv); dst->out_hi = static_cast<unsigned>(outv >> 32);
  dst->zcount = p.od - tz0;
  dst->pitch_b = pitch * es; dst->slice_b = slice_e * es;
  dst->dy_b = n1 > 1 ? pitch * es : 0; dst->dz_b = n2 > 1 ? slice_e * es : 0;
  dst->tile_off = ((tz0 * p.oh + ty0) * p.ow + t0) * es;
  dst->xlim = p.ow - t0; dst->ylim = p.oh - ty0;
  dst->roi = static_cast<int>(n);
  dst->batch = batch;
  dst->vol_lo = static_cast<unsigned>(vol); dst->vol_hi = static_cast<unsigned>(vol >> 32);
}

constexpr unsigned kChunk = 32;     // consecutive items dealt to one XCD
constexpr unsigned kPlanSlots = 16; // items per workgroup: their plan records are kept in LDS

// a wave-uniform value moved to a scalar register
__device__ __forceinline__ float uniform(float v) { return __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(v))); }
__device__ __forceinline__ double uniform(double v) {
  return __hiloint2double(__builtin_amdgcn_readfirstlane(__double2hiint(v)), __builtin_amdgcn_readfirstlane(__double2loint(v)));
}
__device__ __forceinline__ float clamp_ct(float v, float lo, float hi) { return __builtin_amdgcn_fmed3f(v, lo, hi); }
__device__ __forceinline__ double clamp_ct(double v, double lo, double hi) { return fmin(fmax(v, lo), hi); }
__device__ __forceinline__ float frac_of(float v) { return __builtin_amdgcn_fractf(v); }
__device__ __forceinline__ double frac_of(double v) { return __builtin_amdgcn_fract(v); }
__device__ __forceinline__ float mix(float w, float a, float b) { return fmaf(w, b, fmaf(-w, a, a)); }  // exact at w = 0, 1
__device__ __forceinline__ int div_small(int i, float inv) { return static_cast<int>((static_cast<float>(i) + 0.5f) * inv); }

// Box-relative limits (wave-uniform): coordinates clamp to [0, cmax] (a sample the clamp moves by
// more than 1 lies outside [-1, size] of the volume and is void); the low tap index is at most top = max(n - 2, 0) so that the high tap stays inside
// the box (a coordinate on the last voxel gets weight 1 on the high tap).
template <typename CT> struct BoxLimits { CT cmax[3], top[3]; int one; };

// Element index of the low corner and the three fractions.  fp32 coordinates: floor / fraction /
// index all in fp32 (indices stay far below 2^24, so the two FMAs are exact).
__device__ __forceinline__ int corner_index(float lx, float ly, float lz, int pitch, int slice,
                                            float pitch_f, float slice_f) {
  return static_cast<int>(fmaf(lz, slice_f, fmaf(ly, pitch_f, lx)));
}
__device__ __forceinline__ int corner_index(double lx, double ly, double lz, int pitch, int slice,
                                            float, float) {
  return __mul24(static_cast<int>(lz), slice) + __mul24(static_cast<int>(ly), pitch) + static_cast<int>(lx);
}

// Wide variant for samples taken straight from the feature map.
template <typename CT>
__device__ __forceinline__ long corner_index_wide(CT lx, CT ly, CT lz, int pitch, long slice) {
  return static_cast<long>(lz) * slice + static_cast<long>(static_cast<int>(ly)) * pitch + static_cast<int>(lx);
}

// One voxel from the staged box; (rx, ry, rz) are box-relative coordinates, dy / dz the element
// distance to the upper y / z neighbour (0 when the box is one row / slice thick).
// WIDE: `tile` is the feature map itself (box = whole map), indices need 64 bits.
template <typename T, typename CT, bool INTERIOR, int ORDER, bool WIDE = false>
__device__ __forceinline__ float staged_sample(const T *__restrict__ tile, CT rx, CT ry, CT rz,
                                               const BoxLimits<CT> &b, int pitch, long slice,
                                               float pitch_f, float slice_f, int dy, long dz) {
  bool ok = true;
  CT lx, ly, lz;
  if (INTERIOR) {  // all taps of all samples lie inside the box
    lx = floor(rx); ly = floor(ry); lz = floor(rz);
  } else {
    // void outside [vmin, vmax] = [-1, size] of the volume: wherever the clamp to [0, cmax] can
    // act it acts at the volume border (vmin = -1, vmax = cmax + 1), so "inside" is "moved by at
    // most 1 by the clamp" (the differences are exact: one operand is 0 or within a factor of 2)
    const CT ux = rx, uy = ry, uz = rz;
    rx = clamp_ct(rx, CT(0), b.cmax[0]);
    ry = clamp_ct(ry, CT(0), b.cmax[1]);
    rz = clamp_ct(rz, CT(0), b.cmax[2]);
    ok = fmax(fmax(fabs(ux - rx), fabs(uy - ry)), fabs(uz - rz)) <= CT(1);
    lx = fmin(floor(rx), b.top[0]); ly = fmin(floor(ry), b.top[1]); lz = fmin(floor(rz), b.top[2]);
  }
  const CT fx = rx - lx, fy = ry - ly, fz = rz - lz;
  const T *t = tile + (WIDE ? corner_index_wide(lx, ly, lz, pitch, slice)
                            : corner_index(lx, ly, lz, pitch, static_cast<int>(slice), pitch_f, slice_f));
  float v;
  if (ORDER == 0) {
    v = load(t + ((fz <= CT(0.5) ? 0 : dz) + (fy <= CT(0.5) ? 0 : dy) + (fx <= CT(0.5) ? 0 : 1)));
  } else {
    const float wx = static_cast<float>(fx), wy = static_cast<float>(fy), wz = static_cast<float>(fz);
    const float x00 = mix(wx, load(t), load(t + 1)), x01 = mix(wx, load(t + dy), load(t + dy + 1));
    const float x10 = mix(wx, load(t + dz), load(t + dz + 1));
    const float x11 = mix(wx, load(t + dz + dy), load(t + dz + dy + 1));
    v = mix(wz, mix(wy, x00, x01), mix(wy, x10, x11));
  }
  return ok ? v : 0.f;
}

// Order 3 from the staged box: clamped Catmull-Rom over 4 x 4 x 4 voxels (see cubic_tap in
// sampling.hpp).  INTERIOR: all 64 taps of all samples are voxels of the box, no test, no clamp.
// Otherwise a sample below -1 or above `size` (box-relative: b.cmax) is void, negatives snap to 0,
// and the tap indices base-1 .. base+2 are clamped into the box, whose clipped sides are the
// volume's own borders.  dy / dz are 0 for boxes one row / slice thick (images: every z tap reads
// slice 0 and the z weights sum to 1).
__device__ __forceinline__ void catmull_rom(float u, float (&w)[4]) {
  const float u2 = u * u, u3 = u2 * u;
  w[0] = -0.5f * u3 + u2 - 0.5f * u;
  w[1] = 1.5f * u3 - 2.5f * u2 + 1.f;
  w[2] = -1.5f * u3 + 2.f * u2 + 0.5f * u;
  w[3] = 0.5f * u3 - 0.5f * u2;
}

// ONE_ROW: the middle axis is one voxel thick (images as volumes of rows): its four taps are that voxel
// with weights that sum to 1 (0, 1, 0, 0 at the coordinate the one cell is sampled at), so they are left out.
template <typename T, typename CT, bool INTERIOR, bool WIDE, bool ONE_ROW = false>
__device__ __forceinline__ float staged_cubic(const T *__restrict__ tile, CT rx, CT ry, CT rz,
                                              const BoxLimits<CT> &b, int pitch, long slice, int dy, long dz) {
  // void samples: an all-zero bit mask applied to the result (kept as data so that the 64 taps
  // stay one straight-line block)
  unsigned keep = 0xffffffffu;
  if (!INTERIOR) {
    const bool ok = rx >= CT(-1) && rx <= b.cmax[0] && ry >= CT(-1) && ry <= b.cmax[1] && rz >= CT(-1) && rz <= b.cmax[2];
    keep = ok ? 0xffffffffu : 0u;
    rx = fmax(rx, CT(0)); ry = fmax(ry, CT(0)); rz = fmax(rz, CT(0));
  }
  const CT lx = floor(rx), ly = floor(ry), lz = floor(rz);
  float wx[4], wy[4], wz[4];
  catmull_rom(static_cast<float>(rx - lx), wx);
  catmull_rom(static_cast<float>(ry - ly), wy);
  catmull_rom(static_cast<float>(rz - lz), wz);
  float acc = 0.f;
  if (INTERIOR) {
    // `one` is 1, but only at run time: the four taps of a row must stay four 2-byte reads (merged
    // into one 8-byte read at 2-byte alignment they take the slow unaligned LDS path)
    const int one = b.one;
    const int ix = static_cast<int>(lx) - 1, iy = static_cast<int>(ly) - 1, iz = static_cast<int>(lz) - 1;
    const T *row = tile + (static_cast<long>(iz) * dz + static_cast<long>(iy) * dy + ix);
#pragma unroll
    for (int a = 0; a < 4; a++) {
      float plane = 0.f;
#pragma unroll
      for (int c = 0; c < 4; c++) {
        plane += wy[c] * (wx[0] * load(row) + wx[1] * load(row + one) + wx[2] * load(row + 2 * one) +
                          wx[3] * load(row + 3 * one));
        row += dy;
      }
      row += dz - 4 * static_cast<long>(dy);
      acc += wz[a] * plane;
    }
  } else {
    // element offsets fit 32 bits: LDS boxes trivially, feature maps by the host's size check
    const int bx = static_cast<int>(lx), by = static_cast<int>(ly), bz = static_cast<int>(lz);
    const int tx = static_cast<int>(b.top[0]), ty = static_cast<int>(b.top[1]), tz = static_cast<int>(b.top[2]);
    const int sy = WIDE ? pitch : dy, sz = static_cast<int>(WIDE ? slice : dz);
    int ox[4];
#pragma unroll
    for (int k = 0; k < 4; k++) ox[k] = min(max(bx - 1 + k, 0), tx);
#pragma unroll
    for (int a = 0; a < 4; a++) {
      const int za = min(max(bz - 1 + a, 0), tz) * sz;
      float plane = 0.f;
      if constexpr (ONE_ROW) {
        const T *row = tile + za;
        plane = wx[0] * load(row + ox[0]) + wx[1] * load(row + ox[1]) + wx[2] * load(row + ox[2]) + wx[3] * load(row + ox[3]);
      } else {
#pragma unroll
        for (int c = 0; c < 4; c++) {
          const T *row = tile + (za + min(max(by - 1 + c, 0), ty) * sy);
          plane += wy[c] * (wx[0] * load(row + ox[0]) + wx[1] * load(row + ox[1]) + wx[2] * load(row + ox[2]) +
                            wx[3] * load(row + ox[3]));
        }
      }
      acc += wz[a] * plane;
    }
  }
  (void)pitch; (void)slice;
  return __uint_as_float(__float_as_uint(acc) & keep);
}

// The lane's column of ZPL voxels, box-relative start b0..b2 and per-slice step s0..s2.
// `before(k)` runs ahead of voxel k while o[k] still holds the previous item's value.
template <typename T, typename CT, bool INTERIOR, int ORDER, int ZPL, bool WIDE = false, typename Hook>
__device__ __forceinline__ void staged_column(const T *__restrict__ tile, float (&o)[ZPL], CT b0, CT b1,
                                              CT b2, CT s0, CT s1, CT s2, const BoxLimits<CT> &lim,
                                              int pitch, long slice, int dy, long dz, Hook before) {
  const float pitch_f = uniform(static_cast<float>(pitch)), slice_f = uniform(static_cast<float>(slice));
#pragma unroll
  for (int k = 0; k < ZPL; k++) {
    const CT kk = static_cast<CT>(k);
    before(k);
    o[k] = staged_sample<T, CT, INTERIOR, ORDER, WIDE>(tile, b0 + kk * s0, b1 + kk * s1, b2 + kk * s2,
                                                       lim, pitch, slice, pitch_f, slice_f, dy, dz);
    // keep the scheduler from interleaving all voxels of the column (registers are scarce while
    // the next box is in flight)
    if (k % 2 == 1) __builtin_amdgcn_sched_barrier(0);
  }
}

// The scalar part of a plan record held by a wavefront: lane l keeps dword l of the first 64; fields
// are pulled into scalar registers with v_readlane.  The records live in LDS, written by the
// workgroup itself.
#define MV_PLAN_DW(field) (static_cast<int>(offsetof(TilePlan, field) / 4))
struct PlanLanes {
  unsigned v;
  __device__ __forceinline__ int i32(int dw) const { return static_cast<int>(__builtin_amdgcn_readlane(v, dw)); }
  __device__ __forceinline__ unsigned long u64(int dw) const {
    return (static_cast<unsigned long>(__builtin_amdgcn_readlane(v, dw + 1)) << 32) | __builtin_amdgcn_readlane(v, dw);
  }
};
// A field of a record read straight from LDS into a scalar register (paths that are not hot).
__device__ __forceinline__ int plan_scalar(const int *field) { return __builtin_amdgcn_readfirstlane(*field); }

// the coordinate map of a record in the coordinate type CT
template <typename CT> __device__ __forceinline__ const CT *plan_map(const TilePlan *r);
template <> __device__ __forceinline__ const float *plan_map<float>(const TilePlan *r) { return r->mapf; }
template <> __device__ __forceinline__ const double *plan_map<double>(const TilePlan *r) { return r->map; }

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

// One element through a buffer descriptor: offsets beyond the buffer drop the store, so lanes
// without an output need no branch.
template <typename T>
__device__ __forceinline__ void store_element(__amdgpu_buffer_rsrc_t rsrc, unsigned voff, int soff, float v) {
  const T t = store_cast<T>(v);
  if constexpr (sizeof(T) == 2) {
    unsigned short bits;
    __builtin_memcpy(&bits, &t, 2);
    __builtin_amdgcn_raw_buffer_store_b16(bits, rsrc, voff, soff, 0);
  } else {
    unsigned bits;
    __builtin_memcpy(&bits, &t, 4);
    __builtin_amdgcn_raw_buffer_store_b32(bits, rsrc, voff, soff, 0);
  }
}

constexpr unsigned kOutOfRange = 0x80000000u;  // beyond every buffer: the load returns zeros

// floor as an integer in one instruction
__device__ __forceinline__ int floor_int(float v) {
  int i;
  asm("v_cvt_flr_i32_f32 %0, %1" : "=v"(i) : "v"(v));
  return i;
}

// The eight taps of one voxel of an INTERIOR tile (all taps of all samples lie inside the staged
// box, coordinates are non-negative) with fp32 coordinates: floor as integer conversion, fraction
// by v_fract, the byte offset of the low corner from two 24-bit multiply-adds.  `issue` sends the
// LDS reads, `finish` blends; a column keeps the reads of the next voxel in flight while it
// blends the current one.  g = (pitch, slice, dy, dz) in bytes.
// fn(integral_constant<int, k>) for k = K .. N - 1
template <int K, int N, typename F> __device__ __forceinline__ void column_steps(F fn) {
  if constexpr (K < N) {
    fn(std::integral_constant<int, K>{});
    column_steps<K + 1, N>(fn);
  }
}

template <typename T> struct Taps {
  T v[8];
  float wx, wy, wz;
};
// (On this hardware a wavefront's v_add_f32 / v_sub_f32 / v_mul_f32 / v_add_u32 take half the time
// of three-operand and conversion instructions, so sums of products are written as separate
// multiplications and additions where that does not cost accuracy: contraction is switched off.)
template <typename T, int ORDER>
__device__ __forceinline__ void interior_issue(Taps<T> &q, const T *__restrict__ tile, float rx, float ry,
                                               float rz, const i32x4 g, float pitch_f, float slice_f) {
#pragma clang fp contract(off)
  const float lx = floorf(rx), ly = floorf(ry), lz = floorf(rz);
  q.wx = rx - lx; q.wy = ry - ly; q.wz = rz - lz;
  constexpr unsigned E = sizeof(T);
  // byte offset of the low corner, exact in fp32 (far below 2^24)
  const float row = ly * pitch_f, sl = lz * slice_f, xb = E == 2 ? lx + lx : lx * static_cast<float>(E);
  const unsigned at = static_cast<unsigned>((xb + row) + sl);
  const char *t = reinterpret_cast<const char *>(tile) + at;
  const unsigned dy = g.z, dz = g.w;
  if (ORDER == 0) {
    const unsigned off = (q.wz <= 0.5f ? 0u : dz) + (q.wy <= 0.5f ? 0u : dy) + (q.wx <= 0.5f ? 0u : E);
    q.v[0] = *reinterpret_cast<const T *>(t + off);
  } else {
    q.v[0] = *reinterpret_cast<const T *>(t);
    q.v[1] = *reinterpret_cast<const T *>(t + E);
    q.v[2] = *reinterpret_cast<const T *>(t + dy);
    q.v[3] = *reinterpret_cast<const T *>(t + dy + E);
    q.v[4] = *reinterpret_cast<const T *>(t + dz);
    q.v[5] = *reinterpret_cast<const T *>(t + dz + E);
    q.v[6] = *reinterpret_cast<const T *>(t + dz + dy);
    q.v[7] = *reinterpret_cast<const T *>(t + dz + dy + E);
  }
}
template <typename T, int ORDER, bool EXACT_ENDS>
__device__ __forceinline__ float interior_finish(const Taps<T> &q) {
  if (ORDER == 0) return load(&q.v[0]);
  // the last tap read comes first: one wait covers all eight
  const float x11 = mix(q.wx, load(&q.v[6]), load(&q.v[7])), x10 = mix(q.wx, load(&q.v[4]), load(&q.v[5]));
  const float x01 = mix(q.wx, load(&q.v[2]), load(&q.v[3])), x00 = mix(q.wx, load(&q.v[0]), load(&q.v[1]));
  if (EXACT_ENDS) return mix(q.wz, mix(q.wy, x00, x01), mix(q.wy, x10, x11));
  // fractions below 1: a + w * (b - a), the difference on the fast path
  const float y0 = fmaf(q.wy, x01 - x00, x00), y1 = fmaf(q.wy, x11 - x10, x10);
  return fmaf(q.wz, y1 - y0, y0);
}

// Coordinate of slice k of a column from that of slice 0 with additions and multiplications by
// 2 and 4 only (at most three roundings for k < 8): r(k) = r(k - 1) + s for odd k, r(k - 2) + 2 s
// for k = 2 mod 4, r(k - 4) + 4 s for multiples of 4.
struct ColumnCoord {
  float last[3], anchor[3];
  __device__ __forceinline__ void start(float b0, float b1, float b2) {
    last[0] = anchor[0] = b0; last[1] = anchor[1] = b1; last[2] = anchor[2] = b2;
  }
  template <int K> __device__ __forceinline__ void step(float s0, float s1, float s2) {
    const float s[3] = {s0, s1, s2};
#pragma unroll
    for (int a = 0; a < 3; a++) {
      if (K % 2 == 1) last[a] = last[a] + s[a];
      else if (K % 4 == 2) last[a] = fmaf(2.0f, s[a], anchor[a]);
      else { last[a] = fmaf(4.0f, s[a], anchor[a]); anchor[a] = last[a]; }
    }
  }
};

// The lane's column of ZPL voxels of an interior tile, fp32 coordinates.  `before(k)` runs ahead
// of voxel k while o[k] still holds the previous item's value.
template <typename T, int ORDER, int ZPL, typename Hook>
__device__ __forceinline__ void interior_column(const T *__restrict__ tile, float (&o)[ZPL], float b0, float b1,
                                                float b2, float s0, float s1, float s2, const i32x4 g, Hook before) {
  const float pitch_f = static_cast<float>(g.x), slice_f = static_cast<float>(g.y);
  Taps<T> cur, nxt;
  ColumnCoord r;
  r.start(b0, b1, b2);
  interior_issue<T, ORDER>(cur, tile, b0, b1, b2, g, pitch_f, slice_f);
  column_steps<0, ZPL>([&](auto kc) {
    constexpr int k = decltype(kc)::value;
    before(k);
    if constexpr (k + 1 < ZPL) {
      r.template step<k + 1>(s0, s1, s2);
      interior_issue<T, ORDER>(nxt, tile, r.last[0], r.last[1], r.last[2], g, pitch_f, slice_f);
    }
    __builtin_amdgcn_sched_barrier(0);
    o[k] = interior_finish<T, ORDER, false>(cur);
    cur = nxt;
    __builtin_amdgcn_sched_barrier(0);
  });
}

// The same for a CLIPPED box (some side of it is the volume's border), fp32 coordinates: the
// coordinate is clamped to [0, cmax]; a sample the clamp moves by more than 1 lies outside [-1, size]
// of the volume and is void (the differences are exact: one operand is 0 or within a factor of
// 2); the low tap index is at most `top`, so that the high tap stays inside the box (a
// coordinate on the last voxel gets weight 1 on the high tap).
template <typename T, int ORDER>
__device__ __forceinline__ bool clipped_issue(Taps<T> &q, const T *__restrict__ tile, float rx, float ry,
                                              float rz, const i32x4 g, const float (&cmax)[3], const float (&top)[3],
                                              float pitch_f, float slice_f) {
#pragma clang fp contract(off)
  const float cx = clamp_ct(rx, 0.f, cmax[0]), cy = clamp_ct(ry, 0.f, cmax[1]), cz = clamp_ct(rz, 0.f, cmax[2]);
  const bool ok = fmaxf(fmaxf(fabsf(rx - cx), fabsf(ry - cy)), fabsf(rz - cz)) <= 1.f;
  const float lx = fminf(floorf(cx), top[0]), ly = fminf(floorf(cy), top[1]), lz = fminf(floorf(cz), top[2]);
  q.wx = cx - lx; q.wy = cy - ly; q.wz = cz - lz;
  constexpr unsigned E = sizeof(T);
  // byte offset of the low corner, exact in fp32 (far below 2^24)
  const float row = ly * pitch_f, sl = lz * slice_f, xb = E == 2 ? lx + lx : lx * static_cast<float>(E);
  const unsigned at = static_cast<unsigned>((xb + row) + sl);
  const char *t = reinterpret_cast<const char *>(tile) + at;
  const unsigned dy = g.z, dz = g.w;
  if (ORDER == 0) {
    const unsigned off = (q.wz <= 0.5f ? 0u : dz) + (q.wy <= 0.5f ? 0u : dy) + (q.wx <= 0.5f ? 0u : E);
    q.v[0] = *reinterpret_cast<const T *>(t + off);
  } else {
    q.v[0] = *reinterpret_cast<const T *>(t);
    q.v[1] = *reinterpret_cast<const T *>(t + E);
    q.v[2] = *reinterpret_cast<const T *>(t + dy);
    q.v[3] = *reinterpret_cast<const T *>(t + dy + E);
    q.v[4] = *reinterpret_cast<const T *>(t + dz);
    q.v[5] = *reinterpret_cast<const T *>(t + dz + E);
    q.v[6] = *reinterpret_cast<const T *>(t + dz + dy);
    q.v[7] = *reinterpret_cast<const T *>(t + dz + dy + E);
  }
  return ok;
}
template <typename T, int ORDER, int ZPL, typename Hook>
__device__ __forceinline__ void clipped_column(const T *__restrict__ tile, float (&o)[ZPL], float b0, float b1,
                                               float b2, float s0, float s1, float s2, const i32x4 g,
                                               const float (&cmax)[3], const float (&top)[3], Hook before) {
  const float pitch_f = static_cast<float>(g.x), slice_f = static_cast<float>(g.y);
  Taps<T> cur, nxt;
  ColumnCoord r;
  r.start(b0, b1, b2);
  bool ok = clipped_issue<T, ORDER>(cur, tile, b0, b1, b2, g, cmax, top, pitch_f, slice_f), ok_next = false;
  column_steps<0, ZPL>([&](auto kc) {
    constexpr int k = decltype(kc)::value;
    before(k);
    if constexpr (k + 1 < ZPL) {
      r.template step<k + 1>(s0, s1, s2);
      ok_next = clipped_issue<T, ORDER>(nxt, tile, r.last[0], r.last[1], r.last[2], g, cmax, top, pitch_f, slice_f);
    }
    __builtin_amdgcn_sched_barrier(0);
    const float v = interior_finish<T, ORDER, true>(cur);
    o[k] = ok ? v : 0.f;
    cur = nxt;
    ok = ok_next;
    __builtin_amdgcn_sched_barrier(0);
  });
}

// Persistent workgroups: each takes every `slots`-th item (tile, channel) of its XCD's contiguous
// range.  Per item:   write the box (loaded into registers during the previous item) to LDS |
// barrier | store the previous item's outputs, issue the global loads of the next item's box |
// interpolate this item from LDS into registers | barrier.  Global latency is thereby covered by
// the interpolation of the previous item, and stores by that of the next.
// Box rows are copied as 16-byte groups with range-checked buffer loads: lane = (slice, row,
// group) within a pass of `span` z-slices, one register quad per pass, passes `span` slices apart.
// Everything that is the same for all lanes of an item (addresses, extents, LDS geometry) is in
// the item's record, so a wavefront spends a handful of v_readlane and broadcast reads per item;
// conditions that hold for a whole wavefront (a pass that exists, an output slice that exists)
// select between the real buffer extent and an empty one on the scalar unit.
// G > 1: the problem handed in is the one on the G times finer grid of the bins' samples (cell * G + sub
// of a fixed sampling grid of G per axis), and every G x G x G block of its voxels leaves as one mean:
// G slices summed in the lane, the x and y neighbours through lane exchanges, one store per block.
// G = 0: any sampling grid, fixed or per roi (ceil(roi extent / cells)): the problem is the one asked for,
// a lane walks the samples of each of its bins in a loop (the plan holds the grid of the item's roi and
// a box that covers every sample) and keeps their sum in a register.
template <typename T, int TX, int TY, int TZ, int THREADS, int LDS_BYTES, int KMAX, int ORDER, int G = 1>
__global__ __launch_bounds__(THREADS, 4) void roi_resample_kernel(
    const T *__restrict__ feat, const float *__restrict__ rois, T *__restrict__ out, const RoiProblem p, const PlanShape ps, const unsigned total, const unsigned work) {
  using CT = typename std::conditional<(sizeof(T) == 2), float, double>::type;
  constexpr int kCap = LDS_BYTES / sizeof(T);
  constexpr int RZ = THREADS / (TX * TY);  // lane layers along z
  static_assert(RZ >= 1 && RZ * TX * TY == THREADS && TZ % RZ == 0, "tile shape");
  static_assert((TX * TY) % kWave == 0, "a wavefront's lanes share their z layer");
  constexpr int ZPL = TZ / RZ;             // consecutive output slices per lane
  constexpr int ES = sizeof(T);
  constexpr int GO = G > 1 ? G : 1;        // output voxels are means of GO^3 (images: GO^2) voxels of the problem
  constexpr int ZO = ZPL / GO;             // slices a lane stores
  // (images as volumes of rows, TY = 1: the middle axis has one cell and takes no part; blocks of G x G)
  constexpr int GY = TY == 1 ? 1 : GO;
  static_assert(G <= 1 || (ZPL % G == 0 && TX % G == 0 && kWave % TX == 0 &&
                           (TY == 1 || ((kWave / TX) % G == 0 && TY % (kWave / TX) == 0))),
                "blocks of G x G x G voxels lie inside a wavefront's lanes and a lane's column");
  __shared__ __attribute__((aligned(16))) T tile[kCap];
  __shared__ __attribute__((aligned(16))) TilePlan lplans[kPlanSlots];
  const int H = p.H, W = p.W, oh = p.oh, ow = p.ow;

  // Work distribution: items (channel * tiles + tile) are dealt to the XCDs in chunks of kChunk
  // consecutive items (workgroup ids go round-robin over the XCDs, each with an L2 of its own, so
  // tiles processed at the same time share their halos there).  In round i the workgroups of an
  // XCD take the next `slots` positions of its queue, each workgroup a different one; the
  // assignment is rotated from round to round so that a workgroup does not get the same tile
  // position (border: cheap, centre: expensive) in every roi.
  const int tid = threadIdx.x;
  MV_TL(0);
  [[maybe_unused]] int tl_item = 0;
  const unsigned per_roi = static_cast<unsigned>(ps.tiles_x) * ps.tiles_y * ps.tiles_z;
  auto fetch_plan = [&](unsigned r) -> PlanLanes {
    PlanLanes pl;
    pl.v = reinterpret_cast<const unsigned *>(&lplans[r])[tid & (kWave - 1)];
    return pl;
  };
  unsigned round = 0;
  int mode = 4;

  // what a lane keeps for the whole kernel: its place in the tile and in the copy passes
  const int lx = tid % TX, ly = (tid / TX) % TY, lz = tid / (TX * TY);
  const CT fx = static_cast<CT>(lx), fy = static_cast<CT>(ly), fz = static_cast<CT>(lz * ZPL);
  const float tid_h = static_cast<float>(tid) + 0.5f;
  const int oh_o = oh / GY, ow_o = ow / GO;   // the volume that is written
  const int zbytes = oh_o * ow_o * ES;
  const int out_bytes = (p.od / GO) * zbytes;   // bytes of one output volume (< 2^31, checked by the host)
  const unsigned lane_out = static_cast<unsigned>(((lz * ZO * oh_o + ly / GY) * ow_o + lx / GO) * ES);
  const bool lane_stores = lx % GO == 0 && ly % GY == 0;
  const int w_bytes = W * ES;
  const unsigned hw_bytes = static_cast<unsigned>(H) * W * ES;   // < 2^31, checked by the host
  // lane `tid` holds group `tid` of every pass: its place in LDS, slices `gap` bytes apart
  unsigned st_off = tid * 16;

  u32x4 val[KMAX];   // the next item's box: 16-byte group (zz0 + u * span, yy, gi) in val[u]
  int st_zz = 0;     // zz0 of this lane (beyond every box for idle lanes)
  float o[ZPL];      // the previous item's outputs
  [[maybe_unused]] float held[ZO];   // G > 1: the previous item's means (o then belongs to the current item)
  auto pending = [&](int k) -> float {
    if constexpr (G <= 1) return o[k];
    else return held[k];
  };
  // outputs waiting to be stored: the (roi, channel) volume, the lane's byte offset in it (out of
  // range for lanes beyond the output's rows / columns)
  const char *pend_base = reinterpret_cast<const char *>(out);
  unsigned pend_voff = kOutOfRange;
  int pend_bytes = 0;   // 0 until there is something to store

  // The loads of one item's box into val[]: the buffer ends with the box's last row.  `prepare`
  // sets the addresses up and returns the item's mode (4: there is no such item).
  const char *ld_base = reinterpret_cast<const char *>(feat);
  int ld_extent = 0;
  unsigned ld_voff = kOutOfRange;
  int ld_stride = 0, ld_passes = 0;
  // `pl`: the record's scalar part, `sp` = (1 / groups, 1 / rows as float bits, groups, rows), `rp`:
  // read by the caller well ahead (one batch of LDS reads per item).
  auto prepare = [&](bool exists, const PlanLanes &pl, const i32x4 sp, int rp, int gap_b) -> int {
    ld_passes = 0;
    ld_extent = 0;    // an empty buffer: every load returns zeros
    if (!exists) return 4;
    const int m = pl.i32(MV_PLAN_DW(mode));
    const int passes = pl.i32(MV_PLAN_DW(passes));
    if (m == 4 || (m & 1) == 0 || passes == 0) return m;   // staged modes are 1 and 3
    const float inv_groups = __int_as_float(sp.x), inv_rows = __int_as_float(sp.y);
    const int groups = sp.z, by = sp.w;
    const int lr = static_cast<int>(tid_h * inv_groups), gi = tid - __mul24(lr, groups);
    const int zz = static_cast<int>((static_cast<float>(lr) + 0.5f) * inv_rows), yy = lr - __mul24(zz, by);
    ld_base = reinterpret_cast<const char *>(feat) + pl.u64(MV_PLAN_DW(src_lo));
    ld_extent = pl.i32(MV_PLAN_DW(extent));
    ld_stride = pl.i32(MV_PLAN_DW(stride));
    ld_passes = passes;
    const bool on = lr < rp;
    ld_voff = on ? static_cast<unsigned>(zz) * hw_bytes + static_cast<unsigned>(__mul24(yy, w_bytes) + gi * 16) : kOutOfRange;
    st_zz = on ? zz : (1 << 28);
    st_off = tid * 16 + __mul24(zz, gap_b);
    return m;
  };
  // Pass u.  The scalar offset takes part in the range check, so a pass beyond the box's last
  // slice (u >= ld_passes) reads zeros without touching memory.
  auto load_pass = [&](int u) {
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(ld_base), 0, ld_extent, 0x00020000);
    val[u] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, ld_voff, u * ld_stride, 0);
  };
  // While the first wavefront plans, the others pull this workgroup's share of a small input through
  // the caches: the workgroups' first boxes, requested all at once when the plans are ready, then
  // come from the caches instead of from memory in one burst.
  if (tid >= kWave && ps.warm_groups > 0) {
    const unsigned per = (ps.warm_groups + gridDim.x - 1) / gridDim.x, first = blockIdx.x * per;
    const unsigned *words = reinterpret_cast<const unsigned *>(feat);
    unsigned seen = 0;
    // (one word per 16-byte group: four neighbouring lanes share a 64-byte sector, which costs four
    // times the instructions of one lane per sector and was measured 1.1 us faster)
    for (unsigned i = tid - kWave; i < per; i += THREADS - kWave)
      if (first + i < ps.warm_groups) seen |= words[static_cast<size_t>(first + i) * kWarmStride];
    asm volatile("" ::"v"(seen));
  }
  // The first wavefront plans this workgroup's items (at most kPlanSlots), four lanes per item.
  if (tid < kWave) {
    static_assert(kPlanSlots * 4 == kWave, "four lanes per plan slot");
    const unsigned parts = gridDim.x >= kXcds ? kXcds : 1;
    const unsigned xcd = parts > 1 ? blockIdx.x % kXcds : 0, slot = parts > 1 ? blockIdx.x / kXcds : blockIdx.x;
    const unsigned slots = gridDim.x / parts;
    const unsigned r = tid >> 2;
    const unsigned sr = slot + r * 27u;
    const unsigned k = r * slots + (sr - ps.by_slots.div(sr) * slots);
    const unsigned item = ((k / kChunk) * parts + xcd) * kChunk + k % kChunk;
    MV_TL(1);
    plan_item_lanes(rois, p, ps, item < work ? item : kDone, total, per_roi, &lplans[r]);
    MV_TL(2);
  }
  __syncthreads();
  MV_TL(3);
  mode = prepare(true, fetch_plan(0), *reinterpret_cast<const i32x4 *>(&lplans[0].inv_groups), lplans[0].rp, lplans[0].gap_b);
  if (mode == 4) return;
#pragma unroll
  for (int u = 0; u < KMAX; u++)
    if (u < ld_passes) load_pass(u);
  while (true) {
    // everything this item needs from its record and the next one's, requested in one batch ahead
    // of the wait for the box (the records are read-only from here on)
    const TilePlan *rec = &lplans[round];
    const bool has_next = round + 1 < kPlanSlots;
    const TilePlan *nrec = &lplans[has_next ? round + 1 : round];
    const PlanLanes plan = fetch_plan(round);
    PlanLanes nplan;
    nplan.v = reinterpret_cast<const unsigned *>(nrec)[tid & (kWave - 1)];
    const i32x4 nsp = *reinterpret_cast<const i32x4 *>(&nrec->inv_groups);
    const int nrp = nrec->rp, ngap = nrec->gap_b;
    const i32x4 cpy = *reinterpret_cast<const i32x4 *>(&rec->rp);          // rp, -, bz, span
    const i32x4 g = *reinterpret_cast<const i32x4 *>(&rec->pitch_b);       // pitch, slice, dy, dz in bytes
    const i32x4 t = *reinterpret_cast<const i32x4 *>(&rec->tile_off);      // tile_off, xlim, ylim, hop_b
    CT m[12];
#pragma unroll
    for (int i = 0; i < 12; i++) m[i] = plan_map<CT>(rec)[i];
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const f32x4 lim4 = *reinterpret_cast<const f32x4 *>(rec->cmaxf), top4 = *reinterpret_cast<const f32x4 *>(rec->topf);
    const bool staged = (mode & 1) != 0;

    // ---- A: the box into LDS ---------------------------------------------------------------
    // All loads issued for this item have to be back; waiting here on every path (vmcnt(0), other
    // counters untouched) keeps the compiler from waiting again after the stores of phase B.
    __builtin_amdgcn_s_waitcnt(0x0F70);
    if (tl_item == 0) MV_TL(4);
    if (staged) {
      if (ld_passes > 0) {   // still this item's: the next `prepare` comes after the barrier
        const int bz = cpy.z, span = cpy.w, hop_b = t.w;
        int zc = st_zz;
        char *dst = reinterpret_cast<char *>(tile) + st_off;
#pragma unroll
        for (int u = 0; u < KMAX; u++) {
          if (u < ld_passes) {   // a scalar branch
            if (zc < bz) *reinterpret_cast<u32x4 *>(dst) = val[u];
            zc += span;
            dst += hop_b;
          }
        }
      } else {
        // boxes with very long rows, very many slices or unaligned rows: straight from global memory
        const int bx = plan_scalar(&rec->n[0]), by = plan_scalar(&rec->n[1]), bz = plan_scalar(&rec->n[2]);
        const int vec = ps.vec, pitch = vec > 0 ? bx : bx + 1, rows = by * bz, gap = cpy.y / ES;
        const T *corner = reinterpret_cast<const T *>(
            reinterpret_cast<const char *>(feat) + plan.u64(MV_PLAN_DW(src_lo)));
        const float inv_by = rec->inv_rows;
        if (vec > 0) {
          const int groups = bx / vec;
          const float inv_groups = rec->inv_groups;
          for (int i = tid; i < rows * groups; i += THREADS) {
            const int r = div_small(i, inv_groups), gi = i - r * groups;
            const int zz = div_small(r, inv_by), yy = r - zz * by;
            *reinterpret_cast<u32x4 *>(tile + r * pitch + zz * gap + gi * vec) =
                *reinterpret_cast<const u32x4 *>(corner + (static_cast<long>(zz) * H + yy) * W + gi * vec);
          }
        } else {
          int lpr = 1;
          while (lpr < pitch && lpr < kWave) lpr *= 2;
          const int lane_e = tid & (lpr - 1), lane_r = tid / lpr;
          for (int r = lane_r; r < rows; r += THREADS / lpr) {
            const int zz = div_small(r, inv_by), yy = r - zz * by;
            const T *row = corner + (static_cast<long>(zz) * H + yy) * W;
            for (int e = lane_e; e < pitch; e += lpr) tile[r * pitch + zz * gap + e] = e < bx ? row[e] : store_cast<T>(0.f);
          }
        }
      }
    }
    __syncthreads();

    if (tl_item < 4) MV_TL(5 + tl_item);
    tl_item++;
    // ---- B + C: this item; ahead of voxel k the previous item's voxel k is stored and a share of
    // the next box's loads is issued, so that neither piles up in the memory pipeline -------------
    const int next_mode = prepare(has_next, nplan, nsp, nrp, ngap);
    auto before = [&](int k) {
      // (slices beyond the volume's last one are beyond the buffer: scalar offsets are range-checked)
      const __amdgpu_buffer_rsrc_t rsrc =
          __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(pend_base), 0, pend_bytes, 0x00020000);
      if (k < ZO) store_element<T>(rsrc, pend_voff, k * zbytes, pending(k));
#pragma unroll
      for (int u = 0; u < KMAX; u++)
        if (u >= k * KMAX / ZPL && u < (k + 1) * KMAX / ZPL) load_pass(u);   // compile-time share of the loads
    };
    if (mode == 0) {
#pragma unroll
      for (int k = 0; k < ZPL; k++) {
        before(k);
        o[k] = 0.f;
      }
    } else {
      // position of this lane's first voxel and the per-slice increment, relative to the box (to
      // the feature map for mode 2), in the coordinate type (the box margin covers the rounding
      // of fp32 arithmetic); the record's values come as broadcast reads.  Lanes beyond the
      // output run the same code: their reads stay inside the box or miss the LDS (zeros), and
      // their stores are dropped.
      CT b[3], st[3];
#pragma unroll
      for (int a = 0; a < 3; a++) {
        b[a] = m[4 * a] + fx * m[4 * a + 1] + fy * m[4 * a + 2] + fz * m[4 * a + 3];
        st[a] = m[4 * a + 3];
      }
      if constexpr (G == 0) {
        // every sample of the bins: sample (ix, iy, iz) of a bin lies ix / gx, iy / gy, iz / gz of a cell
        // further along the output axes (the plan's origin is sample (0, 0, 0) of the tile's first cell)
        const int gx = plan.i32(MV_PLAN_DW(grid)), gy = plan.i32(MV_PLAN_DW(grid) + 1), gz = plan.i32(MV_PLAN_DW(grid) + 2);
        const CT igx = CT(1) / static_cast<CT>(gx), igy = CT(1) / static_cast<CT>(gy), igz = CT(1) / static_cast<CT>(gz);
        CT sx[3], sy[3], sz[3];
#pragma unroll
        for (int a = 0; a < 3; a++) { sx[a] = m[4 * a + 1] * igx; sy[a] = m[4 * a + 2] * igy; sz[a] = m[4 * a + 3] * igz; }
        const float inv_count = 1.f / (static_cast<float>(gx) * static_cast<float>(gy) * static_cast<float>(gz));
        const int size[3] = {W, H, p.D};
        BoxLimits<CT> lim;
#pragma unroll
        for (int a = 0; a < 3; a++) {
          const int lo = mode == 2 ? 0 : plan_scalar(&rec->lo[a]);
          const int n = mode == 2 ? size[a] : plan_scalar(&rec->n[a]);
          lim.cmax[a] = uniform(static_cast<CT>(size[a] - 1 - lo));
          lim.top[a] = uniform(static_cast<CT>(max(n - 2, 0)));
        }
        auto bins = [&](auto wide_tag, const T *base, int pitch, long slice, int dy, long dz) {
          constexpr bool kWide = decltype(wide_tag)::value;
          const float pitch_f = uniform(static_cast<float>(pitch)), slice_f = uniform(static_cast<float>(slice));
#pragma unroll
          for (int k = 0; k < ZPL; k++) {
            before(k);
            const CT kk = static_cast<CT>(k);
            const CT c0 = b[0] + kk * st[0], c1 = b[1] + kk * st[1], c2 = b[2] + kk * st[2];
            float acc = 0.f;
            for (int iz = 0; iz < gz; iz++)
              for (int iy = 0; iy < gy; iy++) {
                const CT fz_ = static_cast<CT>(iz), fy_ = static_cast<CT>(iy);
                const CT r0 = c0 + fy_ * sy[0] + fz_ * sz[0], r1 = c1 + fy_ * sy[1] + fz_ * sz[1], r2 = c2 + fy_ * sy[2] + fz_ * sz[2];
                for (int ix = 0; ix < gx; ix++) {
                  const CT fx_ = static_cast<CT>(ix);
                  acc += staged_sample<T, CT, false, ORDER, kWide>(base, r0 + fx_ * sx[0], r1 + fx_ * sx[1], r2 + fx_ * sx[2],
                                                                   lim, pitch, slice, pitch_f, slice_f, dy, dz);
                }
              }
            o[k] = acc * inv_count;
          }
        };
        if (mode == 2) {   // the box does not fit in LDS: taps straight from the feature map
          for (int a = 0; a < 3; a++) b[a] += static_cast<CT>(plan_scalar(&rec->lo[a]));
          const T *src = reinterpret_cast<const T *>(
              reinterpret_cast<const char *>(feat) +
              ((static_cast<unsigned long>(static_cast<unsigned>(plan_scalar(reinterpret_cast<const int *>(&rec->vol_hi)))) << 32) |
               static_cast<unsigned>(plan_scalar(reinterpret_cast<const int *>(&rec->vol_lo)))));
          const long hw = static_cast<long>(H) * W;
          bins(std::true_type{}, src, W, hw, H > 1 ? W : 0, p.D > 1 ? hw : 0);
        } else {
          bins(std::false_type{}, tile, g.x / ES, g.y / ES, g.z / ES, g.w / ES);
        }
      } else if (mode == 3 && sizeof(CT) == 4) {
        if constexpr (sizeof(CT) == 4)
          interior_column<T, ORDER, ZPL>(tile, o, b[0], b[1], b[2], st[0], st[1], st[2], g, before);
      } else if (mode == 1 && sizeof(CT) == 4) {
        if constexpr (sizeof(CT) == 4) {
          const float cmax[3] = {lim4.x, lim4.y, lim4.z}, top[3] = {top4.x, top4.y, top4.z};
          clipped_column<T, ORDER, ZPL>(tile, o, b[0], b[1], b[2], st[0], st[1], st[2], g, cmax, top, before);
        }
      } else {
        const int pitch = g.x / ES, slice = g.y / ES, dy = g.z / ES, dz = g.w / ES;
        BoxLimits<CT> lim;
        if (mode == 3) {
          staged_column<T, CT, true, ORDER, ZPL>(tile, o, b[0], b[1], b[2], st[0], st[1], st[2], lim, pitch, slice, dy, dz, before);
        } else {
          const int size[3] = {W, H, p.D};
#pragma unroll
          for (int a = 0; a < 3; a++) {
            const int lo = mode == 2 ? 0 : plan_scalar(&rec->lo[a]);
            const int n = mode == 2 ? size[a] : plan_scalar(&rec->n[a]);
            lim.cmax[a] = uniform(static_cast<CT>(size[a] - 1 - lo));
            lim.top[a] = uniform(static_cast<CT>(max(n - 2, 0)));
          }
          if (mode == 2) {  // the box does not fit in LDS: taps straight from the feature map
            for (int a = 0; a < 3; a++) b[a] += static_cast<CT>(plan_scalar(&rec->lo[a]));
            const T *src = reinterpret_cast<const T *>(
                reinterpret_cast<const char *>(feat) +
                ((static_cast<unsigned long>(static_cast<unsigned>(plan_scalar(reinterpret_cast<const int *>(&rec->vol_hi)))) << 32) |
                 static_cast<unsigned>(plan_scalar(reinterpret_cast<const int *>(&rec->vol_lo)))));
            const long hw = static_cast<long>(H) * W;
            const int dyw = H > 1 ? W : 0;
            const long dzw = p.D > 1 ? hw : 0;
            staged_column<T, CT, false, ORDER, ZPL, true>(src, o, b[0], b[1], b[2], st[0], st[1], st[2], lim, W, hw, dyw, dzw, before);
          } else {
            staged_column<T, CT, false, ORDER, ZPL>(tile, o, b[0], b[1], b[2], st[0], st[1], st[2], lim, pitch, slice, dy, dz, before);
          }
        }
      }
    }
    if constexpr (G <= 1) {
      pend_base = reinterpret_cast<const char *>(out) + plan.u64(MV_PLAN_DW(out_lo));
      pend_voff = (lx < t.y && ly < t.z) ? lane_out + static_cast<unsigned>(t.x) : kOutOfRange;
      pend_bytes = out_bytes;
    } else {
      // means of the blocks: slices in the lane, then the lanes G - 1 to the right and G - 1 rows on
#pragma unroll
      for (int kk = 0; kk < ZO; kk++) {
        float sum = o[kk * G];
#pragma unroll
        for (int j = 1; j < G; j++) sum += o[kk * G + j];
        sum += __shfl_down(sum, 1);
        if (G == 4) sum += __shfl_down(sum, 2);
        if constexpr (GY > 1) {
          sum += __shfl_down(sum, TX);
          if (G == 4) sum += __shfl_down(sum, 2 * TX);
        }
        held[kk] = sum * (1.f / static_cast<float>(G * GY * G));
      }
      // the (roi, channel) volume and the tile's first block in it (tile origins are multiples of G)
      const int bx = plan_scalar(&rec->t0[0]) / G, by0 = plan_scalar(&rec->t0[1]) / GY, bz0 = plan_scalar(&rec->t0[2]) / G;
      pend_base = reinterpret_cast<const char *>(out) + plan.u64(MV_PLAN_DW(out_lo)) / (G * GY * G);
      pend_voff = (lane_stores && lx < t.y && ly < t.z)
                      ? lane_out + static_cast<unsigned>(((bz0 * oh_o + by0) * ow_o + bx) * ES) : kOutOfRange;
      pend_bytes = out_bytes;
    }
    if (next_mode == 4) break;
    __syncthreads();  // every lane is done with the box
    mode = next_mode;
    round++;
  }
#pragma unroll
  for (int k = 0; k < ZO; k++) {
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(pend_base), 0, pend_bytes, 0x00020000);
    store_element<T>(rsrc, pend_voff, k * zbytes, pending(k));
  }
#ifdef MV_RESAMPLE_TIMELINE
  MV_TL(9);
  __builtin_amdgcn_s_waitcnt(0);
  MV_TL(10);
#endif
}

// Compute units of the current device (workgroups resident at once = units * LDS share).

// One output index of an axis-aligned order-3 tile: the four clamped box indices and weights of its taps
struct AxisTaps3 {
  int idx[4];
  float w[4];
};

// Order-3 twin of the kernel above, kept simple because 64 taps per voxel dominate everything
// else: same items, same work distribution and plans (boxes carry a halo of 1 / 2 voxels), but
// the box is copied to LDS in place (no register prefetch) and every lane walks its column of
// voxels in a rolled loop, storing as it goes.
// A roi without rotation (resizes, the control-grid upsampling of the elastic deformation) has
// separable taps: the tile then contracts x, y and z one after the other through two fp32
// intermediates in the unused part of the LDS tile (4 + 4 + 4 taps per voxel and less instead of 64),
// with the same per-axis weights, indices and void rule as the general form.
template <typename T, int TX, int TY, int TZ, int THREADS, int LDS_BYTES>
__global__ __launch_bounds__(THREADS, 4) void roi_resample_cubic_kernel(
    const T *__restrict__ feat, const float *__restrict__ rois, T *__restrict__ out, const RoiProblem p,
    const PlanShape ps, const unsigned total, const unsigned work) {
  using CT = typename std::conditional<(sizeof(T) == 2), float, double>::type;
  constexpr int kCap = LDS_BYTES / sizeof(T);
  constexpr int RZ = THREADS / (TX * TY), ZPL = TZ / RZ, V = 16 / sizeof(T);
  __shared__ __attribute__((aligned(16))) T tile[kCap];
  __shared__ TilePlan lplans[kPlanSlots];
  const int C = p.C, D = p.D, H = p.H, W = p.W, od = p.od, oh = p.oh, ow = p.ow;
  const int vec = ps.vec;
  const unsigned parts = gridDim.x >= kXcds ? kXcds : 1;
  const unsigned xcd = blockIdx.x % parts, slot = blockIdx.x / parts, slots = gridDim.x / parts;
  auto item_of = [&](unsigned round) -> unsigned {
    const unsigned k = round * slots + (slot + round * 27u) % slots;
    const unsigned item = ((k / kChunk) * parts + xcd) * kChunk + k % kChunk;
    return item < work ? item : kDone;
  };
  const int tid = threadIdx.x;
  if (item_of(0) == kDone) return;
  const unsigned per_roi = static_cast<unsigned>(ps.tiles_x) * ps.tiles_y * ps.tiles_z;
  if (tid < kWave) plan_item_lanes(rois, p, ps, item_of(tid >> 2), total, per_roi, &lplans[tid >> 2]);
  __syncthreads();
  const int lx = tid % TX, ly = (tid / TX) % TY, lz = tid / (TX * TY);
  const long zstride = static_cast<long>(oh) * ow, plane = static_cast<long>(D) * H * W;
  for (unsigned round = 0;; round++) {
    const unsigned w = item_of(round);
    if (w == kDone) break;
    const unsigned c = C > 1 ? w / total : 0;
    const TilePlan *rec = &lplans[round];
    const int mode = plan_scalar(&rec->mode);
    const int bx = plan_scalar(&rec->n[0]), by = plan_scalar(&rec->n[1]), bz = plan_scalar(&rec->n[2]);
    const int lo[3] = {plan_scalar(&rec->lo[0]), plan_scalar(&rec->lo[1]), plan_scalar(&rec->lo[2])};
    const int pitch = vec > 0 ? bx : bx + 1, slice = by * pitch;
    const T *src = feat + (static_cast<long>(plan_scalar(&rec->batch)) * C + c) * plane;
    if (mode == 1 || mode == 3) {   // the box into LDS
      const int rows = by * bz;
      const T *corner = src + (static_cast<long>(lo[2]) * H + lo[1]) * W + lo[0];
      const float inv_by = 1.0f / static_cast<float>(by);
      if (vec > 0) {
        const int groups = bx / V;
        const float inv_groups = 1.0f / static_cast<float>(groups);
        // eight independent 16-byte loads in flight per lane before the first LDS store
        for (int i0 = tid; i0 < rows * groups; i0 += THREADS * 8) {
          u32x4 v[8];
#pragma unroll
          for (int u = 0; u < 8; u++) {
            const int i = i0 + u * THREADS;
            if (i < rows * groups) {
              const int r = div_small(i, inv_groups), gi = i - r * groups;
              const int zz = div_small(r, inv_by), yy = r - zz * by;
              v[u] = *reinterpret_cast<const u32x4 *>(corner + (static_cast<long>(zz) * H + yy) * W + gi * V);
            }
          }
#pragma unroll
          for (int u = 0; u < 8; u++) {
            const int i = i0 + u * THREADS;
            if (i < rows * groups) {
              const int r = div_small(i, inv_groups), gi = i - r * groups;
              *reinterpret_cast<u32x4 *>(tile + r * pitch + gi * V) = v[u];
            }
          }
        }
      } else {
        for (int i = tid; i < rows * pitch; i += THREADS) {
          const int r = i / pitch, e = i - r * pitch;
          const int zz = div_small(r, inv_by), yy = r - zz * by;
          tile[i] = e < bx ? corner[(static_cast<long>(zz) * H + yy) * W + e] : store_cast<T>(0.f);
        }
      }
    }
    // separable form: axis-aligned map, box in LDS, room for the intermediates behind it
    const int first_f = static_cast<int>((static_cast<size_t>(by) * bz * pitch * sizeof(T) + 15) / 16 * 4);
    float *t1 = reinterpret_cast<float *>(tile) + first_f;   // [bz][by][TX]
    float *t2 = t1 + bz * by * TX;                           // [bz][TY][TX]
    constexpr int TS = TZ > 16 ? TZ : 16;                               // table entries per axis
    static_assert(TX <= TS && TY <= TS, "table entries per axis");
    AxisTaps3 *tab = reinterpret_cast<AxisTaps3 *>(t2 + bz * TY * TX);   // [3][TS]
    bool sep = false;
    if (mode == 1 || mode == 3) {
      const CT *m = plan_map<CT>(rec);
      // (images as volumes of rows: 16 taps per pixel are cheaper than three passes of which one copies)
      sep = TY > 1 && m[2] == CT(0) && m[3] == CT(0) && m[5] == CT(0) && m[7] == CT(0) && m[9] == CT(0) && m[10] == CT(0) &&
            (static_cast<long>(first_f) + bz * by * TX + bz * TY * TX) * 4 + 3 * TS * static_cast<long>(sizeof(AxisTaps3)) <= LDS_BYTES;
      if (sep && tid < TX + TY + TZ) {
        const int a = tid < TX ? 0 : (tid < TX + TY ? 1 : 2), o = tid - (a == 0 ? 0 : (a == 1 ? TX : TX + TY));
        CT r;
        if (a == 0) r = m[0] + static_cast<CT>(o) * m[1];
        else if (a == 1) r = m[4] + static_cast<CT>(o) * m[6];
        else r = (m[8] + static_cast<CT>(o / ZPL * ZPL) * m[11]) + static_cast<CT>(o % ZPL) * m[11];
        const int size_a = a == 0 ? W : (a == 1 ? H : D), n_a = a == 0 ? bx : (a == 1 ? by : bz);
        const CT cmax = static_cast<CT>(size_a - (a == 0 ? lo[0] : (a == 1 ? lo[1] : lo[2])));
        const int top = max(n_a - 1, 0);
        const bool ok = r >= CT(-1) && r <= cmax;
        r = fmax(r, CT(0));
        const CT l = floor(r);
        AxisTaps3 e;
        catmull_rom(static_cast<float>(r - l), e.w);
#pragma unroll
        for (int k = 0; k < 4; k++) {
          e.idx[k] = min(max(static_cast<int>(l) - 1 + k, 0), top);
          if (!ok) e.w[k] = 0.f;
        }
        tab[a * TS + o] = e;
      }
    }
    __syncthreads();
    const int ox = plan_scalar(&rec->t0[0]) + lx, oy = plan_scalar(&rec->t0[1]) + ly, zb = plan_scalar(&rec->t0[2]) + lz * ZPL;
    const int count = (ox < ow && oy < oh) ? min(ZPL, od - zb) : 0;
    T *drow = out + (static_cast<long>(plan_scalar(&rec->roi)) * C + c) * od * zstride + (static_cast<long>(zb) * oh + oy) * ow + ox;
    if (sep) {
      {
        const AxisTaps3 e = tab[lx];   // (tid % TX == lx)
        for (int i = tid; i < bz * by * TX; i += THREADS) {
          const T *row = tile + (i / TX) * pitch;
          t1[i] = e.w[0] * load(row + e.idx[0]) + e.w[1] * load(row + e.idx[1]) + e.w[2] * load(row + e.idx[2]) +
                  e.w[3] * load(row + e.idx[3]);
        }
      }
      __syncthreads();
      {
        const AxisTaps3 e = tab[TS + ly];   // ((tid / TX) % TY == ly)
        for (int i = tid; i < bz * TY * TX; i += THREADS) {
          const float *col = t1 + (i / (TY * TX)) * by * TX + lx;
          t2[i] = e.w[0] * col[e.idx[0] * TX] + e.w[1] * col[e.idx[1] * TX] + e.w[2] * col[e.idx[2] * TX] +
                  e.w[3] * col[e.idx[3] * TX];
        }
      }
      __syncthreads();
      for (int k = 0; k < count; k++) {
        const AxisTaps3 e = tab[2 * TS + lz * ZPL + k];
        const float *col = t2 + ly * TX + lx;
        drow[k * zstride] = store_cast<T>(e.w[0] * col[e.idx[0] * TY * TX] + e.w[1] * col[e.idx[1] * TY * TX] +
                                          e.w[2] * col[e.idx[2] * TY * TX] + e.w[3] * col[e.idx[3] * TY * TX]);
      }
    } else if (count > 0) {
      const CT fx = static_cast<CT>(lx), fy = static_cast<CT>(ly), fz = static_cast<CT>(lz * ZPL);
      CT b[3], st[3];
#pragma unroll
      for (int a = 0; a < 3; a++) {
        const CT *m = plan_map<CT>(rec) + 4 * a;
        b[a] = m[0] + fx * m[1] + fy * m[2] + fz * m[3];
        st[a] = m[3];
      }
      BoxLimits<CT> lim;
      lim.one = ps.halo_lo;
      const int size[3] = {W, H, D};
      const int n[3] = {mode == 2 ? W : bx, mode == 2 ? H : by, mode == 2 ? D : bz};
      for (int a = 0; a < 3; a++) {  // the volume's far end (inclusive) and the last index of the box
        lim.cmax[a] = static_cast<CT>(size[a] - (mode == 2 ? 0 : lo[a]));
        lim.top[a] = static_cast<CT>(max(n[a] - 1, 0));
      }
      if (mode == 0) {
        for (int k = 0; k < count; k++) drow[k * zstride] = store_cast<T>(0.f);
      } else if (mode == 3) {
        const int dy = by > 1 ? pitch : 0, dz = bz > 1 ? slice : 0;
#pragma unroll 1
        for (int k = 0; k < count; k++) {
          const CT kk = static_cast<CT>(k);
          drow[k * zstride] = store_cast<T>(staged_cubic<T, CT, true, false>(
              tile, b[0] + kk * st[0], b[1] + kk * st[1], b[2] + kk * st[2], lim, pitch, slice, dy, dz));
        }
      } else if (mode == 2) {  // the box does not fit in LDS: taps straight from the feature map
        for (int a = 0; a < 3; a++) b[a] += static_cast<CT>(lo[a]);
        const long hw = static_cast<long>(H) * W;
#pragma unroll 1
        for (int k = 0; k < count; k++) {
          const CT kk = static_cast<CT>(k);
          drow[k * zstride] = store_cast<T>(staged_cubic<T, CT, false, true, TY == 1>(
              src, b[0] + kk * st[0], b[1] + kk * st[1], b[2] + kk * st[2], lim, W, hw, W, hw));
        }
      } else {
        const int dy = by > 1 ? pitch : 0, dz = bz > 1 ? slice : 0;
#pragma unroll 1
        for (int k = 0; k < count; k++) {
          const CT kk = static_cast<CT>(k);
          drow[k * zstride] = store_cast<T>(staged_cubic<T, CT, false, false, TY == 1>(
              tile, b[0] + kk * st[0], b[1] + kk * st[1], b[2] + kk * st[2], lim, pitch, slice, dy, dz));
        }
      }
    }
    __syncthreads();  // every lane is done with the box
  }
}

static unsigned compute_units() {
  static int cus[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (dev < 0 || dev >= 64) return 256;
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev] = n;
  }
  return static_cast<unsigned>(cus[dev]);
}

// G > 1: `p` is the problem on the finer grid of a fixed sampling grid of G per axis (order 1), `out` the
// volume of the bins' means.
template <typename T, int TX, int TY, int TZ, int THREADS, int LDS_BYTES, int KMAX, bool CUBIC = false, int G = 1>
static int launch_resample(const T *feat, const float *rois, T *out, const RoiProblem &p,
                           void *workspace, size_t *need, hipStream_t s) {
  const long tx = (p.ow + TX - 1) / TX, ty = (p.oh + TY - 1) / TY, tz = (p.od + TZ - 1) / TZ;
  const long per_roi = tx * ty * tz, total = per_roi * static_cast<long>(p.R), work = total * p.C;
  if (work >= (1L << 31) || static_cast<long>(p.D) * p.H * p.W * sizeof(T) >= (1L << 31)) return -1;
  if (need) { *need = 0; return MV_OK; }
  constexpr int V = 16 / sizeof(T);
  PlanShape ps;
  ps.tiles_x = static_cast<int>(tx); ps.tiles_y = static_cast<int>(ty); ps.tiles_z = static_cast<int>(tz);
  ps.tx = TX; ps.ty = TY; ps.tz = TZ;
  ps.vec = ((p.W % V == 0) && (reinterpret_cast<uintptr_t>(feat) % 16 == 0)) ? V : 0;
  ps.cap = LDS_BYTES / sizeof(T);
  ps.threads = THREADS; ps.max_items = KMAX;
  ps.halo_lo = CUBIC ? 1 : 0; ps.halo_hi = CUBIC ? 2 : 1;
  ps.grids = G == 0 ? 1 : 0;
  ps.flat_axis = TY == 1 ? 1 : 0;
  {
    // inputs that fit the L2s and are read about once (resampling: no more rois than images)
    const long in_bytes = static_cast<long>(p.N) * p.C * p.D * p.H * p.W * static_cast<long>(sizeof(T));
    ps.warm_groups = (!CUBIC && ps.vec > 0 && p.R <= p.N && in_bytes <= (24L << 20)) ? static_cast<unsigned>(in_bytes / (4 * kWarmStride)) : 0u;
  }
  ps.es = static_cast<int>(sizeof(T));
  ps.pad_slices = (!CUBIC && sizeof(T) == 2) ? 1 : 0;   // (fp32 tensors: modelled gain 12 %, measured none)
  ps.by_per_roi.set(static_cast<unsigned>(per_roi));
  ps.by_tiles_x.set(static_cast<unsigned>(tx));
  ps.by_tiles_y.set(static_cast<unsigned>(ty));
  ps.by_total.set(static_cast<unsigned>(total));
  unsigned blocks = compute_units() * (160u * 1024u / (LDS_BYTES + sizeof(TilePlan) * kPlanSlots + 64u));
  // As many workgroups as are resident at once, more when that would give one more than
  // kPlanSlots items (the later ones start as the first finish).
  if (work < blocks) blocks = static_cast<unsigned>(work);
  // (a queue holds at most work / 8 + kChunk items and gets blocks / 8 workgroups)
  const long by_slots = ((work + kPlanSlots - 1) / kPlanSlots + 2 * kXcds + kXcds - 1) / kXcds * kXcds;
  if (blocks >= kXcds) blocks = blocks / kXcds * kXcds;  // the same number of workgroups on every XCD
  if (by_slots > blocks && work > kPlanSlots) blocks = static_cast<unsigned>(by_slots);
  ps.by_slots.set(blocks >= kXcds ? blocks / kXcds : blocks);
  if constexpr (CUBIC)
    hipLaunchKernelGGL((roi_resample_cubic_kernel<T, TX, TY, TZ, THREADS, LDS_BYTES>), dim3(blocks),
                       dim3(THREADS), 0, s, feat, rois, out, p, ps, static_cast<unsigned>(total),
                       static_cast<unsigned>(work));
  else if constexpr (G == 0) {
    if (p.order == 0)
      hipLaunchKernelGGL((roi_resample_kernel<T, TX, TY, TZ, THREADS, LDS_BYTES, KMAX, 0, 0>), dim3(blocks),
                         dim3(THREADS), 0, s, feat, rois, out, p, ps, static_cast<unsigned>(total),
                         static_cast<unsigned>(work));
    else
      hipLaunchKernelGGL((roi_resample_kernel<T, TX, TY, TZ, THREADS, LDS_BYTES, KMAX, 1, 0>), dim3(blocks),
                         dim3(THREADS), 0, s, feat, rois, out, p, ps, static_cast<unsigned>(total),
                         static_cast<unsigned>(work));
  } else if constexpr (G > 1)
    hipLaunchKernelGGL((roi_resample_kernel<T, TX, TY, TZ, THREADS, LDS_BYTES, KMAX, 1, G>), dim3(blocks),
                       dim3(THREADS), 0, s, feat, rois, out, p, ps, static_cast<unsigned>(total),
                       static_cast<unsigned>(work));
  else if (p.order == 0)
    hipLaunchKernelGGL((roi_resample_kernel<T, TX, TY, TZ, THREADS, LDS_BYTES, KMAX, 0>), dim3(blocks),
                       dim3(THREADS), 0, s, feat, rois, out, p, ps, static_cast<unsigned>(total),
                       static_cast<unsigned>(work));
  else
    hipLaunchKernelGGL((roi_resample_kernel<T, TX, TY, TZ, THREADS, LDS_BYTES, KMAX, 1>), dim3(blocks),
                       dim3(THREADS), 0, s, feat, rois, out, p, ps, static_cast<unsigned>(total),
                       static_cast<unsigned>(work));
  return check_launch("roi_resample_kernel");
}

int roi_forward_tiled(const void *input, const void *rois, void *output, int dtype,
                      const RoiProblem &p, void *workspace, size_t capacity, size_t *need, hipStream_t s);

// Mean over the g^ndim samples of a bin: `fine` holds one sample per element, [planes][od*g][oh*g][ow*g]
// ([planes][oh*g][ow*g] for images, gz = 1).
template <typename T>
__global__ __launch_bounds__(256) void roi_bin_mean_kernel(const T *__restrict__ fine, T *__restrict__ out,
                                                           long cells, int od, int oh, int ow, int g,
                                                           int gz) {
  const long i = blockIdx.x * 256L + threadIdx.x;
  if (i >= cells) return;
  const int x = i % ow, y = (i / ow) % oh, z = (i / (static_cast<long>(ow) * oh)) % od;
  const long plane = i / (static_cast<long>(ow) * oh * od);
  const long fw = static_cast<long>(ow) * g, fh = static_cast<long>(oh) * g, fd = static_cast<long>(od) * gz;
  const T *src = fine + ((plane * fd + static_cast<long>(z) * gz) * fh + static_cast<long>(y) * g) * fw +
                 static_cast<long>(x) * g;
  float sum = 0.f;
  for (int a = 0; a < gz; a++)
    for (int b = 0; b < g; b++)
      for (int c = 0; c < g; c++) sum += static_cast<float>(load(src + (a * fh + b) * fw + c));
  out[i] = store_cast<T>(sum / static_cast<float>(gz * g * g));
}

// A fixed sampling grid of 2..4 per axis on a large output: the bins' samples are exactly the voxels
// of the same roi resampled at grid 1 onto an output g times finer (start + (cell * g + sub + 0.5) *
// bin / g).  Images at order 1 with a grid of 2 or 4 run the tiled kernel on that finer grid and take the
// means inside it (template argument G).  Order 3, and images with a grid of 3, write the finer volume
// into the workspace and a second pass takes the means: 16-bit samples are then rounded before the mean
// is; fp16's two roundings stay within its tolerance, bf16's would not.  Volumes at orders 0 and 1 are
// not taken here: the kernel that walks the samples of a bin in a loop is as fast or faster for them
// (config 2, fp16: grid 2 0.111 against 0.130 ms, grid 3 0.314 against 0.524 ms through the two passes,
// grid 4 0.678 against 0.677 ms), for images it is slower (0.033 / 0.056 / 0.086 against 0.024 / 0.048 /
// 0.049 ms).  Returns -1 for what it does not take.  (The workspace query does not know the order and
// answers for the two passes.)
static int roi_forward_tiled_image(const void *input, const void *rois, void *output, int dtype, const RoiProblem &p,
                                   void *workspace, size_t capacity, size_t *need, hipStream_t s, int pool);

static int roi_forward_tiled_grid(const void *input, const void *rois, void *output, int dtype,
                                  const RoiProblem &p, void *workspace, size_t capacity, size_t *need, hipStream_t s) {
  const int g = p.sampling_ratio, gz = p.ndim == 3 ? g : 1;
  // the means inside the kernel: images, grids of 2 and 4 at order 1 (their rewritten rois are in the workspace)
  const bool means = p.ndim == 2 && (g == 2 || g == 4) && p.R > 0 && (dtype == MV_F16 || dtype == MV_BF16 || dtype == MV_F32);
  const bool in_kernel = !need && means && p.order == 1;
  if (!need && p.ndim == 3 && p.order != 3) return -1;   // volumes at orders 0 and 1: the loop over the samples
  if (dtype != MV_F16 && dtype != MV_F32 && !means) return -1;
  if (!need && p.order != 1 && p.order != 3) return -1;
  // Outputs that the grid-1 rule sends here, except those of <= 16 cells per axis (the pooled kernels
  // take plain boxes of that size).  Only values that the workspace query also knows may decide.
  if (static_cast<long>(p.od) * p.oh * p.ow < 4096 || p.ow < 16) return -1;
  if (p.od <= 16 && p.oh <= 16 && p.ow <= 16) return -1;
  RoiProblem f = p;
  f.sampling_ratio = 1;
  f.od = p.od * gz; f.oh = p.oh * g; f.ow = p.ow * g;
  const long cells = static_cast<long>(p.R) * p.C * p.od * p.oh * p.ow;
  const long fine = cells * gz * g * g;
  // (32-bit byte offsets inside one finer volume, as in the grid-1 rule)
  if (in_kernel && static_cast<long>(f.od) * f.oh * f.ow * 4 < (1L << 31)) {
    const int st = roi_forward_tiled_image(input, rois, output, dtype, f, workspace, capacity, nullptr, s, g);
    if (st != -1) return st;
  }
  if (dtype != MV_F16 && dtype != MV_F32) {   // bf16: the means inside the kernel or nothing
    if (need && p.ndim == 2) return roi_forward_tiled_image(nullptr, nullptr, nullptr, dtype, f, nullptr, 0, need, nullptr, g);
    return -1;
  }
  if (fine >= (1L << 31) || (cells + 255) / 256 >= (1L << 31)) return -1;
  size_t inner = 0;
  if (roi_forward_tiled(nullptr, nullptr, nullptr, dtype, f, nullptr, 0, &inner, nullptr) != MV_OK) return -1;
  inner = (inner + 255) & ~static_cast<size_t>(255);
  if (need) { *need = inner + static_cast<size_t>(fine) * dtype_size(dtype); return MV_OK; }
  if (workspace == nullptr || capacity < inner + static_cast<size_t>(fine) * dtype_size(dtype)) return -1;
  void *samples = static_cast<char *>(workspace) + inner;
  const int st = roi_forward_tiled(input, rois, samples, dtype, f, workspace, inner, nullptr, s);
  if (st != MV_OK) return st;   // -1: the finer problem does not fit the tiled kernel after all
  const dim3 grid(static_cast<unsigned>((cells + 255) / 256)), block(256);
  if (dtype == MV_F16)
    hipLaunchKernelGGL((roi_bin_mean_kernel<__half>), grid, block, 0, s, static_cast<const __half *>(samples),
                       static_cast<__half *>(output), cells, p.od, p.oh, p.ow, g, gz);
  else
    hipLaunchKernelGGL((roi_bin_mean_kernel<float>), grid, block, 0, s, static_cast<const float *>(samples),
                       static_cast<float *>(output), cells, p.od, p.oh, p.ow, g, gz);
  return check_launch("roi_bin_mean_kernel");
}

// ---- images --------------------------------------------------------------------------------------
// A lane's column runs along z, so an image as a depth-1 volume would give every lane one pixel per
// item.  Images are therefore resampled as volumes with the image rows as slices: [N, C, H, W] is read
// as [N, C, D = H, 1, W], the output [R, C, oh, ow] as [R, C, od = oh, 1, ow], and a roi
// (x, y, w, h, theta) becomes the volume roi (x, y', y, w, h', h, 0, -theta, 0) whose middle axis has one
// cell that samples row 0 exactly (aligned: y' = 0.5 / scale, h' = 1 / scale; otherwise y' = 0).  With
// the angles (0, -theta, 0) the volume's rotation rows are (cos, 0, -sin) and (sin, 0, cos) with the
// very values of the image's rotation (sin is odd in the routine used; products with exact 0 and 1 are
// exact), so the planner forms the same fp64 map as for the image.  Tiles of 64 x 1 x 64 (fp32: 32)
// outputs, a column of 8 (4) rows per lane.
__global__ void roi_rows_as_slices_kernel(const float *__restrict__ flat, float *__restrict__ vol, int R, int rotated,
                                          int aligned, float scale) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= R) return;
  const float *r = flat + static_cast<long>(i) * (rotated ? 6 : 5);
  float *o = vol + static_cast<long>(i) * (rotated ? 10 : 7);
  o[0] = r[0];
  if (rotated) {
    o[1] = r[1]; o[2] = aligned ? 0.5f / scale : 0.f; o[3] = r[2];
    o[4] = r[3]; o[5] = 1.f / scale; o[6] = r[4];
    o[7] = 0.f; o[8] = -r[5]; o[9] = 0.f;
  } else {   // corners: the middle axis runs from -0.5 to 0.5, one cell sampled at its centre
    o[1] = r[1]; o[2] = -0.5f / scale; o[3] = r[2];
    o[4] = r[3]; o[5] = 0.5f / scale; o[6] = r[4];
  }
}

// pool = 2 or 4: `p` is the problem on the finer grid of a fixed sampling grid (order 1) and `output` takes
// the bins' means (see roi_forward_tiled_grid).
static int roi_forward_tiled_image(const void *input, const void *rois, void *output, int dtype, const RoiProblem &p,
                                   void *workspace, size_t capacity, size_t *need, hipStream_t s, int pool) {
  const long vox = static_cast<long>(p.oh) * p.ow;
  // pool = 0: `p` is the problem asked for, with any sampling grid, and the kernel walks the samples of a bin
  if ((pool != 0 && p.sampling_ratio != 1) || vox < 4096 || p.ow < 16 || p.R == 0) return -1;
  if (pool > 1 && ((!need && p.order != 1) || (pool != 2 && pool != 4))) return -1;   // (a size query is not told the order)
  if (pool == 0 && !need && p.order == 3) return -1;
  if (vox * 4 >= (1L << 31)) return -1;
  if (dtype != MV_F16 && dtype != MV_BF16 && dtype != MV_F32) return -1;
  // (the workspace query does not know whether the rois are rotated: room for the wider rows)
  const size_t bytes = (static_cast<size_t>(p.R) * 10 * sizeof(float) + 255) / 256 * 256;
  RoiProblem v = p;
  v.ndim = 3;
  v.D = p.H; v.H = 1; v.W = p.W;
  v.od = p.oh; v.oh = 1; v.ow = p.ow;
  float *vol_rois = static_cast<float *>(workspace);
  if (!need) {
    if (workspace == nullptr || capacity < bytes) return -1;
    hipLaunchKernelGGL(roi_rows_as_slices_kernel, dim3((p.R + 255) / 256), dim3(256), 0, s, static_cast<const float *>(rois),
                       vol_rois, p.R, p.rotated, p.aligned, static_cast<float>(p.scale));
  }
  int st;
  if (p.order == 3) {
    // (the one cell of the middle axis samples row 0 exactly: its four taps are that row with weights 0, 1, 0, 0)
    switch (dtype) {
      case MV_F16:
        st = launch_resample<__half, 64, 1, 64, 512, 74 * 1024, 8, true>(static_cast<const __half *>(input), vol_rois,
                                                                          static_cast<__half *>(output), v, nullptr, need, s);
        break;
      case MV_BF16:
        st = launch_resample<__hip_bfloat16, 64, 1, 64, 512, 74 * 1024, 8, true>(
            static_cast<const __hip_bfloat16 *>(input), vol_rois, static_cast<__hip_bfloat16 *>(output), v, nullptr, need, s);
        break;
      default:
        st = launch_resample<float, 64, 1, 64, 512, 74 * 1024, 6, true>(static_cast<const float *>(input), vol_rois,
                                                                         static_cast<float *>(output), v, nullptr, need, s);
    }
    if (need && st == MV_OK) *need = bytes;
    return st;
  }
  if (pool == 0) {
    switch (dtype) {
      case MV_F16:
        st = launch_resample<__half, 64, 1, 64, 512, 74 * 1024, 8, false, 0>(static_cast<const __half *>(input), vol_rois,
                                                                              static_cast<__half *>(output), v, nullptr, need, s);
        break;
      case MV_BF16:
        st = launch_resample<__hip_bfloat16, 64, 1, 64, 512, 74 * 1024, 8, false, 0>(
            static_cast<const __hip_bfloat16 *>(input), vol_rois, static_cast<__hip_bfloat16 *>(output), v, nullptr, need, s);
        break;
      default:
        st = launch_resample<float, 64, 1, 32, 512, 74 * 1024, 6, false, 0>(static_cast<const float *>(input), vol_rois,
                                                                             static_cast<float *>(output), v, nullptr, need, s);
    }
    if (need && st == MV_OK) *need = bytes;
    return st;
  }
  if (pool != 1) {
#define MV_IMAGE_MEANS(TYPE, TZV, KMAXV, GV)                                                                         \
  launch_resample<TYPE, 64, 1, TZV, 512, 74 * 1024, KMAXV, false, GV>(static_cast<const TYPE *>(input), vol_rois, \
                                                                       static_cast<TYPE *>(output), v, nullptr, need, s)
    switch (dtype) {
      case MV_F16: st = pool == 2 ? MV_IMAGE_MEANS(__half, 64, 8, 2) : MV_IMAGE_MEANS(__half, 64, 8, 4); break;
      case MV_BF16: st = pool == 2 ? MV_IMAGE_MEANS(__hip_bfloat16, 64, 8, 2) : MV_IMAGE_MEANS(__hip_bfloat16, 64, 8, 4); break;
      default: st = pool == 2 ? MV_IMAGE_MEANS(float, 32, 6, 2) : MV_IMAGE_MEANS(float, 32, 6, 4);
    }
#undef MV_IMAGE_MEANS
    if (need && st == MV_OK) *need = bytes;
    return st;
  }
  switch (dtype) {
    case MV_F16:
      st = launch_resample<__half, 64, 1, 64, 512, 74 * 1024, 8>(static_cast<const __half *>(input), vol_rois,
                                                                  static_cast<__half *>(output), v, nullptr, need, s);
      break;
    case MV_BF16:
      st = launch_resample<__hip_bfloat16, 64, 1, 64, 512, 74 * 1024, 8>(static_cast<const __hip_bfloat16 *>(input), vol_rois,
                                                                          static_cast<__hip_bfloat16 *>(output), v, nullptr, need, s);
      break;
    case MV_I32:
      st = launch_resample<int, 64, 1, 32, 512, 74 * 1024, 6>(static_cast<const int *>(input), vol_rois,
                                                               static_cast<int *>(output), v, nullptr, need, s);
      break;
    default:
      st = launch_resample<float, 64, 1, 32, 512, 74 * 1024, 6>(static_cast<const float *>(input), vol_rois,
                                                                 static_cast<float *>(output), v, nullptr, need, s);
  }
  if (need && st == MV_OK) *need = bytes;
  return st;
}

// The tiled path pays when one (roi, channel) yields many voxels and the sampling grid is 1 (or a
// fixed 2..4, in two passes).  With `need` set only the workspace size is computed.  Returns -1
// when the path does not apply.
int roi_forward_tiled(const void *input, const void *rois, void *output, int dtype,
                      const RoiProblem &p, void *workspace, size_t capacity, size_t *need, hipStream_t s) {
  // int32 label maps: one sample per cell at order 0 (the voxel's value passes through fp32, which holds
  // labels below 2^24 exactly, as the float copy did that such maps used to be resampled through)
  if (dtype == MV_I32 && (p.order != 0 || p.sampling_ratio != 1)) return -1;
  if (p.sampling_ratio >= 2 && p.sampling_ratio <= 4) {
    const int st = roi_forward_tiled_grid(input, rois, output, dtype, p, workspace, capacity, need, s);
    if (st != -1) return st;
  }
  // Every other grid at orders 0 and 1 - volumes with any grid, images with 3 (without a workspace or in
  // bf16), 5 and more, ceil(roi extent / cells) per roi: the samples of a bin in a loop inside the kernel.
  const bool any_grid = p.sampling_ratio != 1;
  if (any_grid && p.order == 3) return -1;
  // images: rows as slices
  if (p.ndim == 2) return roi_forward_tiled_image(input, rois, output, dtype, p, workspace, capacity, need, s, any_grid ? 0 : 1);
  const long vox = static_cast<long>(p.od) * p.oh * p.ow;
  if (vox < 4096 || p.ow < 16 || p.R == 0) return -1;
  if (vox * 4 >= (1L << 31)) return -1;   // 32-bit byte offsets inside one output volume
  const float *r = static_cast<const float *>(rois);
  if (any_grid) {
    switch (dtype) {
      case MV_F16:
        return launch_resample<__half, 16, 16, 16, 512, 74 * 1024, 8, false, 0>(
            static_cast<const __half *>(input), r, static_cast<__half *>(output), p, workspace, need, s);
      case MV_BF16:
        return launch_resample<__hip_bfloat16, 16, 16, 16, 512, 74 * 1024, 8, false, 0>(
            static_cast<const __hip_bfloat16 *>(input), r, static_cast<__hip_bfloat16 *>(output), p, workspace, need, s);
      case MV_F32:
        return launch_resample<float, 16, 16, 8, 512, 74 * 1024, 6, false, 0>(
            static_cast<const float *>(input), r, static_cast<float *>(output), p, workspace, need, s);
      default:
        return -1;
    }
  }
  if (p.order == 3) {
    // A source of a few hundred voxels per channel (the control grid of the elastic deformation) needs
    // no 74 KB tile: the instance with a small one keeps twice as many workgroups per compute unit busy.
    const long rows = static_cast<long>(p.D) * p.H;
    const long small_f32 = rows * (p.W + 1) * 4 + (rows * 16 + p.D * 256L) * 4 + 3 * 32 * 32;
    if (small_f32 <= 20 * 1024) {
      switch (dtype) {
        case MV_F16:
          return launch_resample<__half, 16, 16, 32, 512, 20 * 1024, 8, true>(
              static_cast<const __half *>(input), r, static_cast<__half *>(output), p, workspace, need, s);
        case MV_BF16:
          return launch_resample<__hip_bfloat16, 16, 16, 32, 512, 20 * 1024, 8, true>(
              static_cast<const __hip_bfloat16 *>(input), r, static_cast<__hip_bfloat16 *>(output), p,
              workspace, need, s);
        case MV_F32:
          return launch_resample<float, 16, 16, 32, 512, 20 * 1024, 6, true>(
              static_cast<const float *>(input), r, static_cast<float *>(output), p, workspace, need, s);
        default:
          return -1;
      }
    }
    switch (dtype) {
      case MV_F16:
        return launch_resample<__half, 16, 16, 8, 512, 74 * 1024, 8, true>(
            static_cast<const __half *>(input), r, static_cast<__half *>(output), p, workspace, need, s);
      case MV_BF16:
        return launch_resample<__hip_bfloat16, 16, 16, 8, 512, 74 * 1024, 8, true>(
            static_cast<const __hip_bfloat16 *>(input), r, static_cast<__hip_bfloat16 *>(output), p,
            workspace, need, s);
      case MV_F32:
        return launch_resample<float, 16, 16, 8, 512, 74 * 1024, 6, true>(
            static_cast<const float *>(input), r, static_cast<float *>(output), p, workspace, need, s);
      default:
        return -1;
    }
  }
  switch (dtype) {
    case MV_F16:
      return launch_resample<__half, 16, 16, 16, 512, 74 * 1024, 8>(
          static_cast<const __half *>(input), r, static_cast<__half *>(output), p, workspace, need, s);
    case MV_BF16:
      return launch_resample<__hip_bfloat16, 16, 16, 16, 512, 74 * 1024, 8>(
          static_cast<const __hip_bfloat16 *>(input), r, static_cast<__hip_bfloat16 *>(output), p,
          workspace, need, s);
    case MV_F32:
      return launch_resample<float, 16, 16, 8, 512, 74 * 1024, 6>(
          static_cast<const float *>(input), r, static_cast<float *>(output), p, workspace, need, s);
    case MV_I32:
      return launch_resample<int, 16, 16, 8, 512, 74 * 1024, 6>(
          static_cast<const int *>(input), r, static_cast<int *>(output), p, workspace, need, s);
    default:
      return -1;
  }
}

// ---------------------------------------------------------------------------------------------
// Backward of the same problems (any sampling grid, orders 0 and 1).  The forward's plan is used in reverse: an
// item is (output tile, channel), its source box becomes an LDS tile of 32-bit FIXED-POINT sums, every
// output voxel of the tile adds weight * grad_output to the <= 8 voxels its sample touches, and the
// tile's non-zero sums go to the fp32 gradient buffer as one atomic per voxel, contiguous along x
// (one request per 64-byte sector instead of eight scattered ones per output voxel).  Integer sums
// because an LDS fp32 atomic retires one lane at a time.  Scale: |term| <= max|grad_output| < 2^e
// is mapped to 2^t quanta, t = 30 - ceil(log2(terms a voxel can get from one tile)) >= 19 (a tile has
// 2^11 voxels; bins of about a voxel give t = 23), so no sum leaves 31 bits and a term is rounded by
// at most 2^-(t+1) of that bound.  Sample coordinates and the tap decisions are fp64, as in the general
// kernel.  Boxes beyond the LDS tile, and every term when grad_output holds a NaN or an infinity,
// go to the buffer as single fp32 atomics.
constexpr int kScatterThreads = 512;
#ifndef MV_SCATTER_SHAPE
#define MV_SCATTER_SHAPE 16, 16, 8
#define MV_SCATTER_SHAPE_2D 32, 64, 1
#define MV_SCATTER_LDS (74 * 1024)
#define MV_SCATTER_WGS 2
#endif
constexpr int kScatterLds = MV_SCATTER_LDS;
constexpr int kScatterWgs = MV_SCATTER_WGS;     // workgroups per compute unit
constexpr int kTermBits = 19;

// fp16 sums straight into the gradient tensor: one packed atomic adds to the two voxels of an aligned
// pair (`pair`: the even voxel).  A voxel's sum is then rounded once per tile that reaches it (a few)
// instead of once at the end.
__device__ __forceinline__ void atomic_add_pair(__half *pair, float lo, float hi) {
  typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
  half2_t v;
  v.x = static_cast<_Float16>(lo); v.y = static_cast<_Float16>(hi);
  __builtin_amdgcn_global_atomic_fadd_v2f16((__attribute__((address_space(1))) half2_t *)pair, v);
}
__device__ __forceinline__ void atomic_add_element(__half *base, long i, float v) {
  atomic_add_pair(base + (i & ~1L), (i & 1) ? 0.f : v, (i & 1) ? v : 0.f);
}
__device__ __forceinline__ void atomic_add_element(float *base, long i, float v) { atomic_add(base + i, v); }

// DIRECT (fp16 only; rows of an even number of voxels, a 4-byte aligned tensor): `acc` is the gradient
// tensor itself, otherwise an fp32 buffer of its shape.
// GRIDS: the instance for sampling ratios other than 1 (a lane walks the samples of its bins); the one
// for ratio 1 is compiled without that code (it has no scalar registers to spare).
template <typename T, int TX, int TY, int TZ, bool DIRECT = false, bool GRIDS = false>
__global__ __launch_bounds__(kScatterThreads, 2 * kScatterWgs) void roi_backward_tiles_kernel(
    const T *__restrict__ gout, const float *__restrict__ rois, void *__restrict__ acc, const RoiProblem p,
    const PlanShape ps, const unsigned total, const unsigned work) {
  using A = typename std::conditional<DIRECT, T, float>::type;
  static_assert(!DIRECT || std::is_same<T, __half>::value, "packed atomics of fp16 pairs");
  constexpr int kScatterCells = TX * TY * TZ;   // output voxels per item
  static_assert(kScatterCells % kScatterThreads == 0 && kScatterCells <= (1 << (30 - kTermBits)), "tile shape");
  constexpr int kPerThread = kScatterCells / kScatterThreads, kWaves = kScatterThreads / kWave;
  __shared__ TilePlan plans[kPlanSlots];
  __shared__ __attribute__((aligned(16))) int tile[kScatterLds / 4];
  __shared__ unsigned bound_part[2][kWaves];
  const unsigned per_roi = static_cast<unsigned>(ps.tiles_x) * ps.tiles_y * ps.tiles_z;
  if (threadIdx.x < kWave) {
    const unsigned item = blockIdx.x + (threadIdx.x >> 2) * gridDim.x;
    plan_item_lanes(rois, p, ps, item < work ? item : kDone, total, per_roi, &plans[threadIdx.x >> 2]);
  }
  // the tile starts at zero; the flush of an item leaves it at zero for the next one
  for (int i = threadIdx.x * 4; i < kScatterLds / 4; i += kScatterThreads * 4)
    *reinterpret_cast<int4 *>(tile + i) = int4{0, 0, 0, 0};
  __syncthreads();
  const long plane = static_cast<long>(p.D) * p.H * p.W, ovol = static_cast<long>(p.od) * p.oh * p.ow;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  int turn = 0;
  for (unsigned slot = 0; slot < kPlanSlots; slot++) {
    const unsigned item = blockIdx.x + slot * gridDim.x;
    if (item >= work) break;
    const TilePlan &r = plans[slot];
    const int mode = plan_scalar(&r.mode);
    if (mode == 0 || mode == 4) continue;
    // the record's values in scalar registers: the LDS atomics below keep the compiler from holding
    // anything it reads from LDS across them
    const int n0 = plan_scalar(&r.n[0]), n1 = plan_scalar(&r.n[1]), n2 = plan_scalar(&r.n[2]);
    const int l0 = plan_scalar(&r.lo[0]), l1 = plan_scalar(&r.lo[1]), l2 = plan_scalar(&r.lo[2]);
    const int t0x = plan_scalar(&r.t0[0]), t0y = plan_scalar(&r.t0[1]), t0z = plan_scalar(&r.t0[2]);
    // samples per bin (the fixed ratio, or ceil(roi extent / cells) of this roi); every sample carries
    // grad_output / count
    const float inv_count = GRIDS ? 1.f / (static_cast<float>(plan_scalar(&r.grid[0])) * static_cast<float>(plan_scalar(&r.grid[1])) *
                                          static_cast<float>(plan_scalar(&r.grid[2])))
                                  : 1.f;
    double map[12];
#pragma unroll
    for (int i = 0; i < 12; i++) map[i] = uniform(r.map[i]);
    map[0] += l0; map[4] += l1; map[8] += l2;   // to volume coordinates
    const unsigned chan = p.C > 1 ? ps.by_total.div(item) : 0u;
    A *const vol = static_cast<A *>(acc) + (static_cast<long>(plan_scalar(&r.batch)) * p.C + chan) * plane;
    const T *const gsrc = gout + (static_cast<long>(plan_scalar(&r.roi)) * p.C + chan) * ovol;
    // The item's grad_output, and the largest magnitude in it as the bit pattern of a float (patterns
    // of non-negative floats order like unsigned integers, NaNs above infinity).
    float gv[kPerThread];
    unsigned bits = 0;
#pragma unroll
    for (int k = 0; k < kPerThread; k++) {
      const int c = threadIdx.x + k * kScatterThreads;
      const int ox = t0x + c % TX, oy = t0y + (c / TX) % TY, oz = t0z + c / (TX * TY);
      const bool in = ox < p.ow && oy < p.oh && oz < p.od;
      gv[k] = in ? static_cast<float>(load(gsrc + (static_cast<long>(oz) * p.oh + oy) * p.ow + ox)) * inv_count : 0.f;
      bits = max(bits, __float_as_uint(fabsf(gv[k])));
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) bits = max(bits, static_cast<unsigned>(__shfl_xor(static_cast<int>(bits), d)));
    // two buffers taken in turn: between two uses of one lies the barrier of the use in between
    // (items that were skipped above pass no barrier and take no turn)
    if (lane == 0) bound_part[turn][wave] = bits;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kWaves; w++) bits = max(bits, bound_part[turn][w]);
    turn ^= 1;
    bits = __builtin_amdgcn_readfirstlane(bits);
    if (bits == 0) continue;                                  // nothing to add
    // Quanta per unit: a voxel gets at most one term from each sample that lies within one voxel of it
    // on every axis, i.e. inside a ball of radius sqrt(3); along output axis j (samples b_j / g_j apart,
    // b_j = length of column j of the map) that leaves floor(2 sqrt(3) g_j / b_j) + 1 of them.
    int terms = 1;
    float u[3][3];   // the lattice of the samples: u[j] = step of one sample along output axis j, in source voxels
#pragma unroll
    for (int j = 0; j < 3; j++) {
      const float c0 = static_cast<float>(map[1 + j]), c1 = static_cast<float>(map[5 + j]), c2 = static_cast<float>(map[9 + j]);
      const float bj = sqrtf(c0 * c0 + c1 * c1 + c2 * c2);
      const int ext = j == 0 ? TX : (j == 1 ? TY : TZ), gj = GRIDS ? plan_scalar(&r.grid[j]) : 1;
      terms *= static_cast<int>(fminf(3.4642f * static_cast<float>(gj) / bj * 1.00001f + 1.f, static_cast<float>(ext * gj)));
      const float ig = 1.f / static_cast<float>(gj);
      u[j][0] = c0 * ig; u[j][1] = c1 * ig; u[j][2] = c2 * ig;
    }
    // The sum of the WEIGHTS of those terms is smaller still where the samples are dense: every sample owns a cell
    // of the lattice (volume |det u|, extent e_a = sum_j |u[j][a]| along source axis a), over which the tent
    // function widened by e_a / 2 on either side is at least the sample's own weight, so the weights that reach a
    // voxel add up to at most prod_a (1 + e_a) / |det u| in a box that the volume does not clip.  (Volumes only: an
    // image's middle axis has one sample.)
    if (TY > 1) {
      const float det = fabsf(u[0][0] * (u[1][1] * u[2][2] - u[1][2] * u[2][1]) - u[0][1] * (u[1][0] * u[2][2] - u[1][2] * u[2][0]) +
                              u[0][2] * (u[1][0] * u[2][1] - u[1][1] * u[2][0]));
      float w = 1.f;
      // (a box that the volume clips: samples beyond the first or last voxel are moved onto it with weight 1, which
      // gives that voxel's weight function the integral 1.5 instead of 1, 2 on an axis of one voxel)
      const float edge = mode == 3 ? 1.f : 2.f;
#pragma unroll
      for (int a = 0; a < 3; a++) w *= edge + fabsf(u[0][a]) + fabsf(u[1][a]) + fabsf(u[2][a]);
      const float sum = w / fmaxf(det, 1e-30f) * 1.0001f + 1.f;
      if (sum < static_cast<float>(terms)) terms = max(static_cast<int>(sum), 1);
    }
    const int term_bits = 30 - (32 - __clz(terms - 1));   // 30 - ceil(log2 terms); >= kTermBits at one sample per bin
    // finite terms, box within the tile, enough bits per term: 18 for fp32 tensors, 12 for 16-bit ones (a
    // term is rounded to 2^-19 / 2^-13 of the largest; grids of many samples over small bins leave less,
    // and their terms go out one by one as fp32 atomics - the direct fp16 path is not taken for such grids)
    const bool in_lds = bits < 0x7f800000u && mode != 2 && terms <= (sizeof(T) == 2 ? (1 << 18) : (1 << 12));
    const int ex = min(max(127 + 126 + term_bits - static_cast<int>(bits >> 23), 1), 253);   // 2^(ex - 127) = 2^term_bits / 2^e
    const float to_quanta = __uint_as_float(static_cast<unsigned>(ex) << 23);
    const float from_quanta = __uint_as_float(static_cast<unsigned>(254 - ex) << 23);
    // One copy of the loop per (interior, order): a box that is not clipped holds samples in
    // [0, size - 1) only, so the low tap is the floor and neither the void test nor the clamps are needed.
    // 16-bit tensors at order 1 whose box is in LDS: box-relative fp32 coordinates with the forward
    // kernel's rules (clipped boxes: the coordinate clamps to [0, cmax], a sample the clamp moves by
    // more than 1 is void, the low tap is at most top = max(n - 2, 0)); the box's margin covers their
    // rounding.
    auto scatter_cells32 = [&](auto interior_tag, auto grids_tag) {
    constexpr bool kInterior = decltype(interior_tag)::value;
    constexpr bool kGrids = decltype(grids_tag)::value;
    // (the grid is read here, not kept from above: the copy without grids has no scalar registers to spare)
    const int sgx = kGrids ? plan_scalar(&r.grid[0]) : 1, sgy = kGrids ? plan_scalar(&r.grid[1]) : 1, sgz = kGrids ? plan_scalar(&r.grid[2]) : 1;
    const float igx = 1.f / static_cast<float>(sgx), igy = 1.f / static_cast<float>(sgy), igz = 1.f / static_cast<float>(sgz);
    float mf[12], cmax[3], top[3];
#pragma unroll
    for (int i = 0; i < 12; i++) mf[i] = uniform(r.mapf[i]);
#pragma unroll
    for (int a = 0; a < 3; a++) { cmax[a] = uniform(r.cmaxf[a]); top[a] = uniform(r.topf[a]); }
    const float gq_scale = to_quanta;
#pragma unroll
    for (int k = 0; k < kPerThread; k++) {
      const int c = threadIdx.x + k * kScatterThreads;
      const float x = static_cast<float>(c % TX), y = static_cast<float>((c / TX) % TY), z = static_cast<float>(c / (TX * TY));
      const float g = gv[k];
      if (g == 0.f) continue;
      float v0[3];
#pragma unroll
      for (int a = 0; a < 3; a++) v0[a] = fmaf(mf[4 * a + 3], z, fmaf(mf[4 * a + 2], y, fmaf(mf[4 * a + 1], x, mf[4 * a])));
      for (int iz = 0; iz < sgz; iz++)
      for (int iy = 0; iy < sgy; iy++)
      for (int ix = 0; ix < sgx; ix++) {
      float v[3], f[3];
      int b0[3];
#pragma unroll
      for (int a = 0; a < 3; a++)
        v[a] = kGrids ? fmaf(mf[4 * a + 3] * igz, static_cast<float>(iz), fmaf(mf[4 * a + 2] * igy, static_cast<float>(iy), fmaf(mf[4 * a + 1] * igx, static_cast<float>(ix), v0[a]))) : v0[a];
      if constexpr (kInterior) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
          const float l = floorf(v[a]);
          f[a] = v[a] - l;
          b0[a] = static_cast<int>(l);
        }
      } else {
        float moved = 0.f;
#pragma unroll
        for (int a = 0; a < 3; a++) {
          const float cl = clamp_ct(v[a], 0.f, cmax[a]);
          moved = fmaxf(moved, fabsf(v[a] - cl));
          const float l = fminf(floorf(cl), top[a]);
          f[a] = cl - l;
          b0[a] = static_cast<int>(l);
        }
        if (!(moved <= 1.f)) continue;
      }
      const float wx[2] = {1.f - f[0], f[0]}, wy[2] = {1.f - f[1], f[1]}, wz[2] = {1.f - f[2], f[2]};
      const float wzy[4] = {wz[0] * wy[0], wz[0] * wy[1], wz[1] * wy[0], wz[1] * wy[1]};
      // (an axis one voxel thick: both taps are that voxel, the high one with weight 0)
      const unsigned bx[2] = {static_cast<unsigned>(b0[0]), static_cast<unsigned>(min(b0[0] + 1, kInterior ? b0[0] + 1 : max(n0 - 1, 0)))};
      const unsigned by[2] = {static_cast<unsigned>(b0[1]), static_cast<unsigned>(min(b0[1] + 1, kInterior ? b0[1] + 1 : max(n1 - 1, 0)))};
      const unsigned bz[2] = {static_cast<unsigned>(b0[2]), static_cast<unsigned>(min(b0[2] + 1, kInterior ? b0[2] + 1 : max(n2 - 1, 0)))};
      const bool inside = max(bx[0], bx[1]) < static_cast<unsigned>(n0) && max(by[0], by[1]) < static_cast<unsigned>(n1) &&
                          max(bz[0], bz[1]) < static_cast<unsigned>(n2);
      if (inside) {
        const float gq = g * gq_scale;
        const int rows[4] = {__mul24(__mul24(bz[0], n1) + by[0], n0), __mul24(__mul24(bz[0], n1) + by[1], n0),
                             __mul24(__mul24(bz[1], n1) + by[0], n0), __mul24(__mul24(bz[1], n1) + by[1], n0)};
#pragma unroll
        for (int n = 0; n < 8; n++)
          __hip_atomic_fetch_add(tile + rows[n >> 1] + static_cast<int>(bx[n & 1]),
                                 __float2int_rn(gq * (wzy[n >> 1] * wx[n & 1])), __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_WORKGROUP);
      } else {   // (rounding beyond the box's margin: not expected; the voxels exist in the volume)
#pragma unroll 1
        for (int n = 0; n < 8; n++) {
          const float w = wzy[n >> 1] * wx[n & 1];
          const long zi = l2 + static_cast<int>(bz[n >> 2]), yi = l1 + static_cast<int>(by[(n >> 1) & 1]), xi = l0 + static_cast<int>(bx[n & 1]);
          if (w != 0.f && zi >= 0 && zi < p.D && yi >= 0 && yi < p.H && xi >= 0 && xi < p.W)
            atomic_add_element(vol, (zi * p.H + yi) * p.W + xi, g * w);
        }
      }
      }   // samples of the bin
    }
    };
    auto scatter_cells = [&](auto interior_tag, auto order_tag, auto grids_tag) {
    constexpr bool kInterior = decltype(interior_tag)::value;
    constexpr int kOrder = decltype(order_tag)::value;
    constexpr bool kGrids = decltype(grids_tag)::value;
    const int sgx = kGrids ? plan_scalar(&r.grid[0]) : 1, sgy = kGrids ? plan_scalar(&r.grid[1]) : 1, sgz = kGrids ? plan_scalar(&r.grid[2]) : 1;
    const double dgx = 1.0 / sgx, dgy = 1.0 / sgy, dgz = 1.0 / sgz;
#pragma unroll
    for (int k = 0; k < kPerThread; k++) {
      const int c = threadIdx.x + k * kScatterThreads;
      const int x = c % TX, y = (c / TX) % TY, z = c / (TX * TY);
      const float g = gv[k];
      if (g == 0.f) continue;
      for (int iz = 0; iz < sgz; iz++)
      for (int iy = 0; iy < sgy; iy++)
      for (int ix = 0; ix < sgx; ix++) {
      const double sx_ = kGrids ? x + ix * dgx : x, sy_ = kGrids ? y + iy * dgy : y, sz_ = kGrids ? z + iz * dgz : z;
      const double vx = map[0] + map[1] * sx_ + map[2] * sy_ + map[3] * sz_;
      const double vy = map[4] + map[5] * sx_ + map[6] * sy_ + map[7] * sz_;
      const double vz = map[8] + map[9] * sx_ + map[10] * sy_ + map[11] * sz_;
      int xi[2], yi[2], zi[2];
      float fx, fy, fz;
      if constexpr (kInterior) {
        const double flx = floor(vx), fly = floor(vy), flz = floor(vz);
        xi[0] = static_cast<int>(flx); yi[0] = static_cast<int>(fly); zi[0] = static_cast<int>(flz);
        xi[1] = xi[0] + 1; yi[1] = yi[0] + 1; zi[1] = zi[0] + 1;
        const double dx = vx - flx, dy = vy - fly, dz = vz - flz;
        if constexpr (kOrder == 0) {
          fx = (1.0 - dx >= 0.5) ? 0.f : 1.f; fy = (1.0 - dy >= 0.5) ? 0.f : 1.f; fz = (1.0 - dz >= 0.5) ? 0.f : 1.f;
        } else {
          fx = static_cast<float>(dx); fy = static_cast<float>(dy); fz = static_cast<float>(dz);
        }
      } else if (!clamped_tap<float>(vx, p.W, xi[0], xi[1], fx, kOrder) || !clamped_tap<float>(vy, p.H, yi[0], yi[1], fy, kOrder) ||
                 !clamped_tap<float>(vz, p.D, zi[0], zi[1], fz, kOrder)) {
        continue;
      }
      const float wx[2] = {1.f - fx, fx}, wy[2] = {1.f - fy, fy}, wz[2] = {1.f - fz, fz};
      const float wzy[4] = {wz[0] * wy[0], wz[0] * wy[1], wz[1] * wy[0], wz[1] * wy[1]};
      const unsigned bx[2] = {static_cast<unsigned>(xi[0] - l0), static_cast<unsigned>(xi[1] - l0)};
      const unsigned by[2] = {static_cast<unsigned>(yi[0] - l1), static_cast<unsigned>(yi[1] - l1)};
      const unsigned bz[2] = {static_cast<unsigned>(zi[0] - l2), static_cast<unsigned>(zi[1] - l2)};
      // the box holds every voxel a sample of the tile touches; a cell that disagrees takes the slow way
      const bool inside = in_lds && max(bx[0], bx[1]) < static_cast<unsigned>(n0) &&
                          max(by[0], by[1]) < static_cast<unsigned>(n1) && max(bz[0], bz[1]) < static_cast<unsigned>(n2);
      if (inside) {
        const float gq = g * to_quanta;   // a power of two: the products below are the terms in quanta
        const int rows[4] = {__mul24(__mul24(bz[0], n1) + by[0], n0), __mul24(__mul24(bz[0], n1) + by[1], n0),
                             __mul24(__mul24(bz[1], n1) + by[0], n0), __mul24(__mul24(bz[1], n1) + by[1], n0)};
#pragma unroll
        for (int n = 0; n < 8; n++)
          __hip_atomic_fetch_add(tile + rows[n >> 1] + static_cast<int>(bx[n & 1]),
                                 __float2int_rn(gq * (wzy[n >> 1] * wx[n & 1])), __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_WORKGROUP);
      } else {
#pragma unroll 1
        for (int n = 0; n < 8; n++) {
          const float w = wzy[n >> 1] * wx[n & 1];
          if (w != 0.f)
            atomic_add_element(vol, (static_cast<long>(zi[n >> 2]) * p.H + yi[(n >> 1) & 1]) * p.W + xi[n & 1], g * w);
        }
      }
      }   // samples of the bin
    }
    };
    using Yes = std::true_type;
    using No = std::false_type;
    if constexpr (GRIDS) {   // (one copy of the loops for grids: the clamped form covers unclipped boxes too)
      if (sizeof(T) == 2 && p.order == 1 && in_lds) scatter_cells32(No{}, Yes{});
      else if (p.order == 0) scatter_cells(No{}, std::integral_constant<int, 0>{}, Yes{});
      else scatter_cells(No{}, std::integral_constant<int, 1>{}, Yes{});
    } else if (sizeof(T) == 2 && p.order == 1 && in_lds) {
      if (mode == 3 && p.ndim == 3) scatter_cells32(Yes{}, No{});
      else scatter_cells32(No{}, No{});
    } else if (mode == 3 && p.ndim == 3) {
      if (p.order == 0) scatter_cells(Yes{}, std::integral_constant<int, 0>{}, No{});
      else scatter_cells(Yes{}, std::integral_constant<int, 1>{}, No{});
    } else {
      if (p.order == 0) scatter_cells(No{}, std::integral_constant<int, 0>{}, No{});
      else scatter_cells(No{}, std::integral_constant<int, 1>{}, No{});
    }
    if (in_lds) {
      __syncthreads();
      // Lanes run along the box's cells in memory order (consecutive lanes = consecutive voxels of a
      // row = one request per 64-byte sector); several independent reads per lane are in flight
      // before the first is looked at.
      constexpr int kAtOnce = 8;
      const int box = n0 * n1 * n2;
      if constexpr (DIRECT) {
        // a lane takes an aligned pair of voxels (volume x even): cells first - l0 and first - l0 + 1 of a
        // box row, either of which may lie outside the row
        const int first = l0 & ~1, pairs = ((l0 + n0 + 1) >> 1) - (l0 >> 1), rows = n1 * n2;
        const float inv_pairs = 1.f / static_cast<float>(pairs), inv_rows = 1.f / static_cast<float>(n1);
        for (int base = threadIdx.x; base < rows * pairs; base += kScatterThreads * kAtOnce) {
          int q0[kAtOnce], q1[kAtOnce], cell[kAtOnce], row_[kAtOnce];
#pragma unroll
          for (int u = 0; u < kAtOnce; u++) {
            const int i = base + u * kScatterThreads;
            const int row = div_small(i, inv_pairs), bx = first - l0 + 2 * (i - row * pairs);
            const bool on = i < rows * pairs;
            cell[u] = row * n0 + bx;
            row_[u] = row;
            q0[u] = (on && bx >= 0) ? tile[cell[u]] : 0;
            q1[u] = (on && bx + 1 < n0) ? tile[cell[u] + 1] : 0;
          }
#pragma unroll
          for (int u = 0; u < kAtOnce; u++) {
            if ((q0[u] | q1[u]) == 0) continue;
            if (q0[u] != 0) tile[cell[u]] = 0;
            if (q1[u] != 0) tile[cell[u] + 1] = 0;
            const int row = row_[u], bx = cell[u] - row * n0;
            const int bz = div_small(row, inv_rows), by = row - bz * n1;
            atomic_add_pair(vol + (static_cast<long>(bz + l2) * p.H + (by + l1)) * p.W + (l0 + bx),
                            static_cast<float>(q0[u]) * from_quanta, static_cast<float>(q1[u]) * from_quanta);
          }
        }
        __syncthreads();
        continue;
      }
      const float inv_row = 1.f / static_cast<float>(n0), inv_rows = 1.f / static_cast<float>(n1);
      for (int base = threadIdx.x; base < box; base += kScatterThreads * kAtOnce) {
        int q[kAtOnce];
#pragma unroll
        for (int u = 0; u < kAtOnce; u++) {
          const int i = base + u * kScatterThreads;
          q[u] = i < box ? tile[i] : 0;
        }
#pragma unroll
        for (int u = 0; u < kAtOnce; u++) {
          if (q[u] == 0) continue;
          const int i = base + u * kScatterThreads;
          tile[i] = 0;
          const int row = div_small(i, inv_row), bx = i - row * n0;
          const int bz = div_small(row, inv_rows), by = row - bz * n1;
          atomic_add_element(vol, (static_cast<long>(bz + l2) * p.H + (by + l1)) * p.W + (l0 + bx),
                             static_cast<float>(q[u]) * from_quanta);
        }
      }
      __syncthreads();
    }
  }
}

struct ScatterTiling { int TX, TY, TZ; long tx, ty, tz, per_roi, total, work; };
static ScatterTiling scatter_tiling(const RoiProblem &p) {
  ScatterTiling t;
  const bool flat = p.ndim == 2;
  const int vol[3] = {MV_SCATTER_SHAPE}, img[3] = {MV_SCATTER_SHAPE_2D};
  t.TX = flat ? img[0] : vol[0]; t.TY = flat ? img[1] : vol[1]; t.TZ = flat ? img[2] : vol[2];
  t.tx = (p.ow + t.TX - 1) / t.TX; t.ty = (p.oh + t.TY - 1) / t.TY; t.tz = (p.od + t.TZ - 1) / t.TZ;
  t.per_roi = t.tx * t.ty * t.tz; t.total = t.per_roi * static_cast<long>(p.R); t.work = t.total * p.C;
  return t;
}

bool roi_backward_tiled_applies(int dtype, const RoiProblem &p) {
  const long vox = static_cast<long>(p.od) * p.oh * p.ow;
  if ((p.order != 0 && p.order != 1) || vox < 4096 || p.ow < 16 || p.R == 0) return false;
  if (dtype != MV_F16 && dtype != MV_BF16 && dtype != MV_F32) return false;
  return scatter_tiling(p).work < (1L << 31) && static_cast<long>(p.D) * p.H * p.W * 4 < (1L << 31);
}

// fp16 gradients whose rows hold an even number of voxels need no fp32 buffer: the tiles' sums go
// straight into the gradient tensor as packed atomics on pairs of voxels.
bool roi_backward_tiled_direct(int dtype, const RoiProblem &p, const void *grad_input) {
  // (grids of up to 3 per axis: a tile's voxel then gets at most 48 x 48 x 24 terms, which its 32-bit sums
  // hold at 14 bits each; larger and adaptive grids may need single terms, which want the fp32 buffer)
  return dtype == MV_F16 && p.W % 2 == 0 && reinterpret_cast<uintptr_t>(grad_input) % 4 == 0 &&
         p.sampling_ratio >= 1 && p.sampling_ratio <= 3 && roi_backward_tiled_applies(dtype, p);
}

// `acc`: fp32 gradient buffer [N, C, D, H, W] that the terms are added to, or (`direct`, see above) the
// fp16 gradient tensor itself.  Returns -1 when the path does not apply.
int roi_backward_tiled(const void *grad_output, const void *rois, void *acc, int dtype,
                       const RoiProblem &p, hipStream_t s, bool direct) {
  if (!roi_backward_tiled_applies(dtype, p)) return -1;
  if (direct && !roi_backward_tiled_direct(dtype, p, acc)) return -1;
  const ScatterTiling t = scatter_tiling(p);
  const bool flat = p.ndim == 2;
  const int TX = t.TX, TY = t.TY, TZ = t.TZ;
  const long tx = t.tx, ty = t.ty, tz = t.tz, per_roi = t.per_roi, total = t.total, work = t.work;
  PlanShape ps;
  ps.tiles_x = static_cast<int>(tx); ps.tiles_y = static_cast<int>(ty); ps.tiles_z = static_cast<int>(tz);
  ps.tx = TX; ps.ty = TY; ps.tz = TZ;
  ps.vec = 0;
  ps.cap = kScatterLds / 4;
  ps.threads = kScatterThreads; ps.max_items = 0;
  ps.halo_lo = 0; ps.halo_hi = 1;
  ps.grids = 1; ps.flat_axis = 0;
  ps.warm_groups = 0;
  ps.pad_slices = 0;
  ps.es = 4;
  ps.by_per_roi.set(static_cast<unsigned>(per_roi));
  ps.by_tiles_x.set(static_cast<unsigned>(tx));
  ps.by_tiles_y.set(static_cast<unsigned>(ty));
  ps.by_total.set(static_cast<unsigned>(total));
  ps.by_slots.set(1);
  long blocks = std::min<long>(work, static_cast<long>(kScatterWgs) * compute_units());
  blocks = std::max(blocks, (work + kPlanSlots - 1) / kPlanSlots);
  const bool grids = p.sampling_ratio != 1;
#define MV_SCATTER_LAUNCH(TYPE, DIRECTV, GRIDSV)                                                                       \
  do {                                                                                                                \
    if (flat)                                                                                                         \
      hipLaunchKernelGGL((roi_backward_tiles_kernel<TYPE, MV_SCATTER_SHAPE_2D, DIRECTV, GRIDSV>),                    \
                         dim3(static_cast<unsigned>(blocks)), dim3(kScatterThreads), 0, s,                            \
                         static_cast<const TYPE *>(grad_output), static_cast<const float *>(rois), acc, p, ps,        \
                         static_cast<unsigned>(total), static_cast<unsigned>(work));                                  \
    else                                                                                                              \
      hipLaunchKernelGGL((roi_backward_tiles_kernel<TYPE, MV_SCATTER_SHAPE, DIRECTV, GRIDSV>),                       \
                         dim3(static_cast<unsigned>(blocks)), dim3(kScatterThreads), 0, s,                            \
                         static_cast<const TYPE *>(grad_output), static_cast<const float *>(rois), acc, p, ps,        \
                         static_cast<unsigned>(total), static_cast<unsigned>(work));                                  \
  } while (0)
  if (direct) {
    if (grids) MV_SCATTER_LAUNCH(__half, true, true);
    else MV_SCATTER_LAUNCH(__half, true, false);
  } else if (dtype == MV_F16) {
    if (grids) MV_SCATTER_LAUNCH(__half, false, true);
    else MV_SCATTER_LAUNCH(__half, false, false);
  } else if (dtype == MV_BF16) {
    if (grids) MV_SCATTER_LAUNCH(__hip_bfloat16, false, true);
    else MV_SCATTER_LAUNCH(__hip_bfloat16, false, false);
  } else {
    if (grids) MV_SCATTER_LAUNCH(float, false, true);
    else MV_SCATTER_LAUNCH(float, false, false);
  }
#undef MV_SCATTER_LAUNCH
  return check_launch("roi_backward_tiles_kernel");
}

}  // namespace mv

#ifdef MV_RESAMPLE_TIMELINE
// Copies the time stamps of the last tiled forward launches to `host` (kTimelineGroups x kTimelineSlots
// 64-bit words, 100 MHz ticks); synchronises the device.
extern "C" int mv_debug_resample_timeline(void *host, size_t bytes) {
  const size_t all = sizeof(unsigned long long) * mv::kTimelineGroups * mv::kTimelineSlots;
  return static_cast<int>(hipMemcpyFromSymbol(host, HIP_SYMBOL(mv::mv_timeline), bytes < all ? bytes : all));
}

// The tap reads of the tiled forward kernel on their own (a measuring aid like the time stamps above): 512
// threads and two workgroups per compute unit as in the kernel, a 16-bit box in LDS, every lane a column of
// eight voxels whose low corners follow a rotation by `degrees` about all three axes; the corner addresses
// are worked out before the timed loop, which holds little besides the reads.  FORM 0: eight 2-byte reads per
// voxel (what the kernel does); 1: four `ds_read2_b32` (two dwords each, the first at the even voxel at or
// below the low tap); 2: four `ds_read_b64` at those 4-byte-aligned addresses; 3: four aligned dword reads,
// as a second copy of the box shifted by one voxel would allow (the odd lanes read elsewhere in the tile).
namespace mv {
struct TapReadShape { float m[12]; int n0, n1, n2, pitch, slice, iters, one; };
template <int FORM>
__global__ __launch_bounds__(512, 2) void lds_tap_reads_kernel(const TapReadShape p, unsigned *out) {
  __shared__ __attribute__((aligned(16))) unsigned short box[74 * 1024 / 2];
  for (int i = threadIdx.x; i < 74 * 1024 / 2; i += 512) box[i] = static_cast<unsigned short>(i * 7 + 1);
  __syncthreads();
  const int ox = threadIdx.x % 16, oy = threadIdx.x / 16 % 16, zb = threadIdx.x / 256 * 8;
  unsigned acc = 0;
  int base_k[8], x_k[8];
#pragma unroll
  for (int k = 0; k < 8; k++) {
    const float x = ox, y = oy, z = zb + k;
    const float sx = p.m[0] + p.m[1] * x + p.m[2] * y + p.m[3] * z, sy = p.m[4] + p.m[5] * x + p.m[6] * y + p.m[7] * z;
    const float sz = p.m[8] + p.m[9] * x + p.m[10] * y + p.m[11] * z;
    const int x0 = min(max(static_cast<int>(sx), 0), p.n0 - 3), y0 = min(max(static_cast<int>(sy), 0), p.n1 - 3);
    const int z0 = min(max(static_cast<int>(sz), 0), p.n2 - 3);
    base_k[k] = z0 * p.slice + y0 * p.pitch;
    x_k[k] = x0;
  }
  for (int it = 0; it < p.iters; it++) {
    const int shift = (it & 1) * p.pitch;
#pragma unroll
    for (int k = 0; k < 8; k++) {
      const int base = base_k[k] + shift, x0 = x_k[k];
      if (FORM == 0) {
        const unsigned short *b = box + base + x0;
        const int o = p.one;   // (a run-time 1: the compiler would merge b[0] and b[1] into one misaligned dword read)
        acc ^= b[0] ^ b[o] ^ b[p.pitch] ^ b[p.pitch + o] ^ b[p.slice] ^ b[p.slice + o] ^ b[p.slice + p.pitch] ^ b[p.slice + p.pitch + o];
      } else if (FORM == 3) {
        const unsigned *w = reinterpret_cast<const unsigned *>(box) + ((base + (x0 & ~1)) >> 1) + (x0 & 1) * 4096;
        acc ^= w[0] ^ w[p.pitch >> 1] ^ w[p.slice >> 1] ^ w[(p.slice + p.pitch) >> 1];
      } else {
        unsigned long long v[4];
        const int offs[4] = {0, p.pitch, p.slice, p.slice + p.pitch};
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const unsigned addr = static_cast<unsigned>(reinterpret_cast<size_t>(box + base + offs[q] + (x0 & ~1)));
          if (FORM == 1) asm volatile("ds_read2_b32 %0, %1 offset1:1" : "=v"(v[q]) : "v"(addr));
          else asm volatile("ds_read_b64 %0, %1" : "=v"(v[q]) : "v"(addr));
        }
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]));
        acc ^= static_cast<unsigned>(v[0]) ^ static_cast<unsigned>(v[1] >> 32) ^ static_cast<unsigned>(v[2]) ^ static_cast<unsigned>(v[3] >> 32);
      }
    }
  }
  out[blockIdx.x * 512 + threadIdx.x] = acc;
}
}  // namespace mv

// Runs form `form` (0..3) on 2 x the compute units' workgroups, `iters` rounds of eight voxels per lane; `out` holds
// 1024 x compute units words of device memory.  `*ms`: the launch's duration by HIP events (synchronises the stream).
extern "C" int mv_debug_lds_tap_reads(int form, int iters, float degrees, unsigned *out, float *ms, void *stream) {
  mv::TapReadShape p;
  const double a = degrees * 3.14159265358979323846 / 180.0, ca = cos(a), sa = sin(a);
  const double rot[9] = {ca * ca, ca * sa * sa - sa * ca, ca * sa * ca + sa * sa, sa * ca, sa * sa * sa + ca * ca,
                         sa * sa * ca - ca * sa, -sa, ca * sa, ca * ca};
  for (int r = 0; r < 3; r++) {
    p.m[4 * r] = 8.f;
    for (int c = 0; c < 3; c++) p.m[4 * r + 1 + c] = static_cast<float>(rot[3 * r + c]);
  }
  p.n0 = 24; p.n1 = 24; p.n2 = 24; p.pitch = 24; p.slice = 24 * 24 + 16; p.iters = iters; p.one = 1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(2 * mv::compute_units()), block(512);
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return 1;
  (void)hipEventRecord(e0, s);
  switch (form) {
    case 0: hipLaunchKernelGGL(mv::lds_tap_reads_kernel<0>, grid, block, 0, s, p, out); break;
    case 1: hipLaunchKernelGGL(mv::lds_tap_reads_kernel<1>, grid, block, 0, s, p, out); break;
    case 2: hipLaunchKernelGGL(mv::lds_tap_reads_kernel<2>, grid, block, 0, s, p, out); break;
    default: hipLaunchKernelGGL(mv::lds_tap_reads_kernel<3>, grid, block, 0, s, p, out);
  }
  (void)hipEventRecord(e1, s);
  const hipError_t st = hipEventSynchronize(e1);
  if (st == hipSuccess) (void)hipEventElapsedTime(ms, e0, e1);
  (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
  return st == hipSuccess ? 0 : 1;
}
#endif
