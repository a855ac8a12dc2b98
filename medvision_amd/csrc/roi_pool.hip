// RoIAlign for plain (axis-aligned) boxes with SMALL outputs per roi (detection heads: thousands of
// rois, 7x7x7 cells, hundreds of channels), forward and backward.  Same results as the reference's
// one-thread-per-output kernels (csrc/cuda/roi_align_3d_cuda_kernel.cuh:11-86 forward, :90-202
// backward with eight atomicAdd per sample, :189-196; 2-D twin roi_align_2d_cuda_kernel.cuh).
//
// For an axis-aligned box the sample coordinates are separable: x depends only on (pw, ix), y on
// (ph, iy), z on (pd, iz).  Each axis therefore has a short tap table (cells * grid entries of
// {low index, high index, two weights}; validity and the 1/grid factor folded into the weights)
// and the pooled output is the source sub-box contracted with three small sparse matrices:
//     out[pd,ph,pw] = sum_z Wz[pd,z] sum_y Wy[ph,y] sum_x Wx[pw,x] * box[z,y,x]
// One workgroup = (roi, chunk of channels).  It builds the tables, copies the roi's source sub-box
// of its channels into LDS (every feature voxel is read once per roi instead of once per sample
// corner), runs the three contractions through LDS and writes the outputs with coalesced stores.
// The backward runs the transposed contractions and adds the sub-box gradient to global memory:
// one atomic per touched feature voxel and (roi, channel) instead of one per sample corner
// (config 5: ~64 instead of 21 952).
// rois whose sub-box or tables exceed the LDS budget are handled in the same workgroup by a plain
// per-output gather / scatter.
// fp16 heads with up to 8 cells per axis (7 x 7 x 7 detection heads) take matrix-core forms of the
// same contractions instead (pool_forward_mfma, pool_backward_mfma): the (y, x) contraction as a
// GEMM against the products Wy[y][ph] Wx[x][pw] held in LDS, operands read straight from global
// memory, no barrier after the set-up; the forward pass optionally from a blocked copy of the
// features (pool_block_features_kernel) in which the few voxels of a box row share their memory
// sectors with the other channels.
#include "common.hpp"
#include "roi_geometry.hpp"
#include "sampling.hpp"
#include "dcn_mfma.hpp"

namespace mv {

constexpr int kPoolThreads = 256;
constexpr int kPoolEntries = 128;              // tap-table entries per axis (cells * grid)
constexpr int kPoolFirst = 256;                // widest box (voxels per axis) of the transposed contractions
constexpr int kPoolLdsBytes = 40 * 1024;       // staged data + intermediates of one channel chunk

// i / d for 0 <= i < 2^21 and 0 < d < 2^12, with inv = 1.0f / d (exact: the product is at least
// 0.5 / d away from an integer and its rounding error is below that)
__device__ __forceinline__ int fdiv(int i, float inv) { return static_cast<int>((static_cast<float>(i) + 0.5f) * inv); }

struct AxisTaps {
  short lo[kPoolEntries], hi[kPoolEntries];    // box-relative tap indices (16 bits: the tables decide how many workgroups share a compute unit's LDS)
  float wlo[kPoolEntries], whi[kPoolEntries];  // weights (0 for void samples), include 1 / grid
  short first[kPoolFirst + 4];                 // first[i] = first entry whose low tap is >= i (box-relative)
  int box_lo, box_hi;                          // inclusive source range covered by valid taps
  int entries, grid;
};

struct PoolShared {
  RoiGeom g;
  AxisTaps ax[3];  // x, y, z
};

// The tap entries of one output cell (grid <= kTapRegs samples) in registers; unused entries have
// weight 0 and index 0.
constexpr int kTapRegs = 2;
struct TapRegs {
  int lo[kTapRegs], hi[kTapRegs];
  float wlo[kTapRegs], whi[kTapRegs];
  __device__ __forceinline__ void load(const AxisTaps &t, int cell) {
#pragma unroll
    for (int s = 0; s < kTapRegs; s++) {
      const bool on = s < t.grid;
      const int e = on ? cell * t.grid + s : 0;
      lo[s] = on ? t.lo[e] : 0; hi[s] = on ? t.hi[e] : 0;
      wlo[s] = on ? t.wlo[e] : 0.f; whi[s] = on ? t.whi[e] : 0.f;
    }
  }
  // sum over the entries of w * row[index * stride]
  template <typename E>
  __device__ __forceinline__ float apply(const E *row, int stride) const {
    float acc = 0.f;
#pragma unroll
    for (int s = 0; s < kTapRegs; s++)
      acc += wlo[s] * load_any(row + lo[s] * stride) + whi[s] * load_any(row + hi[s] * stride);
    return acc;
  }
  static __device__ __forceinline__ float load_any(const float *p) { return *p; }
  static __device__ __forceinline__ float load_any(const __half *p) { return mv::load(p); }
  static __device__ __forceinline__ float load_any(const __hip_bfloat16 *p) { return mv::load(p); }
};

struct PoolPlan {
  int staged;      // 1: LDS path, 0: per-output gather, -1: every output is zero
  int chunk;       // channels per LDS pass
};

static_assert(kPoolEntries % kWave == 0, "one wavefront builds the tap table of one axis, kPoolEntries / kWave entries per lane");
constexpr int kDenseSrc = 32;   // source voxels per axis of the dense weight matrices (see below)

// Builds geometry and tap tables for roi `roi`; all threads must call it (contains barriers).
// Wavefront a (0..2) works out axis a on its own: the axis geometry (the same expressions as
// build_geom), one tap entry per lane, the box bounds by a reduction inside the wavefront and, when
// `wd` is given and the axis fits, the dense weight matrix wd[a][source index][cell] = sum of the
// weights of the cell's samples that touch the source index (samples in their order; a wavefront's
// LDS operations execute in order).  The fourth wavefront writes the whole geometry for the plain
// gather / scatter paths.  One barrier.
template <typename RT, int CELLS>
__device__ inline PoolPlan pool_setup(PoolShared &sh, const RT *roi, const RoiProblem &p, size_t elem_bytes,
                                      float (*wd)[kDenseSrc][CELLS], bool slabs = false, bool sparse_gather = false) {
  const int nd = p.ndim;
  const int cells[3] = {p.ow, p.oh, p.od};
  const int size[3] = {p.W, p.H, p.D};
  const int b = static_cast<int>(roi[0]);
  // extents and sampling grids of all axes (every lane the same): they decide the path
  double start[3], ext[3];
  int grid[3], entries[3];
  PoolPlan plan{1, 0};
  if (b < 0 || b >= p.N) plan.staged = -1;
#pragma unroll
  for (int a = 0; a < 3; a++) {
    start[a] = 0.0; ext[a] = 0.0; grid[a] = 1;
    if (a < nd) {
      const double lo = static_cast<double>(roi[1 + a]) * p.scale;
      const double hi = static_cast<double>(roi[1 + nd + a]) * p.scale;
      ext[a] = fmax(hi - lo, 1.0);
      start[a] = lo;
      grid[a] = p.sampling_ratio > 0 ? p.sampling_ratio
                                     : static_cast<int>(ceil(ext[a] / static_cast<double>(cells[a])));
    }
    entries[a] = cells[a] * max(grid[a], 0);
    if (entries[a] > kPoolEntries) plan.staged = min(plan.staged, 0);
  }
#pragma unroll
  for (int a = 0; a < 3; a++)
    if (entries[a] <= 0) plan.staged = -1;  // empty sampling grid: outputs are zero
  const int a = threadIdx.x / kWave, i = threadIdx.x % kWave;
  if (a == 3 || plan.staged <= 0) {
    if (a == 3 || plan.staged == 0) {   // (plan.staged == 0: every wavefront the same values)
      const double sn[3] = {0, 0, 0}, cs[3] = {1, 1, 1};
      RoiGeom g;
      build_geom(g, roi, p, sn, cs);
      if (i == 0) sh.g = g;
    }
  } else {
    AxisTaps &t = sh.ax[a];
    const int gr = a == 0 ? grid[0] : (a == 1 ? grid[1] : grid[2]);
    const int en = a == 0 ? entries[0] : (a == 1 ? entries[1] : entries[2]);
    const int sz = a == 0 ? size[0] : (a == 1 ? size[1] : size[2]);
    const int nc = a == 0 ? cells[0] : (a == 1 ? cells[1] : cells[2]);
    const double st = a == 0 ? start[0] : (a == 1 ? start[1] : start[2]);
    const double ex = a == 0 ? ext[0] : (a == 1 ? ext[1] : ext[2]);
    const double bin = a < nd ? ex / static_cast<double>(nc) : 0.0;
    const double sub_step = bin / static_cast<double>(gr > 0 ? gr : 1);
    // entries e = i, i + 64, ...: the coordinates grow with the entry (plain boxes have positive
    // extents), so the box runs from the low tap of the first valid sample to the high tap of the last
    constexpr int kPer = kPoolEntries / kWave;
    const float inv = 1.f / static_cast<float>(gr);
    int lo_[kPer], hi_[kPer], cell_[kPer], sub_[kPer];
    float frac_[kPer];
    bool ok_[kPer], up_[kPer];
    int box_lo = 1 << 30, box_hi = -1;
#pragma unroll
    for (int h = 0; h < kPer; h++) {
      const int e = i + h * kWave;
      const bool on = e < en;
      cell_[h] = on ? e / gr : 0; sub_[h] = on ? e % gr : 0;
      // (local_coord's expression)
      const double v = a < nd ? st + cell_[h] * bin + static_cast<double>(static_cast<float>(sub_[h]) + .5f) * sub_step : 0.0;
      lo_[h] = 0; hi_[h] = 0; frac_[h] = 0.f;
      ok_[h] = clamped_tap<float>(v, sz, lo_[h], hi_[h], frac_[h], p.order) && on;
      up_[h] = v > 0.0;
      const unsigned long long valid = __ballot(ok_[h]);
      if (valid) {
        if (box_hi < 0) box_lo = __builtin_amdgcn_readlane(lo_[h], __builtin_ctzll(valid));
        box_hi = __builtin_amdgcn_readlane(hi_[h], 63 - __builtin_clzll(valid));
      }
    }
    const int top = box_hi - box_lo;
    const bool on = i < en;   // (first entry of the lane: what the dense matrices below are built from)
    const bool ok = ok_[0];
    const int cell = cell_[0], sub = sub_[0];
    const float wlo = ok ? (1.f - frac_[0]) * inv : 0.f, whi = ok ? frac_[0] * inv : 0.f;
    const int rlo = ok ? lo_[0] - box_lo : (up_[0] ? top : 0), rhi = ok ? hi_[0] - box_lo : (up_[0] ? top : 0);
#pragma unroll
    for (int h = 0; h < kPer; h++) {
      const int e = i + h * kWave;
      if (e < en) {
        // void samples keep weight 0; they are parked at the matching end so that `lo` stays monotonic
        t.lo[e] = ok_[h] ? lo_[h] - box_lo : (up_[h] ? top : 0);
        t.hi[e] = ok_[h] ? hi_[h] - box_lo : (up_[h] ? top : 0);
        t.wlo[e] = ok_[h] ? (1.f - frac_[h]) * inv : 0.f;
        t.whi[e] = ok_[h] ? frac_[h] * inv : 0.f;
      }
    }
    (void)on;
    if (i == 0) {
      t.box_lo = box_lo; t.box_hi = box_hi;
      t.entries = en; t.grid = gr;
    }
    if (wd != nullptr && box_hi >= 0 && top < kDenseSrc && nc <= CELLS && en <= kWave) {
      float *m = &wd[a][0][0];
      for (int k = i; k < kDenseSrc * CELLS / 4; k += kWave) reinterpret_cast<float4 *>(m)[k] = float4{0.f, 0.f, 0.f, 0.f};
      for (int sidx = 0; sidx < gr; sidx++) {
        __builtin_amdgcn_wave_barrier();   // (keeps the samples' read-modify-write rounds apart)
        if (ok && sub == sidx) {
          m[rlo * CELLS + cell] += wlo;
          m[rhi * CELLS + cell] += whi;
        }
      }
    }
  }
  __syncthreads();
  if (plan.staged <= 0) return plan;
  long vol = 1;
#pragma unroll
  for (int k = 0; k < 3; k++) {
    if (sh.ax[k].box_hi < 0) plan.staged = -1;  // no valid sample on this axis
    vol *= sh.ax[k].box_hi - sh.ax[k].box_lo + 1;
  }
  if (plan.staged != 1) return plan;
  if (sparse_gather) {
    // A box that holds more than half as many voxels as the roi's samples have taps is read sparsely (bins
    // of several voxels with a small grid: large rois on fine feature maps): staging and contracting the
    // whole box costs more than fetching the taps.  Measured on 1000 rois of 16 - 116 pixels x 256 channels
    // x 7^2 cells, grid 2: 1.58 -> 0.38 ms (fp16), 1.55 -> 0.47 ms (fp32); 500 rois of 8 - 32 voxels x 64
    // channels x 7^3, grid 1: 0.50 -> 0.10 ms; dense heads (bins of a voxel or less) are not affected.
    long taps = 1;
    for (int k = 0; k < nd; k++) taps *= 2L * entries[k];
    if (2 * vol > taps) { plan.staged = 0; return plan; }
  }
  {
    const long nz = sh.ax[2].box_hi - sh.ax[2].box_lo + 1, ny = sh.ax[1].box_hi - sh.ax[1].box_lo + 1;
    const long per_channel = vol * static_cast<long>(elem_bytes) + (nz * ny * p.ow + nz * p.oh * p.ow) * 4 + 16;
    const long chunk = kPoolLdsBytes / per_channel;
    if (chunk < 1 && !slabs) plan.staged = 0;   // (a caller that works in slabs of box planes sizes them itself)
    plan.chunk = static_cast<int>(min(chunk, 64L));
  }
  return plan;
}

// The entry ranges per source index (`first`) of a staged roi; all threads, ends with a barrier.
__device__ inline void pool_first(PoolShared &sh) {
  for (int e = threadIdx.x; e < 3 * (kPoolFirst + 4); e += kPoolThreads) {
    const int k = e / (kPoolFirst + 4), j = e % (kPoolFirst + 4);
    AxisTaps &t = sh.ax[k];
    if (j > t.box_hi - t.box_lo + 1) continue;
    int f = 0;
    while (f < t.entries && t.lo[f] < j) f++;
    t.first[j] = f;
  }
  __syncthreads();
}

// Dense form of the tap tables for the usual small boxes (<= CELLS cells per axis, box of
// <= kDenseSrc voxels per axis): per axis a matrix Wd[source index][cell] = sum of the weights of
// the cell's samples that touch the source index.  A contraction then is "walk the line, multiply
// each value into all cells" (forward) or "load the cells of a line, one dot product per source
// index" (backward): no per-entry branches, the matrix rows are LDS broadcasts.
// The kernels are instantiated for CELLS = 8 (7^3 detection heads) and 16 (14 x 14 mask heads).
template <int CELLS>
__device__ __forceinline__ bool dense_applies(const PoolShared &sh, const RoiProblem &p) {
  for (int a = 0; a < 3; a++)
    if (sh.ax[a].box_hi - sh.ax[a].box_lo + 1 > kDenseSrc || sh.ax[a].entries > kWave) return false;
  return p.ow <= CELLS && p.oh <= CELLS && p.od <= CELLS;
}

// all threads of the workgroup; followed by a barrier
template <int CELLS>
__device__ inline void dense_build(const PoolShared &sh, const RoiProblem &p, float (&wd)[3][kDenseSrc][CELLS]) {
  const int ncell[3] = {p.ow, p.oh, p.od};
  for (int i = threadIdx.x; i < 3 * kDenseSrc * CELLS; i += kPoolThreads) {
    const int a = i / (kDenseSrc * CELLS), src_i = (i / CELLS) % kDenseSrc, cell = i % CELLS;
    const AxisTaps &t = sh.ax[a];
    float w = 0.f;
    if (src_i <= t.box_hi - t.box_lo && cell < ncell[a])
      for (int e = cell * t.grid; e < (cell + 1) * t.grid; e++) {
        if (t.lo[e] == src_i) w += t.wlo[e];
        if (t.hi[e] == src_i) w += t.whi[e];
      }
    wd[a][src_i][cell] = w;
  }
  __syncthreads();
}

// acc[k] += Wd row[k] * v for the CELLS cells
template <int CELLS>
__device__ __forceinline__ void dense_axpy(float (&acc)[CELLS], const float *row, float v) {
  static_assert(CELLS % 4 == 0, "rows are read as 16-byte groups");
#pragma unroll
  for (int q = 0; q < CELLS / 4; q++) {
    const float4 w = *reinterpret_cast<const float4 *>(row + 4 * q);
    acc[4 * q] += w.x * v; acc[4 * q + 1] += w.y * v; acc[4 * q + 2] += w.z * v; acc[4 * q + 3] += w.w * v;
  }
}

// Forward pass of one (roi, channel block) on the matrix cores, fp16 tensors, <= 8 cells per axis,
// box rows times padded box columns <= kMfmaYx.  The contraction over (y, x) is one GEMM per group
// of four box slices,
//     T[(slice, channel)][(ph, pw)] = sum_(y, x) box[(slice, channel)][(y, x)] * (Wy[y][ph] Wx[x][pw]),
// K = y * NXP + x with the box row padded to NXP = a multiple of four columns (zero weights on the
// pad).  The weight products sit in LDS as 16-byte K pieces; the box does not: a lane's 8-element K
// piece of the left operand is two 4-voxel pieces of a box row, which it reads straight from the
// feature map with two 2-byte-aligned 8-byte buffer loads (per-lane offset = (slice, channel) of its
// row plus the pieces of the K step, the tile's channels in the scalar offset; slices or channels
// outside the box or the block read zeros through the range check, columns beyond the box row are
// masked).  Rows are ordered (slice % 4, channel), so the 16 x 16 accumulator hands every lane one
// slice of the tile's four channels at one (ph, pw): for two slice groups that is exactly the
// 8-element K piece of a second matrix product with rows (ph, pw), K = (slice, channel) and a
// block-diagonal right-hand side
//     out[(ph, pw)][(channel', pd)] = sum_(z, channel) T[(ph, pw)][(z, channel)] * (channel == channel') Wz[z][pd],
// whose pieces (two non-zero elements) every lane forms from the z matrix by itself (as an fp16 pair
// high + low, so the z weights keep 22 bits).  The contraction over z thereby runs on the matrix
// cores too, without moving T (it is rounded to fp16 once); a lane ends up with four neighbouring
// cells of one (channel, pd).
// A wavefront owns tiles of four channels and shares nothing but the weights with the others: no
// barrier after the set-up.
constexpr int kMfmaYx = 224;
template <typename T>
__device__ inline void pool_forward_mfma(const T *__restrict__ src_any, T *__restrict__ dst, const RoiProblem &p,
                                         const PoolShared &sh, const float (&wd)[3][kDenseSrc][8],
                                         unsigned char *lds, int c_count, long range_bytes, bool blocked, int Wb) {
  using M = Mfma<T>;
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  constexpr int ES = static_cast<int>(sizeof(T));
  auto uni = [](int v) { return __builtin_amdgcn_readfirstlane(v); };   // values read from LDS are the same in every lane
  const int nx = uni(sh.ax[0].box_hi - sh.ax[0].box_lo + 1), ny = uni(sh.ax[1].box_hi - sh.ax[1].box_lo + 1),
            nz = uni(sh.ax[2].box_hi - sh.ax[2].box_lo + 1);
  const int x_lo = uni(sh.ax[0].box_lo), y_lo = uni(sh.ax[1].box_lo), z_lo = uni(sh.ax[2].box_lo);
  // 8-byte pieces of one box row: four voxels from the row's first column on, or (blocked copy of the
  // features) the aligned units of four columns that the row touches, the box starting x_shift
  // columns into the first
  const int xb_lo = x_lo >> 2, x_shift = blocked ? x_lo - 4 * xb_lo : 0;
  const int QX = blocked ? ((x_lo + nx - 1) >> 2) - xb_lo + 1 : (nx + 3) / 4, NXP = 4 * QX, pieces = ny * QX;
  const int KP = (ny * NXP + 31) / 32 * 32, WS = KP + 8;             // weight rows: KP products + a pad against bank conflicts
  const int ohw = p.oh * p.ow, cells = p.od * ohw;
  const long plane = static_cast<long>(p.D) * p.H * p.W;
  const int hw = p.H * p.W;
  T *w = reinterpret_cast<T *>(lds);            // [64 cells (ph, pw)][WS]
  const int zgroups = (nz + 3) / 4;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);   // (a scalar for the compiler too)
  const float inv_ow = 1.f / p.ow, inv_qx = 1.f / QX;
  const int col = lane % 16, quad = lane / 16;
  const unsigned long long sp = reinterpret_cast<unsigned long long>(src_any);
  const T *src = reinterpret_cast<const T *>(static_cast<unsigned long long>(static_cast<unsigned>(uni(static_cast<int>(sp)))) |
                                             static_cast<unsigned long long>(static_cast<unsigned>(uni(static_cast<int>(sp >> 32)))) << 32);
  const __amdgpu_buffer_rsrc_t fr = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(src), 0, static_cast<int>(range_bytes), 0x00020000);
  const int plane_bytes = static_cast<int>(plane) * ES;
  constexpr unsigned kNowhere = 0x80000000u;
  // The row of the left operand this lane LOADS: channel col % 4 of the tile, slice col / 4 of the
  // group, so that four neighbouring lanes read the four channels of one place (32 contiguous bytes
  // of the blocked copy: one request instead of four).  The accumulator rows come out as (slice,
  // channel), the order of the second product's K index.
  // (blocked copy: [slice][row][unit of four columns][channel][4], a unit of one channel is 8 bytes)
  const unsigned unit_row = static_cast<unsigned>(Wb) * p.C * 8u;   // bytes of one row of units
  const unsigned row_off =
      blocked ? static_cast<unsigned>((static_cast<long>(z_lo + col / 4) * p.H + y_lo) * unit_row) +
                    static_cast<unsigned>(xb_lo) * p.C * 8u + static_cast<unsigned>(col % 4) * 8u
              : static_cast<unsigned>(((static_cast<long>(z_lo + col / 4) * p.H + y_lo) * p.W + x_lo) * ES) +
                    static_cast<unsigned>(col % 4) * static_cast<unsigned>(plane_bytes);
  const int tile_bytes = blocked ? 4 * 8 : 4 * plane_bytes;                       // from one tile of four channels to the next
  const int group_bytes = blocked ? 4 * p.H * static_cast<int>(unit_row) : 4 * hw * ES;   // from one group of four slices to the next
  // the two pieces of the lane's K positions in step ks: byte offset inside the slice and the masks
  // that clear the columns beyond the box row
  struct Piece { unsigned off, keep_lo, keep_hi; };
  auto piece = [&](int m) {
    const int y = fdiv(m, inv_qx), x0 = (m - y * QX) * 4, left = nx - x0;
    Piece e;
    if (blocked) {   // whole units; the columns outside the box meet zero weights
      e.off = m < pieces ? static_cast<unsigned>(y) * unit_row + static_cast<unsigned>(m - y * QX) * p.C * 8u : kNowhere;
      e.keep_lo = e.keep_hi = 0xffffffffu;
      return e;
    }
    e.off = m < pieces ? static_cast<unsigned>((y * p.W + x0) * ES) : kNowhere;
    e.keep_lo = left >= 2 ? 0xffffffffu : 0x0000ffffu;
    e.keep_hi = left >= 4 ? 0xffffffffu : (left == 3 ? 0x0000ffffu : 0u);
    return e;
  };
  // Right-hand side of the z product for the stage that starts with slice group zg.  The accumulator
  // of the first product hands lane group `quad` the rows (slice quad, channels 0..3) of each of the
  // two slice groups: packed, that is the K piece {(slice 4 zg + quad, channel i), i = 0..3;
  // (slice 4 zg + 4 + quad, channel i)} of the second product.  Column n = 16 h + col of its
  // right-hand side is (channel' = n / 8, pd = n % 8), block-diagonal in the channel: of the lane's
  // eight elements only i = channel' and i = channel' + 4 are non-zero, Wz[slice][pd] each.  As fp16
  // pairs: dword h, half col / 8 for the first slice group, dword 2 + h for the second; the two
  // weights are kept as a high and a low fp16 part.
  struct ZPair { unsigned a_hi, b_hi, a_lo, b_lo; };
  auto z_pair = [&](int zg) {
    const int pd = col % 8, za_i = zg * 4 + quad, zb_i = za_i + 4;
    const bool up = col / 8 != 0;
    const float za = za_i < nz ? wd[2][za_i < kDenseSrc ? za_i : 0][pd] : 0.f;
    const float zb = zb_i < nz ? wd[2][zb_i < kDenseSrc ? zb_i : 0][pd] : 0.f;
    ZPair z;
    z.a_hi = M::pack2(up ? 0.f : za, up ? za : 0.f);
    z.b_hi = M::pack2(up ? 0.f : zb, up ? zb : 0.f);
    const float ra = za - (up ? M::hi(z.a_hi) : M::lo(z.a_hi)), rb = zb - (up ? M::hi(z.b_hi) : M::lo(z.b_hi));
    z.a_lo = M::pack2(up ? 0.f : ra, up ? ra : 0.f);
    z.b_lo = M::pack2(up ? 0.f : rb, up ? rb : 0.f);
    return z;
  };
  const ZPair z0 = z_pair(0);
  // The steps (tile, slice-group pair, K step of 32) of this wavefront form one sequence; the loads
  // of a step are issued one step ahead, so they are in flight during the previous step's products
  // and stores.
  const int tiles = (c_count + 3) / 4;
  struct Step { int tile, zg, k0; };
  struct Loaded { u32x2 va[2], vb[2]; };
  auto next_of = [&](Step st) {
    st.k0 += 32;
    if (st.k0 >= KP) {
      st.k0 = 0; st.zg += 2;
      if (st.zg >= zgroups) { st.zg = 0; st.tile += st.tile % 2 == 0 ? 1 : 2 * (kPoolThreads / kWave) - 1; }
    }
    return st;
  };
  const Piece pa0 = piece(quad * 2), pb0 = piece(quad * 2 + 1);   // the pieces of the first K step
  auto issue = [&](const Step &st, Loaded &ld) {
    // rows whose slice lies outside the box read zeros
    // (a step beyond the last tile loads nothing: the number of loads per step stays fixed, so the
    // wait before a step's products can leave the loads of the next step in flight)
    const bool any = st.tile < tiles;
    const unsigned row0 = any && st.zg * 4 + col / 4 < nz ? row_off : kNowhere;
    const unsigned row1 = any && st.zg * 4 + 4 + col / 4 < nz ? row_off : kNowhere;
    const int soff = any ? st.tile * tile_bytes + st.zg * group_bytes : 0;
    Piece pa = pa0, pb = pb0;   // (most boxes have one K step)
    if (st.k0 != 0) { pa = piece(st.k0 / 4 + quad * 2); pb = piece(st.k0 / 4 + quad * 2 + 1); }
#pragma unroll
    for (int zs = 0; zs < 2; zs++) {
      const unsigned row = zs == 0 ? row0 : row1;
      // (an offset with the top bit set is beyond the range, whatever the other term adds)
      const unsigned at_a = (row + pa.off) | ((row | pa.off) & kNowhere);
      if (QX % 2 == 0 && !blocked) {   // both pieces lie in one box row: one 16-byte load
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(fr, at_a, soff + zs * group_bytes, 0);
        ld.va[zs] = u32x2{v.x, v.y};
        ld.vb[zs] = u32x2{v.z, v.w};
      } else {
        ld.va[zs] = __builtin_amdgcn_raw_buffer_load_b64(fr, at_a, soff + zs * group_bytes, 0);
        ld.vb[zs] = __builtin_amdgcn_raw_buffer_load_b64(fr, (row + pb.off) | ((row | pb.off) & kNowhere), soff + zs * group_bytes, 0);
      }
    }
  };
  // kAhead sets of load registers used in turn: while a step's products run, the loads of the next
  // kAhead - 1 steps are in flight (a wavefront spends most of a tile waiting for memory otherwise).
  constexpr int kAhead = 3;
  Step q[kAhead];
  Loaded ld[kAhead];
  q[0] = Step{2 * wave, 0, 0};   // tiles 2 w, 2 w + 1, then 2 (w + 4), ...: neighbours in memory back to back
#pragma unroll
  for (int u = 0; u < kAhead; u++) {
    if (u > 0) q[u] = next_of(q[u - 1]);
    issue(q[u], ld[u]);
  }
  // (the first loads are under way while the weight products are formed)
  {  // weight products: thread = (cell, every fourth piece of four neighbouring K); the iterations
     // are independent, so their LDS reads overlap
    const int n = tid / 4, q = tid % 4, ph = fdiv(n, inv_ow), pw = n - ph * p.ow;
    const bool nv = n < ohw;
    uint2 *wr = reinterpret_cast<uint2 *>(w + n * WS);
    for (int m0 = q; m0 < KP / 4; m0 += 8) {   // (KP / 4 is a multiple of eight)
#pragma unroll
      for (int u = 0; u < 2; u++) {
        const int m = m0 + 4 * u;
        const int y = fdiv(m, inv_qx), x0 = (m - y * QX) * 4 - x_shift;   // first column of the piece in the box
        const float wy = (nv && y < ny) ? wd[1][y < ny ? y : 0][ph & 7] : 0.f;
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const bool in = x0 + j >= 0 && x0 + j < nx;
          v[j] = in ? wy * wd[0][in ? x0 + j : 0][pw] : 0.f;
        }
        wr[m] = uint2{M::pack2(v[0], v[1]), M::pack2(v[2], v[3])};
      }
    }
  }
  __syncthreads();
  float4_t oacc[4][2];   // [cell tile][half of the (channel', pd) columns]: cells 4 * quad .. + 3 of the tile
  float4_t acc[2][4];    // [slice group][cell tile]
  // A finished tile (4 channels x cells outputs, contiguous in memory) is laid out in a piece of LDS
  // of this wavefront as it lies in memory, and goes out during the next step as aligned 8-byte
  // pieces, 512 contiguous bytes per instruction: a lane's own results are runs of eight cells at
  // 2-byte-aligned addresses, and such a 16-byte store is two cache accesses per lane.
  const int stage_bytes = (4 * cells * ES + 64 + 15) & ~15;   // (+ room behind the last row, see below)
  const int w_bytes = (64 * WS * ES + 15) & ~15;
  const bool staged = ohw >= 32 && w_bytes + (kPoolThreads / kWave) * stage_bytes <= kPoolLdsBytes &&
                      c_count % 4 == 0 && reinterpret_cast<unsigned long long>(dst) % 8 == 0;
  unsigned char *const stage = lds + w_bytes + wave * stage_bytes;
  int kept_tile = -1;    // the tile waiting in the stage
  T *const lane_dst = dst + (col / 8) * cells + (col % 8) * ohw;   // the lane's (channel, pd) in tile 0
  auto products = [&](const Step &cur, const Loaded &ld) {
    if (cur.k0 == 0) {
#pragma unroll
      for (int i = 0; i < 8; i++) acc[i / 4][i % 4] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    if (cur.k0 == 0 && cur.zg == 0) {
#pragma unroll
      for (int i = 0; i < 8; i++) oacc[i / 2][i % 2] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    {
      Piece pa = pa0, pb = pb0;   // (for the masks)
      if (cur.k0 != 0) { pa = piece(cur.k0 / 4 + quad * 2); pb = piece(cur.k0 / 4 + quad * 2 + 1); }
      u32x4 b[4];
#pragma unroll
      for (int nt = 0; nt < 4; nt++)
        b[nt] = *reinterpret_cast<const u32x4 *>(w + ((nt / 2) * 32 + (col / 4) * 8 + (nt % 2) * 4 + col % 4) * WS + cur.k0 + quad * 8);
#pragma unroll
      for (int zs = 0; zs < 2; zs++) {
        if (cur.zg + zs < zgroups) {
          const u32x4 a = u32x4{ld.va[zs].x & pa.keep_lo, ld.va[zs].y & pa.keep_hi,
                                ld.vb[zs].x & pb.keep_lo, ld.vb[zs].y & pb.keep_hi};
#pragma unroll
          for (int nt = 0; nt < 4; nt++) acc[zs][nt] = M::run16(a, b[nt], acc[zs][nt]);
        }
      }
    }
    if (cur.k0 + 32 >= KP) {
      // contraction over the (up to eight) slices of the two groups
      ZPair z = z0;
      if (cur.zg > 0) z = z_pair(cur.zg);
      const u32x4 zh[2] = {u32x4{z.a_hi, 0u, z.b_hi, 0u}, u32x4{0u, z.a_hi, 0u, z.b_hi}};
      const u32x4 zl[2] = {u32x4{z.a_lo, 0u, z.b_lo, 0u}, u32x4{0u, z.a_lo, 0u, z.b_lo}};
#pragma unroll
      for (int nt = 0; nt < 4; nt++) {
        const u32x4 ta = u32x4{M::pack2(acc[0][nt][0], acc[0][nt][1]), M::pack2(acc[0][nt][2], acc[0][nt][3]),
                               M::pack2(acc[1][nt][0], acc[1][nt][1]), M::pack2(acc[1][nt][2], acc[1][nt][3])};
#pragma unroll
        for (int h = 0; h < 2; h++) {
          oacc[nt][h] = M::run16(ta, zl[h], oacc[nt][h]);
          oacc[nt][h] = M::run16(ta, zh[h], oacc[nt][h]);
        }
      }
      if (cur.zg + 2 >= zgroups) {
        // register r of oacc[nt][h]: cell (nt / 2) * 32 + 8 * quad + (nt % 2) * 4 + r (the order in which
        // the weight rows were read) of (channel 4 tile + 2 h + col / 8, pd col % 8): a lane holds
        // two runs of eight neighbouring cells.
        const int pd = col % 8;
#pragma unroll
        for (int h = 0; h < 2; h++) {
          u32x4 run[2];
#pragma unroll
          for (int half = 0; half < 2; half++)
            run[half] = u32x4{M::pack2(oacc[2 * half][h][0], oacc[2 * half][h][1]),
                              M::pack2(oacc[2 * half][h][2], oacc[2 * half][h][3]),
                              M::pack2(oacc[2 * half + 1][h][0], oacc[2 * half + 1][h][1]),
                              M::pack2(oacc[2 * half + 1][h][2], oacc[2 * half + 1][h][3])};
          if (staged) {
            // Cells at and beyond oh * ow of a run land on the first cells of the NEXT row (at most
            // 32 of them, as oh * ow >= 32; behind the last row: the spare room): the runs of the
            // second half are written first, and the first halves of all rows overwrite what spilt.
            if (pd < p.od) {
              // A run of eight cells starts at a 2-byte-aligned place.  Where that is a multiple of
              // 4 bytes the lane writes dwords 0..2 and the two halves of dword 3, elsewhere cell 0,
              // the three dwords of cells 1..6 and cell 7: three 4-byte and two 2-byte writes either way
              // (2-byte LDS writes take several times as long as 4-byte ones).
              const int first = (2 * h + col / 8) * cells + pd * ohw + 8 * quad;   // in cells
              const bool odd = first & 1;
              unsigned short *row = reinterpret_cast<unsigned short *>(stage) + first;
#pragma unroll
              for (int half = 1; half >= 0; half--) {
                const u32x4 v = run[half];
                unsigned short *at = row + half * 32;
                unsigned *mid = reinterpret_cast<unsigned *>(at + (odd ? 1 : 0));
                mid[0] = odd ? __builtin_amdgcn_alignbit(v.y, v.x, 16) : v.x;
                mid[1] = odd ? __builtin_amdgcn_alignbit(v.z, v.y, 16) : v.y;
                mid[2] = odd ? __builtin_amdgcn_alignbit(v.w, v.z, 16) : v.z;
                at[odd ? 0 : 6] = static_cast<unsigned short>(odd ? v.x : v.w);
                at[7] = static_cast<unsigned short>(v.w >> 16);
                // (the order matters across lanes, which the compiler does not see: it may not move
                // or merge writes of the two halves past each other)
                asm volatile("" ::: "memory");
              }
            }
          } else {
            const int c = cur.tile * 4 + 2 * h + col / 8;
            if (c < c_count && pd < p.od) {
              T *o = lane_dst + (cur.tile * 4 + 2 * h) * cells;   // (the same step for every lane)
#pragma unroll
              for (int half = 0; half < 2; half++) {
                const int n = half * 32 + 8 * quad;
                const u32x4 v = run[half];
                struct __attribute__((packed, aligned(2))) Cells8 { unsigned v[4]; };
                struct __attribute__((packed, aligned(2))) Cells4 { unsigned v[2]; };
                struct __attribute__((packed, aligned(2))) Cells2 { unsigned v; };
                const int left = ohw - n;   // cells of this run that exist
                if (left >= 8) {            // eight neighbouring cells as one 16-byte store (2-byte aligned)
                  *reinterpret_cast<Cells8 *>(o + n) = Cells8{{v.x, v.y, v.z, v.w}};
                } else if (left > 0) {      // 4 + 2 + 1 cells
                  const bool l4 = left & 4, l2 = left & 2;
                  if (l4) *reinterpret_cast<Cells4 *>(o + n) = Cells4{{v.x, v.y}};
                  if (l2) *reinterpret_cast<Cells2 *>(o + n + (left & 4)) = Cells2{l4 ? v.z : v.x};
                  if (left & 1)
                    reinterpret_cast<unsigned short *>(o)[n + (left & 6)] =
                        static_cast<unsigned short>(l4 ? (l2 ? v.w : v.z) : (l2 ? v.y : v.x));
                }
              }
            }
          }
        }
        if (staged) kept_tile = cur.tile;
      }
    }
  };
  // The stores of a staged tile wait until the loads of the following step have arrived: a wait for
  // loads also waits for every store issued before it, and a store takes as long as a load.
  // (Stores to nowhere in the steps that have none, which would let the waits count exactly the
  // operations issued after a set of loads, cost more than the waits they shorten: 371 against
  // 343 µs for 4000 rois of 256 channels.)
  auto store_kept = [&]() {
    if (kept_tile < 0) return;
    const int bytes = 4 * cells * ES;
    unsigned char *to = reinterpret_cast<unsigned char *>(dst) + static_cast<long>(kept_tile) * bytes;
    for (int at = lane * 8; at < bytes; at += kWave * 8)
      // (written once and not read here again: nontemporal, so that the output, larger than the
      // last-level cache, does not push the features out of it)
      __builtin_nontemporal_store(*reinterpret_cast<const unsigned long long *>(stage + at),
                                  reinterpret_cast<unsigned long long *>(to + at));
    kept_tile = -1;
  };
  // a use of the loaded registers that the compiler cannot move: the wait for them lands here
  auto arrived = [&](Loaded &ld) {
    asm volatile("" : "+v"(ld.va[0]), "+v"(ld.va[1]), "+v"(ld.vb[0]), "+v"(ld.vb[1]) : : "memory");
  };
  while (q[0].tile < tiles) {   // (q[0] is the oldest step here)
#pragma unroll
    for (int u = 0; u < kAhead; u++) {
      arrived(ld[u]);
      if (q[u].tile < tiles) {
        store_kept();
        products(q[u], ld[u]);
      }
      q[u] = next_of(q[(u + kAhead - 1) % kAhead]);
      issue(q[u], ld[u]);
    }
  }
  store_kept();
}

template <typename T, typename RT, int CELLS>
__global__ __launch_bounds__(kPoolThreads) void roi_pool_forward_kernel(
    const T *__restrict__ feat, const RT *__restrict__ rois, T *__restrict__ out, const RoiProblem p,
    const int channels_per_block, const T *__restrict__ blocked, const int Wb, const unsigned *__restrict__ order) {
  __shared__ PoolShared sh;
  __shared__ __attribute__((aligned(16))) unsigned char lds[kPoolLdsBytes];
  const unsigned n = order ? order[blockIdx.x] : blockIdx.x;   // (largest rois first, see pool_order_rois)
  const int c_begin = blockIdx.y * channels_per_block, c_end = min(c_begin + channels_per_block, p.C);
  __shared__ __attribute__((aligned(16))) float wd[3][kDenseSrc][CELLS];
  PoolPlan plan = pool_setup<RT, CELLS>(sh, rois + static_cast<long>(n) * roi_columns(p.ndim, 0), p, sizeof(T),
                                        CELLS == 8 ? wd : nullptr, true, true);
  const int cells = p.od * p.oh * p.ow;
  const long plane = static_cast<long>(p.D) * p.H * p.W;
  T *dst = out + (static_cast<long>(n) * p.C + c_begin) * cells;
  const int total = (c_end - c_begin) * cells;
  if (plan.staged < 0) {
    for (int i = threadIdx.x; i < total; i += kPoolThreads) dst[i] = store_cast<T>(0.f);
    return;
  }
  const T *src = feat + (static_cast<long>(sh.g.batch) * p.C + c_begin) * plane;
  if (plan.staged == 1 && plan.chunk < 1) {
    // A box too large for LDS with all its planes is worked through in slabs of planes: x and y are
    // contracted per slab, and the z contraction adds each slab's share to sums kept per output.
    const AxisTaps &tx = sh.ax[0], &ty = sh.ax[1], &tz = sh.ax[2];
    const int nx = tx.box_hi - tx.box_lo + 1, ny = ty.box_hi - ty.box_lo + 1, nz = tz.box_hi - tz.box_lo + 1;
    const int gx = tx.grid, gy = ty.grid, gz = tz.grid, ohw = p.oh * p.ow;
    const long box_plane = (static_cast<long>(ny) * nx * sizeof(T) + 15) / 16 * 16;
    const long per_plane = box_plane + (static_cast<long>(ny) * p.ow + ohw) * 4;
    int cs = 0, zs = 0;
    // (measured on 24^3 - 32^3 boxes: the per-output gather below costs about as much as the slabs with
    // 27 samples per output, a third with 8, twice with 64)
    // (one channel per slab, so that a slab holds as many planes as LDS takes: with 8 channels and a plane or two
    // per slab the passes were 20 - 30 % slower — 200 rois of 24 - 32 voxels x 256 channels, grid 4: 7.0 -> 5.0 ms)
    for (int c = gx * gy * gz > 27 ? 1 : 0; c >= 1 && cs == 0; c >>= 1) {
      const int cn = min(c, c_end - c_begin);
      const long planes = (kPoolLdsBytes - 32 - cn * static_cast<long>(cells) * 4) / (cn * per_plane);
      if (planes >= 1) { cs = cn; zs = static_cast<int>(min(planes, static_cast<long>(nz))); }
    }
    if (cs == 0) {
      plan.staged = 0;   // not even one plane: per-output gather below
    } else {
      float *sums = reinterpret_cast<float *>(lds);                                   // [cs][cells]
      T *box = reinterpret_cast<T *>(sums + cs * cells);                              // [cs][zs][ny][nx]
      float *t1 = reinterpret_cast<float *>(lds + ((static_cast<size_t>(cs) * cells * 4 + static_cast<size_t>(cs) * zs * box_plane + 15) / 16) * 16);  // [cs][zs][ny][ow]
      float *t2 = t1 + cs * zs * ny * p.ow;                                           // [cs][zs][oh][ow]
      for (int cb = c_begin; cb < c_end; cb += cs) {
        const int cn = min(cs, c_end - cb);
        for (int i = threadIdx.x; i < cn * cells; i += kPoolThreads) sums[i] = 0.f;
        for (int z0 = 0; z0 < nz; z0 += zs) {
          const int nzs = min(zs, nz - z0), rows = nzs * ny, vol_s = rows * nx;
          __syncthreads();   // the slab before has been read
          const T *corner = src + static_cast<long>(cb - c_begin) * plane +
                            (static_cast<long>(tz.box_lo + z0) * p.H + ty.box_lo) * p.W + tx.box_lo;
          for (int i = threadIdx.x; i < cn * vol_s; i += kPoolThreads) {
            const int c = i / vol_s, r0 = i - c * vol_s, row = r0 / nx, x = r0 - row * nx, z = row / ny, y = row - z * ny;
            box[i] = corner[c * plane + (static_cast<long>(z) * p.H + y) * p.W + x];
          }
          __syncthreads();
          for (int i = threadIdx.x; i < cn * rows * p.ow; i += kPoolThreads) {        // contract x
            const int row = i / p.ow, pw = i - row * p.ow;                             // row = (c, z, y)
            const T *r = box + row * nx;
            float acc = 0.f;
            for (int k = 0; k < gx; k++) {
              const int e = pw * gx + k;
              acc += tx.wlo[e] * load(r + tx.lo[e]) + tx.whi[e] * load(r + tx.hi[e]);
            }
            t1[i] = acc;
          }
          __syncthreads();
          for (int i = threadIdx.x; i < cn * nzs * ohw; i += kPoolThreads) {          // contract y
            const int cz = i / ohw, hw = i - cz * ohw, ph = hw / p.ow, pw = hw - ph * p.ow;   // cz = (c, z)
            const float *r = t1 + cz * ny * p.ow + pw;
            float acc = 0.f;
            for (int k = 0; k < gy; k++) {
              const int e = ph * gy + k;
              acc += ty.wlo[e] * r[ty.lo[e] * p.ow] + ty.whi[e] * r[ty.hi[e] * p.ow];
            }
            t2[i] = acc;
          }
          __syncthreads();
          for (int i = threadIdx.x; i < cn * cells; i += kPoolThreads) {              // the slab's share of z
            const int c = i / cells, r0 = i - c * cells, pd = r0 / ohw, hw = r0 - pd * ohw;
            const float *r = t2 + c * nzs * ohw + hw;
            float acc = 0.f;
            for (int k = 0; k < gz; k++) {
              const int e = pd * gz + k;
              const unsigned zl = static_cast<unsigned>(tz.lo[e] - z0), zh = static_cast<unsigned>(tz.hi[e] - z0);
              if (zl < static_cast<unsigned>(nzs)) acc += tz.wlo[e] * r[zl * ohw];
              if (zh < static_cast<unsigned>(nzs)) acc += tz.whi[e] * r[zh * ohw];
            }
            sums[i] += acc;   // (element i belongs to this thread in every slab)
          }
        }
        T *o = dst + static_cast<long>(cb - c_begin) * cells;
        for (int i = threadIdx.x; i < cn * cells; i += kPoolThreads) o[i] = store_cast<T>(sums[i]);
      }
      return;
    }
  }
  if (plan.staged == 0) {  // per-output gather
    const int gz = p.ndim == 3 ? sh.g.grid[2] : 1, gy = sh.g.grid[1], gx = sh.g.grid[0];
    for (int i = threadIdx.x; i < total; i += kPoolThreads) {
      const int pw = i % p.ow, ph = (i / p.ow) % p.oh, pd = (i / (p.ow * p.oh)) % p.od, c = i / cells;
      float acc = 0.f;
      for (int iz = 0; iz < gz; iz++) {
        const double z = p.ndim == 3 ? local_coord(sh.g, 2, pd, iz) : 0.0;
        for (int iy = 0; iy < gy; iy++) {
          const double y = local_coord(sh.g, 1, ph, iy);
          for (int ix = 0; ix < gx; ix++)
            acc += sample_clamped<T>(src + c * plane, p.D, p.H, p.W, z, y, local_coord(sh.g, 0, pw, ix), p.order);
        }
      }
      dst[i] = store_cast<T>(acc / static_cast<float>(sh.g.count));
    }
    return;
  }
  const AxisTaps &tx = sh.ax[0], &ty = sh.ax[1], &tz = sh.ax[2];
  const int nx = tx.box_hi - tx.box_lo + 1, ny = ty.box_hi - ty.box_lo + 1, nz = tz.box_hi - tz.box_lo + 1;
  const int vol = nx * ny * nz;
  const int gx = tx.grid, gy = ty.grid, gz = tz.grid;
  const int ohw = p.oh * p.ow;
  const float inv_vol = 1.f / vol, inv_nxy = 1.f / (nx * ny), inv_nx = 1.f / nx, inv_ow = 1.f / p.ow,
              inv_ohw = 1.f / ohw, inv_cells = 1.f / cells;
  // (with 9..16 cells per axis a row of the matrix is mostly zeros: the tap-register form below is
  // faster for the forward pass; the backward pass still gains from the dense form)
  const bool dense = CELLS == 8 && dense_applies<CELLS>(sh, p);   // (the set-up has built the matrices)
  // (fp16 only: weight products rounded to bf16's 8 bits would cost the output half its tolerance)
  if constexpr (CELLS == 8 && std::is_same<T, __half>::value) {
    // The staging addresses a block's channels with 32-bit byte offsets and reads box rows as 8-byte
    // pieces that may reach up to three voxels past the row: the buffer range ends with the tensor
    // (or 64 channels after the block), and a box whose last piece would cross that end takes the
    // plain path below.
    const int nxp = (nx + 3) & ~3;
    const long es = sizeof(T), near = (c_end - c_begin + 64) * plane * es;
    const long left = (static_cast<long>(p.N - sh.g.batch) * p.C - c_begin) * plane * es;
    const long last = ((c_end - c_begin - 1) * plane + (static_cast<long>(tz.box_hi) * p.H + ty.box_hi) * p.W + tx.box_lo + nxp) * es;
    const int kp = (ny * nxp + 31) / 32 * 32;
    const bool room = 64 * (kp + 8) * es <= kPoolLdsBytes;   // the weight products
    if (blocked != nullptr && dense) {   // from the blocked copy (the host has checked its size)
      const int units = ((tx.box_hi >> 2) - (tx.box_lo >> 2) + 1) * 4;
      const long image = static_cast<long>(p.D) * p.H * Wb * p.C * 4;   // elements of one image of the copy
      if (ny * units <= kMfmaYx && 64 * ((ny * units + 31) / 32 * 32 + 8) * es <= kPoolLdsBytes) {
        pool_forward_mfma<T>(blocked + sh.g.batch * image + c_begin * 4, dst, p, sh, wd, lds, c_end - c_begin,
                             (image - c_begin * 4) * es, true, Wb);
        return;
      }
    }
    if (dense && ny * nxp <= kMfmaYx && room && near < (1L << 31) && last <= left) {
      pool_forward_mfma<T>(src, dst, p, sh, wd, lds, c_end - c_begin, min(near, left), false, 0);
      return;
    }
  }
  for (int cb = c_begin; cb < c_end; cb += plan.chunk) {
    const int cs = min(plan.chunk, c_end - cb);
    T *box = reinterpret_cast<T *>(lds);                                            // [cs][nz][ny][nx]
    float *t1 = reinterpret_cast<float *>(lds + ((static_cast<size_t>(cs) * vol * sizeof(T) + 15) / 16) * 16);  // [cs][nz][ny][ow]
    float *t2 = t1 + cs * nz * ny * p.ow;                                           // [cs][nz][oh][ow]
    const T *corner = src + static_cast<long>(cb - c_begin) * plane +
                      (static_cast<long>(tz.box_lo) * p.H + ty.box_lo) * p.W + tx.box_lo;
    // copy the sub-box: eight independent loads in flight per lane before the first LDS store
    for (int i0 = threadIdx.x; i0 < cs * vol; i0 += kPoolThreads * 8) {
      T val[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int i = i0 + u * kPoolThreads;
        if (i < cs * vol) {
          const int c = fdiv(i, inv_vol), r0 = i - c * vol, z = fdiv(r0, inv_nxy), r1 = r0 - z * nx * ny;
          const int y = fdiv(r1, inv_nx), x = r1 - y * nx;
          val[u] = corner[c * plane + (static_cast<long>(z) * p.H + y) * p.W + x];
        }
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int i = i0 + u * kPoolThreads;
        if (i < cs * vol) box[i] = val[u];
      }
    }
    __syncthreads();
    // Each pass gives a thread a FIXED output coordinate on the contracted axis, so its (at most
    // kTapRegs) tap entries stay in registers while it walks over the rows; per element that leaves
    // 2 * grid LDS reads, 2 * grid FMAs and one store.
    if (dense) {
      // x: thread = one (c, z, y) row of the box, all its cells at once
      for (int r = threadIdx.x; r < cs * nz * ny; r += kPoolThreads) {
        float a[CELLS] = {};
        const T *row = box + r * nx;
        for (int x = 0; x < nx; x++) dense_axpy(a, wd[0][x], load(row + x));
#pragma unroll
        for (int k = 0; k < CELLS; k++)
          if (k < p.ow) t1[r * p.ow + k] = a[k];
      }
      __syncthreads();
      // y: thread = (c, z, pw)
      for (int i = threadIdx.x; i < cs * nz * p.ow; i += kPoolThreads) {
        const int cz = fdiv(i, inv_ow), pw = i - cz * p.ow;
        float a[CELLS] = {};
        const float *col = t1 + cz * ny * p.ow + pw;
        for (int yy = 0; yy < ny; yy++) dense_axpy(a, wd[1][yy], col[yy * p.ow]);
#pragma unroll
        for (int k = 0; k < CELLS; k++)
          if (k < p.oh) t2[cz * ohw + k * p.ow + pw] = a[k];
      }
      __syncthreads();
      // z, store: thread = (c, ph, pw)
      T *o = dst + static_cast<long>(cb - c_begin) * cells;
      for (int i = threadIdx.x; i < cs * ohw; i += kPoolThreads) {
        const int c = fdiv(i, inv_ohw), hw = i - c * ohw;
        float a[CELLS] = {};
        const float *col = t2 + c * nz * ohw + hw;
        for (int zz = 0; zz < nz; zz++) dense_axpy(a, wd[2][zz], col[zz * ohw]);
#pragma unroll
        for (int k = 0; k < CELLS; k++)
          if (k < p.od) o[c * cells + k * ohw + hw] = store_cast<T>(a[k]);
      }
    } else if (gx <= kTapRegs && gy <= kTapRegs && gz <= kTapRegs) {
      {  // contract x: thread = (row chunk, pw); rows are (c, z, y)
        int lanes = 1;
        while (lanes < p.ow) lanes *= 2;
        const int pw = threadIdx.x % lanes, r0 = threadIdx.x / lanes, step = kPoolThreads / lanes;
        const int rows = cs * nz * ny;
        if (pw < p.ow) {
          TapRegs t;
          t.load(tx, pw);
          for (int r = r0; r < rows; r += step) t1[r * p.ow + pw] = t.apply(box + r * nx, 1);
        }
      }
      __syncthreads();
      {  // contract y: thread = (row chunk, ph, pw); rows are (c, z)
        int lanes = 1;
        while (lanes < ohw) lanes *= 2;
        const int cell = threadIdx.x % lanes, r0 = threadIdx.x / lanes, step = kPoolThreads / lanes;
        const int rows = cs * nz;
        if (cell < ohw) {
          const int ph = fdiv(cell, inv_ow), pw = cell - ph * p.ow;
          TapRegs t;
          t.load(ty, ph);
          for (int r = r0; r < rows; r += step) t2[r * ohw + cell] = t.apply(t1 + r * ny * p.ow + pw, p.ow);
        }
      }
      __syncthreads();
      {  // contract z, store: a wavefront takes (pd, half of the channels) items, its lanes run over
         // (ph, pw): the taps of pd stay in registers over the channels and the stores are coalesced
        T *o = dst + static_cast<long>(cb - c_begin) * cells;
        const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
        const int half = (cs + 1) / 2;
        for (int item = wave; item < 2 * p.od; item += kPoolThreads / kWave) {
          const int pd = item >> 1, c_lo = (item & 1) * half, c_hi = min(cs, c_lo + half);
          TapRegs t;
          t.load(tz, pd);
          for (int c = c_lo; c < c_hi; c++)
            for (int hw = lane; hw < ohw; hw += kWave)
              o[c * cells + pd * ohw + hw] = store_cast<T>(t.apply(t2 + c * nz * ohw + hw, ohw));
        }
      }
    } else {
      for (int i = threadIdx.x; i < cs * nz * ny * p.ow; i += kPoolThreads) {  // contract x
        const int row = fdiv(i, inv_ow), pw = i - row * p.ow;                 // row = (c, z, y)
        const T *r = box + row * nx;
        float acc = 0.f;
        for (int s = 0; s < gx; s++) {
          const int e = pw * gx + s;
          acc += tx.wlo[e] * load(r + tx.lo[e]) + tx.whi[e] * load(r + tx.hi[e]);
        }
        t1[i] = acc;
      }
      __syncthreads();
      for (int i = threadIdx.x; i < cs * nz * p.oh * p.ow; i += kPoolThreads) {  // contract y
        const int cz = fdiv(i, inv_ohw), hw = i - cz * ohw, ph = fdiv(hw, inv_ow), pw = hw - ph * p.ow;  // cz = (c, z)
        const float *r = t1 + cz * ny * p.ow + pw;
        float acc = 0.f;
        for (int s = 0; s < gy; s++) {
          const int e = ph * gy + s;
          acc += ty.wlo[e] * r[ty.lo[e] * p.ow] + ty.whi[e] * r[ty.hi[e] * p.ow];
        }
        t2[i] = acc;
      }
      __syncthreads();
      T *o = dst + static_cast<long>(cb - c_begin) * cells;
      for (int i = threadIdx.x; i < cs * cells; i += kPoolThreads) {  // contract z, store
        const int c = fdiv(i, inv_cells), r0 = i - c * cells, pd = fdiv(r0, inv_ohw), hw = r0 - pd * ohw;
        const float *r = t2 + c * nz * ohw + hw;
        float acc = 0.f;
        for (int s = 0; s < gz; s++) {
          const int e = pd * gz + s;
          acc += tz.wlo[e] * r[tz.lo[e] * ohw] + tz.whi[e] * r[tz.hi[e] * ohw];
        }
        o[i] = store_cast<T>(acc);
      }
    }
    __syncthreads();
  }
}

// Backward pass of one (roi, channel block) on the matrix cores: fp16 gradients, <= 8 cells per
// axis, channels-last fp32 accumulation buffer.  Per 16 channels and box slice z,
//     dBox[(y, x)][channel] = sum_(ph, pw) (Wy[y][ph] Wx[x][pw]) * U_z[(ph, pw)][channel],
//     U_z[(ph, pw)][channel] = sum_pd Wz[z][pd] * gout[channel][pd][(ph, pw)],
// with the weight products in LDS (rows (y, x) as in the forward pass: box rows padded to a multiple of
// four columns) and U_z formed by every lane in registers straight from its 16-byte loads of the
// gradient, already in the layout of the right-hand operand (column = channel, K = cell).  The
// accumulator then holds, per lane, four neighbouring voxels of one box row for one channel: lanes
// 0..15 are 16 neighbouring channels of the channels-last buffer, so an atomic instruction adds runs
// of 64 contiguous bytes.  Wavefronts work on different channel blocks and share nothing but the
// weights: no barrier after the set-up.
constexpr int kPoolBwdRow = 72;   // fp16 elements per row of the transposed weights: 64 cells + pad
template <typename T>
__device__ inline void pool_backward_mfma(const T *__restrict__ src_any, float *__restrict__ dst_any, const RoiProblem &p,
                                          const PoolShared &sh, const float (&wd)[3][kDenseSrc][8],
                                          unsigned char *lds, int c_count) {
  using M = Mfma<T>;
  auto uni = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
  const int nx = uni(sh.ax[0].box_hi - sh.ax[0].box_lo + 1), ny = uni(sh.ax[1].box_hi - sh.ax[1].box_lo + 1),
            nz = uni(sh.ax[2].box_hi - sh.ax[2].box_lo + 1);
  const int x_lo = uni(sh.ax[0].box_lo), y_lo = uni(sh.ax[1].box_lo), z_lo = uni(sh.ax[2].box_lo);
  const int NXP = (nx + 3) & ~3, QX = NXP / 4, KT = (ny * NXP + 15) / 16;
  const int ohw = p.oh * p.ow, cells = p.od * ohw;
  const int KS = ohw > 32 ? 2 : 1;                    // K steps of 32 cells
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);   // (a scalar for the compiler too)
  const int col = lane % 16, quad = lane / 16;
  T *wt = reinterpret_cast<T *>(lds);                 // [KT * 16 rows (y, x)][kPoolBwdRow]
  {  // weight products: thread = (row of the pass, quarter of the cells)
    const float inv_ow = 1.f / p.ow, inv_nxp = 1.f / NXP;
    const int q = tid % 4;
    float wxy[2][16];   // not kept: the cells' (ph, pw) are the same for every row
    int phs[16], pws[16];
#pragma unroll
    for (int j = 0; j < 16; j++) {
      const int n = q * 16 + j;
      phs[j] = fdiv(n, inv_ow);
      pws[j] = n - phs[j] * p.ow;
      if (n >= ohw) { phs[j] = -1; pws[j] = 0; }
    }
    (void)wxy;
    for (int k = tid / 4; k < KT * 16; k += kPoolThreads / 4) {
      const int y = fdiv(k, inv_nxp), x = k - y * NXP;
      const bool kv = y < ny && x < nx;
      const float *wy = wd[1][kv ? y : 0], *wx = wd[0][kv ? x : 0];
      unsigned packed[8];
#pragma unroll
      for (int j = 0; j < 16; j += 2) {
        const float a = (kv && phs[j] >= 0) ? wy[phs[j]] * wx[pws[j]] : 0.f;
        const float b = (kv && phs[j + 1] >= 0) ? wy[phs[j + 1]] * wx[pws[j + 1]] : 0.f;
        packed[j / 2] = M::pack2(a, b);
      }
      u32x4 *row = reinterpret_cast<u32x4 *>(wt + k * kPoolBwdRow + q * 16);
      row[0] = u32x4{packed[0], packed[1], packed[2], packed[3]};
      row[1] = u32x4{packed[4], packed[5], packed[6], packed[7]};
    }
  }
  __syncthreads();
  auto uni_ptr = [&](const void *ptr) {
    const unsigned long long v = reinterpret_cast<unsigned long long>(ptr);
    return static_cast<unsigned long long>(static_cast<unsigned>(uni(static_cast<int>(v)))) |
           static_cast<unsigned long long>(static_cast<unsigned>(uni(static_cast<int>(v >> 32)))) << 32;
  };
  const T *src = reinterpret_cast<const T *>(uni_ptr(src_any));
  float *dst = reinterpret_cast<float *>(uni_ptr(dst_any));
  // this roi's gradient rows of the block; reads beyond the block's channels return zeros
  const __amdgpu_buffer_rsrc_t gr = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(src), 0, c_count * cells * 2 + 16, 0x00020000);
  const int blocks = (c_count + 15) / 16;
  for (int blk = wave; blk < blocks; blk += kPoolThreads / kWave) {
    const int c = blk * 16 + col;
    const bool cv = c < c_count;
    // the lane's gradient pieces: cells quad * 8 .. + 7 (+ 32) of every pd of its channel
    u32x4 g[8][2];
    const unsigned g0 = cv ? static_cast<unsigned>(c * cells + quad * 8) * 2u : 0x80000000u;
    // a piece that reaches past its plane of cells brings the next plane's, channel's or roi's values:
    // their weights are zero, but 0 x inf is not, so they are cleared
    u32x4 keep[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
      const int c0 = ks * 32 + quad * 8;
      auto two = [&](int j) { return (c0 + j < ohw ? 0xffffu : 0u) | (c0 + j + 1 < ohw ? 0xffff0000u : 0u); };
      keep[ks] = u32x4{two(0), two(2), two(4), two(6)};
    }
#pragma unroll
    for (int pd = 0; pd < 8; pd++)
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {
        g[pd][ks] = u32x4{0u, 0u, 0u, 0u};
        if (pd < p.od && ks * 32 + quad * 8 < ohw)
          g[pd][ks] = __builtin_amdgcn_raw_buffer_load_b128(gr, g0, (pd * ohw + ks * 32) * 2, 0);
      }
    // (all loads first, then the masks: a mask right behind its load would wait for it there)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int pd = 0; pd < 8; pd++)
#pragma unroll
      for (int ks = 0; ks < 2; ks++) g[pd][ks] &= keep[ks];
    for (int z = 0; z < nz; z++) {
      float wz[8];
      {
        const float4 lo4 = *reinterpret_cast<const float4 *>(&wd[2][z][0]), hi4 = *reinterpret_cast<const float4 *>(&wd[2][z][4]);
        wz[0] = lo4.x; wz[1] = lo4.y; wz[2] = lo4.z; wz[3] = lo4.w; wz[4] = hi4.x; wz[5] = hi4.y; wz[6] = hi4.z; wz[7] = hi4.w;
      }
      u32x4 bop[2];
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {
        float u[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (ks < KS) {
#pragma unroll
          for (int pd = 0; pd < 8; pd++)
            if (pd < p.od) M::fma_piece(u, wz[pd], g[pd][ks]);
        }
        bop[ks] = M::pack(u);
      }
      const unsigned slice = static_cast<unsigned>((z_lo + z) * p.H + y_lo) * p.W + x_lo;   // voxel index of the slice's box corner
      for (int kt = 0; kt < KT; kt++) {
        float4_t acc = float4_t{0.f, 0.f, 0.f, 0.f};
        const T *arow = wt + (kt * 16 + col) * kPoolBwdRow + quad * 8;
        acc = M::run16(*reinterpret_cast<const u32x4 *>(arow), bop[0], acc);
        if (KS == 2) acc = M::run16(*reinterpret_cast<const u32x4 *>(arow + 32), bop[1], acc);
        // rows 4 * quad .. + 3 of the tile = piece m of the padded box rows: four neighbouring x
        const int m = kt * 4 + quad, y = m / QX, x0 = (m - y * QX) * 4;
        if (cv && y < ny) {
          float *at = dst + (static_cast<size_t>(slice + static_cast<unsigned>(y * p.W + x0)) * p.C + c);
#pragma unroll
          for (int r = 0; r < 4; r++)
            if (x0 + r < nx && acc[r] != 0.f) atomic_add(at + static_cast<size_t>(r) * p.C, acc[r]);
        }
      }
    }
  }
}

// G = element type of the accumulation buffer (T for fp32, float for 16-bit T).
// CL: the accumulation buffer is channels-last [N, D*H*W, C] (the fp32 workspace of the 16-bit
// path): the lanes of a wavefront then add neighbouring channels of a voxel, contiguous bytes,
// instead of one element in each of many rows (a scattered atomic moves a whole memory sector).
template <typename T, typename G, typename RT, bool CL, int CELLS>
__global__ __launch_bounds__(kPoolThreads) void roi_pool_backward_kernel(
    const T *__restrict__ gout, const RT *__restrict__ rois, G *__restrict__ gin, const RoiProblem p,
    const int channels_per_block) {
  __shared__ PoolShared sh;
  __shared__ __attribute__((aligned(16))) unsigned char lds[kPoolLdsBytes];
  const unsigned n = blockIdx.x;
  const int c_begin = blockIdx.y * channels_per_block, c_end = min(c_begin + channels_per_block, p.C);
  // intermediates are fp32 here, so size the chunk with 4-byte box elements
  __shared__ __attribute__((aligned(16))) float wd[3][kDenseSrc][CELLS];
  PoolPlan plan = pool_setup<RT, CELLS>(sh, rois + static_cast<long>(n) * roi_columns(p.ndim, 0), p, sizeof(float), wd, true);
  if (plan.staged < 0) return;
  const int cells = p.od * p.oh * p.ow;
  const long plane = static_cast<long>(p.D) * p.H * p.W;
  const T *src = gout + (static_cast<long>(n) * p.C + c_begin) * cells;
  G *dst = gin + (static_cast<long>(sh.g.batch) * p.C + c_begin) * plane;
  G *dst_cl = gin + static_cast<long>(sh.g.batch) * plane * p.C + c_begin;   // CL: voxel v, channel c at v * C + c
  // The transposed contractions below look entries up by source index through `first`, which
  // holds kPoolFirst + 4 indices: a box wider than that on any axis (few cells spread over many
  // voxels) takes the per-output scatter, like a box that does not fit LDS.
  bool wide = false;
  if (plan.staged == 1)
    for (int a = 0; a < 3; a++) wide = wide || sh.ax[a].box_hi - sh.ax[a].box_lo + 1 > kPoolFirst + 2;
  const bool dense = plan.staged == 1 && dense_applies<CELLS>(sh, p);
  // Channels per pass and box planes per pass.  A box too large for a pass of enough channels (an atomic
  // request should carry a sector's worth of them, a planar row of gradients a few) is worked through
  // in slabs of planes: the transposed contractions of different planes do not depend on each other.
  int zs = 0;
  if (plan.staged == 1 && !wide) {
    const long bx = sh.ax[0].box_hi - sh.ax[0].box_lo + 1, by = sh.ax[1].box_hi - sh.ax[1].box_lo + 1;
    zs = sh.ax[2].box_hi - sh.ax[2].box_lo + 1;
    const bool box = !CL && dense;                         // planar sums from the dense matrices: the slab of the box itself is staged
    const long per_plane = (box ? by * bx * 4 : 0L) + (by * p.ow + static_cast<long>(p.oh) * p.ow) * 4;
    const int want = min(CL ? 16 : 4, c_end - c_begin);
    // (the set-up has counted a staged box: planar sums through the tap tables keep none, so that a plane of
    // an image that is larger than LDS still takes this path and not one atomic per tap of every sample)
    if (!CL && !dense) plan.chunk = static_cast<int>(min(kPoolLdsBytes / (zs * per_plane + 16), 64L));
    if (plan.chunk < want) {
      zs = static_cast<int>(min(max((kPoolLdsBytes / want - 16) / per_plane, 1L), static_cast<long>(zs)));
      plan.chunk = static_cast<int>(min(kPoolLdsBytes / (zs * per_plane + 16), 64L));
      if (plan.chunk < 1) plan.staged = 0;
    }
  }
  if (plan.staged == 0 || wide) {  // per-output scatter
    const int total = (c_end - c_begin) * cells;
    const int gz = p.ndim == 3 ? sh.g.grid[2] : 1, gy = sh.g.grid[1], gx = sh.g.grid[0];
    for (int i = threadIdx.x; i < total; i += kPoolThreads) {
      const int pw = i % p.ow, ph = (i / p.ow) % p.oh, pd = (i / (p.ow * p.oh)) % p.od, c = i / cells;
      const float top = load(src + i) / static_cast<float>(sh.g.count);
      for (int iz = 0; iz < gz; iz++) {
        const double z = p.ndim == 3 ? local_coord(sh.g, 2, pd, iz) : 0.0;
        for (int iy = 0; iy < gy; iy++) {
          const double y = local_coord(sh.g, 1, ph, iy);
          for (int ix = 0; ix < gx; ix++) {
            Corners<float> cw;
            if (!clamped_corners<float>(p.D, p.H, p.W, z, y, local_coord(sh.g, 0, pw, ix), p.order, cw)) continue;
#pragma unroll
            for (int k = 0; k < 8; k++)
              if (cw.w[k] != 0.f)
                atomic_add(CL ? dst_cl + cw.idx[k] * p.C + c : dst + c * plane + cw.idx[k], static_cast<G>(top * cw.w[k]));
          }
        }
      }
    }
    return;
  }
  const AxisTaps &tx = sh.ax[0], &ty = sh.ax[1], &tz = sh.ax[2];
  const int nx = tx.box_hi - tx.box_lo + 1, ny = ty.box_hi - ty.box_lo + 1, nz = tz.box_hi - tz.box_lo + 1;
  const int ohw = p.oh * p.ow;
  const int gx = tx.grid, gy = ty.grid, gz = tz.grid;
  const float inv_nxy = 1.f / (nx * ny), inv_nx = 1.f / nx, inv_ow = 1.f / p.ow,
              inv_ohw = 1.f / ohw, inv_nyow = 1.f / (ny * p.ow),
              inv_gx = 1.f / gx, inv_gy = 1.f / gy, inv_gz = 1.f / gz;
  if (dense) {   // (the set-up has built the matrices)
    if constexpr (CL && CELLS == 8 && std::is_same<T, __half>::value && std::is_same<G, float>::value) {
      // matrix-core form: 32-bit offsets into the image's accumulation buffer and into this roi's
      // gradient; its 16-byte loads may reach 14 bytes past a row of cells (what they bring from there
      // is masked out), so blocks whose rows end within 16 bytes of the tensor's end stay with the form below
      const int nxp = (nx + 3) & ~3, kt = (ny * nxp + 15) / 16;
      const bool fits = ny * nxp <= kMfmaYx && kt * 16 * kPoolBwdRow * 2 <= kPoolLdsBytes;
      const bool small = plane * p.C * 4 < (1L << 32) && static_cast<long>(c_end - c_begin) * cells * 2 + 64 < (1L << 31);
      // (16 bytes of gradient must follow the block's rows: with few cells per roi that rules out more
      // than the tensor's last block)
      const long behind = (static_cast<long>(p.R) * p.C - (static_cast<long>(n) * p.C + c_end)) * cells * 2;
      if (fits && small && behind >= 16) {
        pool_backward_mfma(src, dst_cl, p, sh, wd, lds, c_end - c_begin);
        return;
      }
    }
    const float inv_ow = 1.f / p.ow;
    for (int cb = c_begin; cb < c_end; cb += plan.chunk) {
      const int cs = min(plan.chunk, c_end - cb);
      for (int z0 = 0; z0 < nz; z0 += zs) {   // slabs of box planes
      const int nzs = min(zs, nz - z0);
      const int vol_s = nx * ny * nzs;
      const float inv_vol_s = 1.f / vol_s;
      float *t2 = reinterpret_cast<float *>(lds);      // [cs][nzs][oh][ow]
      float *t1 = t2 + cs * nzs * ohw;                  // [cs][nzs][ny][ow]; CL: [nzs][ny][cs][ow]
      float *gbox = t1 + cs * nzs * ny * p.ow;          // [cs][nzs][ny][nx] (planar accumulation only)
      const T *go = src + static_cast<long>(cb - c_begin) * cells;
      const float inv_cs = 1.f / cs;
      // z: thread = (c, ph, pw); its grad_output values stay in registers
      for (int i = threadIdx.x; i < cs * ohw; i += kPoolThreads) {
        const int c = fdiv(i, inv_ohw), hw = i - c * ohw;
        float g[CELLS];
#pragma unroll
        for (int k = 0; k < CELLS; k++) g[k] = k < p.od ? load(go + c * cells + k * ohw + hw) : 0.f;
        for (int z = 0; z < nzs; z++) {
          float acc = 0.f;
#pragma unroll
          for (int k = 0; k < CELLS; k++) acc += wd[2][z0 + z][k] * g[k];
          t2[(c * nzs + z) * ohw + hw] = acc;
        }
      }
      __syncthreads();
      // y: thread = (c, z, pw)
      for (int i = threadIdx.x; i < cs * nzs * p.ow; i += kPoolThreads) {
        const int cz = fdiv(i, inv_ow), pw = i - cz * p.ow;
        const int c = fdiv(cz, 1.f / nzs), z = cz - c * nzs;
        float g[CELLS];
#pragma unroll
        for (int k = 0; k < CELLS; k++) g[k] = k < p.oh ? t2[cz * ohw + k * p.ow + pw] : 0.f;
        for (int y = 0; y < ny; y++) {
          float acc = 0.f;
#pragma unroll
          for (int k = 0; k < CELLS; k++) acc += wd[1][y][k] * g[k];
          t1[(CL ? ((z * ny + y) * cs + c) : (cz * ny + y)) * p.ow + pw] = acc;
        }
      }
      __syncthreads();
      // x: thread = one (c, z, y) line
      const long first = (static_cast<long>(tz.box_lo + z0) * p.H + ty.box_lo) * p.W + tx.box_lo;
      if (CL) {   // channel fastest across the lanes: a wavefront adds runs of cs contiguous floats
        for (int i = threadIdx.x; i < cs * nzs * ny; i += kPoolThreads) {
          const int zy = fdiv(i, inv_cs), c = i - zy * cs, z = fdiv(zy, 1.f / ny), y = zy - z * ny;
          float g[CELLS];
#pragma unroll
          for (int k = 0; k < CELLS; k++) g[k] = k < p.ow ? t1[i * p.ow + k] : 0.f;
          G *row = dst_cl + (first + (static_cast<long>(z) * p.H + y) * p.W) * p.C + (cb - c_begin) + c;
          for (int x = 0; x < nx; x++) {
            float acc = 0.f;
#pragma unroll
            for (int k = 0; k < CELLS; k++) acc += wd[0][x][k] * g[k];
            if (acc != 0.f) atomic_add(row + static_cast<long>(x) * p.C, static_cast<G>(acc));
          }
        }
      } else {    // through LDS, so that the lanes of a wavefront add runs of nx contiguous elements
        for (int i = threadIdx.x; i < cs * nzs * ny; i += kPoolThreads) {
          float g[CELLS];
#pragma unroll
          for (int k = 0; k < CELLS; k++) g[k] = k < p.ow ? t1[i * p.ow + k] : 0.f;
          for (int x = 0; x < nx; x++) {
            float acc = 0.f;
#pragma unroll
            for (int k = 0; k < CELLS; k++) acc += wd[0][x][k] * g[k];
            gbox[i * nx + x] = acc;
          }
        }
        __syncthreads();
        G *corner = dst + static_cast<long>(cb - c_begin) * plane + first;
        for (int i = threadIdx.x; i < cs * vol_s; i += kPoolThreads) {
          const float v = gbox[i];
          if (v == 0.f) continue;
          const int c = fdiv(i, inv_vol_s), r0 = i - c * vol_s, z = fdiv(r0, inv_nxy), r1 = r0 - z * nx * ny;
          const int y = fdiv(r1, inv_nx), x = r1 - y * nx;
          atomic_add(corner + c * plane + (static_cast<long>(z) * p.H + y) * p.W + x, static_cast<G>(v));
        }
      }
      __syncthreads();
    }
    }
    return;
  }
  pool_first(sh);
  for (int cb = c_begin; cb < c_end; cb += plan.chunk) {
    const int cs = min(plan.chunk, c_end - cb);
    for (int z0 = 0; z0 < nz; z0 += zs) {   // slabs of box planes
    const int nzs = min(zs, nz - z0);
    const int vol_s = nx * ny * nzs;
    const float inv_vol_s = 1.f / vol_s, inv_nzsohw = 1.f / (nzs * ohw);
    float *t1 = reinterpret_cast<float *>(lds);       // [cs][nzs][ny][ow]
    float *t2 = t1 + cs * nzs * ny * p.ow;            // [cs][nzs][oh][ow]
    const T *go = src + static_cast<long>(cb - c_begin) * cells;
    // Transposed contractions as gathers.  Entries are sorted by coordinate, so the entries whose
    // low tap is source index i form the range [first[i], first[i+1]) and those whose high tap is
    // i are the low-tap entries of i - 1 (a clamped edge entry has lo == hi and zero high weight).
    for (int i = threadIdx.x; i < cs * nzs * ohw; i += kPoolThreads) {  // transpose of "contract z"
      const int c = fdiv(i, inv_nzsohw), r0 = i - c * nzs * ohw, z = fdiv(r0, inv_ohw), hw = r0 - z * ohw;
      const T *r = go + c * cells + hw;
      const int zq = z0 + z;   // plane of the box
      const int mid = tz.first[zq], e0 = zq > 0 ? tz.first[zq - 1] : mid, e1 = tz.first[zq + 1];
      float acc = 0.f;
      for (int e = e0; e < e1; e++) {
        const float w = e < mid ? (tz.hi[e] == zq ? tz.whi[e] : 0.f) : tz.wlo[e];
        acc += w * load(r + fdiv(e, inv_gz) * ohw);
      }
      t2[i] = acc;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < cs * nzs * ny * p.ow; i += kPoolThreads) {  // transpose of "contract y"
      const int cz = fdiv(i, inv_nyow), r0 = i - cz * ny * p.ow, y = fdiv(r0, inv_ow), pw = r0 - y * p.ow;
      const float *r = t2 + cz * ohw + pw;
      const int mid = ty.first[y], e0 = y > 0 ? ty.first[y - 1] : mid, e1 = ty.first[y + 1];
      float acc = 0.f;
      for (int e = e0; e < e1; e++) {
        const float w = e < mid ? (ty.hi[e] == y ? ty.whi[e] : 0.f) : ty.wlo[e];
        acc += w * r[fdiv(e, inv_gy) * p.ow];
      }
      t1[i] = acc;
    }
    __syncthreads();
    const long first = (static_cast<long>(tz.box_lo + z0) * p.H + ty.box_lo) * p.W + tx.box_lo;
    if (CL) {
      // transpose of "contract x" straight into the buffer: a thread takes one (z, y) row of one channel,
      // channels fastest across the lanes, so that a wavefront's atomics are runs of cs contiguous floats
      const float inv_cs = 1.f / cs;
      for (int i = threadIdx.x; i < cs * nzs * ny; i += kPoolThreads) {
        const int zy = fdiv(i, inv_cs), c = i - zy * cs;
        const int z = fdiv(zy, 1.f / ny), y = zy - z * ny;
        const float *r = t1 + (c * nzs * ny + zy) * p.ow;
        G *row = dst_cl + (first + (static_cast<long>(z) * p.H + y) * p.W) * p.C + (cb - c_begin) + c;
        for (int x = 0; x < nx; x++) {
          const int mid = tx.first[x], e0 = x > 0 ? tx.first[x - 1] : mid, e1 = tx.first[x + 1];
          float acc = 0.f;
          for (int e = e0; e < e1; e++) {
            const float w = e < mid ? (tx.hi[e] == x ? tx.whi[e] : 0.f) : tx.wlo[e];
            acc += w * r[fdiv(e, inv_gx)];
          }
          if (acc != 0.f) atomic_add(row + static_cast<long>(x) * p.C, static_cast<G>(acc));
        }
      }
    } else {
      G *corner = dst + static_cast<long>(cb - c_begin) * plane + first;
      for (int i = threadIdx.x; i < cs * vol_s; i += kPoolThreads) {  // transpose of "contract x"
        const int row = fdiv(i, inv_nx), x = i - row * nx;
        const float *r = t1 + row * p.ow;
        const int mid = tx.first[x], e0 = x > 0 ? tx.first[x - 1] : mid, e1 = tx.first[x + 1];
        float acc = 0.f;
        for (int e = e0; e < e1; e++) {
          const float w = e < mid ? (tx.hi[e] == x ? tx.whi[e] : 0.f) : tx.wlo[e];
          acc += w * r[fdiv(e, inv_gx)];
        }
        // (a lane per voxel of a row: the lanes of a wavefront add runs of contiguous elements as they are)
        if (acc == 0.f) continue;
        const int c = fdiv(i, inv_vol_s), r0 = i - c * vol_s, z = fdiv(r0, inv_nxy), y = fdiv(r0 - z * nx * ny, inv_nx);
        atomic_add(corner + c * plane + (static_cast<long>(z) * p.H + y) * p.W + x, static_cast<G>(acc));
      }
    }
    __syncthreads();
    }
  }
}

// Launch order of the rois for the forward pass: descending estimated cost (box volume), so that the
// few rois that take ten times longer than the rest start first instead of finishing alone after
// the others.  One workgroup, a counting sort over 64 logarithmic buckets; the order inside a bucket
// is whatever the atomics give (it changes the schedule, not the results).
constexpr int kOrderBuckets = 64, kOrderMaxRois = 1 << 17;
__device__ inline void pool_order_rois(const float *__restrict__ rois, unsigned *__restrict__ order, int R, int ndim,
                                       float scale) {
  __shared__ unsigned count[kOrderBuckets], start[kOrderBuckets];
  const int cols = 1 + 2 * ndim, step = blockDim.x;
  auto bucket = [&](int i) {
    const float *r = rois + static_cast<long>(i) * cols;
    float vol = 1.f;
    for (int a = 0; a < ndim; a++) vol *= fmaxf((r[1 + ndim + a] - r[1 + a]) * scale, 1.f) + 2.f;
    const int b = static_cast<int>(4.f * log2f(fminf(fmaxf(vol, 1.f), 6.0e4f)));   // 0 .. 63
    return kOrderBuckets - 1 - min(b, kOrderBuckets - 1);                          // large boxes first
  };
  if (threadIdx.x < kOrderBuckets) count[threadIdx.x] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < R; i += step) atomicAdd(&count[bucket(i)], 1u);
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned sum = 0;
    for (int b = 0; b < kOrderBuckets; b++) { start[b] = sum; sum += count[b]; }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < R; i += step) order[atomicAdd(&start[bucket(i)], 1u)] = static_cast<unsigned>(i);
}

// Blocked copy of fp16 / bf16 features for the pooled forward pass: [N][C][D*H][W] ->
// [N][D*H][W / 4][C][4].  A unit of four columns of one channel is 8 bytes, and the units of all
// channels of one place are neighbours: the rows of a roi's box, a few voxels long, then share their
// 64-byte sectors with the other channels of the same workgroup instead of with voxels nobody asked
// for.  A workgroup moves 64 channels x up to 32 units of one row through LDS (reads along the row,
// writes along the channels).  The first workgroup of the launch orders the rois instead (when `order`
// is given): the two jobs do not depend on each other.
constexpr int kBlockUnits = 32;
__global__ __launch_bounds__(256) void pool_block_features_kernel(const uint2 *__restrict__ src, uint2 *__restrict__ dst,
                                                                   int C, long rows, int Wb,
                                                                   const float *__restrict__ rois, unsigned *__restrict__ order,
                                                                   int R, int ndim, float scale) {
  if (order != nullptr && blockIdx.x == 0) {   // (first, so that it is over long before the copy)
    pool_order_rois(rois, order, R, ndim, scale);
    return;
  }
  __shared__ uint2 tile[kBlockUnits * 65];
  const int ux = min(Wb, kBlockUnits), xchunks = (Wb + ux - 1) / ux, cchunks = (C + 63) / 64;
  unsigned id = blockIdx.x - (order != nullptr ? 1u : 0u);
  const int cz = id % cchunks; id /= cchunks;
  const int xc = id % xchunks;
  const long row = id / xchunks;            // n * D * H + (z * H + y)
  const long nimg = row / rows, r = row - nimg * rows;
  const int xb0 = xc * ux, c0 = cz * 64;
  const int t = threadIdx.x;
  const float inv_ux = 1.f / ux;
  for (int i = t; i < 64 * ux; i += 256) {
    const int cl = fdiv(i, inv_ux), xq = i - cl * ux;
    uint2 v = make_uint2(0u, 0u);
    if (c0 + cl < C && xb0 + xq < Wb) {   // (read once: nontemporal, the cache is for the copy)
      const unsigned long long raw = __builtin_nontemporal_load(
          reinterpret_cast<const unsigned long long *>(src + ((nimg * C + c0 + cl) * rows + r) * Wb + xb0 + xq));
      v = make_uint2(static_cast<unsigned>(raw), static_cast<unsigned>(raw >> 32));
    }
    tile[xq * 65 + cl] = v;
  }
  __syncthreads();
  for (int i = t; i < 64 * ux; i += 256) {
    const int xq = i / 64, cl = i % 64;
    if (c0 + cl < C && xb0 + xq < Wb) dst[(row * Wb + xb0 + xq) * C + c0 + cl] = tile[xq * 65 + cl];
  }
}

// The blocked copy pays when the rois read more than the copy costs: about as many pooled outputs as
// input voxels.  fp16 only (the matrix-core forward pass), rows of a multiple of four voxels.
static size_t pool_blocked_bytes(int dtype, const RoiProblem &p) {
  if (dtype != MV_F16 || p.rotated || p.order == 3 || p.W % 4 != 0) return 0;
  if (p.od > 8 || p.oh > 8 || p.ow > 8) return 0;
  const long voxels = static_cast<long>(p.N) * p.D * p.H * p.W, cells = static_cast<long>(p.od) * p.oh * p.ow;
  if (static_cast<long>(p.R) * cells < voxels) return 0;
  const long image = static_cast<long>(p.D) * p.H * p.W * p.C * 2;
  if (image >= (1L << 31)) return 0;   // 32-bit byte offsets inside one image
  return static_cast<size_t>(voxels) * p.C * 2 + (p.R <= kOrderMaxRois ? static_cast<size_t>(p.R) * 4 : 0);
}

static bool pool_applies(int dtype, const RoiProblem &p) {
  if (p.rotated || dtype == MV_F64) return false;
  const long cells = static_cast<long>(p.od) * p.oh * p.ow;
  if (cells > 1024 || p.od > 16 || p.oh > 16 || p.ow > 16) return false;
  if (p.sampling_ratio > 4) return false;
  return p.R <= 0x7fffffff;
}

// Returns -1 when the pooled kernels do not apply.
// Channels per workgroup: 32, doubled while that still leaves a few thousand workgroups (the tap
// tables are built once per workgroup, so with many rois fewer, longer workgroups are cheaper) and
// halved while there are too few workgroups to fill the compute units (few rois, few channels: a
// workgroup walks its channels in LDS-sized chunks one after the other).
// (`enough`: the number of workgroups that must remain when the channels per workgroup double)
static int pool_channels_per_block(const RoiProblem &p, long enough = 6144) {
  int cpb = 32;
  while (cpb < 256 && cpb < p.C && static_cast<long>(p.R) * ((p.C + 2 * cpb - 1) / (2 * cpb)) >= enough) cpb *= 2;
  while (cpb > 1 && static_cast<long>(p.R) * ((p.C + cpb - 1) / cpb) < 1024) cpb /= 2;
  return cpb;
}

template <typename T, int CELLS>
static void launch_pool_forward(const void *input, const float *r, void *output, const RoiProblem &p, int cpb,
                                dim3 grid, hipStream_t s, const void *blocked = nullptr, const unsigned *order = nullptr) {
  hipLaunchKernelGGL((roi_pool_forward_kernel<T, float, CELLS>), grid, dim3(kPoolThreads), 0, s,
                     static_cast<const T *>(input), r, static_cast<T *>(output), p, cpb,
                     static_cast<const T *>(blocked), p.W / 4, order);
}

template <typename T, bool CL, int CELLS>
static void launch_pool_backward(const void *grad_output, const float *r, void *acc, const RoiProblem &p, int cpb,
                                 dim3 grid, hipStream_t s) {
  hipLaunchKernelGGL((roi_pool_backward_kernel<T, float, float, CL, CELLS>), grid, dim3(kPoolThreads), 0, s,
                     static_cast<const T *>(grad_output), r, static_cast<float *>(acc), p, cpb);
}

// dense-matrix width of the kernel instance: 8 cells per axis when the output allows it
static bool pool_small_cells(const RoiProblem &p) { return p.od <= 8 && p.oh <= 8 && p.ow <= 8; }

size_t roi_pool_forward_workspace(int dtype, const RoiProblem &p) {
  return pool_applies(dtype, p) ? pool_blocked_bytes(dtype, p) : 0;
}

// The blocked copy alone, for callers that pool one feature map several times: bytes of the copy of
// these features (0: the forward pass has no use for one; only N, C, D, H, W of `p` are looked at) ...
size_t roi_pool_prepared_bytes(int dtype, const RoiProblem &p) {
  if (dtype != MV_F16 || p.W % 4 != 0) return 0;
  if (static_cast<long>(p.D) * p.H * p.W * p.C * 2 >= (1L << 31)) return 0;   // 32-bit byte offsets inside one image
  const long rows = static_cast<long>(p.D) * p.H;
  const int Wb = p.W / 4, ux = std::min(Wb, kBlockUnits);
  if (p.N * rows * ((Wb + ux - 1) / ux) * ((p.C + 63) / 64) >= (1L << 31)) return 0;
  return static_cast<size_t>(p.N) * p.D * p.H * p.W * p.C * 2;
}

// ... and the copy itself.  -1: no copy for these features.
int roi_pool_prepare(const void *input, int dtype, const RoiProblem &p, void *prepared, size_t capacity, hipStream_t s) {
  const size_t bytes = roi_pool_prepared_bytes(dtype, p);
  if (bytes == 0 || capacity < bytes || reinterpret_cast<uintptr_t>(input) % 8 != 0 ||
      reinterpret_cast<uintptr_t>(prepared) % 8 != 0)
    return -1;
  const long rows = static_cast<long>(p.D) * p.H;
  const int Wb = p.W / 4, ux = std::min(Wb, kBlockUnits);
  const long copy_blocks = p.N * rows * ((Wb + ux - 1) / ux) * ((p.C + 63) / 64);
  hipLaunchKernelGGL(pool_block_features_kernel, dim3(static_cast<unsigned>(copy_blocks)), dim3(256), 0, s,
                     static_cast<const uint2 *>(input), static_cast<uint2 *>(prepared), p.C, rows, Wb,
                     static_cast<const float *>(nullptr), static_cast<unsigned *>(nullptr), 0, p.ndim, 1.f);
  return check_launch("pool_block_features_kernel");
}

// `prepared`: a copy made by roi_pool_prepare from the same features (then only the order of the rois
// is worked out here, into the workspace when it holds four bytes per roi), or null.
int roi_pool_forward(const void *input, const void *rois, void *output, int dtype,
                     const RoiProblem &p, void *workspace, size_t capacity, hipStream_t s, const void *prepared) {
  if (!pool_applies(dtype, p)) return -1;
  const void *blocked = nullptr;
  const unsigned *order = nullptr;
  if (prepared != nullptr) {
    // the kernels that read a copy: fp16, up to 8 cells per axis, orders 0 and 1
    if (roi_pool_prepared_bytes(dtype, p) == 0 || p.order == 3 || p.od > 8 || p.oh > 8 || p.ow > 8 ||
        reinterpret_cast<uintptr_t>(prepared) % 8 != 0)
      return -1;
    blocked = prepared;
    if (workspace != nullptr && p.R <= kOrderMaxRois && capacity >= static_cast<size_t>(p.R) * 4 &&
        reinterpret_cast<uintptr_t>(workspace) % 4 == 0) {
      unsigned *ord = static_cast<unsigned *>(workspace);
      hipLaunchKernelGGL(pool_block_features_kernel, dim3(1), dim3(256), 0, s, static_cast<const uint2 *>(nullptr),
                         static_cast<uint2 *>(nullptr), p.C, static_cast<long>(p.D) * p.H, p.W / 4,
                         static_cast<const float *>(rois), ord, p.R, p.ndim, static_cast<float>(p.scale));
      order = ord;
    }
  } else if (workspace != nullptr && pool_blocked_bytes(dtype, p) > 0 && capacity >= pool_blocked_bytes(dtype, p) &&
      reinterpret_cast<uintptr_t>(input) % 8 == 0 &&
      reinterpret_cast<uintptr_t>(workspace) % 8 == 0) {
    const long rows = static_cast<long>(p.D) * p.H;
    const int Wb = p.W / 4, ux = std::min(Wb, kBlockUnits);
    const long copy_blocks = p.N * rows * ((Wb + ux - 1) / ux) * ((p.C + 63) / 64);
    if (copy_blocks + 1 < (1L << 31)) {
      unsigned *ord = nullptr;   // (behind the copy; its size is a multiple of 8 bytes)
      if (p.R <= kOrderMaxRois)
        ord = reinterpret_cast<unsigned *>(static_cast<char *>(workspace) + static_cast<size_t>(p.N) * rows * p.W * p.C * 2);
      hipLaunchKernelGGL(pool_block_features_kernel, dim3(static_cast<unsigned>(copy_blocks + (ord ? 1 : 0))), dim3(256), 0, s,
                         static_cast<const uint2 *>(input), static_cast<uint2 *>(workspace), p.C, rows, Wb,
                         static_cast<const float *>(rois), ord, p.R, p.ndim,
                         static_cast<float>(p.scale));
      blocked = workspace;
      order = ord;
    }
  }
  // (from the blocked copy, in launch order, a workgroup's set-up weighs more than the balance of the
  // last wave of workgroups: 256 channels per workgroup from 3072 workgroups on, config 5 0.415 -> 0.39 ms)
  const int cpb = pool_channels_per_block(p, blocked != nullptr && order != nullptr ? 3072 : 6144);
  const long cblocks = (p.C + cpb - 1) / cpb;
  if (cblocks > 65535) return -1;
  const dim3 grid(p.R, static_cast<unsigned>(cblocks));
  const float *r = static_cast<const float *>(rois);
  const bool small = pool_small_cells(p);
  switch (dtype) {
    case MV_F32:
      small ? launch_pool_forward<float, 8>(input, r, output, p, cpb, grid, s)
            : launch_pool_forward<float, 16>(input, r, output, p, cpb, grid, s);
      break;
    case MV_F16:
      small ? launch_pool_forward<__half, 8>(input, r, output, p, cpb, grid, s, blocked, order)
            : launch_pool_forward<__half, 16>(input, r, output, p, cpb, grid, s);
      break;
    default:
      small ? launch_pool_forward<__hip_bfloat16, 8>(input, r, output, p, cpb, grid, s)
            : launch_pool_forward<__hip_bfloat16, 16>(input, r, output, p, cpb, grid, s);
  }
  return check_launch("roi_pool_forward_kernel");
}

bool roi_pool_applies(int dtype, const RoiProblem &p) { return pool_applies(dtype, p) && (p.C + 31) / 32 <= 65535; }

// `acc` is the accumulation buffer: grad_input itself for fp32, the fp32 workspace for 16-bit
// (channels-last [N, D*H*W, C] when `channels_last` is set; 16-bit types only).
int roi_pool_backward(const void *grad_output, const void *rois, void *acc, int dtype,
                      const RoiProblem &p, hipStream_t s, bool channels_last) {
  if (!pool_applies(dtype, p)) return -1;
  const int cpb = pool_channels_per_block(p);
  const long cblocks = (p.C + cpb - 1) / cpb;
  if (cblocks > 65535) return -1;
  const dim3 grid(p.R, static_cast<unsigned>(cblocks));
  const float *r = static_cast<const float *>(rois);
  const bool small = pool_small_cells(p);
#define MV_POOL_BACKWARD(TYPE, CLV)                                                          \
  (small ? launch_pool_backward<TYPE, CLV, 8>(grad_output, r, acc, p, cpb, grid, s)          \
         : launch_pool_backward<TYPE, CLV, 16>(grad_output, r, acc, p, cpb, grid, s))
  switch (dtype) {
    case MV_F32:
      if (channels_last) return fail(MV_INVALID_ARGUMENT, "channels-last accumulation is for 16-bit tensors");
      MV_POOL_BACKWARD(float, false);
      break;
    case MV_F16:
      if (channels_last) MV_POOL_BACKWARD(__half, true);
      else MV_POOL_BACKWARD(__half, false);
      break;
    default:
      if (channels_last) MV_POOL_BACKWARD(__hip_bfloat16, true);
      else MV_POOL_BACKWARD(__hip_bfloat16, false);
  }
#undef MV_POOL_BACKWARD
  return check_launch("roi_pool_backward_kernel");
}

}  // namespace mv
