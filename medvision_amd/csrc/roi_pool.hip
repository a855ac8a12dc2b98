// RoIAlign for plain (axis-aligned) boxes with SMALL outputs per roi (detection heads: thousands of
// rois, 7x7x7 cells, hundreds of channels), forward and backward.
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
#include "common.hpp"
#include "roi_geometry.hpp"
#include "sampling.hpp"

namespace mv {

constexpr int kPoolThreads = 256;
constexpr int kPoolEntries = 64;               // tap-table entries per axis (cells * grid)
constexpr int kPoolLdsBytes = 40 * 1024;       // staged data + intermediates of one channel chunk

// i / d for 0 <= i < 2^21 and 0 < d < 2^12, with inv = 1.0f / d (exact: the product is at least
// 0.5 / d away from an integer and its rounding error is below that)
__device__ __forceinline__ int fdiv(int i, float inv) { return static_cast<int>((static_cast<float>(i) + 0.5f) * inv); }

struct AxisTaps {
  int lo[kPoolEntries], hi[kPoolEntries];      // box-relative tap indices
  float wlo[kPoolEntries], whi[kPoolEntries];  // weights (0 for void samples), include 1 / grid
  int first[kPoolEntries + 4];                 // first[i] = first entry whose low tap is >= i (box-relative)
  int box_lo, box_hi;                          // inclusive source range covered by valid taps
  int entries, grid;
};

struct PoolShared {
  RoiGeom g;
  AxisTaps ax[3];  // x, y, z
  int staged;      // 1: LDS path, 0: per-output gather, -1: every output is zero
  int chunk;       // channels per LDS pass
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

// Builds geometry and tap tables for roi `roi`; all threads must call it (contains barriers).
template <typename RT>
__device__ inline void pool_setup(PoolShared &sh, const RT *roi, const RoiProblem &p, size_t elem_bytes) {
  if (threadIdx.x == 0) {
    const double sn[3] = {0, 0, 0}, cs[3] = {1, 1, 1};
    build_geom(sh.g, roi, p, sn, cs);
    const int cells[3] = {p.ow, p.oh, p.od};
    for (int a = 0; a < 3; a++) {
      sh.ax[a].grid = a < p.ndim ? sh.g.grid[a] : 1;
      sh.ax[a].entries = cells[a] * max(sh.ax[a].grid, 0);
      sh.ax[a].box_lo = 1 << 30;
      sh.ax[a].box_hi = -1;
    }
    sh.staged = 1;
    if (sh.g.batch < 0) sh.staged = -1;
    for (int a = 0; a < 3; a++) {
      if (sh.ax[a].entries > kPoolEntries) sh.staged = min(sh.staged, 0);
      if (sh.ax[a].entries <= 0) sh.staged = -1;  // empty sampling grid: outputs are zero
    }
  }
  __syncthreads();
  if (sh.staged <= 0) return;
  const int size[3] = {p.W, p.H, p.D};
  for (int e = threadIdx.x; e < 3 * kPoolEntries; e += kPoolThreads) {
    const int a = e / kPoolEntries, i = e % kPoolEntries;
    AxisTaps &t = sh.ax[a];
    if (i >= t.entries) continue;
    const int cell = i / t.grid, sub = i % t.grid;
    const double v = a < p.ndim ? local_coord(sh.g, a, cell, sub) : 0.0;
    int lo, hi;
    float frac;
    const bool ok = clamped_tap<float>(v, size[a], lo, hi, frac, p.order);
    const float inv = 1.f / static_cast<float>(t.grid);
    // void samples keep weight 0; park them at the matching end so that `lo` stays monotonic
    t.lo[i] = ok ? lo : (v > 0.0 ? -2 : -1);
    t.hi[i] = t.lo[i] < 0 ? t.lo[i] : hi;
    t.wlo[i] = ok ? (1.f - frac) * inv : 0.f;
    t.whi[i] = ok ? frac * inv : 0.f;
    if (ok) {
      atomicMin(&t.box_lo, lo);
      atomicMax(&t.box_hi, hi);
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    long vol = 1;
    for (int a = 0; a < 3; a++) {
      if (sh.ax[a].box_hi < 0) { sh.staged = -1; break; }  // no valid sample on this axis
      vol *= sh.ax[a].box_hi - sh.ax[a].box_lo + 1;
    }
    if (sh.staged == 1) {
      const long nz = sh.ax[2].box_hi - sh.ax[2].box_lo + 1, ny = sh.ax[1].box_hi - sh.ax[1].box_lo + 1;
      const long per_channel = vol * static_cast<long>(elem_bytes) + (nz * ny * p.ow + nz * p.oh * p.ow) * 4 + 16;
      const long chunk = kPoolLdsBytes / per_channel;
      if (chunk < 1) sh.staged = 0;
      sh.chunk = static_cast<int>(min(chunk, 64L));
    }
  }
  __syncthreads();
  if (sh.staged != 1) return;
  for (int e = threadIdx.x; e < 3 * kPoolEntries; e += kPoolThreads) {  // make indices box-relative
    const int a = e / kPoolEntries, i = e % kPoolEntries;
    AxisTaps &t = sh.ax[a];
    if (i >= t.entries) continue;
    const int top = t.box_hi - t.box_lo;
    t.lo[i] = t.lo[i] == -1 ? 0 : (t.lo[i] == -2 ? top : t.lo[i] - t.box_lo);
    t.hi[i] = t.hi[i] == -1 ? 0 : (t.hi[i] == -2 ? top : t.hi[i] - t.box_lo);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < 3 * (kPoolEntries + 4); e += kPoolThreads) {  // entry ranges per source index
    const int a = e / (kPoolEntries + 4), i = e % (kPoolEntries + 4);
    AxisTaps &t = sh.ax[a];
    if (i > t.box_hi - t.box_lo + 1) continue;
    int f = 0;
    while (f < t.entries && t.lo[f] < i) f++;
    t.first[i] = f;
  }
  __syncthreads();
}

// Dense form of the tap tables for the usual small boxes (<= CELLS cells per axis, box of
// <= kDenseSrc voxels per axis): per axis a matrix Wd[source index][cell] = sum of the weights of
// the cell's samples that touch the source index.  A contraction then is "walk the line, multiply
// each value into all cells" (forward) or "load the cells of a line, one dot product per source
// index" (backward): no per-entry branches, the matrix rows are LDS broadcasts.
// The kernels are instantiated for CELLS = 8 (7^3 detection heads) and 16 (14 x 14 mask heads).
constexpr int kDenseSrc = 32;

template <int CELLS>
__device__ __forceinline__ bool dense_applies(const PoolShared &sh, const RoiProblem &p) {
  for (int a = 0; a < 3; a++)
    if (sh.ax[a].box_hi - sh.ax[a].box_lo + 1 > kDenseSrc) return false;
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

template <typename T, typename RT, int CELLS>
__global__ __launch_bounds__(kPoolThreads) void roi_pool_forward_kernel(
    const T *__restrict__ feat, const RT *__restrict__ rois, T *__restrict__ out, const RoiProblem p,
    const int channels_per_block) {
  __shared__ PoolShared sh;
  __shared__ __attribute__((aligned(16))) unsigned char lds[kPoolLdsBytes];
  const unsigned n = blockIdx.x;
  const int c_begin = blockIdx.y * channels_per_block, c_end = min(c_begin + channels_per_block, p.C);
  pool_setup(sh, rois + static_cast<long>(n) * roi_columns(p.ndim, 0), p, sizeof(T));
  const int cells = p.od * p.oh * p.ow;
  const long plane = static_cast<long>(p.D) * p.H * p.W;
  T *dst = out + (static_cast<long>(n) * p.C + c_begin) * cells;
  const int total = (c_end - c_begin) * cells;
  if (sh.staged < 0) {
    for (int i = threadIdx.x; i < total; i += kPoolThreads) dst[i] = store_cast<T>(0.f);
    return;
  }
  const T *src = feat + (static_cast<long>(sh.g.batch) * p.C + c_begin) * plane;
  if (sh.staged == 0) {  // per-output gather
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
  __shared__ __attribute__((aligned(16))) float wd[3][kDenseSrc][CELLS];
  // (with 9..16 cells per axis a row of the matrix is mostly zeros: the tap-register form below is
  // faster for the forward pass; the backward pass still gains from the dense form)
  const bool dense = CELLS == 8 && dense_applies<CELLS>(sh, p);
  if (dense) dense_build<CELLS>(sh, p, wd);
  for (int cb = c_begin; cb < c_end; cb += sh.chunk) {
    const int cs = min(sh.chunk, c_end - cb);
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
  pool_setup(sh, rois + static_cast<long>(n) * roi_columns(p.ndim, 0), p, sizeof(float));
  if (sh.staged < 0) return;
  const int cells = p.od * p.oh * p.ow;
  const long plane = static_cast<long>(p.D) * p.H * p.W;
  const T *src = gout + (static_cast<long>(n) * p.C + c_begin) * cells;
  G *dst = gin + (static_cast<long>(sh.g.batch) * p.C + c_begin) * plane;
  G *dst_cl = gin + static_cast<long>(sh.g.batch) * plane * p.C + c_begin;   // CL: voxel v, channel c at v * C + c
  // The transposed contractions below look entries up by source index through `first`, which
  // holds kPoolEntries + 4 indices: a box wider than that on any axis (few cells spread over many
  // voxels) takes the per-output scatter, like a box that does not fit LDS.
  bool wide = false;
  if (sh.staged == 1)
    for (int a = 0; a < 3; a++) wide = wide || sh.ax[a].box_hi - sh.ax[a].box_lo + 1 > kPoolEntries + 2;
  if (sh.staged == 0 || wide) {  // per-output scatter
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
  const int vol = nx * ny * nz;
  const int ohw = p.oh * p.ow;
  const int gx = tx.grid, gy = ty.grid, gz = tz.grid;
  const float inv_vol = 1.f / vol, inv_nxy = 1.f / (nx * ny), inv_nx = 1.f / nx, inv_ow = 1.f / p.ow,
              inv_ohw = 1.f / ohw, inv_nzohw = 1.f / (nz * ohw), inv_nyow = 1.f / (ny * p.ow),
              inv_gx = 1.f / gx, inv_gy = 1.f / gy, inv_gz = 1.f / gz;
  __shared__ __attribute__((aligned(16))) float wd[3][kDenseSrc][CELLS];
  if (dense_applies<CELLS>(sh, p)) {
    dense_build<CELLS>(sh, p, wd);
    const float inv_ow = 1.f / p.ow;
    for (int cb = c_begin; cb < c_end; cb += sh.chunk) {
      const int cs = min(sh.chunk, c_end - cb);
      float *t2 = reinterpret_cast<float *>(lds);      // [cs][nz][oh][ow]
      float *t1 = t2 + cs * nz * ohw;                  // [cs][nz][ny][ow]; CL: [nz][ny][cs][ow]
      float *gbox = t1 + cs * nz * ny * p.ow;          // [cs][nz][ny][nx] (planar accumulation only)
      const T *go = src + static_cast<long>(cb - c_begin) * cells;
      const float inv_cs = 1.f / cs;
      // z: thread = (c, ph, pw); its grad_output values stay in registers
      for (int i = threadIdx.x; i < cs * ohw; i += kPoolThreads) {
        const int c = fdiv(i, inv_ohw), hw = i - c * ohw;
        float g[CELLS];
#pragma unroll
        for (int k = 0; k < CELLS; k++) g[k] = k < p.od ? load(go + c * cells + k * ohw + hw) : 0.f;
        for (int z = 0; z < nz; z++) {
          float acc = 0.f;
#pragma unroll
          for (int k = 0; k < CELLS; k++) acc += wd[2][z][k] * g[k];
          t2[(c * nz + z) * ohw + hw] = acc;
        }
      }
      __syncthreads();
      // y: thread = (c, z, pw)
      for (int i = threadIdx.x; i < cs * nz * p.ow; i += kPoolThreads) {
        const int cz = fdiv(i, inv_ow), pw = i - cz * p.ow;
        const int c = fdiv(cz, 1.f / nz), z = cz - c * nz;
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
      const long first = (static_cast<long>(tz.box_lo) * p.H + ty.box_lo) * p.W + tx.box_lo;
      if (CL) {   // channel fastest across the lanes: a wavefront adds runs of cs contiguous floats
        for (int i = threadIdx.x; i < cs * nz * ny; i += kPoolThreads) {
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
        for (int i = threadIdx.x; i < cs * nz * ny; i += kPoolThreads) {
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
        for (int i = threadIdx.x; i < cs * vol; i += kPoolThreads) {
          const float v = gbox[i];
          if (v == 0.f) continue;
          const int c = fdiv(i, inv_vol), r0 = i - c * vol, z = fdiv(r0, inv_nxy), r1 = r0 - z * nx * ny;
          const int y = fdiv(r1, inv_nx), x = r1 - y * nx;
          atomic_add(corner + c * plane + (static_cast<long>(z) * p.H + y) * p.W + x, static_cast<G>(v));
        }
      }
      __syncthreads();
    }
    return;
  }
  for (int cb = c_begin; cb < c_end; cb += sh.chunk) {
    const int cs = min(sh.chunk, c_end - cb);
    float *gbox = reinterpret_cast<float *>(lds);    // [cs][nz][ny][nx]
    float *t1 = gbox + cs * vol;                     // [cs][nz][ny][ow]
    float *t2 = t1 + cs * nz * ny * p.ow;            // [cs][nz][oh][ow]
    const T *go = src + static_cast<long>(cb - c_begin) * cells;
    // Transposed contractions as gathers.  Entries are sorted by coordinate, so the entries whose
    // low tap is source index i form the range [first[i], first[i+1]) and those whose high tap is
    // i are the low-tap entries of i - 1 (a clamped edge entry has lo == hi and zero high weight).
    for (int i = threadIdx.x; i < cs * nz * ohw; i += kPoolThreads) {  // transpose of "contract z"
      const int c = fdiv(i, inv_nzohw), r0 = i - c * nz * ohw, z = fdiv(r0, inv_ohw), hw = r0 - z * ohw;
      const T *r = go + c * cells + hw;
      const int mid = tz.first[z], e0 = z > 0 ? tz.first[z - 1] : mid, e1 = tz.first[z + 1];
      float acc = 0.f;
      for (int e = e0; e < e1; e++) {
        const float w = e < mid ? (tz.hi[e] == z ? tz.whi[e] : 0.f) : tz.wlo[e];
        acc += w * load(r + fdiv(e, inv_gz) * ohw);
      }
      t2[i] = acc;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < cs * nz * ny * p.ow; i += kPoolThreads) {  // transpose of "contract y"
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
    for (int i = threadIdx.x; i < cs * vol; i += kPoolThreads) {  // transpose of "contract x"
      const int row = fdiv(i, inv_nx), x = i - row * nx;
      const float *r = t1 + row * p.ow;
      const int mid = tx.first[x], e0 = x > 0 ? tx.first[x - 1] : mid, e1 = tx.first[x + 1];
      float acc = 0.f;
      for (int e = e0; e < e1; e++) {
        const float w = e < mid ? (tx.hi[e] == x ? tx.whi[e] : 0.f) : tx.wlo[e];
        acc += w * r[fdiv(e, inv_gx)];
      }
      gbox[i] = acc;
    }
    __syncthreads();
    const long first = (static_cast<long>(tz.box_lo) * p.H + ty.box_lo) * p.W + tx.box_lo;
    G *corner = dst + static_cast<long>(cb - c_begin) * plane + first;
    for (int i = threadIdx.x; i < cs * vol; i += kPoolThreads) {
      const float v = gbox[i];
      if (v == 0.f) continue;
      const int c = fdiv(i, inv_vol), r0 = i - c * vol, z = fdiv(r0, inv_nxy), r1 = r0 - z * nx * ny;
      const int y = fdiv(r1, inv_nx), x = r1 - y * nx;
      const long voxel = (static_cast<long>(z) * p.H + y) * p.W + x;
      atomic_add(CL ? dst_cl + (first + voxel) * p.C + (cb - c_begin) + c : corner + c * plane + voxel, static_cast<G>(v));
    }
    __syncthreads();
  }
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
static int pool_channels_per_block(const RoiProblem &p) {
  int cpb = 32;
  while (cpb < 256 && cpb < p.C && static_cast<long>(p.R) * ((p.C + 2 * cpb - 1) / (2 * cpb)) >= 6144) cpb *= 2;
  while (cpb > 1 && static_cast<long>(p.R) * ((p.C + cpb - 1) / cpb) < 1024) cpb /= 2;
  return cpb;
}

template <typename T, int CELLS>
static void launch_pool_forward(const void *input, const float *r, void *output, const RoiProblem &p, int cpb,
                                dim3 grid, hipStream_t s) {
  hipLaunchKernelGGL((roi_pool_forward_kernel<T, float, CELLS>), grid, dim3(kPoolThreads), 0, s,
                     static_cast<const T *>(input), r, static_cast<T *>(output), p, cpb);
}

template <typename T, bool CL, int CELLS>
static void launch_pool_backward(const void *grad_output, const float *r, void *acc, const RoiProblem &p, int cpb,
                                 dim3 grid, hipStream_t s) {
  hipLaunchKernelGGL((roi_pool_backward_kernel<T, float, float, CL, CELLS>), grid, dim3(kPoolThreads), 0, s,
                     static_cast<const T *>(grad_output), r, static_cast<float *>(acc), p, cpb);
}

// dense-matrix width of the kernel instance: 8 cells per axis when the output allows it
static bool pool_small_cells(const RoiProblem &p) { return p.od <= 8 && p.oh <= 8 && p.ow <= 8; }

int roi_pool_forward(const void *input, const void *rois, void *output, int dtype,
                     const RoiProblem &p, hipStream_t s) {
  if (!pool_applies(dtype, p)) return -1;
  const int cpb = pool_channels_per_block(p);
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
      small ? launch_pool_forward<__half, 8>(input, r, output, p, cpb, grid, s)
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
