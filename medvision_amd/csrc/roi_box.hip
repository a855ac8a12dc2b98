// RoIAlign / RoIAlignRotated BACKWARD for small outputs per roi (detection heads: 7^3, 14^2 ... cells)
// that the separable pooled kernels do not take: rotated boxes, sampling grids above 4, heads of more
// than 1024 cells.  Same results as the reference's one-thread-per-output kernel with one atomicAdd per
// sample corner (csrc/cuda/roi_align_rotated_3d_cuda_kernel.cuh:124-265 and the 2-D twin).
//
// A workgroup owns (one roi, a group of channels).  The roi's geometry (fp64) is worked out once; its
// output cells are taken in blocks small enough for the axis-aligned box of source voxels that a
// block's samples touch to fit an LDS tile of 32-bit FIXED-POINT sums (an LDS fp32 atomic retires one
// lane at a time): every sample adds weight * grad_output / count to the <= 8 voxels it touches, and
// the tile's non-zero sums then go to the fp32 gradient buffer as one atomic per voxel with lanes along
// x (one request per 64-byte sector) instead of one scattered atomic per sample corner.  The tile
// holds as many of the workgroup's channels side by side as fit, so a sample's taps are worked out
// once for all of them.  Scale per (roi, channel): max |grad_output| / count < 2^e is mapped to 2^t
// quanta, t = 30 - ceil(log2(samples that can reach one voxel)); a term is rounded by at most
// 2^-(t+1) of that bound.  Rois with t < 20 (fp32 tensors; 12 for 16-bit ones: boxes of about a voxel,
// where thousands of samples meet), blocks of one cell whose box still does not fit, and channels whose
// gradient holds a NaN or an infinity add per sample, as the general kernel does, inside the same launch.
// Sample coordinates, tap decisions and the void rule are those of the general kernels (sampling.hpp,
// fp64).
//
// (The forward pass of the same problems stays on the general kernel: copying a block's box to LDS was
// measured slower -- rotated rois of 6 - 24 voxels read a voxel of the box less than once -- and so was
// sharing a sample's taps between channels with the samples of a cell in neighbouring lanes.)
#include "common.hpp"
#include "roi_geometry.hpp"
#include "sampling.hpp"
#include "roi_taps.hpp"

namespace mv {

constexpr int kBoxThreads = 256;
constexpr int kBoxLds = 48 * 1024;   // three workgroups per compute unit

// The roi's output cells are worked through in blocks of blk[0] x blk[1] x blk[2] cells, small enough for
// the axis-aligned box of source voxels that a block's samples touch (n[0] x n[1] x n[2], the same for
// every block of the roi) to fit the tile.
struct BoxPlan {
  int n[3], blk[3];
  int mode;        // 0: no sample of the roi reads or writes anything, 1: boxes in LDS, 2: per-sample path
  int term_bits;   // backward: binary digits of a term below the channel's bound
  double reach[3]; // half the extent of a block's samples along each source axis (with a margin)
};

// One thread: the block shape and the box extent.
__device__ inline void plan_box(BoxPlan &b, const RoiGeom &g, const RoiProblem &p, int cap_voxels, int min_term_bits) {
  const int cells[3] = {p.ow, p.oh, p.od}, size[3] = {p.W, p.H, p.D};
  bool empty = g.batch < 0 || g.grid[0] <= 0 || g.grid[1] <= 0 || (p.ndim == 3 && g.grid[2] <= 0);
  double edge[3] = {2.0, 2.0, 2.0};
  // the whole roi: void when its samples' bounding box lies outside [-1, size] on some axis
  for (int a = 0; a < p.ndim && !empty; a++) {
    double c = g.centre[a], reach = 0.0;
    for (int j = 0; j < p.ndim; j++) {
      const double first = local_coord(g, j, 0, 0), last = local_coord(g, j, cells[j] - 1, g.grid[j] - 1);
      c += g.rot[3 * a + j] * 0.5 * (first + last);
      reach += fabs(g.rot[3 * a + j] * 0.5 * (last - first));
    }
    const double rmin = c - reach - 1e-6, rmax = c + reach + 1e-6;
    if (rmax < -1.0 || rmin > static_cast<double>(size[a]) || !(rmin == rmin) || !(rmax == rmax)) empty = true;
    // (samples beyond the first or last voxel are moved onto it with their full weight, see the bound below)
    edge[a] = size[a] == 1 ? 2.0 : ((rmin < 0.0 || rmax > static_cast<double>(size[a] - 1)) ? 1.5 : 1.0);
  }
  for (int j = 0; j < 3; j++) { b.blk[j] = j < p.ndim ? cells[j] : 1; b.n[j] = 1; b.reach[j] = 0.0; }
  bool fits = false;
  for (int round = 0; round < 40 && !empty; round++) {
    double half[3] = {0.0, 0.0, 0.0};
    for (int j = 0; j < p.ndim; j++) half[j] = 0.5 * ((b.blk[j] - 1) * g.bin[j] + (g.grid[j] - 1) * g.sub[j]);
    long voxels = 1;
    for (int a = 0; a < p.ndim; a++) {
      double reach = 1e-6;   // (wider than the rounding of the per-sample arithmetic, which evaluates the same affine map)
      for (int j = 0; j < p.ndim; j++) reach += fabs(g.rot[3 * a + j] * half[j]);
      b.reach[a] = reach;
      // integers in [floor(c - reach), floor(c + reach) + 1]: at most floor(2 reach) + 3
      b.n[a] = static_cast<int>(fmin(floor(2.0 * reach) + 3.0, static_cast<double>(size[a])));
      voxels *= b.n[a];
    }
    if (voxels <= cap_voxels) { fits = true; break; }
    int widest = -1;
    for (int j = 0; j < p.ndim; j++)
      if (b.blk[j] > 1 && (widest < 0 || half[j] > half[widest])) widest = j;
    if (widest < 0) break;
    b.blk[widest] = (b.blk[widest] + 1) / 2;
  }
  // What the samples can add up to in one voxel, in units of the largest term: the smaller of
  //  - the number of samples that reach a voxel (those within a ball of radius sqrt(3) on the lattice of spacing
  //    sub, at most all samples along an axis), and
  //  - the sum of their WEIGHTS.  A sample's weight is a product of tent functions of its distance to the voxel;
  //    every sample owns a cell of the lattice (volume sub_x sub_y sub_z, extent e_a = sum_j |rot[a][j]| sub_j along
  //    voxel axis a), over which the tent widened by e_a / 2 on either side is at least the sample's own, so the
  //    sum is at most the integral of the widened tents over the cell volume: prod_a (1 + e_a) / prod_j sub_j
  //    (plain boxes: prod (1 / sub + 1)).  On an axis where the roi reaches past the volume's first or last voxel the
  //    samples out there are moved onto that voxel with weight 1: its weight function has the integral 1.5 instead
  //    of 1 (2 on an axis of one voxel).  Thousands of samples may reach a voxel of a finely sampled roi, but their
  //    weights add up to a few hundred.  (The half quantum that each of the reaching terms may be rounded by is
  //    some tens of quanta per unit of weight, nothing beside the 2^30 quanta that the sums may reach.)
  double count_bound = 1.0, weight_bound = 1.0;
  for (int j = 0; j < p.ndim; j++) {
    const double along = fmax(static_cast<double>(cells[j]) * g.grid[j], 1.0), sub = fmax(g.sub[j], 1e-9);
    count_bound *= floor(fmin(3.4642 / sub + 1.0, along));
    double e = 0.0;
    for (int k = 0; k < p.ndim; k++) e += fabs(g.rot[3 * j + k]) * fmax(g.sub[k], 1e-9);
    weight_bound *= (edge[j] + e) / sub;
  }
  const long terms = static_cast<long>(ceil(fmin(fmin(count_bound, weight_bound), 1e15)));
  int bits = 0;
  while ((1L << bits) < terms && bits < 40) bits++;
  b.term_bits = 30 - bits;
  b.mode = empty ? 0 : ((fits && b.term_bits >= min_term_bits) ? 1 : 2);
}

// A block of cells: its first cell and cell counts per axis, and where its box starts in the volume.
struct BoxBlock {
  int c0[3], cnt[3], lo[3];
  int cells;
};
__device__ __forceinline__ BoxBlock box_block(const RoiGeom &g, const RoiProblem &p, const BoxPlan &b, int block) {
  const int cells[3] = {p.ow, p.oh, p.od}, size[3] = {p.W, p.H, p.D};
  const int nbx = (cells[0] + b.blk[0] - 1) / b.blk[0], nby = (cells[1] + b.blk[1] - 1) / b.blk[1];
  const int idx[3] = {block % nbx, (block / nbx) % nby, block / (nbx * nby)};
  BoxBlock k;
  double mid[3] = {0.0, 0.0, 0.0};
  k.cells = 1;
#pragma unroll
  for (int j = 0; j < 3; j++) {
    k.c0[j] = idx[j] * b.blk[j];
    k.cnt[j] = min(b.blk[j], cells[j] - k.c0[j]);
    k.cells *= k.cnt[j];
    if (j < p.ndim) mid[j] = 0.5 * (local_coord(g, j, k.c0[j], 0) + local_coord(g, j, k.c0[j] + k.cnt[j] - 1, g.grid[j] - 1));
  }
#pragma unroll
  for (int a = 0; a < 3; a++) {
    k.lo[a] = 0;
    if (a >= p.ndim) continue;
    double c = g.centre[a];
#pragma unroll
    for (int j = 0; j < 3; j++)
      if (j < p.ndim) c += g.rot[3 * a + j] * mid[j];
    const int l = static_cast<int>(fmin(floor(fmax(c - b.reach[a], 0.0)), static_cast<double>(size[a] - 1)));
    k.lo[a] = max(min(l, size[a] - b.n[a]), 0);   // (the box stays inside the volume: n <= size)
  }
  return k;
}
__device__ __forceinline__ int box_blocks(const RoiProblem &p, const BoxPlan &b) {
  return ((p.ow + b.blk[0] - 1) / b.blk[0]) * ((p.oh + b.blk[1] - 1) / b.blk[1]) * ((p.od + b.blk[2] - 1) / b.blk[2]);
}
// cell `i` of a block as a cell of the roi
__device__ __forceinline__ unsigned block_cell(const RoiProblem &p, const BoxBlock &k, unsigned i) {
  const unsigned bx = i % k.cnt[0], t = i / k.cnt[0], by = t % k.cnt[1], bz = t / k.cnt[1];
  return ((k.c0[2] + bz) * p.oh + (k.c0[1] + by)) * p.ow + (k.c0[0] + bx);
}

__device__ __forceinline__ BoxPlan uniform_plan(const BoxPlan &shared) {
  BoxPlan u;
#pragma unroll
  for (int a = 0; a < 3; a++) {
    u.n[a] = __builtin_amdgcn_readfirstlane(shared.n[a]);
    u.blk[a] = __builtin_amdgcn_readfirstlane(shared.blk[a]);
    u.reach[a] = uniform_f64(shared.reach[a]);
  }
  u.mode = __builtin_amdgcn_readfirstlane(shared.mode);
  u.term_bits = __builtin_amdgcn_readfirstlane(shared.term_bits);
  return u;
}

// A sample's taps relative to the box: offset of the low corner, the steps to the high taps (0 where
// they collapse onto the low ones at the volume's upper border), the eight weights.
struct BoxSample {
  int at;        // >= 0: inside the box; -1: void; -2: touches voxels beyond the box
  int dx, dy, dz;
  float w[8];    // z-major corner order
};
template <bool ROT>
__device__ __forceinline__ BoxSample box_sample(const RoiGeom &g, const RoiProblem &p, const BoxPlan &b, const int (&lo)[3],
                                                unsigned cell, unsigned sub, BoxTaps &t) {
  BoxSample k;
  k.at = -1; k.dx = k.dy = k.dz = 0;
  if (!box_taps<ROT>(g, p, cell, sub, t)) return k;
  const float wx[2] = {1.f - t.fx, t.fx}, wy[2] = {1.f - t.fy, t.fy}, wz[2] = {1.f - t.fz, t.fz};
#pragma unroll
  for (int m = 0; m < 8; m++) k.w[m] = wz[m >> 2] * wy[(m >> 1) & 1] * wx[m & 1];
  const unsigned bx0 = t.xi[0] - lo[0], bx1 = t.xi[1] - lo[0], by0 = t.yi[0] - lo[1], by1 = t.yi[1] - lo[1];
  const unsigned bz0 = t.zi[0] - lo[2], bz1 = t.zi[1] - lo[2];
  const bool inside = b.mode == 1 && max(bx0, bx1) < static_cast<unsigned>(b.n[0]) && max(by0, by1) < static_cast<unsigned>(b.n[1]) &&
                      max(bz0, bz1) < static_cast<unsigned>(b.n[2]);
  if (!inside) { k.at = -2; return k; }
  k.at = static_cast<int>((bz0 * b.n[1] + by0) * b.n[0] + bx0);
  k.dx = t.xi[1] != t.xi[0] ? 1 : 0;
  k.dy = t.yi[1] != t.yi[0] ? b.n[0] : 0;
  k.dz = t.zi[1] != t.zi[0] ? b.n[0] * b.n[1] : 0;
  return k;
}

// ---- largest rois first ----------------------------------------------------------------------------
// A workgroup's time grows with its roi's box, tenfold between the rois of one detection head, and the
// kernel ends with its slowest workgroup: workgroups therefore take the rois in descending order of size.
// No sorted list exists anywhere: every workgroup works out by itself which roi has its rank, from a
// histogram of size classes (four per octave of the extents' product) and a count within its class, in
// index order -- the same bijection in every workgroup.  Two passes over the roi table (<= kRankRois
// rows, from the caches) and four barriers, a few microseconds per workgroup.
constexpr int kRankBuckets = 128;
constexpr int kRankRois = 4096;   // more rois than this run in index order (the tail of the launch is short then)
constexpr int kRankPerThread = kRankRois / kBoxThreads;
__device__ __forceinline__ unsigned roi_size_class(const float *roi, const RoiProblem &p) {
  float v = 1.f;
  for (int a = 0; a < p.ndim; a++) {
    const float e = p.rotated ? roi[1 + p.ndim + a] : roi[1 + p.ndim + a] - roi[1 + a];
    v *= fmaxf(e * static_cast<float>(p.scale), 1e-3f);
  }
  if (!(v == v)) return kRankBuckets - 1;
  // exponent and two mantissa bits, 2^22 voxels and more in class 0
  const int cls = (127 + 22) * 4 + 3 - static_cast<int>(__float_as_uint(v) >> 21);
  return static_cast<unsigned>(min(max(cls, 0), kRankBuckets - 1));
}
// Every thread of the workgroup must call it; `lds` holds kRankBuckets + 8 words.
__device__ inline unsigned roi_of_rank(const float *__restrict__ rois, const RoiProblem &p, unsigned rank, unsigned *lds) {
  const int cols = roi_columns(p.ndim, p.rotated);
  const unsigned per = (static_cast<unsigned>(p.R) + kBoxThreads - 1) / kBoxThreads;   // <= kRankPerThread
  const unsigned first = threadIdx.x * per;
  unsigned *hist = lds, *wave_total = lds + kRankBuckets, *picked = lds + kRankBuckets + 4;
  if (threadIdx.x < kRankBuckets) hist[threadIdx.x] = 0;
  if (threadIdx.x == 0) { picked[0] = 0; picked[1] = 0; picked[2] = rank; }   // (rank < R: a valid roi whatever follows)
  __syncthreads();
  unsigned cls[kRankPerThread / 4];   // a byte per roi of the thread's run
#pragma unroll
  for (int i = 0; i < kRankPerThread / 4; i++) cls[i] = 0;
#pragma unroll
  for (int i = 0; i < kRankPerThread; i++) {
    const unsigned r = first + i;
    if (static_cast<unsigned>(i) < per && r < static_cast<unsigned>(p.R)) {
      const unsigned c = roi_size_class(rois + static_cast<long>(r) * cols, p);
      cls[i / 4] |= c << (8 * (i % 4));
      atomicAdd(&hist[c], 1u);
    }
  }
  __syncthreads();
  // the class that holds the rank, and the rank within it: lane l of the first wavefront owns classes 2l, 2l + 1
  if (threadIdx.x < 64) {
    const unsigned h0 = hist[2 * threadIdx.x], h1 = hist[2 * threadIdx.x + 1];
    unsigned incl = h0 + h1;
#pragma unroll
    for (int d = 1; d < 64; d *= 2) {
      const unsigned up = __shfl_up(incl, d);
      if (threadIdx.x >= static_cast<unsigned>(d)) incl += up;
    }
    const unsigned excl = incl - h0 - h1;
    if (rank >= excl && rank < excl + h0) { picked[0] = 2 * threadIdx.x; picked[1] = rank - excl; }
    else if (rank >= excl + h0 && rank < incl) { picked[0] = 2 * threadIdx.x + 1; picked[1] = rank - excl - h0; }
  }
  __syncthreads();
  const unsigned want = picked[0], kth = picked[1];
  unsigned mine = 0;
#pragma unroll
  for (int i = 0; i < kRankPerThread; i++)
    if (static_cast<unsigned>(i) < per && first + i < static_cast<unsigned>(p.R) && ((cls[i / 4] >> (8 * (i % 4))) & 0xffu) == want) mine++;
  // exclusive sum of `mine` over the workgroup's threads
  unsigned incl = mine;
  const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
#pragma unroll
  for (int d = 1; d < 64; d *= 2) {
    const unsigned up = __shfl_up(incl, d);
    if (lane >= static_cast<unsigned>(d)) incl += up;
  }
  if (lane == 63) wave_total[wave] = incl;
  __syncthreads();
  unsigned before = incl - mine;
  for (unsigned w = 0; w < wave; w++) before += wave_total[w];
  if (kth >= before && kth < before + mine) {
    unsigned left = kth - before;
#pragma unroll
    for (int i = 0; i < kRankPerThread; i++)
      if (static_cast<unsigned>(i) < per && first + i < static_cast<unsigned>(p.R) && ((cls[i / 4] >> (8 * (i % 4))) & 0xffu) == want) {
        if (left == 0) picked[2] = first + i;
        left--;
      }
  }
  __syncthreads();
  return min(picked[2], static_cast<unsigned>(p.R) - 1u);
}

constexpr int kBoxChannels = 16;   // channels a workgroup's tile holds at most (and a workgroup owns at most)
// Samples per thread whose taps stay in registers while a block's channels pass through the tile: the
// fp64 geometry of a sample is then worked out once per block, not once per pass.
constexpr int kBoxKeep = 12;
// A kept sample in 32 bits: offset of its low corner in the box (14 bits: the tile has 12288 cells), which
// of the high taps differ from the low ones (x, y, z: bits 14 - 16), its output cell (from bit 17; heads of
// up to 4096 cells).  Bit 31: the sample touches voxels beyond the box and is worked out again when used.
constexpr unsigned kKeptVoid = 0xffffffffu, kKeptBeyond = 0x80000000u;
static_assert(kBoxLds / 4 <= (1 << 14), "a kept sample's box offset has 14 bits");

// ---- backward ------------------------------------------------------------------------------------
// `per_group` <= kBoxChannels channels per workgroup; the tile holds `cpt` = as many of them as fit
// side by side, so a sample's taps are applied to cpt channels at a time.
template <typename T, bool ROT>
__global__ __launch_bounds__(kBoxThreads, 3) void roi_box_backward_kernel(const T *__restrict__ gout,
                                                                          const float *__restrict__ rois,
                                                                          float *__restrict__ acc, const RoiProblem p,
                                                                          const int per_group, const int groups, const int ranked) {
  __shared__ RoiGeom gs;
  __shared__ double trig[6];
  __shared__ BoxPlan plan;
  __shared__ __attribute__((aligned(16))) int tile[kBoxLds / 4];
  __shared__ unsigned bound[kBoxChannels];
  __shared__ float to_quanta[kBoxChannels], from_quanta[kBoxChannels];
  __shared__ unsigned rank_scratch[kRankBuckets + 8];
  // the channel groups of a roi run side by side (they read the same gradient rows and roi), and the
  // rois in descending order of size where `ranked` says so
  const unsigned group_index = blockIdx.x % static_cast<unsigned>(groups);
  unsigned n = blockIdx.x / static_cast<unsigned>(groups);
  if (ranked) n = roi_of_rank(rois, p, n, rank_scratch);
  build_geom_block(gs, trig, rois + static_cast<long>(n) * roi_columns(p.ndim, p.rotated), p);
  // fixed-point sums only where a term keeps 20 binary digits below the channel's bound (fp32 tensors; 12
  // for 16-bit ones): boxes of a voxel or less, where thousands of samples meet in one voxel, add per sample
  if (threadIdx.x == 0) plan_box(plan, gs, p, kBoxLds / 4, sizeof(T) == 4 ? 20 : 12);
  for (int i = threadIdx.x * 4; i < kBoxLds / 4; i += kBoxThreads * 4) *reinterpret_cast<int4 *>(tile + i) = int4{0, 0, 0, 0};
  if (threadIdx.x < kBoxChannels) bound[threadIdx.x] = 0;
  __syncthreads();
  const BoxPlan b = uniform_plan(plan);
  if (b.mode == 0) return;
  const RoiGeom g = uniform_geom(gs);
  const int cells = p.od * p.oh * p.ow;
  const unsigned count = static_cast<unsigned>(g.count);
  const long plane = static_cast<long>(p.D) * p.H * p.W;
  const int c_first = group_index * per_group, c_end = min(c_first + per_group, p.C);
  const float inv_count = 1.f / static_cast<float>(g.count);
  const int count_shift = 31 - __clz(g.count);   // floor(log2 count): |g| / count < 2^(e - count_shift)
  const int n0 = b.n[0], box = b.n[0] * b.n[1] * b.n[2];
  const int cpt = b.mode == 1 ? min(per_group, (kBoxLds / 4) / box) : per_group;
  const float inv_row = 1.f / static_cast<float>(n0), inv_rows = 1.f / static_cast<float>(b.n[1]);
  const int blocks = box_blocks(p, b);
  const int row_skip = p.W - n0;
  const long slice_skip = static_cast<long>(p.H - b.n[1]) * p.W;
  const bool narrow = plane < (1L << 31);   // offsets within a channel fit 32 bits
  // Per channel of the workgroup the largest |grad_output| of the roi, as the bit pattern of a float (NaNs
  // order above infinity): |term| <= max |g| / count < 2^(e - 126 - count_shift), and a term is counted in
  // quanta of 2^-term_bits of that power of two.  A channel with a NaN or an infinity in its gradient takes
  // the per-sample path (scale 0).
  {
    const T *gall = gout + (static_cast<long>(n) * p.C + c_first) * cells;
    const int span = (c_end - c_first) * cells;
    const float inv_cells = 1.f / static_cast<float>(cells);
    for (int i = threadIdx.x; i < span; i += kBoxThreads)
      atomicMax(&bound[static_cast<int>((static_cast<float>(i) + 0.5f) * inv_cells)], __float_as_uint(fabsf(static_cast<float>(load(gall + i)))));
    __syncthreads();
    if (static_cast<int>(threadIdx.x) < c_end - c_first) {
      const unsigned bits = bound[threadIdx.x];
      const int ex = min(max(127 + 126 + count_shift + b.term_bits - static_cast<int>(bits >> 23), 1), 253);
      to_quanta[threadIdx.x] = bits < 0x7f800000u ? __uint_as_float(static_cast<unsigned>(ex) << 23) * inv_count : 0.f;
      from_quanta[threadIdx.x] = __uint_as_float(static_cast<unsigned>(254 - ex) << 23);
    }
    __syncthreads();
  }
  for (int block = 0; block < blocks; block++) {
    const BoxBlock k = box_block(g, p, b, block);
    const bool few = static_cast<long>(k.cells) * count < (1L << 31);
    const unsigned total = few ? static_cast<unsigned>(k.cells) * count : 0u;   // sample s = cell * count + sub
    // several passes over the same samples: keep the first kBoxKeep per thread
    const bool keep = few && b.mode == 1 && c_end - c_first > cpt;
    unsigned kept[kBoxKeep];
    float kfx[kBoxKeep], kfy[kBoxKeep], kfz[kBoxKeep];
    if (keep) {
      // worked out last to first, every record moving up one place per round, so that the geometry is
      // compiled once and the records still sit in registers with fixed names
#pragma unroll
      for (int j = 0; j < kBoxKeep; j++) { kept[j] = kKeptVoid; kfx[j] = kfy[j] = kfz[j] = 0.f; }
#pragma unroll 1
      for (int round = kBoxKeep - 1; round >= 0; round--) {
#pragma unroll
        for (int j = kBoxKeep - 1; j > 0; j--) { kept[j] = kept[j - 1]; kfx[j] = kfx[j - 1]; kfy[j] = kfy[j - 1]; kfz[j] = kfz[j - 1]; }
        kept[0] = kKeptVoid;
        const unsigned s = threadIdx.x + static_cast<unsigned>(round) * kBoxThreads;
        if (s < total) {
          BoxTaps t;
          const unsigned cell = block_cell(p, k, s / count);
          const BoxSample q = box_sample<ROT>(g, p, b, k.lo, cell, s % count, t);
          if (q.at >= 0)
            kept[0] = static_cast<unsigned>(q.at) | (q.dx ? 1u << 14 : 0u) | (q.dy ? 1u << 15 : 0u) | (q.dz ? 1u << 16 : 0u) | (cell << 17);
          else if (q.at == -2)
            kept[0] = kKeptBeyond | (cell << 17);
          kfx[0] = t.fx; kfy[0] = t.fy; kfz[0] = t.fz;
        }
      }
    }
    for (int c0 = c_first; c0 < c_end; c0 += cpt) {
      const int nc = min(cpt, c_end - c0);
      const T *gsrc = gout + (static_cast<long>(n) * p.C + c0) * cells;
      float *vol = acc + (static_cast<long>(g.batch) * p.C + c0) * plane;
      const int cq = c0 - c_first;   // the pass's first channel among the workgroup's
      // a sample inside the box: its eight terms per channel into the tile
      auto into_tile = [&](int at, int dx, int dy, int dz, const float (&w)[8], int ch, float gv, float scale) {
        const float gq = gv * scale;
        int *cell0 = tile + ch * box + at;
#pragma unroll
        for (int m = 0; m < 8; m++) {
          const int v = __float2int_rn(gq * w[m]);
          if (v != 0)
            __hip_atomic_fetch_add(cell0 + ((m >> 2) ? dz : 0) + (((m >> 1) & 1) ? dy : 0) + ((m & 1) ? dx : 0), v, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_WORKGROUP);
        }
      };
      auto scatter = [&](unsigned cell, unsigned sub, bool beyond_only) {
        BoxTaps t;
        const BoxSample q = box_sample<ROT>(g, p, b, k.lo, cell, sub, t);
        if (q.at == -1) return;
        for (int ch = 0; ch < nc; ch++) {
          const float gv = static_cast<float>(load(gsrc + static_cast<long>(ch) * cells + cell));
          if (gv == 0.f) continue;
          const float scale = to_quanta[cq + ch];
          if (scale != 0.f && q.at >= 0) {
            if (!beyond_only) into_tile(q.at, q.dx, q.dy, q.dz, q.w, ch, gv, scale);
          } else {
            const float top = gv * inv_count;
            float *dst = vol + static_cast<long>(ch) * plane;
#pragma unroll
            for (int m = 0; m < 8; m++)
              if (q.w[m] != 0.f)
                atomic_add(dst + (static_cast<long>(t.zi[m >> 2]) * p.H + t.yi[(m >> 1) & 1]) * p.W + t.xi[m & 1], top * q.w[m]);
          }
        }
      };
      unsigned first = threadIdx.x;
      unsigned again = 0, apart = 0;   // kept samples to work out again: all their terms / those of channels without a scale
      if (keep) {
        // four records per round, then every record moves down four places: after the last round each is
        // back where the next pass expects it (unrolled over all twelve, the compiler ran out of registers)
#pragma unroll 1
        for (int round = 0; round < kBoxKeep / 4; round++) {
#pragma unroll
          for (int u = 0; u < 4; u++) {
            const int j = round * 4 + u;
            const unsigned rec = kept[u];
            if (static_cast<unsigned>(j) * kBoxThreads >= total || rec == kKeptVoid) continue;
            if (rec & kKeptBeyond) { again |= 1u << j; continue; }
            const unsigned cell = (rec >> 17) & 0x3fffu;
            const float wx[2] = {1.f - kfx[u], kfx[u]}, wy[2] = {1.f - kfy[u], kfy[u]}, wz[2] = {1.f - kfz[u], kfz[u]};
            float w[8];
#pragma unroll
            for (int m = 0; m < 8; m++) w[m] = wz[m >> 2] * wy[(m >> 1) & 1] * wx[m & 1];
            const int at = static_cast<int>(rec & 0x3fffu);
            const int dx = (rec >> 14) & 1, dy = (rec & (1u << 15)) ? n0 : 0, dz = (rec & (1u << 16)) ? n0 * b.n[1] : 0;
            for (int ch = 0; ch < nc; ch++) {
              const float gv = static_cast<float>(load(gsrc + static_cast<long>(ch) * cells + cell));
              if (gv == 0.f) continue;
              const float scale = to_quanta[cq + ch];
              if (scale != 0.f) into_tile(at, dx, dy, dz, w, ch, gv, scale);
              else apart |= 1u << j;   // a channel without a scale: its terms go out one by one
            }
          }
#pragma unroll
          for (int u = 0; u < 4; u++) {
            const unsigned r0 = kept[u];
            const float x0 = kfx[u], y0 = kfy[u], z0 = kfz[u];
#pragma unroll
            for (int j = u; j + 4 < kBoxKeep; j += 4) { kept[j] = kept[j + 4]; kfx[j] = kfx[j + 4]; kfy[j] = kfy[j + 4]; kfz[j] = kfz[j + 4]; }
            kept[kBoxKeep - 4 + u] = r0; kfx[kBoxKeep - 4 + u] = x0; kfy[kBoxKeep - 4 + u] = y0; kfz[kBoxKeep - 4 + u] = z0;
          }
        }
        first += kBoxKeep * kBoxThreads;
      }
      if (few) {
        // neighbouring lanes take neighbouring samples; first what the kept records left over
        unsigned next = first;
        while (true) {
          unsigned s;
          bool beyond_only = false;
          if (again | apart) {
            const int j = __ffs(static_cast<int>(again | apart)) - 1;
            beyond_only = !((again >> j) & 1u);
            again &= ~(1u << j); apart &= ~(1u << j);
            s = threadIdx.x + static_cast<unsigned>(j) * kBoxThreads;
          } else if (next < total) {
            s = next; next += kBoxThreads;
          } else {
            break;
          }
          scatter(block_cell(p, k, s / count), s % count, beyond_only);
        }
      } else {
        for (unsigned i = threadIdx.x; i < static_cast<unsigned>(k.cells); i += kBoxThreads)
          for (unsigned sub = 0; sub < count; sub++) scatter(block_cell(p, k, i), sub, false);
      }
      __syncthreads();
      if (b.mode == 1) {
        // lanes along the box's rows: neighbouring lanes add to neighbouring voxels of the buffer
        for (int ch = 0; ch < nc; ch++) {
          const float unit = from_quanta[cq + ch];
          int *sums = tile + ch * box;
          float *dst = vol + static_cast<long>(ch) * plane + (static_cast<long>(k.lo[2]) * p.H + k.lo[1]) * p.W + k.lo[0];
          // four cells per lane and round, read together; a cell's place in the volume from its place in the
          // box: v + row * (W - n0) + slice * (H - n1) * W
          for (int v0 = threadIdx.x; v0 < box; v0 += 4 * kBoxThreads) {
            int q[4];
#pragma unroll
            for (int u = 0; u < 4; u++) q[u] = v0 + u * kBoxThreads < box ? sums[v0 + u * kBoxThreads] : 0;
#pragma unroll
            for (int u = 0; u < 4; u++) {
              if (q[u] == 0) continue;
              const int v = v0 + u * kBoxThreads;
              sums[v] = 0;
              const int row = static_cast<int>((static_cast<float>(v) + 0.5f) * inv_row);
              const int bz = static_cast<int>((static_cast<float>(row) + 0.5f) * inv_rows);
              const float add = static_cast<float>(q[u]) * unit;
              if (narrow) atomic_add(dst + static_cast<unsigned>(v + row * row_skip + bz * static_cast<int>(slice_skip)), add);
              else atomic_add(dst + (v + static_cast<long>(row) * row_skip + bz * slice_skip), add);
            }
          }
        }
      }
      __syncthreads();   // (the next pass adds to the cells that this one has just cleared)
    }
  }
}

// Small outputs per roi in 16- or 32-bit tensors, orders 0 / 1; what the tiled, gathering and pooled
// backward kernels have not taken arrives here (rotated boxes, large grids, heads of more than 1024 cells).
bool roi_box_applies(int dtype, const RoiProblem &p) {
  if (dtype != MV_F16 && dtype != MV_BF16 && dtype != MV_F32) return false;
  if (p.order != 0 && p.order != 1) return false;
  const long cells = static_cast<long>(p.od) * p.oh * p.ow;
  return cells <= 4096 && p.R <= 0x7fffffff && p.C >= 1;
}

// Channels per workgroup: the set-up (geometry, box, the samples' taps) is shared by them, so as many as
// leave enough workgroups to fill the compute units three times over.
static int box_channels_per_group(const RoiProblem &p) {
  int per = kBoxChannels;
  while (per > 1 && static_cast<long>(p.R) * ((p.C + per - 1) / per) < 3 * 768) per /= 2;
  return per;
}

// `acc`: the fp32 buffer the gradient is added to (grad_input itself for fp32 tensors, the workspace for
// 16-bit ones), laid out like grad_input.
int roi_box_backward(const void *grad_output, const void *rois, float *acc, int dtype, const RoiProblem &p, hipStream_t s) {
  if (!roi_box_applies(dtype, p)) return -1;
  const int per = box_channels_per_group(p);
  const long groups = (p.C + per - 1) / per;
  if (static_cast<long>(p.R) * groups > 0x7fffffffL) return -1;
  const dim3 grid(static_cast<unsigned>(p.R * groups)), block(kBoxThreads);
  // in descending order of size while the launch is a few rounds of workgroups, whose last round the largest rois would stretch
  const int ranked = p.R > 1 && p.R <= kRankRois ? 1 : 0;
  const float *r = static_cast<const float *>(rois);
#define MV_BOX_BACKWARD(TYPE)                                                                                              \
  if (p.rotated)                                                                                                           \
    hipLaunchKernelGGL((roi_box_backward_kernel<TYPE, true>), grid, block, 0, s, static_cast<const TYPE *>(grad_output), r, \
                       acc, p, per, static_cast<int>(groups), ranked);                                                                                       \
  else                                                                                                                     \
    hipLaunchKernelGGL((roi_box_backward_kernel<TYPE, false>), grid, block, 0, s, static_cast<const TYPE *>(grad_output), r, \
                       acc, p, per, static_cast<int>(groups), ranked)
  switch (dtype) {
    case MV_F32: MV_BOX_BACKWARD(float); break;
    case MV_F16: MV_BOX_BACKWARD(__half); break;
    default: MV_BOX_BACKWARD(__hip_bfloat16);
  }
#undef MV_BOX_BACKWARD
  return check_launch("roi_box_backward_kernel");
}

}  // namespace mv
