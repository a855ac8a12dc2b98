// Backward of the 3-D deformable convolution for fp16 / bf16 / fp32 tensors, built around the
// matrix cores and channels-last buffers.
//
//   gcol[c, k, q] = sum_o Wt[o, c, k] * gy[o, q]                    (GEMM, MFMA)
//   gx[corner_n(k, q), c] += w_n * mask * gcol                       (scatter: LDS tiles + fp32 atomics)
//   goff_a[k, q] = mask * sum_c gcol * dZ/dp_a ,  gmask[k, q] = sum_c gcol * Z
//   gw[o, c, k]  = sum_{b, q} gy[o, q] * col[c, k, q]                (GEMM over positions, MFMA)
//
// Data kernel: a wavefront owns 32 output positions.  Per tap it forms the 32 x 32 block
// gcol[position, channel] with MFMA 32x32x16 (A = gy channels-last, B = weight fragments); the
// accumulator layout gives every lane ONE channel and 16 positions.  x at the corners is fetched 16
// bytes per lane into an LDS stage and read back one channel per lane; the fp32 atomic adds into
// the channels-last gradient buffer are 128-byte contiguous per position.  The four per-position
// sums over channels are reduced across the half-wavefront with DPP adds.  The column values
// mask * Z(x) are stored for the weight kernel.
// Scatter kernel (unit-stride layers whose taps fit its tile): the corners that land near their
// position are summed per brick of positions in a 64-bit fixed-point LDS tile and reach the
// gradient buffer as one atomic per (voxel, channel) of the tile; the data kernel then adds only the
// other corners.
// Weight kernels: a workgroup owns (taps, 32-channel block, range of positions); the MFMA B
// fragment is the column values of a channel for 16 positions at a time — read from the column
// buffer, or (layers beyond its budget) rebuilt by the lanes with a second gather of x; A is gy read
// in its own layout.  Accumulators stay in registers over the whole range and are added to a
// tap-major fp32 gradient once per workgroup.
#include "dcn_mfma.hpp"

#include <atomic>
#include <cstdlib>

namespace mv {

constexpr unsigned kOob = 0x80000000u;  // byte offset beyond every buffer: loads give 0, atomics are dropped
constexpr int kRsrcFlags = 0x00020000;

// weight [Cout, cpg, K] -> B pieces [group][tap][32-channel block][row step][lane][kPiece]:
// lane l, element i = Wt[g*opg + step*2*kPiece + (l/32)*kPiece + i, block*32 + l%32, k]
template <typename T>
__device__ __forceinline__ void dcn_weight_bfragments_block(const T *__restrict__ wt, T *__restrict__ wb, const DcnDims s, const unsigned bid) {
  constexpr int PC = Mfma<T>::kPiece;
  const int cblocks = s.cpg / 32, steps = s.opg / (2 * PC);
  const long total = static_cast<long>(s.groups) * s.K * cblocks * steps * 64;
  const long id = bid * 256L + threadIdx.x;
  if (id >= total) return;
  const int lane = id % 64;
  long r = id / 64;
  const int st = r % steps; r /= steps;
  const int cb = r % cblocks; r /= cblocks;
  const int k = r % s.K;
  const int g = static_cast<int>(r / s.K);
  const int cl = cb * 32 + lane % 32;
  const int o = g * s.opg + st * 2 * PC + (lane / 32) * PC;
  for (int i = 0; i < PC; i++) wb[id * PC + i] = wt[(static_cast<long>(o + i) * s.cpg + cl) * s.K + k];
}
template <typename T>
__global__ __launch_bounds__(256) void dcn_weight_bfragments_kernel(const T *__restrict__ wt,
                                                                    T *__restrict__ wb,
                                                                    const DcnDims s) { dcn_weight_bfragments_block<T>(wt, wb, s, blockIdx.x); }

// One element of x (channels-last) through a range-checked buffer load, as fp32.
template <typename T>
__device__ __forceinline__ float load_element(__amdgpu_buffer_rsrc_t rsrc, unsigned byte_offset) {
  if (sizeof(T) == 4) return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, byte_offset, 0, 0));
  return Mfma<T>::lo(__builtin_amdgcn_raw_buffer_load_b16(rsrc, byte_offset, 0, 0));
}

// Sum over the 32 lanes of each half-wavefront; the result is valid in lanes 16..31 and 48..63.
__device__ __forceinline__ float half_wave_sum(float v) {
#define MV_DPP_ADD(ctrl, rmask, bound)                                                             \
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, \
                                                             rmask, 0xf, bound))
  MV_DPP_ADD(0xB1, 0xf, true);    // quad_perm [1,0,3,2]
  MV_DPP_ADD(0x4E, 0xf, true);    // quad_perm [2,3,0,1]
  MV_DPP_ADD(0x141, 0xf, true);   // row_half_mirror
  MV_DPP_ADD(0x140, 0xf, true);   // row_mirror: every lane of a 16-lane row holds the row sum
  MV_DPP_ADD(0x142, 0xa, false);  // row_bcast15 into rows 1 and 3
#undef MV_DPP_ADD
  return v;
}

// ---- bricks and tiles of the LDS scatter (dcn_backward_scatter_kernel below) ----------------------
// A brick is BD x BH x BW output positions; its tile the TD x TH x TW input voxels centred on the
// reach of the brick's undeformed taps.  A corner is "local" when its voxel lies in
// the tile of its position's brick: local corners are summed in LDS by the scatter kernel, all
// others are added to the gradient buffer by the data kernel, 128 bytes per request.
// Volumes use 4 x 8 x 8 bricks with 10 x 14 x 14 tiles, images 32 x 32 bricks with 44 x 44 tiles (a
// workgroup's fixed costs — clearing and flushing the tile — need more than nine taps of 256
// positions to pay: 16 x 16 bricks gained nothing on 256-channel FPN layers).
struct VolumeBricks { static constexpr int BD = 4, BH = 8, BW = 8, TD = 10, TH = 14, TW = 14; };
struct ImageBricks { static constexpr int BD = 1, BH = 32, BW = 32, TD = 1, TH = 44, TW = 44; };
constexpr int kTileVoxMax = 1960;
struct TileOrigin { int d, h, w; };
template <typename S>
__device__ __forceinline__ TileOrigin tile_origin(const DcnDims &s, int bz, int by, int bx) {
  TileOrigin t;
  t.d = bz * S::BD * s.sd - s.pd - (S::TD - ((S::BD - 1) * s.sd + (s.kd - 1) * s.dd + 1)) / 2;
  t.h = by * S::BH * s.sh - s.ph - (S::TH - ((S::BH - 1) * s.sh + (s.kh - 1) * s.dh + 1)) / 2;
  t.w = bx * S::BW * s.sw - s.pw - (S::TW - ((S::BW - 1) * s.sw + (s.kw - 1) * s.dw + 1)) / 2;
  return t;
}
// bit c: corner c (z-major) of the sample whose first corner is voxel (id, ih, iw) lies in the tile;
// `first` its cell index there
template <typename S>
__device__ __forceinline__ unsigned tile_bits(const TileOrigin &t, int id, int ih, int iw, int &first) {
  const int zd = id - t.d, zh = ih - t.h, zw = iw - t.w;
  const bool fd[2] = {zd >= 0 && zd < S::TD, zd >= -1 && zd < S::TD - 1};
  const bool fh[2] = {zh >= 0 && zh < S::TH, zh >= -1 && zh < S::TH - 1};
  const bool fw[2] = {zw >= 0 && zw < S::TW, zw >= -1 && zw < S::TW - 1};
  unsigned bits = 0;
#pragma unroll
  for (int c = 0; c < 8; c++) bits |= (fd[c >> 2] && fh[(c >> 1) & 1] && fw[c & 1]) ? 1u << c : 0u;
  first = (zd * S::TH + zh) * S::TW + zw;
  return bits;
}

// The LDS sums are 64-bit fixed point (LDS float atomics retire one lane at a time, integer ones
// a wavefront in a few clocks).  Every term is w * mask * gcol with 0 <= w <= 1, so
//   |term| <= max|mask| * max|grad_output| * max_{c,k} sum_o |Wt[o,c,k]|  =: bound < 2^ex,
// and a voxel takes at most one corner of each (position, tap) of the brick: positions * taps terms.
// Terms are scaled by 2^(shift - ex), shift = min(50, 62 - ceil(log2(terms))), and rounded to
// integers (adding 1.5 * 2^52 in fp64 leaves round(x) in the low mantissa bits for |x| < 2^51):
// a term loses less than 2^-shift of the bound (2^-49 for up to 4096 terms), and the sum of a
// voxel stays below 2^63.  words[0..2] hold the bit patterns of the three maxima (of |.|, so they
// order like unsigned integers; a NaN or infinity anywhere gives a non-finite bound, and then no
// corner is treated as local).
constexpr double kRoundMagic = 6755399441055744.0;  // 1.5 * 2^52
struct ScatterScale { bool valid; double up, down; };
__device__ __forceinline__ ScatterScale scatter_scale(const unsigned *__restrict__ words, int terms, bool has_mask) {
  const float bound = 1.001f * __uint_as_float(words[0]) * __uint_as_float(words[1]) *
                      (has_mask ? __uint_as_float(words[2]) : 1.f);
  ScatterScale r;
  r.valid = bound < __builtin_inff() && bound == bound;
  int ex = 0;
  frexpf(fmaxf(bound, 1e-30f), &ex);  // bound < 2^ex
  const int shift = min(50, 62 - (32 - __clz(terms - 1)));
  r.up = ldexp(1.0, shift - ex);
  r.down = ldexp(1.0, ex - shift);
  return r;
}
// round(w * scaled) as a 64-bit integer; the low word of the magic number's bit pattern is zero
__device__ __forceinline__ unsigned long long fixed_term(float w, double scaled) {
  const double x = fma(static_cast<double>(w), scaled, kRoundMagic);
  const unsigned lo = static_cast<unsigned>(__double2loint(x)), hi = static_cast<unsigned>(__double2hiint(x)) - 0x43380000u;
  return (static_cast<unsigned long long>(hi) << 32) | lo;
}

// max |p[i]| as a bit pattern, folded into *out (which starts at 0) with one atomic per workgroup
__device__ __forceinline__ void fold_max(unsigned bits, unsigned *out) {
  __shared__ unsigned part[4];
  for (int sh = 32; sh > 0; sh >>= 1) bits = max(bits, static_cast<unsigned>(__shfl_xor(static_cast<int>(bits), sh)));
  if (threadIdx.x % kWave == 0) part[threadIdx.x / kWave] = bits;
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned m = max(max(part[0], part[1]), max(part[2], part[3]));
    // (atomics on one address retire one after the other: a workgroup that cannot raise the value it
    // reads — possibly an older one, which is never above the current one — leaves it alone)
    if (m > __hip_atomic_load(out, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(out, m);
  }
}
// (block `bid` of `nblocks`: the kernels below call these bodies with their own block index or with a
// share of a launch that does several small jobs at once)
template <typename T>
__device__ __forceinline__ void dcn_absmax_block(const T *__restrict__ p, long n, unsigned *out, const unsigned bid,
                                                 const unsigned nblocks) {
  constexpr int V = 16 / sizeof(T);  // elements per 16-byte load
  float m = 0.f;
  bool bad = false;
  auto take = [&](T e) {
    const float v = fabsf(static_cast<float>(load(&e)));
    bad = bad || !(v == v);
    m = fmaxf(m, v);
  };
  const long head = min(n, static_cast<long>((16 - reinterpret_cast<size_t>(p) % 16) % 16 / sizeof(T)));
  const long groups = (n - head) / V, tid = bid * 256L + threadIdx.x;
  // four independent loads per lane and step
  for (long i = bid * 1024L + threadIdx.x; i < groups; i += nblocks * 1024L) {
    union { u32x4 u; T e[V]; } piece[4];
#pragma unroll
    for (int u = 0; u < 4; u++)
      piece[u].u = i + u * 256 < groups ? *reinterpret_cast<const u32x4 *>(p + head + (i + u * 256) * V) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int u = 0; u < 4; u++)
#pragma unroll
      for (int j = 0; j < V; j++) take(piece[u].e[j]);
  }
  if (tid < head) take(p[tid]);
  const long tail = head + groups * V;
  if (tid < n - tail) take(p[tail + tid]);
  fold_max(bad ? 0x7fc00000u : __float_as_uint(m), out);
}
template <typename T>
__global__ __launch_bounds__(256) void dcn_absmax_kernel(const T *__restrict__ p, long n, unsigned *out) {
  dcn_absmax_block<T>(p, n, out, blockIdx.x, gridDim.x);
}
// max over (group, c, k) of sum_o |Wt[o, c, k]|: a workgroup takes 64 columns, its four wavefronts
// a quarter of the rows each
template <typename T>
__device__ __forceinline__ void dcn_weight_colsum_block(const T *__restrict__ wt, const DcnDims s, unsigned *out, const unsigned bid) {
  __shared__ float part[4][64];
  const long cols = static_cast<long>(s.cpg) * s.K, id = bid * 64L + threadIdx.x % 64;
  const int wave = threadIdx.x / 64;
  float sum = 0.f;
  if (id < cols * s.groups) {
    const long g = id / cols, ck = id - g * cols;
    for (int o = wave; o < s.opg; o += 4) sum += fabsf(static_cast<float>(load(wt + (g * s.opg + o) * cols + ck)));
  }
  part[wave][threadIdx.x % 64] = sum;
  __syncthreads();
  if (wave == 0) sum = part[0][threadIdx.x] + part[1][threadIdx.x] + part[2][threadIdx.x] + part[3][threadIdx.x];
  fold_max(wave == 0 ? (sum == sum ? __float_as_uint(sum) : 0x7fc00000u) : 0u, out);
}
template <typename T>
__global__ __launch_bounds__(256) void dcn_weight_colsum_kernel(const T *__restrict__ wt, const DcnDims s, unsigned *out) {
  dcn_weight_colsum_block<T>(wt, s, out, blockIdx.x);
}

constexpr int kTapWords = 28;  // byte offsets of the corners in x [8] and in the gradient buffer [8], w[8], mask, ld, lh, lw

// SPLIT: corners that are local to their brick's tile (shape S) are left to the scatter kernel.
template <typename T, bool SPLIT, typename S>
__global__ __launch_bounds__(256) void dcn_backward_data_mfma_kernel(
    const T *__restrict__ xt, const T *__restrict__ off, const T *__restrict__ mask,
    const T *__restrict__ gyt, const T *__restrict__ wb, float *__restrict__ gxt,
    T *__restrict__ goff, T *__restrict__ gmask, const DcnDims s, const unsigned *__restrict__ bounds,
    T *__restrict__ col, const long qp) {
  using M = Mfma<T>;
  using P = typename std::conditional<(sizeof(T) == 2), float, double>::type;  // position type
  constexpr int PC = M::kPiece, SL = 2 * PC, ES = sizeof(T);
  __shared__ __attribute__((aligned(16))) float taps[4][32][kTapWords];
  __shared__ float sums[4][4][32];
  // x at the 8 corners of the two positions of an accumulator register, 32 channels each, in two
  // alternating buffers per wavefront: fetched 16 bytes per lane, read back one channel per lane
  __shared__ __attribute__((aligned(16))) T stage[4][2][16][32];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int n = lane % 32, h = lane / 32;
  constexpr int LPC = 2 * ES, FETCHES = ES / 2;  // lanes per corner (16 bytes each), fetches per register
  // one contiguous eighth of the positions per XCD (see xcd_contiguous)
  const long q0 = (static_cast<long>(xcd_contiguous(blockIdx.x, gridDim.x)) * 4 + wave) * 32;
  if (q0 >= s.Q) return;  // whole wavefront idle (no workgroup barriers in this kernel)
  const long q = q0 + n;
  const bool live = q < s.Q;
  const long qc = live ? q : s.Q - 1;
  const int dgi = blockIdx.y, b = blockIdx.z;
  const int ow = qc % s.Wo, oh = (qc / s.Wo) % s.Ho, od = qc / (static_cast<long>(s.Wo) * s.Ho);
  const int bd = od * s.sd - s.pd, bh = oh * s.sh - s.ph, bw = ow * s.sw - s.pw;
  const long bg = static_cast<long>(b) * s.dg + dgi;
  const int cblocks = s.cpg / 32, steps = s.opg / SL;

  const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(xt + static_cast<long>(b) * s.P * s.Cin), 0, static_cast<int>(s.P * s.Cin * ES), kRsrcFlags);
  const __amdgpu_buffer_rsrc_t gr = __builtin_amdgcn_make_buffer_rsrc(
      gxt + static_cast<long>(b) * s.P * s.Cin, 0, static_cast<int>(s.P * s.Cin * 4), kRsrcFlags);
  const unsigned cin2 = static_cast<unsigned>(s.Cin) * ES;
  const T *gyrow = gyt + (static_cast<long>(b) * s.Q + qc) * s.Cout + h * PC;
  const T *o = off + bg * s.nd * s.K * s.Q + qc;
  const T *mk = mask ? mask + bg * s.K * s.Q + qc : nullptr;
  float(*tp)[kTapWords] = taps[wave];
  float(*sm)[32] = sums[wave];
  const TileOrigin origin = tile_origin<S>(s, od / S::BD, oh / S::BH, ow / S::BW);
  const bool split = SPLIT && scatter_scale(bounds, S::BD * S::BH * S::BW * s.K, mask != nullptr).valid;

  int ki = 0, kj = 0, kk = 0;
  for (int k = 0; k < s.K; k++) {
    // ---- taps of (k, q0 + n): both half-wavefronts compute them, the lower one publishes -------
    {
      P pd, ph, pw;
      dcn_offsets(s, o, pd, ph, pw);
      pd += static_cast<P>(bd + ki * s.dd); ph += static_cast<P>(bh + kj * s.dh); pw += static_cast<P>(bw + kk * s.dw);
      const float m = mk ? load(mk) : 1.f;
      o += s.nd * s.Q;
      if (mk) mk += s.Q;
      if (++kk == s.kw) { kk = 0; if (++kj == s.kh) { kj = 0; ++ki; } }
      // corner offsets in bytes (x: element size ES, gradient buffer: 4); kOob for a corner outside
      // the volume and, in the gradient buffer, for one the scatter kernel sums
      CornerTaps t;
      corner_taps<P>(s, pd, ph, pw, live, cin2, 0u, kOob, t);
      int first;
      const unsigned local = split ? tile_bits<S>(origin, static_cast<int>(floor(pd)), static_cast<int>(floor(ph)),
                                               static_cast<int>(floor(pw)), first) : 0u;
      unsigned ag[8];
#pragma unroll
      for (int c = 0; c < 8; c++) ag[c] = (t.at[c] == kOob || ((local >> c) & 1u)) ? kOob : t.at[c] * (4u / ES);
      if (h == 0) {
        float4 *dst = reinterpret_cast<float4 *>(tp[n]);
        dst[0] = make_float4(__uint_as_float(t.at[0]), __uint_as_float(t.at[1]), __uint_as_float(t.at[2]), __uint_as_float(t.at[3]));
        dst[1] = make_float4(__uint_as_float(t.at[4]), __uint_as_float(t.at[5]), __uint_as_float(t.at[6]), __uint_as_float(t.at[7]));
        dst[2] = make_float4(t.w[0], t.w[1], t.w[2], t.w[3]);
        dst[3] = make_float4(t.w[4], t.w[5], t.w[6], t.w[7]);
        dst[4] = make_float4(m, t.ld, t.lh, t.lw);
        dst[5] = make_float4(__uint_as_float(ag[0]), __uint_as_float(ag[1]), __uint_as_float(ag[2]), __uint_as_float(ag[3]));
        dst[6] = make_float4(__uint_as_float(ag[4]), __uint_as_float(ag[5]), __uint_as_float(ag[6]), __uint_as_float(ag[7]));
        sm[0][n] = 0.f; sm[1][n] = 0.f; sm[2][n] = 0.f; sm[3][n] = 0.f;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    for (int cc = 0; cc < s.cpd / 32; cc++) {
      const int c0 = dgi * s.cpd + cc * 32, g = c0 / s.cpg, cb = (c0 - g * s.cpg) / 32;
      // ---- gcol[32 positions x 32 channels] = gy[32 x opg] * Wt_k[opg x 32] -----------------------
      float16_t acc;
#pragma unroll
      for (int r = 0; r < 16; r++) acc[r] = 0.f;
      const T *wfrag = wb + ((((static_cast<long>(g) * s.K + k) * cblocks + cb) * steps) * 64 + lane) * PC;
      const T *arow = gyrow + g * s.opg;
      for (int st = 0; st < steps; st++) {
        const u32x4 a = live ? *reinterpret_cast<const u32x4 *>(arow + st * SL) : u32x4{0u, 0u, 0u, 0u};
        const u32x4 bf = *reinterpret_cast<const u32x4 *>(wfrag + static_cast<long>(st) * (64 * PC));
        acc = M::run(a, bf, acc);
      }
      const unsigned cbyte4 = static_cast<unsigned>(c0 + n) * 4u;
      float colv[4];
      T *colrow = col ? col + ((static_cast<long>(b) * s.K + k) * (s.Cin / 32) + c0 / 32) * qp * 32 : nullptr;
      // ---- register r: position 8*(r/4) + 4*h + r%4, channel c0 + n ------------------------------
      // fetch f of register r: lane l holds 16 bytes of corner (f * 64 + l) / LPC of the register's
      // two positions (corners 0..7 of the lower half-wavefront's position, then the upper one's).
      // kOob plus a channel offset stays beyond the buffers: such loads give 0, such adds are dropped
      auto fetch = [&](int r, u32x4 (&dst)[FETCHES]) {
#pragma unroll
        for (int f = 0; f < FETCHES; f++) {
          const int corner = (f * 64 + lane) / LPC, pp = 8 * (r / 4) + 4 * (corner / 8) + (r % 4);
          const unsigned at = __float_as_uint(tp[pp][corner % 8]);
          dst[f] = __builtin_amdgcn_raw_buffer_load_b128(xr, at + static_cast<unsigned>(c0) * ES + (lane % LPC) * 16u, 0, 0);
        }
      };
      u32x4 cur[FETCHES];
      fetch(0, cur);
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int p = 8 * (r / 4) + 4 * h + (r % 4);
        T(*sg)[32] = stage[wave][r & 1];
#pragma unroll
        for (int f = 0; f < FETCHES; f++)
          *reinterpret_cast<u32x4 *>(&sg[(f * 64 + lane) / LPC][(lane % LPC) * (16 / ES)]) = cur[f];
        if (r + 1 < 16) fetch(r + 1, cur);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const float4 *src = reinterpret_cast<const float4 *>(tp[p]);
        const float4 w0 = src[2], w1 = src[3], e = src[4], g0 = src[5], g1 = src[6];
        const unsigned ag[8] = {__float_as_uint(g0.x), __float_as_uint(g0.y), __float_as_uint(g0.z), __float_as_uint(g0.w),
                                __float_as_uint(g1.x), __float_as_uint(g1.y), __float_as_uint(g1.z), __float_as_uint(g1.w)};
        const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
        const float m = e.x, ld = e.y, lh = e.z, lw = e.w;
        const float gm = acc[r] * m;
        float v[8];
#pragma unroll
        for (int c = 0; c < 8; c++) {
          v[c] = load(&sg[h * 8 + c][n]);
          // with the scatter kernel at work most instructions would find no lane with an add left
          if (!SPLIT || ag[c] != kOob)
            __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(w[c] * gm, gr, ag[c] + cbyte4, 0, 0);
        }
        // value and the three partial derivatives of the trilinear form, sharing the differences
        const float x0 = v[1] - v[0], x1 = v[3] - v[2], x2 = v[5] - v[4], x3 = v[7] - v[6];
        const float a0 = fmaf(lw, x0, v[0]), a1 = fmaf(lw, x1, v[2]), a2 = fmaf(lw, x2, v[4]), a3 = fmaf(lw, x3, v[6]);
        const float b0 = fmaf(lh, x1 - x0, x0), b1 = fmaf(lh, x3 - x2, x2);
        const float dw = fmaf(ld, b1 - b0, b0);
        const float y0 = a1 - a0, y1 = a3 - a2;
        const float c0v = fmaf(lh, y0, a0), c1v = fmaf(lh, y1, a2);
        const float dh = fmaf(ld, y1 - y0, y0);
        const float dd = c1v - c0v;
        const float val = fmaf(ld, dd, c0v);
        const float s0 = half_wave_sum(dd * gm), s1 = half_wave_sum(dh * gm), s2 = half_wave_sum(dw * gm);
        const float s3 = half_wave_sum(acc[r] * val);
        if (n == 16) {  // one lane per half-wavefront; the chunks of a deformable group accumulate
          sm[0][p] += s0; sm[1][p] += s1; sm[2][p] += s2; sm[3][p] += s3;
        }
        // ---- the column values mask * Z(x) for the weight kernel: registers 4g .. 4g + 3 are four
        // consecutive positions, pieces are [position / kPiece][channel][kPiece] ----------------------
        colv[r % 4] = m * val;
        if (col && r % 4 == 3) {
          const long first = q0 + 8 * (r / 4) + 4 * h;  // position of colv[0]
          T *dst = colrow + ((first / PC) * 32 + n) * PC + first % PC;
          if constexpr (ES == 2) {
            // (nontemporal: the buffer is larger than the caches and read once, by the weight kernel)
            __builtin_nontemporal_store((static_cast<unsigned long long>(M::pack2(colv[2], colv[3])) << 32) | M::pack2(colv[0], colv[1]),
                                        reinterpret_cast<unsigned long long *>(dst));
          } else {
            *reinterpret_cast<float4 *>(dst) = make_float4(colv[0], colv[1], colv[2], colv[3]);
          }
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (h == 0 && live) {
      T *go = goff + (bg * s.nd * s.K + s.nd * k) * s.Q + q;
      if (s.nd == 3) go[0] = store_cast<T>(sm[0][n]);
      go[(s.nd - 2) * s.Q] = store_cast<T>(sm[1][n]); go[(s.nd - 1) * s.Q] = store_cast<T>(sm[2][n]);
      if (gmask) gmask[(bg * s.K + k) * s.Q + q] = store_cast<T>(sm[3][n]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
}

// ---- the data kernel with one POSITION per lane (layers that run the scatter kernel) --------------
// The product is formed the other way round: A = weight fragments (rows = channels), B = gy (columns
// = positions), so lane l holds position l % 32 and sixteen channels (16 * (l / 32) .. + 15 of the
// 32-channel block, the fragment kernel orders the MFMA rows accordingly).  The taps stay in the
// lane's registers, x at a corner arrives as the lane's own 16-byte loads (no LDS stage), and the
// four sums over channels are serial adds with one exchange between the half-wavefronts per tap.
// The column values pass through an LDS block laid out like the column buffer and leave as
// 16-byte stores.  Corners the scatter kernel does not take are rare here; their channels go through
// a [position][channel] LDS block so that an atomic instruction still adds 128 contiguous bytes:
// the wavefront lists its far corners once per tap and walks the list two entries at a time.
template <typename T>
__device__ __forceinline__ void dcn_weight_afragments32_block(const T *__restrict__ wt, T *__restrict__ wa, const DcnDims s, const unsigned bid) {
  constexpr int PC = Mfma<T>::kPiece;
  const int cblocks = s.cpg / 32, steps = s.opg / (2 * PC);
  const long total = static_cast<long>(s.groups) * s.K * cblocks * steps * 64;
  const long id = bid * 256L + threadIdx.x;
  if (id >= total) return;
  const int lane = id % 64;
  long r = id / 64;
  const int st = r % steps; r /= steps;
  const int cb = r % cblocks; r /= cblocks;
  const int k = r % s.K;
  const int g = static_cast<int>(r / s.K);
  // accumulator register r of half h is MFMA row 8 * (r / 4) + 4 * h + r % 4: that row carries channel 16 * h + r
  const int row = lane % 32, cl = cb * 32 + 16 * ((row / 4) % 2) + 4 * (row / 8) + row % 4;
  const int o = g * s.opg + st * 2 * PC + (lane / 32) * PC;
  for (int i = 0; i < PC; i++) wa[id * PC + i] = wt[(static_cast<long>(o + i) * s.cpg + cl) * s.K + k];
}
template <typename T>
__global__ __launch_bounds__(256) void dcn_weight_afragments32_kernel(const T *__restrict__ wt,
                                                                      T *__restrict__ wa,
                                                                      const DcnDims s) { dcn_weight_afragments32_block<T>(wt, wa, s, blockIdx.x); }

template <typename T, typename S>
__global__ __launch_bounds__(256, sizeof(T) == 2 ? 3 : 2) void dcn_backward_data_lanes_kernel(
    const T *__restrict__ xt, const T *__restrict__ off, const T *__restrict__ mask,
    const T *__restrict__ gyt, const T *__restrict__ wa, float *__restrict__ gxt,
    T *__restrict__ goff, T *__restrict__ gmask, const DcnDims s, const unsigned *__restrict__ bounds,
    T *__restrict__ col, const long qp) {
  using M = Mfma<T>;
  using P = typename std::conditional<(sizeof(T) == 2), float, double>::type;  // position type
  constexpr int PC = M::kPiece, SL = 2 * PC, ES = sizeof(T);
  constexpr int CH = 32 / ES, CHUNKS = 16 / CH;  // channels of a lane per pass: 32 bytes per corner
  // LDS of a wavefront.  Gather stage: rows of 64 bytes (the two halves' 32 bytes of a corner) for 4
  // corners x 32 positions, 80 bytes apart so that the 16-byte reads of 8 lanes cover all banks.
  // The column block and the far corners' channels reuse the stage once x sits in registers; with
  // two passes per block (fp32) the column block outlives a pass and lies behind the stage.
  constexpr int kRow = 80, kStage = 4 * 32 * kRow;
  constexpr int kColAt = CHUNKS > 1 ? kStage : 0, kFarAt = CHUNKS > 1 ? 0 : 4096;
  constexpr int kListAt = kStage + (CHUNKS > 1 ? 32 * 32 * ES : 0), kTapsAt = kListAt + 256 * 8;
  constexpr int kWaveBytes = kTapsAt + 32 * 32;
  static_assert(32 * 32 * ES <= 4096 && 4096 + 32 * 33 * 4 <= kStage, "column block and far channels fit the stage");
  __shared__ __attribute__((aligned(16))) unsigned char lds[4][kWaveBytes];
  const int lane = threadIdx.x % kWave, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int n = lane % 32, h = lane / 32;
  const long q0 = (static_cast<long>(xcd_contiguous(blockIdx.x, gridDim.x)) * 4 + wave) * 32;
  if (q0 >= s.Q) return;  // whole wavefront idle (no workgroup barriers in this kernel)
  const long q = q0 + n;
  const bool live = q < s.Q;
  const long qc = live ? q : s.Q - 1;
  const int dgi = blockIdx.y, b = blockIdx.z;
  const int ow = qc % s.Wo, oh = (qc / s.Wo) % s.Ho, od = qc / (static_cast<long>(s.Wo) * s.Ho);
  const int bd = od * s.sd - s.pd, bh = oh * s.sh - s.ph, bw = ow * s.sw - s.pw;
  const long bg = static_cast<long>(b) * s.dg + dgi;
  const int cblocks = s.cpg / 32, steps = s.opg / SL;

  const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(xt + static_cast<long>(b) * s.P * s.Cin), 0, static_cast<int>(s.P * s.Cin * ES), kRsrcFlags);
  const __amdgpu_buffer_rsrc_t gr = __builtin_amdgcn_make_buffer_rsrc(
      gxt + static_cast<long>(b) * s.P * s.Cin, 0, static_cast<int>(s.P * s.Cin * 4), kRsrcFlags);
  const unsigned cin2 = static_cast<unsigned>(s.Cin) * ES;
  const T *gyrow = gyt + (static_cast<long>(b) * s.Q + qc) * s.Cout + h * PC;
  const T *o = off + bg * s.nd * s.K * s.Q + qc;
  const T *mk = mask ? mask + bg * s.K * s.Q + qc : nullptr;
  unsigned char *const stg = lds[wave];
  float *const fg = reinterpret_cast<float *>(stg + kFarAt);
  T *const cs = reinterpret_cast<T *>(stg + kColAt);
  uint2 *const fl = reinterpret_cast<uint2 *>(stg + kListAt);  // per far (position, corner): {offset in the gradient buffer | position, weight}
  unsigned char *const tp = stg + kTapsAt;                     // the corners' byte offsets in x: [position][8]
  const TileOrigin origin = tile_origin<S>(s, od / S::BD, oh / S::BH, ow / S::BW);
  const bool split = scatter_scale(bounds, S::BD * S::BH * S::BW * s.K, mask != nullptr).valid;
  // the gather fetches a voxel's 64 bytes with four adjacent lanes (one request instead of four):
  // lane l fetches quarter l % 4 of the voxels of positions l / 4 and l / 4 + 16
  const int gp = lane / 4, gq = lane % 4;
  const unsigned gbyte = static_cast<unsigned>((gq / 2) * (16 * ES) + (gq % 2) * 16);
  // grad_output of the lane's position does not change with the tap: kept when the deformable
  // group lies in one weight group and the slices fit four registers each
  const bool hoist = s.cpd <= s.cpg && steps <= 4;
  u32x4 bkeep[4];
#pragma unroll
  for (int st = 0; st < 4; st++)
    bkeep[st] = (hoist && live && st < steps)
                    ? *reinterpret_cast<const u32x4 *>(gyrow + (dgi * s.cpd / s.cpg) * s.opg + st * SL)
                    : u32x4{0u, 0u, 0u, 0u};

  int ki = 0, kj = 0, kk = 0;
  P fd, fh, fw;  // offsets and mask of the coming tap, loaded one tap ahead
  dcn_offsets(s, o, fd, fh, fw);
  float fm = mk ? load(mk) : 1.f;
  for (int k = 0; k < s.K; k++) {
    // ---- taps of (k, q0 + n), in the lane's registers ---------------------------------------------
    const P pd = fd + static_cast<P>(bd + ki * s.dd), ph = fh + static_cast<P>(bh + kj * s.dh),
            pw = fw + static_cast<P>(bw + kk * s.dw);
    const float m = fm;
    o += s.nd * s.Q;
    if (mk) mk += s.Q;
    if (++kk == s.kw) { kk = 0; if (++kj == s.kh) { kj = 0; ++ki; } }
    if (k + 1 < s.K) {
      dcn_offsets(s, o, fd, fh, fw);
      if (mk) fm = load(mk);
    }
    CornerTaps t;  // byte offsets of the corners in x; kOob outside the volume
    corner_taps<P>(s, pd, ph, pw, live, cin2, 0u, kOob, t);
    int first;
    const unsigned local = split ? tile_bits<S>(origin, static_cast<int>(floor(pd)), static_cast<int>(floor(ph)),
                                             static_cast<int>(floor(pw)), first) : 0u;
    unsigned farbits = 0;  // corners inside the volume that the scatter kernel does not sum
#pragma unroll
    for (int c = 0; c < 8; c++) farbits |= (t.at[c] != kOob && !((local >> c) & 1u)) ? 1u << c : 0u;
    const float ld = t.ld, lh = t.lh, lw = t.lw;
    if (h == 0) {
      reinterpret_cast<u32x4 *>(tp + n * 32)[0] = u32x4{t.at[0], t.at[1], t.at[2], t.at[3]};
      reinterpret_cast<u32x4 *>(tp + n * 32)[1] = u32x4{t.at[4], t.at[5], t.at[6], t.at[7]};
    }
    // the far corners of the wavefront's 32 positions, listed once per tap: a voxel's channels start
    // at a multiple of 128 bytes, so the position fits below the offset.  Both half-wavefronts hold
    // the same taps; the lower one writes.
    int far_count = 0;
    if (__ballot(farbits != 0) != 0) {
      const float wd[2] = {1.f - ld, ld}, wh[2] = {1.f - lh, lh}, ww[2] = {1.f - lw, lw};
#pragma unroll
      for (int c = 0; c < 8; c++) {
        const bool is_far = (farbits >> c) & 1u;
        const unsigned owners = static_cast<unsigned>(__ballot(is_far));  // low 32 bits: the positions
        if (is_far && h == 0)
          fl[far_count + __builtin_amdgcn_mbcnt_lo(owners, 0u)] =
              make_uint2(t.at[c] * (4u / ES) | static_cast<unsigned>(n),
                         __float_as_uint(wd[c >> 2] * wh[(c >> 1) & 1] * ww[c & 1]));
        far_count += __builtin_popcount(owners);
      }
    }
    const bool any_far = far_count != 0;
    float t0 = 0.f, t1 = 0.f, t2 = 0.f, t3 = 0.f;  // sums over the lane's channels of gcol * {dZ/dd, dZ/dh, dZ/dw, Z}
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    for (int cc = 0; cc < s.cpd / 32; cc++) {
      const int c0 = dgi * s.cpd + cc * 32, g = c0 / s.cpg, cb = (c0 - g * s.cpg) / 32;
      // x at the 8 corners, the lane's 32 bytes each: fetched a voxel per four lanes, passed through
      // the stage four corners at a time
      u32x4 xv[8][2];
      auto gather = [&](int chunk) {
        const unsigned cbyte = static_cast<unsigned>(c0) * ES + gbyte + static_cast<unsigned>(chunk * 32);
        u32x4 raw[2][2][4];
#pragma unroll
        for (int r = 0; r < 2; r++)
#pragma unroll
          for (int p = 0; p < 2; p++) {
            const u32x4 at4 = *reinterpret_cast<const u32x4 *>(tp + (gp + 16 * p) * 32 + r * 16);
#pragma unroll
            for (int c4 = 0; c4 < 4; c4++)
              raw[r][p][c4] = __builtin_amdgcn_raw_buffer_load_b128(xr, at4[c4] + cbyte, 0, 0);  // kOob + small: reads 0
          }
#pragma unroll
        for (int r = 0; r < 2; r++) {
#pragma unroll
          for (int p = 0; p < 2; p++)
#pragma unroll
            for (int c4 = 0; c4 < 4; c4++)
              *reinterpret_cast<u32x4 *>(stg + (c4 * 32 + gp + 16 * p) * kRow + gq * 16) = raw[r][p][c4];
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
          for (int c4 = 0; c4 < 4; c4++)
#pragma unroll
            for (int j = 0; j < 2; j++)
              xv[4 * r + c4][j] = *reinterpret_cast<const u32x4 *>(stg + (c4 * 32 + n) * kRow + 32 * h + 16 * j);
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
      };
      // ---- gcol[32 channels x 32 positions] = Wt_k^T[32 x opg] * gy^T[opg x 32] -------------------
      float16_t acc;
#pragma unroll
      for (int r = 0; r < 16; r++) acc[r] = 0.f;
      const T *wfrag = wa + ((((static_cast<long>(g) * s.K + k) * cblocks + cb) * steps) * 64 + lane) * PC;
      const T *brow = gyrow + g * s.opg;
#pragma unroll
      for (int st = 0; st < 4; st++)
        if (st < steps) {
          const u32x4 af = *reinterpret_cast<const u32x4 *>(wfrag + static_cast<long>(st) * (64 * PC));
          const u32x4 bf = hoist ? bkeep[st]
                                 : (live ? *reinterpret_cast<const u32x4 *>(brow + st * SL) : u32x4{0u, 0u, 0u, 0u});
          acc = M::run(af, bf, acc);
        }
      for (int st = 4; st < steps; st++) {
        const u32x4 af = *reinterpret_cast<const u32x4 *>(wfrag + static_cast<long>(st) * (64 * PC));
        const u32x4 bf = live ? *reinterpret_cast<const u32x4 *>(brow + st * SL) : u32x4{0u, 0u, 0u, 0u};
        acc = M::run(af, bf, acc);
      }
#pragma unroll
      for (int chunk = 0; chunk < CHUNKS; chunk++) {
        gather(chunk);
#pragma unroll
        for (int i = 0; i < CH; i++) {
          const int r = chunk * CH + i;  // channel c0 + 16 * h + r
          float v[8];
#pragma unroll
          for (int c = 0; c < 8; c++) {
            if constexpr (ES == 4) {
              v[c] = __uint_as_float(xv[c][i / 4][i % 4]);
            } else {
              const unsigned word = xv[c][i / 8][(i % 8) / 2];
              v[c] = (i % 2) ? M::hi(word) : M::lo(word);
            }
          }
          // value and the three partial derivatives of the trilinear form, sharing the differences
          const float x0 = v[1] - v[0], x1 = v[3] - v[2], x2 = v[5] - v[4], x3 = v[7] - v[6];
          const float a0 = fmaf(lw, x0, v[0]), a1 = fmaf(lw, x1, v[2]), a2 = fmaf(lw, x2, v[4]), a3 = fmaf(lw, x3, v[6]);
          const float b0 = fmaf(lh, x1 - x0, x0), b1 = fmaf(lh, x3 - x2, x2);
          const float dw = fmaf(ld, b1 - b0, b0);
          const float y0 = a1 - a0, y1 = a3 - a2;
          const float c0v = fmaf(lh, y0, a0), c1v = fmaf(lh, y1, a2);
          const float dh = fmaf(ld, y1 - y0, y0);
          const float dd = c1v - c0v;
          const float val = fmaf(ld, dd, c0v);
          const float gc = acc[r];
          t0 = fmaf(dd, gc, t0); t1 = fmaf(dh, gc, t1); t2 = fmaf(dw, gc, t2); t3 = fmaf(val, gc, t3);
          // column value of (channel 16 * h + r, position n), pieces [position / kPiece][channel][kPiece]
          cs[((n / PC) * 32 + 16 * h + r) * PC + n % PC] = store_cast<T>(m * val);
          // one channel at a time, its sums formed here (left alone the compiler moves the sums
          // behind the stores below and keeps every channel's differences alive until then)
          asm volatile("" : "+v"(t0), "+v"(t1), "+v"(t2), "+v"(t3));
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if (any_far) {
#pragma unroll
        for (int r = 0; r < 16; r++) fg[n * 33 + 16 * h + r] = acc[r] * m;
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      if (col) {
        // the wavefront's block of the column buffer is contiguous: 32 positions x 32 channels
        T *dst = col + ((static_cast<long>(b) * s.K + k) * (s.Cin / 32) + c0 / 32) * qp * 32 + q0 * 32 + lane * 16;
#pragma unroll
        for (int j = 0; j < ES; j++) {
          const u32x4 piece = *reinterpret_cast<const u32x4 *>(cs + lane * 16 + j * (16 / ES));
          // (nontemporal: the buffer is larger than the caches and read once, by the weight kernel)
          __builtin_nontemporal_store(piece, reinterpret_cast<u32x4 *>(dst + j * (16 / ES)));
        }
      }
      if (any_far) {
        // the lower half adds the 32 channels of list entry i, the upper half those of entry i + 1
        const unsigned cbyte4 = static_cast<unsigned>(c0 + n) * 4u;
        // (four entries per turn, so that the LDS reads of one overlap those of the other)
        for (int i = h; i < far_count; i += 4) {
          const bool two = i + 2 < far_count;
          const uint2 e0 = fl[i], e1 = fl[min(i + 2, 255)];
          const float g0 = fg[(e0.x & 31u) * 33 + n], g1 = fg[(e1.x & 31u) * 33 + n];
          __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(__uint_as_float(e0.y) * g0, gr, (e0.x & ~127u) + cbyte4, 0, 0);
          __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(__uint_as_float(e1.y) * g1, gr,
                                                          two ? (e1.x & ~127u) + cbyte4 : kOob, 0, 0);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    // ---- the other half-wavefront's sixteen channels, then grad offset / grad mask -----------------
    t0 += __shfl_xor(t0, 32); t1 += __shfl_xor(t1, 32); t2 += __shfl_xor(t2, 32); t3 += __shfl_xor(t3, 32);
    if (h == 0 && live) {
      T *go = goff + (bg * s.nd * s.K + s.nd * k) * s.Q + q;
      if (s.nd == 3) go[0] = store_cast<T>(m * t0);
      go[(s.nd - 2) * s.Q] = store_cast<T>(m * t1); go[(s.nd - 1) * s.Q] = store_cast<T>(m * t2);
      if (gmask) gmask[(bg * s.K + k) * s.Q + q] = store_cast<T>(t3);
    }
  }
}

// ---- gradient of the input, local corners: summed in LDS, then added to the buffer ----------------
// A workgroup owns a brick of positions and eight channels; its sixteen wavefronts are kScatterSplit
// groups of eight, every group covers the positions of the brick (32 per wavefront at a time) and
// takes a contiguous share of the taps.  gcol comes from the 16 x 16 MFMA with the channels as
// rows: lane l holds position l % 16 of a 16-position block and the channels l / 16 and l / 16 + 4,
// so one LDS add instruction covers 16 positions x 4 adjacent channels; a voxel's 8 sums are 9
// qwords apart from the next voxel's to spread the banks.  After the taps the tile's non-zero sums are converted and added
// to the gradient buffer: one global atomic per (voxel, channel) of the tile instead of one per
// (position, tap, corner, channel).
constexpr int kScatterSplit = 2, kScatterWaves = 8 * kScatterSplit, kScatterStride = 9;
constexpr int kScatterKeep = 4;  // slices of grad_output a wavefront keeps in registers over the taps (all of them)

// weight [Cout, cpg, K] -> A pieces [group][tap][8-channel block][row step][lane][kPiece]: lane l
// is MFMA row l % 16 = channel (row / 4) + 4 * (row % 2) of the block (rows 4j + 2, 4j + 3 repeat
// rows 4j, 4j + 1 and are not used), element i the output channel g*opg + step*4*kPiece +
// (l/16)*kPiece + i
template <typename T>
__device__ __forceinline__ void dcn_weight_afragments8_block(const T *__restrict__ wt, T *__restrict__ wa, const DcnDims s, const unsigned bid) {
  constexpr int PC = Mfma<T>::kPiece;
  const int cblocks = s.cpg / 8, steps = s.opg / (4 * PC);
  const long total = static_cast<long>(s.groups) * s.K * cblocks * steps * 64;
  const long id = bid * 256L + threadIdx.x;
  if (id >= total) return;
  const int lane = id % 64;
  long r = id / 64;
  const int st = r % steps; r /= steps;
  const int cb = r % cblocks; r /= cblocks;
  const int k = r % s.K;
  const int g = static_cast<int>(r / s.K);
  const int row = lane % 16, cl = cb * 8 + row / 4 + 4 * (row % 2);
  const int o = g * s.opg + st * 4 * PC + (lane / 16) * PC;
  for (int i = 0; i < PC; i++) wa[id * PC + i] = wt[(static_cast<long>(o + i) * s.cpg + cl) * s.K + k];
}
template <typename T>
__global__ __launch_bounds__(256) void dcn_weight_afragments8_kernel(const T *__restrict__ wt,
                                                                     T *__restrict__ wa,
                                                                     const DcnDims s) { dcn_weight_afragments8_block<T>(wt, wa, s, blockIdx.x); }

template <typename T, typename S>
__global__ __launch_bounds__(kScatterWaves * 64) void dcn_backward_scatter_kernel(
    const T *__restrict__ off, const T *__restrict__ mask, const T *__restrict__ gyt,
    const T *__restrict__ wa, float *__restrict__ gxt, const DcnDims s, const int nbh, const int nbw,
    const unsigned *__restrict__ bounds) {
  using M = Mfma<T>;
  using P = typename std::conditional<(sizeof(T) == 2), float, double>::type;
  constexpr int PC = M::kPiece, SL = 4 * PC;
  constexpr int VOX = S::TD * S::TH * S::TW;
  constexpr int GROUPS = S::BD * S::BH * S::BW / 32;  // 32-position groups of the brick
  static_assert(VOX <= kTileVoxMax && GROUPS % 8 == 0, "brick and tile sizes");
  __shared__ unsigned long long tile[VOX * kScatterStride];
  __shared__ __attribute__((aligned(16))) float recs[kScatterWaves][32][8];
  const ScatterScale scale = scatter_scale(bounds, S::BD * S::BH * S::BW * s.K, mask != nullptr);
  if (!scale.valid) return;  // every corner went through the data kernel
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int n = lane % 32, p16 = lane % 16, j = lane / 16;
  const int tg = wave / 8;
  const unsigned brick = xcd_contiguous(blockIdx.x, gridDim.x);
  const int bx = brick % nbw, by = (brick / nbw) % nbh, bz = brick / (nbw * nbh);
  const int c0 = blockIdx.y * 8, b = blockIdx.z;
  const int dgi = c0 / s.cpd, g = c0 / s.cpg, cb = (c0 - g * s.cpg) / 8;
  const long bg = static_cast<long>(b) * s.dg + dgi;
  const int cblocks = s.cpg / 8, steps = s.opg / SL;
  const TileOrigin origin = tile_origin<S>(s, bz, by, bx);

  for (int i = threadIdx.x; i < VOX * kScatterStride; i += kScatterWaves * 64) tile[i] = 0ull;
  __syncthreads();

  // position of brick index i, columns fastest
  auto position = [&](int i, bool &live) {
    const int od = bz * S::BD + i / (S::BH * S::BW), oh = by * S::BH + (i / S::BW) % S::BH, ow = bx * S::BW + i % S::BW;
    live = od < s.Do && oh < s.Ho && ow < s.Wo;
    return (static_cast<long>(min(od, s.Do - 1)) * s.Ho + min(oh, s.Ho - 1)) * s.Wo + min(ow, s.Wo - 1);
  };
  for (int pg = wave % 8; pg < GROUPS; pg += 8) {
  // the lane's own position for the taps (both halves of the wavefront compute them)
  bool live;
  const long q = position(pg * 32 + n, live);
  const int ow = q % s.Wo, oh = (q / s.Wo) % s.Ho, od = q / (static_cast<long>(s.Wo) * s.Ho);
  const int bd = od * s.sd - s.pd, bh = oh * s.sh - s.ph, bw = ow * s.sw - s.pw;
  // grad_output of the lane's column in the two 16-position blocks (MFMA B operand)
  bool blive[2];
  const T *grow[2];
  u32x4 keep[2][kScatterKeep];
#pragma unroll
  for (int blk = 0; blk < 2; blk++) {
    const long qb = position(pg * 32 + blk * 16 + p16, blive[blk]);
    grow[blk] = gyt + (static_cast<long>(b) * s.Q + qb) * s.Cout + g * s.opg + j * PC;
#pragma unroll
    for (int st = 0; st < kScatterKeep; st++)
      keep[blk][st] = (blive[blk] && st < steps) ? *reinterpret_cast<const u32x4 *>(grow[blk] + st * SL)
                                                : u32x4{0u, 0u, 0u, 0u};
  }
  const int per = (s.K + kScatterSplit - 1) / kScatterSplit, k0 = min(tg * per, s.K), k1 = min(s.K, k0 + per);
  const T *o = off + (bg * s.nd * s.K + static_cast<long>(s.nd) * k0) * s.Q + q;
  const T *mk = mask ? mask + (bg * s.K + k0) * s.Q + q : nullptr;
  float(*rec)[8] = recs[wave];

  int ki = k0 / (s.kh * s.kw), kj = (k0 / s.kw) % s.kh, kk = k0 % s.kw;
  P fd = P(0), fh = P(0), fw = P(0);
  float fm = 1.f;
  if (k0 < k1) {
    dcn_offsets(s, o, fd, fh, fw);
    if (mk) fm = load(mk);
  }
  // weight pieces of the current tap, loaded one tap ahead
  const long tap_stride = static_cast<long>(cblocks) * steps * 64 * PC;
  const T *afrag = wa + (((static_cast<long>(g) * s.K + k0) * cblocks + cb) * steps * 64 + lane) * PC;
  u32x4 wcur[kScatterKeep];
#pragma unroll
  for (int st = 0; st < kScatterKeep; st++)
    wcur[st] = (k0 < k1 && st < steps) ? *reinterpret_cast<const u32x4 *>(afrag + static_cast<long>(st) * (64 * PC))
                                       : u32x4{0u, 0u, 0u, 0u};
  for (int k = k0; k < k1; k++) {
    u32x4 wnext[kScatterKeep];
#pragma unroll
    for (int st = 0; st < kScatterKeep; st++)
      wnext[st] = (k + 1 < k1 && st < steps)
                      ? *reinterpret_cast<const u32x4 *>(afrag + tap_stride + static_cast<long>(st) * (64 * PC))
                      : u32x4{0u, 0u, 0u, 0u};
    {
      const P pd = fd + static_cast<P>(bd + ki * s.dd), ph = fh + static_cast<P>(bh + kj * s.dh),
              pw = fw + static_cast<P>(bw + kk * s.dw);
      const float m = fm;
      o += s.nd * s.Q;
      if (mk) mk += s.Q;
      if (++kk == s.kw) { kk = 0; if (++kj == s.kh) { kj = 0; ++ki; } }
      if (k + 1 < k1) {  // the next tap's offsets are in flight during this tap's adds
        dcn_offsets(s, o, fd, fh, fw);
        if (mk) fm = load(mk);
      }
      CornerTaps t;
      corner_taps<P>(s, pd, ph, pw, live, 1u, 0u, ~0u, t);
      int first;
      unsigned bits = tile_bits<S>(origin, static_cast<int>(floor(pd)), static_cast<int>(floor(ph)),
                                static_cast<int>(floor(pw)), first);
      unsigned inside = 0;
#pragma unroll
      for (int c = 0; c < 8; c++) inside |= t.at[c] != ~0u ? 1u << c : 0u;
      bits &= inside;
      if (lane < 32) {
        float4 *dst = reinterpret_cast<float4 *>(rec[n]);
        dst[0] = make_float4(__int_as_float(first), __uint_as_float(bits), m, t.ld);
        dst[1] = make_float4(t.lh, t.lw, 0.f, 0.f);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    float4_t acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int st = 0; st < kScatterKeep; st++)
      if (st < steps) {
        acc[0] = M::run16(wcur[st], keep[0][st], acc[0]);
        acc[1] = M::run16(wcur[st], keep[1][st], acc[1]);
      }
#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
      const float4 *src = reinterpret_cast<const float4 *>(rec[blk * 16 + p16]);
      const float4 ra = src[0], rb = src[1];
      const int first = __float_as_int(ra.x);
      const unsigned bits = __float_as_uint(ra.y);
      // the lane's two channels, times the mask and the fixed-point scale
      const double gv[2] = {static_cast<double>(acc[blk][0] * ra.z) * scale.up,
                            static_cast<double>(acc[blk][1] * ra.z) * scale.up};
      const float wd[2] = {1.f - ra.w, ra.w}, wh[2] = {1.f - rb.x, rb.x}, ww[2] = {1.f - rb.y, rb.y};
      // the lane's qword of the first corner, as a 32-bit byte offset worked out once: the corners
      // differ by constants that go into the instructions' offset fields
      char *const cell0 = reinterpret_cast<char *>(tile) + (static_cast<unsigned>(first) * kScatterStride + j) * 8u;
#pragma unroll
      for (int c = 0; c < 8; c++) {
        const int ca = c >> 2, cb2 = (c >> 1) & 1, ce = c & 1;
        if ((S::TD > 1 || ca == 0) && ((bits >> c) & 1u)) {  // images have no second slice
          const float wc = wd[ca] * wh[cb2] * ww[ce];
          unsigned long long *dst = reinterpret_cast<unsigned long long *>(
              cell0 + (ca * (S::TH * S::TW) + cb2 * S::TW + ce) * (kScatterStride * 8));
#pragma unroll
          for (int r = 0; r < 2; r++)
            __hip_atomic_fetch_add(dst + 4 * r, fixed_term(wc, gv[r]), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_WORKGROUP);
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    afrag += tap_stride;
#pragma unroll
    for (int st = 0; st < kScatterKeep; st++) wcur[st] = wnext[st];
  }
  }
  __syncthreads();
  // ---- the tile's voxels inside the volume go to the gradient buffer, 8 channels per voxel --------
  const __amdgpu_buffer_rsrc_t gr = __builtin_amdgcn_make_buffer_rsrc(
      gxt + static_cast<long>(b) * s.P * s.Cin, 0, static_cast<int>(s.P * s.Cin * 4), kRsrcFlags);
  const unsigned cin4 = static_cast<unsigned>(s.Cin) * 4u;
  const int ch = threadIdx.x % 8;
  for (int cell = threadIdx.x / 8; cell < VOX; cell += kScatterWaves * 8) {
    const int zw = cell % S::TW + origin.w, zh = (cell / S::TW) % S::TH + origin.h, zd = cell / (S::TW * S::TH) + origin.d;
    const unsigned long long sum = tile[cell * kScatterStride + ch];
    if (zd >= 0 && zd < s.D && zh >= 0 && zh < s.H && zw >= 0 && zw < s.W && sum != 0ull) {
      const double v = static_cast<double>(static_cast<long long>(sum)) * scale.down;
      __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(
          static_cast<float>(v), gr,
          static_cast<unsigned>((zd * s.H + zh) * s.W + zw) * cin4 + static_cast<unsigned>(c0 + ch) * 4u, 0, 0);
    }
  }
}

// ---- the same sums in 32-bit cells, for 16-bit tensors ---------------------------------------------
// A workgroup owns a brick and SIXTEEN channels (all 16 rows of the 16 x 16 MFMA): the taps, the
// records and grad_output serve twice the channels, an LDS add moves 4 bytes instead of 8 and a term
// costs one fma and one subtraction.  32 bits leave 30 - ceil(log2(positions * taps)) bits for a
// term (17 for 3 x 3 x 3 taps), so the scale comes from the data: a first sweep over the brick's
// taps forms gcol alone (matrix cores, no geometry) and takes max |gcol| of the workgroup; every
// term is then below max |gcol| * max |mask| < 2^ex and is rounded to a multiple of 2^(ex - shift)
// (adding 1.5 * 2^23 in fp32 leaves round(x) in the low mantissa bits for |x| < 2^22).  The error of
// a voxel's sum stays below terms * 2^(ex - shift - 1), about 2^-15 of the values it sums for the
// 3 x 3 x 3 layer — a sixteenth of the last bit of the 16-bit result.
constexpr int kScatter32Stride = 17;    // dwords between voxels: 16 channels and one to spread the banks
constexpr int kScatter32MinShift = 14;  // fewer bits per term: the 64-bit kernel takes the layer
__host__ __device__ constexpr int scatter32_shift(int terms) {
  int bits = 0;
  while ((1L << bits) < terms) bits++;
  return 30 - bits;
}

// weight [Cout, cpg, K] -> A pieces [group][tap][16-channel block][row step][lane][kPiece]: lane l is
// MFMA row l % 16 = channel l % 16 of the block, element i the output channel
// g*opg + step*4*kPiece + (l/16)*kPiece + i
template <typename T>
__device__ __forceinline__ void dcn_weight_afragments16_block(const T *__restrict__ wt, T *__restrict__ wa, const DcnDims s, const unsigned bid) {
  constexpr int PC = Mfma<T>::kPiece;
  const int cblocks = s.cpg / 16, steps = s.opg / (4 * PC);
  const long total = static_cast<long>(s.groups) * s.K * cblocks * steps * 64;
  const long id = bid * 256L + threadIdx.x;
  if (id >= total) return;
  const int lane = id % 64;
  long r = id / 64;
  const int st = r % steps; r /= steps;
  const int cb = r % cblocks; r /= cblocks;
  const int k = r % s.K;
  const int g = static_cast<int>(r / s.K);
  const int cl = cb * 16 + lane % 16;
  const int o = g * s.opg + st * 4 * PC + (lane / 16) * PC;
  for (int i = 0; i < PC; i++) wa[id * PC + i] = wt[(static_cast<long>(o + i) * s.cpg + cl) * s.K + k];
}
template <typename T>
__global__ __launch_bounds__(256) void dcn_weight_afragments16_kernel(const T *__restrict__ wt,
                                                                      T *__restrict__ wa,
                                                                      const DcnDims s) { dcn_weight_afragments16_block<T>(wt, wa, s, blockIdx.x); }

template <typename T, typename S>
__global__ __launch_bounds__(kScatterWaves * 64) void dcn_backward_scatter32_kernel(
    const T *__restrict__ off, const T *__restrict__ mask, const T *__restrict__ gyt,
    const T *__restrict__ wa, float *__restrict__ gxt, const DcnDims s, const int nbh, const int nbw,
    const unsigned *__restrict__ bounds) {
  using M = Mfma<T>;
  using P = typename std::conditional<(sizeof(T) == 2), float, double>::type;
  constexpr int PC = M::kPiece, SL = 4 * PC;
  constexpr int VOX = S::TD * S::TH * S::TW;
  constexpr int GROUPS = S::BD * S::BH * S::BW / 32;  // 32-position groups of the brick
  static_assert(VOX <= kTileVoxMax && GROUPS % 8 == 0, "brick and tile sizes");
  __shared__ int tile[VOX * kScatter32Stride];
  __shared__ __attribute__((aligned(8))) float recs[kScatterWaves][64][6];
  __shared__ unsigned wgmax;
  // (the validity of the data kernel's split: no NaN or infinity anywhere, products finite)
  if (!scatter_scale(bounds, S::BD * S::BH * S::BW * s.K, mask != nullptr).valid) return;
  const float mask_max = mask ? __uint_as_float(bounds[2]) : 1.f;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int n = lane % 32, p16 = lane % 16, j = lane / 16;
  const int tg = wave / 8;
  const unsigned brick = xcd_contiguous(blockIdx.x, gridDim.x);
  const int bx = brick % nbw, by = (brick / nbw) % nbh, bz = brick / (nbw * nbh);
  const int c0 = blockIdx.y * 16, b = blockIdx.z;
  const int dgi = c0 / s.cpd, g = c0 / s.cpg, cb = (c0 - g * s.cpg) / 16;
  const long bg = static_cast<long>(b) * s.dg + dgi;
  const int cblocks = s.cpg / 16, steps = s.opg / SL;
  const TileOrigin origin = tile_origin<S>(s, bz, by, bx);
  const int per = (s.K + kScatterSplit - 1) / kScatterSplit, k0 = min(tg * per, s.K), k1 = min(s.K, k0 + per);
  const long tap_stride = static_cast<long>(cblocks) * steps * 64 * PC;
  const T *afrag0 = wa + (((static_cast<long>(g) * s.K + k0) * cblocks + cb) * steps * 64 + lane) * PC;

  for (int i = threadIdx.x; i < VOX * kScatter32Stride; i += kScatterWaves * 64) tile[i] = 0;
  if (threadIdx.x == 0) wgmax = 0u;
  __syncthreads();

  // position of brick index i, columns fastest
  auto position = [&](int i, bool &live) {
    const int od = bz * S::BD + i / (S::BH * S::BW), oh = by * S::BH + (i / S::BW) % S::BH, ow = bx * S::BW + i % S::BW;
    live = od < s.Do && oh < s.Ho && ow < s.Wo;
    return (static_cast<long>(min(od, s.Do - 1)) * s.Ho + min(oh, s.Ho - 1)) * s.Wo + min(ow, s.Wo - 1);
  };
  // grad_output of the lane's column in the two 16-position blocks of a group (MFMA B operand)
  auto load_keep = [&](int pg, u32x4 (&keep)[2][kScatterKeep]) {
#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
      bool blive;
      const long qb = position(pg * 32 + blk * 16 + p16, blive);
      const T *grow = gyt + (static_cast<long>(b) * s.Q + qb) * s.Cout + g * s.opg + j * PC;
#pragma unroll
      for (int st = 0; st < kScatterKeep; st++)
        keep[blk][st] = (blive && st < steps) ? *reinterpret_cast<const u32x4 *>(grow + st * SL) : u32x4{0u, 0u, 0u, 0u};
    }
  };
  auto load_weights = [&](const T *afrag, bool on, u32x4 (&w)[kScatterKeep]) {
#pragma unroll
    for (int st = 0; st < kScatterKeep; st++)
      w[st] = (on && st < steps) ? *reinterpret_cast<const u32x4 *>(afrag + static_cast<long>(st) * (64 * PC))
                                 : u32x4{0u, 0u, 0u, 0u};
  };

  // ---- first sweep: max |gcol| over the brick's positions, the taps and the 16 channels -----------
  {
    float top = 0.f;
    for (int pg = wave % 8; pg < GROUPS; pg += 8) {
      u32x4 keep[2][kScatterKeep];
      load_keep(pg, keep);
      const T *afrag = afrag0;
      for (int k = k0; k < k1; k++) {
        u32x4 w[kScatterKeep];
        load_weights(afrag, true, w);
        afrag += tap_stride;
        float4_t acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int st = 0; st < kScatterKeep; st++)
          if (st < steps) {
            acc[0] = M::run16(w[st], keep[0][st], acc[0]);
            acc[1] = M::run16(w[st], keep[1][st], acc[1]);
          }
#pragma unroll
        for (int i = 0; i < 4; i++) top = fmaxf(top, fmaxf(fabsf(acc[0][i]), fabsf(acc[1][i])));
      }
    }
    for (int sh = 32; sh > 0; sh >>= 1) top = fmaxf(top, __shfl_xor(top, sh));
    if (lane == 0 && top > 0.f) atomicMax(&wgmax, __float_as_uint(top));
  }
  __syncthreads();
  const float bound = fmaxf(1.001f * __uint_as_float(wgmax), 1e-30f) * mask_max;
  if (!(bound > 0.f)) return;  // nothing but zeros to add (the whole workgroup leaves together)
  const int shift = scatter32_shift(S::BD * S::BH * S::BW * s.K);
  int ex = 0;
  frexpf(bound, &ex);  // bound < 2^ex
  const float up = ldexpf(1.f, shift - ex), down = ldexpf(1.f, ex - shift);
  constexpr float kMagic = 12582912.f;  // 1.5 * 2^23

  for (int pg = wave % 8; pg < GROUPS; pg += 8) {
  // the taps are worked out two at a time: the lower half-wavefront takes tap k of the group's 32
  // positions, the upper half tap k + 1
  const int hh = lane / 32;
  bool live;
  const long q = position(pg * 32 + n, live);
  const int ow = q % s.Wo, oh = (q / s.Wo) % s.Ho, od = q / (static_cast<long>(s.Wo) * s.Ho);
  const int bd = od * s.sd - s.pd, bh = oh * s.sh - s.ph, bw = ow * s.sw - s.pw;
  u32x4 keep[2][kScatterKeep];
  load_keep(pg, keep);
  int kt = k0 + hh;  // the lane's own tap
  const T *o = off + (bg * s.nd * s.K + static_cast<long>(s.nd) * kt) * s.Q + q;
  const T *mk = mask ? mask + (bg * s.K + kt) * s.Q + q : nullptr;
  float(*rec)[6] = recs[wave];

  int ki = kt / (s.kh * s.kw), kj = (kt / s.kw) % s.kh, kk = kt % s.kw;
  P fd = P(0), fh = P(0), fw = P(0);
  float fm = 1.f;
  if (kt < k1) {
    dcn_offsets(s, o, fd, fh, fw);
    if (mk) fm = load(mk);
  }
  const T *afrag = afrag0;
  for (int k = k0; k < k1; k += 2) {
    // weight pieces of the two taps (the taps' geometry below hides their latency)
    u32x4 wpair[2][kScatterKeep];
    load_weights(afrag, true, wpair[0]);
    load_weights(afrag + tap_stride, k + 1 < k1, wpair[1]);
    {
      const P pd = fd + static_cast<P>(bd + ki * s.dd), ph = fh + static_cast<P>(bh + kj * s.dh),
              pw = fw + static_cast<P>(bw + kk * s.dw);
      const float m = fm;
      const bool tap_on = kt < k1;
      kt += 2;
      o += 2 * s.nd * s.Q;
      if (mk) mk += 2 * s.Q;
#pragma unroll
      for (int u = 0; u < 2; u++)
        if (++kk == s.kw) { kk = 0; if (++kj == s.kh) { kj = 0; ++ki; } }
      if (kt < k1) {  // the next pair's offsets are in flight during this pair's adds
        dcn_offsets(s, o, fd, fh, fw);
        if (mk) fm = load(mk);
      }
      CornerTaps t;
      corner_taps<P>(s, pd, ph, pw, live && tap_on, 1u, 0u, ~0u, t);
      int first;
      unsigned bits = tile_bits<S>(origin, static_cast<int>(floor(pd)), static_cast<int>(floor(ph)),
                                static_cast<int>(floor(pw)), first);
      unsigned inside = 0;
#pragma unroll
      for (int c = 0; c < 8; c++) inside |= t.at[c] != ~0u ? 1u << c : 0u;
      bits &= inside;
      float2 *dst = reinterpret_cast<float2 *>(rec[lane]);
      dst[0] = make_float2(__int_as_float(first), __uint_as_float(bits));
      dst[1] = make_float2(m * up, t.ld);
      dst[2] = make_float2(t.lh, t.lw);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

#pragma unroll
    for (int u = 0; u < 2; u++) {
      if (k + u >= k1) break;
      float4_t acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
      for (int st = 0; st < kScatterKeep; st++)
        if (st < steps) {
          acc[0] = M::run16(wpair[u][st], keep[0][st], acc[0]);
          acc[1] = M::run16(wpair[u][st], keep[1][st], acc[1]);
        }
#pragma unroll
      for (int blk = 0; blk < 2; blk++) {
        const float2 *src = reinterpret_cast<const float2 *>(rec[u * 32 + blk * 16 + p16]);
        const float2 ra = src[0], rb = src[1], rc = src[2];
        const int first = __float_as_int(ra.x);
        const unsigned bits = __float_as_uint(ra.y);
        // the lane's four channels 4j .. 4j + 3, times the mask and the fixed-point scale
        const float gv[4] = {acc[blk][0] * rb.x, acc[blk][1] * rb.x, acc[blk][2] * rb.x, acc[blk][3] * rb.x};
        const float wd[2] = {1.f - rb.y, rb.y}, wh[2] = {1.f - rc.x, rc.x}, ww[2] = {1.f - rc.y, rc.y};
        // the lane's first dword of the first corner, as a 32-bit byte offset worked out once: the
        // corners and channels differ by constants that go into the instructions' offset fields
        char *const cell0 = reinterpret_cast<char *>(tile) + (static_cast<unsigned>(first) * kScatter32Stride + 4 * j) * 4u;
#pragma unroll
        for (int c = 0; c < 8; c++) {
          const int ca = c >> 2, cb2 = (c >> 1) & 1, ce = c & 1;
          if ((S::TD > 1 || ca == 0) && ((bits >> c) & 1u)) {  // images have no second slice
            const float wc = wd[ca] * wh[cb2] * ww[ce];
            int *dst = reinterpret_cast<int *>(cell0 + (ca * (S::TH * S::TW) + cb2 * S::TW + ce) * (kScatter32Stride * 4));
#pragma unroll
            for (int r = 0; r < 4; r++)
              __hip_atomic_fetch_add(dst + r, __float_as_int(fmaf(wc, gv[r], kMagic)) - 0x4B400000, __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_WORKGROUP);
          }
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    afrag += 2 * tap_stride;
  }
  }
  __syncthreads();
  // ---- the tile's voxels inside the volume go to the gradient buffer, 16 channels per voxel -------
  const __amdgpu_buffer_rsrc_t gr = __builtin_amdgcn_make_buffer_rsrc(
      gxt + static_cast<long>(b) * s.P * s.Cin, 0, static_cast<int>(s.P * s.Cin * 4), kRsrcFlags);
  const unsigned cin4 = static_cast<unsigned>(s.Cin) * 4u;
  const int ch = threadIdx.x % 16;
  for (int cell = threadIdx.x / 16; cell < VOX; cell += kScatterWaves * 4) {
    const int zw = cell % S::TW + origin.w, zh = (cell / S::TW) % S::TH + origin.h, zd = cell / (S::TW * S::TH) + origin.d;
    const int sum = tile[cell * kScatter32Stride + ch];
    if (zd >= 0 && zd < s.D && zh >= 0 && zh < s.H && zw >= 0 && zw < s.W && sum != 0)
      __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(
          static_cast<float>(sum) * down, gr,
          static_cast<unsigned>((zd * s.H + zh) * s.W + zw) * cin4 + static_cast<unsigned>(c0 + ch) * 4u, 0, 0);
  }
}

// ---- grad wrt weight ---------------------------------------------------------------------------
constexpr int kGwChunk = 2048;  // positions per workgroup

template <typename T, int MT>
__global__ __launch_bounds__(256) void dcn_backward_weight_mfma_kernel(
    const T *__restrict__ xt, const T *__restrict__ off, const T *__restrict__ mask,
    const T *__restrict__ gy, float *__restrict__ gw, const DcnDims s, const int mb0) {
  using M = Mfma<T>;
  using P = typename std::conditional<(sizeof(T) == 2), float, double>::type;  // position type
  constexpr int PC = M::kPiece, SL = 2 * PC, ES = sizeof(T);
  __shared__ __attribute__((aligned(16))) float taps[4][64][16];  // byte offsets in x [8], w[8] * mask
  __shared__ float part[3][MT][16][64];                           // accumulators of wavefronts 1..3
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int n = lane % 32, h = lane / 32;
  const int cblocks_all = s.Cin / 32;
  const int k = blockIdx.x % s.K, cbi = blockIdx.x / s.K;  // tap, 32-channel block of the layer
  const int c0 = cbi * 32, g = c0 / s.cpg, dgi = c0 / s.cpd;
  const int b = blockIdx.z;
  const long qbase = static_cast<long>(blockIdx.y) * kGwChunk;
  const long bg = static_cast<long>(b) * s.dg + dgi;
  const int ki = k / (s.kh * s.kw), kj = (k / s.kw) % s.kh, kk = k % s.kw;
  const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(xt + static_cast<long>(b) * s.P * s.Cin), 0, static_cast<int>(s.P * s.Cin * ES), kRsrcFlags);
  const unsigned cbyte2 = static_cast<unsigned>(c0 + n) * ES, cin2 = static_cast<unsigned>(s.Cin) * ES;
  const T *ob = off + (bg * s.nd * s.K + s.nd * k) * s.Q;
  const T *mb_ = mask ? mask + (bg * s.K + k) * s.Q : nullptr;
  const bool aligned = s.Q % PC == 0;
  float(*tp)[16] = taps[wave];
  (void)cblocks_all;

  float16_t acc[MT];
#pragma unroll
  for (int m = 0; m < MT; m++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[m][r] = 0.f;

  const long qend = min(qbase + kGwChunk, s.Q);
  for (long qg = qbase + wave * 64; qg < qend; qg += 256) {
    // ---- taps of the 64 positions qg + lane ------------------------------------------------------
    {
      const long q = qg + lane;
      const bool live = q < s.Q;
      const long qc = live ? q : s.Q - 1;
      const int ow = qc % s.Wo, oh = (qc / s.Wo) % s.Ho, od = qc / (static_cast<long>(s.Wo) * s.Ho);
      P pd, ph, pw;
      dcn_offsets(s, ob + qc, pd, ph, pw);
      pd += static_cast<P>(od * s.sd - s.pd + ki * s.dd); ph += static_cast<P>(oh * s.sh - s.ph + kj * s.dh);
      pw += static_cast<P>(ow * s.sw - s.pw + kk * s.dw);
      const float m = mb_ ? load(mb_ + qc) : 1.f;
      CornerTaps t;
      corner_taps<P>(s, pd, ph, pw, live, cin2, 0u, kOob, t);  // byte offsets in x; kOob outside the volume
      float4 *dst = reinterpret_cast<float4 *>(tp[lane]);
      dst[0] = make_float4(__uint_as_float(t.at[0]), __uint_as_float(t.at[1]), __uint_as_float(t.at[2]), __uint_as_float(t.at[3]));
      dst[1] = make_float4(__uint_as_float(t.at[4]), __uint_as_float(t.at[5]), __uint_as_float(t.at[6]), __uint_as_float(t.at[7]));
      dst[2] = make_float4(m * t.w[0], m * t.w[1], m * t.w[2], m * t.w[3]);
      dst[3] = make_float4(m * t.w[4], m * t.w[5], m * t.w[6], m * t.w[7]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll 1
    for (int st = 0; st < kWave / SL; st++) {  // SL positions per step
      // B piece: column n = channel c0 + n, rows = positions st*SL + h*PC + i
      float colv[PC];
#pragma unroll
      for (int i = 0; i < PC; i++) {
        const float4 *src = reinterpret_cast<const float4 *>(tp[st * SL + h * PC + i]);
        const float4 v0 = src[0], v1 = src[1], w0 = src[2], w1 = src[3];
        const unsigned ax[8] = {__float_as_uint(v0.x), __float_as_uint(v0.y), __float_as_uint(v0.z), __float_as_uint(v0.w),
                                __float_as_uint(v1.x), __float_as_uint(v1.y), __float_as_uint(v1.z), __float_as_uint(v1.w)};
        const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
        float a = 0.f;
#pragma unroll
        for (int c = 0; c < 8; c++) a += w[c] * load_element<T>(xr, ax[c] + cbyte2);  // kOob + channel: reads 0
        colv[i] = a;
      }
      const u32x4 bf = M::pack(colv);
      // A pieces: row n = output channel, columns = the same PC positions
      const long qa = qg + st * SL + h * PC;
#pragma unroll
      for (int m = 0; m < MT; m++) {
        const T *grow = gy + (static_cast<long>(b) * s.Cout + g * s.opg + (mb0 + m) * 32 + n) * s.Q + qa;
        union { u32x4 u; T e[PC]; } a;
        if (aligned && qa + PC <= s.Q) {
          a.u = *reinterpret_cast<const u32x4 *>(grow);
        } else {
          a.u = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
          for (int i = 0; i < PC; i++)
            if (qa + i < s.Q) a.e[i] = grow[i];
        }
        acc[m] = M::run(a.u, bf, acc[m]);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  // ---- reduce the four wavefronts, then one atomic per (o, c) ------------------------------------
  if (wave > 0) {
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
      for (int r = 0; r < 16; r++) part[wave - 1][m][r][lane] = acc[m][r];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float v = acc[m][r] + part[0][m][r][lane] + part[1][m][r][lane] + part[2][m][r][lane];
        // accumulator layout: register r of lane l = row 8*(r/4) + 4*(l/32) + r%4, column l%32
        const int o = g * s.opg + (mb0 + m) * 32 + 8 * (r / 4) + 4 * h + (r % 4);
        const int cl = c0 - g * s.cpg + n;
        // tap-major accumulator [K][Cout][cpg]: the 32 lanes of a row add to 128 contiguous bytes
        atomicAdd(gw + (static_cast<long>(k) * s.Cout + o) * s.cpg + cl, v);
      }
  }
}

// The same contraction with the column values read from the buffer the data kernel wrote (pieces
// [position / kPiece][channel][kPiece] per (sample, tap, 32-channel block), `qp` positions each): no
// gather, and a workgroup takes TPW taps at once so that a piece of grad_output (16 useful bytes of
// a 64-byte request per lane) serves TPW products.
template <typename T, int MT, int TPW>
__global__ __launch_bounds__(256) void dcn_backward_weight_columns_kernel(
    const T *__restrict__ col, const T *__restrict__ gy, float *__restrict__ gw, const DcnDims s,
    const int mb0, const long qp) {
  using M = Mfma<T>;
  constexpr int PC = M::kPiece, SL = 2 * PC;
  __shared__ float part[3][16][64];  // an accumulator of wavefronts 1..3
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int n = lane % 32, h = lane / 32;
  const int tgroups = (s.K + TPW - 1) / TPW, cblocks_all = s.Cin / 32;
  const int k0 = (blockIdx.x % tgroups) * TPW, cbi = blockIdx.x / tgroups;
  const int c0 = cbi * 32, g = c0 / s.cpg, b = blockIdx.z;
  const long qbase = static_cast<long>(blockIdx.y) * kGwChunk, qend = min(qbase + kGwChunk, s.Q);
  const bool aligned = s.Q % PC == 0;
  const T *colrow[TPW];  // taps beyond the last one repeat it; their products are not used
#pragma unroll
  for (int t = 0; t < TPW; t++)
    colrow[t] = col + ((static_cast<long>(b) * s.K + min(k0 + t, s.K - 1)) * cblocks_all + cbi) * qp * 32;

  float16_t acc[TPW][MT];
#pragma unroll
  for (int t = 0; t < TPW; t++)
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[t][m][r] = 0.f;

  for (long qg = qbase + wave * 64; qg < qend; qg += 256) {
#pragma unroll
    for (int st = 0; st < kWave / SL; st++) {  // SL positions per step
      const long qa = qg + st * SL + h * PC;
      // A pieces: row n = output channel, columns = PC positions
      u32x4 a[MT];
#pragma unroll
      for (int m = 0; m < MT; m++) {
        const T *grow = gy + (static_cast<long>(b) * s.Cout + g * s.opg + (mb0 + m) * 32 + n) * s.Q + qa;
        union { u32x4 u; T e[PC]; } piece;
        if (aligned && qa + PC <= s.Q) {
          piece.u = *reinterpret_cast<const u32x4 *>(grow);
        } else {
          piece.u = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
          for (int i = 0; i < PC; i++)
            if (qa + i < s.Q) piece.e[i] = grow[i];
        }
        a[m] = piece.u;
      }
      // B pieces: column n = channel c0 + n, rows = the same PC positions.  Positions beyond Q
      // contribute nothing because their A elements are zero, but the buffer must not be read
      // where nothing was written.
#pragma unroll
      for (int t = 0; t < TPW; t++) {
        union { u32x4 u; T e[PC]; } piece;
        piece.u = u32x4{0u, 0u, 0u, 0u};
        if (qa < s.Q) {
          piece.u = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(colrow[t] + ((qa / PC) * 32 + n) * PC));   // (read once)
          if (qa + PC > s.Q) {
#pragma unroll
            for (int i = 0; i < PC; i++)
              if (qa + i >= s.Q) piece.e[i] = store_cast<T>(0.f);
          }
        }
#pragma unroll
        for (int m = 0; m < MT; m++) acc[t][m] = M::run(a[m], piece.u, acc[t][m]);
      }
    }
  }
  // ---- reduce the four wavefronts, then one atomic per (o, c, tap) -------------------------------
#pragma unroll
  for (int t = 0; t < TPW; t++) {
    if (k0 + t >= s.K) break;  // the same for every thread
#pragma unroll
    for (int m = 0; m < MT; m++) {
      __syncthreads();
      if (wave > 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) part[wave - 1][r][lane] = acc[t][m][r];
      }
      __syncthreads();
      if (wave == 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const float v = acc[t][m][r] + part[0][r][lane] + part[1][r][lane] + part[2][r][lane];
          // accumulator layout: register r of lane l = row 8*(r/4) + 4*(l/32) + r%4, column l%32
          const int o = g * s.opg + (mb0 + m) * 32 + 8 * (r / 4) + 4 * h + (r % 4);
          const int cl = c0 - g * s.cpg + n;
          atomicAdd(gw + (static_cast<long>(k0 + t) * s.Cout + o) * s.cpg + cl, v);
        }
      }
    }
  }
}

// gxt [B, P, C] fp32 -> gx [B, C, P] T, added to what gx holds; 64 positions x up to kAddChunk
// channels per workgroup
constexpr int kAddChunk = 64;
template <typename T>
__global__ __launch_bounds__(256) void dcn_planar_add_kernel(const float *__restrict__ gxt,
                                                             T *__restrict__ gx, int C, long P) {
  __shared__ float stagef[64][kAddChunk + 1];
  const int b = blockIdx.y;
  const long p0 = static_cast<long>(blockIdx.x) * 64;
  const int c0 = blockIdx.z * kAddChunk, cn = min(kAddChunk, C - c0);
  const int count = static_cast<int>(min(static_cast<long>(64), P - p0)) * cn;
  const float *src = gxt + (static_cast<long>(b) * P + p0) * C + c0;
  for (int i = threadIdx.x; i < count; i += 256) {
    const int pp = i / cn, c = i % cn;
    stagef[pp][c] = src[static_cast<long>(pp) * C + c];
  }
  __syncthreads();
  const int lp = threadIdx.x % 64;
  if (p0 + lp < P)
    for (int c = threadIdx.x / 64; c < cn; c += 4) {
      T *d = gx + (static_cast<long>(b) * C + c0 + c) * P + p0 + lp;
      *d = store_cast<T>(load(d) + stagef[lp][c]);
    }
}

// The same move with 16-byte accesses on both sides (whole tiles of 64 positions x 64 channels, P a
// multiple of 64, 16-byte aligned tensors): a lane reads four channels of one position, then adds
// V = 16 / sizeof(T) neighbouring positions of one channel to the gradient in one read-modify-write.
template <typename T>
__device__ __forceinline__ void dcn_planar_add_wide_block(const float *__restrict__ gxt, T *__restrict__ gx, int C, long P,
                                                          const unsigned bx, const int b, const int bz) {
  constexpr int V = 16 / static_cast<int>(sizeof(T));
  __shared__ __attribute__((aligned(16))) float stagef[64][kAddChunk + 4];
  const long p0 = static_cast<long>(bx) * 64;
  const int c0 = bz * kAddChunk, cn = min(kAddChunk, C - c0);   // cn: a multiple of 4
  const float *src = gxt + (static_cast<long>(b) * P + p0) * C + c0;
  float4 in[4];
#pragma unroll
  for (int u = 0; u < 4; u++) {
    const int i = threadIdx.x + u * 256, pp = i / 16, cq = i % 16;
    in[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (cq * 4 < cn) {   // (the accumulation buffer is read once and the result not read here again: nontemporal)
      typedef float f32x4 __attribute__((ext_vector_type(4)));
      const f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src + static_cast<long>(pp) * C + cq * 4));
      in[u] = make_float4(t.x, t.y, t.z, t.w);
    }
  }
#pragma unroll
  for (int u = 0; u < 4; u++) {
    const int i = threadIdx.x + u * 256, pp = i / 16, cq = i % 16;
    *reinterpret_cast<float4 *>(&stagef[pp][cq * 4]) = in[u];
  }
  __syncthreads();
  constexpr int PG = 64 / V;   // position groups per channel
  for (int i = threadIdx.x; i < cn * PG; i += 256) {
    const int c = i / PG, pg = i % PG;
    T *d = gx + (static_cast<long>(b) * C + c0 + c) * P + p0 + pg * V;
    union { u32x4 u; T e[V]; } piece;
    piece.u = *reinterpret_cast<const u32x4 *>(d);
#pragma unroll
    for (int e = 0; e < V; e++) piece.e[e] = store_cast<T>(load(&piece.e[e]) + stagef[pg * V + e][c]);
    __builtin_nontemporal_store(piece.u, reinterpret_cast<u32x4 *>(d));
  }
}
template <typename T>
__global__ __launch_bounds__(256) void dcn_planar_add_wide_kernel(const float *__restrict__ gxt,
                                                                  T *__restrict__ gx, int C, long P) {
  dcn_planar_add_wide_block<T>(gxt, gx, C, P, blockIdx.x, blockIdx.y, blockIdx.z);
}

__device__ __forceinline__ void dcn_zero_f32_block(float *p, long n, const unsigned bid, const unsigned nblocks) {
  for (long i = bid * 256L + threadIdx.x; i < n; i += nblocks * 256L) p[i] = 0.f;
}
__global__ __launch_bounds__(256) void dcn_zero_f32_kernel(float *p, long n) { dcn_zero_f32_block(p, n, blockIdx.x, gridDim.x); }

// One pass over a slab of grad_output[b, o, .]: its sum into the fp32 bias accumulator and (`out`
// given) its largest magnitude as a bit pattern into *out.  Workgroup = (o, b, slab of `slab_len`
// positions); about 512 workgroups in all — enough loads in flight for the memory system, and few enough
// for the atomics on the one word of the maximum, which retire one after the other (~10 ns each).
static long gy_slab_len(const DcnDims &s) {
  const long rows = static_cast<long>(s.Cout) * s.B;
  const long slabs = std::max(1L, std::min((s.Q + 2047) / 2048, (512 + rows - 1) / rows));
  return ((s.Q + slabs - 1) / slabs + 1023) / 1024 * 1024;
}
template <typename T>
__device__ __forceinline__ void dcn_gy_sum_max_block(const T *__restrict__ gy, float *__restrict__ gb32, unsigned *out,
                                                     const DcnDims s, const long slab_len, const unsigned bid) {
  constexpr int V = 16 / static_cast<int>(sizeof(T));
  __shared__ float sums[4];
  const unsigned slabs = static_cast<unsigned>((s.Q + slab_len - 1) / slab_len);
  const unsigned slab = bid % slabs, r = bid / slabs;
  const int b = static_cast<int>(r % s.B), o = static_cast<int>(r / s.B);
  const T *src = gy + (static_cast<long>(b) * s.Cout + o) * s.Q;
  long q0 = static_cast<long>(slab) * slab_len;
  const long q_end = min(q0 + slab_len, s.Q);
  float v = 0.f, m = 0.f;
  bool bad = false;
  auto take = [&](T e) {
    const float x = static_cast<float>(load(&e));
    v += x;
    bad = bad || !(x == x);
    m = fmaxf(m, fabsf(x));
  };
  if (reinterpret_cast<uintptr_t>(src + q0) % 16 == 0) {
    // 16-byte pieces, four independent loads per lane and step
    const long groups = (q_end - q0) / V;
    const u32x4 *pieces = reinterpret_cast<const u32x4 *>(src + q0);
    for (long i = threadIdx.x; i < groups; i += 1024) {
      union { u32x4 u; T e[V]; } raw[4];
#pragma unroll
      for (int u = 0; u < 4; u++) raw[u].u = i + u * 256 < groups ? pieces[i + u * 256] : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
      for (int u = 0; u < 4; u++)
#pragma unroll
        for (int e = 0; e < V; e++) take(raw[u].e[e]);
    }
    q0 += groups * V;
  }
  for (long q = q0 + threadIdx.x; q < q_end; q += 256) take(src[q]);
  for (int sh = 32; sh > 0; sh >>= 1) v += __shfl_xor(v, sh);
  if (threadIdx.x % kWave == 0) sums[threadIdx.x / kWave] = v;
  if (out) fold_max(bad ? 0x7fc00000u : __float_as_uint(m), out);   // (contains the barrier)
  else __syncthreads();
  if (threadIdx.x == 0) atomicAdd(gb32 + o, (sums[0] + sums[1]) + (sums[2] + sums[3]));
}
template <typename T>
__global__ __launch_bounds__(256) void dcn_gy_sum_kernel(const T *__restrict__ gy, float *__restrict__ gb32, const DcnDims s,
                                                         const long slab_len) {
  dcn_gy_sum_max_block<T>(gy, gb32, nullptr, s, slab_len, blockIdx.x);
}

// The small jobs in front of the data kernel of a layer with tiles, in two launches instead of eight
// (a dependent launch costs ~2.7 us before its first instruction, and kernels of a few microseconds do
// not fill the machine): first the two layout passes, the weight fragments and the zero fill of the
// accumulators and of the maxima's words; then the maxima, which need those words at zero.
struct PrepareJobs {
  unsigned x_end, gy_end, f32_end, fsc_end, zero_end;   // block ranges of the first launch
  unsigned wbx, wbq;                                    // 128-position blocks of the input / the output
  int wide16;                                           // scatter fragments: 16-channel blocks (else 8)
};
template <typename T>
__global__ __launch_bounds__(256) void dcn_backward_prepare_kernel(const T *__restrict__ x, T *__restrict__ xt,
                                                                   const T *__restrict__ gy, T *__restrict__ gyt,
                                                                   const T *__restrict__ wt, T *__restrict__ wb,
                                                                   T *__restrict__ wa, float *__restrict__ zero,
                                                                   const long nz, const DcnDims s, const PrepareJobs j) {
  using U = typename std::conditional<(sizeof(T) == 2), unsigned short, unsigned int>::type;
  const unsigned id = blockIdx.x;
  if (id < j.x_end) {
    channels_last_wide_block<U>(reinterpret_cast<const U *>(x), reinterpret_cast<U *>(xt), s.Cin, s.P, id % j.wbx,
                                static_cast<int>((id / j.wbx) % s.B), static_cast<int>(id / (j.wbx * s.B)));
  } else if (id < j.gy_end) {
    const unsigned r = id - j.x_end;
    channels_last_wide_block<U>(reinterpret_cast<const U *>(gy), reinterpret_cast<U *>(gyt), s.Cout, s.Q, r % j.wbq,
                                static_cast<int>((r / j.wbq) % s.B), static_cast<int>(r / (j.wbq * s.B)));
  } else if (id < j.f32_end) {
    dcn_weight_afragments32_block<T>(wt, wb, s, id - j.gy_end);
  } else if (id < j.fsc_end) {
    if (j.wide16) dcn_weight_afragments16_block<T>(wt, wa, s, id - j.f32_end);
    else dcn_weight_afragments8_block<T>(wt, wa, s, id - j.f32_end);
  } else {
    dcn_zero_f32_block(zero, nz, id - j.fsc_end, j.zero_end - j.fsc_end);
  }
}
template <typename T>
__global__ __launch_bounds__(256) void dcn_backward_maxima_kernel(const T *__restrict__ gy, const long ngy,
                                                                  const T *__restrict__ mask, const long nmask,
                                                                  const T *__restrict__ wt, const DcnDims s,
                                                                  unsigned *__restrict__ bounds, float *__restrict__ gb32,
                                                                  const long slab_len, const unsigned gy_blocks,
                                                                  const unsigned mask_blocks) {
  const unsigned id = blockIdx.x;
  if (id < gy_blocks) {
    // with a bias gradient to form the pass over grad_output also sums it, a workgroup per (o, b, slab)
    if (gb32) dcn_gy_sum_max_block<T>(gy, gb32, bounds, s, slab_len, id);
    else dcn_absmax_block<T>(gy, ngy, bounds, id, gy_blocks);
  } else if (id < gy_blocks + mask_blocks) dcn_absmax_block<T>(mask, nmask, bounds + 2, id - gy_blocks, mask_blocks);
  else dcn_weight_colsum_block<T>(wt, s, bounds + 1, id - gy_blocks - mask_blocks);
}

// The LDS scatter pays when its tile holds the reach of a brick's undeformed taps with a voxel to
// spare on either side (offsets beyond the tile still work, through the data kernel's atomics).
template <typename S>
static bool scatter_tile_applies(const DcnDims &s, int dtype) {
  // the scatter kernel keeps grad_output of its positions in registers: up to kScatterKeep slices
  // of 4 * kPiece output channels per group (128 for 16-bit tensors, 64 for fp32); wider layers
  // would repeat too much per 8-channel workgroup and keep the atomics
  if (s.opg > kScatterKeep * (dtype == MV_F32 ? 16 : 32)) return false;
  const int ed = (S::BD - 1) * s.sd + (s.kd - 1) * s.dd + 1, eh = (S::BH - 1) * s.sh + (s.kh - 1) * s.dh + 1,
            ew = (S::BW - 1) * s.sw + (s.kw - 1) * s.dw + 1;
  return (S::TD == 1 || ed + 2 <= S::TD) && eh + 2 <= S::TH && ew + 2 <= S::TW &&
         static_cast<long>(S::BD * S::BH * S::BW) * s.K < (1L << 20);
}

static size_t align256b(size_t v) { return (v + 255) / 256 * 256; }

bool dcn_mfma_backward_supported(const DcnDims &s, int dtype) {
  if (dtype != MV_F16 && dtype != MV_BF16 && dtype != MV_F32) return false;
  if (s.cpg % 32 || s.opg % 32 || s.cpd % 32) return false;
  if (s.B > 65535 || s.dg > 65535) return false;
  if (static_cast<long>(s.P) * s.Cin * 4 >= (1L << 31)) return false;  // 32-bit byte offsets
  if (static_cast<long>(s.Cin / 32) * s.K >= (1L << 31) || (s.Q + kGwChunk - 1) / kGwChunk > 65535) return false;
  return true;
}

// workspace: xt | gyt | weight fragments (32- and 8-channel blocks) | gxt (fp32) | gw (fp32) | gb (fp32) |
// the three maxima of the scatter scale; everything from gxt on starts at zero
struct BackwardLayout {
  size_t xt, gyt, wb, wa, col, gxt, gw, gb, bounds, total;
  long qp;  // positions per row of the column buffer; 0: no buffer (the weight kernel gathers again)
};
// The column buffer holds mask * Z(x) for every (sample, tap, channel, position): it saves the
// weight kernel the second gather of x.  Layers whose columns exceed the budget do without.  The
// budget is 1 GiB unless the environment variable MV_DCN_COLUMN_BYTES (read once, when the library
// is first asked) or mv_dcn_set_column_budget() says otherwise.
static std::atomic<size_t> &column_budget_cell() {
  static std::atomic<size_t> cell{[] {
    const char *e = getenv("MV_DCN_COLUMN_BYTES");
    return e ? static_cast<size_t>(strtoull(e, nullptr, 10)) : (static_cast<size_t>(1) << 30);
  }()};
  return cell;
}
static size_t column_budget() { return column_budget_cell().load(std::memory_order_relaxed); }
void dcn_set_column_budget(size_t bytes) { column_budget_cell().store(bytes, std::memory_order_relaxed); }
size_t dcn_column_budget() { return column_budget(); }
static BackwardLayout backward_layout(const DcnDims &s, int dtype) {
  BackwardLayout l;
  const size_t es = dtype == MV_F32 ? 4 : 2;
  size_t at = 0;
  l.xt = at; at += align256b(static_cast<size_t>(s.B) * s.P * s.Cin * es);
  l.gyt = at; at += align256b(static_cast<size_t>(s.B) * s.Q * s.Cout * es);
  l.wb = at; at += align256b(static_cast<size_t>(s.Cout) * s.cpg * s.K * es);
  l.wa = at; at += align256b(2 * static_cast<size_t>(s.Cout) * s.cpg * s.K * es);  // 16 MFMA rows per 8 channels
  const long qp = (s.Q + 63) / 64 * 64;
  const size_t col_bytes = static_cast<size_t>(s.B) * s.K * s.Cin * qp * es;
  l.qp = col_bytes <= column_budget() ? qp : 0;
  l.col = at; at += l.qp ? align256b(col_bytes) : 0;
  l.gxt = at; at += align256b(static_cast<size_t>(s.B) * s.P * s.Cin * 4);
  l.gw = at; at += align256b(static_cast<size_t>(s.Cout) * s.cpg * s.K * 4);
  l.gb = at; at += align256b(static_cast<size_t>(s.Cout) * 4);
  l.bounds = at; at += 256;
  l.total = at;
  return l;
}

size_t dcn_mfma_backward_workspace_bytes(const DcnDims &s, int dtype) { return backward_layout(s, dtype).total; }

template <typename T>
static int backward_run(const void *x, const void *off, const void *mask, const void *wt,
                        const void *gy, void *goff, void *gmask, const DcnDims &s, void *workspace,
                        float **gx32, float **gw32, float **gb32, int dtype, bool want_bias, hipStream_t stream) {
  const BackwardLayout l = backward_layout(s, dtype);
  char *ws = static_cast<char *>(workspace);
  T *xt = reinterpret_cast<T *>(ws + l.xt), *gyt = reinterpret_cast<T *>(ws + l.gyt), *wb = reinterpret_cast<T *>(ws + l.wb);
  float *gxt = reinterpret_cast<float *>(ws + l.gxt);
  T *col = l.qp ? reinterpret_cast<T *>(ws + l.col) : nullptr;
  *gx32 = gxt; *gw32 = reinterpret_cast<float *>(ws + l.gw); *gb32 = reinterpret_cast<float *>(ws + l.gb);
  const bool image = s.nd == 2;
  const bool tiles = image ? scatter_tile_applies<ImageBricks>(s, dtype) : scatter_tile_applies<VolumeBricks>(s, dtype);
  // 16-bit tensors: 32-bit cells and 16 channels per workgroup, while a term keeps enough bits
  const int terms = (image ? ImageBricks::BD * ImageBricks::BH * ImageBricks::BW
                           : VolumeBricks::BD * VolumeBricks::BH * VolumeBricks::BW) * s.K;
  const bool narrow = sizeof(T) == 2 && scatter32_shift(terms) >= kScatter32MinShift;
  const int wch = narrow ? 16 : 8;
  T *wa = reinterpret_cast<T *>(ws + l.wa);
  unsigned *bounds = reinterpret_cast<unsigned *>(ws + l.bounds);
  // 32-channel weight fragments: B operands (columns = channels) for the data kernel with a channel
  // per lane, A operands (rows = channels) for the one with a position per lane
  const long frag_lanes = static_cast<long>(s.groups) * s.K * (s.cpg / 32) * (s.opg / (2 * Mfma<T>::kPiece)) * 64;
  const long scatter_lanes = static_cast<long>(s.groups) * s.K * (s.cpg / wch) * (s.opg / (4 * Mfma<T>::kPiece)) * 64;
  const long nz = static_cast<long>((l.total - l.gxt) / 4);
  const long ngy = static_cast<long>(s.B) * s.Cout * s.Q, nmask = static_cast<long>(s.B) * s.dg * s.K * s.Q;
  const long ncols = static_cast<long>(s.groups) * s.cpg * s.K;
  constexpr int V = 16 / static_cast<int>(sizeof(T)), CH = 256 / static_cast<int>(sizeof(T));
  auto aligned16 = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const long wbx = (s.P + kLayoutPos - 1) / kLayoutPos, wbq = (s.Q + kLayoutPos - 1) / kLayoutPos;
  const long nx = wbx * s.B * ((s.Cin + CH - 1) / CH), ngyb = wbq * s.B * ((s.Cout + CH - 1) / CH);
  const long nf32 = (frag_lanes + 255) / 256, nfsc = (scatter_lanes + 255) / 256, nzb = min((nz + 1023) / 1024, 4096L);
  int st = MV_OK;
  bool bias_summed = false;
  if (tiles && aligned16(x) && aligned16(xt) && aligned16(gy) && aligned16(gyt) && s.P % V == 0 && s.Q % V == 0 &&
      s.Cin % V == 0 && s.Cout % V == 0 && nx + ngyb + nf32 + nfsc + nzb < (1L << 31)) {
    PrepareJobs j;
    j.x_end = static_cast<unsigned>(nx); j.gy_end = j.x_end + static_cast<unsigned>(ngyb);
    j.f32_end = j.gy_end + static_cast<unsigned>(nf32); j.fsc_end = j.f32_end + static_cast<unsigned>(nfsc);
    j.zero_end = j.fsc_end + static_cast<unsigned>(nzb);
    j.wbx = static_cast<unsigned>(wbx); j.wbq = static_cast<unsigned>(wbq); j.wide16 = narrow;
    hipLaunchKernelGGL((dcn_backward_prepare_kernel<T>), dim3(j.zero_end), dim3(256), 0, stream, static_cast<const T *>(x), xt,
                       static_cast<const T *>(gy), gyt, static_cast<const T *>(wt), wb, wa, gxt, nz, s, j);
    const long slab_len = gy_slab_len(s);
    const long sum_blocks = static_cast<long>(s.Cout) * s.B * ((s.Q + slab_len - 1) / slab_len);
    const bool sums = want_bias && sum_blocks < (1L << 30);
    const unsigned gy_blocks = sums ? static_cast<unsigned>(sum_blocks) : static_cast<unsigned>(min((ngy + 8191) / 8192, 256L));
    const unsigned mask_blocks = mask ? static_cast<unsigned>(min((nmask + 8191) / 8192, 256L)) : 0u;
    hipLaunchKernelGGL((dcn_backward_maxima_kernel<T>), dim3(gy_blocks + mask_blocks + static_cast<unsigned>((ncols + 63) / 64)),
                       dim3(256), 0, stream, static_cast<const T *>(gy), ngy, static_cast<const T *>(mask), nmask,
                       static_cast<const T *>(wt), s, bounds, sums ? *gb32 : nullptr, slab_len, gy_blocks, mask_blocks);
    bias_summed = sums;
  } else {
    st = dcn_channels_last(x, xt, s.B, s.Cin, s.P, sizeof(T), stream);
    if (st) return st;
    st = dcn_channels_last(gy, gyt, s.B, s.Cout, s.Q, sizeof(T), stream);
    if (st) return st;
    if (tiles)
      hipLaunchKernelGGL((dcn_weight_afragments32_kernel<T>), dim3(static_cast<unsigned>(nf32)), dim3(256), 0, stream,
                         static_cast<const T *>(wt), wb, s);
    else
      hipLaunchKernelGGL((dcn_weight_bfragments_kernel<T>), dim3(static_cast<unsigned>(nf32)), dim3(256), 0, stream,
                         static_cast<const T *>(wt), wb, s);
    hipLaunchKernelGGL(dcn_zero_f32_kernel, dim3(static_cast<unsigned>(min((nz + 1023) / 1024, 65536L))), dim3(256),
                       0, stream, gxt, nz);
    if (tiles) {
      hipLaunchKernelGGL((dcn_absmax_kernel<T>), dim3(static_cast<unsigned>(min((ngy + 8191) / 8192, 256L))), dim3(256),
                         0, stream, static_cast<const T *>(gy), ngy, bounds);
      hipLaunchKernelGGL((dcn_weight_colsum_kernel<T>), dim3(static_cast<unsigned>((ncols + 63) / 64)), dim3(256), 0,
                         stream, static_cast<const T *>(wt), s, bounds + 1);
      if (mask)
        hipLaunchKernelGGL((dcn_absmax_kernel<T>), dim3(static_cast<unsigned>(min((nmask + 8191) / 8192, 256L))),
                           dim3(256), 0, stream, static_cast<const T *>(mask), nmask, bounds + 2);
      if (narrow)
        hipLaunchKernelGGL((dcn_weight_afragments16_kernel<T>), dim3(static_cast<unsigned>(nfsc)), dim3(256), 0, stream,
                           static_cast<const T *>(wt), wa, s);
      else
        hipLaunchKernelGGL((dcn_weight_afragments8_kernel<T>), dim3(static_cast<unsigned>(nfsc)), dim3(256), 0, stream,
                           static_cast<const T *>(wt), wa, s);
    }
  }
  if (want_bias && !bias_summed) {
    const long slab_len = gy_slab_len(s);
    const long sum_blocks = static_cast<long>(s.Cout) * s.B * ((s.Q + slab_len - 1) / slab_len);
    MV_REQUIRE(sum_blocks < (1L << 31), "grid too large");
    hipLaunchKernelGGL((dcn_gy_sum_kernel<T>), dim3(static_cast<unsigned>(sum_blocks)), dim3(256), 0, stream,
                       static_cast<const T *>(gy), *gb32, s, slab_len);
  }
  const long qblocks = (s.Q + 127) / 128;
  MV_REQUIRE(qblocks < (1L << 31), "grid too large");
  if (tiles) {
    MV_REQUIRE(s.Cin / 8 <= 65535, "grid too large");
#define MV_LAUNCH_SPLIT(S)                                                                                        \
  {                                                                                                               \
    hipLaunchKernelGGL((dcn_backward_data_lanes_kernel<T, S>), dim3(static_cast<unsigned>(qblocks), s.dg, s.B),   \
                       dim3(256), 0, stream, xt, static_cast<const T *>(off), static_cast<const T *>(mask), gyt,  \
                       wb, gxt, static_cast<T *>(goff), static_cast<T *>(gmask), s, bounds, col, l.qp);           \
    const long nbd = (s.Do + S::BD - 1) / S::BD, nbh = (s.Ho + S::BH - 1) / S::BH, nbw = (s.Wo + S::BW - 1) / S::BW; \
    MV_REQUIRE(nbd * nbh * nbw < (1L << 31), "grid too large");                                                   \
    if (narrow)                                                                                                   \
      hipLaunchKernelGGL((dcn_backward_scatter32_kernel<T, S>),                                                   \
                         dim3(static_cast<unsigned>(nbd * nbh * nbw), s.Cin / 16, s.B), dim3(kScatterWaves * 64), 0, \
                         stream, static_cast<const T *>(off), static_cast<const T *>(mask), gyt, wa, gxt, s,      \
                         static_cast<int>(nbh), static_cast<int>(nbw), bounds);                                   \
    else                                                                                                          \
      hipLaunchKernelGGL((dcn_backward_scatter_kernel<T, S>),                                                     \
                         dim3(static_cast<unsigned>(nbd * nbh * nbw), s.Cin / 8, s.B), dim3(kScatterWaves * 64), 0, \
                         stream, static_cast<const T *>(off), static_cast<const T *>(mask), gyt, wa, gxt, s,      \
                         static_cast<int>(nbh), static_cast<int>(nbw), bounds);                                   \
  }
    if (image) MV_LAUNCH_SPLIT(ImageBricks) else MV_LAUNCH_SPLIT(VolumeBricks)
#undef MV_LAUNCH_SPLIT
  } else {
    hipLaunchKernelGGL((dcn_backward_data_mfma_kernel<T, false, VolumeBricks>),
                       dim3(static_cast<unsigned>(qblocks), s.dg, s.B), dim3(256), 0, stream, xt,
                       static_cast<const T *>(off), static_cast<const T *>(mask), gyt, wb, gxt,
                       static_cast<T *>(goff), static_cast<T *>(gmask), s, nullptr, col, l.qp);
  }
  const dim3 wgrid(static_cast<unsigned>(static_cast<long>(s.Cin / 32) * s.K),
                   static_cast<unsigned>((s.Q + kGwChunk - 1) / kGwChunk), s.B);
#define MV_LAUNCH_GW(MTV, TPW)                                                                         \
  if (col) {                                                                                           \
    const dim3 cgrid(static_cast<unsigned>(static_cast<long>(s.Cin / 32) * ((s.K + TPW - 1) / TPW)), wgrid.y, s.B); \
    hipLaunchKernelGGL((dcn_backward_weight_columns_kernel<T, MTV, TPW>), cgrid, dim3(256), 0, stream, \
                       col, static_cast<const T *>(gy), *gw32, s, mb0, l.qp);                          \
  } else                                                                                               \
    hipLaunchKernelGGL((dcn_backward_weight_mfma_kernel<T, MTV>), wgrid, dim3(256), 0, stream, xt,     \
                       static_cast<const T *>(off), static_cast<const T *>(mask),                      \
                       static_cast<const T *>(gy), *gw32, s, mb0)
  // up to four 32-row blocks of output channels per pass over the positions when gathering; with
  // the column buffer two blocks and three taps per workgroup (the accumulators fill the registers)
  const int mstep = col ? 2 : 4;
  for (int mb0 = 0; mb0 < s.opg / 32; mb0 += mstep)
    switch (min(s.opg / 32 - mb0, mstep)) {
      case 1: MV_LAUNCH_GW(1, 3); break;
      case 2: MV_LAUNCH_GW(2, 3); break;
      case 3: MV_LAUNCH_GW(3, 1); break;
      default: MV_LAUNCH_GW(4, 1); break;
    }
#undef MV_LAUNCH_GW
  return check_launch("dcn3d mfma backward");
}

// Runs the data and weight kernels; grad_offset / grad_mask are written, the fp32 gradients of
// input (channels-last; dcn_planar_add) and weight (tap-major; dcn_weight_add) and the bias
// accumulator (zero; with `want_bias` the sums of grad_output over samples and positions) are returned
// for the caller to fold in.
int dcn_mfma_backward(const void *x, const void *off, const void *mask, const void *wt,
                      const void *gy, void *goff, void *gmask, const DcnDims &s, int dtype,
                      void *workspace, bool want_bias, float **gx32, float **gw32, float **gb32,
                      hipStream_t stream) {
  if (dtype == MV_F16)
    return backward_run<__half>(x, off, mask, wt, gy, goff, gmask, s, workspace, gx32, gw32, gb32, dtype, want_bias, stream);
  if (dtype == MV_F32)
    return backward_run<float>(x, off, mask, wt, gy, goff, gmask, s, workspace, gx32, gw32, gb32, dtype, want_bias, stream);
  return backward_run<__hip_bfloat16>(x, off, mask, wt, gy, goff, gmask, s, workspace, gx32, gw32, gb32, dtype, want_bias, stream);
}

// dst [B, C, P] (element type of `dtype`) += src [B, P, C] fp32
int planar_add_f32(const float *src, void *dst, int B, int C, long P, int dtype, hipStream_t stream) {
  const long pblocks = (P + 63) / 64;
  MV_REQUIRE(pblocks < (1L << 31) && B <= 65535 && (C + kAddChunk - 1) / kAddChunk <= 65535, "volume too large");
  const dim3 grid(static_cast<unsigned>(pblocks), B, (C + kAddChunk - 1) / kAddChunk);
  if (P % 64 == 0 && C % 4 == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(dst) % 16 == 0) {
    if (dtype == MV_F16)
      hipLaunchKernelGGL((dcn_planar_add_wide_kernel<__half>), grid, dim3(256), 0, stream, src,
                         static_cast<__half *>(dst), C, P);
    else if (dtype == MV_F32)
      hipLaunchKernelGGL((dcn_planar_add_wide_kernel<float>), grid, dim3(256), 0, stream, src,
                         static_cast<float *>(dst), C, P);
    else
      hipLaunchKernelGGL((dcn_planar_add_wide_kernel<__hip_bfloat16>), grid, dim3(256), 0, stream, src,
                         static_cast<__hip_bfloat16 *>(dst), C, P);
    return check_launch("dcn_planar_add_wide_kernel");
  }
  if (dtype == MV_F16)
    hipLaunchKernelGGL((dcn_planar_add_kernel<__half>), grid, dim3(256), 0, stream, src,
                       static_cast<__half *>(dst), C, P);
  else if (dtype == MV_F32)
    hipLaunchKernelGGL((dcn_planar_add_kernel<float>), grid, dim3(256), 0, stream, src,
                       static_cast<float *>(dst), C, P);
  else
    hipLaunchKernelGGL((dcn_planar_add_kernel<__hip_bfloat16>), grid, dim3(256), 0, stream, src,
                       static_cast<__hip_bfloat16 *>(dst), C, P);
  return check_launch("dcn_planar_add_kernel");
}

// grad_weight [Cout][cpg][K] += the tap-major fp32 accumulator [K][Cout][cpg] of the weight kernel
template <typename T>
__device__ __forceinline__ void dcn_weight_add_block(const float *__restrict__ acc, T *__restrict__ gw, const DcnDims s,
                                                     const unsigned bid, const unsigned nblocks) {
  const long n = static_cast<long>(s.Cout) * s.cpg * s.K;
  for (long i = bid * 256L + threadIdx.x; i < n; i += nblocks * 256L) {
    const long k = i % s.K, oc = i / s.K;
    gw[i] = store_cast<T>(load(gw + i) + acc[k * s.Cout * s.cpg + oc]);
  }
}
template <typename T>
__global__ __launch_bounds__(256) void dcn_weight_add_kernel(const float *__restrict__ acc, T *__restrict__ gw,
                                                             const DcnDims s) {
  dcn_weight_add_block<T>(acc, gw, s, blockIdx.x, gridDim.x);
}

// The folds behind the backward kernels in one launch: channels-last fp32 grad input -> grad_input,
// tap-major fp32 grad weight -> grad_weight, the fp32 bias sums -> grad_bias.
template <typename T>
__global__ __launch_bounds__(256) void dcn_backward_fold_kernel(const float *__restrict__ gxt, T *__restrict__ gx,
                                                                const float *__restrict__ gw32, T *__restrict__ gw,
                                                                const float *__restrict__ gb32, T *__restrict__ gb,
                                                                const DcnDims s, const unsigned pblocks,
                                                                const unsigned add_end, const unsigned weight_end) {
  const unsigned id = blockIdx.x;
  if (id < add_end)
    dcn_planar_add_wide_block<T>(gxt, gx, s.Cin, s.P, id % pblocks, static_cast<int>((id / pblocks) % s.B),
                                 static_cast<int>(id / (pblocks * s.B)));
  else if (id < weight_end)
    dcn_weight_add_block<T>(gw32, gw, s, id - add_end, weight_end - add_end);
  else
    for (int o = threadIdx.x; o < s.Cout; o += 256) gb[o] = store_cast<T>(static_cast<float>(load(gb + o)) + gb32[o]);
}

// All three folds of a layer on the matrix-core path.  Returns -1 when the tensors do not allow the
// 16-byte accesses of the one-launch form (the caller then folds one by one).
int dcn_backward_fold(const float *gxt, const float *gw32, const float *gb32, void *grad_input, void *grad_weight,
                      void *grad_bias, const DcnDims &s, int dtype, hipStream_t stream) {
  if (dtype != MV_F16 && dtype != MV_BF16 && dtype != MV_F32) return -1;
  auto aligned16 = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  if (s.P % 64 || s.Cin % 4 || !aligned16(gxt) || !aligned16(grad_input)) return -1;
  const long pblocks = s.P / 64, add_blocks = pblocks * s.B * ((s.Cin + kAddChunk - 1) / kAddChunk);
  const long n = static_cast<long>(s.Cout) * s.cpg * s.K, weight_blocks = min((n + 255) / 256, 1024L);
  const long bias_blocks = grad_bias ? 1 : 0;
  if (add_blocks + weight_blocks + bias_blocks >= (1L << 31)) return -1;
  const unsigned add_end = static_cast<unsigned>(add_blocks), weight_end = add_end + static_cast<unsigned>(weight_blocks);
#define MV_FOLD(T)                                                                                                  \
  hipLaunchKernelGGL((dcn_backward_fold_kernel<T>), dim3(weight_end + static_cast<unsigned>(bias_blocks)), dim3(256), 0, \
                     stream, gxt, static_cast<T *>(grad_input), gw32, static_cast<T *>(grad_weight),               \
                     gb32, static_cast<T *>(grad_bias), s,                                                         \
                     static_cast<unsigned>(pblocks), add_end, weight_end)
  if (dtype == MV_F16) MV_FOLD(__half);
  else if (dtype == MV_BF16) MV_FOLD(__hip_bfloat16);
  else MV_FOLD(float);
#undef MV_FOLD
  return check_launch("dcn_backward_fold_kernel");
}
int dcn_weight_add(const float *acc, void *gw, const DcnDims &s, int dtype, hipStream_t stream) {
  const long n = static_cast<long>(s.Cout) * s.cpg * s.K;
  const dim3 grid(static_cast<unsigned>(min((n + 255) / 256, 4096L)));
  if (dtype == MV_F16)
    hipLaunchKernelGGL((dcn_weight_add_kernel<__half>), grid, dim3(256), 0, stream, acc, static_cast<__half *>(gw), s);
  else if (dtype == MV_F32)
    hipLaunchKernelGGL((dcn_weight_add_kernel<float>), grid, dim3(256), 0, stream, acc, static_cast<float *>(gw), s);
  else
    hipLaunchKernelGGL((dcn_weight_add_kernel<__hip_bfloat16>), grid, dim3(256), 0, stream, acc,
                       static_cast<__hip_bfloat16 *>(gw), s);
  return check_launch("dcn_weight_add_kernel");
}

int dcn_planar_add(const float *gxt, void *gx, const DcnDims &s, int dtype, hipStream_t stream) {
  return planar_add_f32(gxt, gx, s.B, s.Cin, s.P, dtype, stream);
}

}  // namespace mv
