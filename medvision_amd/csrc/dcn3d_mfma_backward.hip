// Backward of the 3-D deformable convolution for fp16 / bf16 tensors, built around the matrix
// cores and channels-last buffers.
//
//   gcol[c, k, q] = sum_o Wt[o, c, k] * gy[o, q]                    (GEMM, MFMA)
//   gx[corner_n(k, q), c] += w_n * mask * gcol                       (scatter, fp32 atomics)
//   goff_a[k, q] = mask * sum_c gcol * dZ/dp_a ,  gmask[k, q] = sum_c gcol * Z
//   gw[o, c, k]  = sum_{b, q} gy[o, q] * col[c, k, q]                (GEMM over positions, MFMA)
//
// Data kernel: a wavefront owns 32 output positions.  Per tap it forms the 32 x 32 block
// gcol[position, channel] with MFMA 32x32x16 (A = gy channels-last, B = weight fragments); the
// accumulator layout gives every lane ONE channel and 16 positions, so for each position the 32
// lanes of a half-wavefront touch 32 consecutive channels of a channels-last voxel: the reads of
// x (for the offset / mask gradients) and the fp32 atomic adds into the channels-last gradient
// buffer are 64- and 128-byte contiguous.  The four per-position sums over channels are reduced
// across the half-wavefront with DPP adds.
// Weight kernel: a workgroup owns (tap, 32-channel block, range of positions); lanes rebuild the
// column values of their channel for 16 positions at a time (same coalesced corner reads), which
// is exactly the MFMA B fragment; A is gy read in its own layout.  Accumulators stay in registers
// over the whole range and are added to the fp32 gradient once per workgroup.
#include "dcn_mfma.hpp"

namespace mv {

constexpr unsigned kOob = 0x80000000u;  // byte offset beyond every buffer: loads give 0, atomics are dropped
constexpr int kRsrcFlags = 0x00020000;

// weight [Cout, cpg, K] -> B pieces [group][tap][32-channel block][row step][lane][kPiece]:
// lane l, element i = Wt[g*opg + step*2*kPiece + (l/32)*kPiece + i, block*32 + l%32, k]
template <typename T>
__global__ __launch_bounds__(256) void dcn_weight_bfragments_kernel(const T *__restrict__ wt,
                                                                    T *__restrict__ wb,
                                                                    const DcnDims s) {
  constexpr int PC = Mfma<T>::kPiece;
  const int cblocks = s.cpg / 32, steps = s.opg / (2 * PC);
  const long total = static_cast<long>(s.groups) * s.K * cblocks * steps * 64;
  const long id = blockIdx.x * 256L + threadIdx.x;
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

constexpr int kTapWords = 20;  // vox[8], w[8], mask, ld, lh, lw

template <typename T>
__global__ __launch_bounds__(256) void dcn_backward_data_mfma_kernel(
    const T *__restrict__ xt, const T *__restrict__ off, const T *__restrict__ mask,
    const T *__restrict__ gyt, const T *__restrict__ wb, float *__restrict__ gxt,
    T *__restrict__ goff, T *__restrict__ gmask, const DcnDims s) {
  using M = Mfma<T>;
  using P = typename std::conditional<(sizeof(T) == 2), float, double>::type;  // position type
  constexpr int PC = M::kPiece, SL = 2 * PC, ES = sizeof(T);
  __shared__ __attribute__((aligned(16))) float taps[4][32][kTapWords];
  __shared__ float sums[4][4][32];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int n = lane % 32, h = lane / 32;
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
  const T *gyrow = gyt + (static_cast<long>(b) * s.Q + qc) * s.Cout + h * PC;
  const T *o = off + bg * s.nd * s.K * s.Q + qc;
  const T *mk = mask ? mask + bg * s.K * s.Q + qc : nullptr;
  float(*tp)[kTapWords] = taps[wave];
  float(*sm)[32] = sums[wave];

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
      CornerTaps t;
      corner_taps<P>(s, pd, ph, pw, live, 1u, 0u, ~0u, t);
      if (h == 0) {
        float4 *dst = reinterpret_cast<float4 *>(tp[n]);
        dst[0] = make_float4(__uint_as_float(t.at[0]), __uint_as_float(t.at[1]), __uint_as_float(t.at[2]), __uint_as_float(t.at[3]));
        dst[1] = make_float4(__uint_as_float(t.at[4]), __uint_as_float(t.at[5]), __uint_as_float(t.at[6]), __uint_as_float(t.at[7]));
        dst[2] = make_float4(t.w[0], t.w[1], t.w[2], t.w[3]);
        dst[3] = make_float4(t.w[4], t.w[5], t.w[6], t.w[7]);
        dst[4] = make_float4(m, t.ld, t.lh, t.lw);
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
      const unsigned cbyte2 = static_cast<unsigned>(c0 + n) * ES, cbyte4 = static_cast<unsigned>(c0 + n) * 4u;
      const unsigned cin2 = static_cast<unsigned>(s.Cin) * ES, cin4 = static_cast<unsigned>(s.Cin) * 4u;
      // ---- register r: position 8*(r/4) + 4*h + r%4, channel c0 + n ------------------------------
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int p = 8 * (r / 4) + 4 * h + (r % 4);
        const float4 *src = reinterpret_cast<const float4 *>(tp[p]);
        const float4 v0 = src[0], v1 = src[1], w0 = src[2], w1 = src[3], e = src[4];
        const unsigned vox[8] = {__float_as_uint(v0.x), __float_as_uint(v0.y), __float_as_uint(v0.z), __float_as_uint(v0.w),
                                 __float_as_uint(v1.x), __float_as_uint(v1.y), __float_as_uint(v1.z), __float_as_uint(v1.w)};
        const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
        const float m = e.x, ld = e.y, lh = e.z, lw = e.w;
        const float gm = acc[r] * m;
        float v[8];
#pragma unroll
        for (int c = 0; c < 8; c++) {
          const bool in = vox[c] != ~0u;
          v[c] = load_element<T>(xr, in ? vox[c] * cin2 + cbyte2 : kOob);
          __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(w[c] * gm, gr, in ? vox[c] * cin4 + cbyte4 : kOob, 0, 0);
        }
        float val = 0.f;
#pragma unroll
        for (int c = 0; c < 8; c++) val += w[c] * v[c];
        const float hd = 1.f - ld, hh = 1.f - lh, hw = 1.f - lw;
        const float dd = hh * (hw * (v[4] - v[0]) + lw * (v[5] - v[1])) + lh * (hw * (v[6] - v[2]) + lw * (v[7] - v[3]));
        const float dh = hd * (hw * (v[2] - v[0]) + lw * (v[3] - v[1])) + ld * (hw * (v[6] - v[4]) + lw * (v[7] - v[5]));
        const float dw = hd * (hh * (v[1] - v[0]) + lh * (v[3] - v[2])) + ld * (hh * (v[5] - v[4]) + lh * (v[7] - v[6]));
        const float s0 = half_wave_sum(dd * gm), s1 = half_wave_sum(dh * gm), s2 = half_wave_sum(dw * gm);
        const float s3 = half_wave_sum(acc[r] * val);
        if (n == 16) {  // one lane per half-wavefront; the chunks of a deformable group accumulate
          sm[0][p] += s0; sm[1][p] += s1; sm[2][p] += s2; sm[3][p] += s3;
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

// ---- grad wrt weight ---------------------------------------------------------------------------
constexpr int kGwChunk = 2048;  // positions per workgroup

template <typename T, int MT>
__global__ __launch_bounds__(256) void dcn_backward_weight_mfma_kernel(
    const T *__restrict__ xt, const T *__restrict__ off, const T *__restrict__ mask,
    const T *__restrict__ gy, float *__restrict__ gw, const DcnDims s, const int mb0) {
  using M = Mfma<T>;
  using P = typename std::conditional<(sizeof(T) == 2), float, double>::type;  // position type
  constexpr int PC = M::kPiece, SL = 2 * PC, ES = sizeof(T);
  __shared__ __attribute__((aligned(16))) float taps[4][64][16];  // vox[8], w[8] * mask
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
      corner_taps<P>(s, pd, ph, pw, live, 1u, 0u, ~0u, t);
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
      float col[PC];
#pragma unroll
      for (int i = 0; i < PC; i++) {
        const float4 *src = reinterpret_cast<const float4 *>(tp[st * SL + h * PC + i]);
        const float4 v0 = src[0], v1 = src[1], w0 = src[2], w1 = src[3];
        const unsigned vox[8] = {__float_as_uint(v0.x), __float_as_uint(v0.y), __float_as_uint(v0.z), __float_as_uint(v0.w),
                                 __float_as_uint(v1.x), __float_as_uint(v1.y), __float_as_uint(v1.z), __float_as_uint(v1.w)};
        const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
        float a = 0.f;
#pragma unroll
        for (int c = 0; c < 8; c++)
          a += w[c] * load_element<T>(xr, vox[c] != ~0u ? vox[c] * cin2 + cbyte2 : kOob);
        col[i] = a;
      }
      const u32x4 bf = M::pack(col);
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
        atomicAdd(gw + (static_cast<long>(o) * s.cpg + cl) * s.K + k, v);
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

__global__ void dcn_zero_f32_kernel(float *p, long n) {
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<long>(gridDim.x) * blockDim.x)
    p[i] = 0.f;
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

// workspace: xt | gyt | weight fragments | gxt (fp32) | gw (fp32) | gb (fp32)
struct BackwardLayout {
  size_t xt, gyt, wb, gxt, gw, gb, total;
};
static BackwardLayout backward_layout(const DcnDims &s, int dtype) {
  BackwardLayout l;
  const size_t es = dtype == MV_F32 ? 4 : 2;
  size_t at = 0;
  l.xt = at; at += align256b(static_cast<size_t>(s.B) * s.P * s.Cin * es);
  l.gyt = at; at += align256b(static_cast<size_t>(s.B) * s.Q * s.Cout * es);
  l.wb = at; at += align256b(static_cast<size_t>(s.Cout) * s.cpg * s.K * es);
  l.gxt = at; at += align256b(static_cast<size_t>(s.B) * s.P * s.Cin * 4);
  l.gw = at; at += align256b(static_cast<size_t>(s.Cout) * s.cpg * s.K * 4);
  l.gb = at; at += align256b(static_cast<size_t>(s.Cout) * 4);
  l.total = at;
  return l;
}

size_t dcn_mfma_backward_workspace_bytes(const DcnDims &s, int dtype) { return backward_layout(s, dtype).total; }

template <typename T>
static int backward_run(const void *x, const void *off, const void *mask, const void *wt,
                        const void *gy, void *goff, void *gmask, const DcnDims &s, void *workspace,
                        float **gx32, float **gw32, float **gb32, int dtype, hipStream_t stream) {
  const BackwardLayout l = backward_layout(s, dtype);
  char *ws = static_cast<char *>(workspace);
  T *xt = reinterpret_cast<T *>(ws + l.xt), *gyt = reinterpret_cast<T *>(ws + l.gyt), *wb = reinterpret_cast<T *>(ws + l.wb);
  float *gxt = reinterpret_cast<float *>(ws + l.gxt);
  *gx32 = gxt; *gw32 = reinterpret_cast<float *>(ws + l.gw); *gb32 = reinterpret_cast<float *>(ws + l.gb);
  int st = dcn_channels_last(x, xt, s.B, s.Cin, s.P, sizeof(T), stream);
  if (st) return st;
  st = dcn_channels_last(gy, gyt, s.B, s.Cout, s.Q, sizeof(T), stream);
  if (st) return st;
  const long frag_lanes = static_cast<long>(s.groups) * s.K * (s.cpg / 32) * (s.opg / (2 * Mfma<T>::kPiece)) * 64;
  hipLaunchKernelGGL((dcn_weight_bfragments_kernel<T>), dim3(static_cast<unsigned>((frag_lanes + 255) / 256)),
                     dim3(256), 0, stream, static_cast<const T *>(wt), wb, s);
  const long nz = static_cast<long>((l.total - l.gxt) / 4);
  hipLaunchKernelGGL(dcn_zero_f32_kernel, dim3(static_cast<unsigned>(min((nz + 1023) / 1024, 65536L))), dim3(256),
                     0, stream, gxt, nz);
  const long qblocks = (s.Q + 127) / 128;
  MV_REQUIRE(qblocks < (1L << 31), "grid too large");
  hipLaunchKernelGGL((dcn_backward_data_mfma_kernel<T>), dim3(static_cast<unsigned>(qblocks), s.dg, s.B),
                     dim3(256), 0, stream, xt, static_cast<const T *>(off), static_cast<const T *>(mask), gyt,
                     wb, gxt, static_cast<T *>(goff), static_cast<T *>(gmask), s);
  const dim3 wgrid(static_cast<unsigned>(static_cast<long>(s.Cin / 32) * s.K),
                   static_cast<unsigned>((s.Q + kGwChunk - 1) / kGwChunk), s.B);
#define MV_LAUNCH_GW(MTV)                                                                          \
  hipLaunchKernelGGL((dcn_backward_weight_mfma_kernel<T, MTV>), wgrid, dim3(256), 0, stream, xt,   \
                     static_cast<const T *>(off), static_cast<const T *>(mask),                    \
                     static_cast<const T *>(gy), *gw32, s, mb0)
  // up to four 32-row blocks of output channels per pass over the positions
  for (int mb0 = 0; mb0 < s.opg / 32; mb0 += 4)
    switch (min(s.opg / 32 - mb0, 4)) {
      case 1: MV_LAUNCH_GW(1); break;
      case 2: MV_LAUNCH_GW(2); break;
      case 3: MV_LAUNCH_GW(3); break;
      default: MV_LAUNCH_GW(4); break;
    }
#undef MV_LAUNCH_GW
  return check_launch("dcn3d mfma backward");
}

// Runs the data and weight kernels; grad_offset / grad_mask are written, the fp32 gradients of
// input (channels-last), weight and bias accumulators are returned for the caller to fold in.
int dcn_mfma_backward(const void *x, const void *off, const void *mask, const void *wt,
                      const void *gy, void *goff, void *gmask, const DcnDims &s, int dtype,
                      void *workspace, float **gx32, float **gw32, float **gb32,
                      hipStream_t stream) {
  if (dtype == MV_F16)
    return backward_run<__half>(x, off, mask, wt, gy, goff, gmask, s, workspace, gx32, gw32, gb32, dtype, stream);
  if (dtype == MV_F32)
    return backward_run<float>(x, off, mask, wt, gy, goff, gmask, s, workspace, gx32, gw32, gb32, dtype, stream);
  return backward_run<__hip_bfloat16>(x, off, mask, wt, gy, goff, gmask, s, workspace, gx32, gw32, gb32, dtype, stream);
}

// dst [B, C, P] (element type of `dtype`) += src [B, P, C] fp32
int planar_add_f32(const float *src, void *dst, int B, int C, long P, int dtype, hipStream_t stream) {
  const long pblocks = (P + 63) / 64;
  MV_REQUIRE(pblocks < (1L << 31) && B <= 65535 && (C + kAddChunk - 1) / kAddChunk <= 65535, "volume too large");
  const dim3 grid(static_cast<unsigned>(pblocks), B, (C + kAddChunk - 1) / kAddChunk);
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

int dcn_planar_add(const float *gxt, void *gx, const DcnDims &s, int dtype, hipStream_t stream) {
  return planar_add_f32(gxt, gx, s.B, s.Cin, s.P, dtype, stream);
}

}  // namespace mv
