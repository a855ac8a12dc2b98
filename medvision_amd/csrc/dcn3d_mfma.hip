// Matrix-core (MFMA) forward of the 3-D deformable convolution for fp16 / bf16 / fp32 tensors.
//
//   y[b, o, q] = sum_{k, c} Wt[o, c, k] * col[c, k, q] + bias[o],
//   col[c, k, q] = mask[k, q] * Z(x[b, c], p(k, q))           (zero-padded trilinear sample)
//
// is a GEMM whose B operand (the column matrix, Cin*K x positions) is never written to memory:
// wavefronts build the fragment of one (tap, channel slice) directly in registers from the gathered
// corners and multiply it with weight fragments, accumulating in fp32.  Three kernels share that plan:
//   * dcn_forward_shared_taps_kernel: 16-bit tensors with 32 or 64 channels per group (the usual
//     layers).  A workgroup owns 64 positions; per group of four taps one wavefront per tap works
//     the tap geometry out with one position per lane and leaves a 64-byte record per (tap,
//     position) in LDS; then each wavefront gathers and blends 16 positions in the load layout
//     (position l / 4, 16-byte piece l % 4: the four pieces of a voxel in one cache look-up), moves
//     the piece to the matrix layout with ds_bpermute and issues v_mfma_f32_16x16x32_{f16,bf16}.
//   * dcn_forward_mfma16_kernel: the same 16 x 16 x 32 tiling with the geometry worked out by the
//     lanes that load (other channel counts that are multiples of 32, fp32 through 16x16x4).
//   * dcn_forward_mfma_kernel: 32 positions per wavefront and v_mfma_f32_32x32x16, for channel
//     counts that are multiples of 16 but not of 32.
//
// Data layout chosen for the gather, not for the GEMM:
//   * x is first transposed to channels-last [B, D*H*W, Cin] (workspace), so that ONE 16-byte load
//     per trilinear corner brings the 8 consecutive channels a lane contributes to a fragment;
//   * the 8 corner offsets / weights (x mask) of a (tap, position) are computed once and reused for
//     every channel slice of the deformable group (positions are exact in fp32 for 16-bit offsets);
//   * weights are re-laid out once per call into fragment order (workspace) so that a fragment is
//     one coalesced 16-byte load per lane, or one LDS read where a workgroup shares them.
// The sampling gather, not the matrix core, bounds these kernels: per (tap, position) 8 corners x
// Cin channels are fetched, 8 x more bytes than the fragment holds.
#include <cstdint>
#include <cstdlib>

#include "dcn_mfma.hpp"

namespace mv {

// x [B, Cin, P] -> xt [B, P, Cin]; one workgroup moves 64 positions of up to kLayoutChunk
// channels through LDS (U = unsigned short / unsigned int: only the element size matters)
constexpr int kLayoutChunk = 128;
template <typename U>
__global__ void dcn_channels_last_kernel(const U *__restrict__ x, U *__restrict__ xt, int Cin, long P) {
  __shared__ U stage[64][kLayoutChunk + 2];
  const int b = blockIdx.y;
  const long p0 = static_cast<long>(blockIdx.x) * 64;
  const int c0 = blockIdx.z * kLayoutChunk, cn = min(kLayoutChunk, Cin - c0);
  const U *src = x + (static_cast<long>(b) * Cin + c0) * P;
  U *dst = xt + (static_cast<long>(b) * P + p0) * Cin + c0;
  const int lp = threadIdx.x % 64;
  for (int c = threadIdx.x / 64; c < cn; c += 4)
    if (p0 + lp < P) stage[lp][c] = src[static_cast<long>(c) * P + p0 + lp];
  __syncthreads();
  const int count = static_cast<int>(min(static_cast<long>(64), P - p0)) * cn;
  for (int i = threadIdx.x; i < count; i += 256) {
    const int pp = i / cn, c = i % cn;
    dst[static_cast<long>(pp) * Cin + c] = stage[pp][c];
  }
}

template <typename U>
__global__ __launch_bounds__(256) void dcn_channels_last_wide_kernel(const U *__restrict__ x, U *__restrict__ xt,
                                                                     int Cin, long P) {
  channels_last_wide_block<U>(x, xt, Cin, P, blockIdx.x, blockIdx.y, blockIdx.z);
}

// weight [Cout, cpg, K] -> A pieces [group][tap][slice][row block][lane][kPiece]
template <typename T>
__global__ __launch_bounds__(256) void dcn_weight_fragments_kernel(const T *__restrict__ wt,
                                                                   T *__restrict__ wf,
                                                                   const DcnDims s) {
  constexpr int PC = Mfma<T>::kPiece;
  const int slices = s.cpg / (2 * PC), blocks = s.opg / 32;
  const long total = static_cast<long>(s.groups) * s.K * slices * blocks * 64;
  const long id = blockIdx.x * 256L + threadIdx.x;
  if (id >= total) return;
  const int lane = id % 64;
  long r = id / 64;
  const int mb = r % blocks; r /= blocks;
  const int cc = r % slices; r /= slices;
  const int k = r % s.K;
  const int g = static_cast<int>(r / s.K);
  const int o = g * s.opg + mb * 32 + lane % 32;
  const int cl = cc * 2 * PC + (lane / 32) * PC;
  for (int i = 0; i < PC; i++) wf[id * PC + i] = wt[(static_cast<long>(o) * s.cpg + cl + i) * s.K + k];
}

template <typename T, int MT>
__global__ __launch_bounds__(256, MT <= 2 ? 4 : 3) void dcn_forward_mfma_kernel(
    const T *__restrict__ xt, const T *__restrict__ off, const T *__restrict__ mask,
    const T *__restrict__ wf, const T *__restrict__ bias, T *__restrict__ y, const DcnDims s) {
  using M = Mfma<T>;
  using P = typename std::conditional<(sizeof(T) == 2), float, double>::type;  // position type
  constexpr int PC = M::kPiece, SL = 2 * PC, ES = sizeof(T);
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int n = lane % 32, h = lane / 32;
  const long q0 = (static_cast<long>(xcd_contiguous(blockIdx.x, gridDim.x)) * 4 + wave) * 32;
  if (q0 >= s.Q) return;  // whole wave idle (no barriers in this kernel)
  const long q = q0 + n;
  const bool live = q < s.Q;
  const long qc = live ? q : s.Q - 1;
  const int slices = s.cpg / SL, blocks = s.opg / 32;
  const int chunks = (blocks + MT - 1) / MT;
  const int g = blockIdx.y / chunks, mb0 = (blockIdx.y % chunks) * MT;
  const int b = blockIdx.z;
  const int ow = qc % s.Wo, oh = (qc / s.Wo) % s.Ho, od = qc / (static_cast<long>(s.Wo) * s.Ho);
  const int bd = od * s.sd - s.pd, bh = oh * s.sh - s.ph, bw = ow * s.sw - s.pw;
  const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(xt + static_cast<long>(b) * s.P * s.Cin), 0, static_cast<int>(s.P * s.Cin * ES), 0x00020000);

  float16_t acc[MT];
#pragma unroll
  for (int m = 0; m < MT; m++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[m][r] = 0.f;

  // deformable groups that intersect this convolution group's channels, and the channel slices
  // of each (cpd % 16 == 0, so a slice never straddles two deformable groups)
  const int dg_first = g * s.cpg / s.cpd, dg_last = (g * s.cpg + s.cpg - 1) / s.cpd;
  const unsigned cin = s.Cin;
  const T *wfg = wf + ((static_cast<long>(g) * s.K * slices) * blocks + mb0) * (64 * PC) + lane * PC;
  for (int dgi = dg_first; dgi <= dg_last; dgi++) {
    const int c_lo = max(g * s.cpg, dgi * s.cpd), c_hi = min(g * s.cpg + s.cpg, (dgi + 1) * s.cpd);
    const int cc_lo = (c_lo - g * s.cpg) / SL, cc_hi = (c_hi - g * s.cpg) / SL;
    const long bg = static_cast<long>(b) * s.dg + dgi;
    const T *o = off + bg * s.nd * s.K * s.Q + qc;
    const T *mk = mask ? mask + bg * s.K * s.Q + qc : nullptr;
    int ki = 0, kj = 0, kk = 0;
    for (int k = 0; k < s.K; k++) {
      P pd, ph, pw;
      dcn_offsets(s, o, pd, ph, pw);
      pd += static_cast<P>(bd + ki * s.dd); ph += static_cast<P>(bh + kj * s.dh); pw += static_cast<P>(bw + kk * s.dw);
      const float m = mk ? load(mk) : 1.f;
      o += s.nd * s.Q;
      if (mk) mk += s.Q;
      if (++kk == s.kw) { kk = 0; if (++kj == s.kh) { kj = 0; ++ki; } }
      // byte offsets of the corners' channel vectors in xt (beyond the buffer when outside: such
      // loads return zeros) and corner weights times the mask
      CornerTaps t;
      corner_taps<P>(s, pd, ph, pw, true, cin * ES, static_cast<unsigned>(h) * 16u, 0x80000000u, t);
      float cw[8];
#pragma unroll
      for (int c = 0; c < 8; c++) cw[c] = m * t.w[c];
      const unsigned *coff = t.at;
      for (int cc = cc_lo; cc < cc_hi; cc++) {
        const unsigned c0 = g * s.cpg + cc * SL;
        // this lane's channels of the slice: c0 + h * PC .. + PC - 1, one 16-byte load per corner
        u32x4 raw[8];
#pragma unroll
        for (int c = 0; c < 8; c++) raw[c] = __builtin_amdgcn_raw_buffer_load_b128(xr, coff[c], c0 * ES, 0);
        const T *wfk = wfg + (static_cast<long>(k) * slices + cc) * blocks * (64 * PC);
        u32x4 araw[MT];
#pragma unroll
        for (int mm = 0; mm < MT; mm++)
          if (mb0 + mm < blocks) araw[mm] = *reinterpret_cast<const u32x4 *>(wfk + mm * (64 * PC));
        float v[PC];
#pragma unroll
        for (int i = 0; i < PC; i++) v[i] = 0.f;
#pragma unroll
        for (int c = 0; c < 8; c++) M::fma_piece(v, cw[c], raw[c]);
        const u32x4 bfrag = M::pack(v);
#pragma unroll
        for (int mm = 0; mm < MT; mm++)
          if (mb0 + mm < blocks) acc[mm] = M::run(araw[mm], bfrag, acc[mm]);
      }
    }
  }
  if (!live) return;
#pragma unroll
  for (int m = 0; m < MT; m++) {
    if (mb0 + m >= blocks) continue;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      // 32x32 accumulator layout: register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32
      const int o = g * s.opg + (mb0 + m) * 32 + (r / 4) * 8 + h * 4 + (r % 4);
      const float val = acc[m][r] + (bias ? load(bias + o) : 0.f);
      y[(static_cast<long>(b) * s.Cout + o) * s.Q + q] = store_cast<T>(val);
    }
  }
}

// ---- 16 x 16 tiling ----------------------------------------------------------------------------
// The gather is bound by the number of cache-line look-ups: with the 32 x 32 tiling above a lane
// pair fetches 32 of the 64 (fp16: Cin = 32) bytes of a voxel per instruction, i.e. every voxel is
// looked up once per 16-channel slice.  With v_mfma_f32_16x16x32 (fp32: 16x16x4) the B operand
// gives lane l column l % 16 and K piece l / 16: four lanes fetch the four 16-byte pieces of ONE
// voxel, a load instruction covers 16 positions x 4 * kPiece channels and a voxel is looked up
// once per 32 (fp32: 16) channels.  The weight pieces of a tap come from LDS (filled by the
// workgroup one tap ahead) instead of from the vector memory path.
// weight [Cout, cpg, K] -> A pieces [group][tap][slice][16-row block][lane][kPiece]
template <typename T>
__device__ __forceinline__ void weight_fragments16_block(const T *__restrict__ wt, T *__restrict__ wf, const DcnDims &s,
                                                         unsigned block) {
  constexpr int PC = 16 / static_cast<int>(sizeof(T));   // = Mfma<T>::kPiece
  const int slices = s.cpg / (4 * PC), blocks = s.opg / 16;
  const long total = static_cast<long>(s.groups) * s.K * slices * blocks * 64;
  const long id = block * 256L + threadIdx.x;
  if (id >= total) return;
  const int lane = id % 64;
  long r = id / 64;
  const int mb = r % blocks; r /= blocks;
  const int cc = r % slices; r /= slices;
  const int k = r % s.K;
  const int g = static_cast<int>(r / s.K);
  const int o = g * s.opg + mb * 16 + lane % 16;
  const int cl = cc * 4 * PC + (lane / 16) * PC;
  for (int i = 0; i < PC; i++) wf[id * PC + i] = wt[(static_cast<long>(o) * s.cpg + cl + i) * s.K + k];
}
template <typename T>
__global__ __launch_bounds__(256) void dcn_weight_fragments16_kernel(const T *__restrict__ wt,
                                                                     T *__restrict__ wf,
                                                                     const DcnDims s) {
  weight_fragments16_block<T>(wt, wf, s, blockIdx.x);
}
// Both layout moves of a forward call in one launch (the weights are a few thousand pieces: a
// launch of their own costs more than the move): the first `nt` workgroups transpose x, the others
// order the weight pieces.  U = the element as an integer of its size.
template <typename U>
__global__ __launch_bounds__(256) void dcn_forward_layout_kernel(const U *__restrict__ x, U *__restrict__ xt,
                                                                 const U *__restrict__ wt, U *__restrict__ wf,
                                                                 const DcnDims s, unsigned wblocks, unsigned nt) {
  if (blockIdx.x < nt) {
    const unsigned bx = blockIdx.x % wblocks, r = blockIdx.x / wblocks;
    channels_last_wide_block<U>(x, xt, s.Cin, s.P, bx, static_cast<int>(r % s.B), static_cast<int>(r / s.B));
  } else {
    weight_fragments16_block<U>(wt, wf, s, blockIdx.x - nt);
  }
}

// blocks of 16 positions per wavefront: one keeps the kernel at 96 registers = 5 wavefronts per
// SIMD, which hides more of the gather latency than the reuse of two blocks would save
#ifndef MV_DCN_NB
#define MV_DCN_NB 1
#endif
#ifndef MV_DCN_WAVES_2D
#define MV_DCN_WAVES_2D 6
#endif
// bytes per weight buffer (two per workgroup): 12 KB lets five workgroups share a CU's LDS, 16 KB
// (four workgroups) serves layers whose tap does not fit the smaller one
constexpr int kWeightLdsSmall = 12 * 1024, kWeightLds = 16 * 1024;

// NC: corners per sample, 8 for volumes, 4 for images (a depth-1 volume: the upper z slice never
// exists, so its loads, weights and blend steps are left out at compile time).
// UNITS: a tap's weight pieces do not fit one LDS buffer and are walked in units of fewer channel
// slices (layers with many channels per group); otherwise a refill brings whole taps.
template <typename T, int MB, int NB, int WBYTES, int NC, bool UNITS>
__global__ __launch_bounds__(256, NB == 1 ? (NC == 4 && WBYTES <= 12 * 1024 ? MV_DCN_WAVES_2D : 5) : 4) void dcn_forward_mfma16_kernel(
    const T *__restrict__ xt, const T *__restrict__ off, const T *__restrict__ mask,
    const T *__restrict__ wf, const T *__restrict__ bias, T *__restrict__ y, const DcnDims s) {
  using M = Mfma<T>;
  using P = typename std::conditional<(sizeof(T) == 2), float, double>::type;  // position type
  constexpr int PC = M::kPiece, SL = 4 * PC, ES = sizeof(T);
  __shared__ __attribute__((aligned(16))) unsigned char wlds[2][WBYTES];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int j = lane % 16, kc = lane / 16;   // matrix layout: position (column) and piece of this lane
  const int lj = lane / 4, lk = lane % 4;    // load layout
  const int from = (4 * j + kc) * 4;         // ds_bpermute byte address of the lane holding this lane's piece
  // every XCD takes one contiguous eighth of the positions: its L2 then holds an eighth of the
  // input (plus the reach of the offsets) instead of every XCD streaming the whole volume
  const long q0 = (static_cast<long>(xcd_contiguous(blockIdx.x, gridDim.x)) * 4 + wave) * (NB * 16);
  const int slices = s.cpg / SL, blocks = s.opg / 16;
  const int chunks = (blocks + MB - 1) / MB;
  const int g = blockIdx.y / chunks, mb0 = (blockIdx.y % chunks) * MB;
  const int b = blockIdx.z;
  const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(xt + static_cast<long>(b) * s.P * s.Cin), 0, static_cast<int>(s.P * s.Cin * ES), 0x00020000);

  long qc[NB];   // position this lane gathers for (load layout), clamped
  int bd[NB], bh[NB], bw[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    const long q = q0 + nb * 16 + lj;
    qc[nb] = q < s.Q ? q : s.Q - 1;
    const int ow = qc[nb] % s.Wo, oh = (qc[nb] / s.Wo) % s.Ho, od = qc[nb] / (static_cast<long>(s.Wo) * s.Ho);
    bd[nb] = od * s.sd - s.pd; bh[nb] = oh * s.sh - s.ph; bw[nb] = ow * s.sw - s.pw;
  }
  float4_t acc[NB][MB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++)
#pragma unroll
    for (int m = 0; m < MB; m++) acc[nb][m] = float4_t{0.f, 0.f, 0.f, 0.f};

  // Weight pieces in LDS, double-buffered: a "unit" is one tap restricted to `sc` channel slices,
  // [slice][block of this chunk][lane] 16 bytes.  Usually sc = all slices and a refill brings as
  // many whole taps as fit (one workgroup barrier per refill); layers with many channels per group
  // walk a tap in several units (nunits > 1), the tap's corner offsets and weights staying in
  // registers in between.
  const int sc = UNITS ? min(slices, WBYTES / 16 / (MB * 64)) : slices;
  const int nunits = UNITS ? (slices + sc - 1) / sc : 1;         // units per tap
  const int unit_pieces = sc * MB * 64;
  const int total_units = s.K * nunits;
  const T *wfg = wf + static_cast<long>(g) * s.K * slices * blocks * (64 * PC);
  const int group = nunits == 1 ? max(1, min(s.K, WBYTES / 16 / unit_pieces)) : 1;   // units per refill
  auto fill = [&](int u0, int buf) {
    const int count = min(group, total_units - u0) * unit_pieces;
    for (int i = threadIdx.x; i < count; i += 256) {
      const int u = u0 + i / unit_pieces, rem = i % unit_pieces;
      const int ln = rem % 64, m = (rem / 64) % MB, cc = (u % nunits) * sc + rem / (64 * MB), k = u / nunits;
      u32x4 v = u32x4{0u, 0u, 0u, 0u};
      if (mb0 + m < blocks && cc < slices)
        v = *reinterpret_cast<const u32x4 *>(wfg + (((static_cast<long>(k) * slices + cc) * blocks + mb0 + m) * 64 + ln) * PC);
      reinterpret_cast<u32x4 *>(wlds[buf])[i] = v;
    }
  };
  fill(0, 0);
  __syncthreads();

  const int dg_first = g * s.cpg / s.cpd, dg_last = (g * s.cpg + s.cpg - 1) / s.cpd;
  const bool one_dg = dg_first == dg_last;   // then a tap's corners are kept from unit to unit
  const unsigned cin = s.Cin;
  int ki = 0, kj = 0, kk = 0;
  float cw[NB][NC];
  unsigned at[NB][NC];
  for (int u = 0, k = 0, unit = 0, in_group = 0, buf = 0; u < total_units; u++) {
    if (in_group == 0 && u + group < total_units) fill(u + group, buf ^ 1);
    const u32x4 *wl = reinterpret_cast<const u32x4 *>(wlds[buf]) + in_group * unit_pieces;
    const int s_lo = UNITS ? unit * sc : 0, s_hi = UNITS ? min(slices, s_lo + sc) : slices;   // slices of this unit
    for (int dgi = dg_first; dgi <= dg_last; dgi++) {
      const int c_lo = max(g * s.cpg, dgi * s.cpd), c_hi = min(g * s.cpg + s.cpg, (dgi + 1) * s.cpd);
      const int cc_lo = max((c_lo - g * s.cpg) / SL, s_lo), cc_hi = min((c_hi - g * s.cpg) / SL, s_hi);
      if (cc_lo >= cc_hi) continue;
      const long bg = static_cast<long>(b) * s.dg + dgi;
#pragma unroll
      for (int nb = 0; nb < NB; nb++) {
        if (!UNITS || unit == 0 || !one_dg) {
          P pd, ph, pw;
          dcn_offsets(s, off + (bg * s.nd * s.K + s.nd * k) * s.Q + qc[nb], pd, ph, pw);
          pd += static_cast<P>(bd[nb] + ki * s.dd); ph += static_cast<P>(bh[nb] + kj * s.dh); pw += static_cast<P>(bw[nb] + kk * s.dw);
          if (NC == 4) pd = P(0);   // images: the only slice
          const float m = mask ? load(mask + (bg * s.K + k) * s.Q + qc[nb]) : 1.f;
          CornerTaps t;
          corner_taps<P>(s, pd, ph, pw, true, cin * ES, static_cast<unsigned>(lk) * 16u, 0x80000000u, t);
#pragma unroll
          for (int c = 0; c < NC; c++) { cw[nb][c] = m * t.w[c]; at[nb][c] = t.at[c]; }
        }
        for (int cc = cc_lo; cc < cc_hi; cc++) {
          const unsigned c0 = g * s.cpg + cc * SL;
          u32x4 raw[NC];
#pragma unroll
          for (int c = 0; c < NC; c++) raw[c] = __builtin_amdgcn_raw_buffer_load_b128(xr, at[nb][c], c0 * ES, 0);
          float v[PC];
#pragma unroll
          for (int i = 0; i < PC; i++) v[i] = 0.f;
#pragma unroll
          for (int c = 0; c < NC; c++) M::fma_piece(v, cw[nb][c], raw[c]);
          const u32x4 mine = M::pack(v);   // piece lk of position lj; wanted: piece kc of position j
          const u32x4 bpiece = u32x4{
              static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(from, static_cast<int>(mine.x))),
              static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(from, static_cast<int>(mine.y))),
              static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(from, static_cast<int>(mine.z))),
              static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(from, static_cast<int>(mine.w)))};
#pragma unroll
          for (int mm = 0; mm < MB; mm++)
            acc[nb][mm] = M::run16(wl[((cc - s_lo) * MB + mm) * 64 + lane], bpiece, acc[nb][mm]);
        }
      }
    }
    if (!UNITS || ++unit == nunits) {
      unit = 0;
      k++;
      if (++kk == s.kw) { kk = 0; if (++kj == s.kh) { kj = 0; ++ki; } }
    }
    if (++in_group == group) {
      in_group = 0;
      buf ^= 1;
      __syncthreads();  // the other buffer is complete, this one may be refilled
    }
  }
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    if (q0 + nb * 16 + j >= s.Q) continue;
#pragma unroll
    for (int m = 0; m < MB; m++) {
      if (mb0 + m >= blocks) continue;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        // 16x16 accumulator layout: register r of lane l holds row 4 * (l / 16) + r, column l % 16
        const int o = g * s.opg + (mb0 + m) * 16 + kc * 4 + r;
        const float val = acc[nb][m][r] + (bias ? load(bias + o) : 0.f);
        y[(static_cast<long>(b) * s.Cout + o) * s.Q + q0 + nb * 16 + j] = store_cast<T>(val);
      }
    }
  }
}

// ---- taps worked out once per position ------------------------------------------------------------
// In the kernel above the four lanes that share a position each repeat the tap's geometry (offsets,
// floor / fraction, 8 corner offsets, 8 weights: about as many vector instructions as the blend of
// 32 channels).  Here a workgroup of four wavefronts owns 64 positions and alternates two phases
// per group of TG = 4 taps:
//   G  wavefront w takes tap w of the group with ONE position per lane (the offset planes are read
//      as 128 contiguous bytes), and leaves the 8 corner offsets and 8 mask-scaled weights as a
//      64-byte record in LDS; all lanes also bring the group's weight pieces into LDS;
//   B  wavefront w takes positions 16 w .. 16 w + 15 in the load layout (position l / 4, piece
//      l % 4), reads each tap's record as four broadcast 16-byte LDS reads, gathers, blends and
//      feeds the matrix core as above.
// The geometry then costs a quarter of what it did per (tap, 16 positions), and the offsets of
// the next group are requested a whole B phase ahead.  One convolution group must lie inside one
// deformable group, and a tap's weight pieces (SLICES x MB x 1 KB) are kept to 8 KB.
template <typename T, int MB, int SLICES, int NC>
__global__ __launch_bounds__(256, 5) void dcn_forward_shared_taps_kernel(
    const T *__restrict__ xt, const T *__restrict__ off, const T *__restrict__ mask,
    const T *__restrict__ wf, const T *__restrict__ bias, T *__restrict__ y, const DcnDims s) {
  using M = Mfma<T>;
  constexpr int PC = M::kPiece, SL = 4 * PC, ES = sizeof(T), TG = 4;
  static_assert(sizeof(T) == 2, "16-bit tensors");
  constexpr int REC = 2 * NC;                     // dwords per record: NC corner offsets, NC weights
  constexpr int WT = SLICES * MB * 64;            // 16-byte weight pieces per tap
  constexpr int WREG = (TG * WT + 255) / 256;     // pieces a thread moves per group
  constexpr unsigned kOutside = 0x80000000u;      // beyond the buffer: such loads return zeros
  __shared__ __attribute__((aligned(16))) unsigned rec[TG][64][REC];
  __shared__ __attribute__((aligned(16))) u32x4 wl[TG * WT];
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int j = lane % 16, kc = lane / 16;   // matrix layout: position (column) and piece of this lane
  const int lj = lane / 4, lk = lane % 4;    // load layout
  const int from = (4 * j + kc) * 4;         // ds_bpermute byte address of the lane holding this lane's piece
  // The workgroup's 64 positions are a brick of 8 x 4 x 2 output voxels (8 x 8 of a single slice):
  // their corners overlap far more than those of 64 positions along a row, which is what the vector
  // L1 sees.  Local index l of the brick is voxel (l / 32, (l / 8) % 4, l % 8); positions of a
  // brick that reach past the volume are dead.
  const int bdz = s.Do > 1 ? 2 : 1, bhy = 8 / bdz;
  const int nbw = (s.Wo + 7) / 8, nbh = (s.Ho + bhy - 1) / bhy;
  const int wg = xcd_contiguous(blockIdx.x, gridDim.x);
  const int w0 = (wg % nbw) * 8, h0 = ((wg / nbw) % nbh) * bhy, d0 = (wg / (nbw * nbh)) * bdz;
  auto position = [&](int l) -> long {   // linear output position of local index l, -1 when dead
    const int ow = w0 + l % 8, oh = h0 + (l / 8) % bhy, od = d0 + l / (8 * bhy);
    return (ow < s.Wo && oh < s.Ho && od < s.Do) ? (static_cast<long>(od) * s.Ho + oh) * s.Wo + ow : -1;
  };
  const int blocks = s.opg / 16;
  const int chunks = (blocks + MB - 1) / MB;
  const int g = blockIdx.y / chunks, mb0 = (blockIdx.y % chunks) * MB;
  const int b = blockIdx.z;
  const int dgi = g * s.cpg / s.cpd;
  const long bg = static_cast<long>(b) * s.dg + dgi;
  const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(xt + static_cast<long>(b) * s.P * s.Cin), 0, static_cast<int>(s.P * s.Cin * ES), 0x00020000);

  // phase G: this lane's position, its grid origin, and the planes it reads (scalar offsets per
  // tap and component; sizes below 2^31 bytes are checked by the host)
  const long qg = position(lane);
  const bool live = qg >= 0;
  const long qgc = live ? qg : s.Q - 1;
  float base_d, base_h, base_w;
  {
    const int ow = qgc % s.Wo, oh = (qgc / s.Wo) % s.Ho, od = qgc / (static_cast<long>(s.Wo) * s.Ho);
    base_d = static_cast<float>(od * s.sd - s.pd); base_h = static_cast<float>(oh * s.sh - s.ph);
    base_w = live ? static_cast<float>(ow * s.sw - s.pw) : -1e30f;   // a dead lane's samples are void
  }
  const int plane_bytes = static_cast<int>(s.Q) * ES;
  const __amdgpu_buffer_rsrc_t offr = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(off + bg * s.nd * s.K * s.Q), 0, s.nd * s.K * plane_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t maskr = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(mask ? mask + bg * s.K * s.Q : off), 0, mask ? s.K * plane_bytes : 0, 0x00020000);
  const unsigned q_bytes = static_cast<unsigned>(qgc) * ES;
  auto as_float = [](unsigned short bits) { T t; __builtin_memcpy(&t, &bits, 2); return load(&t); };
  // (d), h, w offsets and the mask value of tap k, requested one group ahead (a tap beyond the
  // last one reads zeros: scalar offsets take part in the range check)
  unsigned short rd = 0, rh = 0, rw = 0, rm = 0;
  auto request = [&](int k) {
    const int first = s.nd * k * plane_bytes;
    if (s.nd == 3) rd = __builtin_amdgcn_raw_buffer_load_b16(offr, q_bytes, first, 0);
    rh = __builtin_amdgcn_raw_buffer_load_b16(offr, q_bytes, first + (s.nd - 2) * plane_bytes, 0);
    rw = __builtin_amdgcn_raw_buffer_load_b16(offr, q_bytes, first + (s.nd - 1) * plane_bytes, 0);
    rm = __builtin_amdgcn_raw_buffer_load_b16(maskr, q_bytes, k * plane_bytes, 0);
  };
  // element strides of the channels-last input in bytes, and the corner offsets relative to the first
  const unsigned cb = s.Cin * ES, wb = static_cast<unsigned>(s.W) * cb, hwb = static_cast<unsigned>(s.H) * wb;
  // the group's weight pieces: piece `id` of the group = (tap id / WT, slice, block, lane)
  const int tap_bytes = SLICES * blocks * 64 * 16;   // bytes of one tap's pieces in wf
  const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(wf + static_cast<long>(g) * s.K * SLICES * blocks * (64 * PC)), 0, s.K * tap_bytes, 0x00020000);
  unsigned wsrc[WREG];
#pragma unroll
  for (int i = 0; i < WREG; i++) {
    const int id = i * 256 + tid, t = id / WT, rem = id % WT;
    const int ln = rem % 64, m = (rem / 64) % MB, cc = rem / (64 * MB);
    wsrc[i] = (id < TG * WT && mb0 + m < blocks) ? static_cast<unsigned>(t * tap_bytes + ((cc * blocks + mb0 + m) * 64 + ln) * 16)
                                                 : kOutside;
  }

  float4_t acc[MB];
#pragma unroll
  for (int m = 0; m < MB; m++) acc[m] = float4_t{0.f, 0.f, 0.f, 0.f};

  // tap of this wavefront in the current group as (i, j, k) kernel indices: advanced by TG per group
  const int khw = s.kh * s.kw;
  int ki = wave / khw, kj = (wave % khw) / s.kw, kk = wave % s.kw;
  request(wave);
  for (int k0 = 0; k0 < s.K; k0 += TG) {
    const int taps = min(TG, s.K - k0);
    // ---- G: the group's weight pieces (requested first, stored last) and this wavefront's tap ----
    u32x4 wreg[WREG];
#pragma unroll
    for (int i = 0; i < WREG; i++) wreg[i] = __builtin_amdgcn_raw_buffer_load_b128(wr, wsrc[i], k0 * tap_bytes, 0);
    const int k = k0 + wave;
    if (k < s.K) {
      const float m = mask ? as_float(rm) : 1.f;
      float pd = base_d + static_cast<float>(ki * s.dd) + as_float(rd);
      const float ph = base_h + static_cast<float>(kj * s.dh) + as_float(rh);
      const float pw = base_w + static_cast<float>(kk * s.dw) + as_float(rw);
      if (NC == 4) pd = 0.f;   // images: the only slice
      // A corner is inside iff its index is: with f = floor(p) the low one iff 0 <= f < size, the
      // high one iff 0 <= f + 1 < size (a sample at -1 exactly keeps a high corner of weight 0).
      const float fd = floorf(pd), fh = floorf(ph), fw = floorf(pw);
      const float ld = pd - fd, lh = ph - fh, lw = pw - fw;
      // (huge positions saturate in the conversion and fail the unsigned comparisons)
      const int id = static_cast<int>(fd), ih = static_cast<int>(fh), iw = static_cast<int>(fw);
      const bool vd0 = static_cast<unsigned>(id) < static_cast<unsigned>(s.D), vd1 = static_cast<unsigned>(id + 1) < static_cast<unsigned>(s.D);
      const bool vh0 = static_cast<unsigned>(ih) < static_cast<unsigned>(s.H), vh1 = static_cast<unsigned>(ih + 1) < static_cast<unsigned>(s.H);
      const bool vw0 = static_cast<unsigned>(iw) < static_cast<unsigned>(s.W), vw1 = static_cast<unsigned>(iw + 1) < static_cast<unsigned>(s.W);
      const unsigned first = static_cast<unsigned>(id) * hwb + static_cast<unsigned>(ih) * wb + static_cast<unsigned>(iw) * cb;
      const float md1 = m * ld, md0 = m - md1;   // mask times the depth weights
      const float wh1 = lh, wh0 = 1.f - lh, ww1 = lw, ww0 = 1.f - lw;
      const float hw00 = wh0 * ww0, hw01 = wh0 * ww1, hw10 = wh1 * ww0, hw11 = wh1 * ww1;
      unsigned at[8];
      float w[8];
      at[0] = (vd0 && vh0 && vw0) ? first : kOutside;                 w[0] = md0 * hw00;
      at[1] = (vd0 && vh0 && vw1) ? first + cb : kOutside;            w[1] = md0 * hw01;
      at[2] = (vd0 && vh1 && vw0) ? first + wb : kOutside;            w[2] = md0 * hw10;
      at[3] = (vd0 && vh1 && vw1) ? first + wb + cb : kOutside;       w[3] = md0 * hw11;
      at[4] = (vd1 && vh0 && vw0) ? first + hwb : kOutside;           w[4] = md1 * hw00;
      at[5] = (vd1 && vh0 && vw1) ? first + hwb + cb : kOutside;      w[5] = md1 * hw01;
      at[6] = (vd1 && vh1 && vw0) ? first + hwb + wb : kOutside;      w[6] = md1 * hw10;
      at[7] = (vd1 && vh1 && vw1) ? first + hwb + wb + cb : kOutside; w[7] = md1 * hw11;
      unsigned *r = rec[wave][lane];
#pragma unroll
      for (int c = 0; c < NC; c += 4) {
        *reinterpret_cast<u32x4 *>(r + c) = u32x4{at[c], at[c + 1], at[c + 2], at[c + 3]};
        *reinterpret_cast<u32x4 *>(r + NC + c) = u32x4{__float_as_uint(w[c]), __float_as_uint(w[c + 1]),
                                                      __float_as_uint(w[c + 2]), __float_as_uint(w[c + 3])};
      }
    }
    request(k + TG);
    kk += TG;
    while (kk >= s.kw) { kk -= s.kw; kj++; }
    while (kj >= s.kh) { kj -= s.kh; ki++; }
#pragma unroll
    for (int i = 0; i < WREG; i++)
      if (i * 256 + tid < TG * WT) wl[i * 256 + tid] = wreg[i];
    __syncthreads();
    // ---- B: positions 16 * wave .. + 15, every tap of the group -----------------------------------
    for (int t = 0; t < taps; t++) {
      const unsigned *r = rec[t][16 * wave + lj];
      unsigned at[NC];
      float cw[NC];
#pragma unroll
      for (int c = 0; c < NC; c += 4) {
        const u32x4 a = *reinterpret_cast<const u32x4 *>(r + c), w4 = *reinterpret_cast<const u32x4 *>(r + NC + c);
        at[c] = a.x + lk * 16u; at[c + 1] = a.y + lk * 16u; at[c + 2] = a.z + lk * 16u; at[c + 3] = a.w + lk * 16u;
        cw[c] = __uint_as_float(w4.x); cw[c + 1] = __uint_as_float(w4.y);
        cw[c + 2] = __uint_as_float(w4.z); cw[c + 3] = __uint_as_float(w4.w);
      }
#pragma unroll
      for (int cc = 0; cc < SLICES; cc++) {
        const unsigned c0 = g * s.cpg + cc * SL;
        u32x4 raw[NC];
#pragma unroll
        for (int c = 0; c < NC; c++) raw[c] = __builtin_amdgcn_raw_buffer_load_b128(xr, at[c], c0 * ES, 0);
        float v[PC];
#pragma unroll
        for (int i = 0; i < PC; i++) v[i] = 0.f;
#pragma unroll
        for (int c = 0; c < NC; c++) M::fma_piece(v, cw[c], raw[c]);
        const u32x4 mine = M::pack(v);   // piece lk of position lj; wanted: piece kc of position j
        const u32x4 bpiece = u32x4{
            static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(from, static_cast<int>(mine.x))),
            static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(from, static_cast<int>(mine.y))),
            static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(from, static_cast<int>(mine.z))),
            static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(from, static_cast<int>(mine.w)))};
#pragma unroll
        for (int mm = 0; mm < MB; mm++) acc[mm] = M::run16(wl[t * WT + (cc * MB + mm) * 64 + lane], bpiece, acc[mm]);
      }
    }
    __syncthreads();   // records and weight pieces may be overwritten
  }
  const long qo = position(16 * wave + j);
  if (qo < 0) return;
  // 16x16 accumulator layout: register r of lane l holds row 4 * (l / 16) + r, column l % 16.
  // All bias values first (the lane's four channels of a block are 8 contiguous bytes; no bias: an
  // empty range), then the stores: a load between two stores would wait for the first.
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  const __amdgpu_buffer_rsrc_t br = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(bias), 0, bias ? s.Cout * ES : 0, 0x00020000);
  u32x2 braw[MB];
#pragma unroll
  for (int m = 0; m < MB; m++)
    braw[m] = __builtin_amdgcn_raw_buffer_load_b64(br, (g * s.opg + (mb0 + m) * 16 + kc * 4) * ES, 0, 0);
#pragma unroll
  for (int m = 0; m < MB; m++) {
    if (mb0 + m >= blocks) continue;
    const float bv[4] = {M::lo(braw[m].x), M::hi(braw[m].x), M::lo(braw[m].y), M::hi(braw[m].y)};
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int o = g * s.opg + (mb0 + m) * 16 + kc * 4 + r;
      y[(static_cast<long>(b) * s.Cout + o) * s.Q + qo] = store_cast<T>(acc[m][r] + bv[r]);
    }
  }
}

// [B, C, P] -> [B, P, C] for elements of 2 or 4 bytes
int dcn_channels_last(const void *x, void *xt, int B, int C, long P, int elem_bytes, hipStream_t stream) {
  const int vec = 16 / elem_bytes;
  const bool aligned = reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(xt) % 16 == 0;
  if (aligned && P % vec == 0 && C % vec == 0) {
    const long wblocks = (P + kLayoutPos - 1) / kLayoutPos;
    const int ch = 256 / elem_bytes;
    MV_REQUIRE(wblocks < (1L << 31) && B <= 65535 && (C + ch - 1) / ch <= 65535, "volume too large");
    const dim3 wgrid(static_cast<unsigned>(wblocks), B, (C + ch - 1) / ch);
    if (elem_bytes == 2)
      hipLaunchKernelGGL((dcn_channels_last_wide_kernel<unsigned short>), wgrid, dim3(256), 0, stream,
                         static_cast<const unsigned short *>(x), static_cast<unsigned short *>(xt), C, P);
    else
      hipLaunchKernelGGL((dcn_channels_last_wide_kernel<unsigned int>), wgrid, dim3(256), 0, stream,
                         static_cast<const unsigned int *>(x), static_cast<unsigned int *>(xt), C, P);
    return check_launch("dcn_channels_last_wide_kernel");
  }
  const long pblocks = (P + 63) / 64;
  MV_REQUIRE(pblocks < (1L << 31) && B <= 65535, "volume too large");
  const dim3 grid(static_cast<unsigned>(pblocks), B, (C + kLayoutChunk - 1) / kLayoutChunk);
  if (elem_bytes == 2)
    hipLaunchKernelGGL((dcn_channels_last_kernel<unsigned short>), grid, dim3(256), 0, stream,
                       static_cast<const unsigned short *>(x), static_cast<unsigned short *>(xt), C, P);
  else
    hipLaunchKernelGGL((dcn_channels_last_kernel<unsigned int>), grid, dim3(256), 0, stream,
                       static_cast<const unsigned int *>(x), static_cast<unsigned int *>(xt), C, P);
  return check_launch("dcn_channels_last_kernel");
}

static size_t align256(size_t v) { return (v + 255) / 256 * 256; }
// MV_DCN_SHARED_TAPS=0 keeps every layer on the kernels that work the taps out per lane
static bool dcn_shared_taps_enabled() {
  static const bool on = [] { const char *e = getenv("MV_DCN_SHARED_TAPS"); return !(e && e[0] == '0'); }();
  return on;
}
static int elem_size(int dtype) { return dtype == MV_F32 ? 4 : 2; }

bool dcn_mfma_supported(const DcnDims &s, int dtype) {
  if (dtype != MV_F16 && dtype != MV_BF16 && dtype != MV_F32) return false;
  if (s.cpg % 16 || s.opg % 32 || s.cpd % 16) return false;
  if (s.Cin > 4096 || s.B > 65535) return false;
  if (static_cast<long>(s.P) * s.Cin * elem_size(dtype) >= (1L << 31)) return false;  // 32-bit byte offsets
  return true;
}

size_t dcn_mfma_workspace_bytes(const DcnDims &s, int dtype) {
  const size_t es = elem_size(dtype);
  const size_t xt = static_cast<size_t>(s.B) * s.P * s.Cin * es;
  const size_t wf = static_cast<size_t>(s.Cout) * s.cpg * s.K * es;
  return align256(xt) + align256(wf);
}

template <typename T>
static int dcn_mfma_run(const void *x, const void *off, const void *mask, const void *wt,
                        const void *bias, void *y, const DcnDims &s, void *workspace,
                        hipStream_t stream) {
  constexpr int PC = Mfma<T>::kPiece;
  T *xt = static_cast<T *>(workspace);
  T *wf = reinterpret_cast<T *>(static_cast<char *>(workspace) +
                                align256(static_cast<size_t>(s.B) * s.P * s.Cin * sizeof(T)));
  // 16 x 16 tiling: whole 4-piece slices per (deformable) group and a tap's weight pieces fit LDS
  bool fused = false;   // x and the weights laid out by one launch
  {
    using U = typename std::conditional<(sizeof(T) == 2), unsigned short, unsigned int>::type;
    const int blocks16 = s.opg / 16;
    const int mb = (blocks16 >= 8 && s.nd == 2) ? 8 : (blocks16 >= 4 ? 4 : (blocks16 >= 2 ? 2 : 1));
    const long tap_bytes = static_cast<long>(s.cpg / (4 * PC)) * mb * 64 * 16;
    const bool tiling16 = s.cpg % (4 * PC) == 0 && s.cpd % (4 * PC) == 0 && (tap_bytes <= kWeightLds || s.cpd % s.cpg == 0);
    constexpr int V = 16 / static_cast<int>(sizeof(T)), CH = 256 / static_cast<int>(sizeof(T));
    const bool aligned = reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(xt) % 16 == 0;
    const long wblocks = (s.P + kLayoutPos - 1) / kLayoutPos;
    const long nt = wblocks * s.B * ((s.Cin + CH - 1) / CH);
    const long lanes = static_cast<long>(s.groups) * s.K * (s.cpg / (4 * PC)) * blocks16 * 64;
    const long nw = (lanes + 255) / 256;
    if (tiling16 && aligned && s.P % V == 0 && s.Cin % V == 0 && nt + nw < (1L << 31)) {
      hipLaunchKernelGGL((dcn_forward_layout_kernel<U>), dim3(static_cast<unsigned>(nt + nw)), dim3(256), 0, stream,
                         reinterpret_cast<const U *>(x), reinterpret_cast<U *>(xt), reinterpret_cast<const U *>(wt),
                         reinterpret_cast<U *>(wf), s, static_cast<unsigned>(wblocks), static_cast<unsigned>(nt));
      const int st = check_launch("dcn_forward_layout_kernel");
      if (st) return st;
      fused = true;
    }
  }
  if (!fused) {
    const int st = dcn_channels_last(x, xt, s.B, s.Cin, s.P, sizeof(T), stream);
    if (st) return st;
  }
  {
    const int blocks16 = s.opg / 16;
    // output blocks of 16 per wavefront: up to 8 (128 output channels: every pass over the output
    // channels repeats the gather, so wide layers want few passes)
    const int mb = (blocks16 >= 8 && s.nd == 2) ? 8 : (blocks16 >= 4 ? 4 : (blocks16 >= 2 ? 2 : 1));
    const long tap_bytes = static_cast<long>(s.cpg / (4 * PC)) * mb * 64 * 16;
    // a tap that does not fit one weight buffer is walked in units of fewer channel slices; that
    // keeps the tap's corners in registers, which needs one deformable group per convolution group
    const bool fits = tap_bytes <= kWeightLds || s.cpd % s.cpg == 0;
    if (s.cpg % (4 * PC) == 0 && s.cpd % (4 * PC) == 0 && fits) {
      const long lanes = static_cast<long>(s.groups) * s.K * (s.cpg / (4 * PC)) * blocks16 * 64;
      if (!fused)
        hipLaunchKernelGGL((dcn_weight_fragments16_kernel<T>), dim3(static_cast<unsigned>((lanes + 255) / 256)),
                           dim3(256), 0, stream, static_cast<const T *>(wt), wf, s);
      const int chunks = (blocks16 + mb - 1) / mb;
      if constexpr (sizeof(T) == 2) {
        // volumes with 32 or 64 channels per group inside one deformable group: taps shared through LDS
        const int slices = s.cpg / (4 * PC);
        const bool volume = !(s.nd == 2 && s.D == 1 && s.kd == 1 && s.pd == 0);
        const bool small = static_cast<long>(s.nd) * s.K * s.Q * 2 < (1L << 31) &&
                           static_cast<long>(s.K) * slices * blocks16 * 1024 < (1L << 31);
        if (dcn_shared_taps_enabled() && (slices == 1 || slices == 2) && s.cpd % s.cpg == 0 && blocks16 >= 4 && volume && small) {
          const int chunks4 = (blocks16 + 3) / 4;
          // bricks of 8 x 4 x 2 output voxels (8 x 8 of a single slice), one per workgroup
          const int bdz = s.Do > 1 ? 2 : 1, bhy = 8 / bdz;
          const long qb = static_cast<long>((s.Wo + 7) / 8) * ((s.Ho + bhy - 1) / bhy) * ((s.Do + bdz - 1) / bdz);
          MV_REQUIRE(qb < (1L << 31) && static_cast<long>(s.groups) * chunks4 <= 65535, "grid too large");
          const dim3 grid(static_cast<unsigned>(qb), s.groups * chunks4, s.B), block(256);
          if (slices == 1)
            hipLaunchKernelGGL((dcn_forward_shared_taps_kernel<T, 4, 1, 8>), grid, block, 0, stream, xt,
                               static_cast<const T *>(off), static_cast<const T *>(mask), wf,
                               static_cast<const T *>(bias), static_cast<T *>(y), s);
          else
            hipLaunchKernelGGL((dcn_forward_shared_taps_kernel<T, 4, 2, 8>), grid, block, 0, stream, xt,
                               static_cast<const T *>(off), static_cast<const T *>(mask), wf,
                               static_cast<const T *>(bias), static_cast<T *>(y), s);
          return check_launch("dcn_forward_shared_taps_kernel");
        }
      }
      constexpr int kNb = MV_DCN_NB;
      const long qblocks = (s.Q + 64 * kNb - 1) / (64 * kNb);
      MV_REQUIRE(qblocks < (1L << 31) && static_cast<long>(s.groups) * chunks <= 65535, "grid too large");
      const dim3 grid(static_cast<unsigned>(qblocks), s.groups * chunks, s.B), block(256);
#define MV_LAUNCH_MFMA16_K(MBV, WB, NCV, UV)                                                          \
  hipLaunchKernelGGL((dcn_forward_mfma16_kernel<T, MBV, kNb, WB, NCV, UV>), grid, block, 0, stream, xt, \
                     static_cast<const T *>(off), static_cast<const T *>(mask), wf,                  \
                     static_cast<const T *>(bias), static_cast<T *>(y), s)
      // whole taps per refill unless the tap is larger than the (large) buffer
#define MV_LAUNCH_MFMA16_NC(MBV, WB, NCV)                                                             \
  do {                                                                                                \
    if (WB == kWeightLds && static_cast<long>(s.cpg / (4 * PC)) * MBV * 64 * 16 > kWeightLds)         \
      MV_LAUNCH_MFMA16_K(MBV, kWeightLds, NCV, true);                                                 \
    else                                                                                              \
      MV_LAUNCH_MFMA16_K(MBV, WB, NCV, false);                                                        \
  } while (0)
#define MV_LAUNCH_MFMA16(MBV, WB)                                                                \
  do {                                                                                            \
    if (s.nd == 2 && s.D == 1 && s.kd == 1 && s.pd == 0)                                          \
      MV_LAUNCH_MFMA16_NC(MBV, WB, 4);                                                            \
    else                                                                                          \
      MV_LAUNCH_MFMA16_NC(MBV, WB, 8);                                                            \
  } while (0)
      if (mb == 8) MV_LAUNCH_MFMA16(8, kWeightLds);
      else if (tap_bytes <= kWeightLdsSmall) {
        if (mb == 4) MV_LAUNCH_MFMA16(4, kWeightLdsSmall);
        else if (mb == 2) MV_LAUNCH_MFMA16(2, kWeightLdsSmall);
        else MV_LAUNCH_MFMA16(1, kWeightLdsSmall);
      } else {
        if (mb == 4) MV_LAUNCH_MFMA16(4, kWeightLds);
        else if (mb == 2) MV_LAUNCH_MFMA16(2, kWeightLds);
        else MV_LAUNCH_MFMA16(1, kWeightLds);
      }
#undef MV_LAUNCH_MFMA16
#undef MV_LAUNCH_MFMA16_NC
#undef MV_LAUNCH_MFMA16_K
      return check_launch("dcn_forward_mfma16_kernel");
    }
  }
  const long frag_lanes = static_cast<long>(s.groups) * s.K * (s.cpg / (2 * PC)) * (s.opg / 32) * 64;
  hipLaunchKernelGGL((dcn_weight_fragments_kernel<T>), dim3(static_cast<unsigned>((frag_lanes + 255) / 256)),
                     dim3(256), 0, stream, static_cast<const T *>(wt), wf, s);
  const int blocks = s.opg / 32;
  const int mt = blocks >= 4 ? 4 : (blocks >= 2 ? 2 : 1);
  const int chunks = (blocks + mt - 1) / mt;
  const long qblocks = (s.Q + 127) / 128;
  MV_REQUIRE(qblocks < (1L << 31) && static_cast<long>(s.groups) * chunks <= 65535, "grid too large");
  const dim3 grid(static_cast<unsigned>(qblocks), s.groups * chunks, s.B), block(256);
#define MV_LAUNCH_MFMA(MTV)                                                                      \
  hipLaunchKernelGGL((dcn_forward_mfma_kernel<T, MTV>), grid, block, 0, stream, xt,              \
                     static_cast<const T *>(off), static_cast<const T *>(mask), wf,              \
                     static_cast<const T *>(bias), static_cast<T *>(y), s)
  if (mt == 4) MV_LAUNCH_MFMA(4);
  else if (mt == 2) MV_LAUNCH_MFMA(2);
  else MV_LAUNCH_MFMA(1);
#undef MV_LAUNCH_MFMA
  return check_launch("dcn_forward_mfma_kernel");
}

int dcn_mfma_forward(const void *x, const void *off, const void *mask, const void *wt,
                     const void *bias, void *y, const DcnDims &s, int dtype, void *workspace,
                     hipStream_t stream) {
  if (dtype == MV_F16) return dcn_mfma_run<__half>(x, off, mask, wt, bias, y, s, workspace, stream);
  if (dtype == MV_F32) return dcn_mfma_run<float>(x, off, mask, wt, bias, y, s, workspace, stream);
  return dcn_mfma_run<__hip_bfloat16>(x, off, mask, wt, bias, y, s, workspace, stream);
}

}  // namespace mv
