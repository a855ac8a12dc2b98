// Pieces shared by the matrix-core (MFMA) kernels of the 3-D deformable convolution.
#pragma once
#include "dcn_common.hpp"

namespace mv {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Element-type traits of the matrix-core kernels.  Every operand piece is 16 bytes per lane
// (`kPiece` elements): for the 16-bit types one piece is the lane's share of a K = 16 fragment of
// v_mfma_f32_32x32x16 (lane l: row / column l % 32, K indices (l / 32) * 8 .. + 7); for fp32 one
// piece feeds four v_mfma_f32_32x32x2_f32 (K = 2: lane l holds K index l / 32), element t of the
// piece in instruction t.  A "slice" is the 2 * kPiece channels (or rows) one such step covers:
// lane half h = l / 32 owns elements h * kPiece .. + kPiece - 1 of the slice.
// `run16` is the 16 x 16 counterpart (v_mfma_f32_16x16x32 / four v_mfma_f32_16x16x4_f32): lane l holds
// row / column l % 16 and the piece l / 16 of a slice of 4 * kPiece; accumulator register r of lane l
// is row 4 * (l / 16) + r, column l % 16.
template <typename T> struct Mfma;
template <> struct Mfma<__half> {
  static constexpr int kPiece = 8;
  static __device__ __forceinline__ float16_t run(u32x4 a, u32x4 b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float4_t run16(u32x4 a, u32x4 b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float lo(unsigned w) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(w & 0xffffu)));
  }
  static __device__ __forceinline__ float hi(unsigned w) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(w >> 16)));
  }
  // two values rounded to nearest even and packed, in one instruction
  static __device__ __forceinline__ unsigned pack2(float a, float b) {
    unsigned r;
    asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
  }
  // v[0..7] += w * piece
  static __device__ __forceinline__ void fma_piece(float (&v)[8], float w, u32x4 r) {
    v[0] += w * lo(r.x); v[1] += w * hi(r.x); v[2] += w * lo(r.y); v[3] += w * hi(r.y);
    v[4] += w * lo(r.z); v[5] += w * hi(r.z); v[6] += w * lo(r.w); v[7] += w * hi(r.w);
  }
  static __device__ __forceinline__ u32x4 pack(const float (&v)[8]) {
    return u32x4{pack2(v[0], v[1]), pack2(v[2], v[3]), pack2(v[4], v[5]), pack2(v[6], v[7])};
  }
};
template <> struct Mfma<__hip_bfloat16> {
  static constexpr int kPiece = 8;
  static __device__ __forceinline__ float16_t run(u32x4 a, u32x4 b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float4_t run16(u32x4 a, u32x4 b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float lo(unsigned w) { return __uint_as_float(w << 16); }
  static __device__ __forceinline__ float hi(unsigned w) { return __uint_as_float(w & 0xffff0000u); }
  // two values rounded to nearest even and packed, in one instruction
  static __device__ __forceinline__ unsigned pack2(float a, float b) {
    unsigned r;
    asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
  }
  static __device__ __forceinline__ void fma_piece(float (&v)[8], float w, u32x4 r) {
    v[0] += w * lo(r.x); v[1] += w * hi(r.x); v[2] += w * lo(r.y); v[3] += w * hi(r.y);
    v[4] += w * lo(r.z); v[5] += w * hi(r.z); v[6] += w * lo(r.w); v[7] += w * hi(r.w);
  }
  static __device__ __forceinline__ u32x4 pack(const float (&v)[8]) {
    return u32x4{pack2(v[0], v[1]), pack2(v[2], v[3]), pack2(v[4], v[5]), pack2(v[6], v[7])};
  }
};
template <> struct Mfma<float> {
  static constexpr int kPiece = 4;
  static __device__ __forceinline__ float16_t run(u32x4 a, u32x4 b, float16_t c) {
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float4_t run16(u32x4 a, u32x4 b, float4_t c) {
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float lo(unsigned w) { return __uint_as_float(w); }
  static __device__ __forceinline__ void fma_piece(float (&v)[4], float w, u32x4 r) {
    v[0] += w * __uint_as_float(r.x); v[1] += w * __uint_as_float(r.y);
    v[2] += w * __uint_as_float(r.z); v[3] += w * __uint_as_float(r.w);
  }
  static __device__ __forceinline__ u32x4 pack(const float (&v)[4]) {
    return u32x4{__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])};
  }
};

// x [B, C, P] -> xt [B, P, C], elements of `elem_bytes` (2 or 4); defined in dcn3d_mfma.hip
int dcn_channels_last(const void *x, void *xt, int B, int C, long P, int elem_bytes, hipStream_t stream);

// The same move with 16-byte global accesses: rows of x are read as groups of 16 bytes (V
// positions of one channel), kept in LDS as [channel][position], and every lane writes V channels
// of one position.  Needs P and Cin to be multiples of V and 16-byte aligned tensors.
constexpr int kLayoutPos = 128;
template <typename U>
__device__ __forceinline__ void channels_last_wide_block(const U *__restrict__ x, U *__restrict__ xt, int Cin, long P,
                                                         unsigned bx, int b, int bz) {
  constexpr int V = 16 / sizeof(U), CH = 256 / sizeof(U);   // CH channels per workgroup: 128 (2 bytes), 64 (4 bytes)
  constexpr int PITCH = kLayoutPos + V;
  __shared__ __attribute__((aligned(16))) U stage[CH * PITCH];
  const long p0 = static_cast<long>(bx) * kLayoutPos;
  const int c0 = bz * CH, cn = min(CH, Cin - c0);
  const int np = static_cast<int>(min(static_cast<long>(kLayoutPos), P - p0));   // a multiple of V
  const U *src = x + (static_cast<long>(b) * Cin + c0) * P + p0;
  U *dst = xt + (static_cast<long>(b) * P + p0) * Cin + c0;
  constexpr int PG = kLayoutPos / V;
  for (int i = threadIdx.x; i < cn * PG; i += 256) {
    const int c = i / PG, pg = i % PG;
    if (pg * V < np)
      *reinterpret_cast<u32x4 *>(stage + c * PITCH + pg * V) = *reinterpret_cast<const u32x4 *>(src + static_cast<long>(c) * P + pg * V);
  }
  __syncthreads();
  const int cg_n = cn / V;
  for (int i = threadIdx.x; i < np * cg_n; i += 256) {
    const int pp = i / cg_n, cg = i % cg_n;
    U out[V];
#pragma unroll
    for (int e = 0; e < V; e++) out[e] = stage[(cg * V + e) * PITCH + pp];
    u32x4 packed;
    __builtin_memcpy(&packed, out, 16);
    *reinterpret_cast<u32x4 *>(dst + static_cast<long>(pp) * Cin + cg * V) = packed;
  }
}
// The 8 trilinear corners of one (tap, position), z-major order: `at[c]` = voxel index * scale + add
// for a corner inside the volume, `outside` otherwise (also when the sample itself is void, i.e.
// not -1 < p < size on every axis, or the lane is not live); w[c] the trilinear weight; ld/lh/lw
// the fractions.  Branch-free: a corner is inside iff its index is, which per axis reads
//   low  index valid  <=>  0 <= p < size        high index valid  <=>  -1 < p < size - 1.
// Positions are exact in fp32 for 16-bit offsets (integer grid position + offset); fp32 tensors
// pass them in fp64 (floor and fraction taken there, the fraction rounded once to fp32).
struct CornerTaps {
  unsigned at[8];
  float w[8];
  float ld, lh, lw;
};
template <typename P>
__device__ __forceinline__ void corner_taps(const DcnDims &s, P pd, P ph, P pw, bool live,
                                            unsigned scale, unsigned add, unsigned outside,
                                            CornerTaps &t) {
  const P fd = floor(pd), fh = floor(ph), fw = floor(pw);
  t.ld = static_cast<float>(pd - fd); t.lh = static_cast<float>(ph - fh); t.lw = static_cast<float>(pw - fw);
  const bool vd[2] = {pd >= P(0) && pd < static_cast<P>(s.D), pd > P(-1) && pd < static_cast<P>(s.D - 1)};
  const bool vh[2] = {ph >= P(0) && ph < static_cast<P>(s.H), ph > P(-1) && ph < static_cast<P>(s.H - 1)};
  const bool vw[2] = {live && pw >= P(0) && pw < static_cast<P>(s.W), live && pw > P(-1) && pw < static_cast<P>(s.W - 1)};
  const int base = (static_cast<int>(fd) * s.H + static_cast<int>(fh)) * s.W + static_cast<int>(fw);
  const unsigned first = static_cast<unsigned>(base) * scale + add;  // wraps harmlessly when base < 0
  const unsigned sw = scale, sh = static_cast<unsigned>(s.W) * scale, sd = static_cast<unsigned>(s.H * s.W) * scale;
  const float wd[2] = {1.f - t.ld, t.ld}, wh[2] = {1.f - t.lh, t.lh}, ww[2] = {1.f - t.lw, t.lw};
#pragma unroll
  for (int c = 0; c < 8; c++) {
    const int a = c >> 2, bb = (c >> 1) & 1, e = c & 1;
    t.at[c] = (vd[a] && vh[bb] && vw[e]) ? first + a * sd + bb * sh + e * sw : outside;
    t.w[c] = wd[a] * wh[bb] * ww[e];
  }
}

}  // namespace mv
