// Pieces shared by the matrix-core (MFMA) kernels of the 3-D deformable convolution.
#pragma once
#include "dcn_common.hpp"

namespace mv {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

template <typename T> struct Mfma;
template <> struct Mfma<__half> {
  using frag = half8_t;
  static __device__ __forceinline__ float16_t run(frag a, frag b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float lo(unsigned w) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(w & 0xffffu)));
  }
  static __device__ __forceinline__ float hi(unsigned w) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(w >> 16)));
  }
  static __device__ __forceinline__ unsigned pack(float a, float b) {
    return static_cast<unsigned>(__half_as_ushort(__float2half_rn(a))) |
           (static_cast<unsigned>(__half_as_ushort(__float2half_rn(b))) << 16);
  }
};
template <> struct Mfma<__hip_bfloat16> {
  using frag = bf16x8_t;
  static __device__ __forceinline__ float16_t run(frag a, frag b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float lo(unsigned w) { return __uint_as_float(w << 16); }
  static __device__ __forceinline__ float hi(unsigned w) { return __uint_as_float(w & 0xffff0000u); }
  static __device__ __forceinline__ unsigned pack(float a, float b) {
    // round to nearest even on the upper 16 bits
    const unsigned ua = __float_as_uint(a), ub = __float_as_uint(b);
    const unsigned ra = (ua + 0x7fffu + ((ua >> 16) & 1u)) >> 16;
    const unsigned rb = (ub + 0x7fffu + ((ub >> 16) & 1u)) & 0xffff0000u;
    return ra | rb;
  }
};

// x [B, C, P] -> xt [B, P, C] for 16-bit elements; defined in dcn3d_mfma.hip
int dcn_channels_last(const void *x, void *xt, int B, int C, long P, hipStream_t stream);

// The 8 trilinear corners of one (tap, position), z-major order: `at[c]` = voxel index * scale + add
// for a corner inside the volume, `outside` otherwise (also when the sample itself is void, i.e.
// not -1 < p < size on every axis, or the lane is not live); w[c] the trilinear weight; ld/lh/lw
// the fractions.  Branch-free: a corner is inside iff its index is, which per axis reads
//   low  index valid  <=>  0 <= p < size        high index valid  <=>  -1 < p < size - 1.
// Positions are exact in fp32 for 16-bit offsets (integer grid position + offset).
struct CornerTaps {
  unsigned at[8];
  float w[8];
  float ld, lh, lw;
};
__device__ __forceinline__ void corner_taps(const DcnDims &s, float pd, float ph, float pw, bool live,
                                            unsigned scale, unsigned add, unsigned outside,
                                            CornerTaps &t) {
  const float fd = floorf(pd), fh = floorf(ph), fw = floorf(pw);
  t.ld = pd - fd; t.lh = ph - fh; t.lw = pw - fw;
  const bool vd[2] = {pd >= 0.f && pd < static_cast<float>(s.D), pd > -1.f && pd < static_cast<float>(s.D - 1)};
  const bool vh[2] = {ph >= 0.f && ph < static_cast<float>(s.H), ph > -1.f && ph < static_cast<float>(s.H - 1)};
  const bool vw[2] = {live && pw >= 0.f && pw < static_cast<float>(s.W), live && pw > -1.f && pw < static_cast<float>(s.W - 1)};
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
