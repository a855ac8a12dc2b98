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

// The 8 trilinear corners of one (tap, position): voxel index (~0u outside the volume or when the
// sample is void) and weight; fractions for the derivative.  Positions are exact in fp32 for
// 16-bit offsets (integer grid position + offset).
struct CornerTaps {
  unsigned vox[8];
  float w[8];
  float ld, lh, lw;
};
__device__ __forceinline__ void corner_taps(const DcnDims &s, float pd, float ph, float pw, bool live,
                                            CornerTaps &t) {
  const bool ok = live && pd > -1.f && ph > -1.f && pw > -1.f && pd < s.D && ph < s.H && pw < s.W;
  const float fd = floorf(pd), fh = floorf(ph), fw = floorf(pw);
  const int d0 = static_cast<int>(fd), h0 = static_cast<int>(fh), w0 = static_cast<int>(fw);
  t.ld = pd - fd; t.lh = ph - fh; t.lw = pw - fw;
#pragma unroll
  for (int c = 0; c < 8; c++) {
    const int a = c >> 2, bb = (c >> 1) & 1, e = c & 1;
    const int zd = d0 + a, zh = h0 + bb, zw = w0 + e;
    const bool in = ok && zd >= 0 && zd < s.D && zh >= 0 && zh < s.H && zw >= 0 && zw < s.W;
    t.vox[c] = in ? static_cast<unsigned>((zd * s.H + zh) * s.W + zw) : ~0u;
    t.w[c] = (a ? t.ld : 1.f - t.ld) * (bb ? t.lh : 1.f - t.lh) * (e ? t.lw : 1.f - t.lw);
  }
}

}  // namespace mv
