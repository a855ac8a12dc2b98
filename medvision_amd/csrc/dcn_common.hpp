// Shapes and the zero-padded sampler of the deformable convolution kernels (3-D, and 2-D as a
// depth-1 volume whose offsets carry two components per tap instead of three).
//
// For output position q = (od,oh,ow), kernel tap k = (i*kh + j)*kw + kk and input channel c in
// deformable group dgi = c / (Cin/dg):
//   p = q*stride - pad + (i,j,kk)*dil + offset[b, dgi*3K + 3k + {0:d, 1:h, 2:w}, q]
//       (images, nd = 2: offset[b, dgi*2K + 2k + {0:h, 1:w}, q] and p_d = 0)
//   col[c*K + k, q] = mask[b, dgi*K + k, q] * Z(x[b,c], p)        (mask == 1 for DCNv1)
//   y[b,o,q] = sum_{c in group(o), k} Wt[o, c_local, k] * col[c*K + k, q] + bias[o]
// Z is trilinear interpolation with ZERO padding, evaluated only when -1 < p < size on all axes
// (reference: csrc/cuda/modulated_deform_conv_3d_cuda_kernel.cuh:9-54,201-251).
#pragma once
#include "common.hpp"

namespace mv {

struct DcnDims {
  int B, Cin, D, H, W, Cout;
  int kd, kh, kw, sd, sh, sw, pd, ph, pw, dd, dh, dw;
  int groups, dg;
  int nd;             // offset components per tap: 3 (d,h,w) for volumes, 2 (h,w) for images
  int Do, Ho, Wo, K;
  int cpg, opg, cpd;  // in-channels / out-channels per group, in-channels per deformable group
  long Q, P;          // output / input positions per (sample, channel)
};

inline int make_dcn_dims(DcnDims &d, const mv_dcn3d_shape *s, int nd = 3) {
  MV_REQUIRE(s != nullptr, "shape is null");
  MV_REQUIRE(s->batch > 0 && s->in_channels > 0 && s->depth > 0 && s->height > 0 && s->width > 0 &&
                 s->out_channels > 0, "tensor dims must be positive");
  MV_REQUIRE(s->kernel_d > 0 && s->kernel_h > 0 && s->kernel_w > 0, "kernel dims must be positive");
  MV_REQUIRE(s->stride_d > 0 && s->stride_h > 0 && s->stride_w > 0, "strides must be positive");
  MV_REQUIRE(s->dil_d > 0 && s->dil_h > 0 && s->dil_w > 0, "dilations must be positive");
  MV_REQUIRE(s->pad_d >= 0 && s->pad_h >= 0 && s->pad_w >= 0, "paddings must be >= 0");
  MV_REQUIRE(s->groups > 0 && s->deformable_groups > 0, "groups must be positive");
  MV_REQUIRE(s->in_channels % s->groups == 0 && s->out_channels % s->groups == 0,
             "channels(%d) and channels_out(%d) must divide group(%d)", s->in_channels,
             s->out_channels, s->groups);
  MV_REQUIRE(s->in_channels % s->deformable_groups == 0,
             "channels(%d) must divide deformable_group(%d)", s->in_channels, s->deformable_groups);
  d.B = s->batch; d.Cin = s->in_channels; d.D = s->depth; d.H = s->height; d.W = s->width;
  d.Cout = s->out_channels;
  d.kd = s->kernel_d; d.kh = s->kernel_h; d.kw = s->kernel_w;
  d.sd = s->stride_d; d.sh = s->stride_h; d.sw = s->stride_w;
  d.pd = s->pad_d; d.ph = s->pad_h; d.pw = s->pad_w;
  d.dd = s->dil_d; d.dh = s->dil_h; d.dw = s->dil_w;
  d.groups = s->groups; d.dg = s->deformable_groups;
  d.nd = nd;
  d.Do = (d.D + 2 * d.pd - (d.dd * (d.kd - 1) + 1)) / d.sd + 1;
  d.Ho = (d.H + 2 * d.ph - (d.dh * (d.kh - 1) + 1)) / d.sh + 1;
  d.Wo = (d.W + 2 * d.pw - (d.dw * (d.kw - 1) + 1)) / d.sw + 1;
  MV_REQUIRE(d.Do > 0 && d.Ho > 0 && d.Wo > 0, "empty output (%d x %d x %d)", d.Do, d.Ho, d.Wo);
  d.K = d.kd * d.kh * d.kw;
  d.cpg = d.Cin / d.groups; d.opg = d.Cout / d.groups; d.cpd = d.Cin / d.dg;
  d.Q = static_cast<long>(d.Do) * d.Ho * d.Wo;
  d.P = static_cast<long>(d.D) * d.H * d.W;
  MV_REQUIRE(d.Q < (1L << 31) && d.P < (1L << 31), "per-channel volume must be < 2^31 voxels");
  return MV_OK;
}

// Zero-padded trilinear taps of one sample.  `off[n]` is the plane offset of corner n (z-major
// order) or -1 when the corner lies outside the volume; `w[n]` its weight.
template <typename A> struct ZTaps {
  bool ok;
  int off[8];
  A w[8];
  A fd, fh, fw;
};

// Positions are formed and split into floor + fraction in fp64 (integer grid position plus the
// offset is exact there), the fractions are then rounded once to the arithmetic type A.
template <typename A>
__device__ __forceinline__ void zero_pad_taps(const DcnDims &s, double pd, double ph, double pw,
                                              ZTaps<A> &t) {
  t.ok = pd > -1.0 && ph > -1.0 && pw > -1.0 && pd < s.D && ph < s.H && pw < s.W;
  if (!t.ok) return;
  const double fl_d = floor(pd), fl_h = floor(ph), fl_w = floor(pw);
  const int d0 = static_cast<int>(fl_d), h0 = static_cast<int>(fl_h), w0 = static_cast<int>(fl_w);
  t.fd = static_cast<A>(pd - fl_d); t.fh = static_cast<A>(ph - fl_h); t.fw = static_cast<A>(pw - fl_w);
#pragma unroll
  for (int n = 0; n < 8; n++) {
    const int a = n >> 2, b = (n >> 1) & 1, c = n & 1;
    const int zd = d0 + a, zh = h0 + b, zw = w0 + c;
    const bool in = zd >= 0 && zd < s.D && zh >= 0 && zh < s.H && zw >= 0 && zw < s.W;
    t.off[n] = in ? (zd * s.H + zh) * s.W + zw : -1;
    t.w[n] = (a ? t.fd : A(1) - t.fd) * (b ? t.fh : A(1) - t.fh) * (c ? t.fw : A(1) - t.fw);
  }
}

// Offset components of one (tap, position); `o` points at the tap's first component.
template <typename P, typename T>
__device__ __forceinline__ void dcn_offsets(const DcnDims &s, const T *__restrict__ o, P &fd, P &fh,
                                            P &fw) {
  // three unconditional loads (for images the first one re-reads the row component and is dropped)
  const long step = (s.nd - 2) * s.Q;
  const P first = static_cast<P>(load(o));
  fd = s.nd == 3 ? first : P(0);
  fh = static_cast<P>(load(o + step));
  fw = static_cast<P>(load(o + step + s.Q));
}

// Sample position of tap k at output position (od,oh,ow) for (b, dgi).
template <typename T>
__device__ __forceinline__ void dcn_position(const DcnDims &s, const T *__restrict__ off_bg,
                                             int k, int od, int oh, int ow, long q, double &pd,
                                             double &ph, double &pw) {
  const int i = k / (s.kh * s.kw), j = (k / s.kw) % s.kh, kk = k % s.kw;
  double fd, fh, fw;
  dcn_offsets(s, off_bg + static_cast<long>(s.nd * k) * s.Q + q, fd, fh, fw);
  pd = static_cast<double>(od * s.sd - s.pd + i * s.dd) + fd;
  ph = static_cast<double>(oh * s.sh - s.ph + j * s.dh) + fh;
  pw = static_cast<double>(ow * s.sw - s.pw + kk * s.dw) + fw;
}

template <typename T, typename A>
__device__ __forceinline__ A zsample(const T *__restrict__ plane, const ZTaps<A> &t) {
  A v = A(0);
#pragma unroll
  for (int n = 0; n < 8; n++)
    if (t.off[n] >= 0) v += t.w[n] * load(plane + t.off[n]);
  return v;
}

}  // namespace mv
