// Channel padding for the matrix-core deformable-convolution kernels.
//
// Those kernels take channel counts that are multiples of 32 per convolution group, per deformable
// group and per group of output channels (dcn3d_mfma.hip, dcn3d_mfma_backward.hip).  Any other layer
// (16, 24, 40, 48 ... channels, with any number of groups as long as convolution groups and
// deformable groups nest) is run as the next larger layer that they do take: the input, the weight
// and the output gradient are copied with zero channels added, the kernels run on the padded shapes,
// and outputs and gradients are taken from the real channels only.  Zero inputs, zero weight rows and
// zero weight columns add nothing to any output or gradient, so the results are those of the layer
// itself.  The copies live in the caller's workspace; they cost one pass over the tensors, against
// kernels that are 50 - 100 times slower without the matrix cores.
//
// Channel map: with unit = min(channels per convolution group, channels per deformable group) (the
// smaller divides the larger) real input channel c sits at (c / unit) * unit_p + c % unit of the
// padded tensor, unit_p = unit rounded up to 32; output channel o at (o / opg) * opg_p + o % opg.
#include "dcn_pad.hpp"

namespace mv {

static int round_up32(int v) { return (v + 31) / 32 * 32; }

bool dcn_pad_plan(const DcnDims &s, int dtype, DcnPad &pad) {
  pad.on = false;
  if (dtype != MV_F16 && dtype != MV_BF16 && dtype != MV_F32) return false;
  const int unit = s.cpg < s.cpd ? s.cpg : s.cpd, other = s.cpg < s.cpd ? s.cpd : s.cpg;
  if (other % unit != 0) return false;   // groups that do not nest keep the general kernels
  const int unit_p = round_up32(unit), opg_p = round_up32(s.opg);
  if (unit_p == unit && opg_p == s.opg) return false;
  // Which small layers pay for the copies, measured on [2, C, 64^3] .. [2, C, 4^3] with 3^3 taps: the general kernels'
  // time grows with Cin x Cout (8 -> 8 channels on 64^3: 1.9 ms forward, 40 ms backward, against 0.5 and 2.7 ms padded
  // to 32 channels; 3 -> 8 on 32^3: 1.9 -> 0.9 ms per training step; even on a 4^3 volume 0.3 -> 0.06 ms forward), and
  // only below 16 weights per tap are they the faster ones (1 -> 1 and 1 -> 8 channels: 0.35 against 1.1 ms forward
  // in fp32) -- those stay, which also keeps fp32 columns for layers whose one or two weight gradients are sums
  // that may nearly cancel.  bf16 layers stay below 256 as before: with 8-bit products such a weight gradient was
  // off by several per cent of itself in random layers.
  if (static_cast<long>(s.Cin) * s.Cout < (dtype == MV_BF16 ? 256 : 16)) return false;
  DcnDims p = s;
  p.cpg = s.cpg / unit * unit_p;
  p.cpd = s.cpd / unit * unit_p;
  p.Cin = s.Cin / unit * unit_p;
  p.opg = opg_p;
  p.Cout = s.groups * opg_p;
  pad.p = p;
  pad.unit = unit; pad.unit_p = unit_p;
  pad.on = true;
  return true;
}

// dst [B, C / unit * unit_p, P] <- src [B, C, P]; elements moved as integers of their size
template <typename U>
__global__ __launch_bounds__(256) void dcn_pad_channels_kernel(const U *__restrict__ src, U *__restrict__ dst,
                                                               int Cp, long P, int unit, int unit_p, int C, long n) {
  for (long i = blockIdx.x * 256L + threadIdx.x; i < n; i += gridDim.x * 256L) {
    const long row = i / P, pos = i - row * P;
    const int cp = static_cast<int>(row % Cp);
    const long b = row / Cp;
    const int u = cp / unit_p, r = cp - u * unit_p;
    dst[i] = r < unit ? src[(b * C + u * unit + r) * P + pos] : U(0);
  }
}

int dcn_pad_channels(const void *src, void *dst, int B, int C, long P, int unit, int unit_p, int es, hipStream_t stream) {
  const int Cp = C / unit * unit_p;
  const long n = static_cast<long>(B) * Cp * P;
  const dim3 grid(static_cast<unsigned>(std::min<long>((n + 1023) / 1024, 1 << 20)));
  if (es == 2)
    hipLaunchKernelGGL((dcn_pad_channels_kernel<unsigned short>), grid, dim3(256), 0, stream,
                       static_cast<const unsigned short *>(src), static_cast<unsigned short *>(dst), Cp, P, unit, unit_p, C, n);
  else
    hipLaunchKernelGGL((dcn_pad_channels_kernel<unsigned int>), grid, dim3(256), 0, stream,
                       static_cast<const unsigned int *>(src), static_cast<unsigned int *>(dst), Cp, P, unit, unit_p, C, n);
  return check_launch("dcn_pad_channels_kernel");
}

// dst [Cout_p, cpg_p, K] <- src [Cout, cpg, K]
template <typename U>
__global__ __launch_bounds__(256) void dcn_pad_weight_kernel(const U *__restrict__ src, U *__restrict__ dst,
                                                             const DcnDims s, const DcnDims p, int unit, int unit_p) {
  const long n = static_cast<long>(p.Cout) * p.cpg * p.K;
  for (long i = blockIdx.x * 256L + threadIdx.x; i < n; i += gridDim.x * 256L) {
    const int k = static_cast<int>(i % p.K);
    const long oc = i / p.K;
    const int clp = static_cast<int>(oc % p.cpg), op = static_cast<int>(oc / p.cpg);
    const int g = op / p.opg, ol = op - g * p.opg;
    const int u = clp / unit_p, r = clp - u * unit_p;
    const bool real = ol < s.opg && r < unit;
    dst[i] = real ? src[(static_cast<long>(g * s.opg + ol) * s.cpg + u * unit + r) * s.K + k] : U(0);
  }
}

int dcn_pad_weight(const void *src, void *dst, const DcnDims &s, const DcnPad &pad, int es, hipStream_t stream) {
  const long n = static_cast<long>(pad.p.Cout) * pad.p.cpg * pad.p.K;
  const dim3 grid(static_cast<unsigned>(std::min<long>((n + 255) / 256, 65536)));
  if (es == 2)
    hipLaunchKernelGGL((dcn_pad_weight_kernel<unsigned short>), grid, dim3(256), 0, stream,
                       static_cast<const unsigned short *>(src), static_cast<unsigned short *>(dst), s, pad.p, pad.unit, pad.unit_p);
  else
    hipLaunchKernelGGL((dcn_pad_weight_kernel<unsigned int>), grid, dim3(256), 0, stream,
                       static_cast<const unsigned int *>(src), static_cast<unsigned int *>(dst), s, pad.p, pad.unit, pad.unit_p);
  return check_launch("dcn_pad_weight_kernel");
}

// dst [B, C, P] <- the real channels of src [B, C / unit * unit_p, P]
template <typename U>
__global__ __launch_bounds__(256) void dcn_unpad_channels_kernel(const U *__restrict__ src, U *__restrict__ dst,
                                                                 int C, long P, int unit, int unit_p, long n) {
  const int Cp = C / unit * unit_p;
  for (long i = blockIdx.x * 256L + threadIdx.x; i < n; i += gridDim.x * 256L) {
    const long row = i / P, pos = i - row * P;
    const int c = static_cast<int>(row % C);
    const long b = row / C;
    const int u = c / unit, r = c - u * unit;
    dst[i] = src[(b * Cp + u * unit_p + r) * P + pos];
  }
}

int dcn_unpad_channels(const void *src, void *dst, int B, int C, long P, int unit, int unit_p, int es, hipStream_t stream) {
  const long n = static_cast<long>(B) * C * P;
  const dim3 grid(static_cast<unsigned>(std::min<long>((n + 1023) / 1024, 1 << 20)));
  if (es == 2)
    hipLaunchKernelGGL((dcn_unpad_channels_kernel<unsigned short>), grid, dim3(256), 0, stream,
                       static_cast<const unsigned short *>(src), static_cast<unsigned short *>(dst), C, P, unit, unit_p, n);
  else
    hipLaunchKernelGGL((dcn_unpad_channels_kernel<unsigned int>), grid, dim3(256), 0, stream,
                       static_cast<const unsigned int *>(src), static_cast<unsigned int *>(dst), C, P, unit, unit_p, n);
  return check_launch("dcn_unpad_channels_kernel");
}

// gx [B, C, P] (T) += the real channels of gxt [B, P, C / unit * unit_p] (fp32, channels-last);
// 64 positions x 64 real channels per workgroup through LDS
template <typename T>
__global__ __launch_bounds__(256) void dcn_planar_add_padded_kernel(const float *__restrict__ gxt, T *__restrict__ gx,
                                                                    int C, long P, int unit, int unit_p) {
  __shared__ float stagef[64][65];
  const int Cp = C / unit * unit_p;
  const int b = blockIdx.y;
  const long p0 = static_cast<long>(blockIdx.x) * 64;
  const int c0 = blockIdx.z * 64, cn = min(64, C - c0);
  const int count = static_cast<int>(min(static_cast<long>(64), P - p0)) * cn;
  const float *src = gxt + (static_cast<long>(b) * P + p0) * Cp;
  for (int i = threadIdx.x; i < count; i += 256) {
    const int pp = i / cn, c = c0 + i % cn;
    const int u = c / unit, r = c - u * unit;
    stagef[pp][i % cn] = src[static_cast<long>(pp) * Cp + u * unit_p + r];
  }
  __syncthreads();
  const int lp = threadIdx.x % 64;
  if (p0 + lp < P)
    for (int c = threadIdx.x / 64; c < cn; c += 4) {
      T *d = gx + (static_cast<long>(b) * C + c0 + c) * P + p0 + lp;
      *d = store_cast<T>(load(d) + stagef[lp][c]);
    }
}

int dcn_planar_add_padded(const float *gxt, void *gx, const DcnDims &s, const DcnPad &pad, int dtype, hipStream_t stream) {
  const long pblocks = (s.P + 63) / 64;
  MV_REQUIRE(pblocks < (1L << 31) && s.B <= 65535 && (s.Cin + 63) / 64 <= 65535, "volume too large");
  const dim3 grid(static_cast<unsigned>(pblocks), s.B, (s.Cin + 63) / 64);
  if (dtype == MV_F16)
    hipLaunchKernelGGL((dcn_planar_add_padded_kernel<__half>), grid, dim3(256), 0, stream, gxt, static_cast<__half *>(gx),
                       s.Cin, s.P, pad.unit, pad.unit_p);
  else if (dtype == MV_F32)
    hipLaunchKernelGGL((dcn_planar_add_padded_kernel<float>), grid, dim3(256), 0, stream, gxt, static_cast<float *>(gx),
                       s.Cin, s.P, pad.unit, pad.unit_p);
  else
    hipLaunchKernelGGL((dcn_planar_add_padded_kernel<__hip_bfloat16>), grid, dim3(256), 0, stream, gxt,
                       static_cast<__hip_bfloat16 *>(gx), s.Cin, s.P, pad.unit, pad.unit_p);
  return check_launch("dcn_planar_add_padded_kernel");
}

// grad_weight [Cout][cpg][K] (T) += the real entries of the tap-major fp32 accumulator
// [K][Cout_p][cpg_p] of the padded layer; grad_bias [Cout] += the real entries of gb [Cout_p]
template <typename T>
__global__ __launch_bounds__(256) void dcn_weight_add_padded_kernel(const float *__restrict__ acc, T *__restrict__ gw,
                                                                    const float *__restrict__ gb_acc, T *__restrict__ gb,
                                                                    const DcnDims s, const DcnDims p, int unit, int unit_p) {
  const long n = static_cast<long>(s.Cout) * s.cpg * s.K;
  for (long i = blockIdx.x * 256L + threadIdx.x; i < n; i += gridDim.x * 256L) {
    const int k = static_cast<int>(i % s.K);
    const long oc = i / s.K;
    const int cl = static_cast<int>(oc % s.cpg), o = static_cast<int>(oc / s.cpg);
    const int g = o / s.opg, ol = o - g * s.opg;
    const int u = cl / unit, r = cl - u * unit;
    gw[i] = store_cast<T>(load(gw + i) + acc[(static_cast<long>(k) * p.Cout + g * p.opg + ol) * p.cpg + u * unit_p + r]);
  }
  if (gb != nullptr)
    for (long o = blockIdx.x * 256L + threadIdx.x; o < s.Cout; o += gridDim.x * 256L) {
      const int g = static_cast<int>(o) / s.opg, ol = static_cast<int>(o) - g * s.opg;
      gb[o] = store_cast<T>(load(gb + o) + gb_acc[g * p.opg + ol]);
    }
}

int dcn_weight_add_padded(const float *acc, void *gw, const float *gb_acc, void *gb, const DcnDims &s,
                          const DcnPad &pad, int dtype, hipStream_t stream) {
  const long n = static_cast<long>(s.Cout) * s.cpg * s.K;
  const dim3 grid(static_cast<unsigned>(std::min<long>((n + 255) / 256, 4096L)));
  if (dtype == MV_F16)
    hipLaunchKernelGGL((dcn_weight_add_padded_kernel<__half>), grid, dim3(256), 0, stream, acc, static_cast<__half *>(gw),
                       gb_acc, static_cast<__half *>(gb), s, pad.p, pad.unit, pad.unit_p);
  else if (dtype == MV_F32)
    hipLaunchKernelGGL((dcn_weight_add_padded_kernel<float>), grid, dim3(256), 0, stream, acc, static_cast<float *>(gw),
                       gb_acc, static_cast<float *>(gb), s, pad.p, pad.unit, pad.unit_p);
  else
    hipLaunchKernelGGL((dcn_weight_add_padded_kernel<__hip_bfloat16>), grid, dim3(256), 0, stream, acc,
                       static_cast<__hip_bfloat16 *>(gw), gb_acc, static_cast<__hip_bfloat16 *>(gb), s, pad.p, pad.unit,
                       pad.unit_p);
  return check_launch("dcn_weight_add_padded_kernel");
}

}  // namespace mv
