// Displacement-field warp: out[b,c,q] = S(img[b,c], q + off[b,:,q]) for -1 < p < size, else 0,
// with S the border-replicating sampler (order 0 / 1) or the clamped Catmull-Rom one (order 3).  This is what the reference obtains from
// its augmentation DCN with a 1x1x1 kernel and an identity weight (ops/cuda_fun_tools.py:94-167,
// csrc/cuda_aug/deform_3d_cuda_kernel.cuh:58-85) -- here without the column matrix, the C x C
// GEMM and the permute copy.  One thread owns one voxel position and reuses its taps for all
// channels; lanes run along W so offset loads and output stores are coalesced.
#include "common.hpp"
#include "sampling.hpp"

namespace mv {

template <typename T>
__global__ __launch_bounds__(256) void deform_warp_kernel(const T *__restrict__ img,
                                                          const T *__restrict__ off,
                                                          T *__restrict__ out, int ndim, int C,
                                                          int D, int H, int W, int order) {
  using A = typename Acc<T>::type;
  const long P = static_cast<long>(D) * H * W;
  const long q = blockIdx.x * 256L + threadIdx.x;
  const int b = blockIdx.y;
  if (q >= P) return;
  const int w = q % W, h = (q / W) % H, d = q / (static_cast<long>(W) * H);
  const T *o = off + static_cast<long>(b) * ndim * P + q;
  const double pd = ndim == 3 ? d + static_cast<double>(load(o)) : 0.0;
  const double ph = h + static_cast<double>(load(o + (ndim - 2) * P));
  const double pw = w + static_cast<double>(load(o + (ndim - 1) * P));
  const bool ok = ph > -1.0 && pw > -1.0 && ph < H && pw < W && (ndim == 2 || (pd > -1.0 && pd < D));
  if (order == 3) {
    for (int c = 0; c < C; c++) {
      const long base = (static_cast<long>(b) * C + c) * P;
      out[base + q] =
          store_cast<T>(ok ? sample_cubic<T>(img + base, ndim, D, H, W, pd, ph, pw) : A(0));
    }
    return;
  }
  Corners<A> cw;
  const bool live = ok && clamped_corners<A>(D, H, W, pd, ph, pw, order, cw);
  for (int c = 0; c < C; c++) {
    const long base = (static_cast<long>(b) * C + c) * P;
    A v = A(0);
    if (live) {
      const T *plane = img + base;
#pragma unroll
      for (int n = 0; n < 8; n++) v += cw.w[n] * load(plane + cw.idx[n]);
    }
    out[base + q] = store_cast<T>(v);
  }
}

static int deform_warp(const void *img, const void *offset, void *output, int dtype, int ndim,
                       int batch, int channels, int depth, int height, int width, int order,
                       void *stream) {
  MV_REQUIRE(batch > 0 && channels > 0 && depth > 0 && height > 0 && width > 0,
             "tensor dims must be positive");
  MV_REQUIRE(order == 0 || order == 1 || order == 3,
             "order %d is not supported (0 nearest, 1 linear, 3 cubic)", order);
  MV_REQUIRE(img && offset && output, "null pointer argument");
  const long P = static_cast<long>(depth) * height * width;
  MV_REQUIRE(P < (1L << 31) && batch <= 65535, "volume too large");
  const dim3 grid(static_cast<unsigned>((P + 255) / 256), batch), block(256);
  MV_DISPATCH(dtype, {
    hipLaunchKernelGGL((deform_warp_kernel<T>), grid, block, 0, static_cast<hipStream_t>(stream),
                       static_cast<const T *>(img), static_cast<const T *>(offset),
                       static_cast<T *>(output), ndim, channels, depth, height, width, order);
  });
  return check_launch("deform_warp_kernel");
}

}  // namespace mv

extern "C" {

int mv_deform_warp_2d(const void *img, const void *offset, void *output, int dtype, int batch,
                      int channels, int height, int width, int order, void *stream) {
  return mv::deform_warp(img, offset, output, dtype, 2, batch, channels, 1, height, width, order, stream);
}

int mv_deform_warp_3d(const void *img, const void *offset, void *output, int dtype, int batch,
                      int channels, int depth, int height, int width, int order, void *stream) {
  return mv::deform_warp(img, offset, output, dtype, 3, batch, channels, depth, height, width, order,
                         stream);
}

}  // extern "C"
