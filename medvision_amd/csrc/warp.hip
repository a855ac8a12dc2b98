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
  // Images (one slice: the four taps of the upper slice have weight 0 and are not loaded) in 16-bit types:
  // the two x taps of a row are neighbours in memory and come in one 4-byte load at 2-byte alignment; where
  // they collapse onto one pixel (the last column) the high tap has weight 0 and the low pixel stands in for
  // it.  (Measured on [8,3,512,512] fp16: 0.048 -> 0.023 ms, both together.  For volumes the paired loads
  // were slower, 0.031 -> 0.036 ms on [2,1,128^3], and are not used.)
  const bool pairs = sizeof(T) == 2 && cw.idx[1] == cw.idx[0] + 1;
  for (int c = 0; c < C; c++) {
    const long base = (static_cast<long>(b) * C + c) * P;
    A v = A(0);
    if (live) {
      const T *plane = img + base;
      if (ndim == 2) {
#pragma unroll
        for (int n = 0; n < 4; n += 2) {
          T lo, hi;
          if constexpr (sizeof(T) == 2) {
            if (pairs) {
              unsigned two;
              __builtin_memcpy(&two, plane + cw.idx[n], sizeof(two));
              const unsigned short l = static_cast<unsigned short>(two & 0xffffu), h = static_cast<unsigned short>(two >> 16);
              __builtin_memcpy(&lo, &l, sizeof(l));
              __builtin_memcpy(&hi, &h, sizeof(h));
            } else {
              lo = plane[cw.idx[n]]; hi = plane[cw.idx[n + 1]];
            }
          } else {
            lo = plane[cw.idx[n]]; hi = plane[cw.idx[n + 1]];
          }
          v += cw.w[n] * load(&lo);
          v += cw.w[n + 1] * load(&hi);
        }
      } else {
#pragma unroll
        for (int n = 0; n < 8; n++) v += cw.w[n] * load(plane + cw.idx[n]);
      }
    }
    out[base + q] = store_cast<T>(v);
  }
}

// Order 0 on int32 label maps with fp32 offsets: the voxel the float path picks (low index when
// 1 - frac >= 0.5, csrc/cuda/interpolation_helpers_3d.h:186-194), copied as an integer.
__global__ __launch_bounds__(256) void deform_warp_labels_kernel(const int *__restrict__ img,
                                                                 const float *__restrict__ off,
                                                                 int *__restrict__ out, int ndim, int C,
                                                                 int D, int H, int W) {
  const long P = static_cast<long>(D) * H * W;
  const long q = blockIdx.x * 256L + threadIdx.x;
  const int b = blockIdx.y;
  if (q >= P) return;
  const int w = q % W, h = (q / W) % H, d = q / (static_cast<long>(W) * H);
  const float *o = off + static_cast<long>(b) * ndim * P + q;
  const double pd = ndim == 3 ? d + static_cast<double>(o[0]) : 0.0;
  const double ph = h + static_cast<double>(o[(ndim - 2) * P]);
  const double pw = w + static_cast<double>(o[(ndim - 1) * P]);
  bool ok = ph > -1.0 && pw > -1.0 && ph < H && pw < W && (ndim == 2 || (pd > -1.0 && pd < D));
  int z0 = 0, z1 = 0, y0 = 0, y1 = 0, x0 = 0, x1 = 0;
  float lz = 0.f, ly = 0.f, lx = 0.f;
  ok = ok && clamped_tap<float>(pd, D, z0, z1, lz, 0) && clamped_tap<float>(ph, H, y0, y1, ly, 0) &&
       clamped_tap<float>(pw, W, x0, x1, lx, 0);
  const long at = (static_cast<long>(lz == 0.f ? z0 : z1) * H + (ly == 0.f ? y0 : y1)) * W + (lx == 0.f ? x0 : x1);
  for (int c = 0; c < C; c++) {
    const long base = (static_cast<long>(b) * C + c) * P;
    out[base + q] = ok ? img[base + at] : 0;
  }
}

// Order 3 for volumes: 64 taps per sample make the plain kernel above a stream of scattered 2-byte
// global loads.  Here a workgroup owns a tile of TX x TY x TZ positions (a thread: one column along
// z), finds the box of source voxels its samples touch (minimum and maximum of floor(p) over the
// tile, one voxel below and two above, clipped to the volume), copies that box of one channel at a
// time to LDS and takes the taps from there.  Tiles whose box does not fit (very large
// displacements) sample from global memory as above.  Same arithmetic as sample_cubic.
template <typename T, int TX, int TY, int TZ, int LDS_BYTES>
__global__ __launch_bounds__(TX * TY, 4) void deform_warp_cubic_tiled_kernel(
    const T *__restrict__ img, const T *__restrict__ off, T *__restrict__ out, int C, int D, int H, int W,
    int tiles_z) {
  using A = typename Acc<T>::type;
  constexpr int THREADS = TX * TY, kCap = LDS_BYTES / static_cast<int>(sizeof(T));
  __shared__ T tile[kCap];
  __shared__ int lo_s[3], hi_s[3];
  const int tid = threadIdx.x, lx = tid % TX, ly = tid / TX;
  const int b = blockIdx.z / tiles_z, tz = blockIdx.z % tiles_z;
  const int x = blockIdx.x * TX + lx, y = blockIdx.y * TY + ly, z0 = tz * TZ;
  const long P = static_cast<long>(D) * H * W, HW = static_cast<long>(H) * W;
  const bool in_xy = x < W && y < H;
  if (tid < 3) { lo_s[tid] = 1 << 30; hi_s[tid] = -(1 << 30); }
  __syncthreads();
  // sample positions of this thread's column (fp64: grid position + offset is exact there)
  float oz[TZ], oy[TZ], ox[TZ];   // the offsets (exact in fp32 for every storage type)
  bool ok[TZ];
  int mn[3] = {1 << 30, 1 << 30, 1 << 30}, mx[3] = {-(1 << 30), -(1 << 30), -(1 << 30)};
#pragma unroll
  for (int k = 0; k < TZ; k++) {
    const int z = z0 + k;
    ok[k] = in_xy && z < D;
    oz[k] = oy[k] = ox[k] = 0.f;
    double pz = 0.0, py = 0.0, px = 0.0;
    if (ok[k]) {
      const T *o = off + static_cast<long>(b) * 3 * P + (static_cast<long>(z) * H + y) * W + x;
      oz[k] = static_cast<float>(load(o)); oy[k] = static_cast<float>(load(o + P)); ox[k] = static_cast<float>(load(o + 2 * P));
      pz = z + static_cast<double>(oz[k]); py = y + static_cast<double>(oy[k]); px = x + static_cast<double>(ox[k]);
      ok[k] = pz > -1.0 && py > -1.0 && px > -1.0 && pz < D && py < H && px < W;
    }
    if (ok[k]) {
      const int f[3] = {static_cast<int>(fmax(px, 0.0)), static_cast<int>(fmax(py, 0.0)), static_cast<int>(fmax(pz, 0.0))};
#pragma unroll
      for (int a = 0; a < 3; a++) { mn[a] = min(mn[a], f[a]); mx[a] = max(mx[a], f[a]); }
    }
  }
#pragma unroll
  for (int a = 0; a < 3; a++) {
    if (mn[a] <= mx[a]) { atomicMin(&lo_s[a], mn[a]); atomicMax(&hi_s[a], mx[a]); }
  }
  __syncthreads();
  const int size[3] = {W, H, D};
  int lo[3], n[3];
  bool any = true;
#pragma unroll
  for (int a = 0; a < 3; a++) {
    any = any && lo_s[a] <= hi_s[a];
    lo[a] = max(lo_s[a] - 1, 0);
    n[a] = min(hi_s[a] + 2, size[a] - 1) - lo[a] + 1;
  }
  const bool fits = any && static_cast<long>(n[0]) * n[1] * n[2] <= kCap;
  const int rows = fits ? n[1] * n[2] : 0;
  for (int c = 0; c < C; c++) {
    const T *plane = img + (static_cast<long>(b) * C + c) * P;
    T *oplane = out + (static_cast<long>(b) * C + c) * P;
    if (fits) {
      // element i of the box = (row i / n0, column i % n0); eight independent loads in flight per
      // thread (small integers: the float quotients are exact)
      const int total = rows * n[0];
      const float inv0 = 1.0f / static_cast<float>(n[0]), inv1 = 1.0f / static_cast<float>(n[1]);
      const T *corner = plane + (static_cast<long>(lo[2]) * H + lo[1]) * W + lo[0];
      for (int i0 = tid; i0 < total; i0 += THREADS * 8) {
        T v8[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
          const int i = i0 + u * THREADS;
          if (i < total) {
            const int r = static_cast<int>((static_cast<float>(i) + 0.5f) * inv0), e = i - r * n[0];
            const int zz = static_cast<int>((static_cast<float>(r) + 0.5f) * inv1), yy = r - zz * n[1];
            v8[u] = corner[(static_cast<long>(zz) * H + yy) * W + e];
          }
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
          const int i = i0 + u * THREADS;
          if (i < total) tile[i] = v8[u];
        }
      }
      __syncthreads();
    }
#pragma unroll 1
    for (int k = 0; k < TZ; k++) {
      if (!(in_xy && z0 + k < D)) continue;
      A v = A(0);
      if (ok[k]) {
        const double pz = z0 + k + static_cast<double>(oz[k]), py = y + static_cast<double>(oy[k]),
                     px = x + static_cast<double>(ox[k]);
        if (fits) {
          int zi[4], yi[4], xi[4];
          A wz[4], wy[4], wx[4];
          cubic_tap<A>(pz, D, zi, wz);
          cubic_tap<A>(py, H, yi, wy);
          cubic_tap<A>(px, W, xi, wx);
#pragma unroll
          for (int j = 0; j < 4; j++) { zi[j] = (zi[j] - lo[2]) * n[1]; yi[j] -= lo[1]; xi[j] -= lo[0]; }
#pragma unroll
          for (int a = 0; a < 4; a++) {
            A slab = A(0);
#pragma unroll
            for (int bb = 0; bb < 4; bb++) {
              const T *row = tile + (zi[a] + yi[bb]) * n[0];
              slab += wy[bb] * (wx[0] * load(row + xi[0]) + wx[1] * load(row + xi[1]) +
                                wx[2] * load(row + xi[2]) + wx[3] * load(row + xi[3]));
            }
            v += wz[a] * slab;
          }
        } else {
          v = sample_cubic<T>(plane, 3, D, H, W, pz, py, px);
        }
      }
      oplane[(static_cast<long>(z0 + k) * H + y) * W + x] = store_cast<T>(v);
    }
    if (fits && c + 1 < C) __syncthreads();   // the box may be overwritten
  }
  (void)HW;
}

template <typename T>
static int launch_warp_cubic_tiled(const void *img, const void *offset, void *output, int batch, int channels,
                                   int depth, int height, int width, hipStream_t stream) {
  constexpr int TX = 16, TY = 16, TZ = 8, LDS = 40000;
  const int tx = (width + TX - 1) / TX, ty = (height + TY - 1) / TY, tz = (depth + TZ - 1) / TZ;
  MV_REQUIRE(ty <= 65535 && static_cast<long>(tz) * batch <= 65535, "volume too large");
  hipLaunchKernelGGL((deform_warp_cubic_tiled_kernel<T, TX, TY, TZ, LDS>), dim3(tx, ty, tz * batch), dim3(TX * TY), 0,
                     stream, static_cast<const T *>(img), static_cast<const T *>(offset), static_cast<T *>(output),
                     channels, depth, height, width, tz);
  return check_launch("deform_warp_cubic_tiled_kernel");
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
  if (dtype == MV_I32) {
    MV_REQUIRE(order == 0, "int32 label maps are warped at order 0 only (got %d)", order);
    hipLaunchKernelGGL(deform_warp_labels_kernel, dim3(static_cast<unsigned>((P + 255) / 256), batch), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const int *>(img),
                       static_cast<const float *>(offset), static_cast<int *>(output), ndim, channels, depth,
                       height, width);
    return check_launch("deform_warp_labels_kernel");
  }
  if (order == 3 && ndim == 3 && P >= 4096 && dtype != MV_F64) {
    const int th = (height + 15) / 16;
    const long tzb = static_cast<long>((depth + 7) / 8) * batch;
    if (th <= 65535 && tzb <= 65535) {
      hipStream_t st = static_cast<hipStream_t>(stream);
      if (dtype == MV_F16) return launch_warp_cubic_tiled<__half>(img, offset, output, batch, channels, depth, height, width, st);
      if (dtype == MV_BF16) return launch_warp_cubic_tiled<__hip_bfloat16>(img, offset, output, batch, channels, depth, height, width, st);
      if (dtype == MV_F32) return launch_warp_cubic_tiled<float>(img, offset, output, batch, channels, depth, height, width, st);
    }
  }
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
