// RoIAlign / RoIAlignRotated 2-D and 3-D, forward and backward: general-shape kernels.
//
// Work decomposition: one workgroup = (one roi, one chunk of kChunk consecutive output elements
// of that roi in [C, od, oh, ow] order).  Lane 0 turns the roi row into the sample-grid geometry
// (fp64, 3 sincos) once per workgroup and shares it through LDS, so the per-element work is only
// the sample loop.  Consecutive lanes own consecutive pw, so output stores (forward) and
// grad_output loads (backward) are coalesced along W.
#include "common.hpp"
#include "roi_geometry.hpp"
#include "sampling.hpp"

namespace mv {

constexpr int kRoiThreads = 256;
constexpr int kRoiChunk = kRoiThreads * 4;

template <typename T, typename RT, bool ROT>
__global__ __launch_bounds__(kRoiThreads) void roi_forward_kernel(const T *__restrict__ feat,
                                                                  const RT *__restrict__ rois,
                                                                  T *__restrict__ out,
                                                                  const RoiProblem p) {
  using A = typename Acc<T>::type;
  __shared__ RoiGeom g;
  __shared__ double trig[6];
  const unsigned n = blockIdx.x / p.chunks, chunk = blockIdx.x % p.chunks;
  build_geom_block(g, trig, rois + static_cast<long>(n) * roi_columns(p.ndim, p.rotated), p);
  const unsigned begin = chunk * kRoiChunk;
  const unsigned end = min(begin + kRoiChunk, p.per_roi);
  const long plane = static_cast<long>(p.D) * p.H * p.W;
  const int gz = p.ndim == 3 ? g.grid[2] : 1, gy = g.grid[1], gx = g.grid[0];
  for (unsigned e = begin + threadIdx.x; e < end; e += kRoiThreads) {
    const unsigned pw = e % p.ow, t1 = e / p.ow;
    const unsigned ph = t1 % p.oh, t2 = t1 / p.oh;
    const unsigned pd = t2 % p.od, c = t2 / p.od;
    A acc = A(0);
    if (g.batch >= 0) {
      const T *src = feat + (static_cast<long>(g.batch) * p.C + c) * plane;
      for (int iz = 0; iz < gz; iz++) {
        const double z = p.ndim == 3 ? local_coord(g, 2, pd, iz) : 0.0;
        for (int iy = 0; iy < gy; iy++) {
          const double y = local_coord(g, 1, ph, iy);
          for (int ix = 0; ix < gx; ix++) {
            const double x = local_coord(g, 0, pw, ix);
            double rx = x, ry = y, rz = z;
            if (ROT) {
              rx = g.rot[0] * x + g.rot[1] * y + g.rot[2] * z + g.centre[0];
              ry = g.rot[3] * x + g.rot[4] * y + g.rot[5] * z + g.centre[1];
              rz = p.ndim == 3 ? g.rot[6] * x + g.rot[7] * y + g.rot[8] * z + g.centre[2] : 0.0;
            }
            acc += p.order == 3 ? sample_cubic<T>(src, p.ndim, p.D, p.H, p.W, rz, ry, rx)
                                : sample_clamped<T>(src, p.D, p.H, p.W, rz, ry, rx, p.order);
          }
        }
      }
    }
    out[static_cast<long>(n) * p.per_roi + e] = store_cast<T>(acc / static_cast<A>(g.count));
  }
}

// G = element type of the accumulation buffer (T itself for fp32/fp64, float for 16-bit T).
template <typename T, typename G, typename RT, bool ROT>
__global__ __launch_bounds__(kRoiThreads) void roi_backward_kernel(const T *__restrict__ gout,
                                                                   const RT *__restrict__ rois,
                                                                   G *__restrict__ gin,
                                                                   const RoiProblem p) {
  using A = typename Acc<T>::type;
  __shared__ RoiGeom g;
  __shared__ double trig[6];
  // a contiguous eighth of the chunks per XCD: the atomics of neighbouring chunks then meet in
  // fewer places at a time (11 % faster on large outputs; the forward kernel lost by it)
  const unsigned wg = xcd_contiguous(blockIdx.x, gridDim.x);
  const unsigned n = wg / p.chunks, chunk = wg % p.chunks;
  build_geom_block(g, trig, rois + static_cast<long>(n) * roi_columns(p.ndim, p.rotated), p);
  if (g.batch < 0) return;
  const unsigned begin = chunk * kRoiChunk;
  const unsigned end = min(begin + kRoiChunk, p.per_roi);
  const long plane = static_cast<long>(p.D) * p.H * p.W;
  const int gz = p.ndim == 3 ? g.grid[2] : 1, gy = g.grid[1], gx = g.grid[0];
  for (unsigned e = begin + threadIdx.x; e < end; e += kRoiThreads) {
    const unsigned pw = e % p.ow, t1 = e / p.ow;
    const unsigned ph = t1 % p.oh, t2 = t1 / p.oh;
    const unsigned pd = t2 % p.od, c = t2 / p.od;
    const A top = load(gout + static_cast<long>(n) * p.per_roi + e) / static_cast<A>(g.count);
    G *dst = gin + (static_cast<long>(g.batch) * p.C + c) * plane;
    for (int iz = 0; iz < gz; iz++) {
      const double z = p.ndim == 3 ? local_coord(g, 2, pd, iz) : 0.0;
      for (int iy = 0; iy < gy; iy++) {
        const double y = local_coord(g, 1, ph, iy);
        for (int ix = 0; ix < gx; ix++) {
          const double x = local_coord(g, 0, pw, ix);
          double rx = x, ry = y, rz = z;
          if (ROT) {
            rx = g.rot[0] * x + g.rot[1] * y + g.rot[2] * z + g.centre[0];
            ry = g.rot[3] * x + g.rot[4] * y + g.rot[5] * z + g.centre[1];
            rz = p.ndim == 3 ? g.rot[6] * x + g.rot[7] * y + g.rot[8] * z + g.centre[2] : 0.0;
          }
          Corners<A> cw;
          if (!clamped_corners<A>(p.D, p.H, p.W, rz, ry, rx, p.order, cw)) continue;
#pragma unroll
          for (int k = 0; k < 8; k++)
            if (cw.w[k] != A(0)) atomic_add(dst + cw.idx[k], static_cast<G>(top * cw.w[k]));
        }
      }
    }
  }
}

__global__ void fill_zero_kernel(float *p, long n) {
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<long>(gridDim.x) * blockDim.x)
    p[i] = 0.f;
}

template <typename T>
__global__ void add_from_f32_kernel(T *dst, const float *src, long n) {
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<long>(gridDim.x) * blockDim.x)
    dst[i] = store_cast<T>(load(dst + i) + src[i]);
}

// roi_resample.hip: tiled LDS-staged forward; returns -1 when it does not apply
int roi_forward_tiled(const void *input, const void *rois, void *output, int dtype,
                      const RoiProblem &p, void *workspace, size_t capacity, size_t *need, hipStream_t s);

// roi_resample.hip: backward of the same problems through LDS tiles of the source boxes; `acc` is the
// fp32 buffer the gradient is added to; -1 when it does not apply
bool roi_backward_tiled_applies(int dtype, const RoiProblem &p);
int roi_backward_tiled(const void *grad_output, const void *rois, void *acc, int dtype,
                       const RoiProblem &p, hipStream_t s, bool direct = false);
// fp16 gradients with even rows: the tiles add to the gradient tensor itself (packed atomics on pairs)
bool roi_backward_tiled_direct(int dtype, const RoiProblem &p, const void *grad_input);

// roi_pool.hip: separable LDS kernels for plain boxes with small outputs; -1 when not applicable
size_t roi_pool_forward_workspace(int dtype, const RoiProblem &p);
int roi_pool_forward(const void *input, const void *rois, void *output, int dtype,
                     const RoiProblem &p, void *workspace, size_t capacity, hipStream_t s,
                     const void *prepared = nullptr);
// the re-ordered copy of the features alone (callers that pool one feature map several times)
size_t roi_pool_prepared_bytes(int dtype, const RoiProblem &p);
int roi_pool_prepare(const void *input, int dtype, const RoiProblem &p, void *prepared, size_t capacity, hipStream_t s);
int roi_pool_backward(const void *grad_output, const void *rois, void *acc, int dtype,
                      const RoiProblem &p, hipStream_t s, bool channels_last);
bool roi_pool_applies(int dtype, const RoiProblem &p);
// roi_gather_backward.hip: atomic-free backward for resampling-sized problems; -1 when not applicable
// roi_box.hip: backward of small outputs that the pooled kernels do not take (rotated boxes, large
// grids), one workgroup per (roi, channel group) with LDS tiles of the source boxes; -1 when not applicable
int roi_box_backward(const void *grad_output, const void *rois, float *acc, int dtype, const RoiProblem &p, hipStream_t s);
// Many small outputs over wide feature maps, read from a channels-last copy in the workspace (roi_cl.hip).
size_t roi_forward_cl_workspace(int dtype, const RoiProblem &p);
int roi_forward_cl(const void *input, const void *rois, void *output, int dtype, const RoiProblem &p,
                   void *workspace, size_t capacity, hipStream_t s);

int roi_backward_gather(const void *grad_output, const void *rois, void *grad_input, int dtype,
                        const RoiProblem &p, hipStream_t s);
// dcn3d_mfma_backward.hip: dst [B, C, P] += src [B, P, C] fp32
int planar_add_f32(const float *src, void *dst, int B, int C, long P, int dtype, hipStream_t stream);

static int make_problem(RoiProblem &p, int ndim, int rotated, int batch, int channels, int depth,
                        int height, int width, int num_rois, int out_d, int out_h, int out_w,
                        float spatial_scale, int sampling_ratio, int aligned, int order,
                        bool cubic_ok = false) {
  MV_REQUIRE(batch > 0 && channels > 0 && depth > 0 && height > 0 && width > 0,
             "feature dims must be positive (got %d,%d,%d,%d,%d)", batch, channels, depth, height, width);
  MV_REQUIRE(num_rois >= 0, "num_rois must be >= 0");
  MV_REQUIRE(out_d > 0 && out_h > 0 && out_w > 0, "output size must be positive");
  MV_REQUIRE(order == 0 || order == 1 || (cubic_ok && order == 3),
             cubic_ok ? "order %d is not supported (0 nearest, 1 linear, 3 cubic)"
                      : "only support order = 0 (nearest) or 1 (linear), got %d", order);
  const long per_roi = static_cast<long>(channels) * out_d * out_h * out_w;
  MV_REQUIRE(per_roi < (1L << 31), "channels*out_d*out_h*out_w must be < 2^31");
  const long chunks = (per_roi + kRoiChunk - 1) / kRoiChunk;
  MV_REQUIRE(chunks * static_cast<long>(num_rois) < (1L << 31), "too many workgroups");
  p.ndim = ndim; p.rotated = rotated;
  p.N = batch; p.C = channels; p.D = depth; p.H = height; p.W = width; p.R = num_rois;
  p.od = out_d; p.oh = out_h; p.ow = out_w;
  p.scale = static_cast<double>(spatial_scale);
  p.sampling_ratio = sampling_ratio; p.aligned = aligned; p.order = order;
  p.per_roi = static_cast<unsigned>(per_roi);
  p.chunks = static_cast<unsigned>(chunks);
  return MV_OK;
}

int roi_forward(const void *input, const void *rois, void *output, int dtype, int ndim,
                int rotated, int batch, int channels, int depth, int height, int width,
                int num_rois, int out_d, int out_h, int out_w, float spatial_scale,
                int sampling_ratio, int aligned, int order, void *workspace, size_t workspace_bytes,
                void *stream, bool cubic_ok = false, const void *prepared = nullptr) {
  RoiProblem p;
  int st = make_problem(p, ndim, rotated, batch, channels, depth, height, width, num_rois, out_d,
                        out_h, out_w, spatial_scale, sampling_ratio, aligned, order, cubic_ok);
  if (st) return st;
  if (num_rois == 0) return MV_OK;
  MV_REQUIRE(input && rois && output, "null pointer argument");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == MV_I32) {
    // int32 label maps (the augmentation layer's segmentations): the voxel that order 0 picks, one sample per
    // cell.  The reference resamples a float copy of the map and converts back
    // (aug_cuda/aug_spatial.py: `.float()` ... `.int()`); here the two conversion passes happen in the loads
    // and stores of the kernel.
    MV_REQUIRE(order == 0 && sampling_ratio == 1 && prepared == nullptr,
               "int32 label maps are resampled at order 0 with a sampling grid of one");
    const int tiled = roi_forward_tiled(input, rois, output, dtype, p, workspace, workspace ? workspace_bytes : 0, nullptr, s);
    if (tiled >= 0) return tiled;
    const dim3 grid(p.chunks * num_rois), block(kRoiThreads);
    if (rotated)
      hipLaunchKernelGGL((roi_forward_kernel<int, float, true>), grid, block, 0, s, static_cast<const int *>(input),
                         static_cast<const float *>(rois), static_cast<int *>(output), p);
    else
      hipLaunchKernelGGL((roi_forward_kernel<int, float, false>), grid, block, 0, s, static_cast<const int *>(input),
                         static_cast<const float *>(rois), static_cast<int *>(output), p);
    return check_launch("roi_forward_kernel");
  }
  {
    // (a workspace too small for a path selects the kernels that need none)
    const size_t capacity = workspace ? workspace_bytes : 0;
    if (prepared != nullptr) {   // (a copy the pooled kernels have no use for is left alone)
      const int pooled = roi_pool_forward(input, rois, output, dtype, p, workspace, capacity, s, prepared);
      if (pooled >= 0) return pooled;
    }
    const int tiled = roi_forward_tiled(input, rois, output, dtype, p, workspace, capacity, nullptr, s);
    if (tiled >= 0) return tiled;
    const int pooled = order != 3 ? roi_pool_forward(input, rois, output, dtype, p, workspace, capacity, s) : -1;
    if (pooled >= 0) return pooled;
    const int wide = order != 3 ? roi_forward_cl(input, rois, output, dtype, p, workspace, capacity, s) : -1;
    if (wide >= 0) return wide;
  }
  const dim3 grid(p.chunks * num_rois), block(kRoiThreads);
  MV_DISPATCH(dtype, {
    using RT = typename std::conditional<std::is_same<T, double>::value, double, float>::type;
    if (rotated)
      hipLaunchKernelGGL((roi_forward_kernel<T, RT, true>), grid, block, 0, s,
                         static_cast<const T *>(input), static_cast<const RT *>(rois),
                         static_cast<T *>(output), p);
    else
      hipLaunchKernelGGL((roi_forward_kernel<T, RT, false>), grid, block, 0, s,
                         static_cast<const T *>(input), static_cast<const RT *>(rois),
                         static_cast<T *>(output), p);
  });
  return check_launch("roi_forward_kernel");
}

int roi_backward(const void *grad_output, const void *rois, void *grad_input, int dtype, int ndim,
                 int rotated, int batch, int channels, int depth, int height, int width,
                 int num_rois, int out_d, int out_h, int out_w, float spatial_scale,
                 int sampling_ratio, int aligned, int order, void *workspace, void *stream) {
  RoiProblem p;
  int st = make_problem(p, ndim, rotated, batch, channels, depth, height, width, num_rois, out_d,
                        out_h, out_w, spatial_scale, sampling_ratio, aligned, order);
  if (st) return st;
  if (num_rois == 0) return MV_OK;
  MV_REQUIRE(grad_output && rois && grad_input, "null pointer argument");
  const bool narrow = dtype == MV_F16 || dtype == MV_BF16;
  MV_REQUIRE(!narrow || workspace, "16-bit backward needs an fp32 workspace");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long total = static_cast<long>(batch) * channels * depth * height * width;
  const int fill_blocks = static_cast<int>(std::min<long>((total + 1023) / 1024, 65536));
  if (roi_backward_tiled_direct(dtype, p, grad_input))
    return roi_backward_tiled(grad_output, rois, grad_input, dtype, p, s, true);
  if (roi_backward_tiled_applies(dtype, p)) {
    // 16-bit tensors: sums in the fp32 workspace; fp32: sums in grad_input
    float *ws = static_cast<float *>(workspace);
    if (narrow) hipLaunchKernelGGL(fill_zero_kernel, dim3(fill_blocks), dim3(256), 0, s, ws, total);
    st = roi_backward_tiled(grad_output, rois, narrow ? ws : static_cast<float *>(grad_input), dtype, p, s);
    if (st) return st;
    if (!narrow) return MV_OK;
    MV_DISPATCH(dtype, {
      if constexpr (sizeof(T) == 2)
        hipLaunchKernelGGL((add_from_f32_kernel<T>), dim3(fill_blocks), dim3(256), 0, s,
                           static_cast<T *>(grad_input), static_cast<const float *>(workspace), total);
    });
    return check_launch("add_from_f32_kernel");
  }
  const int gathered = roi_backward_gather(grad_output, rois, grad_input, dtype, p, s);
  if (gathered >= 0) return gathered;
  const dim3 grid(p.chunks * num_rois), block(kRoiThreads);
  if (narrow) {
    hipLaunchKernelGGL(fill_zero_kernel, dim3(fill_blocks), dim3(256), 0, s,
                       static_cast<float *>(workspace), total);
  }
  // 16-bit pooled path: the fp32 workspace is used channels-last and folded in by a transposing add
  const bool channels_last = narrow && roi_pool_applies(dtype, p);
  const int pooled = roi_pool_backward(grad_output, rois, narrow ? workspace : grad_input, dtype, p, s, channels_last);
  if (pooled > 0) return pooled;
  if (pooled == 0 && channels_last)
    return planar_add_f32(static_cast<const float *>(workspace), grad_input, batch, channels,
                          static_cast<long>(depth) * height * width, dtype, s);
  const int boxed = pooled < 0 ? roi_box_backward(grad_output, rois, static_cast<float *>(narrow ? workspace : grad_input), dtype, p, s) : -1;
  if (boxed > 0) return boxed;
  MV_DISPATCH(dtype, {
    using RT = typename std::conditional<std::is_same<T, double>::value, double, float>::type;
    using G = typename std::conditional<(sizeof(T) == 2), float, T>::type;
    G *acc = narrow ? static_cast<G *>(workspace) : static_cast<G *>(grad_input);
    if (pooled == 0 || boxed == 0) {
      // gradient already accumulated by the pooled / box kernel
    } else if (rotated)
      hipLaunchKernelGGL((roi_backward_kernel<T, G, RT, true>), grid, block, 0, s,
                         static_cast<const T *>(grad_output), static_cast<const RT *>(rois), acc, p);
    else
      hipLaunchKernelGGL((roi_backward_kernel<T, G, RT, false>), grid, block, 0, s,
                         static_cast<const T *>(grad_output), static_cast<const RT *>(rois), acc, p);
    if (sizeof(T) == 2)
      hipLaunchKernelGGL((add_from_f32_kernel<T>), dim3(fill_blocks), dim3(256), 0, s,
                         static_cast<T *>(grad_input), static_cast<const float *>(workspace), total);
  });
  return check_launch("roi_backward_kernel");
}

}  // namespace mv

// ---------------------------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------------------------
using mv::roi_backward;
using mv::roi_forward;

extern "C" {

int mv_roi_align_2d_forward(const void *input, const void *rois, void *output, int dtype,
                            int batch, int channels, int height, int width, int num_rois,
                            int out_h, int out_w, float spatial_scale, int sampling_ratio,
                            int order, void *workspace,
                            size_t workspace_bytes, void *stream) {
  return roi_forward(input, rois, output, dtype, 2, 0, batch, channels, 1, height, width, num_rois,
                     1, out_h, out_w, spatial_scale, sampling_ratio, 1, order, workspace, workspace_bytes, stream);
}

size_t mv_roi_align_prepared_bytes(int dtype, int ndim, int batch, int channels, int depth, int height, int width) {
  if ((ndim != 2 && ndim != 3) || batch <= 0 || channels <= 0 || depth <= 0 || height <= 0 || width <= 0) return 0;
  mv::RoiProblem p{};
  p.ndim = ndim; p.N = batch; p.C = channels; p.D = ndim == 2 ? 1 : depth; p.H = height; p.W = width;
  return mv::roi_pool_prepared_bytes(dtype, p);
}

int mv_roi_align_prepare_features(const void *input, int dtype, int ndim, int batch, int channels, int depth,
                                  int height, int width, void *prepared, size_t prepared_bytes, void *stream) {
  MV_REQUIRE(ndim == 2 || ndim == 3, "ndim must be 2 or 3");
  MV_REQUIRE(batch > 0 && channels > 0 && depth > 0 && height > 0 && width > 0,
             "feature dims must be positive (got %d,%d,%d,%d,%d)", batch, channels, depth, height, width);
  MV_REQUIRE(input && prepared, "null pointer argument");
  mv::RoiProblem p{};
  p.ndim = ndim; p.N = batch; p.C = channels; p.D = ndim == 2 ? 1 : depth; p.H = height; p.W = width;
  const size_t bytes = mv::roi_pool_prepared_bytes(dtype, p);
  MV_REQUIRE(bytes > 0, "no prepared copy for these features (mv_roi_align_prepared_bytes is 0)");
  MV_REQUIRE(prepared_bytes >= bytes, "prepared buffer too small");
  MV_REQUIRE(reinterpret_cast<uintptr_t>(input) % 8 == 0 && reinterpret_cast<uintptr_t>(prepared) % 8 == 0,
             "input and prepared must be 8-byte aligned");
  return mv::roi_pool_prepare(input, dtype, p, prepared, prepared_bytes, static_cast<hipStream_t>(stream));
}

int mv_roi_align_forward_prepared(const void *input, const void *prepared, const void *rois, void *output,
                                  int dtype, int ndim, int batch, int channels, int depth, int height, int width,
                                  int num_rois, int out_d, int out_h, int out_w, float spatial_scale,
                                  int sampling_ratio, int order, void *workspace, size_t workspace_bytes,
                                  void *stream) {
  MV_REQUIRE(ndim == 2 || ndim == 3, "ndim must be 2 or 3");
  return roi_forward(input, rois, output, dtype, ndim, 0, batch, channels, ndim == 2 ? 1 : depth, height, width,
                     num_rois, ndim == 2 ? 1 : out_d, out_h, out_w, spatial_scale, sampling_ratio, 1, order,
                     workspace, workspace_bytes, stream, false, prepared);
}

int mv_roi_align_2d_backward(const void *grad_output, const void *rois, void *grad_input,
                             int dtype, int batch, int channels, int height, int width,
                             int num_rois, int out_h, int out_w, float spatial_scale,
                             int sampling_ratio, int order, void *workspace, void *stream) {
  return roi_backward(grad_output, rois, grad_input, dtype, 2, 0, batch, channels, 1, height,
                      width, num_rois, 1, out_h, out_w, spatial_scale, sampling_ratio, 1, order,
                      workspace, stream);
}

int mv_roi_align_3d_forward(const void *input, const void *rois, void *output, int dtype,
                            int batch, int channels, int depth, int height, int width,
                            int num_rois, int out_d, int out_h, int out_w, float spatial_scale,
                            int sampling_ratio, int order, void *workspace,
                            size_t workspace_bytes, void *stream) {
  return roi_forward(input, rois, output, dtype, 3, 0, batch, channels, depth, height, width,
                     num_rois, out_d, out_h, out_w, spatial_scale, sampling_ratio, 1, order, workspace, workspace_bytes, stream);
}

int mv_roi_align_3d_backward(const void *grad_output, const void *rois, void *grad_input,
                             int dtype, int batch, int channels, int depth, int height, int width,
                             int num_rois, int out_d, int out_h, int out_w, float spatial_scale,
                             int sampling_ratio, int order, void *workspace, void *stream) {
  return roi_backward(grad_output, rois, grad_input, dtype, 3, 0, batch, channels, depth, height,
                      width, num_rois, out_d, out_h, out_w, spatial_scale, sampling_ratio, 1,
                      order, workspace, stream);
}

int mv_roi_align_rotated_2d_forward(const void *input, const void *rois, void *output, int dtype,
                                    int batch, int channels, int height, int width, int num_rois,
                                    int out_h, int out_w, float spatial_scale, int sampling_ratio,
                                    int aligned, int order, void *workspace,
                                    size_t workspace_bytes, void *stream) {
  return roi_forward(input, rois, output, dtype, 2, 1, batch, channels, 1, height, width, num_rois,
                     1, out_h, out_w, spatial_scale, sampling_ratio, aligned, order, workspace, workspace_bytes, stream);
}

int mv_roi_align_rotated_2d_backward(const void *grad_output, const void *rois, void *grad_input,
                                     int dtype, int batch, int channels, int height, int width,
                                     int num_rois, int out_h, int out_w, float spatial_scale,
                                     int sampling_ratio, int aligned, int order, void *workspace,
                                     void *stream) {
  return roi_backward(grad_output, rois, grad_input, dtype, 2, 1, batch, channels, 1, height,
                      width, num_rois, 1, out_h, out_w, spatial_scale, sampling_ratio, aligned,
                      order, workspace, stream);
}

int mv_roi_align_rotated_3d_forward(const void *input, const void *rois, void *output, int dtype,
                                    int batch, int channels, int depth, int height, int width,
                                    int num_rois, int out_d, int out_h, int out_w,
                                    float spatial_scale, int sampling_ratio, int aligned,
                                    int order, void *workspace,
                                    size_t workspace_bytes, void *stream) {
  return roi_forward(input, rois, output, dtype, 3, 1, batch, channels, depth, height, width,
                     num_rois, out_d, out_h, out_w, spatial_scale, sampling_ratio, aligned, order,
                     workspace, workspace_bytes, stream);
}

int mv_roi_align_rotated_3d_backward(const void *grad_output, const void *rois, void *grad_input,
                                     int dtype, int batch, int channels, int depth, int height,
                                     int width, int num_rois, int out_d, int out_h, int out_w,
                                     float spatial_scale, int sampling_ratio, int aligned,
                                     int order, void *workspace, void *stream) {
  return roi_backward(grad_output, rois, grad_input, dtype, 3, 1, batch, channels, depth, height,
                      width, num_rois, out_d, out_h, out_w, spatial_scale, sampling_ratio, aligned,
                      order, workspace, stream);
}

size_t mv_roi_align_forward_workspace_bytes(int dtype, int ndim, int channels, int num_rois,
                                            int out_d, int out_h, int out_w, int sampling_ratio) {
  mv::RoiProblem p = {};
  p.ndim = ndim; p.C = channels; p.R = num_rois;
  p.od = ndim == 2 ? 1 : out_d; p.oh = out_h; p.ow = out_w; p.sampling_ratio = sampling_ratio;
  size_t need = 0;
  if (mv::roi_forward_tiled(nullptr, nullptr, nullptr, dtype, p, nullptr, 0, &need, nullptr) != MV_OK) return 0;
  return need;
}

size_t mv_roi_align_forward_workspace_bytes_for_input(int dtype, int ndim, int batch, int channels, int depth,
                                                      int height, int width, int num_rois, int out_d,
                                                      int out_h, int out_w, int sampling_ratio) {
  const size_t basic = mv_roi_align_forward_workspace_bytes(dtype, ndim, channels, num_rois, out_d, out_h, out_w,
                                                            sampling_ratio);
  mv::RoiProblem p = {};
  p.ndim = ndim; p.N = batch; p.C = channels; p.D = ndim == 2 ? 1 : depth; p.H = height; p.W = width; p.R = num_rois;
  p.od = ndim == 2 ? 1 : out_d; p.oh = out_h; p.ow = out_w; p.sampling_ratio = sampling_ratio; p.order = 1;
  if (batch <= 0 || channels <= 0 || p.D <= 0 || height <= 0 || width <= 0 || num_rois <= 0) return basic;
  if (basic || dtype == MV_I32) return basic;   // (the tiled resampler takes the problem; label maps have no other path that wants memory)
  const size_t pooled = mv::roi_pool_forward_workspace(dtype, p);
  return pooled ? pooled : mv::roi_forward_cl_workspace(dtype, p);
}

size_t mv_roi_align_backward_workspace_bytes(int dtype, int batch, int channels, int depth,
                                             int height, int width) {
  if (dtype != MV_F16 && dtype != MV_BF16) return 0;
  return sizeof(float) * static_cast<size_t>(batch) * channels * depth * height * width;
}

int mv_affine_2d(const void *input, const void *rois, void *output, int dtype, int batch,
                 int channels, int height, int width, int num_rois, int out_h, int out_w,
                 float spatial_scale, int sampling_ratio, int aligned, int order, void *workspace,
                 size_t workspace_bytes, void *stream) {
  return roi_forward(input, rois, output, dtype, 2, 1, batch, channels, 1, height, width, num_rois,
                     1, out_h, out_w, spatial_scale, sampling_ratio, aligned, order, workspace, workspace_bytes, stream, true);
}

int mv_affine_3d(const void *input, const void *rois, void *output, int dtype, int batch,
                 int channels, int depth, int height, int width, int num_rois, int out_d,
                 int out_h, int out_w, float spatial_scale, int sampling_ratio, int aligned,
                 int order, void *workspace,
                 size_t workspace_bytes, void *stream) {
  return roi_forward(input, rois, output, dtype, 3, 1, batch, channels, depth, height, width,
                     num_rois, out_d, out_h, out_w, spatial_scale, sampling_ratio, aligned, order,
                     workspace, workspace_bytes, stream, true);
}

}  // extern "C"
