// RoIAlign / RoIAlignRotated FORWARD for many small outputs over wide feature maps (detection heads
// that the separable pooled kernels do not take: rotated boxes, 2-D and 3-D, orders 0 and 1).  Same
// results as the reference's one-thread-per-output kernel
// (csrc/cuda/roi_align_rotated_3d_cuda_kernel.cuh:16-122, roi_align_3d_cuda_kernel.cuh and the 2-D twins).
//
// The one-thread-per-(channel, cell) kernel works a sample's taps out again for every channel and
// reads 2 or 4 bytes per tap and lane from planes that lie megabytes apart.  Here the features are
// first copied channels-last into the workspace ([N][voxel][C]: one pass over the input), and a
// workgroup owns a roi: a lane takes one output cell and 16 bytes of channels (8 16-bit or 4 fp32
// ones), the lanes of a cell sit side by side, so a tap is one 16-byte load per lane from the run of
// C contiguous channels of its voxel, and the taps of a sample serve all of the lane's channels.
// The lanes of a cell split its samples' geometry between them.
// Sample coordinates, tap decisions and the void rule are those of the general kernels
// (sampling.hpp, fp64); sums in fp32 in the order of the general kernel's sample loop.
#include "common.hpp"
#include "roi_geometry.hpp"
#include "sampling.hpp"
#include "roi_taps.hpp"

namespace mv {

// [B, C, P] -> [B, P, C] for elements of 2 or 4 bytes (dcn3d_mfma.hip)
int dcn_channels_last(const void *x, void *xt, int B, int C, long P, int elem_bytes, hipStream_t stream);

constexpr int kClThreads = 256;

struct ClShape {
  int lanes;    // lanes per cell (each 16 bytes of channels)
  int slots;    // cells per wavefront
  int passes;   // passes over the channels when a cell's channels exceed a wavefront
  int chunk;    // cells per workgroup
  int chunks;   // workgroups per roi
};

template <typename T, bool ROT>
__global__ __launch_bounds__(kClThreads) void roi_forward_cl_kernel(const T *__restrict__ xt, const float *__restrict__ rois,
                                                                  T *__restrict__ out, const RoiProblem p,
                                                                  const ClShape cs) {
  constexpr int ES = sizeof(T), V = 16 / ES;
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  __shared__ RoiGeom gs;
  __shared__ double trig[6];
  const unsigned n = blockIdx.y;
  build_geom_block(gs, trig, rois + static_cast<long>(n) * roi_columns(p.ndim, p.rotated), p);
  const RoiGeom g = uniform_geom(gs);
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int slot = lane / cs.lanes, part = lane - slot * cs.lanes;
  const unsigned cells = static_cast<unsigned>(p.od) * p.oh * p.ow;
  const unsigned begin = blockIdx.x * cs.chunk, end = min(begin + cs.chunk, cells);
  const long plane = static_cast<long>(p.D) * p.H * p.W;
  const int samples = g.batch >= 0 ? g.grid[0] * g.grid[1] * (p.ndim == 3 ? g.grid[2] : 1) : 0;
  const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(xt + static_cast<long>(max(g.batch, 0)) * plane * p.C), 0, static_cast<int>(plane * p.C * ES), 0x00020000);
  const unsigned cbytes = static_cast<unsigned>(p.C) * ES;
  const float count = static_cast<float>(g.count);
  const unsigned sy = static_cast<unsigned>(p.W) * cbytes, sz = static_cast<unsigned>(p.H) * sy;
  for (int pass = 0; pass < cs.passes; pass++) {
    const int c0 = (pass * cs.lanes + part) * V;   // the lane's first channel
    const bool loads = slot < cs.slots && c0 < p.C;
    for (unsigned first = begin + wave * cs.slots; first < end; first += (kClThreads / kWave) * cs.slots) {
      const unsigned cell = first + slot;
      const bool cell_on = slot < cs.slots && cell < end;
      float acc[V];
#pragma unroll
      for (int i = 0; i < V; i++) acc[i] = 0.f;
      // The lanes of a cell share its samples: lane j of the group works out the taps of samples j,
      // j + lanes, ... (fp64 geometry, once per sample instead of once per lane) and hands them to
      // the others through ds_bpermute; every lane then adds the sample for its own channels.
      for (int s0 = 0; s0 < samples; s0 += cs.lanes) {
        int rec_at = -1;           // byte offset of the low corner's channels; -1: void sample
        unsigned rec_step = 0;     // bit 0 / 1 / 2: the high tap differs from the low one along x / y / z
        float rec_fx = 0.f, rec_fy = 0.f, rec_fz = 0.f;
        if (cell_on && s0 + part < samples) {
          BoxTaps t;
          if (box_taps<ROT>(g, p, cell, s0 + part, t)) {
            int zi = t.zi[0], yi = t.yi[0], xi = t.xi[0];
            if (p.order == 0) {   // the picked voxel becomes the low corner
              zi = t.fz == 0.f ? t.zi[0] : t.zi[1]; yi = t.fy == 0.f ? t.yi[0] : t.yi[1]; xi = t.fx == 0.f ? t.xi[0] : t.xi[1];
            }
            rec_at = static_cast<int>(static_cast<unsigned>((zi * p.H + yi) * p.W + xi) * cbytes);
            rec_step = (t.xi[1] != t.xi[0] ? 1u : 0u) | (t.yi[1] != t.yi[0] ? 2u : 0u) | (t.zi[1] != t.zi[0] ? 4u : 0u);
            rec_fx = t.fx; rec_fy = t.fy; rec_fz = t.fz;
          }
        }
        const int turns = min(cs.lanes, samples - s0);
        for (int j = 0; j < turns; j++) {
          const int from = min(slot * cs.lanes + j, kWave - 1);
          const int at0 = __shfl(rec_at, from);
          const unsigned step = __shfl(rec_step, from);
          const float lx = __shfl(rec_fx, from), ly = __shfl(rec_fy, from), lz = __shfl(rec_fz, from);
          if (at0 < 0 || !loads) continue;
          const unsigned at = static_cast<unsigned>(at0) + static_cast<unsigned>(c0) * ES;
          auto take = [&](u32x4 r, float (&v)[V]) {
            if constexpr (ES == 4) {
              v[0] = __uint_as_float(r.x); v[1] = __uint_as_float(r.y); v[2] = __uint_as_float(r.z); v[3] = __uint_as_float(r.w);
            } else {
              union { u32x4 u; T e[8]; } w;
              w.u = r;
#pragma unroll
              for (int i = 0; i < 8; i++) v[i] = static_cast<float>(load(&w.e[i]));
            }
          };
          if (p.order == 0) {
            float v[V];
            take(__builtin_amdgcn_raw_buffer_load_b128(xr, at, 0, 0), v);
#pragma unroll
            for (int i = 0; i < V; i++) acc[i] += v[i];
            continue;
          }
          const unsigned dx = (step & 1u) ? cbytes : 0u, dy = (step & 2u) ? sy : 0u, dz = (step & 4u) ? sz : 0u;
          u32x4 raw[8];
#pragma unroll
          for (int k = 0; k < 8; k++)
            raw[k] = __builtin_amdgcn_raw_buffer_load_b128(xr, at + ((k & 4) ? dz : 0u) + ((k & 2) ? dy : 0u) + ((k & 1) ? dx : 0u), 0, 0);
          const float hx = 1.f - lx, hy = 1.f - ly, hz = 1.f - lz;
          float v[8][V];
#pragma unroll
          for (int k = 0; k < 8; k++) take(raw[k], v[k]);
#pragma unroll
          for (int i = 0; i < V; i++)
            acc[i] += hz * (hy * (hx * v[0][i] + lx * v[1][i]) + ly * (hx * v[2][i] + lx * v[3][i])) +
                      lz * (hy * (hx * v[4][i] + lx * v[5][i]) + ly * (hx * v[6][i] + lx * v[7][i]));
        }
      }
      if (cell_on && loads) {
        T *dst = out + (static_cast<long>(n) * p.C + c0) * cells + cell;
#pragma unroll
        for (int i = 0; i < V; i++) dst[static_cast<long>(i) * cells] = store_cast<T>(acc[i] / count);
      }
    }
  }
}

// The path pays when the taps read outnumber the voxels copied: small outputs per roi (larger ones
// belong to the tiled resampler), channels in whole 16-byte pieces, many samples per input voxel.
static bool roi_cl_applies(int dtype, const RoiProblem &p) {
  if (dtype != MV_F16 && dtype != MV_BF16 && dtype != MV_F32) return false;
  const int v = dtype == MV_F32 ? 4 : 8;
  if (p.order == 3 || p.C < 16 || p.C % v) return false;
  const long cells = static_cast<long>(p.od) * p.oh * p.ow, plane = static_cast<long>(p.D) * p.H * p.W;
  if (cells > 4096 || p.R <= 0 || p.N <= 0 || plane <= 0) return false;
  if (plane * p.C * (dtype == MV_F32 ? 4 : 2) >= (1L << 31)) return false;   // 32-bit byte offsets inside one image
  const long grid = p.sampling_ratio > 0 ? p.sampling_ratio : 2;            // (the adaptive grid is not known here)
  long samples = static_cast<long>(p.R) * cells;
  for (int a = 0; a < p.ndim; a++) samples *= grid;
  return samples >= static_cast<long>(p.N) * plane && p.R <= 65535;
}

size_t roi_forward_cl_workspace(int dtype, const RoiProblem &p) {
  if (!roi_cl_applies(dtype, p)) return 0;
  return static_cast<size_t>(p.N) * p.C * p.D * p.H * p.W * (dtype == MV_F32 ? 4 : 2);
}

// Returns -1 when the path does not apply or the workspace cannot hold the copy.
int roi_forward_cl(const void *input, const void *rois, void *output, int dtype, const RoiProblem &p,
                   void *workspace, size_t capacity, hipStream_t s) {
  const size_t need = roi_forward_cl_workspace(dtype, p);
  if (need == 0 || workspace == nullptr || capacity < need) return -1;
  const int es = dtype == MV_F32 ? 4 : 2, v = 16 / es;
  const long plane = static_cast<long>(p.D) * p.H * p.W;
  const int st = dcn_channels_last(input, workspace, p.N, p.C, plane, es, s);
  if (st) return st;
  ClShape cs;
  const int pieces = p.C / v;
  cs.lanes = pieces < kWave ? pieces : kWave;
  cs.slots = kWave / cs.lanes;
  cs.passes = (pieces + cs.lanes - 1) / cs.lanes;
  const long cells = static_cast<long>(p.od) * p.oh * p.ow;
  const int per_turn = (kClThreads / kWave) * cs.slots;   // cells a workgroup takes at a time
  // a roi per workgroup when there are many; few rois are split so that ~1024 workgroups exist
  long chunks = (1024 + p.R - 1) / p.R;
  chunks = std::max(1L, std::min(chunks, (cells + per_turn - 1) / per_turn));
  cs.chunk = static_cast<int>(((cells + chunks - 1) / chunks + per_turn - 1) / per_turn * per_turn);
  cs.chunks = static_cast<int>((cells + cs.chunk - 1) / cs.chunk);
  const dim3 grid(cs.chunks, p.R), block(kClThreads);
#define MV_LAUNCH_CL(T)                                                                                     \
  if (p.rotated)                                                                                            \
    hipLaunchKernelGGL((roi_forward_cl_kernel<T, true>), grid, block, 0, s, static_cast<const T *>(workspace), \
                       static_cast<const float *>(rois), static_cast<T *>(output), p, cs);                  \
  else                                                                                                      \
    hipLaunchKernelGGL((roi_forward_cl_kernel<T, false>), grid, block, 0, s, static_cast<const T *>(workspace), \
                       static_cast<const float *>(rois), static_cast<T *>(output), p, cs)
  if (dtype == MV_F16) { MV_LAUNCH_CL(__half); }
  else if (dtype == MV_BF16) { MV_LAUNCH_CL(__hip_bfloat16); }
  else { MV_LAUNCH_CL(float); }
#undef MV_LAUNCH_CL
  return check_launch("roi_forward_cl_kernel");
}

}  // namespace mv
