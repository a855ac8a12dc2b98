// 3-D deformable convolution (DCNv1 when mask == nullptr, DCNv2 otherwise): general-shape
// kernels for every dtype / group configuration, plus the entry points that choose between them
// and the matrix-core forward for 16-bit tensors (dcn3d_mfma.hip).
//
// Nothing here materialises the reference's column matrix: the trilinear gather feeds the weight
// contraction directly, and the 8 corner offsets / weights of a (tap, position) pair are computed
// once and reused for all channels of the deformable group.
#include <atomic>

#include "dcn_common.hpp"
#include "dcn_pad.hpp"
#include "sampling.hpp"

namespace mv {

constexpr int kDcnThreads = 128;
constexpr int kOutTile = 32;  // output channels accumulated per thread in the general forward

// ---- forward: thread = (output position, tile of <= 32 output channels of one group) --------
template <typename T>
__global__ __launch_bounds__(kDcnThreads) void dcn_forward_kernel(
    const T *__restrict__ x, const T *__restrict__ off, const T *__restrict__ mask,
    const T *__restrict__ wt, const T *__restrict__ bias, T *__restrict__ y, const DcnDims s) {
  using A = typename Acc<T>::type;
  const long q = blockIdx.x * static_cast<long>(kDcnThreads) + threadIdx.x;
  const int tiles_per_group = (s.opg + kOutTile - 1) / kOutTile;
  const int grp = blockIdx.y / tiles_per_group, tile = blockIdx.y % tiles_per_group;
  const int b = blockIdx.z;
  if (q >= s.Q) return;
  const int ow = q % s.Wo, oh = (q / s.Wo) % s.Ho, od = q / (static_cast<long>(s.Wo) * s.Ho);
  const int o_begin = grp * s.opg + tile * kOutTile;
  const int o_count = min(kOutTile, grp * s.opg + s.opg - o_begin);
  A acc[kOutTile];
#pragma unroll
  for (int i = 0; i < kOutTile; i++) acc[i] = A(0);
  const int c_begin = grp * s.cpg, c_end = c_begin + s.cpg;
  for (int dgi = c_begin / s.cpd; dgi <= (c_end - 1) / s.cpd; dgi++) {
    const int c_lo = max(c_begin, dgi * s.cpd), c_hi = min(c_end, (dgi + 1) * s.cpd);
    const T *off_bg = off + (static_cast<long>(b) * s.dg + dgi) * s.nd * s.K * s.Q;
    const T *mask_bg = mask ? mask + (static_cast<long>(b) * s.dg + dgi) * s.K * s.Q : nullptr;
    for (int k = 0; k < s.K; k++) {
      double pd, ph, pw;
      dcn_position(s, off_bg, k, od, oh, ow, q, pd, ph, pw);
      ZTaps<A> t;
      zero_pad_taps(s, pd, ph, pw, t);
      if (!t.ok) continue;
      const A m = mask_bg ? load(mask_bg + static_cast<long>(k) * s.Q + q) : A(1);
      for (int c = c_lo; c < c_hi; c++) {
        const A col = zsample<T, A>(x + (static_cast<long>(b) * s.Cin + c) * s.P, t) * m;
        const T *wrow = wt + (static_cast<long>(o_begin) * s.cpg + (c - c_begin)) * s.K + k;
#pragma unroll
        for (int i = 0; i < kOutTile; i++)
          if (i < o_count) acc[i] += load(wrow + static_cast<long>(i) * s.cpg * s.K) * col;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < kOutTile; i++)
    if (i < o_count) {
      const int o = o_begin + i;
      y[(static_cast<long>(b) * s.Cout + o) * s.Q + q] =
          store_cast<T>(acc[i] + (bias ? load(bias + o) : A(0)));
    }
}

// ---- augmentation DCN: the v1 forward with the border-replicating samplers ---------------------
// Column value = S(x[b,c], p) when -1 < p < size on every axis, else 0, with S nearest, linear
// or cubic by `order` (reference: csrc/cuda_aug/deform_3d_cuda_kernel.cuh:8-89, contraction with
// the weight and bias csrc/cuda_aug/deform_3d_cuda.cu:43-152).  Same thread layout as above.
template <typename T>
__global__ __launch_bounds__(kDcnThreads) void deform_conv_clamped_kernel(
    const T *__restrict__ x, const T *__restrict__ off, const T *__restrict__ wt,
    const T *__restrict__ bias, T *__restrict__ y, const DcnDims s, const int order) {
  using A = typename Acc<T>::type;
  const long q = blockIdx.x * static_cast<long>(kDcnThreads) + threadIdx.x;
  const int tiles_per_group = (s.opg + kOutTile - 1) / kOutTile;
  const int grp = blockIdx.y / tiles_per_group, tile = blockIdx.y % tiles_per_group;
  const int b = blockIdx.z;
  if (q >= s.Q) return;
  const int ow = q % s.Wo, oh = (q / s.Wo) % s.Ho, od = q / (static_cast<long>(s.Wo) * s.Ho);
  const int o_begin = grp * s.opg + tile * kOutTile;
  const int o_count = min(kOutTile, grp * s.opg + s.opg - o_begin);
  A acc[kOutTile];
#pragma unroll
  for (int i = 0; i < kOutTile; i++) acc[i] = A(0);
  const int c_begin = grp * s.cpg, c_end = c_begin + s.cpg;
  for (int dgi = c_begin / s.cpd; dgi <= (c_end - 1) / s.cpd; dgi++) {
    const int c_lo = max(c_begin, dgi * s.cpd), c_hi = min(c_end, (dgi + 1) * s.cpd);
    const T *off_bg = off + (static_cast<long>(b) * s.dg + dgi) * s.nd * s.K * s.Q;
    for (int k = 0; k < s.K; k++) {
      double pd, ph, pw;
      dcn_position(s, off_bg, k, od, oh, ow, q, pd, ph, pw);
      if (!(ph > -1.0 && pw > -1.0 && ph < s.H && pw < s.W && (s.nd == 2 || (pd > -1.0 && pd < s.D))))
        continue;
      Corners<A> cw;
      if (order != 3 && !clamped_corners<A>(s.D, s.H, s.W, pd, ph, pw, order, cw)) continue;
      for (int c = c_lo; c < c_hi; c++) {
        const T *plane = x + (static_cast<long>(b) * s.Cin + c) * s.P;
        A col = A(0);
        if (order == 3) {
          col = sample_cubic<T>(plane, s.nd, s.D, s.H, s.W, pd, ph, pw);
        } else {
#pragma unroll
          for (int n = 0; n < 8; n++) col += cw.w[n] * load(plane + cw.idx[n]);
        }
        const T *wrow = wt + (static_cast<long>(o_begin) * s.cpg + (c - c_begin)) * s.K + k;
#pragma unroll
        for (int i = 0; i < kOutTile; i++)
          if (i < o_count) acc[i] += load(wrow + static_cast<long>(i) * s.cpg * s.K) * col;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < kOutTile; i++)
    if (i < o_count) {
      const int o = o_begin + i;
      y[(static_cast<long>(b) * s.Cout + o) * s.Q + q] =
          store_cast<T>(acc[i] + (bias ? load(bias + o) : A(0)));
    }
}

// ---- backward 1: thread = (b, dgi, k, q): grad wrt input (atomic scatter), offset and mask ---
//   gcol[c] = sum_o Wt[o,c_l,k] * gy[b,o,q];  gx += gcol*m*w_corner;  goff_a = sum_c gcol*m*dZ/dp_a;
//   gm = sum_c gcol*Z.   G = accumulation element type of gx (T, or float for 16-bit T).
template <typename T, typename G>
__global__ __launch_bounds__(kDcnThreads) void dcn_backward_data_kernel(
    const T *__restrict__ x, const T *__restrict__ off, const T *__restrict__ mask,
    const T *__restrict__ wt, const T *__restrict__ gy, G *__restrict__ gx, T *__restrict__ goff,
    T *__restrict__ gmask, const DcnDims s) {
  using A = typename Acc<T>::type;
  const long q = blockIdx.x * static_cast<long>(kDcnThreads) + threadIdx.x;
  const int k = blockIdx.y % s.K, dgi = blockIdx.y / s.K;
  const int b = blockIdx.z;
  if (q >= s.Q) return;
  const int ow = q % s.Wo, oh = (q / s.Wo) % s.Ho, od = q / (static_cast<long>(s.Wo) * s.Ho);
  const long bg = static_cast<long>(b) * s.dg + dgi;
  double pd, ph, pw;
  dcn_position(s, off + bg * s.nd * s.K * s.Q, k, od, oh, ow, q, pd, ph, pw);
  ZTaps<A> t;
  zero_pad_taps(s, pd, ph, pw, t);
  A go_d = A(0), go_h = A(0), go_w = A(0), gm = A(0);
  if (t.ok) {
    const A m = mask ? load(mask + (bg * s.K + k) * s.Q + q) : A(1);
    for (int c = dgi * s.cpd; c < (dgi + 1) * s.cpd; c++) {
      const int grp = c / s.cpg, cl = c % s.cpg;
      A gcol = A(0);
      const T *wcol = wt + (static_cast<long>(grp) * s.opg * s.cpg + cl) * s.K + k;
      const T *gyo = gy + (static_cast<long>(b) * s.Cout + grp * s.opg) * s.Q + q;
      for (int o = 0; o < s.opg; o++)
        gcol += load(wcol + static_cast<long>(o) * s.cpg * s.K) * load(gyo + o * s.Q);
      const T *plane = x + (static_cast<long>(b) * s.Cin + c) * s.P;
      G *gplane = gx + (static_cast<long>(b) * s.Cin + c) * s.P;
      A v[8];
      A val = A(0);
#pragma unroll
      for (int n = 0; n < 8; n++) {
        v[n] = t.off[n] >= 0 ? load(plane + t.off[n]) : A(0);
        val += t.w[n] * v[n];
        if (t.off[n] >= 0) atomic_add(gplane + t.off[n], static_cast<G>(t.w[n] * gcol * m));
      }
      gm += gcol * val;
      const A hd = A(1) - t.fd, hh = A(1) - t.fh, hw = A(1) - t.fw;
      // d/dp of the trilinear blend: the differentiated axis contributes -1 (low) / +1 (high)
      const A dd = hh * (hw * (v[4] - v[0]) + t.fw * (v[5] - v[1])) +
                   t.fh * (hw * (v[6] - v[2]) + t.fw * (v[7] - v[3]));
      const A dh = hd * (hw * (v[2] - v[0]) + t.fw * (v[3] - v[1])) +
                   t.fd * (hw * (v[6] - v[4]) + t.fw * (v[7] - v[5]));
      const A dw = hd * (hh * (v[1] - v[0]) + t.fh * (v[3] - v[2])) +
                   t.fd * (hh * (v[5] - v[4]) + t.fh * (v[7] - v[6]));
      go_d += dd * gcol * m; go_h += dh * gcol * m; go_w += dw * gcol * m;
    }
  }
  T *o = goff + (bg * s.nd * s.K + s.nd * k) * s.Q + q;
  if (s.nd == 3) o[0] = store_cast<T>(go_d);
  o[(s.nd - 2) * s.Q] = store_cast<T>(go_h); o[(s.nd - 1) * s.Q] = store_cast<T>(go_w);
  if (gmask) gmask[(bg * s.K + k) * s.Q + q] = store_cast<T>(gm);
}

// ---- backward 2: grad wrt weight.  workgroup = (input channel c, tap k, slab of positions) ----
// every thread rebuilds col[c,k,q] for its positions, multiplies with gy[b,o,q] for the <= 32
// output channels of the tile, the workgroup reduces and adds one value per (o,c,k) atomically.
constexpr int kGwThreads = 256;
constexpr int kGwPositions = 4096;

template <typename T, typename G>
__global__ __launch_bounds__(kGwThreads) void dcn_backward_weight_kernel(
    const T *__restrict__ x, const T *__restrict__ off, const T *__restrict__ mask,
    const T *__restrict__ gy, G *__restrict__ gw, const DcnDims s, const int slabs) {
  using A = typename Acc<T>::type;
  const int k = blockIdx.x % s.K, c = blockIdx.x / s.K;
  const int tiles = (s.opg + kOutTile - 1) / kOutTile;
  const int tile = blockIdx.y % tiles, slab = blockIdx.y / tiles;
  const int b = blockIdx.z;
  const int grp = c / s.cpg, cl = c % s.cpg, dgi = c / s.cpd;
  const int o_begin = grp * s.opg + tile * kOutTile;
  const int o_count = min(kOutTile, grp * s.opg + s.opg - o_begin);
  const long bg = static_cast<long>(b) * s.dg + dgi;
  const T *plane = x + (static_cast<long>(b) * s.Cin + c) * s.P;
  A acc[kOutTile];
#pragma unroll
  for (int i = 0; i < kOutTile; i++) acc[i] = A(0);
  const long q_end = min(static_cast<long>(slab + 1) * kGwPositions, s.Q);
  for (long q = static_cast<long>(slab) * kGwPositions + threadIdx.x; q < q_end; q += kGwThreads) {
    const int ow = q % s.Wo, oh = (q / s.Wo) % s.Ho, od = q / (static_cast<long>(s.Wo) * s.Ho);
    double pd, ph, pw;
    dcn_position(s, off + bg * s.nd * s.K * s.Q, k, od, oh, ow, q, pd, ph, pw);
    ZTaps<A> t;
    zero_pad_taps(s, pd, ph, pw, t);
    if (!t.ok) continue;
    const A m = mask ? load(mask + (bg * s.K + k) * s.Q + q) : A(1);
    const A col = zsample<T, A>(plane, t) * m;
    const T *gyo = gy + (static_cast<long>(b) * s.Cout + o_begin) * s.Q + q;
#pragma unroll
    for (int i = 0; i < kOutTile; i++)
      if (i < o_count) acc[i] += col * load(gyo + i * s.Q);
  }
  __shared__ A part[kGwThreads / kWave][kOutTile];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
#pragma unroll
  for (int i = 0; i < kOutTile; i++) {
    A v = acc[i];
    for (int d = kWave / 2; d > 0; d >>= 1) v += __shfl_down(v, d, kWave);
    if (lane == 0) part[wave][i] = v;
  }
  __syncthreads();
  if (threadIdx.x < o_count) {
    A v = A(0);
    for (int w = 0; w < kGwThreads / kWave; w++) v += part[w][threadIdx.x];
    atomic_add(gw + (static_cast<long>(o_begin + threadIdx.x) * s.cpg + cl) * s.K + k,
               static_cast<G>(v));
  }
  (void)slabs;
}

// ---- backward 3: grad wrt bias: workgroup = (o, b, slab of positions) ----------------------------
constexpr int kBiasSlab = 8192;
template <typename T, typename G>
__global__ __launch_bounds__(256) void dcn_backward_bias_kernel(const T *__restrict__ gy,
                                                                G *__restrict__ gb,
                                                                const DcnDims s) {
  using A = typename Acc<T>::type;
  const int o = blockIdx.x, b = blockIdx.y;
  const T *src = gy + (static_cast<long>(b) * s.Cout + o) * s.Q;
  const long q_end = min(static_cast<long>(blockIdx.z + 1) * kBiasSlab, s.Q);
  A v = A(0);
  long q0 = static_cast<long>(blockIdx.z) * kBiasSlab;
  if constexpr (sizeof(T) <= 4) {
    // 16-byte pieces, four independent loads per lane and step (one load in flight per wavefront
    // leaves the memory system idle most of the time)
    constexpr int V = 16 / sizeof(T);
    if (reinterpret_cast<uintptr_t>(src + q0) % 16 == 0) {
      const long groups = (q_end - q0) / V;
      const uint4 *pieces = reinterpret_cast<const uint4 *>(src + q0);
      for (long i = threadIdx.x; i < groups; i += 1024) {
        uint4 raw[4];
#pragma unroll
        for (int u = 0; u < 4; u++) raw[u] = i + u * 256 < groups ? pieces[i + u * 256] : uint4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int u = 0; u < 4; u++) {
          const T *e = reinterpret_cast<const T *>(&raw[u]);
#pragma unroll
          for (int j = 0; j < V; j++) v += load(e + j);
        }
      }
      q0 += groups * V;
    }
  }
  for (long q = q0 + threadIdx.x; q < q_end; q += 256) v += load(src + q);
  __shared__ A part[4];
  for (int d = kWave / 2; d > 0; d >>= 1) v += __shfl_down(v, d, kWave);
  if (threadIdx.x % kWave == 0) part[threadIdx.x / kWave] = v;
  __syncthreads();
  if (threadIdx.x == 0) atomic_add(gb + o, static_cast<G>(part[0] + part[1] + part[2] + part[3]));
}

__global__ void dcn_fill_zero_kernel(float *p, long n) {
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<long>(gridDim.x) * blockDim.x)
    p[i] = 0.f;
}

template <typename T>
__global__ void dcn_add_from_f32_kernel(T *dst, const float *src, long n) {
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<long>(gridDim.x) * blockDim.x)
    dst[i] = store_cast<T>(load(dst + i) + src[i]);
}

// matrix-core forward for 16-bit tensors (dcn3d_mfma.hip)
bool dcn_mfma_supported(const DcnDims &s, int dtype);
size_t dcn_mfma_workspace_bytes(const DcnDims &s, int dtype);
int dcn_mfma_forward(const void *x, const void *off, const void *mask, const void *wt,
                     const void *bias, void *y, const DcnDims &s, int dtype, void *workspace,
                     hipStream_t stream);

// matrix-core backward for 16-bit tensors (dcn3d_mfma_backward.hip)
bool dcn_mfma_backward_supported(const DcnDims &s, int dtype);
size_t dcn_mfma_backward_workspace_bytes(const DcnDims &s, int dtype);
int dcn_mfma_backward(const void *x, const void *off, const void *mask, const void *wt,
                      const void *gy, void *goff, void *gmask, const DcnDims &s, int dtype,
                      void *workspace, bool want_bias, float **gx32, float **gw32, float **gb32,
                      hipStream_t stream);
void dcn_set_column_budget(size_t bytes);
size_t dcn_column_budget();
int dcn_planar_add(const float *gxt, void *gx, const DcnDims &s, int dtype, hipStream_t stream);
int dcn_weight_add(const float *acc, void *gw, const DcnDims &s, int dtype, hipStream_t stream);
int dcn_backward_fold(const float *gxt, const float *gw32, const float *gb32, void *grad_input, void *grad_weight,
                      void *grad_bias, const DcnDims &s, int dtype, hipStream_t stream);

static inline int blocks_for(long n, int per_block, int cap) {
  return static_cast<int>(std::min<long>((n + per_block - 1) / per_block, cap));
}

}  // namespace mv

using namespace mv;

extern "C" {

int mv_dcn3d_output_dims(const mv_dcn3d_shape *shape, int *out_d, int *out_h, int *out_w) {
  DcnDims s;
  int st = make_dcn_dims(s, shape);
  if (st) return st;
  *out_d = s.Do; *out_h = s.Ho; *out_w = s.Wo;
  return MV_OK;
}

// Layers whose channel counts the matrix-core kernels do not take run as the next larger layer
// that they do (dcn_pad.hip).  Workspace of such a call: padded copies first, then the workspace
// of the padded layer.
static size_t align256p(size_t v) { return (v + 255) / 256 * 256; }
struct PadLayout {
  size_t x, w, b, y, gy, inner, total;   // byte offsets (x, w, b / gy, y: padded copies; y only when Cout is padded)
  bool x_padded, y_padded;
};
static PadLayout pad_layout(const DcnDims &s, const DcnPad &pad, int dtype, bool backward) {
  const size_t es = dtype == MV_F32 ? 4 : 2;
  const DcnDims &p = pad.p;
  PadLayout l;
  l.x_padded = p.Cin != s.Cin; l.y_padded = p.Cout != s.Cout;
  size_t at = 0;
  l.x = at; at += l.x_padded ? align256p(static_cast<size_t>(p.B) * p.Cin * p.P * es) : 0;
  l.w = at; at += align256p(static_cast<size_t>(p.Cout) * p.cpg * p.K * es);
  l.b = at; at += align256p(static_cast<size_t>(p.Cout) * es);
  l.y = at; at += (!backward && l.y_padded) ? align256p(static_cast<size_t>(p.B) * p.Cout * p.Q * es) : 0;
  l.gy = at; at += (backward && l.y_padded) ? align256p(static_cast<size_t>(p.B) * p.Cout * p.Q * es) : 0;
  l.inner = at;
  at += backward ? dcn_mfma_backward_workspace_bytes(p, dtype) : dcn_mfma_workspace_bytes(p, dtype);
  l.total = at;
  return l;
}
static bool forward_pads(const DcnDims &s, int dtype, DcnPad &pad) {
  return !dcn_mfma_supported(s, dtype) && dcn_pad_plan(s, dtype, pad) && dcn_mfma_supported(pad.p, dtype);
}
static bool backward_pads(const DcnDims &s, int dtype, DcnPad &pad) {
  return !dcn_mfma_backward_supported(s, dtype) && dcn_pad_plan(s, dtype, pad) && dcn_mfma_backward_supported(pad.p, dtype);
}

static size_t forward_workspace(const DcnDims &s, int dtype) {
  if (dcn_mfma_supported(s, dtype)) return dcn_mfma_workspace_bytes(s, dtype);
  DcnPad pad;
  return forward_pads(s, dtype, pad) ? pad_layout(s, pad, dtype, false).total : 0;
}

static size_t backward_workspace(const DcnDims &s, int dtype) {
  if (dcn_mfma_backward_supported(s, dtype)) return dcn_mfma_backward_workspace_bytes(s, dtype);
  DcnPad pad;
  if (backward_pads(s, dtype, pad)) return pad_layout(s, pad, dtype, true).total;
  if (dtype != MV_F16 && dtype != MV_BF16) return 0;
  // fp32 accumulators for grad_input, grad_weight, grad_bias
  const size_t n = static_cast<size_t>(s.B) * s.Cin * s.P + static_cast<size_t>(s.Cout) * s.cpg * s.K + s.Cout;
  return n * sizeof(float);
}

static int dcn_forward_any(const void *input, const void *offset, const void *mask,
                           const void *weight, const void *bias, void *output, const DcnDims &s,
                           int dtype, void *workspace, void *stream) {
  MV_REQUIRE(input && offset && weight && output, "null pointer argument");
  hipStream_t hs = static_cast<hipStream_t>(stream);
  if (dcn_mfma_supported(s, dtype)) {
    MV_REQUIRE(workspace, "this shape needs a workspace of mv_dcn3d_forward_workspace_bytes()");
    return dcn_mfma_forward(input, offset, mask, weight, bias, output, s, dtype, workspace, hs);
  }
  DcnPad pad;
  if (forward_pads(s, dtype, pad)) {
    MV_REQUIRE(workspace, "this shape needs a workspace of mv_dcn3d_forward_workspace_bytes()");
    const PadLayout l = pad_layout(s, pad, dtype, false);
    const int es = dtype == MV_F32 ? 4 : 2;
    char *ws = static_cast<char *>(workspace);
    const void *xp = input;
    int st = MV_OK;
    if (l.x_padded) {
      st = dcn_pad_channels(input, ws + l.x, s.B, s.Cin, s.P, pad.unit, pad.unit_p, es, hs);
      if (st) return st;
      xp = ws + l.x;
    }
    st = dcn_pad_weight(weight, ws + l.w, s, pad, es, hs);
    if (st) return st;
    if (bias) {
      st = dcn_pad_channels(bias, ws + l.b, 1, s.Cout, 1, s.opg, pad.p.opg, es, hs);
      if (st) return st;
    }
    void *yp = l.y_padded ? static_cast<void *>(ws + l.y) : output;
    st = dcn_mfma_forward(xp, offset, mask, ws + l.w, bias ? ws + l.b : nullptr, yp, pad.p, dtype, ws + l.inner, hs);
    if (st || !l.y_padded) return st;
    return dcn_unpad_channels(yp, output, s.B, s.Cout, s.Q, s.opg, pad.p.opg, es, hs);
  }
  const long qb = (s.Q + kDcnThreads - 1) / kDcnThreads;
  const long yb = static_cast<long>(s.groups) * ((s.opg + kOutTile - 1) / kOutTile);
  MV_REQUIRE(qb < (1L << 31) && yb <= 65535 && s.B <= 65535, "grid too large");
  const dim3 grid(static_cast<unsigned>(qb), static_cast<unsigned>(yb), s.B), block(kDcnThreads);
  MV_DISPATCH(dtype, {
    hipLaunchKernelGGL((dcn_forward_kernel<T>), grid, block, 0, hs, static_cast<const T *>(input),
                       static_cast<const T *>(offset), static_cast<const T *>(mask),
                       static_cast<const T *>(weight), static_cast<const T *>(bias),
                       static_cast<T *>(output), s);
  });
  return check_launch("dcn_forward_kernel");
}

static int deform_conv_any(const void *input, const void *offset, const void *weight,
                           const void *bias, void *output, const DcnDims &s, int dtype, int order,
                           void *stream) {
  MV_REQUIRE(input && offset && weight && output, "null pointer argument");
  MV_REQUIRE(order == 0 || order == 1 || order == 3,
             "order %d is not supported (0 nearest, 1 linear, 3 cubic)", order);
  const long qb = (s.Q + kDcnThreads - 1) / kDcnThreads;
  const long yb = static_cast<long>(s.groups) * ((s.opg + kOutTile - 1) / kOutTile);
  MV_REQUIRE(qb < (1L << 31) && yb <= 65535 && s.B <= 65535, "grid too large");
  const dim3 grid(static_cast<unsigned>(qb), static_cast<unsigned>(yb), s.B), block(kDcnThreads);
  MV_DISPATCH(dtype, {
    hipLaunchKernelGGL((deform_conv_clamped_kernel<T>), grid, block, 0,
                       static_cast<hipStream_t>(stream), static_cast<const T *>(input),
                       static_cast<const T *>(offset), static_cast<const T *>(weight),
                       static_cast<const T *>(bias), static_cast<T *>(output), s, order);
  });
  return check_launch("deform_conv_clamped_kernel");
}

static int dcn_backward_any(const void *input, const void *offset, const void *mask,
                            const void *weight, const void *grad_output, void *grad_input,
                            void *grad_offset, void *grad_mask, void *grad_weight, void *grad_bias,
                            const DcnDims &s, int dtype, void *workspace, void *stream) {
  int st = MV_OK;
  MV_REQUIRE(input && offset && weight && grad_output && grad_input && grad_offset && grad_weight,
             "null pointer argument");
  MV_REQUIRE((mask == nullptr) == (grad_mask == nullptr) || grad_mask == nullptr,
             "grad_mask given without mask");
  const bool narrow = dtype == MV_F16 || dtype == MV_BF16;
  DcnPad pad;
  const bool padded = backward_pads(s, dtype, pad);
  MV_REQUIRE((!narrow && !dcn_mfma_backward_supported(s, dtype) && !padded) || workspace,
             "this backward needs a workspace of mv_dcn3d_backward_workspace_bytes()");
  hipStream_t hs = static_cast<hipStream_t>(stream);
  if (padded) {
    const PadLayout l = pad_layout(s, pad, dtype, true);
    const int es = dtype == MV_F32 ? 4 : 2;
    char *wsb = static_cast<char *>(workspace);
    const void *xp = input, *gyp = grad_output;
    if (l.x_padded) {
      st = dcn_pad_channels(input, wsb + l.x, s.B, s.Cin, s.P, pad.unit, pad.unit_p, es, hs);
      if (st) return st;
      xp = wsb + l.x;
    }
    st = dcn_pad_weight(weight, wsb + l.w, s, pad, es, hs);
    if (st) return st;
    if (l.y_padded) {
      st = dcn_pad_channels(grad_output, wsb + l.gy, s.B, s.Cout, s.Q, s.opg, pad.p.opg, es, hs);
      if (st) return st;
      gyp = wsb + l.gy;
    }
    float *gx32, *gw32, *gb32;
    st = dcn_mfma_backward(xp, offset, mask, wsb + l.w, gyp, grad_offset, grad_mask, pad.p, dtype, wsb + l.inner,
                           false, &gx32, &gw32, &gb32, hs);
    if (st) return st;
    st = dcn_planar_add_padded(gx32, grad_input, s, pad, dtype, hs);
    if (st) return st;
    MV_DISPATCH(dtype, {
      if (sizeof(T) <= 4) {
        if (grad_bias) {   // from the real output gradient, into the (zeroed) accumulator of the padded layer
          hipLaunchKernelGGL((dcn_backward_bias_kernel<T, float>), dim3(s.Cout, s.B, static_cast<unsigned>((s.Q + kBiasSlab - 1) / kBiasSlab)), dim3(256), 0, hs,
                             static_cast<const T *>(grad_output), gb32, s);
          hipLaunchKernelGGL((dcn_add_from_f32_kernel<T>), dim3(1), dim3(256), 0, hs,
                             static_cast<T *>(grad_bias), gb32, static_cast<long>(s.Cout));
        }
      }
    });
    st = dcn_weight_add_padded(gw32, grad_weight, nullptr, nullptr, s, pad, dtype, hs);
    if (st) return st;
    return check_launch("dcn3d backward (padded channels)");
  }
  const long n_gx = static_cast<long>(s.B) * s.Cin * s.P, n_gw = static_cast<long>(s.Cout) * s.cpg * s.K;
  float *ws = static_cast<float *>(workspace);
  if (dcn_mfma_backward_supported(s, dtype)) {
    float *gx32, *gw32, *gb32;
    st = dcn_mfma_backward(input, offset, mask, weight, grad_output, grad_offset, grad_mask, s, dtype,
                           workspace, grad_bias != nullptr, &gx32, &gw32, &gb32, hs);
    if (st) return st;
    st = dcn_backward_fold(gx32, gw32, gb32, grad_input, grad_weight, grad_bias, s, dtype, hs);
    if (st >= 0) return st;   // (one launch for the three folds; -1: not with these tensors)
    st = dcn_planar_add(gx32, grad_input, s, dtype, hs);
    if (st) return st;
    MV_DISPATCH(dtype, {
      if (sizeof(T) <= 4) {
        if (grad_bias)   // (the sums of grad_output are in the accumulator already)
          hipLaunchKernelGGL((dcn_add_from_f32_kernel<T>), dim3(1), dim3(256), 0, hs,
                             static_cast<T *>(grad_bias), gb32, static_cast<long>(s.Cout));
      }
    });
    st = dcn_weight_add(gw32, grad_weight, s, dtype, hs);
    if (st) return st;
    return check_launch("dcn3d backward");
  }
  if (narrow) {
    const long n = n_gx + n_gw + s.Cout;
    hipLaunchKernelGGL(dcn_fill_zero_kernel, dim3(blocks_for(n, 1024, 65536)), dim3(256), 0, hs, ws, n);
  }
  const long qb = (s.Q + kDcnThreads - 1) / kDcnThreads;
  const long kb = static_cast<long>(s.dg) * s.K;
  const int tiles = (s.opg + kOutTile - 1) / kOutTile;
  const int slabs = static_cast<int>((s.Q + kGwPositions - 1) / kGwPositions);
  MV_REQUIRE(qb < (1L << 31) && kb <= 65535 && s.B <= 65535 &&
                 static_cast<long>(tiles) * slabs <= 65535 &&
                 static_cast<long>(s.Cin) * s.K < (1L << 31), "grid too large");
  MV_DISPATCH(dtype, {
    using G = typename std::conditional<(sizeof(T) == 2), float, T>::type;
    G *gx = narrow ? reinterpret_cast<G *>(ws) : static_cast<G *>(grad_input);
    G *gw = narrow ? reinterpret_cast<G *>(ws + n_gx) : static_cast<G *>(grad_weight);
    G *gb = narrow ? reinterpret_cast<G *>(ws + n_gx + n_gw) : static_cast<G *>(grad_bias);
    hipLaunchKernelGGL((dcn_backward_data_kernel<T, G>),
                       dim3(static_cast<unsigned>(qb), static_cast<unsigned>(kb), s.B),
                       dim3(kDcnThreads), 0, hs, static_cast<const T *>(input),
                       static_cast<const T *>(offset), static_cast<const T *>(mask),
                       static_cast<const T *>(weight), static_cast<const T *>(grad_output), gx,
                       static_cast<T *>(grad_offset), static_cast<T *>(grad_mask), s);
    hipLaunchKernelGGL((dcn_backward_weight_kernel<T, G>),
                       dim3(static_cast<unsigned>(s.Cin * s.K), static_cast<unsigned>(tiles * slabs), s.B),
                       dim3(kGwThreads), 0, hs, static_cast<const T *>(input),
                       static_cast<const T *>(offset), static_cast<const T *>(mask),
                       static_cast<const T *>(grad_output), gw, s, slabs);
    if (grad_bias)
      hipLaunchKernelGGL((dcn_backward_bias_kernel<T, G>), dim3(s.Cout, s.B, static_cast<unsigned>((s.Q + kBiasSlab - 1) / kBiasSlab)), dim3(256), 0, hs,
                         static_cast<const T *>(grad_output), gb, s);
    if (sizeof(T) == 2) {
      hipLaunchKernelGGL((dcn_add_from_f32_kernel<T>), dim3(blocks_for(n_gx, 1024, 65536)), dim3(256),
                         0, hs, static_cast<T *>(grad_input), ws, n_gx);
      hipLaunchKernelGGL((dcn_add_from_f32_kernel<T>), dim3(blocks_for(n_gw, 1024, 65536)), dim3(256),
                         0, hs, static_cast<T *>(grad_weight), ws + n_gx, n_gw);
      if (grad_bias)
        hipLaunchKernelGGL((dcn_add_from_f32_kernel<T>), dim3(1), dim3(256), 0, hs,
                           static_cast<T *>(grad_bias), ws + n_gx + n_gw, static_cast<long>(s.Cout));
    }
  });
  return check_launch("dcn3d backward");
}

// An image layer as a depth-1 volume with a 1 x kh x kw kernel and two offset components per tap.
static int make_dcn_dims_2d(DcnDims &d, const mv_dcn2d_shape *s) {
  MV_REQUIRE(s != nullptr, "shape is null");
  const mv_dcn3d_shape v = {s->batch, s->in_channels, 1, s->height, s->width, s->out_channels,
                            1, s->kernel_h, s->kernel_w, 1, s->stride_h, s->stride_w,
                            0, s->pad_h, s->pad_w, 1, s->dil_h, s->dil_w,
                            s->groups, s->deformable_groups};
  return make_dcn_dims(d, &v, 2);
}

void mv_dcn_set_column_budget(size_t bytes) { dcn_set_column_budget(bytes); }
size_t mv_dcn_column_budget(void) { return dcn_column_budget(); }

size_t mv_dcn3d_forward_workspace_bytes(const mv_dcn3d_shape *shape, int dtype) {
  DcnDims s;
  return make_dcn_dims(s, shape) ? 0 : forward_workspace(s, dtype);
}

size_t mv_dcn3d_backward_workspace_bytes(const mv_dcn3d_shape *shape, int dtype) {
  DcnDims s;
  return make_dcn_dims(s, shape) ? 0 : backward_workspace(s, dtype);
}

int mv_dcn3d_forward(const void *input, const void *offset, const void *mask, const void *weight,
                     const void *bias, void *output, const mv_dcn3d_shape *shape, int dtype,
                     void *workspace, void *stream) {
  DcnDims s;
  const int st = make_dcn_dims(s, shape);
  return st ? st : dcn_forward_any(input, offset, mask, weight, bias, output, s, dtype, workspace, stream);
}

int mv_dcn3d_backward(const void *input, const void *offset, const void *mask, const void *weight,
                      const void *grad_output, void *grad_input, void *grad_offset,
                      void *grad_mask, void *grad_weight, void *grad_bias,
                      const mv_dcn3d_shape *shape, int dtype, void *workspace, void *stream) {
  DcnDims s;
  const int st = make_dcn_dims(s, shape);
  return st ? st
            : dcn_backward_any(input, offset, mask, weight, grad_output, grad_input, grad_offset,
                               grad_mask, grad_weight, grad_bias, s, dtype, workspace, stream);
}

// ---- forward without any allocation --------------------------------------------------------
// Callers that cannot allocate (code under graph capture, serving loops, harnesses that forbid
// hipMalloc) get the forward pass with the workspace taken from a fixed array in device memory.
// Each GPU the library runs on holds its own copy of the array at its own address; the address is
// looked up once per device, on the first call there, and only that pointer is handed to kernels.
constexpr size_t kStaticScratchBytes = MV_DCN3D_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kScratchDevices = 64;
static std::atomic<void *> scratch_address[kScratchDevices];

static int static_scratch(void **ptr) {
  int dev = -1;
  MV_HIP_CHECK(hipGetDevice(&dev));
  MV_REQUIRE(dev >= 0 && dev < kScratchDevices, "device index beyond the table of scratch addresses");
  void *p = scratch_address[dev].load(std::memory_order_acquire);
  if (p == nullptr) {   // first call on this device (two threads racing resolve the same address)
    MV_HIP_CHECK(hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch)));
    MV_REQUIRE(p != nullptr, "the static scratch array has no address on this device");
    scratch_address[dev].store(p, std::memory_order_release);
  }
  *ptr = p;
  return MV_OK;
}

int mv_dcn3d_forward_static(const void *input, const void *offset, const void *mask,
                            const void *weight, const void *bias, void *output,
                            const mv_dcn3d_shape *shape, int dtype, void *stream) {
  DcnDims s;
  const int st = make_dcn_dims(s, shape);
  if (st) return st;
  const size_t need = forward_workspace(s, dtype);
  MV_REQUIRE(need <= kStaticScratchBytes,
             "mv_dcn3d_forward_static: this layer needs a workspace of %zu bytes, the static scratch holds "
             "%zu; use mv_dcn3d_forward with a caller-provided workspace", need, kStaticScratchBytes);
  void *ws = nullptr;
  if (need > 0) {
    const int sc = static_scratch(&ws);
    if (sc) return sc;
  }
  return dcn_forward_any(input, offset, mask, weight, bias, output, s, dtype, ws, stream);
}

int mv_dcn2d_output_dims(const mv_dcn2d_shape *shape, int *out_h, int *out_w) {
  DcnDims s;
  const int st = make_dcn_dims_2d(s, shape);
  if (st) return st;
  *out_h = s.Ho; *out_w = s.Wo;
  return MV_OK;
}

size_t mv_dcn2d_forward_workspace_bytes(const mv_dcn2d_shape *shape, int dtype) {
  DcnDims s;
  return make_dcn_dims_2d(s, shape) ? 0 : forward_workspace(s, dtype);
}

size_t mv_dcn2d_backward_workspace_bytes(const mv_dcn2d_shape *shape, int dtype) {
  DcnDims s;
  return make_dcn_dims_2d(s, shape) ? 0 : backward_workspace(s, dtype);
}

int mv_dcn2d_forward(const void *input, const void *offset, const void *mask, const void *weight,
                     const void *bias, void *output, const mv_dcn2d_shape *shape, int dtype,
                     void *workspace, void *stream) {
  DcnDims s;
  const int st = make_dcn_dims_2d(s, shape);
  return st ? st : dcn_forward_any(input, offset, mask, weight, bias, output, s, dtype, workspace, stream);
}

int mv_dcn2d_backward(const void *input, const void *offset, const void *mask, const void *weight,
                      const void *grad_output, void *grad_input, void *grad_offset,
                      void *grad_mask, void *grad_weight, void *grad_bias,
                      const mv_dcn2d_shape *shape, int dtype, void *workspace, void *stream) {
  DcnDims s;
  const int st = make_dcn_dims_2d(s, shape);
  return st ? st
            : dcn_backward_any(input, offset, mask, weight, grad_output, grad_input, grad_offset,
                               grad_mask, grad_weight, grad_bias, s, dtype, workspace, stream);
}

int mv_deform_conv_3d(const void *input, const void *offset, const void *weight, const void *bias,
                      void *output, const mv_dcn3d_shape *shape, int dtype, int order, void *stream) {
  DcnDims s;
  const int st = make_dcn_dims(s, shape);
  return st ? st : deform_conv_any(input, offset, weight, bias, output, s, dtype, order, stream);
}

int mv_deform_conv_2d(const void *input, const void *offset, const void *weight, const void *bias,
                      void *output, const mv_dcn2d_shape *shape, int dtype, int order, void *stream) {
  DcnDims s;
  const int st = make_dcn_dims_2d(s, shape);
  return st ? st : deform_conv_any(input, offset, weight, bias, output, s, dtype, order, stream);
}

}  // extern "C"
