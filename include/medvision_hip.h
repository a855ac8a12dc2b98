/*
 * C ABI of libmedvision_hip.so -- MI355X (gfx950) kernels for MedVision's trilinear-sampling
 * operator family.  One entry point per function that the reference registers in its pybind11
 * module `medvision._C` for this path (/root/reference/medvision/csrc/vision.cpp:26-77).
 *
 * Conventions (all entry points):
 *   - every pointer is a DEVICE pointer to a dense, contiguous NC(D)HW tensor of element type
 *     `dtype` (mv_dtype); shapes are passed as plain ints;
 *   - `rois` are float32 [num_rois, cols] -- except when dtype == MV_F64, then float64 -- with the
 *     reference's column layouts (5 | 7 | 6 | 10 columns);
 *   - coordinates are computed in fp64 and interpolation weights / accumulation in fp32 (fp64 for
 *     MV_F64) regardless of the storage type;
 *   - `stream` is a hipStream_t (NULL = the null stream); launches are asynchronous, nothing
 *     synchronises;
 *   - return value 0 = success, otherwise an mv_status; mv_last_error() gives the message of the
 *     last failure on the calling thread.  No entry point allocates device memory: scratch is
 *     passed in as `workspace` (size queried with the matching *_workspace_bytes function).
 */
#ifndef MEDVISION_HIP_H
#define MEDVISION_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { MV_F32 = 0, MV_F16 = 1, MV_BF16 = 2, MV_F64 = 3,
               MV_I32 = 4 /* label maps: mv_deform_warp_2d / _3d and mv_affine_2d / _3d, order 0 with one sample per cell only */ } mv_dtype;
typedef enum { MV_OK = 0, MV_INVALID_ARGUMENT = 1, MV_HIP_ERROR = 2 } mv_status;

const char *mv_last_error(void);
int mv_version(void);

/* ---- RoIAlign, plain boxes --------------------------------------------------------------
 * replaces roi_align_2d_forward / roi_align_2d_backward   csrc/roi_align_2d.h (vision.cpp:31-34)
 *          roi_align_3d_forward / roi_align_3d_backward   csrc/roi_align_3d.h:71,98 (vision.cpp:36-39)
 * input  [batch, channels, (depth,) height, width], rois [num_rois, 5 | 7], output
 * [num_rois, channels, (out_d,) out_h, out_w].  order: 0 nearest, 1 linear.
 * backward ACCUMULATES into grad_input (callers pass a zero-filled buffer, like the reference's
 * Python wrapper ops/roi_align_nd.py:139 does).  For MV_F16 / MV_BF16 the backward needs an fp32
 * workspace of mv_roi_align_backward_workspace_bytes(); other dtypes accept NULL.  (fp16 outputs of
 * resampling size whose gradient rows hold an even number of voxels, at sampling ratios 1..3, leave it untouched: the sums of
 * their tiles go to grad_input as packed fp16 atomics, rounded once per tile that reaches a voxel.) */
int mv_roi_align_2d_forward(const void *input, const void *rois, void *output, int dtype,
                            int batch, int channels, int height, int width, int num_rois,
                            int out_h, int out_w, float spatial_scale, int sampling_ratio,
                            int order, void *workspace,
                            size_t workspace_bytes, void *stream);
int mv_roi_align_2d_backward(const void *grad_output, const void *rois, void *grad_input,
                             int dtype, int batch, int channels, int height, int width,
                             int num_rois, int out_h, int out_w, float spatial_scale,
                             int sampling_ratio, int order, void *workspace, void *stream);
int mv_roi_align_3d_forward(const void *input, const void *rois, void *output, int dtype,
                            int batch, int channels, int depth, int height, int width,
                            int num_rois, int out_d, int out_h, int out_w, float spatial_scale,
                            int sampling_ratio, int order, void *workspace,
                            size_t workspace_bytes, void *stream);
int mv_roi_align_3d_backward(const void *grad_output, const void *rois, void *grad_input,
                             int dtype, int batch, int channels, int depth, int height, int width,
                             int num_rois, int out_d, int out_h, int out_w, float spatial_scale,
                             int sampling_ratio, int order, void *workspace, void *stream);

/* ---- RoIAlignRotated ---------------------------------------------------------------------
 * replaces roi_align_rotated_2d_forward/backward  csrc/roi_align_rotated_2d.h (vision.cpp:41-44)
 *          roi_align_rotated_3d_forward/backward  csrc/roi_align_rotated_3d.h:71,98 (vision.cpp:45-48)
 * rois [num_rois, 6] = (b, cx, cy, w, h, theta) or [num_rois, 10] = (b, cx, cy, cz, w, h, d,
 * angle_x, angle_y, angle_z), radians.                                                        */
int mv_roi_align_rotated_2d_forward(const void *input, const void *rois, void *output, int dtype,
                                    int batch, int channels, int height, int width, int num_rois,
                                    int out_h, int out_w, float spatial_scale, int sampling_ratio,
                                    int aligned, int order, void *workspace,
                                    size_t workspace_bytes, void *stream);
int mv_roi_align_rotated_2d_backward(const void *grad_output, const void *rois, void *grad_input,
                                     int dtype, int batch, int channels, int height, int width,
                                     int num_rois, int out_h, int out_w, float spatial_scale,
                                     int sampling_ratio, int aligned, int order, void *workspace,
                                     void *stream);
int mv_roi_align_rotated_3d_forward(const void *input, const void *rois, void *output, int dtype,
                                    int batch, int channels, int depth, int height, int width,
                                    int num_rois, int out_d, int out_h, int out_w,
                                    float spatial_scale, int sampling_ratio, int aligned,
                                    int order, void *workspace,
                                    size_t workspace_bytes, void *stream);
int mv_roi_align_rotated_3d_backward(const void *grad_output, const void *rois, void *grad_input,
                                     int dtype, int batch, int channels, int depth, int height,
                                     int width, int num_rois, int out_d, int out_h, int out_w,
                                     float spatial_scale, int sampling_ratio, int aligned,
                                     int order, void *workspace, void *stream);
size_t mv_roi_align_backward_workspace_bytes(int dtype, int batch, int channels, int depth,
                                             int height, int width);
/* Workspace of the forward entry points (plain, rotated and affine).  0 for a sampling grid of 1 on
 * volumes (the kernels keep their per-call state in LDS), 40 bytes per roi for images of resampling
 * size (their rois are rewritten for the tiled kernel); for fp16 / fp32 outputs of resampling size with a
 * fixed sampling_ratio of 2..4 the bytes of the bins' samples (sampling_ratio^ndim per output
 * element), which a second pass averages (orders 0 and 1 sum the samples of a bin inside the
 * kernel, for any grid, fixed or per roi, and any of the three types: volumes leave the workspace
 * untouched, images use 40 bytes per roi of it; the query is not told the order and answers for order 3).  The forward entry points take the workspace together
 * with its size in bytes (`workspace_bytes`) and use a path only when the workspace holds what that
 * path needs: NULL, or a workspace that is too small, selects the kernels that need none (same
 * results, slower), never an access beyond `workspace_bytes`.  ndim = 2 or 3 (out_d ignored for 2). */
size_t mv_roi_align_forward_workspace_bytes(int dtype, int ndim, int channels, int num_rois,
                                            int out_d, int out_h, int out_w, int sampling_ratio);
/* The same query with the input's shape: the value above when it is not 0; otherwise, for fp16
 * detection heads (plain rois, outputs of up to 8 cells per axis, about as many pooled outputs as
 * input voxels or more, width a multiple of four) the size of a re-ordered copy of the features that
 * mv_roi_align_2d_forward / _3d_forward then read instead of the input (a few voxels of a box row no
 * longer cost a whole memory sector each); and for the heads those kernels do not take (rotated
 * boxes, sampling grids above 4, more than 16 cells per axis; fp16 / bf16 / fp32 with channels in
 * whole 16-byte pieces, at least as many samples as input voxels; plain and rotated entry points) the
 * size of a channels-last copy of the features.  An entry point makes its copy only when
 * `workspace_bytes` is at least this value.  depth ignored for ndim 2.
 * No counterpart in the reference.                                                              */
size_t mv_roi_align_forward_workspace_bytes_for_input(int dtype, int ndim, int batch, int channels, int depth,
                                                      int height, int width, int num_rois, int out_d,
                                                      int out_h, int out_w, int sampling_ratio);

/* Detection heads that pool ONE feature map several times (cascade stages, several batches of rois):
 * the re-ordered copy that mv_roi_align_2d_forward / _3d_forward make in their workspace on every call
 * (fp16 features whose width is a multiple of four) can be made once and handed in.
 * mv_roi_align_prepared_bytes: size of that copy, 0 when the forward pass has no use for one.
 * mv_roi_align_prepare_features: writes it (8-byte aligned pointers; an error when the size is 0 or
 * `prepared_bytes` is smaller).  mv_roi_align_forward_prepared: mv_roi_align_{2,3}d_forward (plain
 * rois; replaces the same reference functions) reading `prepared`, which must have been written from
 * the very contents `input` has now; outputs equal those of the plain entry points bit for bit.  Its
 * workspace wants 4 bytes per roi (the order the rois are worked in; without it they run in the given
 * order).  Heads the copy does not serve (more than 8 cells per axis, order 3, other types) run as
 * through the plain entry points and then want their workspace.  depth / out_d ignored for ndim 2.
 * No counterpart in the reference.                                                              */
size_t mv_roi_align_prepared_bytes(int dtype, int ndim, int batch, int channels, int depth, int height, int width);
int mv_roi_align_prepare_features(const void *input, int dtype, int ndim, int batch, int channels, int depth,
                                  int height, int width, void *prepared, size_t prepared_bytes, void *stream);
int mv_roi_align_forward_prepared(const void *input, const void *prepared, const void *rois, void *output,
                                  int dtype, int ndim, int batch, int channels, int depth, int height, int width,
                                  int num_rois, int out_d, int out_h, int out_w, float spatial_scale,
                                  int sampling_ratio, int order, void *workspace, size_t workspace_bytes,
                                  void *stream);

/* ---- affine resampling engine (forward only) ----------------------------------------------
 * replaces affine_2d  csrc/affine_2d.h (vision.cpp:74), affine_3d  csrc/affine_3d.h:40 (vision.cpp:75)
 * Same arguments and results as the rotated forward for order 0 / 1 (the reference kernel text
 * is identical, csrc/cuda_aug/affine_3d_cuda_kernel.cuh:14-120).  order 3 = clamped Catmull-Rom
 * over 4 x 4 (x 4) voxels (csrc/cuda_aug/interpolation_helpers_3d.h:571-792); the RoIAlign entry
 * points above reject it, as the reference's do.                                              */
int mv_affine_2d(const void *input, const void *rois, void *output, int dtype, int batch,
                 int channels, int height, int width, int num_rois, int out_h, int out_w,
                 float spatial_scale, int sampling_ratio, int aligned, int order, void *workspace,
                 size_t workspace_bytes, void *stream);
int mv_affine_3d(const void *input, const void *rois, void *output, int dtype, int batch,
                 int channels, int depth, int height, int width, int num_rois, int out_d,
                 int out_h, int out_w, float spatial_scale, int sampling_ratio, int aligned,
                 int order, void *workspace,
                 size_t workspace_bytes, void *stream);

/* ---- deformable convolution 3-D -----------------------------------------------------------
 * replaces deform_conv_3d_forward / _backward                 csrc/deform_conv_3d.h:48,87
 *          modulated_deform_conv_3d_forward / _backward       csrc/modulated_deform_conv_3d.h:61,89
 * One shape record serves v1 (mask == NULL) and v2.  Layouts: input [B,Cin,D,H,W], offset
 * [B, dg*3*K, Do,Ho,Wo] (channel 3k+0 = depth, +1 = height, +2 = width displacement of tap k),
 * mask [B, dg*K, Do,Ho,Wo], weight [Cout, Cin/groups, kd,kh,kw], bias [Cout] or NULL, output
 * [B,Cout,Do,Ho,Wo] with Do = (D + 2*pad_d - (dil_d*(kd-1)+1)) / stride_d + 1 etc.
 * The backward accumulates into grad_weight / grad_bias / grad_input and overwrites
 * grad_offset / grad_mask; grad_mask and grad_bias may be NULL.                               */
typedef struct {
  int batch, in_channels, depth, height, width;
  int out_channels, kernel_d, kernel_h, kernel_w;
  int stride_d, stride_h, stride_w;
  int pad_d, pad_h, pad_w;
  int dil_d, dil_h, dil_w;
  int groups, deformable_groups;
} mv_dcn3d_shape;

int mv_dcn3d_output_dims(const mv_dcn3d_shape *shape, int *out_d, int *out_h, int *out_w);
size_t mv_dcn3d_forward_workspace_bytes(const mv_dcn3d_shape *shape, int dtype);
/* The backward workspace of 16-bit / fp32 layers on the matrix-core path includes a buffer of column
 * values (batch x taps x in_channels x positions elements) while that stays below 1 GiB or the number
 * of bytes set with mv_dcn_set_column_budget() / the environment variable MV_DCN_COLUMN_BYTES. */
size_t mv_dcn3d_backward_workspace_bytes(const mv_dcn3d_shape *shape, int dtype);
int mv_dcn3d_forward(const void *input, const void *offset, const void *mask, const void *weight,
                     const void *bias, void *output, const mv_dcn3d_shape *shape, int dtype,
                     void *workspace, void *stream);
int mv_dcn3d_backward(const void *input, const void *offset, const void *mask, const void *weight,
                      const void *grad_output, void *grad_input, void *grad_offset,
                      void *grad_mask, void *grad_weight, void *grad_bias,
                      const mv_dcn3d_shape *shape, int dtype, void *workspace, void *stream);

/* Budget of the backward pass's column buffer in bytes (default 1 GiB, or MV_DCN_COLUMN_BYTES in the
 * environment when the library is first asked).  Changing it changes what
 * mv_dcn{2,3}d_backward_workspace_bytes() returns: query again.  No counterpart in the reference
 * (its column buffer is a tensor argument, csrc/modulated_deform_conv_3d.h:89).               */
void mv_dcn_set_column_budget(size_t bytes);
size_t mv_dcn_column_budget(void);

/* mv_dcn3d_forward for callers that cannot allocate or provide device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): no counterpart in the reference.
 * Same arguments and results as mv_dcn3d_forward without `workspace`: the layout buffers live in a
 * fixed array of MV_DCN3D_STATIC_SCRATCH_BYTES in the library's device image (every GPU the
 * library runs on holds it until the process ends).  Calls no hipMalloc / hipFree or allocating
 * library routine; the first call on a device looks the array's address up (hipGetSymbolAddress,
 * which may load the code object): make that call once OUTSIDE any graph capture.  Every process that
 * loads the library holds the array on each GPU it runs kernels on.  Layers whose
 * mv_dcn3d_forward_workspace_bytes() exceeds the array are rejected with MV_INVALID_ARGUMENT.
 * All calls on one GPU share the array: calls that overlap on one GPU (two streams, two threads)
 * race; serialise them.                                                                        */
#define MV_DCN3D_STATIC_SCRATCH_BYTES ((size_t)32 << 20)
int mv_dcn3d_forward_static(const void *input, const void *offset, const void *mask,
                            const void *weight, const void *bias, void *output,
                            const mv_dcn3d_shape *shape, int dtype, void *stream);

/* ---- deformable convolution 2-D -----------------------------------------------------------
 * replaces deform_conv_2d_forward / _backward                 csrc/deform_conv_2d.h:41,76
 *          modulated_deform_conv_2d_forward / _backward       csrc/modulated_deform_conv_2d.h:23,47
 * (vision.cpp:50-51,56-59).  Same conventions as the 3-D entry points with images instead of
 * volumes: input [B,Cin,H,W], offset [B, dg*2*K, Ho,Wo] (channel 2k+0 = height, 2k+1 = width
 * displacement of tap k = i*kw + j), mask [B, dg*K, Ho,Wo], weight [Cout, Cin/groups, kh,kw].
 * The same kernels run (an image is a depth-1 volume).                                        */
typedef struct {
  int batch, in_channels, height, width;
  int out_channels, kernel_h, kernel_w;
  int stride_h, stride_w;
  int pad_h, pad_w;
  int dil_h, dil_w;
  int groups, deformable_groups;
} mv_dcn2d_shape;

int mv_dcn2d_output_dims(const mv_dcn2d_shape *shape, int *out_h, int *out_w);
size_t mv_dcn2d_forward_workspace_bytes(const mv_dcn2d_shape *shape, int dtype);
size_t mv_dcn2d_backward_workspace_bytes(const mv_dcn2d_shape *shape, int dtype);
int mv_dcn2d_forward(const void *input, const void *offset, const void *mask, const void *weight,
                     const void *bias, void *output, const mv_dcn2d_shape *shape, int dtype,
                     void *workspace, void *stream);
int mv_dcn2d_backward(const void *input, const void *offset, const void *mask, const void *weight,
                      const void *grad_output, void *grad_input, void *grad_offset,
                      void *grad_mask, void *grad_weight, void *grad_bias,
                      const mv_dcn2d_shape *shape, int dtype, void *workspace, void *stream);

/* ---- displacement-field warp (elastic engine) -----------------------------------------------
 * replaces deform_2d / deform_3d  csrc/deform_2d.h, csrc/deform_3d.h:27 (vision.cpp:71-72) for the
 * way the reference calls them (ops/cuda_fun_tools.py:94-167: 1x1x1 kernel, identity weight,
 * zero bias): out[b,c,q] = S(img[b,c], q + off[b,:,q]) on the open interval (-1, size), else 0;
 * order 0, 1 or 3 as for the affine engine.
 * img/out [B,C,(D,)H,W], offset [B, 2|3, (D,)H,W] (3-D: 0 = depth, 1 = height, 2 = width).
 * dtype MV_I32 (order 0 only): img/out are int32 label maps and offset is float32 -- the voxel the
 * reference picks after converting the labels to float (aug_cuda/aug_spatial.py:664-668), without
 * the two conversion passes.                                                                      */
int mv_deform_warp_2d(const void *img, const void *offset, void *output, int dtype, int batch,
                      int channels, int height, int width, int order, void *stream);
int mv_deform_warp_3d(const void *img, const void *offset, void *output, int dtype, int batch,
                      int channels, int depth, int height, int width, int order, void *stream);

/* ---- augmentation DCN in general ----------------------------------------------------------------
 * replaces deform_2d / deform_3d  csrc/deform_2d.h, csrc/deform_3d.h:27 (vision.cpp:71-72; host
 * csrc/cuda_aug/deform_3d_cuda.cu:43-152, kernel csrc/cuda_aug/deform_3d_cuda_kernel.cuh:8-89) for
 * any kernel, stride, padding, dilation, groups and weight: the DCNv1 forward whose column value is
 * the border-replicating sampler of the affine engine, S(x[b,c], p) when -1 < p < size on every
 * axis and 0 otherwise (order 0, 1 or 3), instead of the zero-padded trilinear form.
 * Tensors as for mv_dcn3d_forward / mv_dcn2d_forward without mask; bias may be NULL.            */
int mv_deform_conv_3d(const void *input, const void *offset, const void *weight, const void *bias,
                      void *output, const mv_dcn3d_shape *shape, int dtype, int order, void *stream);
int mv_deform_conv_2d(const void *input, const void *offset, const void *weight, const void *bias,
                      void *output, const mv_dcn2d_shape *shape, int dtype, int order, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MEDVISION_HIP_H */
