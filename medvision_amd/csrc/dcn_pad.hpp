// Zero-channel padding of deformable-convolution layers whose channel counts the matrix-core kernels
// do not take (see dcn_pad.hip).
#pragma once
#include <algorithm>

#include "dcn_common.hpp"

namespace mv {

struct DcnPad {
  bool on;
  DcnDims p;          // the padded layer
  int unit, unit_p;   // input channels: real channel c sits at (c / unit) * unit_p + c % unit
};

// True (and `pad` filled in) when the layer has channel counts to pad and groups that nest.
bool dcn_pad_plan(const DcnDims &s, int dtype, DcnPad &pad);

// planar tensors [B, C, P] <-> [B, C / unit * unit_p, P], es = bytes per element (2 or 4)
int dcn_pad_channels(const void *src, void *dst, int B, int C, long P, int unit, int unit_p, int es, hipStream_t stream);
int dcn_unpad_channels(const void *src, void *dst, int B, int C, long P, int unit, int unit_p, int es, hipStream_t stream);
// weight [Cout, cpg, K] -> [Cout_p, cpg_p, K]
int dcn_pad_weight(const void *src, void *dst, const DcnDims &s, const DcnPad &pad, int es, hipStream_t stream);
// the matrix-core backward's fp32 accumulators of the padded layer, folded into the real gradients
int dcn_planar_add_padded(const float *gxt, void *gx, const DcnDims &s, const DcnPad &pad, int dtype, hipStream_t stream);
int dcn_weight_add_padded(const float *acc, void *gw, const float *gb_acc, void *gb, const DcnDims &s,
                          const DcnPad &pad, int dtype, hipStream_t stream);

}  // namespace mv
