// Matrix-core (MFMA) forward of the 3-D deformable convolution for fp16 / bf16 tensors.
#include "dcn_common.hpp"

namespace mv {

bool dcn_mfma_supported(const DcnDims &, int) { return false; }
size_t dcn_mfma_workspace_bytes(const DcnDims &, int) { return 0; }
int dcn_mfma_forward(const void *, const void *, const void *, const void *, const void *, void *,
                     const DcnDims &, int, void *, hipStream_t) {
  return fail(MV_INVALID_ARGUMENT, "matrix-core DCN forward is not available for this shape");
}

}  // namespace mv
