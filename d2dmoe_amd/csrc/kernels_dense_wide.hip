// The fused experts kernel ("masked dense sweep") at D = 1024: GPT-2 medium, BERT-large, ViT-L.  Same tile routine as at
// D = 768 with a chunk of 128 neurons (the x tile of 64 tokens takes 128 KB of the 160 KB of LDS) and the routing values
// fetched from global memory one chunk ahead.
#include "dense_sweep.hpp"

namespace d2dmoe {

hipError_t launch_mfma_dense_wide(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                                  const void* last_bias, void* out, const int* skip_flag, void* workspace,
                                  size_t workspace_bytes, hipStream_t s) {
  if (sh.d_model != 1024) return hipErrorInvalidValue;
  switch (sh.activation) {
    case D2DMOE_ACT_RELU:
      return launch_dense_act<1024, D2DMOE_ACT_RELU>(sh, x, routing, packed, last_bias, out, skip_flag, workspace, workspace_bytes, s);
    case D2DMOE_ACT_GELU:
      return launch_dense_act<1024, D2DMOE_ACT_GELU>(sh, x, routing, packed, last_bias, out, skip_flag, workspace, workspace_bytes, s);
    default:
      return launch_dense_act<1024, -1>(sh, x, routing, packed, last_bias, out, skip_flag, workspace, workspace_bytes, s);
  }
}

}  // namespace d2dmoe
