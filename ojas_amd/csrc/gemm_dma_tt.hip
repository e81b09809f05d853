// Direct-to-LDS bf16 GEMM, the instantiations with both operands k-major (weight gradients).
#include "gemm_dma_impl.h"

int32_t omx_gemm_dma_launch_tt(omx_ctx* ctx, const GemmArgs& g, int variant) {
  return launch_variant<true, true>(ctx, g, variant);
}
