// Direct-to-LDS bf16 GEMM, the instantiations with A k-contiguous, B k-major (input gradients).
#include "gemm_dma_impl.h"

int32_t omx_gemm_dma_launch_nt(omx_ctx* ctx, const GemmArgs& g, int variant) {
  return launch_variant<false, true>(ctx, g, variant);
}
