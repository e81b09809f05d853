// Direct-to-LDS bf16 GEMM, the instantiations with both operands k-contiguous (forward products).
#include "gemm_dma_impl.h"

int32_t omx_gemm_dma_launch_nn(omx_ctx* ctx, const GemmArgs& g, int variant) {
  return launch_variant<false, false>(ctx, g, variant);
}

