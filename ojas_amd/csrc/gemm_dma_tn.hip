// Direct-to-LDS bf16 GEMM, the instantiations with A k-major, B k-contiguous.
#include "gemm_dma_impl.h"

int32_t omx_gemm_dma_launch_tn(omx_ctx* ctx, const GemmArgs& g, int variant) {
  return launch_variant<true, false>(ctx, g, variant);
}
