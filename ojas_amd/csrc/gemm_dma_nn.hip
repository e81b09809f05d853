// Direct-to-LDS bf16 GEMM, the instantiations with both operands k-contiguous (forward products).
#include "gemm_dma_impl.h"

int32_t omx_gemm_dma_launch_nn(omx_ctx* ctx, const GemmArgs& g, int variant) {
  return launch_variant<false, false>(ctx, g, variant);
}

#ifdef W4_TRACE
extern "C" int omx_debug_w4_trace(void* buf) {
  long long* p = static_cast<long long*>(buf);
  return static_cast<int>(hipMemcpyToSymbol(HIP_SYMBOL(w4_trace_buf), &p, sizeof(p)));
}
#endif
