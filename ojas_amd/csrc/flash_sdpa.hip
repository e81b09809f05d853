// bf16 MFMA flash attention for head_dim 64 / 128 (placeholder until the
// tiled kernels land: every shape currently takes the row kernels).
#include "omx_common.h"

bool omx_flash_sdpa_supports(uint64_t, int32_t) { return false; }

int32_t omx_flash_sdpa_forward(omx_ctx* ctx, const void*, const void*, const void*, void*, int32_t, float*, uint64_t,
                               uint64_t, uint64_t, uint64_t, uint64_t, uint64_t, float, unsigned long long) {
  return omx_fail(ctx, OMX_UNSUPPORTED, "flash sdpa forward");
}
int32_t omx_flash_sdpa_backward(omx_ctx* ctx, const void*, const void*, const void*, const void*, const float*,
                                const void*, void*, void*, void*, int32_t, uint64_t, uint64_t, uint64_t, uint64_t,
                                uint64_t, uint64_t, float, unsigned long long) {
  return omx_fail(ctx, OMX_UNSUPPORTED, "flash sdpa backward");
}
