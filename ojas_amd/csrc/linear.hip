// BackendModule::linear_forward / linear_backward / linear_backward_input
// (ojas-core/src/backend.rs:1628-1656) over the MFMA GEMM.
//
//   y [rows,out] = x [rows,in] . W[out,in]^T      (ojas-cpu/src/linalg.rs:69-89)
//   gx[rows,in]  = gy[rows,out] . W[out,in]       (linalg.rs:105-184, sum over out)
//   gw[out,in]   = gy[rows,out]^T . x[rows,in]    (sum over rows)
//
// The transposes are strides the GEMM packs through, never copies.
#include "omx_common.h"

namespace {

// A bf16 operand next to an f32 one is widened exactly into the workspace
// (the reference widens bf16 operands the same way, ojas-cpu/src/validate.rs:178-208).
struct Widened {
  const void* x;
  const void* w;
  int32_t dtype;
};

int32_t unify(omx_ctx* ctx, const char* op, const void* x, int32_t x_dtype, uint64_t x_len, const void* w,
              int32_t w_dtype, uint64_t w_len, Widened* out) {
  if (!omx_valid_float_dtype(x_dtype) || !omx_valid_float_dtype(w_dtype))
    return omx_fail(ctx, OMX_DTYPE, "%s: operands must be f32 or bf16", op);
  out->x = x;
  out->w = w;
  out->dtype = x_dtype;
  if (x_dtype == w_dtype) return OMX_OK;
  void* ws = nullptr;
  if (x_dtype == OMX_BF16) {
    int32_t rc = omx_workspace(ctx, x_len * 4, &ws);
    if (rc != OMX_OK) return rc;
    rc = omx_convert(ctx, x, OMX_BF16, ws, OMX_F32, x_len);
    if (rc != OMX_OK) return rc;
    out->x = ws;
  } else {
    int32_t rc = omx_workspace(ctx, w_len * 4, &ws);
    if (rc != OMX_OK) return rc;
    rc = omx_convert(ctx, w, OMX_BF16, ws, OMX_F32, w_len);
    if (rc != OMX_OK) return rc;
    out->w = ws;
  }
  out->dtype = OMX_F32;
  return OMX_OK;
}

}  // namespace

extern "C" {

int32_t omx_linear_forward(omx_ctx* ctx, const void* x, int32_t x_dtype, const void* w, int32_t w_dtype, void* y,
                           int32_t y_dtype, uint64_t rows, uint64_t in_features, uint64_t out_features) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "linear_forward";
  if (!x || !w || !y) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (rows == 0 || in_features == 0 || out_features == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  Widened u;
  int32_t rc = unify(ctx, op, x, x_dtype, rows * in_features, w, w_dtype, out_features * in_features, &u);
  if (rc != OMX_OK) return rc;
  // A(i,p) = x[i*in + p]; B(p,j) = W[j*in + p].
  return omx_gemm_impl(ctx, F_LINEAR_FORWARD, u.x, in_features, 1, u.w, 1, in_features, u.dtype, y, y_dtype,
                       out_features, rows, in_features, out_features, 0);
}

int32_t omx_linear_backward(omx_ctx* ctx, const void* x, const void* w, const void* gy, int32_t operand_dtype,
                            void* gx, int32_t gx_dtype, void* gw, int32_t gw_dtype, uint64_t rows,
                            uint64_t in_features, uint64_t out_features) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "linear_backward";
  if (!gy || (!gx && !gw)) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (gx && !w) return omx_fail(ctx, OMX_PLACEMENT, "%s: weight is null", op);
  if (gw && !x) return omx_fail(ctx, OMX_PLACEMENT, "%s: input is null", op);
  if (rows == 0 || in_features == 0 || out_features == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (gx) {
    // gx(i,j) = sum_o gy[i*out + o] * W[o*in + j]
    int32_t rc = omx_gemm_impl(ctx, F_LINEAR_BACKWARD, gy, out_features, 1, w, in_features, 1, operand_dtype, gx,
                               gx_dtype, in_features, rows, out_features, in_features, 0);
    if (rc != OMX_OK) return rc;
  }
  if (gw) {
    // gw(o,j) = sum_r gy[r*out + o] * x[r*in + j]
    int32_t rc = omx_gemm_impl(ctx, F_LINEAR_BACKWARD, gy, 1, out_features, x, in_features, 1, operand_dtype, gw,
                               gw_dtype, in_features, out_features, rows, in_features, 0);
    if (rc != OMX_OK) return rc;
  }
  return OMX_OK;
}

// linear_forward followed by gelu (ojas-model block: up-projection then activation), the
// activation applied in the product's store pass: u = x W^T and act = gelu(u), both bf16.
int32_t omx_linear_gelu_forward(omx_ctx* ctx, const void* x, const void* w, int32_t operand_dtype, void* u, void* act,
                                uint64_t rows, uint64_t in_features, uint64_t out_features, int32_t tanh_form) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "linear_gelu_forward";
  if (!x || !w || !u || !act) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (operand_dtype != OMX_BF16) return omx_fail(ctx, OMX_UNSUPPORTED, "%s: bf16 operands only", op);
  if (rows == 0 || in_features == 0 || out_features == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  OmxGemmEpilogue epi = {OMX_EPI_GELU_FWD, tanh_form ? 1 : 0, nullptr, act};
  return omx_gemm_impl(ctx, F_LINEAR_FORWARD, x, in_features, 1, w, 1, in_features, operand_dtype, u, OMX_BF16,
                       out_features, rows, in_features, out_features, 0, &epi);
}

// The input gradient of linear_backward followed by gelu_backward: gu = (gy W) * gelu'(u),
// the derivative applied in the product's store pass. gy [rows, out], w [out, in], u / gu [rows, in].
int32_t omx_linear_backward_input_gelu(omx_ctx* ctx, const void* w, const void* gy, int32_t operand_dtype,
                                       const void* u, void* gu, uint64_t rows, uint64_t in_features,
                                       uint64_t out_features, int32_t tanh_form) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "linear_backward_input_gelu";
  if (!w || !gy || !u || !gu) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (operand_dtype != OMX_BF16) return omx_fail(ctx, OMX_UNSUPPORTED, "%s: bf16 operands only", op);
  if (rows == 0 || in_features == 0 || out_features == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  OmxGemmEpilogue epi = {OMX_EPI_GELU_BWD, tanh_form ? 1 : 0, u, nullptr};
  return omx_gemm_impl(ctx, F_LINEAR_BACKWARD, gy, out_features, 1, w, in_features, 1, operand_dtype, gu, OMX_BF16,
                       in_features, rows, out_features, in_features, 0, &epi);
}

}  // extern "C"
