// What the nanolab block does to a fused q | k | v projection output before attention, in one pass
// over HBM each way: per-head RMSNorm of q and k (rms_qk_norm, ojas-cpu/src/norm.rs:60-180), the
// half-split rotary embedding on the result (norm.rs:271-347), and the value-residual blend on v
// (ojas-cpu/src/pointwise.rs:2031-2148); the graph is ojas-model/src/block.rs:225-240. Tensors
// whose token rows are `pitch` elements apart and hold, per token, the query heads, then the key
// heads, then the value heads. The prepared q | k | v and the gradients are bf16 (operands of the
// attention products and of the projection's backward); the projection output itself (and block
// 0's, for the blend) is bf16 or f32: kept in f32 it reaches attention with one rounding.
//
// A head row (64 or 128 values) is held by head_dim / 8 adjacent lanes, 8 values (one 16-byte
// access) each: the row's sum of squares is a shuffle reduction over those lanes and the rotary
// partner of a value sits in the lane half a row away. The normed row is not rounded to bf16
// between the norm and the rotation (the separate ops round there).
#include "omx_common.h"

namespace {

constexpr int QP_THREADS = 256;

struct QkvShape {
  long tokens, pitch, time;
  int heads, kv_heads, dim;
  float eps;
};

__device__ __forceinline__ void unpack8(const uint4& w, float (&v)[8]) {
  const unsigned int ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(ww[i] << 16);
    v[2 * i + 1] = __uint_as_float(ww[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ uint4 pack8(const float (&v)[8]) {
  unsigned int w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = dev_pack_bf16_pair(v[2 * i], v[2 * i + 1]);
  return make_uint4(w[0], w[1], w[2], w[3]);
}
__device__ __forceinline__ void load8f(const float* __restrict__ p, float (&v)[8]);
// Eight consecutive values of a projection output stored as bf16 or as f32.
__device__ __forceinline__ void load_lin(const unsigned short* __restrict__ p, float (&v)[8]) {
  unpack8(*reinterpret_cast<const uint4*>(p), v);
}
__device__ __forceinline__ void load_lin(const float* __restrict__ p, float (&v)[8]) { load8f(p, v); }
__device__ __forceinline__ void load8f(const float* __restrict__ p, float (&v)[8]) {
  const float4 a = reinterpret_cast<const float4*>(p)[0], b = reinterpret_cast<const float4*>(p)[1];
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
// Sum over the LPR adjacent lanes that hold one row.
template <int LPR>
__device__ __forceinline__ float row_sum(float v) {
#pragma unroll
  for (int m = 1; m < LPR; m <<= 1) v += __shfl_xor(v, m, 64);
  return v;
}
// sigmoid(u) and 1 - sigmoid(u), both without cancellation.
__device__ __forceinline__ void sigmoid_both(float u, float* s, float* rest) {
  const float e = __expf(-fabsf(u));
  const float inv = 1.0f / (1.0f + e);
  *s = u >= 0.0f ? inv : e * inv;
  *rest = u >= 0.0f ? e * inv : inv;
}

// Row r of the launch is (token, slot): slot < heads is a query head, the next kv_heads are key
// heads, the rest value heads.
template <int D, typename LIN>
__global__ __launch_bounds__(QP_THREADS) void qkv_prepare_fwd_kernel(
    const LIN* __restrict__ lin, unsigned short* __restrict__ out, const float* __restrict__ q_weight,
    const float* __restrict__ k_weight, const float* __restrict__ cos, const float* __restrict__ sin,
    const LIN* __restrict__ v0, const float* __restrict__ lambda, QkvShape s, OmxFaultWord* fault,
    unsigned long long tag) {
  constexpr int LPR = D / 8, ROWS = QP_THREADS / LPR;
  const int slots = s.heads + 2 * s.kv_heads;
  const long rows = s.tokens * slots;
  const int col = (threadIdx.x % LPR) * 8;
  const bool second_half = col >= D / 2;
  float blend_s = 0.0f, blend_rest = 1.0f;
  bool bad = false;
  if (v0) {
    sigmoid_both(*lambda, &blend_s, &blend_rest);
    bad |= !dev_finite(blend_s);
  }
  for (long r = static_cast<long>(blockIdx.x) * ROWS + threadIdx.x / LPR; r < rows; r += static_cast<long>(gridDim.x) * ROWS) {
    const long token = r / slots;
    const int slot = static_cast<int>(r % slots);
    const long at = token * s.pitch + static_cast<long>(slot) * D + col;
    float x[8], y[8];
    load_lin(lin + at, x);
    if (slot >= s.heads + s.kv_heads) {
      if (v0) {
        float b[8];
        load_lin(v0 + at, b);
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = blend_rest * x[i] + blend_s * b[i];
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = x[i];
      }
    } else {
      float ss = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += x[i] * x[i];
      ss = row_sum<LPR>(ss);
      const float denom = ss / static_cast<float>(D) + s.eps;
      const float rstd = 1.0f / sqrtf(denom);
      bad |= !(dev_finite(denom) && denom > 0.0f && dev_finite(rstd));
      float w[8], c[8], sn[8];
      load8f((slot < s.heads ? q_weight : k_weight) + col, w);
      const long trow = (token % s.time) * D + col;
      load8f(cos + trow, c);
      load8f(sin + trow, sn);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float n = x[i] * rstd * w[i];
        const float partner = __shfl_xor(n, LPR / 2, 64);
        // y = n cos + cat(-n2, n1) sin
        y[i] = second_half ? n * c[i] + partner * sn[i] : n * c[i] + (-partner) * sn[i];
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) bad |= !dev_finite(y[i]);
    *reinterpret_cast<uint4*>(out + at) = pack8(y);
  }
  if (bad) dev_raise_fault(fault, tag);
}

// The backward of the above. g is the gradient of the prepared q | k | v (same layout), g_lin that
// of the projection output. The norm weights' gradients leave as per-workgroup partial sums
// (partial_w: [blocks][2][D], q then k) and the blend's as one partial per workgroup; v0_acc
// (f32 [tokens, kv_heads * D]) collects what the blends send to block 0's value, written when
// `v0_first` and added to otherwise; `add_v` (block 0 only, no blend) is added to the value's gradient.
template <int D, typename LIN>
__global__ __launch_bounds__(QP_THREADS) void qkv_prepare_bwd_kernel(
    const LIN* __restrict__ lin, const unsigned short* __restrict__ g, unsigned short* __restrict__ g_lin,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, const float* __restrict__ cos,
    const float* __restrict__ sin, const LIN* __restrict__ v0, const float* __restrict__ lambda,
    float* __restrict__ v0_acc, int v0_first, const float* __restrict__ add_v, float* __restrict__ partial_w,
    float* __restrict__ partial_lambda, QkvShape s, OmxFaultWord* fault, unsigned long long tag) {
  constexpr int LPR = D / 8, ROWS = QP_THREADS / LPR;
  __shared__ float red[2][ROWS][D];
  __shared__ float red_lambda[QP_THREADS / 64];
  const int slots = s.heads + 2 * s.kv_heads;
  const long rows = s.tokens * slots;
  const int col = (threadIdx.x % LPR) * 8, sub = threadIdx.x / LPR;
  const bool second_half = col >= D / 2;
  float blend_s = 0.0f, blend_rest = 1.0f;
  bool bad = false;
  if (v0) {
    sigmoid_both(*lambda, &blend_s, &blend_rest);
    bad |= !dev_finite(blend_s);
  }
  float acc_w[2][8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc_w[0][i] = acc_w[1][i] = 0.0f;
  float acc_lambda = 0.0f;
  const long kv_cols = static_cast<long>(s.kv_heads) * D;
  for (long r = static_cast<long>(blockIdx.x) * ROWS + sub; r < rows; r += static_cast<long>(gridDim.x) * ROWS) {
    const long token = r / slots;
    const int slot = static_cast<int>(r % slots);
    const long at = token * s.pitch + static_cast<long>(slot) * D + col;
    float x[8], gy[8], out[8];
    load_lin(lin + at, x);
    unpack8(*reinterpret_cast<const uint4*>(g + at), gy);
    if (slot >= s.heads + s.kv_heads) {
      const long vat = token * kv_cols + static_cast<long>(slot - s.heads - s.kv_heads) * D + col;
      if (v0) {
        float b[8];
        load_lin(v0 + at, b);
        float* acc = v0_acc + vat;
        float keep[8];
        if (!v0_first) load8f(acc, keep);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          out[i] = blend_rest * gy[i];
          const float to_v0 = blend_s * gy[i];
          keep[i] = v0_first ? to_v0 : keep[i] + to_v0;
          acc_lambda += (b[i] - x[i]) * gy[i];
        }
        reinterpret_cast<float4*>(acc)[0] = make_float4(keep[0], keep[1], keep[2], keep[3]);
        reinterpret_cast<float4*>(acc)[1] = make_float4(keep[4], keep[5], keep[6], keep[7]);
      } else if (add_v) {
        float a[8];
        load8f(add_v + vat, a);
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = gy[i] + a[i];
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = gy[i];
      }
    } else {
      const int which = slot < s.heads ? 0 : 1;
      float w[8], c[8], sn[8];
      load8f((which == 0 ? q_weight : k_weight) + col, w);
      const long trow = (token % s.time) * D + col;
      load8f(cos + trow, c);
      load8f(sin + trow, sn);
      float ss = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += x[i] * x[i];
      ss = row_sum<LPR>(ss);
      const float denom = ss / static_cast<float>(D) + s.eps;
      const float rstd = 1.0f / sqrtf(denom);
      bad |= !(dev_finite(denom) && denom > 0.0f && dev_finite(rstd));
      float gn[8], dot = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float partner = __shfl_xor(gy[i], LPR / 2, 64);
        // the rotation's transpose: gx1 = g1 c1 + g2 s2, gx2 = -g1 s1 + g2 c2 (both table halves are equal)
        gn[i] = second_half ? gy[i] * c[i] + (-partner) * sn[i] : gy[i] * c[i] + partner * sn[i];
        dot += (gn[i] * w[i]) * (x[i] * rstd);
      }
      const float mean = row_sum<LPR>(dot) / static_cast<float>(D);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float xhat = x[i] * rstd;
        out[i] = (gn[i] * w[i] - xhat * mean) * rstd;
        acc_w[which][i] += gn[i] * xhat;
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) bad |= !dev_finite(out[i]);
    *reinterpret_cast<uint4*>(g_lin + at) = pack8(out);
  }
  // The workgroup's partial sums, added in a fixed order.
#pragma unroll
  for (int which = 0; which < 2; ++which)
#pragma unroll
    for (int i = 0; i < 8; ++i) red[which][sub][col + i] = acc_w[which][i];
  float lam = acc_lambda;
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) lam += __shfl_xor(lam, m, 64);
  if ((threadIdx.x & 63) == 0) red_lambda[threadIdx.x >> 6] = lam;
  __syncthreads();
  for (int i = threadIdx.x; i < 2 * D; i += QP_THREADS) {
    const int which = i / D, c = i % D;
    float sum = 0.0f;
    for (int row = 0; row < ROWS; ++row) sum += red[which][row][c];
    partial_w[(static_cast<long>(blockIdx.x) * 2 + which) * D + c] = sum;
  }
  if (threadIdx.x == 0) partial_lambda[blockIdx.x] = ((red_lambda[0] + red_lambda[1]) + red_lambda[2]) + red_lambda[3];
  if (bad) dev_raise_fault(fault, tag);
}

// g_lambda = s (1 - s) x the sum of the workgroups' partials, added in order by one workgroup.
__global__ __launch_bounds__(256) void qkv_lambda_kernel(const float* __restrict__ partial, int blocks,
                                                         const float* __restrict__ lambda, float* __restrict__ g_lambda,
                                                         OmxFaultWord* fault, unsigned long long tag) {
  __shared__ float red[256];
  float acc = 0.0f;
  for (int b = threadIdx.x; b < blocks; b += 256) acc += partial[b];
  red[threadIdx.x] = acc;
  __syncthreads();
  for (int step = 128; step >= 1; step >>= 1) {
    if (threadIdx.x < step) red[threadIdx.x] += red[threadIdx.x + step];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    float s, rest;
    sigmoid_both(*lambda, &s, &rest);
    const float v = red[0] * s * rest;
    if (!dev_finite(v)) dev_raise_fault(fault, tag);
    *g_lambda = v;
  }
}

int32_t check(omx_ctx* ctx, const char* op, uint64_t pitch, uint64_t tokens, uint64_t time, uint64_t heads,
              uint64_t kv_heads, uint64_t head_dim, float eps, std::initializer_list<const void*> ptrs) {
  for (const void* p : ptrs)
    if (!p) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (tokens == 0 || time == 0 || heads == 0 || kv_heads == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (head_dim != 64 && head_dim != 128)
    return omx_fail(ctx, OMX_UNSUPPORTED, "%s: head_dim %llu (64 and 128 are built)", op, (unsigned long long)head_dim);
  if (pitch % 8 != 0 || pitch < (heads + 2 * kv_heads) * head_dim)
    return omx_fail(ctx, OMX_SHAPE, "%s: pitch %llu must be a multiple of 8 and hold %llu heads of %llu", op,
                    (unsigned long long)pitch, (unsigned long long)(heads + 2 * kv_heads), (unsigned long long)head_dim);
  if (!(eps == eps) || eps == INFINITY || eps == -INFINITY) return omx_fail(ctx, OMX_NON_FINITE, "%s", op);
  if (tokens > 0x7fffffffull || pitch > 0x7fffffffull) return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: axis does not fit in i32", op);
  uintptr_t bits = 0;
  for (const void* p : ptrs) bits |= reinterpret_cast<uintptr_t>(p);
  if (bits & 15u) return omx_fail(ctx, OMX_SHAPE, "%s: pointers must be 16-byte aligned", op);
  return OMX_OK;
}

unsigned grid_for(const omx_ctx* ctx, uint64_t rows, int rows_per_block) {
  const uint64_t want = (rows + rows_per_block - 1) / rows_per_block;
  const uint64_t cap = static_cast<uint64_t>(ctx->cu_count > 0 ? ctx->cu_count : 256) * 8;
  return static_cast<unsigned>(want < cap ? (want > 0 ? want : 1) : cap);
}

}  // namespace

extern "C" {

int32_t omx_qkv_prepare_forward(omx_ctx* ctx, const void* qkv_lin, int32_t lin_dtype, void* qkv_out, uint64_t pitch, const void* q_weight,
                                const void* k_weight, const void* cos, const void* sin, const void* value0,
                                const void* lambda, uint64_t tokens, uint64_t time, uint64_t heads, uint64_t kv_heads,
                                uint64_t head_dim, float eps) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "qkv_prepare_forward";
  if (!omx_valid_float_dtype(lin_dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: the projection output must be f32 or bf16", op);
  int32_t rc = check(ctx, op, pitch, tokens, time, heads, kv_heads, head_dim, eps, {qkv_lin, qkv_out, q_weight, k_weight, cos, sin});
  if (rc != OMX_OK) return rc;
  if ((value0 != nullptr) != (lambda != nullptr)) return omx_fail(ctx, OMX_PLACEMENT, "%s: value0 and lambda come together", op);
  if (value0 && (reinterpret_cast<uintptr_t>(value0) & 15u)) return omx_fail(ctx, OMX_SHAPE, "%s: pointers must be 16-byte aligned", op);
  QkvShape s{static_cast<long>(tokens), static_cast<long>(pitch), static_cast<long>(time), static_cast<int>(heads),
             static_cast<int>(kv_heads), static_cast<int>(head_dim), eps};
  const uint64_t rows = tokens * (heads + 2 * kv_heads);
  const unsigned long long tag = omx_tag(ctx, F_RMS_FORWARD);
#define QP_FWD(D_, LIN_)                                                                                           \
  hipLaunchKernelGGL((qkv_prepare_fwd_kernel<D_, LIN_>), dim3(grid_for(ctx, rows, QP_THREADS / (D_ / 8))),             \
                     dim3(QP_THREADS), 0, ctx->stream, static_cast<const LIN_*>(qkv_lin),                              \
                     static_cast<unsigned short*>(qkv_out), static_cast<const float*>(q_weight),                       \
                     static_cast<const float*>(k_weight), static_cast<const float*>(cos), static_cast<const float*>(sin), \
                     static_cast<const LIN_*>(value0), static_cast<const float*>(lambda), s, ctx->fault, tag)
  if (lin_dtype == OMX_BF16) {
    if (head_dim == 64) QP_FWD(64, unsigned short);
    else QP_FWD(128, unsigned short);
  } else {
    if (head_dim == 64) QP_FWD(64, float);
    else QP_FWD(128, float);
  }
#undef QP_FWD
  OMX_LAUNCH_CHECK(ctx, "qkv_prepare_fwd_kernel");
  return OMX_OK;
}

int32_t omx_qkv_prepare_backward(omx_ctx* ctx, const void* qkv_lin, int32_t lin_dtype, const void* g_qkv, void* g_qkv_lin, uint64_t pitch,
                                 const void* q_weight, const void* k_weight, const void* cos, const void* sin,
                                 const void* value0, const void* lambda, void* value0_grad_f32, int32_t value0_grad_first,
                                 const void* add_value_grad_f32, void* g_q_weight, void* g_k_weight, void* g_lambda,
                                 uint64_t tokens, uint64_t time, uint64_t heads, uint64_t kv_heads, uint64_t head_dim,
                                 float eps) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "qkv_prepare_backward";
  if (!omx_valid_float_dtype(lin_dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: the projection output must be f32 or bf16", op);
  int32_t rc = check(ctx, op, pitch, tokens, time, heads, kv_heads, head_dim, eps,
                     {qkv_lin, g_qkv, g_qkv_lin, q_weight, k_weight, cos, sin, g_q_weight, g_k_weight});
  if (rc != OMX_OK) return rc;
  if (value0 && (!lambda || !value0_grad_f32 || !g_lambda))
    return omx_fail(ctx, OMX_PLACEMENT, "%s: a blend needs lambda, the value0 gradient and the lambda gradient", op);
  if (value0 && add_value_grad_f32) return omx_fail(ctx, OMX_SHAPE, "%s: add_value_grad is for the block without a blend", op);
  for (const void* p : {value0, static_cast<const void*>(value0_grad_f32), add_value_grad_f32})
    if (p && (reinterpret_cast<uintptr_t>(p) & 15u)) return omx_fail(ctx, OMX_SHAPE, "%s: pointers must be 16-byte aligned", op);
  QkvShape s{static_cast<long>(tokens), static_cast<long>(pitch), static_cast<long>(time), static_cast<int>(heads),
             static_cast<int>(kv_heads), static_cast<int>(head_dim), eps};
  const uint64_t rows = tokens * (heads + 2 * kv_heads);
  const int rows_per_block = QP_THREADS / static_cast<int>(head_dim / 8);
  // At most 1024 workgroups, so the partial sums stay short.
  unsigned blocks = grid_for(ctx, rows, rows_per_block);
  if (blocks > 1024) blocks = 1024;
  void* ws = nullptr;
  const uint64_t partial_w_floats = static_cast<uint64_t>(blocks) * 2 * head_dim;
  rc = omx_workspace(ctx, (partial_w_floats + (1 + OMX_COLUMN_SUM_GROUPS) * 2 * head_dim + blocks + 64) * sizeof(float), &ws);
  if (rc != OMX_OK) return rc;
  float* partial_w = static_cast<float*>(ws);
  float* summed = partial_w + partial_w_floats;  // [2][D]
  float* stage = summed + 2 * head_dim;          // the column sum's first stage
  float* partial_lambda = stage + OMX_COLUMN_SUM_GROUPS * 2 * head_dim;
  const unsigned long long tag = omx_tag(ctx, F_RMS_BACKWARD);
#define QP_BWD(D_, LIN_)                                                                                               \
  hipLaunchKernelGGL((qkv_prepare_bwd_kernel<D_, LIN_>), dim3(blocks), dim3(QP_THREADS), 0, ctx->stream,               \
                     static_cast<const LIN_*>(qkv_lin), static_cast<const unsigned short*>(g_qkv),                     \
                     static_cast<unsigned short*>(g_qkv_lin), static_cast<const float*>(q_weight),                     \
                     static_cast<const float*>(k_weight), static_cast<const float*>(cos), static_cast<const float*>(sin), \
                     static_cast<const LIN_*>(value0), static_cast<const float*>(lambda),                              \
                     static_cast<float*>(value0_grad_f32), value0_grad_first, static_cast<const float*>(add_value_grad_f32), \
                     partial_w, partial_lambda, s, ctx->fault, tag)
  if (lin_dtype == OMX_BF16) {
    if (head_dim == 64) QP_BWD(64, unsigned short);
    else QP_BWD(128, unsigned short);
  } else {
    if (head_dim == 64) QP_BWD(64, float);
    else QP_BWD(128, float);
  }
#undef QP_BWD
  OMX_LAUNCH_CHECK(ctx, "qkv_prepare_bwd_kernel");
  // partial_w is [blocks][2 D]: one column sum gives both weights' gradients side by side.
  rc = omx_column_sum(ctx, partial_w, summed, blocks, 2 * head_dim, tag, stage);
  if (rc != OMX_OK) return rc;
  rc = omx_copy(ctx, g_q_weight, summed, head_dim * sizeof(float));
  if (rc != OMX_OK) return rc;
  rc = omx_copy(ctx, g_k_weight, summed + head_dim, head_dim * sizeof(float));
  if (rc != OMX_OK) return rc;
  if (value0) {
    hipLaunchKernelGGL(qkv_lambda_kernel, dim3(1), dim3(256), 0, ctx->stream, partial_lambda, static_cast<int>(blocks),
                       static_cast<const float*>(lambda), static_cast<float*>(g_lambda), ctx->fault, tag);
    OMX_LAUNCH_CHECK(ctx, "qkv_lambda_kernel");
  }
  return OMX_OK;
}

}  // extern "C"
