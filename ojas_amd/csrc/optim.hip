// Optimizer kernels: AdamW, Muon NS5 and gradient clipping.
//
// Reference semantics:
//   adamw_step       ojas-cpu/src/optim.rs:302-395 (Fast f32 element math), two-pass
//                    all-or-nothing :513-621; scalars ojas-core/src/backend.rs:312-477
//   muon_ns5_step    ojas-cpu/src/optim.rs:684-743 (momentum, Nesterov, scale, decay),
//                    :841-985 (Newton-Schulz, f32 and bf16)
//   clip_grad_norm   ojas-cpu/src/backend.rs:770-795, optim.rs:61-160, clip_scale backend.rs:277-303
//
// Each element pass reads and writes every word once with 16-byte accesses.
// An optimizer step is all-or-nothing: a check pass decides on the device,
// and the apply pass writes nothing when any value of the call is non-finite.
#include <cmath>

#include "omx_common.h"

namespace {

constexpr int OPT_THREADS = 256;

struct AdamWords {
  float decay, one_minus_b1, lerp_high, beta2, one_minus_b2, step_size, bc2_sqrt, eps;
  int decays, lerp_low;
};

// ojas-core/src/backend.rs:244-257
double pow_u64(double base, uint64_t exp) {
  double result = 1.0, b = base;
  while (exp > 0) {
    if (exp & 1) result *= b;
    exp >>= 1;
    if (exp > 0) b *= b;
  }
  return result;
}

__device__ __forceinline__ void adam_elem(const AdamWords& a, float p, float g, float m, float v, float* np,
                                          float* nm, float* nv, bool* ok) {
  // torch lerp: below weight 0.5 `m + w (g - m)`, else `g - (g - m)(1 - w)`.
  float m1 = a.lerp_low ? m + a.one_minus_b1 * (g - m) : g - (g - m) * a.lerp_high;
  float v1 = a.beta2 * v + a.one_minus_b2 * g * g;
  float denom = sqrtf(v1) / a.bc2_sqrt + a.eps;
  float delta = (-a.step_size) * m1 / denom;
  float q = p;
  if (a.decays) q *= a.decay;
  q += delta;
  // Without decay a zero step keeps the stored bits (-0.0 + 0.0 would flip a negative zero).
  float new_p = (!a.decays && delta == 0.0f) ? p : q;
  *ok = dev_finite(m1) && dev_finite(v1) && dev_finite(denom) && dev_finite(delta) && dev_finite(new_p);
  *np = new_p;
  *nm = m1;
  *nv = v1;
}

// What `omx_adamw_step_bounded` tracks: every stored value below 2^60 in magnitude (false for NaN).
constexpr float ADAM_BOUND = 1152921504606846976.0f;  // 2^60
__device__ __forceinline__ bool within_bound(float p, float m, float v) {
  return fabsf(p) < ADAM_BOUND && fabsf(m) < ADAM_BOUND && fabsf(v) < ADAM_BOUND;
}

__global__ __launch_bounds__(OPT_THREADS) void adamw_check_kernel(const float* __restrict__ p,
                                                                  const float* __restrict__ g,
                                                                  const float* __restrict__ m,
                                                                  const float* __restrict__ v, size_t n, AdamWords a,
                                                                  unsigned int* __restrict__ refuse,
                                                                  unsigned int* __restrict__ unbounded,
                                                                  OmxFaultWord* fault, unsigned long long tag) {
  bool bad = false, big = false;
  size_t stride = static_cast<size_t>(gridDim.x) * OPT_THREADS;
  for (size_t i = static_cast<size_t>(blockIdx.x) * OPT_THREADS + threadIdx.x; i < n; i += stride) {
    float np, nm, nv;
    bool ok;
    const float pi = p[i], mi = m[i], vi = v[i];
    adam_elem(a, pi, g[i], mi, vi, &np, &nm, &nv, &ok);
    bad |= !ok;
    big |= !within_bound(pi, mi, vi);
  }
  if (bad) {
    atomicOr(refuse, 1u);
    dev_raise_fault(fault, tag);
  }
  if (big && unbounded) atomicOr(unbounded, 1u);
}

__global__ __launch_bounds__(OPT_THREADS) void adamw_apply_kernel(float* __restrict__ p, const float* __restrict__ g,
                                                                  float* __restrict__ m, float* __restrict__ v,
                                                                  size_t n, AdamWords a,
                                                                  const unsigned int* __restrict__ refuse,
                                                                  unsigned int* __restrict__ unbounded,
                                                                  unsigned short* __restrict__ p_bf16) {
  if (refuse && *refuse) return;
  bool big = false;
  size_t stride = static_cast<size_t>(gridDim.x) * OPT_THREADS;
  for (size_t i = static_cast<size_t>(blockIdx.x) * OPT_THREADS + threadIdx.x; i < n; i += stride) {
    float np, nm, nv;
    bool ok;
    adam_elem(a, p[i], g[i], m[i], v[i], &np, &nm, &nv, &ok);
    p[i] = np;
    m[i] = nm;
    v[i] = nv;
    if (p_bf16) p_bf16[i] = dev_f32_to_bf16_bits(np);
    big |= !within_bound(np, nm, nv);
  }
  if (big && unbounded) atomicOr(unbounded, 1u);
}

// The same update on four consecutive elements per thread (16-byte accesses); every pointer
// 16-byte aligned (the bf16 copy 8-byte). The last n % 4 elements are thread 0's.
__global__ __launch_bounds__(OPT_THREADS) void adamw_apply_vec_kernel(float* __restrict__ p,
                                                                      const float* __restrict__ g,
                                                                      float* __restrict__ m, float* __restrict__ v,
                                                                      size_t n, AdamWords a,
                                                                      const unsigned int* __restrict__ refuse,
                                                                      unsigned int* __restrict__ unbounded,
                                                                      unsigned short* __restrict__ p_bf16) {
  if (refuse && *refuse) return;
  bool big = false;
  const size_t quads = n / 4;
  const size_t stride = static_cast<size_t>(gridDim.x) * OPT_THREADS;
  float4* p4 = reinterpret_cast<float4*>(p);
  const float4* g4 = reinterpret_cast<const float4*>(g);
  float4* m4 = reinterpret_cast<float4*>(m);
  float4* v4 = reinterpret_cast<float4*>(v);
  for (size_t i = static_cast<size_t>(blockIdx.x) * OPT_THREADS + threadIdx.x; i < quads; i += stride) {
    const float4 pq = p4[i], gq = g4[i], mq = m4[i], vq = v4[i];
    const float pi[4] = {pq.x, pq.y, pq.z, pq.w}, gi[4] = {gq.x, gq.y, gq.z, gq.w};
    const float mi[4] = {mq.x, mq.y, mq.z, mq.w}, vi[4] = {vq.x, vq.y, vq.z, vq.w};
    float np[4], nm[4], nv[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      bool ok;
      adam_elem(a, pi[e], gi[e], mi[e], vi[e], &np[e], &nm[e], &nv[e], &ok);
      big |= !within_bound(np[e], nm[e], nv[e]);
    }
    p4[i] = make_float4(np[0], np[1], np[2], np[3]);
    m4[i] = make_float4(nm[0], nm[1], nm[2], nm[3]);
    v4[i] = make_float4(nv[0], nv[1], nv[2], nv[3]);
    if (p_bf16) {
      uint2 q;
      q.x = dev_pack_bf16_pair(np[0], np[1]);
      q.y = dev_pack_bf16_pair(np[2], np[3]);
      reinterpret_cast<uint2*>(p_bf16)[i] = q;
    }
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    for (size_t i = quads * 4; i < n; ++i) {
      float np, nm, nv;
      bool ok;
      adam_elem(a, p[i], g[i], m[i], v[i], &np, &nm, &nv, &ok);
      p[i] = np;
      m[i] = nm;
      v[i] = nv;
      if (p_bf16) p_bf16[i] = dev_f32_to_bf16_bits(np);
      big |= !within_bound(np, nm, nv);
    }
  }
  if (big && unbounded) atomicOr(unbounded, 1u);
}

// Sum of squares in f64, one partial per 64Ki-element block, summed inside a
// block in a fixed order (lane-strided, then a tree), so the norm does not
// depend on scheduling.
constexpr size_t NORM_BLOCK = 1 << 16;
__device__ __forceinline__ double sumsq4(const float4& u) {
  const double a = u.x, b = u.y, c = u.z, d = u.w;
  return (a * a + b * b) + (c * c + d * d);
}
__global__ __launch_bounds__(OPT_THREADS) void sumsq_partial_kernel(const float* __restrict__ x, size_t n,
                                                                    double* __restrict__ partial) {
  __shared__ double red[OPT_THREADS];
  size_t begin = static_cast<size_t>(blockIdx.x) * NORM_BLOCK;
  size_t end = min(n, begin + NORM_BLOCK);
  double acc = 0.0;
  if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    // 16-byte loads, four of them in flight per thread; the tail of the last block one by one.
    const float4* x4 = reinterpret_cast<const float4*>(x);
    const size_t q_begin = begin / 4, q_end = end / 4;  // NORM_BLOCK is a multiple of 4
    double a0 = 0.0, a1 = 0.0, a2 = 0.0, a3 = 0.0;
    size_t i = q_begin + threadIdx.x;
    for (; i + 3 * OPT_THREADS < q_end; i += 4 * OPT_THREADS) {
      const float4 u0 = x4[i], u1 = x4[i + OPT_THREADS], u2 = x4[i + 2 * OPT_THREADS], u3 = x4[i + 3 * OPT_THREADS];
      a0 += sumsq4(u0);
      a1 += sumsq4(u1);
      a2 += sumsq4(u2);
      a3 += sumsq4(u3);
    }
    for (; i < q_end; i += OPT_THREADS) a0 += sumsq4(x4[i]);
    acc = (a0 + a1) + (a2 + a3);
    for (size_t j = q_end * 4 + threadIdx.x; j < end; j += OPT_THREADS) {
      const double v = static_cast<double>(x[j]);
      acc += v * v;
    }
  } else {
    for (size_t i = begin + threadIdx.x; i < end; i += OPT_THREADS) {
      double v = static_cast<double>(x[i]);
      acc += v * v;
    }
  }
  red[threadIdx.x] = acc;
  __syncthreads();
  for (int s = OPT_THREADS / 2; s > 0; s >>= 1) {
    if (threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0) partial[blockIdx.x] = red[0];
}
__global__ __launch_bounds__(1024) void sumsq_final_kernel(const double* __restrict__ partial, size_t count,
                                                           double* __restrict__ out) {
  __shared__ double red[1024];
  double acc = 0.0;
  for (size_t i = threadIdx.x; i < count; i += 1024) acc += partial[i];
  red[threadIdx.x] = acc;
  __syncthreads();
  for (int s = 512; s > 0; s >>= 1) {
    if (threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0) *out = red[0];
}
__global__ void scale_in_place_kernel(float* __restrict__ x, size_t n, float s) {
  size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) x[i] *= s;
}
// The same on a 16-byte aligned array, four elements per thread; the last n % 4 are thread 0's.
__global__ __launch_bounds__(OPT_THREADS) void scale_in_place_vec_kernel(float* __restrict__ x, size_t n, float s) {
  const size_t quads = n / 4;
  const size_t i = static_cast<size_t>(blockIdx.x) * OPT_THREADS + threadIdx.x;
  if (i < quads) {
    float4 v = reinterpret_cast<float4*>(x)[i];
    v.x *= s;
    v.y *= s;
    v.z *= s;
    v.w *= s;
    reinterpret_cast<float4*>(x)[i] = v;
  }
  if (i == 0)
    for (size_t j = quads * 4; j < n; ++j) x[j] *= s;
}

inline unsigned grid_for(uint64_t n, int cu_count) {
  uint64_t blocks = (n + OPT_THREADS * 4 - 1) / (OPT_THREADS * 4);
  uint64_t cap = static_cast<uint64_t>(cu_count > 0 ? cu_count : 256) * 16;
  if (blocks > cap) blocks = cap;
  return static_cast<unsigned>(blocks ? blocks : 1);
}

}  // namespace

// `unbounded` (device u32 or null) collects whether any stored parameter or moment reaches 2^60;
// `inputs_bounded` is the caller's word that none of the four inputs does.
static int32_t adamw_impl(omx_ctx* ctx, const char* op, void* param, const void* grad, void* moment1, void* moment2,
                   uint64_t n, uint64_t step, const omx_adamw_config* c, void* param_bf16, bool inputs_bounded,
                   unsigned int* unbounded) {
  OMX_REQUIRE_CTX(ctx);
  if (!param || !grad || !moment1 || !moment2 || !c) return omx_fail(ctx, OMX_PLACEMENT, "%s: null pointer", op);
  if (n == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  // check_adamw, ojas-core/src/backend.rs:312-352.
  const double scalars[5] = {c->lr, c->beta1, c->beta2, c->eps, c->weight_decay};
  for (double s : scalars)
    if (!std::isfinite(s)) return omx_fail(ctx, OMX_NON_FINITE, "%s", op);
  if (!(c->beta1 >= 0.0 && c->beta1 < 1.0 && c->beta2 >= 0.0 && c->beta2 < 1.0))
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: adamw beta must be in [0, 1)", op);
  if (c->eps <= 0.0) return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: adamw eps must be > 0", op);
  if (c->lr < 0.0) return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: lr %g is negative", op, c->lr);
  if (c->weight_decay < 0.0)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: weight_decay %g is negative", op, c->weight_decay);
  if (step == UINT64_MAX) return omx_fail(ctx, OMX_OUT_OF_RANGE, "next_step: step counter is u64::MAX");
  const uint64_t next = step + 1;
  const double bc1 = 1.0 - pow_u64(c->beta1, next), bc2 = 1.0 - pow_u64(c->beta2, next);
  if (!(std::isfinite(bc1) && std::isfinite(bc2) && bc1 > 0.0 && bc2 > 0.0))
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: adamw bias correction is not a positive finite value", op);
  // AdamWScalars::from_bias_corrections + f32_words, backend.rs:387-477.
  const double one_minus_b1 = 1.0 - c->beta1;
  AdamWords a;
  a.decay = static_cast<float>(1.0 - c->lr * c->weight_decay);
  a.one_minus_b1 = static_cast<float>(one_minus_b1);
  a.lerp_high = 1.0f - a.one_minus_b1;
  a.beta2 = static_cast<float>(c->beta2);
  a.one_minus_b2 = static_cast<float>(1.0 - c->beta2);
  a.step_size = static_cast<float>(c->lr / bc1);
  a.bc2_sqrt = static_cast<float>(std::sqrt(bc2));
  a.eps = static_cast<float>(c->eps);
  a.decays = c->weight_decay != 0.0;
  a.lerp_low = a.one_minus_b1 < 0.5f;
  const float words[7] = {a.decay, a.one_minus_b1, a.beta2, a.one_minus_b2, a.step_size, a.bc2_sqrt, a.eps};
  for (float wd : words)
    if (!std::isfinite(wd)) return omx_fail(ctx, OMX_NON_FINITE, "%s", op);

  // With every input below 2^60 in magnitude no result can be non-finite, provided the scalars
  // are moderate: |m1| < 2^61, v1 < 2^121, denom >= eps, |delta| = step_size |m1| / denom
  // < 2^20 2^61 2^40 = 2^121, |new p| <= 2 |p| + |delta|. The checking pass has nothing to find then.
  const bool moderate = a.step_size <= 0x1p20f && fabsf(a.decay) <= 2.0f && a.eps >= 0x1p-40f && a.bc2_sqrt >= 0x1p-30f;
  const bool skip_check = inputs_bounded && moderate;
  dim3 grid(grid_for(n, ctx->cu_count)), block(OPT_THREADS);
  unsigned int* refuse = nullptr;
  // Parameter, gradient and both moments read, parameter and moments written: 28 bytes per
  // element, and 2 more with the bf16 copy of the parameter.
  OmxKernelTimer timer(ctx, OMX_K_ADAMW, (param_bf16 ? 30.0 : 28.0) * static_cast<double>(n));
  if (!skip_check) {
    void* ws = nullptr;
    int32_t rc = omx_workspace(ctx, 256, &ws);
    if (rc != OMX_OK) return rc;
    refuse = static_cast<unsigned int*>(ws);
    rc = omx_fill_zero(ctx, refuse, 4);
    if (rc != OMX_OK) return rc;
    omx_launch_timed(ctx, adamw_check_kernel, grid, block, 0, timer.start(), nullptr, static_cast<const float*>(param),
                     static_cast<const float*>(grad), static_cast<const float*>(moment1),
                     static_cast<const float*>(moment2), n, a, refuse, unbounded, ctx->fault, omx_tag(ctx, F_ADAMW));
    OMX_LAUNCH_CHECK(ctx, "adamw_check_kernel");
  }
  const uintptr_t bits = reinterpret_cast<uintptr_t>(param) | reinterpret_cast<uintptr_t>(grad) |
                         reinterpret_cast<uintptr_t>(moment1) | reinterpret_cast<uintptr_t>(moment2) |
                         (reinterpret_cast<uintptr_t>(param_bf16) << 1);
  if ((bits & 15) == 0 && n >= 4) {
    dim3 vec_grid(static_cast<unsigned>((n / 4 + OPT_THREADS - 1) / OPT_THREADS));
    omx_launch_timed(ctx, adamw_apply_vec_kernel, vec_grid, block, 0, skip_check ? timer.start() : nullptr,
                     timer.stop(), static_cast<float*>(param), static_cast<const float*>(grad),
                     static_cast<float*>(moment1), static_cast<float*>(moment2), n, a, refuse, unbounded,
                     static_cast<unsigned short*>(param_bf16));
  } else {
    omx_launch_timed(ctx, adamw_apply_kernel, grid, block, 0, skip_check ? timer.start() : nullptr, timer.stop(),
                     static_cast<float*>(param), static_cast<const float*>(grad), static_cast<float*>(moment1),
                     static_cast<float*>(moment2), n, a, refuse, unbounded, static_cast<unsigned short*>(param_bf16));
  }
  OMX_LAUNCH_CHECK(ctx, "adamw_apply_kernel");
  return OMX_OK;
}

extern "C" {

int32_t omx_adamw_step(omx_ctx* ctx, void* param, const void* grad, void* moment1, void* moment2, uint64_t n,
                       uint64_t step, const omx_adamw_config* c, void* param_bf16) {
  return adamw_impl(ctx, "adamw_step", param, grad, moment1, moment2, n, step, c, param_bf16, false, nullptr);
}

int32_t omx_adamw_step_bounded(omx_ctx* ctx, void* param, const void* grad, void* moment1, void* moment2, uint64_t n,
                               uint64_t step, const omx_adamw_config* c, void* param_bf16, int32_t inputs_bounded,
                               void* unbounded_flag) {
  OMX_REQUIRE_CTX(ctx);
  if (!unbounded_flag) return omx_fail(ctx, OMX_PLACEMENT, "adamw_step_bounded: null pointer");
  return adamw_impl(ctx, "adamw_step_bounded", param, grad, moment1, moment2, n, step, c, param_bf16,
                    inputs_bounded != 0 && ctx->adamw_trust != 0, static_cast<unsigned int*>(unbounded_flag));
}

int32_t omx_clip_grad_norm(omx_ctx* ctx, void* const* grads, const uint64_t* lens, uint64_t count, float max_norm,
                           float* norm_out) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "clip_grad_norm";
  if (!grads || !lens || !norm_out) return omx_fail(ctx, OMX_PLACEMENT, "%s: null pointer", op);
  if (count == 0) return omx_fail(ctx, OMX_SHAPE, "%s: no gradients", op);
  uint64_t blocks = 0;
  for (uint64_t t = 0; t < count; ++t) {
    if (!grads[t]) return omx_fail(ctx, OMX_PLACEMENT, "%s: gradient %llu is null", op, (unsigned long long)t);
    if (lens[t] == 0) return omx_fail(ctx, OMX_SHAPE, "%s: gradient %llu is empty", op, (unsigned long long)t);
    blocks += (lens[t] + NORM_BLOCK - 1) / NORM_BLOCK;
  }
  void* ws = nullptr;
  int32_t rc = omx_workspace(ctx, (blocks + 1) * sizeof(double), &ws);
  if (rc != OMX_OK) return rc;
  double* partial = static_cast<double*>(ws);
  double* total = partial + blocks;
  uint64_t at = 0;
  for (uint64_t t = 0; t < count; ++t) {
    uint64_t nb = (lens[t] + NORM_BLOCK - 1) / NORM_BLOCK;
    hipLaunchKernelGGL(sumsq_partial_kernel, dim3(static_cast<unsigned>(nb)), dim3(OPT_THREADS), 0, ctx->stream,
                       static_cast<const float*>(grads[t]), lens[t], partial + at);
    OMX_LAUNCH_CHECK(ctx, "sumsq_partial_kernel");
    at += nb;
  }
  hipLaunchKernelGGL(sumsq_final_kernel, dim3(1), dim3(1024), 0, ctx->stream, partial, blocks, total);
  OMX_LAUNCH_CHECK(ctx, "sumsq_final_kernel");
  // The norm is a host value: this is the step's first sync point, and it
  // also reports any fault raised by the ops that produced the gradients.
  double sum_sq = 0.0;
  rc = omx_download(ctx, &sum_sq, total, 0, sizeof(double));
  if (rc != OMX_OK) return rc;
  float norm = static_cast<float>(std::sqrt(sum_sq));
  if (!std::isfinite(norm)) return omx_fail(ctx, OMX_NON_FINITE, "%s", op);
  // clip_scale, ojas-core/src/backend.rs:277-303.
  if (std::isnan(max_norm) || max_norm == -INFINITY) return omx_fail(ctx, OMX_NON_FINITE, "%s", op);
  if (max_norm < 0.0f) return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: max_norm %g is negative", op, max_norm);
  float coef = max_norm / (norm + 1e-6f);
  if (std::isnan(coef)) return omx_fail(ctx, OMX_NON_FINITE, "%s", op);
  if (coef > 1.0f) coef = 1.0f;
  if (coef < 1.0f) {
    for (uint64_t t = 0; t < count; ++t) {
      if ((reinterpret_cast<uintptr_t>(grads[t]) & 15u) == 0 && lens[t] >= 4 && lens[t] / 4 / OPT_THREADS < 0x7fffffffull)
        hipLaunchKernelGGL(scale_in_place_vec_kernel,
                           dim3(static_cast<unsigned>((lens[t] / 4 + OPT_THREADS - 1) / OPT_THREADS)), dim3(OPT_THREADS),
                           0, ctx->stream, static_cast<float*>(grads[t]), lens[t], coef);
      else
        hipLaunchKernelGGL(scale_in_place_kernel, dim3(grid_for(lens[t], ctx->cu_count)), dim3(OPT_THREADS), 0,
                           ctx->stream, static_cast<float*>(grads[t]), lens[t], coef);
      OMX_LAUNCH_CHECK(ctx, "scale_in_place_kernel");
    }
  }
  *norm_out = norm;
  return OMX_OK;
}

}  // extern "C"
