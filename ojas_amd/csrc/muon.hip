// Muon NS5 step: BackendModule::muon_ns5_step (ojas-core/src/backend.rs:2480-2491,
// config :548-570). CPU reference: ojas-cpu/src/optim.rs:684-743 (momentum,
// Nesterov blend, scale, decay, update) and :841-985 (Newton-Schulz).
//
//   buf = mom * m + g;  u = nesterov ? fma(mom, buf, g) : buf
//   X = u / (||u||_F + 1e-7)        (norm from an f64 sum of squares; read as the
//                                    short-side-first matrix, a stride choice here)
//   5 x { A = X X^T;  B = b A + c A A;  X = a X + B X }   (a,b,c) = (3.4445, -4.7750, 2.0315)
//   p = fma(-lr * sqrt(max(1, rows/cols)), X, p * (1 - lr * wd));  m = buf
//
// In bf16 mode X, the norm, the sum with the epsilon, the quotient, every GEMM
// output and every scalar multiple and sum are rounded to bf16 (optim.rs:947-971);
// the iterate then lives in bf16 storage and the three products run on the
// bf16 MFMA lane, whose bf16 output store is exactly that rounding.
//
// The step is all-or-nothing: a refuse flag raised by any non-finite
// intermediate keeps the final pass from writing the parameter or the momentum.
#include <algorithm>
#include <cmath>

#include "omx_common.h"

namespace {

constexpr int MU_THREADS = 256;
constexpr size_t MU_BLOCK = 1 << 11;  // elements per sum-of-squares partial (8 per thread: a 768 x 768 matrix fills the chip)

struct MuonScalars {
  float mom, alpha, decay, a, b, c;
  int nesterov, decays, bf16;
};

inline unsigned mu_grid(uint64_t n) {
  uint64_t blocks = (n + MU_THREADS * 4 - 1) / (MU_THREADS * 4);
  if (blocks > 4096) blocks = 4096;
  return static_cast<unsigned>(blocks ? blocks : 1);
}

// One launch serves up to MU_MAX_BATCH matrices of one shape: block (x, y) works on matrix y. The
// tensors the caller owns come as pointer tables in the kernel arguments; the intermediates of
// matrix y live `stride` bytes after matrix y - 1's in the workspace, at the offsets of MuonLayout.
constexpr int MU_MAX_BATCH = 64;
struct MuonTensors {
  float* p[MU_MAX_BATCH];
  const float* g[MU_MAX_BATCH];
  float* m[MU_MAX_BATCH];
  unsigned short* p16[MU_MAX_BATCH];  // entries may be null
};
struct MuonLayout {
  uint64_t buf, u, x, xn, a, a2, partial, scalars, total;
};
struct MuonWork {
  char* ws;
  uint64_t stride;  // bytes between consecutive matrices' blocks
  MuonLayout L;
  unsigned int* refuse;  // one flag for the whole launch
  template <typename T>
  __device__ __forceinline__ T* at(uint64_t offset) const {
    return reinterpret_cast<T*>(ws + blockIdx.y * stride + offset);
  }
};

// buf, the (possibly bf16-rounded) update u, and per-block f64 sums of u^2.
__global__ __launch_bounds__(MU_THREADS) void muon_momentum_kernel(MuonTensors t, MuonWork w, size_t n, MuonScalars s,
                                                                   OmxFaultWord* fault, unsigned long long tag) {
  __shared__ double red[MU_THREADS];
  const float* __restrict__ g = t.g[blockIdx.y];
  const float* __restrict__ m = t.m[blockIdx.y];
  float* __restrict__ buf = w.at<float>(w.L.buf);
  float* __restrict__ u = w.at<float>(w.L.u);
  double* __restrict__ partial = w.at<double>(w.L.partial);
  const size_t begin = static_cast<size_t>(blockIdx.x) * MU_BLOCK, end = min(n, begin + MU_BLOCK);
  double acc = 0.0;
  bool bad = false;
  for (size_t i = begin + threadIdx.x; i < end; i += MU_THREADS) {
    float gi = g[i];
    float b = s.mom * m[i] + gi;
    bad |= !(dev_finite(b) && dev_finite(gi));
    float upd = s.nesterov ? fmaf(s.mom, b, gi) : b;
    if (s.bf16) upd = dev_round_bf16(upd);
    buf[i] = b;
    u[i] = upd;
    acc += static_cast<double>(upd) * static_cast<double>(upd);
  }
  red[threadIdx.x] = acc;
  __syncthreads();
  for (int st = MU_THREADS / 2; st > 0; st >>= 1) {
    if (threadIdx.x < st) red[threadIdx.x] += red[threadIdx.x + st];
    __syncthreads();
  }
  if (threadIdx.x == 0) partial[blockIdx.x] = red[0];
  if (bad) {
    atomicOr(w.refuse, 1u);
    dev_raise_fault(fault, tag);
  }
}

// One block per matrix (blockIdx.y): the norm and the quotient's denominator.
__global__ __launch_bounds__(1024) void muon_norm_kernel(MuonWork w, size_t count, int bf16, OmxFaultWord* fault,
                                                         unsigned long long tag) {
  __shared__ double red[1024];
  const double* __restrict__ partial = w.at<double>(w.L.partial);
  double acc = 0.0;
  for (size_t i = threadIdx.x; i < count; i += 1024) acc += partial[i];
  red[threadIdx.x] = acc;
  __syncthreads();
  for (int st = 512; st > 0; st >>= 1) {
    if (threadIdx.x < st) red[threadIdx.x] += red[threadIdx.x + st];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    float norm = static_cast<float>(sqrt(red[0]));
    const float eps = 1e-7f;
    float denom = bf16 ? dev_round_bf16(dev_round_bf16(norm) + eps) : norm + eps;
    *w.at<float>(w.L.scalars + 16) = denom;
    if (!(dev_finite(denom) && denom != 0.0f)) {
      atomicOr(w.refuse, 1u);
      dev_raise_fault(fault, tag);
    }
  }
}

template <typename TX>
__global__ void muon_normalize_kernel(MuonWork w, uint64_t x_off, size_t n) {
  const float* __restrict__ u = w.at<float>(w.L.u);
  TX* __restrict__ x = w.at<TX>(x_off);
  const float d = *w.at<float>(w.L.scalars + 16);
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * blockDim.x)
    dev_store<TX>(x, i, u[i] / d);  // bf16 storage rounds the quotient
}

// B = b A + c A2 (in place over A2), with the bf16 roundings of optim.rs:913-921.
template <typename TX>
__global__ void muon_combine_b_kernel(MuonWork w, size_t n, MuonScalars s) {
  const TX* __restrict__ am = w.at<TX>(w.L.a);
  TX* __restrict__ a2 = w.at<TX>(w.L.a2);
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    float av = dev_load<TX>(am, i), a2v = dev_load<TX>(a2, i);
    float r;
    if (s.bf16) r = dev_round_bf16(s.b * av) + dev_round_bf16(s.c * a2v);
    else r = s.b * av + s.c * a2v;
    dev_store<TX>(a2, i, r);
  }
}

// X_next = a X + BX (in place over BX), finite-checked (optim.rs:950-962).
template <typename TX>
__global__ void muon_combine_x_kernel(MuonWork w, uint64_t x_off, uint64_t bx_off, size_t n, MuonScalars s,
                                      OmxFaultWord* fault, unsigned long long tag) {
  const TX* __restrict__ x = w.at<TX>(x_off);
  TX* __restrict__ bx = w.at<TX>(bx_off);
  bool bad = false;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    float xv = dev_load<TX>(x, i), bxv = dev_load<TX>(bx, i);
    float r = s.bf16 ? dev_round_bf16(s.a * xv) + bxv : s.a * xv + bxv;
    if (s.bf16) r = dev_round_bf16(r);
    bad |= !dev_finite(r);
    dev_store<TX>(bx, i, r);
  }
  if (bad) {
    atomicOr(w.refuse, 1u);
    dev_raise_fault(fault, tag);
  }
}

template <typename TX>
__global__ void muon_check_update_kernel(MuonTensors t, MuonWork w, uint64_t x_off, size_t n, MuonScalars s,
                                         OmxFaultWord* fault, unsigned long long tag) {
  const float* __restrict__ p = t.p[blockIdx.y];
  const TX* __restrict__ x = w.at<TX>(x_off);
  bool bad = false;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    float base = s.decays ? p[i] * s.decay : p[i];
    bad |= !dev_finite(fmaf(s.alpha, dev_load<TX>(x, i), base));
  }
  if (bad) {
    atomicOr(w.refuse, 1u);
    dev_raise_fault(fault, tag);
  }
}

template <typename TX>
__global__ void muon_apply_kernel(MuonTensors t, MuonWork w, uint64_t x_off, size_t n, MuonScalars s) {
  if (*w.refuse) return;
  float* __restrict__ p = t.p[blockIdx.y];
  float* __restrict__ m = t.m[blockIdx.y];
  unsigned short* __restrict__ p_bf16 = t.p16[blockIdx.y];
  const float* __restrict__ buf = w.at<float>(w.L.buf);
  const TX* __restrict__ x = w.at<TX>(x_off);
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    float base = s.decays ? p[i] * s.decay : p[i];
    float np = fmaf(s.alpha, dev_load<TX>(x, i), base);
    p[i] = np;
    m[i] = buf[i];
    if (p_bf16) p_bf16[i] = dev_f32_to_bf16_bits(np);
  }
}

MuonLayout muon_layout(uint64_t rows, uint64_t cols) {
  auto up = [](uint64_t v) { return (v + 255) & ~255ull; };
  const uint64_t len = rows * cols, r = rows < cols ? rows : cols;
  MuonLayout L;
  uint64_t at = 0;
  L.buf = at;
  at += up(len * 4);
  L.u = at;
  at += up(len * 4);
  L.x = at;
  at += up(len * 4);
  L.xn = at;
  at += up(len * 4);
  L.a = at;
  at += up(r * r * 4);
  L.a2 = at;
  at += up(r * r * 4);
  L.partial = at;
  at += up(((len + MU_BLOCK - 1) / MU_BLOCK) * 8);
  L.scalars = at;
  at += 256;
  L.total = at;
  return L;
}

// `count` (<= MU_MAX_BATCH) matrices of one shape; ws holds count blocks of L.total bytes.
template <typename TX>
int32_t run_muon(omx_ctx* ctx, const MuonTensors& t, unsigned count, uint64_t rows, uint64_t cols, MuonScalars s,
                 char* ws, const MuonLayout& L, unsigned long long tag) {
  const uint64_t len = rows * cols;
  const int32_t XD = sizeof(TX) == 2 ? OMX_BF16 : OMX_F32;
  MuonWork w;
  w.ws = ws;
  w.stride = L.total;
  w.L = L;
  w.refuse = reinterpret_cast<unsigned int*>(ws + L.scalars);
  int32_t rc = omx_fill_zero(ctx, w.refuse, 4);
  if (rc != OMX_OK) return rc;
  uint64_t x_off = L.x, xn_off = L.xn;
  const unsigned nb = static_cast<unsigned>((len + MU_BLOCK - 1) / MU_BLOCK);
  const dim3 block(MU_THREADS), over_len(mu_grid(len), count);
  hipLaunchKernelGGL(muon_momentum_kernel, dim3(nb, count), block, 0, ctx->stream, t, w, len, s, ctx->fault, tag);
  hipLaunchKernelGGL(muon_norm_kernel, dim3(1, count), dim3(1024), 0, ctx->stream, w, static_cast<size_t>(nb), s.bf16,
                     ctx->fault, tag);
  hipLaunchKernelGGL((muon_normalize_kernel<TX>), over_len, block, 0, ctx->stream, w, x_off, len);
  OMX_LAUNCH_CHECK(ctx, "muon prologue");
  const bool tall = rows > cols;
  const uint64_t r = tall ? cols : rows, c = tall ? rows : cols;
  const uint64_t es = L.total / sizeof(TX);  // elements between consecutive matrices' buffers
  const OmxGemmBatch batch{count, es, es, es};
  const OmxGemmBatch* bp = count > 1 ? &batch : nullptr;
  TX* am = reinterpret_cast<TX*>(ws + L.a);
  TX* a2 = reinterpret_cast<TX*>(ws + L.a2);
  // bf16 tier: the two-term sums after the second and third product ride in those products' store
  // passes (the same roundings in the same order as the combine kernels below; a non-finite value
  // raises the fault there and reaches the final check through the remaining products). Strided
  // batches only: a single product may split its reduction, which a store-pass sum cannot follow.
  const bool fused = sizeof(TX) == 2 && s.bf16 && ctx->muon_fused_sums && count > 1;
  for (int it = 0; it < 5; ++it) {
    TX* x = reinterpret_cast<TX*>(ws + x_off);
    TX* xn = reinterpret_cast<TX*>(ws + xn_off);
    // A = X' X'^T with X' the short-side-first reading of X.
    if (!tall) rc = omx_gemm_impl(ctx, F_MUON, x, cols, 1, x, 1, cols, XD, am, XD, r, r, c, r, 0, nullptr, bp);
    else rc = omx_gemm_impl(ctx, F_MUON, x, 1, cols, x, cols, 1, XD, am, XD, r, r, c, r, 0, nullptr, bp);
    if (rc != OMX_OK) return rc;
    // B = b A + c A^2
    const OmxGemmEpilogue sum_b{OMX_EPI_AXPBY, 0, am, nullptr, s.b, s.c};
    rc = omx_gemm_impl(ctx, F_MUON, am, r, 1, am, r, 1, XD, a2, XD, r, r, r, r, 0, fused ? &sum_b : nullptr, bp);
    if (rc != OMX_OK) return rc;
    if (!fused)
      hipLaunchKernelGGL((muon_combine_b_kernel<TX>), dim3(mu_grid(r * r), count), block, 0, ctx->stream, w,
                         static_cast<size_t>(r * r), s);
    // X_next = a X + B X, with BX in X's own physical layout: B X' when wide, X B^T when tall.
    const OmxGemmEpilogue sum_x{OMX_EPI_AXPBY, 0, x, nullptr, s.a, 1.0f};
    const OmxGemmEpilogue* ex = fused ? &sum_x : nullptr;
    if (!tall) rc = omx_gemm_impl(ctx, F_MUON, a2, r, 1, x, cols, 1, XD, xn, XD, cols, r, r, c, 0, ex, bp);
    else rc = omx_gemm_impl(ctx, F_MUON, x, cols, 1, a2, 1, r, XD, xn, XD, cols, rows, cols, cols, 0, ex, bp);
    if (rc != OMX_OK) return rc;
    if (!fused)
      hipLaunchKernelGGL((muon_combine_x_kernel<TX>), over_len, block, 0, ctx->stream, w, x_off, xn_off, len, s,
                         ctx->fault, tag);
    OMX_LAUNCH_CHECK(ctx, "muon newton-schulz step");
    std::swap(x_off, xn_off);
  }
  hipLaunchKernelGGL((muon_check_update_kernel<TX>), over_len, block, 0, ctx->stream, t, w, x_off, len, s, ctx->fault,
                     tag);
  hipLaunchKernelGGL((muon_apply_kernel<TX>), over_len, block, 0, ctx->stream, t, w, x_off, len, s);
  OMX_LAUNCH_CHECK(ctx, "muon apply");
  return OMX_OK;
}

// check_muon (ojas-cpu/src/optim.rs:664-681) and the step's scalars.
int32_t muon_scalars(omx_ctx* ctx, const char* op, const omx_muon_config* c, uint64_t rows, uint64_t cols,
                     MuonScalars* out) {
  if (rows == 0 || cols == 0) return omx_fail(ctx, OMX_SHAPE, "%s: empty tensor", op);
  if (rows > 0x7fffffffull || cols > 0x7fffffffull) return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: axis too large", op);
  if (!std::isfinite(c->lr) || !std::isfinite(c->momentum) || !std::isfinite(c->weight_decay))
    return omx_fail(ctx, OMX_NON_FINITE, "%s", op);
  if (c->lr < 0.0) return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: lr %g is negative", op, c->lr);
  if (c->momentum < 0.0) return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: momentum %g is negative", op, c->momentum);
  if (c->weight_decay < 0.0)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: weight_decay %g is negative", op, c->weight_decay);
  MuonScalars s;
  s.mom = static_cast<float>(c->momentum);
  const double ratio = static_cast<double>(rows) / static_cast<double>(cols);
  s.alpha = static_cast<float>(-c->lr * std::sqrt(ratio > 1.0 ? ratio : 1.0));
  s.decay = static_cast<float>(1.0 - c->lr * c->weight_decay);
  s.a = static_cast<float>(3.4445);
  s.b = static_cast<float>(-4.7750);
  s.c = static_cast<float>(2.0315);
  s.nesterov = c->nesterov != 0;
  s.decays = c->weight_decay != 0.0;
  s.bf16 = c->ns5_bf16 != 0;
  *out = s;
  return OMX_OK;
}

int32_t muon_batch(omx_ctx* ctx, const char* op, void* const* params, const void* const* grads, void* const* momenta,
                   void* const* params_bf16, uint64_t count, uint64_t rows, uint64_t cols, const omx_muon_config* c) {
  MuonScalars s;
  int32_t rc = muon_scalars(ctx, op, c, rows, cols, &s);
  if (rc != OMX_OK) return rc;
  for (uint64_t i = 0; i < count; ++i)
    if (!params[i] || !grads[i] || !momenta[i]) return omx_fail(ctx, OMX_PLACEMENT, "%s: null pointer", op);
  const MuonLayout L = muon_layout(rows, cols);
  for (uint64_t first = 0; first < count; first += MU_MAX_BATCH) {
    const unsigned n = static_cast<unsigned>(std::min<uint64_t>(MU_MAX_BATCH, count - first));
    void* ws = nullptr;
    rc = omx_workspace(ctx, L.total * n, &ws);
    if (rc != OMX_OK) return rc;
    MuonTensors t{};
    for (unsigned i = 0; i < n; ++i) {
      t.p[i] = static_cast<float*>(params[first + i]);
      t.g[i] = static_cast<const float*>(grads[first + i]);
      t.m[i] = static_cast<float*>(momenta[first + i]);
      t.p16[i] = params_bf16 ? static_cast<unsigned short*>(params_bf16[first + i]) : nullptr;
    }
    const unsigned long long tag = omx_tag(ctx, F_MUON);
    rc = s.bf16 ? run_muon<unsigned short>(ctx, t, n, rows, cols, s, static_cast<char*>(ws), L, tag)
                : run_muon<float>(ctx, t, n, rows, cols, s, static_cast<char*>(ws), L, tag);
    if (rc != OMX_OK) return rc;
  }
  return OMX_OK;
}

}  // namespace

extern "C" {

uint64_t omx_muon_scratch_bytes(uint64_t rows, uint64_t cols) {
  if (rows == 0 || cols == 0) return 0;
  return muon_layout(rows, cols).total;
}

int32_t omx_muon_ns5_step(omx_ctx* ctx, void* param, const void* grad, void* momentum, uint64_t rows, uint64_t cols,
                          const omx_muon_config* c, void* param_bf16) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "muon_ns5_step";
  if (!param || !grad || !momentum || !c) return omx_fail(ctx, OMX_PLACEMENT, "%s: null pointer", op);
  void* mirrors[1] = {param_bf16};
  const void* grads[1] = {grad};
  return muon_batch(ctx, op, &param, grads, &momentum, param_bf16 ? mirrors : nullptr, 1, rows, cols, c);
}

int32_t omx_muon_ns5_step_batched(omx_ctx* ctx, void* const* params, const void* const* grads, void* const* momenta,
                                  void* const* params_bf16, uint64_t count, uint64_t rows, uint64_t cols,
                                  const omx_muon_config* c) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "muon_ns5_step";
  if (!params || !grads || !momenta || !c) return omx_fail(ctx, OMX_PLACEMENT, "%s: null pointer", op);
  if (count == 0) return omx_fail(ctx, OMX_SHAPE, "%s: no tensors", op);
  return muon_batch(ctx, op, params, grads, momenta, params_bf16, count, rows, cols, c);
}

}  // extern "C"
