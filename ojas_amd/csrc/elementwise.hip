// Elementwise, cast and layout kernels: one coalesced pass over HBM each.
//
// BackendCore::{cast_bf16,to_bf16,to_f32} (ojas-core/src/backend.rs:975-1090,
// rounding rule autocast.rs:66-101), BackendFloat::{residual_add_forward,
// accumulate_grad, scale_grad, gelu_erf_*, gelu_tanh_*, permute}
// (backend.rs:1115-1220,1473-1510; CPU reference ojas-cpu/src/accum.rs:31-106,
// pointwise.rs:1052, layout.rs:82-118, ojas-core/src/erf_exact.rs:29-110,
// gelu_tanh.rs:27-68).
#include "omx_common.h"

namespace {

constexpr int EW_THREADS = 256;
constexpr int EW_PER_THREAD = 8;

inline dim3 ew_grid(uint64_t n) {
  uint64_t per_block = static_cast<uint64_t>(EW_THREADS) * EW_PER_THREAD;
  uint64_t blocks = (n + per_block - 1) / per_block;
  return dim3(static_cast<unsigned>(blocks > 0 ? blocks : 1));
}

// Block b owns elements [b*2048, (b+1)*2048); thread t touches t, t+256, ...
// so a wave's accesses are contiguous.
#define EW_LOOP(i, n)                                                                      \
  for (size_t i = static_cast<size_t>(blockIdx.x) * (EW_THREADS * EW_PER_THREAD) + threadIdx.x, \
              end_ = min(static_cast<size_t>(n), (static_cast<size_t>(blockIdx.x) + 1) * (EW_THREADS * EW_PER_THREAD)); \
       i < end_; i += EW_THREADS)

template <typename S, typename D>
__global__ void convert_kernel(const S* __restrict__ x, D* __restrict__ y, size_t n) {
  EW_LOOP(i, n) dev_store<D>(y, i, dev_load<S>(x, i));
}
__global__ void round_bf16_kernel(const float* __restrict__ x, float* __restrict__ y, size_t n) {
  EW_LOOP(i, n) y[i] = dev_round_bf16(x[i]);
}
__global__ void fill_zero_kernel(unsigned int* __restrict__ p, size_t words, unsigned char* tail, int tail_bytes) {
  EW_LOOP(i, words) p[i] = 0u;
  if (blockIdx.x == 0 && threadIdx.x < tail_bytes) tail[threadIdx.x] = 0;
}

template <typename TX, typename TY, typename TO>
__global__ void add_kernel(const TX* __restrict__ x, const TY* __restrict__ y, TO* __restrict__ out, size_t n,
                           OmxFaultWord* fault, unsigned long long tag) {
  bool bad = false;
  EW_LOOP(i, n) {
    float v = dev_load<TX>(x, i) + dev_load<TY>(y, i);
    bad |= !dev_finite(v);
    dev_store<TO>(out, i, v);
  }
  if (bad) dev_raise_fault(fault, tag);
}

__global__ void accumulate_kernel(float* __restrict__ acc, const float* __restrict__ g, size_t n, OmxFaultWord* fault,
                                  unsigned long long tag) {
  bool bad = false;
  EW_LOOP(i, n) {
    float v = acc[i] + g[i];
    bad |= !dev_finite(v);
    acc[i] = v;
  }
  if (bad) dev_raise_fault(fault, tag);
}
__global__ void scale_kernel(float* __restrict__ g, float s, size_t n, OmxFaultWord* fault, unsigned long long tag) {
  bool bad = false;
  EW_LOOP(i, n) {
    float v = g[i] * s;
    bad |= !dev_finite(v);
    g[i] = v;
  }
  if (bad) dev_raise_fault(fault, tag);
}

template <typename T, bool TANH>
__global__ void gelu_fwd_kernel(const T* __restrict__ x, T* __restrict__ y, size_t n, OmxFaultWord* fault,
                                unsigned long long tag) {
  bool bad = false;
  EW_LOOP(i, n) {
    float v = dev_load<T>(x, i);
    float r = dev_gelu_of<T, TANH>(v);
    bad |= !dev_finite(r);
    dev_store<T>(y, i, r);
  }
  if (bad) dev_raise_fault(fault, tag);
}
template <typename T, bool TANH>
__global__ void gelu_bwd_kernel(const T* __restrict__ x, const T* __restrict__ gy, T* __restrict__ gx, size_t n,
                                OmxFaultWord* fault, unsigned long long tag) {
  bool bad = false;
  EW_LOOP(i, n) {
    float v = dev_load<T>(x, i);
    float r = dev_load<T>(gy, i) * dev_gelu_grad_of<T, TANH>(v);
    bad |= !dev_finite(r);
    dev_store<T>(gx, i, r);
  }
  if (bad) dev_raise_fault(fault, tag);
}

// [d0,d1,d2,d3] -> [d0,d2,d1,d3]; one thread moves `VEC` contiguous elements
// of the innermost axis, so both sides are coalesced along d3.
template <typename V>
__global__ void permute_0213_kernel(const V* __restrict__ x, V* __restrict__ y, size_t d0, size_t d1, size_t d2,
                                    size_t d3v) {
  size_t total = d0 * d1 * d2 * d3v;
  EW_LOOP(i, total) {
    size_t c = i % d3v, r = i / d3v;
    size_t k = r % d1;  // output is [d0][d2][d1][d3v]
    r /= d1;
    size_t j = r % d2, a = r / d2;
    y[i] = x[((a * d1 + k) * d2 + j) * d3v + c];
  }
}

// x[b, t] = tokens[starts[b] + t], y[b, t] = tokens[starts[b] + t + 1], widened to u32.
template <typename TOK>
__global__ void token_windows_kernel(const TOK* __restrict__ tokens, const unsigned long long* __restrict__ starts,
                                     unsigned int* __restrict__ x, unsigned int* __restrict__ y, size_t batch,
                                     size_t seq_len) {
  const size_t n = batch * seq_len;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t b = i / seq_len, t = i - b * seq_len;
    const TOK* w = tokens + starts[b] + t;
    x[i] = w[0];
    y[i] = w[1];
  }
}

}  // namespace

int32_t omx_convert(omx_ctx* ctx, const void* src, int32_t src_dtype, void* dst, int32_t dst_dtype, uint64_t n) {
  if (n == 0) return OMX_OK;
  dim3 grid = ew_grid(n), block(EW_THREADS);
  if (src_dtype == OMX_F32 && dst_dtype == OMX_BF16)
    hipLaunchKernelGGL((convert_kernel<float, unsigned short>), grid, block, 0, ctx->stream,
                       static_cast<const float*>(src), static_cast<unsigned short*>(dst), n);
  else if (src_dtype == OMX_BF16 && dst_dtype == OMX_F32)
    hipLaunchKernelGGL((convert_kernel<unsigned short, float>), grid, block, 0, ctx->stream,
                       static_cast<const unsigned short*>(src), static_cast<float*>(dst), n);
  else if (src_dtype == dst_dtype)
    return omx_copy(ctx, dst, src, n * omx_dtype_size(src_dtype));
  else
    return omx_fail(ctx, OMX_DTYPE, "convert: unsupported dtype pair");
  OMX_LAUNCH_CHECK(ctx, "convert_kernel");
  return OMX_OK;
}

extern "C" {

int32_t omx_fill_zero(omx_ctx* ctx, void* dst, uint64_t bytes) {
  OMX_REQUIRE_CTX(ctx);
  if (bytes == 0) return OMX_OK;
  if (!dst) return omx_fail(ctx, OMX_PLACEMENT, "fill_zero: null pointer");
  if (reinterpret_cast<uintptr_t>(dst) & 3u) return omx_fail(ctx, OMX_SHAPE, "fill_zero: pointer not 4-byte aligned");
  uint64_t words = bytes / 4;
  int tail = static_cast<int>(bytes % 4);
  hipLaunchKernelGGL(fill_zero_kernel, ew_grid(words), dim3(EW_THREADS), 0, ctx->stream,
                     static_cast<unsigned int*>(dst), words, static_cast<unsigned char*>(dst) + words * 4, tail);
  OMX_LAUNCH_CHECK(ctx, "fill_zero_kernel");
  return OMX_OK;
}

int32_t omx_cast_bf16(omx_ctx* ctx, const void* x, void* y, uint64_t n) {
  OMX_REQUIRE_CTX(ctx);
  if (!x || !y) return omx_fail(ctx, OMX_PLACEMENT, "cast_bf16: null device pointer");
  if (n == 0) return omx_fail(ctx, OMX_SHAPE, "cast_bf16: zero-sized axis");
  hipLaunchKernelGGL(round_bf16_kernel, ew_grid(n), dim3(EW_THREADS), 0, ctx->stream, static_cast<const float*>(x),
                     static_cast<float*>(y), n);
  OMX_LAUNCH_CHECK(ctx, "round_bf16_kernel");
  return OMX_OK;
}
int32_t omx_to_bf16(omx_ctx* ctx, const void* x, void* y, uint64_t n) {
  OMX_REQUIRE_CTX(ctx);
  if (!x || !y) return omx_fail(ctx, OMX_PLACEMENT, "to_bf16: null device pointer");
  if (n == 0) return omx_fail(ctx, OMX_SHAPE, "to_bf16: zero-sized axis");
  return omx_convert(ctx, x, OMX_F32, y, OMX_BF16, n);
}
int32_t omx_to_f32(omx_ctx* ctx, const void* x, void* y, uint64_t n) {
  OMX_REQUIRE_CTX(ctx);
  if (!x || !y) return omx_fail(ctx, OMX_PLACEMENT, "to_f32: null device pointer");
  if (n == 0) return omx_fail(ctx, OMX_SHAPE, "to_f32: zero-sized axis");
  return omx_convert(ctx, x, OMX_BF16, y, OMX_F32, n);
}

int32_t omx_residual_add(omx_ctx* ctx, const void* x, int32_t x_dtype, const void* y, int32_t y_dtype, void* out,
                         int32_t out_dtype, uint64_t n) {
  OMX_REQUIRE_CTX(ctx);
  if (!x || !y || !out) return omx_fail(ctx, OMX_PLACEMENT, "residual_add_forward: null device pointer");
  if (!omx_valid_float_dtype(x_dtype) || !omx_valid_float_dtype(y_dtype) || !omx_valid_float_dtype(out_dtype))
    return omx_fail(ctx, OMX_DTYPE, "residual_add_forward: dtype must be f32 or bf16");
  if (n == 0) return omx_fail(ctx, OMX_SHAPE, "residual_add_forward: zero-sized axis");
  unsigned long long tag = omx_tag(ctx, F_RESIDUAL_ADD);
  dim3 grid = ew_grid(n), block(EW_THREADS);
#define ADD_K(TX, TY, TO)                                                                                   \
  hipLaunchKernelGGL((add_kernel<TX, TY, TO>), grid, block, 0, ctx->stream, static_cast<const TX*>(x),      \
                     static_cast<const TY*>(y), static_cast<TO*>(out), n, ctx->fault, tag)
  typedef unsigned short h16;
  const int key = (x_dtype == OMX_BF16 ? 4 : 0) | (y_dtype == OMX_BF16 ? 2 : 0) | (out_dtype == OMX_BF16 ? 1 : 0);
  switch (key) {
    case 0: ADD_K(float, float, float); break;
    case 1: ADD_K(float, float, h16); break;
    case 2: ADD_K(float, h16, float); break;
    case 3: ADD_K(float, h16, h16); break;
    case 4: ADD_K(h16, float, float); break;
    case 5: ADD_K(h16, float, h16); break;
    case 6: ADD_K(h16, h16, float); break;
    default: ADD_K(h16, h16, h16); break;
  }
#undef ADD_K
  OMX_LAUNCH_CHECK(ctx, "add_kernel");
  return OMX_OK;
}

int32_t omx_accumulate_grad(omx_ctx* ctx, void* acc, const void* grad, uint64_t n) {
  OMX_REQUIRE_CTX(ctx);
  if (!acc || !grad) return omx_fail(ctx, OMX_PLACEMENT, "accumulate_grad: null device pointer");
  if (n == 0) return omx_fail(ctx, OMX_SHAPE, "accumulate_grad: zero-sized axis");
  hipLaunchKernelGGL(accumulate_kernel, ew_grid(n), dim3(EW_THREADS), 0, ctx->stream, static_cast<float*>(acc),
                     static_cast<const float*>(grad), n, ctx->fault, omx_tag(ctx, F_ACCUMULATE));
  OMX_LAUNCH_CHECK(ctx, "accumulate_kernel");
  return OMX_OK;
}

int32_t omx_scale_grad(omx_ctx* ctx, void* grad, float scale, uint64_t n) {
  OMX_REQUIRE_CTX(ctx);
  if (!grad) return omx_fail(ctx, OMX_PLACEMENT, "scale_grad: null device pointer");
  if (n == 0) return omx_fail(ctx, OMX_SHAPE, "scale_grad: zero-sized axis");
  if (!(scale == scale) || scale == INFINITY || scale == -INFINITY)
    return omx_fail(ctx, OMX_NON_FINITE, "scale_grad");
  hipLaunchKernelGGL(scale_kernel, ew_grid(n), dim3(EW_THREADS), 0, ctx->stream, static_cast<float*>(grad), scale, n,
                     ctx->fault, omx_tag(ctx, F_SCALE_GRAD));
  OMX_LAUNCH_CHECK(ctx, "scale_kernel");
  return OMX_OK;
}

int32_t omx_gelu_forward(omx_ctx* ctx, const void* x, void* y, int32_t dtype, uint64_t n, int32_t tanh_form) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = tanh_form ? "gelu_tanh_forward" : "gelu_erf_forward";
  if (!x || !y) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  if (n == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  unsigned long long tag = omx_tag(ctx, F_GELU_FORWARD);
  dim3 grid = ew_grid(n), block(EW_THREADS);
#define GELU_FWD(T, TANH)                                                                                       \
  hipLaunchKernelGGL((gelu_fwd_kernel<T, TANH>), grid, block, 0, ctx->stream, static_cast<const T*>(x), \
                     static_cast<T*>(y), n, ctx->fault, tag)
  if (dtype == OMX_F32) {
    if (tanh_form) GELU_FWD(float, true);
    else GELU_FWD(float, false);
  } else {
    if (tanh_form) GELU_FWD(unsigned short, true);
    else GELU_FWD(unsigned short, false);
  }
#undef GELU_FWD
  OMX_LAUNCH_CHECK(ctx, "gelu_fwd_kernel");
  return OMX_OK;
}

int32_t omx_gelu_backward(omx_ctx* ctx, const void* x, const void* gy, void* gx, int32_t dtype, uint64_t n,
                          int32_t tanh_form) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = tanh_form ? "gelu_tanh_backward" : "gelu_erf_backward";
  if (!x || !gy || !gx) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  if (n == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  unsigned long long tag = omx_tag(ctx, F_GELU_BACKWARD);
  dim3 grid = ew_grid(n), block(EW_THREADS);
#define GELU_BWD(T, TANH)                                                                                       \
  hipLaunchKernelGGL((gelu_bwd_kernel<T, TANH>), grid, block, 0, ctx->stream, static_cast<const T*>(x), \
                     static_cast<const T*>(gy), static_cast<T*>(gx), n, ctx->fault, tag)
  if (dtype == OMX_F32) {
    if (tanh_form) GELU_BWD(float, true);
    else GELU_BWD(float, false);
  } else {
    if (tanh_form) GELU_BWD(unsigned short, true);
    else GELU_BWD(unsigned short, false);
  }
#undef GELU_BWD
  OMX_LAUNCH_CHECK(ctx, "gelu_bwd_kernel");
  return OMX_OK;
}

int32_t omx_permute_0213(omx_ctx* ctx, const void* x, void* y, int32_t dtype, uint64_t d0, uint64_t d1, uint64_t d2,
                         uint64_t d3) {
  OMX_REQUIRE_CTX(ctx);
  if (!x || !y) return omx_fail(ctx, OMX_PLACEMENT, "permute: null device pointer");
  if (!(dtype == OMX_F32 || dtype == OMX_BF16 || dtype == OMX_U32)) return omx_fail(ctx, OMX_DTYPE, "permute: dtype");
  if (d0 == 0 || d1 == 0 || d2 == 0 || d3 == 0) return omx_fail(ctx, OMX_SHAPE, "permute: zero-sized axis");
  size_t esz = omx_dtype_size(dtype);
  size_t row_bytes = d3 * esz;
  bool al16 = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15u) == 0;
  if (row_bytes % 16 == 0 && al16) {
    size_t d3v = row_bytes / 16;
    hipLaunchKernelGGL((permute_0213_kernel<uint4>), ew_grid(d0 * d1 * d2 * d3v), dim3(EW_THREADS), 0, ctx->stream,
                       static_cast<const uint4*>(x), static_cast<uint4*>(y), d0, d1, d2, d3v);
  } else if (esz == 4) {
    hipLaunchKernelGGL((permute_0213_kernel<unsigned int>), ew_grid(d0 * d1 * d2 * d3), dim3(EW_THREADS), 0,
                       ctx->stream, static_cast<const unsigned int*>(x), static_cast<unsigned int*>(y), d0, d1, d2, d3);
  } else {
    hipLaunchKernelGGL((permute_0213_kernel<unsigned short>), ew_grid(d0 * d1 * d2 * d3), dim3(EW_THREADS), 0,
                       ctx->stream, static_cast<const unsigned short*>(x), static_cast<unsigned short*>(y), d0, d1, d2,
                       d3);
  }
  OMX_LAUNCH_CHECK(ctx, "permute_0213_kernel");
  return OMX_OK;
}

int32_t omx_token_windows(omx_ctx* ctx, const void* tokens, int32_t bytes_per_token, uint64_t n_tokens,
                          const uint64_t* starts, uint64_t batch, uint64_t seq_len, void* x, void* y) {
  OMX_REQUIRE_CTX(ctx);
  if (!tokens || !x || !y) return omx_fail(ctx, OMX_PLACEMENT, "token_windows: null device pointer");
  if (!starts) return omx_fail(ctx, OMX_PLACEMENT, "token_windows: null starts");
  if (bytes_per_token != 2 && bytes_per_token != 4)
    return omx_fail(ctx, OMX_DTYPE, "token_windows: tokens are 2 or 4 bytes wide, got %d", bytes_per_token);
  if (batch == 0 || seq_len == 0) return omx_fail(ctx, OMX_SHAPE, "token_windows: zero-sized axis");
  if (seq_len >= n_tokens || batch > (1ull << 32) || seq_len > (1ull << 32))
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "token_windows: a window of %llu + 1 tokens in a bin of %llu",
                    static_cast<unsigned long long>(seq_len), static_cast<unsigned long long>(n_tokens));
  for (uint64_t b = 0; b < batch; ++b)
    if (starts[b] > n_tokens - seq_len - 1)
      return omx_fail(ctx, OMX_OUT_OF_RANGE, "token_windows: window %llu starts at %llu, past the bin's %llu tokens",
                      static_cast<unsigned long long>(b), static_cast<unsigned long long>(starts[b]),
                      static_cast<unsigned long long>(n_tokens));
  void* ws = nullptr;
  int32_t rc = omx_workspace(ctx, batch * sizeof(uint64_t), &ws);
  if (rc != OMX_OK) return rc;
  // The caller may reuse or free `starts` as soon as this returns, and an asynchronous copy from
  // pageable memory is not guaranteed to have read its source by then: wait for it, as omx_upload does.
  OMX_HIP(ctx, hipMemcpyAsync(ws, starts, batch * sizeof(uint64_t), hipMemcpyHostToDevice, ctx->stream));
  OMX_HIP(ctx, hipStreamSynchronize(ctx->stream));
  const uint64_t n = batch * seq_len;
  const unsigned blocks = static_cast<unsigned>(std::min<uint64_t>((n + 255) / 256, 4096));
  if (bytes_per_token == 2)
    hipLaunchKernelGGL((token_windows_kernel<unsigned short>), dim3(blocks), dim3(256), 0, ctx->stream,
                       static_cast<const unsigned short*>(tokens), static_cast<const unsigned long long*>(ws),
                       static_cast<unsigned int*>(x), static_cast<unsigned int*>(y), batch, seq_len);
  else
    hipLaunchKernelGGL((token_windows_kernel<unsigned int>), dim3(blocks), dim3(256), 0, ctx->stream,
                       static_cast<const unsigned int*>(tokens), static_cast<const unsigned long long*>(ws),
                       static_cast<unsigned int*>(x), static_cast<unsigned int*>(y), batch, seq_len);
  OMX_LAUNCH_CHECK(ctx, "token_windows_kernel");
  return OMX_OK;
}

}  // extern "C"
