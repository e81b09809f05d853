// Bandwidth-bound ops of the Llama-shaped block around the frozen int8 projections: the rotary
// embedding applied in place to the q and k column blocks of a fused projection output, and the
// SwiGLU product on a fused gate | up projection output. Single coalesced passes, 16 bytes per lane.
//
// Reference semantics: rope_half_split (ojas-cpu/src/norm.rs:271-312: for i < dim/2,
// y[i] = x[i] cos[i] - x[i + dim/2] sin[i], y[i + dim/2] = x[i + dim/2] cos[i] + x[i] sin[i]; the
// backward is the rotation by the opposite angle); silu and mul (ojas-cpu/src/pointwise.rs:346-366,
// 515-546; ojas-model/src/block.rs:248-262 is where the model composes them).
#include "omx_common.h"

namespace {

__device__ __forceinline__ void unpack8(const uint4& w, float (&f)[8]) {
  const unsigned int u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(u[i] << 16);
    f[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
  unsigned int u[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    u[i] = dev_pack_bf16_pair(f[2 * i], f[2 * i + 1]);
  return make_uint4(u[0], u[1], u[2], u[3]);
}

// One thread rotates 8 pairs: elements [c, c + 8) and [c + dim/2, c + dim/2 + 8) of one head.
__global__ void rope_pitched_kernel(unsigned short* __restrict__ x, long pitch, const float* __restrict__ cos_t,
                                    const float* __restrict__ sin_t, long tokens, int time, int heads, int dim,
                                    float sin_sign, OmxFaultWord* fault, unsigned long long tag) {
  const int half = dim / 2, per_head = half / 8;
  const long total = tokens * heads * per_head;
  const long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int piece = static_cast<int>(i % per_head);
  const int head = static_cast<int>((i / per_head) % heads);
  const long token = i / (static_cast<long>(per_head) * heads);
  const int t = static_cast<int>(token % time);
  unsigned short* lo_p = x + token * pitch + static_cast<long>(head) * dim + piece * 8;
  unsigned short* hi_p = lo_p + half;
  float lo[8], hi[8], c[8], s[8];
  unpack8(*reinterpret_cast<const uint4*>(lo_p), lo);
  unpack8(*reinterpret_cast<const uint4*>(hi_p), hi);
  const float* cp = cos_t + static_cast<long>(t) * dim + piece * 8;
  const float* sp = sin_t + static_cast<long>(t) * dim + piece * 8;
  const float4 c0 = *reinterpret_cast<const float4*>(cp), c1 = *reinterpret_cast<const float4*>(cp + 4);
  const float4 s0 = *reinterpret_cast<const float4*>(sp), s1 = *reinterpret_cast<const float4*>(sp + 4);
  c[0] = c0.x; c[1] = c0.y; c[2] = c0.z; c[3] = c0.w; c[4] = c1.x; c[5] = c1.y; c[6] = c1.z; c[7] = c1.w;
  s[0] = s0.x; s[1] = s0.y; s[2] = s0.z; s[3] = s0.w; s[4] = s1.x; s[5] = s1.y; s[6] = s1.z; s[7] = s1.w;
  float ylo[8], yhi[8];
  bool bad = false;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float sn = s[e] * sin_sign;
    ylo[e] = lo[e] * c[e] - hi[e] * sn;
    yhi[e] = hi[e] * c[e] + lo[e] * sn;
    bad |= !(dev_finite(ylo[e]) && dev_finite(yhi[e]));
  }
  *reinterpret_cast<uint4*>(lo_p) = pack8(ylo);
  *reinterpret_cast<uint4*>(hi_p) = pack8(yhi);
  if (bad) dev_raise_fault(fault, tag);
}

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + __expf(-x)); }

// Eight consecutive values of a bf16 or an f32 tensor as floats (16-byte accesses).
__device__ __forceinline__ void load8(const unsigned short* p, float (&v)[8]) { unpack8(*reinterpret_cast<const uint4*>(p), v); }
__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
}

// The forward rotation out of place, x (bf16 or f32) -> bf16 out at the same pitch: a thread takes
// elements [c, c + 8) and [c + dim/2, c + dim/2 + 8) of one head, rotates them when the head is one
// of the first `heads` and converts them as they are for the `plain` heads behind those.
template <typename TIN>
__global__ void rope_pitched_out_kernel(const TIN* __restrict__ x, unsigned short* __restrict__ out, long pitch,
                                        const float* __restrict__ cos_t, const float* __restrict__ sin_t, long tokens,
                                        int time, int heads, int plain, int dim, OmxFaultWord* fault,
                                        unsigned long long tag) {
  const int half = dim / 2, per_head = half / 8, all = heads + plain;
  const long total = tokens * all * per_head;
  const long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int piece = static_cast<int>(i % per_head);
  const int head = static_cast<int>((i / per_head) % all);
  const long token = i / (static_cast<long>(per_head) * all);
  const long at = token * pitch + static_cast<long>(head) * dim + piece * 8;
  float lo[8], hi[8], ylo[8], yhi[8];
  load8(x + at, lo);
  load8(x + at + half, hi);
  bool bad = false;
  if (head < heads) {
    const int t = static_cast<int>(token % time);
    float c[8], s[8];
    load8(cos_t + static_cast<long>(t) * dim + piece * 8, c);
    load8(sin_t + static_cast<long>(t) * dim + piece * 8, s);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      ylo[e] = lo[e] * c[e] - hi[e] * s[e];
      yhi[e] = hi[e] * c[e] + lo[e] * s[e];
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) ylo[e] = lo[e], yhi[e] = hi[e];
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) bad |= !(dev_finite(ylo[e]) && dev_finite(yhi[e]));
  *reinterpret_cast<uint4*>(out + at) = pack8(ylo);
  *reinterpret_cast<uint4*>(out + at + half) = pack8(yhi);
  if (bad) dev_raise_fault(fault, tag);
}

// gate_up: [rows][2 * hidden] (gate columns first), bf16 or f32 (the projection's output as its
// product left it, so the activation is rounded once, when it is stored as the next product's
// operand). out[r][c] = silu(gate[r][c]) * up[r][c], bf16.
template <typename GU>
__global__ void swiglu_fwd_kernel(const GU* __restrict__ gate_up, unsigned short* __restrict__ out,
                                  long rows, long hidden, OmxFaultWord* fault, unsigned long long tag) {
  const long per_row = hidden / 8, total = rows * per_row;
  const long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long r = i / per_row, c = (i % per_row) * 8;
  float g[8], u[8], y[8];
  load8(gate_up + r * 2 * hidden + c, g);
  load8(gate_up + r * 2 * hidden + hidden + c, u);
  bool bad = false;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    y[e] = g[e] * sigmoid_f(g[e]) * u[e];
    bad |= !dev_finite(y[e]);
  }
  *reinterpret_cast<uint4*>(out + r * hidden + c) = pack8(y);
  if (bad) dev_raise_fault(fault, tag);
}

// g_gate = gm * up * silu'(gate), g_up = gm * silu(gate); silu'(x) = s (1 + x (1 - s)), s = sigmoid(x).
template <typename GU>
__global__ void swiglu_bwd_kernel(const GU* __restrict__ gate_up, const unsigned short* __restrict__ gm,
                                  unsigned short* __restrict__ g_gate_up, long rows, long hidden, OmxFaultWord* fault,
                                  unsigned long long tag) {
  const long per_row = hidden / 8, total = rows * per_row;
  const long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long r = i / per_row, c = (i % per_row) * 8;
  float g[8], u[8], d[8], gg[8], gu[8];
  load8(gate_up + r * 2 * hidden + c, g);
  load8(gate_up + r * 2 * hidden + hidden + c, u);
  unpack8(*reinterpret_cast<const uint4*>(gm + r * hidden + c), d);
  bool bad = false;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float s = sigmoid_f(g[e]);
    gu[e] = d[e] * (g[e] * s);
    gg[e] = d[e] * u[e] * (s * (1.0f + g[e] * (1.0f - s)));
    bad |= !(dev_finite(gu[e]) && dev_finite(gg[e]));
  }
  *reinterpret_cast<uint4*>(g_gate_up + r * 2 * hidden + c) = pack8(gg);
  *reinterpret_cast<uint4*>(g_gate_up + r * 2 * hidden + hidden + c) = pack8(gu);
  if (bad) dev_raise_fault(fault, tag);
}

// Counter-based generator for synthetic weights: SplitMix64's output function of (seed, counter),
// two 24-bit uniforms, Box-Muller. Element i of a tensor is a function of (seed, i) alone.
__device__ __forceinline__ unsigned long long mix64(unsigned long long z) {
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}
__device__ __forceinline__ void normal_pair(unsigned long long seed, unsigned long long pair, float* a, float* b) {
  const unsigned long long bits = mix64(seed + 0x9e3779b97f4a7c15ull * (pair + 1));
  const float u1 = (static_cast<float>(bits & 0xffffffu) + 1.0f) * (1.0f / 16777216.0f);  // (0, 1]
  const float u2 = static_cast<float>((bits >> 24) & 0xffffffu) * (1.0f / 16777216.0f);
  const float rad = sqrtf(-2.0f * __logf(u1));
  float sn, cs;
  __sincosf(6.28318530717958647692f * u2, &sn, &cs);
  *a = rad * cs;
  *b = rad * sn;
}

template <typename T>
__global__ void init_normal_kernel(T* __restrict__ dst, long n, unsigned long long seed, float std) {
  const long pair = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (2 * pair >= n) return;
  float a, b;
  normal_pair(seed, static_cast<unsigned long long>(pair), &a, &b);
  dev_store<T>(dst, 2 * pair, a * std);
  if (2 * pair + 1 < n) dev_store<T>(dst, 2 * pair + 1, b * std);
}

// One thread per group of 32: draws the group's values, then quantises them with the rule of
// ojas-cpu/src/quant_sparse.rs:306-326 applied to the group (scale = abs_max / 127, or 1 for zeros;
// code = round half away from zero of v * 127 / abs_max, clamped to +-127).
__global__ void init_normal_i8_group_kernel(signed char* __restrict__ codes, float* __restrict__ scales, long groups,
                                            unsigned long long seed, float std) {
  const long gi = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gi >= groups) return;
  float v[32];
  float abs_max = 0.0f;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    normal_pair(seed, static_cast<unsigned long long>(gi) * 16 + i, &v[2 * i], &v[2 * i + 1]);
    v[2 * i] *= std;
    v[2 * i + 1] *= std;
    abs_max = fmaxf(abs_max, fmaxf(fabsf(v[2 * i]), fabsf(v[2 * i + 1])));
  }
  scales[gi] = abs_max > 0.0f ? abs_max / 127.0f : 1.0f;
  const float inv = abs_max > 0.0f ? 127.0f / abs_max : 0.0f;
  unsigned int words[8];
#pragma unroll
  for (int w = 0; w < 8; ++w) {
    unsigned int word = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      float q = roundf(v[4 * w + b] * inv);
      q = fminf(fmaxf(q, -127.0f), 127.0f);
      word |= (static_cast<unsigned int>(static_cast<int>(q)) & 0xffu) << (8 * b);
    }
    words[w] = word;
  }
  uint4* out = reinterpret_cast<uint4*>(codes + gi * 32);
  out[0] = make_uint4(words[0], words[1], words[2], words[3]);
  out[1] = make_uint4(words[4], words[5], words[6], words[7]);
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

extern "C" {

int32_t omx_rope_half_split_inplace(omx_ctx* ctx, void* x, int32_t dtype, uint64_t pitch, const void* cos_f32,
                                    const void* sin_f32, uint64_t tokens, uint64_t time, uint64_t heads, uint64_t dim,
                                    int32_t backward) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = backward ? "rope_half_split_backward" : "rope_half_split_forward";
  if (!x || !cos_f32 || !sin_f32) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (dtype != OMX_BF16) return omx_fail(ctx, OMX_DTYPE, "%s: the in-place form takes bf16", op);
  if (tokens == 0 || time == 0 || heads == 0 || dim == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (dim % 16 != 0) return omx_fail(ctx, OMX_SHAPE, "%s: head_dim %llu is not a multiple of 16", op, (unsigned long long)dim);
  if (pitch < heads * dim || pitch % 8 != 0 || !aligned16(x) || !aligned16(cos_f32) || !aligned16(sin_f32))
    return omx_fail(ctx, OMX_SHAPE, "%s: pitch %llu does not hold %llu heads of %llu in 16-byte pieces", op,
                    (unsigned long long)pitch, (unsigned long long)heads, (unsigned long long)dim);
  if (tokens > 0x7fffffffull || heads * dim > 0x7fffffffull)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: axis does not fit in i32", op);
  const long total = static_cast<long>(tokens * heads * (dim / 16));
  hipLaunchKernelGGL(rope_pitched_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, ctx->stream,
                     static_cast<unsigned short*>(x), static_cast<long>(pitch), static_cast<const float*>(cos_f32),
                     static_cast<const float*>(sin_f32), static_cast<long>(tokens), static_cast<int>(time),
                     static_cast<int>(heads), static_cast<int>(dim), backward ? -1.0f : 1.0f, ctx->fault,
                     omx_tag(ctx, backward ? F_ROPE_BACKWARD : F_ROPE_FORWARD));
  OMX_LAUNCH_CHECK(ctx, "rope_pitched_kernel");
  return OMX_OK;
}

int32_t omx_rope_half_split_pitched(omx_ctx* ctx, const void* x, int32_t x_dtype, void* out, uint64_t pitch,
                                    const void* cos_f32, const void* sin_f32, uint64_t tokens, uint64_t time,
                                    uint64_t heads, uint64_t plain_heads, uint64_t dim) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "rope_half_split_forward";
  if (!x || !out || !cos_f32 || !sin_f32) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(x_dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: the input must be f32 or bf16", op);
  if (tokens == 0 || time == 0 || heads + plain_heads == 0 || dim == 0)
    return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (dim % 16 != 0) return omx_fail(ctx, OMX_SHAPE, "%s: head_dim %llu is not a multiple of 16", op, (unsigned long long)dim);
  if (pitch < (heads + plain_heads) * dim || pitch % 8 != 0 || !aligned16(x) || !aligned16(out) || !aligned16(cos_f32) ||
      !aligned16(sin_f32))
    return omx_fail(ctx, OMX_SHAPE, "%s: pitch %llu does not hold %llu heads of %llu in 16-byte pieces", op,
                    (unsigned long long)pitch, (unsigned long long)(heads + plain_heads), (unsigned long long)dim);
  if (tokens > 0x7fffffffull || (heads + plain_heads) * dim > 0x7fffffffull)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: axis does not fit in i32", op);
  const long total = static_cast<long>(tokens * (heads + plain_heads) * (dim / 16));
  const dim3 grid(static_cast<unsigned>((total + 255) / 256));
  const unsigned long long tag = omx_tag(ctx, F_ROPE_FORWARD);
  if (x_dtype == OMX_BF16)
    hipLaunchKernelGGL(rope_pitched_out_kernel<unsigned short>, grid, dim3(256), 0, ctx->stream,
                       static_cast<const unsigned short*>(x), static_cast<unsigned short*>(out), static_cast<long>(pitch),
                       static_cast<const float*>(cos_f32), static_cast<const float*>(sin_f32), static_cast<long>(tokens),
                       static_cast<int>(time), static_cast<int>(heads), static_cast<int>(plain_heads),
                       static_cast<int>(dim), ctx->fault, tag);
  else
    hipLaunchKernelGGL(rope_pitched_out_kernel<float>, grid, dim3(256), 0, ctx->stream, static_cast<const float*>(x),
                       static_cast<unsigned short*>(out), static_cast<long>(pitch), static_cast<const float*>(cos_f32),
                       static_cast<const float*>(sin_f32), static_cast<long>(tokens), static_cast<int>(time),
                       static_cast<int>(heads), static_cast<int>(plain_heads), static_cast<int>(dim), ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "rope_pitched_out_kernel");
  return OMX_OK;
}

int32_t omx_init_normal(omx_ctx* ctx, void* dst, int32_t dtype, uint64_t n, uint64_t seed, float std) {
  OMX_REQUIRE_CTX(ctx);
  if (!dst) return omx_fail(ctx, OMX_PLACEMENT, "init_normal: null device pointer");
  if (!omx_valid_float_dtype(dtype)) return omx_fail(ctx, OMX_DTYPE, "init_normal: dtype must be f32 or bf16");
  if (n == 0) return OMX_OK;
  const long pairs = static_cast<long>((n + 1) / 2);
  dim3 grid(static_cast<unsigned>((pairs + 255) / 256)), block(256);
  if (dtype == OMX_F32)
    hipLaunchKernelGGL(init_normal_kernel<float>, grid, block, 0, ctx->stream, static_cast<float*>(dst),
                       static_cast<long>(n), static_cast<unsigned long long>(seed), std);
  else
    hipLaunchKernelGGL(init_normal_kernel<unsigned short>, grid, block, 0, ctx->stream,
                       static_cast<unsigned short*>(dst), static_cast<long>(n), static_cast<unsigned long long>(seed), std);
  OMX_LAUNCH_CHECK(ctx, "init_normal_kernel");
  return OMX_OK;
}

int32_t omx_init_normal_i8_group(omx_ctx* ctx, void* codes_i8, void* scales_f32, uint64_t nout, uint64_t kin,
                                 uint64_t group, uint64_t seed, float std) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "init_normal_i8_group";
  if (!codes_i8 || !scales_f32) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (group != 32) return omx_fail(ctx, OMX_UNSUPPORTED, "%s: group size %llu (only 32)", op, (unsigned long long)group);
  if (nout == 0 || kin == 0 || kin % 32 != 0) return omx_fail(ctx, OMX_SHAPE, "%s: k_in must be a positive multiple of 32", op);
  if (!aligned16(codes_i8)) return omx_fail(ctx, OMX_SHAPE, "%s: codes must be 16-byte aligned", op);
  const long groups = static_cast<long>(nout * (kin / 32));
  hipLaunchKernelGGL(init_normal_i8_group_kernel, dim3(static_cast<unsigned>((groups + 255) / 256)), dim3(256), 0,
                     ctx->stream, static_cast<signed char*>(codes_i8), static_cast<float*>(scales_f32), groups,
                     static_cast<unsigned long long>(seed), std);
  OMX_LAUNCH_CHECK(ctx, "init_normal_i8_group_kernel");
  return OMX_OK;
}

int32_t omx_swiglu_forward(omx_ctx* ctx, const void* gate_up, void* out, int32_t dtype, uint64_t rows, uint64_t hidden) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "swiglu_forward";
  if (!gate_up || !out) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: gate_up must be f32 or bf16", op);
  if (rows == 0 || hidden == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (hidden % 8 != 0 || !aligned16(gate_up) || !aligned16(out))
    return omx_fail(ctx, OMX_SHAPE, "%s: hidden %llu must be a multiple of 8 and the tensors 16-byte aligned", op,
                    (unsigned long long)hidden);
  const long total = static_cast<long>(rows * (hidden / 8));
  const unsigned long long tag = omx_tag(ctx, F_MUL_FORWARD);
  if (dtype == OMX_BF16)
    hipLaunchKernelGGL(swiglu_fwd_kernel<unsigned short>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                       ctx->stream, static_cast<const unsigned short*>(gate_up), static_cast<unsigned short*>(out),
                       static_cast<long>(rows), static_cast<long>(hidden), ctx->fault, tag);
  else
    hipLaunchKernelGGL(swiglu_fwd_kernel<float>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                       ctx->stream, static_cast<const float*>(gate_up), static_cast<unsigned short*>(out),
                       static_cast<long>(rows), static_cast<long>(hidden), ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "swiglu_fwd_kernel");
  return OMX_OK;
}

int32_t omx_swiglu_backward(omx_ctx* ctx, const void* gate_up, const void* gy, void* g_gate_up, int32_t dtype,
                            uint64_t rows, uint64_t hidden) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "swiglu_backward";
  if (!gate_up || !gy || !g_gate_up) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: gate_up must be f32 or bf16", op);
  if (rows == 0 || hidden == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (hidden % 8 != 0 || !aligned16(gate_up) || !aligned16(gy) || !aligned16(g_gate_up))
    return omx_fail(ctx, OMX_SHAPE, "%s: hidden %llu must be a multiple of 8 and the tensors 16-byte aligned", op,
                    (unsigned long long)hidden);
  const long total = static_cast<long>(rows * (hidden / 8));
  const unsigned long long tag = omx_tag(ctx, F_MUL_BACKWARD);
  if (dtype == OMX_BF16)
    hipLaunchKernelGGL(swiglu_bwd_kernel<unsigned short>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                       ctx->stream, static_cast<const unsigned short*>(gate_up), static_cast<const unsigned short*>(gy),
                       static_cast<unsigned short*>(g_gate_up), static_cast<long>(rows), static_cast<long>(hidden),
                       ctx->fault, tag);
  else
    hipLaunchKernelGGL(swiglu_bwd_kernel<float>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                       ctx->stream, static_cast<const float*>(gate_up), static_cast<const unsigned short*>(gy),
                       static_cast<unsigned short*>(g_gate_up), static_cast<long>(rows), static_cast<long>(hidden),
                       ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "swiglu_bwd_kernel");
  return OMX_OK;
}

}  // extern "C"
