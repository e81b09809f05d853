// Internal declarations shared by the kernel files of libojas_mi355x.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <hip/hip_bf16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <initializer_list>
#include <map>
#include <string>
#include <vector>

#include "ojas_mi355x.h"

// Ops that can raise a deferred non-finite fault, in the order their bits sit
// in the fault word. The name is what OjasError::NonFinite { op } carries.
enum OmxFaultOp : uint32_t {
  F_LINEAR_FORWARD = 0,
  F_LINEAR_BACKWARD,
  F_GEMM,
  F_SDPA_FORWARD,
  F_SDPA_BACKWARD,
  F_RMS_FORWARD,
  F_RMS_BACKWARD,
  F_CE_FORWARD,
  F_CE_BACKWARD,
  F_LINEAR_CE,
  F_EMBEDDING_FORWARD,
  F_EMBEDDING_BACKWARD,
  F_ADAMW,
  F_MUON,
  F_CLIP,
  F_RESIDUAL_ADD,
  F_ACCUMULATE,
  F_SCALE_GRAD,
  F_GELU_FORWARD,
  F_GELU_BACKWARD,
  F_ARGMAX,
  F_TOPK,
  F_SILU_FORWARD,
  F_SILU_BACKWARD,
  F_MUL_FORWARD,
  F_MUL_BACKWARD,
  F_ROPE_FORWARD,
  F_ROPE_BACKWARD,
  F_RMS_QK_FORWARD,
  F_RMS_QK_BACKWARD,
  F_GATE_FORWARD,
  F_GATE_BACKWARD,
  F_VRES_FORWARD,
  F_VRES_BACKWARD,
  F_CACHED_ATTENTION,
  F_KV_CACHE_WRITE,
  F_COUNT
};
const char* omx_fault_name(uint32_t op);

// Device-side fault record: a bit mask plus the launch sequence number of the
// first op that faulted (lowest sequence wins), so the error can name it.
struct OmxFaultWord {
  unsigned long long mask;
  unsigned long long first;  // (sequence << 8) | op, ~0 when clear
};

struct omx_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  uint64_t budget_limit = 0, budget_live = 0, budget_peak = 0;
  std::map<void*, uint64_t> allocations;
  // Freed blocks kept for reuse by size (see omx_free); not charged to the budget.
  std::multimap<uint64_t, void*> pool;
  uint64_t pooled_bytes = 0;
  OmxFaultWord* fault = nullptr;  // device
  OmxFaultWord* fault_host = nullptr;  // pinned
  uint64_t sequence = 0;
  std::string last_error;
  std::string arch;
  // Scratch the library owns (charged to the budget); grown on demand.
  // Slot 0: per-op scratch. Slot 1: split-K partials of the GEMM (which an op
  // may call while it holds slot 0) and operands converted for an op that holds slot 0.
  // Slot 2: tensors an op keeps across calls into other ops (a recomputed attention output).
  void* workspace[3] = {nullptr, nullptr, nullptr};
  uint64_t workspace_bytes[3] = {0, 0, 0};
  int cu_count = 0;
  // This device's copy of the static scratch of omx_cross_entropy_mean_forward_static, looked up
  // when the context is opened (the lookup is not stream work and may load the code object).
  void* ce_static_scratch = nullptr;
  // Optional per-launch timing of the GEMM kernel (benchmark only).
  // 0: 128x128 kernel only; 1: choose by shape; 2 / 3: force the 256x256 / 256x128 direct-to-LDS kernel where eligible.
  int gemm_dma_mode = 1;
  int gemm_row_split = 1;    // 0: a product whose last round of 256 x 256 tiles is mostly empty is not cut by rows
  bool gemm_in_row_split = false;  // set while omx_gemm_impl runs the two halves of a cut product
  int gemm_forced_tiling = -1;     // the tiling the first half keeps, whatever its own tile count says
  int gemm_thin = 1;         // outputs of at most 64 columns over many rows take gemm_thin_kernel
  int flash_schedule = 0;     // 0: by the chip's workgroup places; 1: one 128-row block per workgroup; 2: mirrored pairs
  int kv_attention_mode = 0;  // 1: cached attention always takes the LDS-tiled kernel
  int adamw_trust = 1;        // 0: omx_adamw_step_bounded always runs its checking pass
  int ce_fused = 1;           // 0: linear-CE always takes the separate statistics and gradient kernels
  int sdpa_tiled = 1;         // 0: f32 attention always takes the one-wave-per-row kernels
  int muon_fused_sums = 1;    // 0: Newton-Schulz forms b A + c A^2 and a X + B X in kernels of their own (bf16 tier)
  bool profile_gemm = false;
  uint32_t profile_classes = 0;  // bit per OmxKernelClass other than the products (omx_profile_kernels)
  // The events of the product being launched (null when not timing): the first kernel of the
  // product takes `timing_start`, its last one `timing_stop`.
  hipEvent_t timing_start = nullptr, timing_stop = nullptr;
  struct TimedLaunch {
    hipEvent_t start, stop;
    double flops;  // the launch's algorithmic work: FLOPs for the matrix-unit classes, bytes for the others
    int cls = 0;
  };
  std::vector<TimedLaunch> timed;
  std::vector<hipEvent_t> event_pool;
};

// A kernel launch on the context's stream; with events, the dispatch itself carries them (its own
// begin and end timestamps, no extra packets in the queue).
template <typename F, typename... Args>
inline void omx_launch_timed(omx_ctx* ctx, F kernel, dim3 grid, dim3 block, unsigned smem, hipEvent_t start,
                             hipEvent_t stop, Args... args) {
  if (start || stop) hipExtLaunchKernelGGL(kernel, grid, block, smem, ctx->stream, start, stop, 0, args...);
  else hipLaunchKernelGGL(kernel, grid, block, smem, ctx->stream, args...);
}

int32_t omx_fail(omx_ctx* ctx, omx_status code, const char* fmt, ...);
void omx_release_pool(omx_ctx* ctx);
// The device address of the static cross-entropy scratch on the current device (loss.hip), or null.
void* omx_ce_static_scratch_address();
// Per-product timing for callers outside gemm.hip: takes a pair of events for the product about
// to be launched (when omx_profile_gemm is on) and files them with its FLOP count afterwards.
int32_t omx_timing_begin(omx_ctx* ctx, double flops, omx_ctx::TimedLaunch* timed);
void omx_timing_end(omx_ctx* ctx, bool launched, const omx_ctx::TimedLaunch& timed);

// Kernel classes that can be timed per launch (benchmark only); the values are those of
// omx_profile_kernels in the public header.
enum OmxKernelClass {
  OMX_K_GEMM = 0, OMX_K_FLASH_FWD = 1, OMX_K_FLASH_BWD = 2, OMX_K_CE = 3, OMX_K_ADAMW = 4, OMX_K_RMS_FWD = 5,
  OMX_K_RMS_BWD = 6, OMX_K_EMBED_BWD = 7, OMX_K_CLASSES = 8
};
// Events for one launch (or one run of launches) of a timed class: the first kernel is launched
// with start(), the last with stop() (both null while the class is off, which makes
// omx_launch_timed an ordinary launch); the destructor files the pair with `work`.
struct OmxKernelTimer {
  omx_ctx* ctx;
  omx_ctx::TimedLaunch t{};
  bool on = false;
  OmxKernelTimer(omx_ctx* ctx, int cls, double work);
  ~OmxKernelTimer();
  OmxKernelTimer(const OmxKernelTimer&) = delete;
  OmxKernelTimer& operator=(const OmxKernelTimer&) = delete;
  hipEvent_t start() const { return on ? t.start : nullptr; }
  hipEvent_t stop() const { return on ? t.stop : nullptr; }
};

int32_t omx_hip_fail(omx_ctx* ctx, hipError_t err, const char* what);
// Grows workspace `slot` to at least `bytes` (budget-charged).
int32_t omx_workspace(omx_ctx* ctx, uint64_t bytes, void** out, int slot = 0);
// Next launch tag for fault attribution: (sequence << 8) | op.
inline unsigned long long omx_tag(omx_ctx* ctx, uint32_t op) {
  return (static_cast<unsigned long long>(++ctx->sequence) << 8) | op;
}

// C[m,n] (+)= A.B with element strides; `ldc` is C's row pitch in elements.
// Optional elementwise work in the GEMM's store pass (bf16 outputs only; `aux` shares C's row pitch):
//   OMX_EPI_GELU_FWD: C = u (rounded to bf16) and aux_out = gelu(u);
//   OMX_EPI_GELU_BWD: C = round_bf16(A.B) * gelu'(aux_in);
//   OMX_EPI_AXPBY: C = round_bf16(s1 aux_in) + round_bf16(s2 round_bf16(A.B)): the product stored as
//     bf16, then the two-term sum a separate pass over it would form, in one store.
// aux tensors have C's layout (pitch, and batch stride in a strided batch).
enum { OMX_EPI_NONE = 0, OMX_EPI_GELU_FWD = 1, OMX_EPI_GELU_BWD = 2, OMX_EPI_AXPBY = 3 };
struct OmxGemmEpilogue {
  int mode;
  int tanh_form;
  const void* aux_in;
  void* aux_out;
  float s1 = 0.0f, s2 = 0.0f;  // OMX_EPI_AXPBY
};
// `count` products of one shape whose operands lie `stride_*` ELEMENTS apart (16-byte multiples), one launch.
struct OmxGemmBatch {
  uint64_t count, stride_a, stride_b, stride_c;
};
int32_t omx_gemm_impl(omx_ctx* ctx, uint32_t fault_op, const void* a, uint64_t a_rs, uint64_t a_cs, const void* b,
                      uint64_t b_rs, uint64_t b_cs, int32_t operand_dtype, void* c, int32_t c_dtype, uint64_t ldc,
                      uint64_t m, uint64_t k, uint64_t n, int32_t accumulate, const OmxGemmEpilogue* epi = nullptr,
                      const OmxGemmBatch* batch = nullptr);
// out[c] = sum over b < blocks of partial[b * dim + c], added in a fixed order.
// `scratch` (OMX_COLUMN_SUM_GROUPS * dim floats, may be null) lets a tall `partial` be added in two stages.
constexpr int OMX_COLUMN_SUM_GROUPS = 32;
// Up to this many rows a tall sum is one launch of 1024-thread workgroups.
constexpr int OMX_COLUMN_SUM_WIDE_ROWS = 1024;
int32_t omx_column_sum(omx_ctx* ctx, const float* partial, float* out, uint64_t blocks, uint64_t dim,
                       unsigned long long tag, float* scratch = nullptr, hipEvent_t stop = nullptr);
// RMSNorm with 16-byte accesses for row widths 256..2048 (rmsvec.hip). `add` (forward) and
// `add_in` / `gx16` (backward) are optional fused operands.
bool omx_rms_vec_eligible(uint64_t dim, std::initializer_list<const void*> ptrs);
int32_t omx_rms_forward_vec(omx_ctx* ctx, const void* x, int32_t x_dtype, const void* add, int32_t add_dtype,
                            const float* w, float* sum_out, void* y, int32_t y_dtype, uint64_t rows, uint64_t dim,
                            float eps, unsigned long long tag);
int32_t omx_rms_backward_vec(omx_ctx* ctx, const void* x, int32_t x_dtype, const float* w, const void* gy,
                             int32_t gy_dtype, const float* add_in, void* gx, int32_t gx_dtype, void* gx16, float* gw,
                             uint64_t rows, uint64_t dim, float eps, unsigned long long tag);
// Elementwise conversions on the context's stream (no fault reporting).
int32_t omx_convert(omx_ctx* ctx, const void* src, int32_t src_dtype, void* dst, int32_t dst_dtype, uint64_t n);

#define OMX_HIP(ctx, expr)                                   \
  do {                                                       \
    hipError_t e_ = (expr);                                  \
    if (e_ != hipSuccess) return omx_hip_fail(ctx, e_, #expr); \
  } while (0)

#define OMX_LAUNCH_CHECK(ctx, what)                               \
  do {                                                            \
    hipError_t e_ = hipGetLastError();                            \
    if (e_ != hipSuccess) return omx_hip_fail(ctx, e_, what);     \
  } while (0)

#define OMX_REQUIRE_CTX(ctx) \
  do {                       \
    if (!(ctx)) return OMX_BACKEND; \
  } while (0)

// ---- device helpers ----
typedef __hip_bfloat16 bf16_t;

__device__ __forceinline__ bool dev_finite(float x) {
  return (__float_as_uint(x) & 0x7fffffffu) < 0x7f800000u;
}

// Round to nearest even on the dropped 16 bits; NaN keeps sign and payload and
// sets the quiet bit (ojas-core/src/autocast.rs:70-96). The integer form of the rule:
__device__ __forceinline__ unsigned short dev_f32_to_bf16_bits_integer_rule(float v) {
  unsigned int b = __float_as_uint(v);
  if (v != v) return static_cast<unsigned short>((b >> 16) | 0x0040u);
  unsigned int round = 0x7fffu + ((b >> 16) & 1u);
  return static_cast<unsigned short>((b + round) >> 16);
}
// The conversion instruction (v_cvt_pk_bf16_f32) gives the bits of that rule on every one of the
// 2^32 f32 patterns, NaN payloads and denormals included (checked exhaustively on the device;
// tests/test_gpu_parity_ops.py holds the casts to the rule over every exponent and the special
// values), at one instruction per pair instead of seven per value.
__device__ __forceinline__ unsigned int dev_pack_bf16_pair(float lo, float hi) {
  typedef __bf16 omx_bf16x2 __attribute__((ext_vector_type(2)));
  typedef float omx_floatx2 __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(unsigned int, __builtin_convertvector(omx_floatx2{lo, hi}, omx_bf16x2));
}
__device__ __forceinline__ unsigned short dev_f32_to_bf16_bits(float v) {
  return static_cast<unsigned short>(dev_pack_bf16_pair(v, 0.0f) & 0xffffu);
}
__device__ __forceinline__ float dev_bf16_bits_to_f32(unsigned short b) {
  return __uint_as_float(static_cast<unsigned int>(b) << 16);
}
__device__ __forceinline__ float dev_round_bf16(float v) {
  return dev_bf16_bits_to_f32(dev_f32_to_bf16_bits(v));
}

// The low byte of a tag is the op (bits 0-6) and the fault kind (bit 7:
// 0 = non-finite value, 1 = index out of range).
__device__ __forceinline__ void dev_raise_fault(OmxFaultWord* fault, unsigned long long tag) {
  atomicOr(&fault->mask, 1ull << (tag & 0x3full));
  atomicMin(&fault->first, tag);
}
__device__ __forceinline__ void dev_raise_range(OmxFaultWord* fault, unsigned long long tag) {
  atomicOr(&fault->mask, 1ull << (tag & 0x3full));
  atomicMin(&fault->first, tag | 0x80ull);
}

// Loads element i of a tensor stored as f32 or bf16, widened exactly.
template <typename T>
__device__ __forceinline__ float dev_load(const T* p, size_t i);
template <>
__device__ __forceinline__ float dev_load<float>(const float* p, size_t i) {
  return p[i];
}
template <>
__device__ __forceinline__ float dev_load<unsigned short>(const unsigned short* p, size_t i) {
  return dev_bf16_bits_to_f32(p[i]);
}
template <typename T>
__device__ __forceinline__ void dev_store(T* p, size_t i, float v);
template <>
__device__ __forceinline__ void dev_store<float>(float* p, size_t i, float v) {
  p[i] = v;
}
template <>
__device__ __forceinline__ void dev_store<unsigned short>(unsigned short* p, size_t i, float v) {
  p[i] = dev_f32_to_bf16_bits(v);
}

// Four consecutive elements starting at element index i (a multiple of 4; the
// address must be 16-byte aligned for f32 and 8-byte aligned for bf16).
template <typename T>
__device__ __forceinline__ void dev_load4(const T* p, size_t i, float (&v)[4]) {
  if constexpr (sizeof(T) == 4) {
    const float4 q = *reinterpret_cast<const float4*>(p + i);
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
  } else {
    const uint2 q = *reinterpret_cast<const uint2*>(p + i);
    v[0] = __uint_as_float(q.x << 16); v[1] = __uint_as_float(q.x & 0xffff0000u);
    v[2] = __uint_as_float(q.y << 16); v[3] = __uint_as_float(q.y & 0xffff0000u);
  }
}
template <typename T>
__device__ __forceinline__ void dev_store4(T* p, size_t i, const float (&v)[4]) {
  if constexpr (sizeof(T) == 4) {
    *reinterpret_cast<float4*>(p + i) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
    uint2 q;
    q.x = dev_pack_bf16_pair(v[0], v[1]);
    q.y = dev_pack_bf16_pair(v[2], v[3]);
    *reinterpret_cast<uint2*>(p + i) = q;
  }
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// GELU in f32. The erf form is 0.5 x (1 + erf(x / sqrt 2)); the tanh form is
// x * sigmoid(2 sqrt(2/pi) (x + 0.044715 x^3)), which has no cancellation in
// the negative tail (ojas-core/src/gelu_tanh.rs:8-15).
__device__ __forceinline__ float dev_gelu_erf(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752f)); }
__device__ __forceinline__ float dev_gelu_erf_grad(float x) {
  float cdf = 0.5f * (1.0f + erff(x * 0.70710678118654752f));
  float pdf = 0.3989422804014327f * __expf(-0.5f * x * x);
  return cdf + x * pdf;
}
__device__ __forceinline__ void dev_sigmoid_pair(float u, float* s, float* slope) {
  float e = __expf(-fabsf(u));
  float denom = 1.0f + e;
  *s = u >= 0.0f ? 1.0f / denom : e / denom;
  *slope = e / (denom * denom);
}
__device__ __forceinline__ float dev_gelu_tanh(float x) {
  float u = 2.0f * 0.7978845608028654f * (x + 0.044715f * x * x * x);
  float s, slope;
  dev_sigmoid_pair(u, &s, &slope);
  return x * s;
}
__device__ __forceinline__ float dev_gelu_tanh_grad(float x) {
  float u = 2.0f * 0.7978845608028654f * (x + 0.044715f * x * x * x);
  float s, slope;
  dev_sigmoid_pair(u, &s, &slope);
  float du = 2.0f * 0.7978845608028654f * (1.0f + 3.0f * 0.044715f * x * x);
  return s + x * slope * du;
}

// The same four functions for values stored in bf16 (8 bits of mantissa): the exact forms above cost
// 40 to 60 instructions per element (erff, IEEE divisions) and made the products that apply them in
// their store pass half as long again. These take one hardware exp2, one hardware reciprocal
// (1 ulp) and a few fmas. erf: Abramowitz & Stegun 7.1.26, |error| <= 1.5e-7, evaluated as erfc so
// the negative tail x * Phi(x) has no cancellation; exp(-z^2) doubles as the density in the
// derivative.
// tail = Phi(-|x|) and e = exp(-x^2 / 2). With w = |x| sqrt(log2(e) / 2): e = exp2(-w^2), and the
// series' argument |x| / sqrt 2 is w / sqrt(log2 e), so its constant folds into the fma that feeds
// the reciprocal; the 1/2 of erfc / 2 is folded into the coefficients.
__device__ __forceinline__ void dev_normal_tail_fast(float x, float* tail, float* e) {
  const float w = fabsf(x) * 0.84932180028801904f;
  const float t = __builtin_amdgcn_rcpf(fmaf(0.27273748087922250f, w, 1.0f));
  *e = __builtin_amdgcn_exp2f(-(w * w));
  float poly = fmaf(t, 0.5307027145f, -0.7265760135f);
  poly = fmaf(t, poly, 0.7107068705f);
  poly = fmaf(t, poly, -0.142248368f);
  poly = fmaf(t, poly, 0.127414796f);
  *tail = (poly * t) * *e;
}
// x Phi(x) = max(x, 0) - |x| Phi(-|x|): no branch on the sign and no 1 - tail.
__device__ __forceinline__ float dev_gelu_erf_fast(float x) {
  float tail, e;
  dev_normal_tail_fast(x, &tail, &e);
  return fmaf(-fabsf(x), tail, fmaxf(x, 0.0f));
}
__device__ __forceinline__ float dev_gelu_erf_grad_fast(float x) {
  float tail, e;
  dev_normal_tail_fast(x, &tail, &e);
  const float cdf = x >= 0.0f ? 1.0f - tail : tail;
  return fmaf(x, 0.3989422804014327f * e, cdf);
}
__device__ __forceinline__ void dev_sigmoid_pair_fast(float u, float* s, float* slope) {
  const float e = __builtin_amdgcn_exp2f(fabsf(u) * -1.4426950408889634f);
  const float r = __builtin_amdgcn_rcpf(1.0f + e);
  *s = u >= 0.0f ? r : e * r;
  *slope = e * r * r;
}
// 2 sqrt(2/pi) (x + 0.044715 x^3) as x (c0 + c1 x^2).
__device__ __forceinline__ float dev_gelu_tanh_arg_fast(float x) {
  return x * fmaf(0.07135481627260025f, x * x, 1.5957691216057308f);
}
__device__ __forceinline__ float dev_gelu_tanh_fast(float x) {
  const float u = dev_gelu_tanh_arg_fast(x);
  float s, slope;
  dev_sigmoid_pair_fast(u, &s, &slope);
  return x * s;
}
__device__ __forceinline__ float dev_gelu_tanh_grad_fast(float x) {
  const float u = dev_gelu_tanh_arg_fast(x);
  float s, slope;
  dev_sigmoid_pair_fast(u, &s, &slope);
  const float du = fmaf(0.21406444881780074f, x * x, 1.5957691216057308f);
  return fmaf(x * slope, du, s);
}
// GELU of a value whose storage type is T: exact for f32, the fast forms for bf16.
template <typename T, bool TANH>
__device__ __forceinline__ float dev_gelu_of(float x) {
  if constexpr (sizeof(T) == 2) return TANH ? dev_gelu_tanh_fast(x) : dev_gelu_erf_fast(x);
  else return TANH ? dev_gelu_tanh(x) : dev_gelu_erf(x);
}
template <typename T, bool TANH>
__device__ __forceinline__ float dev_gelu_grad_of(float x) {
  if constexpr (sizeof(T) == 2) return TANH ? dev_gelu_tanh_grad_fast(x) : dev_gelu_erf_grad_fast(x);
  else return TANH ? dev_gelu_tanh_grad(x) : dev_gelu_erf_grad(x);
}

inline bool omx_valid_float_dtype(int32_t d) { return d == OMX_F32 || d == OMX_BF16; }
inline size_t omx_dtype_size(int32_t d) { return d == OMX_BF16 ? 2 : 4; }
