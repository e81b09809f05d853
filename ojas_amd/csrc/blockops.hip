// Ops that only the nanolab block uses: SiLU, elementwise product, half-split
// RoPE, the per-head sigmoid gate and the value-residual blend. All are
// bandwidth-bound: each tensor is read once and written once, 16 bytes per
// lane where the shape allows it. The gate's three small matrix products run
// on the library's GEMM.
//
// Reference semantics (CPU backend):
//   silu_*                     ojas-cpu/src/pointwise.rs:346-366,515-546
//   mul_*                      ojas-cpu/src/pointwise.rs:579-620,770-905
//   rope_half_split_*          ojas-cpu/src/norm.rs:271-347
//   per_head_sigmoid_gate_*    ojas-cpu/src/pointwise.rs:1395-1470,1678-1781,1853-1894
//   value_residual_blend_*     ojas-cpu/src/pointwise.rs:2031-2148
// Trait: ojas-core/src/backend.rs:1151-1163,1674-1686,1860-1920.
#include "omx_common.h"

namespace {

constexpr int BK_THREADS = 256;
constexpr int BK_PACKS = 4;  // packs per thread

// A pack is V consecutive elements: one 16-byte (f32) or 8-byte (bf16) access
// when V == 4, one element when V == 1.
template <typename T, int V>
__device__ __forceinline__ void load_pack(const T* __restrict__ p, size_t pack, float (&v)[V]) {
  if constexpr (V == 1) {
    v[0] = dev_load<T>(p, pack);
  } else if constexpr (sizeof(T) == 4) {
    float4 q = reinterpret_cast<const float4*>(p)[pack];
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
  } else {
    uint2 q = reinterpret_cast<const uint2*>(p)[pack];
    v[0] = __uint_as_float(q.x << 16); v[1] = __uint_as_float(q.x & 0xffff0000u);
    v[2] = __uint_as_float(q.y << 16); v[3] = __uint_as_float(q.y & 0xffff0000u);
  }
}
template <typename T, int V>
__device__ __forceinline__ void store_pack(T* __restrict__ p, size_t pack, const float (&v)[V]) {
  if constexpr (V == 1) {
    dev_store<T>(p, pack, v[0]);
  } else if constexpr (sizeof(T) == 4) {
    reinterpret_cast<float4*>(p)[pack] = make_float4(v[0], v[1], v[2], v[3]);
  } else {
    uint2 q;
    q.x = dev_pack_bf16_pair(v[0], v[1]);
    q.y = dev_pack_bf16_pair(v[2], v[3]);
    reinterpret_cast<uint2*>(p)[pack] = q;
  }
}

inline dim3 pack_grid(uint64_t packs) {
  uint64_t per_block = static_cast<uint64_t>(BK_THREADS) * BK_PACKS;
  uint64_t blocks = (packs + per_block - 1) / per_block;
  return dim3(static_cast<unsigned>(blocks > 0 ? blocks : 1));
}
#define PACK_LOOP(p, packs)                                                                          \
  for (size_t p = static_cast<size_t>(blockIdx.x) * (BK_THREADS * BK_PACKS) + threadIdx.x,           \
              end_ = min(static_cast<size_t>(packs), (static_cast<size_t>(blockIdx.x) + 1) * (BK_THREADS * BK_PACKS)); \
       p < end_; p += BK_THREADS)

// Whether every pointer allows 4-element packs of `esz`-byte elements.
inline bool packs_of_four(uint64_t n, size_t esz, std::initializer_list<const void*> ptrs) {
  if (n % 4 != 0) return false;
  uintptr_t mask = esz * 4 - 1, bits = 0;
  for (const void* p : ptrs) bits |= reinterpret_cast<uintptr_t>(p);
  return (bits & mask) == 0;
}

// sigmoid(u) and 1 - sigmoid(u), both without cancellation.
__device__ __forceinline__ void sigmoid_pair(float u, float* s, float* rest) {
  float e = __expf(-fabsf(u));
  float inv = 1.0f / (1.0f + e);
  float big = inv, small = e * inv;
  *s = u >= 0.0f ? big : small;
  *rest = u >= 0.0f ? small : big;
}

// ------------------------------------------------------------ silu and mul
template <typename T, int V>
__global__ __launch_bounds__(BK_THREADS) void silu_fwd_kernel(const T* __restrict__ x, T* __restrict__ y, size_t packs,
                                                              OmxFaultWord* fault, unsigned long long tag) {
  bool bad = false;
  PACK_LOOP(p, packs) {
    float v[V], r[V];
    load_pack<T, V>(x, p, v);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      float s, rest;
      sigmoid_pair(v[j], &s, &rest);
      r[j] = v[j] * s;
      bad |= !dev_finite(r[j]);
    }
    store_pack<T, V>(y, p, r);
  }
  if (bad) dev_raise_fault(fault, tag);
}
template <typename T, int V>
__global__ __launch_bounds__(BK_THREADS) void silu_bwd_kernel(const T* __restrict__ x, const T* __restrict__ gy,
                                                              T* __restrict__ gx, size_t packs, OmxFaultWord* fault,
                                                              unsigned long long tag) {
  bool bad = false;
  PACK_LOOP(p, packs) {
    float v[V], g[V], r[V];
    load_pack<T, V>(x, p, v);
    load_pack<T, V>(gy, p, g);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      float s, rest;
      sigmoid_pair(v[j], &s, &rest);
      r[j] = g[j] * s * (1.0f + v[j] * rest);
      bad |= !dev_finite(r[j]);
    }
    store_pack<T, V>(gx, p, r);
  }
  if (bad) dev_raise_fault(fault, tag);
}
template <typename T, int V>
__global__ __launch_bounds__(BK_THREADS) void mul_fwd_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                             T* __restrict__ out, size_t packs, OmxFaultWord* fault,
                                                             unsigned long long tag) {
  bool bad = false;
  PACK_LOOP(p, packs) {
    float x[V], y[V], r[V];
    load_pack<T, V>(a, p, x);
    load_pack<T, V>(b, p, y);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      r[j] = x[j] * y[j];
      bad |= !dev_finite(r[j]);
    }
    store_pack<T, V>(out, p, r);
  }
  if (bad) dev_raise_fault(fault, tag);
}
template <typename T, int V>
__global__ __launch_bounds__(BK_THREADS) void mul_bwd_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                             const T* __restrict__ gy, T* __restrict__ ga,
                                                             T* __restrict__ gb, size_t packs, OmxFaultWord* fault,
                                                             unsigned long long tag) {
  bool bad = false;
  PACK_LOOP(p, packs) {
    float x[V], y[V], g[V], ra[V], rb[V];
    load_pack<T, V>(a, p, x);
    load_pack<T, V>(b, p, y);
    load_pack<T, V>(gy, p, g);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      ra[j] = g[j] * y[j];
      rb[j] = g[j] * x[j];
      bad |= !(dev_finite(ra[j]) && dev_finite(rb[j]));
    }
    store_pack<T, V>(ga, p, ra);
    store_pack<T, V>(gb, p, rb);
  }
  if (bad) dev_raise_fault(fault, tag);
}

// ------------------------------------------------------------------- RoPE
// One thread owns V columns of the first half of a row and the matching V of
// the second half. y = x cos + cat(-x2, x1) sin; the backward is its
// transpose: gx1 = g1 c1 + g2 s2, gx2 = -g1 s1 + g2 c2.
template <typename T, int V, bool BACKWARD>
__global__ __launch_bounds__(BK_THREADS) void rope_kernel(const T* __restrict__ x, const float* __restrict__ cos,
                                                          const float* __restrict__ sin, T* __restrict__ y,
                                                          size_t rows, int dim, size_t time, size_t heads,
                                                          OmxFaultWord* fault, unsigned long long tag) {
  const int half_packs = dim / 2 / V;
  const size_t row_packs = static_cast<size_t>(half_packs) * 2;
  const size_t packs = rows * half_packs;
  bool bad = false;
  PACK_LOOP(p, packs) {
    size_t row = p / half_packs;
    int c = static_cast<int>(p % half_packs);
    size_t trow = heads ? (row / heads) % time : row;
    float a[V], b[V], c1[V], s1[V], c2[V], s2[V], lo[V], hi[V];
    load_pack<T, V>(x, row * row_packs + c, a);
    load_pack<T, V>(x, row * row_packs + half_packs + c, b);
    load_pack<float, V>(cos, trow * row_packs + c, c1);
    load_pack<float, V>(sin, trow * row_packs + c, s1);
    load_pack<float, V>(cos, trow * row_packs + half_packs + c, c2);
    load_pack<float, V>(sin, trow * row_packs + half_packs + c, s2);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      if (BACKWARD) {
        lo[j] = a[j] * c1[j] + b[j] * s2[j];
        hi[j] = -a[j] * s1[j] + b[j] * c2[j];
      } else {
        lo[j] = a[j] * c1[j] + (-b[j]) * s1[j];
        hi[j] = b[j] * c2[j] + a[j] * s2[j];
      }
      bad |= !(dev_finite(lo[j]) && dev_finite(hi[j]));
    }
    store_pack<T, V>(y, row * row_packs + c, lo);
    store_pack<T, V>(y, row * row_packs + half_packs + c, hi);
  }
  if (bad) dev_raise_fault(fault, tag);
}

// ------------------------------------------------------------------- gate
// z[r, h] (the product input . weight^T) becomes sigmoid(z + bias[h]) in place.
__global__ __launch_bounds__(BK_THREADS) void gate_sigmoid_kernel(float* __restrict__ z, const float* __restrict__ bias,
                                                                  size_t n, int heads, OmxFaultWord* fault,
                                                                  unsigned long long tag) {
  bool bad = false;
  PACK_LOOP(i, n) {
    float u = z[i] + bias[i % heads];
    bad |= !dev_finite(u);
    float s, rest;
    sigmoid_pair(u, &s, &rest);
    z[i] = s;
  }
  if (bad) dev_raise_fault(fault, tag);
}
// y[r, h, :] = attn[r, h, :] * gates[r, h]; head_dim is a multiple of V.
template <typename TA, typename TY, int V>
__global__ __launch_bounds__(BK_THREADS) void gate_apply_kernel(const TA* __restrict__ attn,
                                                                const float* __restrict__ gates, TY* __restrict__ y,
                                                                size_t packs, int head_packs, OmxFaultWord* fault,
                                                                unsigned long long tag) {
  bool bad = false;
  PACK_LOOP(p, packs) {
    float a[V], r[V];
    load_pack<TA, V>(attn, p, a);
    float g = gates[p / head_packs];
#pragma unroll
    for (int j = 0; j < V; ++j) {
      r[j] = a[j] * g;
      bad |= !dev_finite(r[j]);
    }
    store_pack<TY, V>(y, p, r);
  }
  if (bad) dev_raise_fault(fault, tag);
}

// Backward over (row, head) items. A group of `group` lanes (a power of two,
// at most 64) owns one item at a time: g_attn = gy * g, and the group's sum of
// gy * attn gives gz = dot * g * (1 - g). A block covers `block_rows` whole
// rows; once its gz values sit in LDS, thread h adds column h in row order,
// so the bias gradient needs no atomics.
template <typename TA, typename TG, typename TO, typename TZ, int V>
__global__ __launch_bounds__(BK_THREADS) void gate_bwd_kernel(const TA* __restrict__ attn, const TG* __restrict__ gy,
                                                              const float* __restrict__ gates, TO* __restrict__ g_attn,
                                                              TZ* __restrict__ gz, float* __restrict__ partial,
                                                              size_t rows, int heads, int head_packs, int group,
                                                              int block_rows, OmxFaultWord* fault,
                                                              unsigned long long tag) {
  extern __shared__ float lds_gz[];  // [block_rows * heads]
  const int groups = BK_THREADS / group;
  const int sub = threadIdx.x / group, lane = threadIdx.x % group;
  const size_t first_row = static_cast<size_t>(blockIdx.x) * block_rows;
  const int live_rows = static_cast<int>(min(static_cast<size_t>(block_rows), rows - first_row));
  const int items = live_rows * heads;
  bool bad = false;
  for (int it = sub; it < items; it += groups) {
    const size_t item = first_row * heads + it;
    const float g = gates[item];
    float dot = 0.0f;
    for (int c = lane; c < head_packs; c += group) {
      float a[V], d[V], r[V];
      load_pack<TA, V>(attn, item * head_packs + c, a);
      load_pack<TG, V>(gy, item * head_packs + c, d);
#pragma unroll
      for (int j = 0; j < V; ++j) {
        r[j] = d[j] * g;
        dot += d[j] * a[j];
        bad |= !dev_finite(r[j]);
      }
      store_pack<TO, V>(g_attn, item * head_packs + c, r);
    }
    for (int off = group >> 1; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
    float z = dot * g * (1.0f - g);
    if (lane == 0) {
      bad |= !dev_finite(z);
      lds_gz[it] = z;
      dev_store<TZ>(gz, item, z);
    }
  }
  __syncthreads();
  for (int h = threadIdx.x; h < heads; h += BK_THREADS) {
    float s = 0.0f;
    for (int r = 0; r < live_rows; ++r) s += lds_gz[r * heads + h];
    partial[static_cast<size_t>(blockIdx.x) * heads + h] = s;
  }
  if (bad) dev_raise_fault(fault, tag);
}

// --------------------------------------------------- value-residual blend
template <typename T, int V>
__global__ __launch_bounds__(BK_THREADS) void vres_fwd_kernel(const T* __restrict__ v, const T* __restrict__ v0,
                                                              const float* __restrict__ lambda, T* __restrict__ out,
                                                              size_t packs, OmxFaultWord* fault,
                                                              unsigned long long tag) {
  float s, rest;
  sigmoid_pair(*lambda, &s, &rest);
  bool bad = !dev_finite(s);
  PACK_LOOP(p, packs) {
    float a[V], b[V], r[V];
    load_pack<T, V>(v, p, a);
    load_pack<T, V>(v0, p, b);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      r[j] = rest * a[j] + s * b[j];
      bad |= !dev_finite(r[j]);
    }
    store_pack<T, V>(out, p, r);
  }
  if (bad) dev_raise_fault(fault, tag);
}
// gv = (1 - s) gy, gv0 = s gy, and this block's sum of (v0 - v) gy.
template <typename T, int V>
__global__ __launch_bounds__(BK_THREADS) void vres_bwd_kernel(const T* __restrict__ v, const T* __restrict__ v0,
                                                              const T* __restrict__ gy,
                                                              const float* __restrict__ lambda, T* __restrict__ gv,
                                                              T* __restrict__ gv0, float* __restrict__ partial,
                                                              size_t packs, OmxFaultWord* fault,
                                                              unsigned long long tag) {
  __shared__ float red[BK_THREADS / 64];
  float s, rest;
  sigmoid_pair(*lambda, &s, &rest);
  bool bad = !dev_finite(s);
  float acc = 0.0f;
  PACK_LOOP(p, packs) {
    float a[V], b[V], g[V], ra[V], rb[V];
    load_pack<T, V>(v, p, a);
    load_pack<T, V>(v0, p, b);
    load_pack<T, V>(gy, p, g);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      ra[j] = rest * g[j];
      rb[j] = s * g[j];
      acc += (b[j] - a[j]) * g[j];
      bad |= !(dev_finite(ra[j]) && dev_finite(rb[j]));
    }
    store_pack<T, V>(gv, p, ra);
    store_pack<T, V>(gv0, p, rb);
  }
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) partial[blockIdx.x] = ((red[0] + red[1]) + red[2]) + red[3];
  if (bad) dev_raise_fault(fault, tag);
}
// One block: thread t adds partials t, t + 256, ... in order, then a fixed
// tree over the 256 sums; the result is scaled by s (1 - s).
__global__ __launch_bounds__(BK_THREADS) void vres_lambda_kernel(const float* __restrict__ partial, int blocks,
                                                                 const float* __restrict__ lambda,
                                                                 float* __restrict__ g_lambda, OmxFaultWord* fault,
                                                                 unsigned long long tag) {
  __shared__ float red[BK_THREADS];
  float acc = 0.0f;
  for (int b = threadIdx.x; b < blocks; b += BK_THREADS) acc += partial[b];
  red[threadIdx.x] = acc;
  __syncthreads();
  for (int w = BK_THREADS / 2; w > 0; w >>= 1) {
    if (threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    float s, rest;
    sigmoid_pair(*lambda, &s, &rest);
    float r = red[0] * s * rest;
    *g_lambda = r;
    if (!dev_finite(r)) dev_raise_fault(fault, tag);
  }
}

int32_t check_unary(omx_ctx* ctx, const char* op, int32_t dtype, uint64_t n, std::initializer_list<const void*> ptrs) {
  for (const void* p : ptrs)
    if (!p) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  if (n == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  return OMX_OK;
}

// Launches KERNEL<T, V> with T from `dtype` and V = 4 when `vec`.
#define LAUNCH_TV(KERNEL, dtype, vec, grid, ...)                                                        \
  do {                                                                                                  \
    if ((dtype) == OMX_F32) {                                                                           \
      typedef float T_;                                                                                 \
      if (vec) hipLaunchKernelGGL((KERNEL<T_, 4>), grid, dim3(BK_THREADS), 0, ctx->stream, __VA_ARGS__); \
      else hipLaunchKernelGGL((KERNEL<T_, 1>), grid, dim3(BK_THREADS), 0, ctx->stream, __VA_ARGS__);    \
    } else {                                                                                            \
      typedef unsigned short T_;                                                                        \
      if (vec) hipLaunchKernelGGL((KERNEL<T_, 4>), grid, dim3(BK_THREADS), 0, ctx->stream, __VA_ARGS__); \
      else hipLaunchKernelGGL((KERNEL<T_, 1>), grid, dim3(BK_THREADS), 0, ctx->stream, __VA_ARGS__);    \
    }                                                                                                   \
  } while (0)

template <bool BACKWARD>
int32_t launch_rope(omx_ctx* ctx, const char* op, uint32_t fault_op, const void* x, const void* cos, const void* sin,
                    void* y, int32_t dtype, uint64_t rows, uint64_t dim, uint64_t time, uint64_t heads) {
  int32_t rc = check_unary(ctx, op, dtype, rows * dim, {x, cos, sin, y});
  if (rc != OMX_OK) return rc;
  if (dim % 2 != 0) return omx_fail(ctx, OMX_SHAPE, "%s: rope last dim %llu is odd", op, (unsigned long long)dim);
  if (dim > (1u << 30)) return omx_fail(ctx, OMX_SHAPE, "%s: rope last dim too large", op);
  if (heads != 0 && (time == 0 || rows % (time * heads) != 0))
    return omx_fail(ctx, OMX_SHAPE, "%s: cos/sin [%llu, %llu] does not broadcast onto %llu rows of %llu heads", op,
                    (unsigned long long)time, (unsigned long long)dim, (unsigned long long)rows,
                    (unsigned long long)heads);
  const uint64_t half = dim / 2;
  const bool vec = half % 4 == 0 && packs_of_four(4, omx_dtype_size(dtype), {x, y}) && packs_of_four(4, 4, {cos, sin});
  const int v = vec ? 4 : 1;
  unsigned long long tag = omx_tag(ctx, fault_op);
  dim3 grid = pack_grid(rows * (half / v));
#define ROPE_K(T_, V_)                                                                                           \
  hipLaunchKernelGGL((rope_kernel<T_, V_, BACKWARD>), grid, dim3(BK_THREADS), 0, ctx->stream,                    \
                     static_cast<const T_*>(x), static_cast<const float*>(cos), static_cast<const float*>(sin), \
                     static_cast<T_*>(y), static_cast<size_t>(rows), static_cast<int>(dim),                      \
                     static_cast<size_t>(time), static_cast<size_t>(heads), ctx->fault, tag)
  if (dtype == OMX_F32) {
    if (vec) ROPE_K(float, 4);
    else ROPE_K(float, 1);
  } else {
    if (vec) ROPE_K(unsigned short, 4);
    else ROPE_K(unsigned short, 1);
  }
#undef ROPE_K
  OMX_LAUNCH_CHECK(ctx, "rope_kernel");
  return OMX_OK;
}

inline uint64_t round_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

int32_t check_gate(omx_ctx* ctx, const char* op, int32_t operand_dtype, std::initializer_list<int32_t> dtypes,
                   uint64_t rows, uint64_t d_model, uint64_t heads, uint64_t head_dim) {
  if (!omx_valid_float_dtype(operand_dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  for (int32_t d : dtypes)
    if (!omx_valid_float_dtype(d)) return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  if (rows == 0 || d_model == 0 || heads == 0 || head_dim == 0)
    return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (heads > (1u << 16) || head_dim > (1u << 24)) return omx_fail(ctx, OMX_SHAPE, "%s: head axes too large", op);
  return OMX_OK;
}

// gates[rows, heads] = sigmoid(input . weight^T + bias) into `gates`.
int32_t compute_gates(omx_ctx* ctx, uint32_t fault_op, const void* input, const void* weight, int32_t operand_dtype,
                      const void* bias, float* gates, uint64_t rows, uint64_t d_model, uint64_t heads) {
  int32_t rc = omx_gemm_impl(ctx, fault_op, input, d_model, 1, weight, 1, d_model, operand_dtype, gates, OMX_F32, heads,
                             rows, d_model, heads, 0);
  if (rc != OMX_OK) return rc;
  hipLaunchKernelGGL(gate_sigmoid_kernel, pack_grid(rows * heads), dim3(BK_THREADS), 0, ctx->stream, gates,
                     static_cast<const float*>(bias), static_cast<size_t>(rows * heads), static_cast<int>(heads),
                     ctx->fault, omx_tag(ctx, fault_op));
  OMX_LAUNCH_CHECK(ctx, "gate_sigmoid_kernel");
  return OMX_OK;
}

// out[r, c] = add[r, c] + sum_h gz[r, h] w[h, c]: the gate's input gradient (a product with a reduction
// of `heads` terms) joined to another gradient of the same input. A thread owns four columns and
// keeps their weights in registers as bf16 pairs of consecutive heads; a wave reads a row's gz once
// (lane p holds heads 2p and 2p + 1, packed) and hands the pairs round through readlane, so a
// column takes heads / 2 v_dot2c_f32_bf16 (bf16 x bf16 products are exact in f32; the sum runs
// pair by pair in f32). The block is d / 4 threads rounded up to whole waves.
constexpr int GATE_JOIN_HEADS = 16;
__device__ __forceinline__ float gate_join_dot(unsigned int a, unsigned int b, float acc) {
  typedef __bf16 bf16_pair __attribute__((ext_vector_type(2)));
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16_pair, a), __builtin_bit_cast(bf16_pair, b), acc, false);
}
template <typename TA>
__global__ __launch_bounds__(256) void gate_input_grad_add_kernel(const unsigned short* __restrict__ gz,
                                                                  const unsigned short* __restrict__ w,
                                                                  const TA* __restrict__ add, float* __restrict__ out,
                                                                  size_t rows, int d, int heads, int rows_per_block,
                                                                  OmxFaultWord* fault, unsigned long long tag) {
  constexpr int PAIRS = GATE_JOIN_HEADS / 2;
  const int c = static_cast<int>(threadIdx.x) * 4, lane = threadIdx.x & 63;
  const bool live = c < d;
  const int pairs = (heads + 1) / 2;
  unsigned int wp[PAIRS][4];  // (w[2p][c + e], w[2p + 1][c + e]) as a bf16 pair
#pragma unroll
  for (int p = 0; p < PAIRS; ++p) {
#pragma unroll
    for (int e = 0; e < 4; ++e) wp[p][e] = 0u;
    if (live && p < pairs) {
      const uint2 lo = *reinterpret_cast<const uint2*>(w + static_cast<size_t>(2 * p) * d + c);
      uint2 hi = make_uint2(0u, 0u);
      if (2 * p + 1 < heads) hi = *reinterpret_cast<const uint2*>(w + static_cast<size_t>(2 * p + 1) * d + c);
      wp[p][0] = (lo.x & 0xffffu) | (hi.x << 16);
      wp[p][1] = (lo.x >> 16) | (hi.x & 0xffff0000u);
      wp[p][2] = (lo.y & 0xffffu) | (hi.y << 16);
      wp[p][3] = (lo.y >> 16) | (hi.y & 0xffff0000u);
    }
  }
  const size_t r0 = static_cast<size_t>(blockIdx.x) * rows_per_block;
  const size_t r1 = r0 + rows_per_block < rows ? r0 + rows_per_block : rows;
  bool bad = false;
  constexpr int G = 4;  // rows whose loads are in flight together
  for (size_t rg = r0; rg < r1; rg += G) {
    unsigned int zv[G];
    float a[G][4];
#pragma unroll
    for (int i = 0; i < G; ++i) {
      const size_t r = rg + i < r1 ? rg + i : r1 - 1;
      const unsigned short* zr = gz + r * heads;
      zv[i] = 0u;
      if (2 * lane < heads) zv[i] = zr[2 * lane];
      if (2 * lane + 1 < heads) zv[i] |= static_cast<unsigned int>(zr[2 * lane + 1]) << 16;
#pragma unroll
      for (int e = 0; e < 4; ++e) a[i][e] = 0.0f;
      if (live) dev_load4<TA>(add + r * d, c, a[i]);
    }
#pragma unroll
    for (int i = 0; i < G; ++i) {
      float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int p = 0; p < PAIRS; ++p) {
        if (p < pairs) {
          const unsigned int z = static_cast<unsigned int>(__builtin_amdgcn_readlane(static_cast<int>(zv[i]), p));
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[e] = gate_join_dot(z, wp[p][e], acc[e]);
        }
      }
      if (live && rg + i < r1) {
        float4 o = make_float4(a[i][0] + acc[0], a[i][1] + acc[1], a[i][2] + acc[2], a[i][3] + acc[3]);
        bad |= !(dev_finite(o.x) && dev_finite(o.y) && dev_finite(o.z) && dev_finite(o.w));
        *reinterpret_cast<float4*>(out + (rg + i) * d + c) = o;
      }
    }
  }
  if (bad) dev_raise_fault(fault, tag);
}

}  // namespace

extern "C" {

int32_t omx_silu_forward(omx_ctx* ctx, const void* x, void* y, int32_t dtype, uint64_t n) {
  OMX_REQUIRE_CTX(ctx);
  int32_t rc = check_unary(ctx, "silu_forward", dtype, n, {x, y});
  if (rc != OMX_OK) return rc;
  const bool vec = packs_of_four(n, omx_dtype_size(dtype), {x, y});
  const size_t packs = vec ? n / 4 : n;
  unsigned long long tag = omx_tag(ctx, F_SILU_FORWARD);
  LAUNCH_TV(silu_fwd_kernel, dtype, vec, pack_grid(packs), static_cast<const T_*>(x), static_cast<T_*>(y), packs,
            ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "silu_fwd_kernel");
  return OMX_OK;
}

int32_t omx_silu_backward(omx_ctx* ctx, const void* x, const void* gy, void* gx, int32_t dtype, uint64_t n) {
  OMX_REQUIRE_CTX(ctx);
  int32_t rc = check_unary(ctx, "silu_backward", dtype, n, {x, gy, gx});
  if (rc != OMX_OK) return rc;
  const bool vec = packs_of_four(n, omx_dtype_size(dtype), {x, gy, gx});
  const size_t packs = vec ? n / 4 : n;
  unsigned long long tag = omx_tag(ctx, F_SILU_BACKWARD);
  LAUNCH_TV(silu_bwd_kernel, dtype, vec, pack_grid(packs), static_cast<const T_*>(x), static_cast<const T_*>(gy),
            static_cast<T_*>(gx), packs, ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "silu_bwd_kernel");
  return OMX_OK;
}

int32_t omx_mul_forward(omx_ctx* ctx, const void* a, const void* b, void* out, int32_t dtype, uint64_t n) {
  OMX_REQUIRE_CTX(ctx);
  int32_t rc = check_unary(ctx, "mul_forward", dtype, n, {a, b, out});
  if (rc != OMX_OK) return rc;
  const bool vec = packs_of_four(n, omx_dtype_size(dtype), {a, b, out});
  const size_t packs = vec ? n / 4 : n;
  unsigned long long tag = omx_tag(ctx, F_MUL_FORWARD);
  LAUNCH_TV(mul_fwd_kernel, dtype, vec, pack_grid(packs), static_cast<const T_*>(a), static_cast<const T_*>(b),
            static_cast<T_*>(out), packs, ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "mul_fwd_kernel");
  return OMX_OK;
}

int32_t omx_mul_backward(omx_ctx* ctx, const void* a, const void* b, const void* gy, void* ga, void* gb, int32_t dtype,
                         uint64_t n) {
  OMX_REQUIRE_CTX(ctx);
  int32_t rc = check_unary(ctx, "mul_backward", dtype, n, {a, b, gy, ga, gb});
  if (rc != OMX_OK) return rc;
  const bool vec = packs_of_four(n, omx_dtype_size(dtype), {a, b, gy, ga, gb});
  const size_t packs = vec ? n / 4 : n;
  unsigned long long tag = omx_tag(ctx, F_MUL_BACKWARD);
  LAUNCH_TV(mul_bwd_kernel, dtype, vec, pack_grid(packs), static_cast<const T_*>(a), static_cast<const T_*>(b),
            static_cast<const T_*>(gy), static_cast<T_*>(ga), static_cast<T_*>(gb), packs, ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "mul_bwd_kernel");
  return OMX_OK;
}

int32_t omx_rope_half_split_forward(omx_ctx* ctx, const void* x, const void* cos, const void* sin, void* y,
                                    int32_t dtype, uint64_t rows, uint64_t dim, uint64_t time, uint64_t heads) {
  OMX_REQUIRE_CTX(ctx);
  return launch_rope<false>(ctx, "rope_half_split_forward", F_ROPE_FORWARD, x, cos, sin, y, dtype, rows, dim, time,
                            heads);
}
int32_t omx_rope_half_split_backward(omx_ctx* ctx, const void* gy, const void* cos, const void* sin, void* gx,
                                     int32_t dtype, uint64_t rows, uint64_t dim, uint64_t time, uint64_t heads) {
  OMX_REQUIRE_CTX(ctx);
  return launch_rope<true>(ctx, "rope_half_split_backward", F_ROPE_BACKWARD, gy, cos, sin, gx, dtype, rows, dim, time,
                           heads);
}

int32_t omx_per_head_sigmoid_gate_forward(omx_ctx* ctx, const void* input, const void* weight, int32_t operand_dtype,
                                          const void* bias, const void* attn, int32_t attn_dtype, void* y,
                                          int32_t y_dtype, void* gates_out, uint64_t rows, uint64_t d_model,
                                          uint64_t heads, uint64_t head_dim) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "per_head_sigmoid_gate_forward";
  if (!input || !weight || !bias || !attn || !y) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  int32_t rc = check_gate(ctx, op, operand_dtype, {attn_dtype, y_dtype}, rows, d_model, heads, head_dim);
  if (rc != OMX_OK) return rc;
  float* gates = static_cast<float*>(gates_out);
  if (!gates) {
    void* ws = nullptr;
    rc = omx_workspace(ctx, rows * heads * sizeof(float), &ws);
    if (rc != OMX_OK) return rc;
    gates = static_cast<float*>(ws);
  }
  rc = compute_gates(ctx, F_GATE_FORWARD, input, weight, operand_dtype, bias, gates, rows, d_model, heads);
  if (rc != OMX_OK) return rc;
  const bool vec = head_dim % 4 == 0 && packs_of_four(4, omx_dtype_size(attn_dtype), {attn}) &&
                   packs_of_four(4, omx_dtype_size(y_dtype), {y});
  const int v = vec ? 4 : 1;
  const size_t packs = rows * heads * (head_dim / v);
  const int head_packs = static_cast<int>(head_dim / v);
  unsigned long long tag = omx_tag(ctx, F_GATE_FORWARD);
  dim3 grid = pack_grid(packs);
#define GATE_APPLY(TA, TY, V_)                                                                                    \
  hipLaunchKernelGGL((gate_apply_kernel<TA, TY, V_>), grid, dim3(BK_THREADS), 0, ctx->stream,                     \
                     static_cast<const TA*>(attn), gates, static_cast<TY*>(y), packs, head_packs, ctx->fault, tag)
  typedef unsigned short h16;
  const int key = (attn_dtype == OMX_BF16 ? 2 : 0) | (y_dtype == OMX_BF16 ? 1 : 0);
  if (vec) {
    switch (key) {
      case 0: GATE_APPLY(float, float, 4); break;
      case 1: GATE_APPLY(float, h16, 4); break;
      case 2: GATE_APPLY(h16, float, 4); break;
      default: GATE_APPLY(h16, h16, 4); break;
    }
  } else {
    switch (key) {
      case 0: GATE_APPLY(float, float, 1); break;
      case 1: GATE_APPLY(float, h16, 1); break;
      case 2: GATE_APPLY(h16, float, 1); break;
      default: GATE_APPLY(h16, h16, 1); break;
    }
  }
#undef GATE_APPLY
  OMX_LAUNCH_CHECK(ctx, "gate_apply_kernel");
  return OMX_OK;
}

// The backward of the gate. `g_weight` may be null (the weight gradient is then left to the caller)
// and `gz_out` may be null (gz then lives in the workspace only).
static int32_t gate_backward_impl(omx_ctx* ctx, const char* op, const void* input, const void* weight,
                                  int32_t operand_dtype, const void* bias, const void* attn, int32_t attn_dtype,
                                  const void* gy, int32_t gy_dtype, const void* gates_saved, void* g_input,
                                  int32_t g_input_dtype, void* g_weight, void* gz_out, void* g_bias, void* g_attn,
                                  int32_t g_attn_dtype, uint64_t rows, uint64_t d_model, uint64_t heads,
                                  uint64_t head_dim) {
  OMX_REQUIRE_CTX(ctx);
  // The deferred form may leave the input gradient to the caller as well (it has gz for it).
  if (!input || !weight || !bias || !attn || !gy || (!g_input && !gz_out) || !g_bias || !g_attn || (!g_weight && !gz_out))
    return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  int32_t rc = check_gate(ctx, op, operand_dtype, {attn_dtype, gy_dtype, g_input_dtype, g_attn_dtype}, rows, d_model,
                          heads, head_dim);
  if (rc != OMX_OK) return rc;
  if (attn_dtype != gy_dtype)
    return omx_fail(ctx, OMX_DTYPE, "%s: attn and grad_output must share a dtype", op);

  // Workspace: [gates f32][gz in the operand dtype][per-block bias partials][two-stage sum scratch].
  const int block_rows = 16;
  const uint64_t blocks = (rows + block_rows - 1) / block_rows;
  const uint64_t items = rows * heads;
  const uint64_t gates_bytes = round_up(items * sizeof(float), 256);
  const uint64_t gz_bytes = round_up(items * omx_dtype_size(operand_dtype), 256);
  const uint64_t partial_bytes = round_up(blocks * heads * sizeof(float), 256);
  const uint64_t stage_bytes = OMX_COLUMN_SUM_GROUPS * heads * sizeof(float);
  const size_t lds_bytes = static_cast<size_t>(block_rows) * heads * sizeof(float);
  if (lds_bytes > 64 * 1024) return omx_fail(ctx, OMX_UNSUPPORTED, "%s: %llu heads above 1024", op, (unsigned long long)heads);
  void* ws = nullptr;
  rc = omx_workspace(ctx, gates_bytes + gz_bytes + partial_bytes + stage_bytes, &ws);
  if (rc != OMX_OK) return rc;
  char* base = static_cast<char*>(ws);
  const float* gates = static_cast<const float*>(gates_saved);
  if (!gates) {
    float* fresh = reinterpret_cast<float*>(base);
    rc = compute_gates(ctx, F_GATE_BACKWARD, input, weight, operand_dtype, bias, fresh, rows, d_model, heads);
    if (rc != OMX_OK) return rc;
    gates = fresh;
  }
  void* gz = gz_out ? gz_out : static_cast<void*>(base + gates_bytes);
  float* partial = reinterpret_cast<float*>(base + gates_bytes + gz_bytes);
  float* stage = reinterpret_cast<float*>(base + gates_bytes + gz_bytes + partial_bytes);

  const bool vec = head_dim % 4 == 0 && packs_of_four(4, omx_dtype_size(attn_dtype), {attn, gy}) &&
                   packs_of_four(4, omx_dtype_size(g_attn_dtype), {g_attn});
  const int v = vec ? 4 : 1;
  const int head_packs = static_cast<int>(head_dim / v);
  int group = 1;
  while (group < 64 && group < head_packs) group <<= 1;
  unsigned long long tag = omx_tag(ctx, F_GATE_BACKWARD);
  dim3 grid(static_cast<unsigned>(blocks));
#define GATE_BWD(TA, TO, TZ, V_)                                                                                 \
  hipLaunchKernelGGL((gate_bwd_kernel<TA, TA, TO, TZ, V_>), grid, dim3(BK_THREADS), lds_bytes, ctx->stream,      \
                     static_cast<const TA*>(attn), static_cast<const TA*>(gy), gates, static_cast<TO*>(g_attn),  \
                     static_cast<TZ*>(gz), partial, static_cast<size_t>(rows), static_cast<int>(heads),          \
                     head_packs, group, block_rows, ctx->fault, tag)
#define GATE_BWD_V(TA, TO, TZ)      \
  do {                              \
    if (vec) GATE_BWD(TA, TO, TZ, 4); \
    else GATE_BWD(TA, TO, TZ, 1);   \
  } while (0)
  typedef unsigned short h16;
  const int key = (attn_dtype == OMX_BF16 ? 4 : 0) | (g_attn_dtype == OMX_BF16 ? 2 : 0) |
                  (operand_dtype == OMX_BF16 ? 1 : 0);
  switch (key) {
    case 0: GATE_BWD_V(float, float, float); break;
    case 1: GATE_BWD_V(float, float, h16); break;
    case 2: GATE_BWD_V(float, h16, float); break;
    case 3: GATE_BWD_V(float, h16, h16); break;
    case 4: GATE_BWD_V(h16, float, float); break;
    case 5: GATE_BWD_V(h16, float, h16); break;
    case 6: GATE_BWD_V(h16, h16, float); break;
    default: GATE_BWD_V(h16, h16, h16); break;
  }
#undef GATE_BWD_V
#undef GATE_BWD
  OMX_LAUNCH_CHECK(ctx, "gate_bwd_kernel");
  rc = omx_column_sum(ctx, partial, static_cast<float*>(g_bias), blocks, heads, tag, stage);
  if (rc != OMX_OK) return rc;
  // grad_input[r, i] = sum_h gz[r, h] weight[h, i]
  if (g_input) {
    rc = omx_gemm_impl(ctx, F_GATE_BACKWARD, gz, heads, 1, weight, d_model, 1, operand_dtype, g_input, g_input_dtype,
                       d_model, rows, heads, d_model, 0);
    if (rc != OMX_OK) return rc;
  }
  // grad_weight[h, i] = sum_r gz[r, h] input[r, i]
  if (!g_weight) return OMX_OK;
  return omx_gemm_impl(ctx, F_GATE_BACKWARD, gz, 1, heads, input, d_model, 1, operand_dtype, g_weight, OMX_F32, d_model,
                       heads, rows, d_model, 0);
}

int32_t omx_per_head_sigmoid_gate_backward(omx_ctx* ctx, const void* input, const void* weight, int32_t operand_dtype,
                                           const void* bias, const void* attn, int32_t attn_dtype, const void* gy,
                                           int32_t gy_dtype, const void* gates_saved, void* g_input,
                                           int32_t g_input_dtype, void* g_weight, void* g_bias, void* g_attn,
                                           int32_t g_attn_dtype, uint64_t rows, uint64_t d_model, uint64_t heads,
                                           uint64_t head_dim) {
  if (ctx && !g_weight) return omx_fail(ctx, OMX_PLACEMENT, "per_head_sigmoid_gate_backward: null device pointer");
  return gate_backward_impl(ctx, "per_head_sigmoid_gate_backward", input, weight, operand_dtype, bias, attn, attn_dtype,
                            gy, gy_dtype, gates_saved, g_input, g_input_dtype, g_weight, nullptr, g_bias, g_attn,
                            g_attn_dtype, rows, d_model, heads, head_dim);
}

int32_t omx_per_head_sigmoid_gate_backward_deferred(omx_ctx* ctx, const void* input, const void* weight,
                                                    int32_t operand_dtype, const void* bias, const void* attn,
                                                    int32_t attn_dtype, const void* gy, int32_t gy_dtype,
                                                    const void* gates_saved, void* g_input, int32_t g_input_dtype,
                                                    void* gz_out, void* g_bias, void* g_attn, int32_t g_attn_dtype,
                                                    uint64_t rows, uint64_t d_model, uint64_t heads,
                                                    uint64_t head_dim) {
  if (ctx && !gz_out)
    return omx_fail(ctx, OMX_PLACEMENT, "per_head_sigmoid_gate_backward_deferred: null device pointer");
  return gate_backward_impl(ctx, "per_head_sigmoid_gate_backward_deferred", input, weight, operand_dtype, bias, attn,
                            attn_dtype, gy, gy_dtype, gates_saved, g_input, g_input_dtype, nullptr, gz_out, g_bias,
                            g_attn, g_attn_dtype, rows, d_model, heads, head_dim);
}

int32_t omx_per_head_sigmoid_gate_input_grad_add(omx_ctx* ctx, const void* gz, const void* weight, int32_t operand_dtype,
                                                 const void* add_in, int32_t add_dtype, void* out, uint64_t rows,
                                                 uint64_t d_model, uint64_t heads) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "per_head_sigmoid_gate_input_grad_add";
  if (!gz || !weight || !add_in || !out) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(operand_dtype) || !omx_valid_float_dtype(add_dtype))
    return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  if (rows == 0 || d_model == 0 || heads == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (out == add_in) return omx_fail(ctx, OMX_SHAPE, "%s: the output may not be the gradient it is added to", op);
  const bool aligned = ((reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(add_in)) & 7u) == 0 &&
                       (reinterpret_cast<uintptr_t>(out) & 15u) == 0 &&
                       (add_dtype == OMX_BF16 || (reinterpret_cast<uintptr_t>(add_in) & 15u) == 0);
  if (operand_dtype == OMX_BF16 && d_model % 4 == 0 && d_model <= 1024 && heads <= GATE_JOIN_HEADS && aligned) {
    const int rows_per_block = 8;
    const unsigned threads = static_cast<unsigned>((d_model / 4 + 63) / 64 * 64);
    const unsigned long long tag = omx_tag(ctx, F_GATE_BACKWARD);
    dim3 grid(static_cast<unsigned>((rows + rows_per_block - 1) / rows_per_block));
#define GATE_JOIN(TA_)                                                                                        \
  hipLaunchKernelGGL(gate_input_grad_add_kernel<TA_>, grid, dim3(threads), 0, ctx->stream,                    \
                     static_cast<const unsigned short*>(gz), static_cast<const unsigned short*>(weight),      \
                     static_cast<const TA_*>(add_in), static_cast<float*>(out), rows, static_cast<int>(d_model), \
                     static_cast<int>(heads), rows_per_block, ctx->fault, tag)
    if (add_dtype == OMX_BF16) GATE_JOIN(unsigned short);
    else GATE_JOIN(float);
#undef GATE_JOIN
    OMX_LAUNCH_CHECK(ctx, "gate_input_grad_add_kernel");
    return OMX_OK;
  }
  // Any other shape: the product, then the sum.
  int32_t rc = omx_gemm_impl(ctx, F_GATE_BACKWARD, gz, heads, 1, weight, d_model, 1, operand_dtype, out, OMX_F32, d_model,
                             rows, heads, d_model, 0);
  if (rc != OMX_OK) return rc;
  return omx_residual_add(ctx, out, OMX_F32, add_in, add_dtype, out, OMX_F32, rows * d_model);
}

int32_t omx_value_residual_blend_forward(omx_ctx* ctx, const void* value, const void* value0, const void* lambda,
                                         void* out, int32_t dtype, uint64_t n) {
  OMX_REQUIRE_CTX(ctx);
  int32_t rc = check_unary(ctx, "value_residual_blend_forward", dtype, n, {value, value0, lambda, out});
  if (rc != OMX_OK) return rc;
  const bool vec = packs_of_four(n, omx_dtype_size(dtype), {value, value0, out});
  const size_t packs = vec ? n / 4 : n;
  unsigned long long tag = omx_tag(ctx, F_VRES_FORWARD);
  LAUNCH_TV(vres_fwd_kernel, dtype, vec, pack_grid(packs), static_cast<const T_*>(value),
            static_cast<const T_*>(value0), static_cast<const float*>(lambda), static_cast<T_*>(out), packs,
            ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "vres_fwd_kernel");
  return OMX_OK;
}

int32_t omx_value_residual_blend_backward(omx_ctx* ctx, const void* value, const void* value0, const void* lambda,
                                          const void* gy, void* g_value, void* g_value0, int32_t dtype,
                                          void* g_lambda, uint64_t n) {
  OMX_REQUIRE_CTX(ctx);
  int32_t rc = check_unary(ctx, "value_residual_blend_backward", dtype, n,
                           {value, value0, lambda, gy, g_value, g_value0, g_lambda});
  if (rc != OMX_OK) return rc;
  const bool vec = packs_of_four(n, omx_dtype_size(dtype), {value, value0, gy, g_value, g_value0});
  const size_t packs = vec ? n / 4 : n;
  dim3 grid = pack_grid(packs);
  void* ws = nullptr;
  rc = omx_workspace(ctx, static_cast<uint64_t>(grid.x) * sizeof(float), &ws);
  if (rc != OMX_OK) return rc;
  float* partial = static_cast<float*>(ws);
  unsigned long long tag = omx_tag(ctx, F_VRES_BACKWARD);
  LAUNCH_TV(vres_bwd_kernel, dtype, vec, grid, static_cast<const T_*>(value), static_cast<const T_*>(value0),
            static_cast<const T_*>(gy), static_cast<const float*>(lambda), static_cast<T_*>(g_value),
            static_cast<T_*>(g_value0), partial, packs, ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "vres_bwd_kernel");
  hipLaunchKernelGGL(vres_lambda_kernel, dim3(1), dim3(BK_THREADS), 0, ctx->stream, partial, static_cast<int>(grid.x),
                     static_cast<const float*>(lambda), static_cast<float*>(g_lambda), ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "vres_lambda_kernel");
  return OMX_OK;
}

}  // extern "C"
