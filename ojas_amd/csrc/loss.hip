// Softmax cross-entropy: plain (logits in HBM) and fused with the LM head.
//
// Reference semantics:
//   cross_entropy_mean_forward/backward  ojas-cpu/src/pointwise.rs:2172-2438
//                                        (trait ojas-core/src/backend.rs:2451-2466)
//   linear_cross_entropy_mean            ojas-cpu/src/fused_ce.rs:97-158,290-452
//                                        (trait backend.rs:2493-2524, CeChunk :3081)
//
// Per row: loss = max + ln(sum e^(x - max)) - x_t, grad = (softmax - onehot) / valid,
// ignored rows contribute nothing, an all-ignored batch is NonFinite. The
// collapse rule (pointwise.rs:2305-2325) is kept: when the target holds the
// whole mass (x_t == max and the sum rounds to 1), S = sum_{j != t} e^(x_j - x_t)
// is used instead: loss = log1p(S), grad = e / (1 + S) / valid, target -S / (1 + S) / valid.
//
// The row statistics are carried as (max, sum without the target, target
// logit) so they can be updated one vocabulary tile at a time (online
// softmax); the fused op therefore never holds more than one
// chunk_rows x chunk_cols tile of logits.
#include "omx_common.h"

namespace {

constexpr int CE_THREADS = 256;

struct CeState {
  float* max;    // running row maximum
  float* other;  // sum of e^(x - max) over columns other than the target
  float* picked; // target logit
};

__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  return ((red[0] + red[1]) + red[2]) + red[3];
}

__global__ void ce_count_valid_kernel(const unsigned int* __restrict__ targets, size_t rows, size_t vocab,
                                      int has_ignore, unsigned int ignore, unsigned int* __restrict__ valid,
                                      OmxFaultWord* fault, unsigned long long tag) {
  size_t n = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  bool counts = false;
  if (n < rows) {
    unsigned int t = targets[n];
    if (!(has_ignore && t == ignore)) {
      if (t >= vocab) dev_raise_range(fault, tag);
      else counts = true;
    }
  }
  unsigned long long ballot = __ballot(counts);
  if ((threadIdx.x & 63) == 0 && ballot) atomicAdd(valid, static_cast<unsigned int>(__popcll(ballot)));
}

// Loads VEC consecutive logits (one 16-byte access when VEC > 1).
template <typename T, int VEC>
__device__ __forceinline__ void ce_load(const T* __restrict__ r, unsigned int c, float (&v)[VEC]) {
  if constexpr (VEC == 1) {
    v[0] = dev_load<T>(r, c);
  } else if constexpr (sizeof(T) == 4) {
    float4 q = *reinterpret_cast<const float4*>(r + c);
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
  } else {
    uint4 q = *reinterpret_cast<const uint4*>(r + c);
    const unsigned int w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[2 * j] = __uint_as_float(w[j] << 16);
      v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    }
  }
}
template <typename T, int VEC>
__device__ __forceinline__ void ce_store(T* __restrict__ g, unsigned int c, const float (&v)[VEC]) {
  if constexpr (VEC == 1) {
    dev_store<T>(g, c, v[0]);
  } else if constexpr (sizeof(T) == 4) {
    *reinterpret_cast<float4*>(g + c) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
    unsigned int w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      w[j] = dev_pack_bf16_pair(v[2 * j], v[2 * j + 1]);
    *reinterpret_cast<uint4*>(g + c) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}
// Elements per 16-byte access of T.
template <typename T>
constexpr int ce_vec() { return 16 / static_cast<int>(sizeof(T)); }

// exp for the running sums and the gradients of a tile. bf16 logits carry 8 bits of mantissa, the
// bf16 tier's loss gate is 1e-3 and its gradients are stored in bf16, so their exponentials take
// the hardware exp2 (two instructions; about 1e-6 relative with the rounding of the scaled
// argument) instead of expf's full-precision sequence, which made the passes compute-bound
// (2.9 TB/s for the statistics, 3.4 for statistics and gradients in one). f32 logits keep expf.
template <typename T>
__device__ __forceinline__ float ce_exp(float x) {
  if constexpr (sizeof(T) == 2) return __builtin_amdgcn_exp2f(x * 1.4426950408889634f);
  else return expf(x);
}

// One block per row. Folds the tile's columns [col0, col0 + ncols) into the
// row's running (max, other, picked) in ONE pass over the row: every thread
// keeps an online (max, sum) pair that is rescaled when its maximum grows,
// and the pairs are merged once at the end. `first` starts the state.
template <typename T, int VEC>
__global__ __launch_bounds__(CE_THREADS) void ce_tile_stats_kernel(const T* __restrict__ tile, size_t ld,
                                                                   size_t row0, unsigned int col0,
                                                                   unsigned int ncols,
                                                                   const unsigned int* __restrict__ targets,
                                                                   CeState st, int first, OmxFaultWord* fault,
                                                                   unsigned long long tag) {
  __shared__ float red[4];
  const size_t local = blockIdx.x, row = row0 + local;
  const T* r = tile + local * ld;
  const unsigned int target = targets[row];
  const unsigned int tcol = target - col0;  // wraps to a huge value when the target is left of this tile
  float mx = -INFINITY, sum = 0.0f;
  bool bad = false;
  for (unsigned int c = threadIdx.x * VEC; c < ncols; c += CE_THREADS * VEC) {
    float v[VEC];
    ce_load<T, VEC>(r, c, v);
    float top = v[0];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      bad |= !dev_finite(v[j]);
      top = fmaxf(top, v[j]);
    }
    if (top > mx) {
      sum *= ce_exp<T>(mx - top);
      mx = top;
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j)
      if (c + j != tcol) sum += ce_exp<T>(v[j] - mx);
  }
  const float row_max = block_max(mx, red);
  sum = block_sum(mx == -INFINITY ? 0.0f : sum * expf(mx - row_max), red);
  if (__syncthreads_or(bad)) {
    if (threadIdx.x == 0) dev_raise_fault(fault, tag);
  }
  if (threadIdx.x == 0) {
    float old_max = first ? -INFINITY : st.max[row];
    float new_max = fmaxf(old_max, row_max);
    float other = first ? 0.0f : st.other[row] * expf(old_max - new_max);
    st.max[row] = new_max;
    st.other[row] = other + sum * expf(row_max - new_max);
    if (target >= col0 && target < col0 + ncols) st.picked[row] = dev_load<T>(r, tcol);
  }
}

// Single block: per-row losses from the final state, summed in a fixed tree
// order, divided by the valid count.
__global__ __launch_bounds__(1024) void ce_mean_kernel(CeState st, const unsigned int* __restrict__ targets,
                                                       size_t rows, int has_ignore, unsigned int ignore,
                                                       const unsigned int* __restrict__ valid,
                                                       float* __restrict__ loss, OmxFaultWord* fault,
                                                       unsigned long long tag) {
  __shared__ float red[1024];
  float acc = 0.0f;
  for (size_t n = threadIdx.x; n < rows; n += 1024) {
    unsigned int t = targets[n];
    if (has_ignore && t == ignore) continue;
    float m = st.max[n], other = st.other[n], p = st.picked[n];
    float sum = other + expf(p - m);
    float term;
    if (p == m && sum == 1.0f && other > 0.0f) term = log1pf(other);
    else term = m + logf(sum) - p;
    acc += term;
  }
  red[threadIdx.x] = acc;
  __syncthreads();
  for (int s = 512; s > 0; s >>= 1) {
    if (threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    unsigned int v = *valid;
    float l = red[0] / static_cast<float>(v);
    *loss = l;
    // An all-ignored batch divides by zero: NonFinite, as on the CPU.
    if (v == 0 || !dev_finite(l)) dev_raise_fault(fault, tag);
  }
}

// One block per row: tile of logits -> tile of gradients (may be in place).
template <typename TL, typename TG, int VEC>
__global__ __launch_bounds__(CE_THREADS) void ce_tile_grad_kernel(const TL* __restrict__ tile, TG* __restrict__ grad,
                                                                  size_t ld, size_t ld_grad, size_t row0,
                                                                  unsigned int col0, unsigned int ncols,
                                                                  const unsigned int* __restrict__ targets,
                                                                  int has_ignore, unsigned int ignore, CeState st,
                                                                  const unsigned int* __restrict__ valid) {
  const size_t local = blockIdx.x, row = row0 + local;
  const TL* r = tile + local * ld;
  TG* g = grad + local * ld_grad;
  const unsigned int target = targets[row];
  if (has_ignore && target == ignore) {
    float zero[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) zero[j] = 0.0f;
    for (unsigned int c = threadIdx.x * VEC; c < ncols; c += CE_THREADS * VEC) ce_store<TG, VEC>(g, c, zero);
    return;
  }
  const unsigned int tcol = target - col0;
  const float m = st.max[row], other = st.other[row], p = st.picked[row];
  const float denom = static_cast<float>(*valid);
  const float sum = other + expf(p - m);
  const bool collapse = (p == m && sum == 1.0f && other > 0.0f);
  const float d = collapse ? 1.0f + other : sum;
  const float target_grad = collapse ? -(other / d) / denom : (expf(p - m) / d) / denom - 1.0f / denom;
  const float scale = (1.0f / d) / denom;
  for (unsigned int c = threadIdx.x * VEC; c < ncols; c += CE_THREADS * VEC) {
    float v[VEC], out[VEC];
    ce_load<TL, VEC>(r, c, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) out[j] = (c + j == tcol) ? target_grad : ce_exp<TL>(v[j] - m) * scale;
    ce_store<TG, VEC>(g, c, out);
  }
}

// One block per row, for a tile that holds the row's whole vocabulary: the statistics pass and the
// gradient pass of the two kernels above over ONE read of the logits, which wait in registers in
// between (MAXV 16-byte packs per thread), gradients written in place. 1024 threads keep that to
// 32 registers per thread for 65536 bf16 logits, so eight waves per SIMD overlap one row's loads
// with another's exponentials. Same formulas as ce_tile_stats_kernel (first tile) followed by
// ce_tile_grad_kernel; the row sum is formed over 1024 partial sums instead of 256, so it agrees
// with theirs to rounding, not to the bit.
constexpr int CE_FUSED_THREADS = 1024;
// max / min of three in one instruction (NaNs are skipped, as by fmaxf / fminf).
__device__ __forceinline__ float ce_max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ float ce_min3(float a, float b, float c) {
  float r;
  asm("v_min3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ float fused_block_max(float v, float* red) {
  v = wave_max(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float r = red[0];
#pragma unroll
  for (int i = 1; i < CE_FUSED_THREADS / 64; ++i) r = fmaxf(r, red[i]);
  return r;
}
__device__ __forceinline__ float fused_block_sum(float v, float* red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float r = red[0];
#pragma unroll
  for (int i = 1; i < CE_FUSED_THREADS / 64; ++i) r += red[i];
  return r;
}
template <typename T, int MAXV>
__global__ __launch_bounds__(CE_FUSED_THREADS, 8) void ce_row_fused_kernel(T* __restrict__ tile, size_t ld, size_t row0,
                                                                  unsigned int ncols,
                                                                  const unsigned int* __restrict__ targets,
                                                                  int has_ignore, unsigned int ignore, CeState st,
                                                                  const unsigned int* __restrict__ valid,
                                                                  OmxFaultWord* fault, unsigned long long tag) {
  constexpr int VEC = ce_vec<T>();
  __shared__ float red[CE_FUSED_THREADS / 64];
  __shared__ float picked;
  const size_t local = blockIdx.x, row = row0 + local;
  T* r = tile + local * ld;
  const unsigned int target = targets[row];
  if (threadIdx.x == 0) picked = target < ncols ? 0.0f : st.picked[row];
  // Every pack of the row, all loads in flight together. Packs past the end re-read the last one
  // (unconditional loads; they are masked out below).
  uint4 q[MAXV];
  const unsigned int last = ncols - VEC;
#pragma unroll
  for (int k = 0; k < MAXV; ++k) {
    const unsigned int c = (threadIdx.x + k * CE_FUSED_THREADS) * VEC;
    q[k] = *reinterpret_cast<const uint4*>(r + (c < ncols ? c : last));
  }
  auto unpack = [](const uint4& w, float (&v)[VEC]) {
    const unsigned int u[4] = {w.x, w.y, w.z, w.w};
    if constexpr (sizeof(T) == 4) {
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = __uint_as_float(u[j]);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[2 * j] = __uint_as_float(u[j] << 16);
        v[2 * j + 1] = __uint_as_float(u[j] & 0xffff0000u);
      }
    }
  };
  float mx = -INFINITY, sum = 0.0f;
  bool bad = false;
  __syncthreads();  // `picked` is initialised before its owner overwrites it
  if constexpr (sizeof(T) == 2) {
    // bf16 logits: a pack's largest and smallest value through three-input max / min, the
    // exponent as one fma (v log2e - max log2e) into the hardware exp2, and the comparison with
    // the target column only in the one pack that holds it. A NaN or an infinity among the logits
    // shows in the smallest / largest value, in the sum or in the picked logit.
    constexpr float LOG2E = 1.4426950408889634f;
    float mn = INFINITY, mine = 0.0f;
#pragma unroll
    for (int k = 0; k < MAXV; ++k) {
      const unsigned int c = (threadIdx.x + k * CE_FUSED_THREADS) * VEC;
      if (c < ncols) {
        float v[VEC];
        unpack(q[k], v);
        const float top = fmaxf(ce_max3(ce_max3(ce_max3(v[0], v[1], v[2]), v[3], v[4]), v[5], v[6]), v[7]);
        mn = fminf(ce_min3(ce_min3(ce_min3(mn, v[0], v[1]), v[2], v[3]), v[4], v[5]), fminf(v[6], v[7]));
        if (top > mx) {
          sum *= __builtin_amdgcn_exp2f((mx - top) * LOG2E);
          mx = top;
        }
        const float shift = -mx * LOG2E;
        if (target - c >= static_cast<unsigned int>(VEC)) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) sum += __builtin_amdgcn_exp2f(fmaf(v[j], LOG2E, shift));
        } else {
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            if (c + j != target) sum += __builtin_amdgcn_exp2f(fmaf(v[j], LOG2E, shift));
            else picked = mine = v[j];
          }
        }
      }
    }
    bad = !(mn > -INFINITY && mx < INFINITY && sum == sum && dev_finite(mine));
  } else {
#pragma unroll
    for (int k = 0; k < MAXV; ++k) {
      const unsigned int c = (threadIdx.x + k * CE_FUSED_THREADS) * VEC;
      if (c < ncols) {
        float v[VEC];
        unpack(q[k], v);
        float top = v[0];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          bad |= !dev_finite(v[j]);
          top = fmaxf(top, v[j]);
        }
        if (top > mx) {
          sum *= ce_exp<T>(mx - top);
          mx = top;
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          if (c + j != target) sum += ce_exp<T>(v[j] - mx);
          else picked = v[j];
        }
      }
    }
  }
  const float row_max = fused_block_max(mx, red);
  sum = fused_block_sum(mx == -INFINITY ? 0.0f : sum * expf(mx - row_max), red);
  if (__syncthreads_or(bad)) {
    if (threadIdx.x == 0) dev_raise_fault(fault, tag);
  }
  const float m = row_max, other = 0.0f + sum * expf(row_max - row_max), p = picked;
  if (threadIdx.x == 0) {
    st.max[row] = m;
    st.other[row] = other;
    if (target < ncols) st.picked[row] = p;
  }
  if (has_ignore && target == ignore) {
#pragma unroll
    for (int k = 0; k < MAXV; ++k) {
      const unsigned int c = (threadIdx.x + k * CE_FUSED_THREADS) * VEC;
      if (c < ncols) *reinterpret_cast<uint4*>(r + c) = make_uint4(0u, 0u, 0u, 0u);
    }
    return;
  }
  const float denom = static_cast<float>(*valid);
  const float total = other + expf(p - m);
  const bool collapse = (p == m && total == 1.0f && other > 0.0f);
  const float d = collapse ? 1.0f + other : total;
  const float target_grad = collapse ? -(other / d) / denom : (expf(p - m) / d) / denom - 1.0f / denom;
  const float scale = (1.0f / d) / denom;
#pragma unroll
  for (int k = 0; k < MAXV; ++k) {
    const unsigned int c = (threadIdx.x + k * CE_FUSED_THREADS) * VEC;
    if (c < ncols) {
      float v[VEC], out[VEC];
      unpack(q[k], v);
      if constexpr (sizeof(T) == 2) {
        constexpr float LOG2E = 1.4426950408889634f;
        const float shift = -m * LOG2E;
#pragma unroll
        for (int j = 0; j < VEC; ++j) out[j] = __builtin_amdgcn_exp2f(fmaf(v[j], LOG2E, shift)) * scale;
        if (target - c < static_cast<unsigned int>(VEC)) {
#pragma unroll
          for (int j = 0; j < VEC; ++j)
            if (c + j == target) out[j] = target_grad;
        }
        uint4 w;
        w.x = dev_pack_bf16_pair(out[0], out[1]);
        w.y = dev_pack_bf16_pair(out[2], out[3]);
        w.z = dev_pack_bf16_pair(out[4], out[5]);
        w.w = dev_pack_bf16_pair(out[6], out[7]);
        *reinterpret_cast<uint4*>(r + c) = w;
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) out[j] = (c + j == target) ? target_grad : ce_exp<T>(v[j] - m) * scale;
        ce_store<T, VEC>(r, c, out);
      }
    }
  }
}
constexpr int CE_FUSED_PACKS = 8;  // per thread: rows of up to 65536 bf16 or 32768 f32 logits

// Whether rows of `ld` elements starting at `base` (+ col offset) allow 16-byte accesses of T.
template <typename T>
bool ce_vector_ok(const void* base, size_t ld, unsigned int ncols) {
  return (reinterpret_cast<uintptr_t>(base) & 15u) == 0 && (ld * sizeof(T)) % 16 == 0 && ncols % ce_vec<T>() == 0;
}

template <typename T>
void launch_stats(omx_ctx* ctx, const void* tile, size_t ld, size_t row0, size_t nrows, unsigned int col0,
                  unsigned int ncols, const unsigned int* targets, CeState st, int first, unsigned long long tag) {
  dim3 grid(static_cast<unsigned>(nrows)), block(CE_THREADS);
  if (ce_vector_ok<T>(tile, ld, ncols))
    hipLaunchKernelGGL((ce_tile_stats_kernel<T, ce_vec<T>()>), grid, block, 0, ctx->stream,
                       static_cast<const T*>(tile), ld, row0, col0, ncols, targets, st, first, ctx->fault, tag);
  else
    hipLaunchKernelGGL((ce_tile_stats_kernel<T, 1>), grid, block, 0, ctx->stream, static_cast<const T*>(tile), ld,
                       row0, col0, ncols, targets, st, first, ctx->fault, tag);
}
template <typename TL, typename TG>
void launch_grad(omx_ctx* ctx, const void* tile, void* grad, size_t ld, size_t ld_grad, size_t row0, size_t nrows,
                 unsigned int col0, unsigned int ncols, const unsigned int* targets, int has_ignore,
                 unsigned int ignore, CeState st, const unsigned int* valid) {
  dim3 grid(static_cast<unsigned>(nrows)), block(CE_THREADS);
  // 16-byte packs on both sides need logits and gradients of one element size.
  if constexpr (sizeof(TL) == sizeof(TG)) {
    if (ce_vector_ok<TL>(tile, ld, ncols) && ce_vector_ok<TG>(grad, ld_grad, ncols)) {
      hipLaunchKernelGGL((ce_tile_grad_kernel<TL, TG, ce_vec<TL>()>), grid, block, 0, ctx->stream,
                         static_cast<const TL*>(tile), static_cast<TG*>(grad), ld, ld_grad, row0, col0, ncols, targets,
                         has_ignore, ignore, st, valid);
      return;
    }
  }
  hipLaunchKernelGGL((ce_tile_grad_kernel<TL, TG, 1>), grid, block, 0, ctx->stream, static_cast<const TL*>(tile),
                     static_cast<TG*>(grad), ld, ld_grad, row0, col0, ncols, targets, has_ignore, ignore, st, valid);
}

// State + valid counter carved out of a workspace block.
struct CeScratch {
  CeState st;
  unsigned int* valid;
};
inline size_t ce_scratch_bytes(uint64_t rows) { return (3 * rows + 4) * sizeof(float); }
inline CeScratch carve(void* base, uint64_t rows) {
  float* f = static_cast<float*>(base);
  CeScratch s;
  s.st.max = f;
  s.st.other = f + rows;
  s.st.picked = f + 2 * rows;
  s.valid = reinterpret_cast<unsigned int*>(f + 3 * rows);
  return s;
}

int32_t count_valid(omx_ctx* ctx, const unsigned int* targets, uint64_t rows, uint64_t vocab, int has_ignore,
                    unsigned int ignore, unsigned int* valid, unsigned long long tag) {
  int32_t rc = omx_fill_zero(ctx, valid, 4);
  if (rc != OMX_OK) return rc;
  hipLaunchKernelGGL(ce_count_valid_kernel, dim3(static_cast<unsigned>((rows + 255) / 256)), dim3(256), 0,
                     ctx->stream, targets, rows, vocab, has_ignore, ignore, valid, ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "ce_count_valid_kernel");
  return OMX_OK;
}

int32_t check_ce_args(omx_ctx* ctx, const char* op, const void* logits, const void* targets, uint64_t rows,
                      uint64_t vocab, int32_t dtype) {
  if (!logits || !targets) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: logits must be f32 or bf16", op);
  if (rows == 0 || vocab == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (vocab > 0xfffffffeull || rows > 0x7fffffffull)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: axis does not fit in u32", op);
  return OMX_OK;
}

// cross_entropy_mean_forward over caller-chosen scratch (ce_scratch_bytes(rows) bytes at `ws`):
// every word of the scratch that is read is written first (the valid counter by a fill kernel,
// the row state by the statistics kernel started with `first`), so stale contents do not matter.
int32_t ce_forward_in(omx_ctx* ctx, const void* logits, int32_t logits_dtype, const void* targets, uint64_t rows,
                      uint64_t vocab, int32_t has_ignore, uint32_t ignore_index, void* loss, void* ws) {
  CeScratch s = carve(ws, rows);
  const unsigned int* tg = static_cast<const unsigned int*>(targets);
  unsigned long long tag = omx_tag(ctx, F_CE_FORWARD);
  int32_t rc = count_valid(ctx, tg, rows, vocab, has_ignore, ignore_index, s.valid, tag);
  if (rc != OMX_OK) return rc;
  if (logits_dtype == OMX_F32) launch_stats<float>(ctx, logits, vocab, 0, rows, 0, vocab, tg, s.st, 1, tag);
  else launch_stats<unsigned short>(ctx, logits, vocab, 0, rows, 0, vocab, tg, s.st, 1, tag);
  OMX_LAUNCH_CHECK(ctx, "ce_tile_stats_kernel");
  hipLaunchKernelGGL(ce_mean_kernel, dim3(1), dim3(1024), 0, ctx->stream, s.st, tg, rows, has_ignore, ignore_index,
                     s.valid, static_cast<float*>(loss), ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "ce_mean_kernel");
  return OMX_OK;
}

}  // namespace

// Scratch of omx_cross_entropy_mean_forward_static: row state (max, sum, target logit) and the
// valid counter for up to CE_STATIC_MAX_ROWS rows, 786,688 bytes held by every device the library
// runs on until the process ends. All calls on a device share it.
constexpr uint64_t CE_STATIC_MAX_ROWS = 65536;
static __device__ __align__(256) float g_ce_static_scratch[3 * CE_STATIC_MAX_ROWS + 64];

// The array's name is a host-side handle; each device holds its own copy at its own address.
// omx_open calls this once per context with the context's device current and keeps the result.
void* omx_ce_static_scratch_address() {
  void* p = nullptr;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_ce_static_scratch)) != hipSuccess) return nullptr;
  return p;
}

extern "C" {

int32_t omx_cross_entropy_mean_forward(omx_ctx* ctx, const void* logits, int32_t logits_dtype, const void* targets,
                                       uint64_t rows, uint64_t vocab, int32_t has_ignore, uint32_t ignore_index,
                                       void* loss) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "cross_entropy_mean_forward";
  int32_t rc = check_ce_args(ctx, op, logits, targets, rows, vocab, logits_dtype);
  if (rc != OMX_OK) return rc;
  if (!loss) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  void* ws = nullptr;
  rc = omx_workspace(ctx, ce_scratch_bytes(rows), &ws);
  if (rc != OMX_OK) return rc;
  return ce_forward_in(ctx, logits, logits_dtype, targets, rows, vocab, has_ignore, ignore_index, loss, ws);
}

int32_t omx_cross_entropy_mean_forward_static(omx_ctx* ctx, const void* logits, int32_t logits_dtype,
                                              const void* targets, uint64_t rows, uint64_t vocab, int32_t has_ignore,
                                              uint32_t ignore_index, void* loss) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "cross_entropy_mean_forward_static";
  int32_t rc = check_ce_args(ctx, op, logits, targets, rows, vocab, logits_dtype);
  if (rc != OMX_OK) return rc;
  if (!loss) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (rows > CE_STATIC_MAX_ROWS)
    return omx_fail(ctx, OMX_CAPACITY_EXCEEDED, "%s: %llu rows, the static scratch holds at most %llu", op,
                    (unsigned long long)rows, (unsigned long long)CE_STATIC_MAX_ROWS);
  // Looked up when the context was opened: nothing here but launches on the context's stream.
  void* ws = ctx->ce_static_scratch;
  if (!ws) return omx_fail(ctx, OMX_BACKEND, "%s: the scratch symbol has no device address", op);
  return ce_forward_in(ctx, logits, logits_dtype, targets, rows, vocab, has_ignore, ignore_index, loss, ws);
}

int32_t omx_cross_entropy_mean_backward(omx_ctx* ctx, const void* logits, int32_t logits_dtype, const void* targets,
                                        uint64_t rows, uint64_t vocab, int32_t has_ignore, uint32_t ignore_index,
                                        void* grad, int32_t grad_dtype) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "cross_entropy_mean_backward";
  int32_t rc = check_ce_args(ctx, op, logits, targets, rows, vocab, logits_dtype);
  if (rc != OMX_OK) return rc;
  if (!grad) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(grad_dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: grad must be f32 or bf16", op);
  void* ws = nullptr;
  rc = omx_workspace(ctx, ce_scratch_bytes(rows) + 16, &ws);
  if (rc != OMX_OK) return rc;
  CeScratch s = carve(ws, rows);
  float* loss_scratch = reinterpret_cast<float*>(s.valid + 2);
  const unsigned int* tg = static_cast<const unsigned int*>(targets);
  unsigned long long tag = omx_tag(ctx, F_CE_BACKWARD);
  rc = count_valid(ctx, tg, rows, vocab, has_ignore, ignore_index, s.valid, tag);
  if (rc != OMX_OK) return rc;
  if (logits_dtype == OMX_F32) launch_stats<float>(ctx, logits, vocab, 0, rows, 0, vocab, tg, s.st, 1, tag);
  else launch_stats<unsigned short>(ctx, logits, vocab, 0, rows, 0, vocab, tg, s.st, 1, tag);
  OMX_LAUNCH_CHECK(ctx, "ce_tile_stats_kernel");
  // The mean kernel also raises the all-ignored fault, as the forward does.
  hipLaunchKernelGGL(ce_mean_kernel, dim3(1), dim3(1024), 0, ctx->stream, s.st, tg, rows, has_ignore, ignore_index,
                     s.valid, loss_scratch, ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "ce_mean_kernel");
  if (logits_dtype == OMX_F32 && grad_dtype == OMX_F32)
    launch_grad<float, float>(ctx, logits, grad, vocab, vocab, 0, rows, 0, vocab, tg, has_ignore, ignore_index, s.st,
                              s.valid);
  else if (logits_dtype == OMX_F32)
    launch_grad<float, unsigned short>(ctx, logits, grad, vocab, vocab, 0, rows, 0, vocab, tg, has_ignore,
                                       ignore_index, s.st, s.valid);
  else if (grad_dtype == OMX_F32)
    launch_grad<unsigned short, float>(ctx, logits, grad, vocab, vocab, 0, rows, 0, vocab, tg, has_ignore,
                                       ignore_index, s.st, s.valid);
  else
    launch_grad<unsigned short, unsigned short>(ctx, logits, grad, vocab, vocab, 0, rows, 0, vocab, tg, has_ignore,
                                                ignore_index, s.st, s.valid);
  OMX_LAUNCH_CHECK(ctx, "ce_tile_grad_kernel");
  return OMX_OK;
}

int32_t omx_linear_cross_entropy_mean(omx_ctx* ctx, const void* x, const void* w, int32_t operand_dtype,
                                      const void* targets, uint64_t rows, uint64_t dim, uint64_t vocab,
                                      int32_t has_ignore, uint32_t ignore_index, uint64_t chunk_rows,
                                      uint64_t chunk_cols, void* loss, void* gx, int32_t gx_dtype, void* gw) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "linear_cross_entropy_mean";
  if (!x || !w || !targets || !loss) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(operand_dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: operands must be f32 or bf16", op);
  if (gx && !omx_valid_float_dtype(gx_dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: grad_input dtype", op);
  if (rows == 0 || dim == 0 || vocab == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (chunk_rows == 0 || chunk_cols == 0) return omx_fail(ctx, OMX_SHAPE, "%s: chunk has a zero axis", op);
  if (vocab > 0xfffffffeull || rows > 0x7fffffffull)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: axis does not fit in u32", op);
  const uint64_t R = chunk_rows < rows ? chunk_rows : rows;
  // Column tiles start on multiples of 8 so every tile of W stays 16-byte aligned.
  uint64_t C = chunk_cols < vocab ? chunk_cols : vocab;
  if (C < vocab && C >= 8) C &= ~7ull;
  const bool one_tile = C >= vocab;
  const bool want_grads = gx || gw;
  const size_t esz = omx_dtype_size(operand_dtype);
  // Workspace: [tile R x C] [gx accumulator R x dim f32, only with several column tiles] [state].
  const uint64_t tile_bytes = (R * C * esz + 255) & ~255ull;
  const uint64_t gxacc_bytes = (gx && !one_tile) ? ((R * dim * 4 + 255) & ~255ull) : 0;
  void* ws = nullptr;
  int32_t rc = omx_workspace(ctx, tile_bytes + gxacc_bytes + ce_scratch_bytes(rows), &ws);
  if (rc != OMX_OK) return rc;
  char* base = static_cast<char*>(ws);
  void* tile = base;
  float* gxacc = reinterpret_cast<float*>(base + tile_bytes);
  CeScratch s = carve(base + tile_bytes + gxacc_bytes, rows);
  const unsigned int* tg = static_cast<const unsigned int*>(targets);
  unsigned long long tag = omx_tag(ctx, F_LINEAR_CE);
  rc = count_valid(ctx, tg, rows, vocab, has_ignore, ignore_index, s.valid, tag);
  if (rc != OMX_OK) return rc;
  const char* xb = static_cast<const char*>(x);
  const char* wb = static_cast<const char*>(w);

  auto logits_tile = [&](uint64_t r0, uint64_t nr, uint64_t c0, uint64_t nc) -> int32_t {
    // tile[nr, nc] = x[r0.., :] . W[c0.., :]^T
    return omx_gemm_impl(ctx, F_LINEAR_CE, xb + r0 * dim * esz, dim, 1, wb + c0 * dim * esz, 1, dim, operand_dtype,
                         tile, operand_dtype, nc, nr, dim, nc, 0);
  };
  for (uint64_t r0 = 0; r0 < rows; r0 += R) {
    const uint64_t nr = (rows - r0) < R ? (rows - r0) : R;
    // The whole vocabulary in one tile, with gradients wanted: one kernel reads the logits once.
    const bool fuse = ctx->ce_fused && one_tile && want_grads && vocab <= static_cast<uint64_t>(CE_FUSED_THREADS) * CE_FUSED_PACKS * (16 / esz) &&
                      (operand_dtype == OMX_F32 ? ce_vector_ok<float>(tile, vocab, static_cast<unsigned>(vocab))
                                                : ce_vector_ok<unsigned short>(tile, vocab, static_cast<unsigned>(vocab)));
    // Pass 1: row statistics over every vocabulary tile.
    for (uint64_t c0 = 0; c0 < vocab; c0 += C) {
      const uint64_t nc = (vocab - c0) < C ? (vocab - c0) : C;
      rc = logits_tile(r0, nr, c0, nc);
      if (rc != OMX_OK) return rc;
      if (fuse) {
        dim3 grid(static_cast<unsigned>(nr)), block(CE_FUSED_THREADS);
        // One read of the logits tile and one write of the gradient over it.
        OmxKernelTimer timer(ctx, OMX_K_CE, 2.0 * static_cast<double>(nr) * static_cast<double>(nc) * esz);
        // As many 16-byte packs per thread as the row needs (fewer registers for shorter rows).
        const uint64_t packs = (nc * esz / 16 + CE_FUSED_THREADS - 1) / CE_FUSED_THREADS;
#define CE_FUSED(T_, P_)                                                                                          \
  omx_launch_timed(ctx, ce_row_fused_kernel<T_, P_>, grid, block, 0, timer.start(), timer.stop(),                 \
                   static_cast<T_*>(tile), nc, r0, static_cast<unsigned>(nc), tg, has_ignore, ignore_index, s.st, \
                   s.valid, ctx->fault, tag)
#define CE_FUSED_P(T_)                              \
  do {                                              \
    if (packs <= 2) CE_FUSED(T_, 2);                \
    else if (packs <= 4) CE_FUSED(T_, 4);           \
    else if (packs <= 6) CE_FUSED(T_, 6);           \
    else if (packs <= 7) CE_FUSED(T_, 7);           \
    else CE_FUSED(T_, CE_FUSED_PACKS);              \
  } while (0)
        if (operand_dtype == OMX_F32) CE_FUSED_P(float);
        else CE_FUSED_P(unsigned short);
#undef CE_FUSED_P
#undef CE_FUSED
        OMX_LAUNCH_CHECK(ctx, "ce_row_fused_kernel");
        continue;
      }
      if (operand_dtype == OMX_F32)
        launch_stats<float>(ctx, tile, nc, r0, nr, static_cast<unsigned>(c0), static_cast<unsigned>(nc), tg, s.st,
                            c0 == 0, tag);
      else
        launch_stats<unsigned short>(ctx, tile, nc, r0, nr, static_cast<unsigned>(c0), static_cast<unsigned>(nc), tg,
                                     s.st, c0 == 0, tag);
      OMX_LAUNCH_CHECK(ctx, "ce_tile_stats_kernel");
    }
    if (!want_grads) continue;
    // Pass 2: gradient tiles and their two products.
    for (uint64_t c0 = 0; c0 < vocab; c0 += C) {
      const uint64_t nc = (vocab - c0) < C ? (vocab - c0) : C;
      if (!one_tile) {
        rc = logits_tile(r0, nr, c0, nc);
        if (rc != OMX_OK) return rc;
      }
      if (fuse) {
        // the gradients are already in the tile
      } else if (operand_dtype == OMX_F32)
        launch_grad<float, float>(ctx, tile, tile, nc, nc, r0, nr, static_cast<unsigned>(c0),
                                  static_cast<unsigned>(nc), tg, has_ignore, ignore_index, s.st, s.valid);
      else
        launch_grad<unsigned short, unsigned short>(ctx, tile, tile, nc, nc, r0, nr, static_cast<unsigned>(c0),
                                                    static_cast<unsigned>(nc), tg, has_ignore, ignore_index, s.st,
                                                    s.valid);
      OMX_LAUNCH_CHECK(ctx, "ce_tile_grad_kernel");
      if (gx) {
        // gx[r0.., :] (+)= G[nr, nc] . W[c0.., :]
        if (one_tile) {
          rc = omx_gemm_impl(ctx, F_LINEAR_CE, tile, nc, 1, wb + c0 * dim * esz, dim, 1, operand_dtype,
                             static_cast<char*>(gx) + r0 * dim * omx_dtype_size(gx_dtype), gx_dtype, dim, nr, nc, dim,
                             0);
        } else {
          rc = omx_gemm_impl(ctx, F_LINEAR_CE, tile, nc, 1, wb + c0 * dim * esz, dim, 1, operand_dtype, gxacc,
                             OMX_F32, dim, nr, nc, dim, c0 != 0);
        }
        if (rc != OMX_OK) return rc;
      }
      if (gw) {
        // gw[c0.., :] (+)= G^T[nc, nr] . x[r0.., :]
        rc = omx_gemm_impl(ctx, F_LINEAR_CE, tile, 1, nc, xb + r0 * dim * esz, dim, 1, operand_dtype,
                           static_cast<float*>(gw) + c0 * dim, OMX_F32, dim, nc, nr, dim, r0 != 0);
        if (rc != OMX_OK) return rc;
      }
    }
    if (gx && !one_tile) {
      rc = omx_convert(ctx, gxacc, OMX_F32, static_cast<char*>(gx) + r0 * dim * omx_dtype_size(gx_dtype), gx_dtype,
                       nr * dim);
      if (rc != OMX_OK) return rc;
    }
  }
  hipLaunchKernelGGL(ce_mean_kernel, dim3(1), dim3(1024), 0, ctx->stream, s.st, tg, rows, has_ignore, ignore_index,
                     s.valid, static_cast<float*>(loss), ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "ce_mean_kernel");
  return OMX_OK;
}

}  // extern "C"
