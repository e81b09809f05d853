// Causal scaled-dot-product attention, forward and backward.
//
// Reference semantics: ojas-cpu/src/attn.rs:47-124,176-227 (forward),
// :437-597 (backward from the saved output and log-sum-exp); trait
// ojas-core/src/backend.rs:1729-1792. Layout [B, H, T, D]; query t sees keys
// max(0, t + 1 - window) ..= t; query head h reads KV head h / (H / Hkv);
// scale = 1 / sqrt(D) formed in f32 (backend.rs:159). lse = max + ln(sum).
// Backward: P = e^(S - lse), Dr = dO . O, dS = scale * P * (dP - Dr);
// dQ = dS K, dK = dS^T Q, dV = P^T dO, with the query heads of one KV head
// summed in ascending head order.
//
// Two families of kernels:
//   * row kernels (this file, first part): one wavefront per query row (or per
//     key row in the dK/dV pass), any head_dim up to 256, f32 arithmetic. They
//     serve the f32 tier and every head_dim the MFMA kernels do not cover.
//   * flash kernels (flash_sdpa.hip): bf16 MFMA tiles for head_dim 64 / 128.
// Neither forms a T x T matrix; no atomics are used, so results do not depend
// on scheduling.
#include <algorithm>

#include "omx_common.h"

int32_t omx_flash_sdpa_forward(omx_ctx* ctx, const void* q, const void* k, const void* v, void* out,
                               int32_t out_dtype, void* out_residual, float* lse, uint64_t batch, uint64_t heads,
                               uint64_t kv_heads, uint64_t time, uint64_t dim, uint64_t window, float scale,
                               unsigned long long tag, const long* strides);
int32_t omx_flash_sdpa_backward(omx_ctx* ctx, const void* q, const void* k, const void* v, const void* out,
                                const void* out_residual, const float* lse, const void* gy, void* gq, void* gk,
                                void* gv, int32_t grad_dtype,
                                uint64_t batch, uint64_t heads, uint64_t kv_heads, uint64_t time, uint64_t dim,
                                uint64_t window, float scale, unsigned long long tag, const long* strides);
bool omx_flash_sdpa_supports(uint64_t dim, int32_t operand_dtype);

namespace {

constexpr int SD_THREADS = 256;  // 4 waves: 4 rows per block
constexpr int MAXD = 256;

struct SdpaShape {
  int batch, heads, kv_heads, time, dim, window, rep;
  float scale;
};

__device__ __forceinline__ int first_key(const SdpaShape& s, int t) {
  return s.window > 0 ? max(0, t + 1 - s.window) : 0;
}
__device__ __forceinline__ int last_query(const SdpaShape& s, int j) {
  // Queries that see key j: j ..= min(T-1, j + window - 1).
  return s.window > 0 ? min(s.time - 1, j + s.window - 1) : s.time - 1;
}

// One wave per query row. Lane l scores keys j0 + l of each 64-key block
// (dot over D from LDS-broadcast q), the block is folded into the running
// softmax, and lanes then switch to owning output dims for the P.V update.
template <typename TI, typename TO>
__global__ __launch_bounds__(SD_THREADS) void sdpa_fwd_rows_kernel(const TI* __restrict__ q, const TI* __restrict__ k,
                                                                   const TI* __restrict__ v, TO* __restrict__ out,
                                                                   float* __restrict__ lse, SdpaShape s,
                                                                   OmxFaultWord* fault, unsigned long long tag) {
  __shared__ float q_lds[4][MAXD];
  __shared__ float p_lds[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long row = static_cast<long>(blockIdx.x) * 4 + wave;  // (b*H + h)*T + t
  const long total = static_cast<long>(s.batch) * s.heads * s.time;
  if (row >= total) return;
  const int t = static_cast<int>(row % s.time);
  const long plane = row / s.time;
  const int h = static_cast<int>(plane % s.heads), b = static_cast<int>(plane / s.heads);
  const long kv_plane = static_cast<long>(b) * s.kv_heads + h / s.rep;
  const TI* qr = q + row * s.dim;
  const TI* kh = k + kv_plane * s.time * s.dim;
  const TI* vh = v + kv_plane * s.time * s.dim;
  const int D = s.dim;
  for (int d = lane; d < D; d += 64) q_lds[wave][d] = dev_load<TI>(qr, d);
  constexpr int ND = MAXD / 64;
  float acc[ND];
#pragma unroll
  for (int i = 0; i < ND; ++i) acc[i] = 0.0f;
  float run_max = -INFINITY, run_sum = 0.0f;
  bool bad = false;
  const int j_begin = first_key(s, t), j_end = t + 1;
  for (int j0 = j_begin; j0 < j_end; j0 += 64) {
    const int j = j0 + lane;
    float sc = -INFINITY;
    if (j < j_end) {
      const TI* kr = kh + static_cast<long>(j) * D;
      float dot = 0.0f;
      for (int d = 0; d < D; ++d) dot += q_lds[wave][d] * dev_load<TI>(kr, d);
      sc = dot * s.scale;
      bad |= !dev_finite(sc);
    }
    float blk_max = wave_max(sc);
    float new_max = fmaxf(run_max, blk_max);
    float p = j < j_end ? expf(sc - new_max) : 0.0f;
    float blk_sum = wave_sum(p);
    float rescale = expf(run_max - new_max);  // 0 on the first block (run_max = -inf)
    run_sum = run_sum * rescale + blk_sum;
    run_max = new_max;
    p_lds[wave][lane] = p;
    // Same-wave LDS traffic: the wave executes in lockstep, a fence orders it.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const int nk = min(64, j_end - j0);
#pragma unroll
    for (int i = 0; i < ND; ++i) {
      const int d = i * 64 + lane;
      if (d < D) {
        float a = acc[i] * rescale;
        for (int jj = 0; jj < nk; ++jj) a += p_lds[wave][jj] * dev_load<TI>(vh, static_cast<long>(j0 + jj) * D + d);
        acc[i] = a;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  bad |= !(dev_finite(run_sum) && run_sum > 0.0f);
  const float inv = 1.0f / run_sum;
  TO* orow = out + row * D;
#pragma unroll
  for (int i = 0; i < ND; ++i) {
    const int d = i * 64 + lane;
    if (d < D) {
      float o = acc[i] * inv;
      bad |= !dev_finite(o);
      dev_store<TO>(orow, d, o);
    }
  }
  if (lane == 0) lse[row] = run_max + logf(run_sum);
  if (bad) dev_raise_fault(fault, tag);
}

// Dr[row] = dO[row] . O[row] (f32), one wave per row.
template <typename TOUT, typename TGY>
__global__ __launch_bounds__(SD_THREADS) void sdpa_delta_kernel(const TOUT* __restrict__ out,
                                                                const TGY* __restrict__ gy,
                                                                float* __restrict__ delta, long rows, int D) {
  const int lane = threadIdx.x & 63;
  const long row = static_cast<long>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  float acc = 0.0f;
  for (int d = lane; d < D; d += 64) acc += dev_load<TGY>(gy, row * D + d) * dev_load<TOUT>(out, row * D + d);
  acc = wave_sum(acc);
  if (lane == 0) delta[row] = acc;
}

// An f32 attention output as the pair the bf16 MFMA backward reads: hi = bf16(x) and
// residual = bf16(x - hi), so hi + residual carries x to 2^-17.
__global__ void sdpa_split_output_kernel(const float* __restrict__ x, unsigned short* __restrict__ hi,
                                         unsigned short* __restrict__ residual, long n) {
  for (long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<long>(gridDim.x) * blockDim.x) {
    const float v = x[i];
    const unsigned short h = dev_f32_to_bf16_bits(v);
    hi[i] = h;
    residual[i] = dev_f32_to_bf16_bits(v - dev_bf16_bits_to_f32(h));
  }
}

// dQ: one wave per query row, the forward's structure with dS in place of P.
template <typename TI, typename TO>
__global__ __launch_bounds__(SD_THREADS) void sdpa_bwd_dq_rows_kernel(
    const TI* __restrict__ q, const TI* __restrict__ k, const TI* __restrict__ v, const float* __restrict__ lse,
    const float* __restrict__ delta, const TI* __restrict__ gy, TO* __restrict__ gq, SdpaShape s, OmxFaultWord* fault,
    unsigned long long tag) {
  __shared__ float q_lds[4][MAXD];
  __shared__ float g_lds[4][MAXD];
  __shared__ float c_lds[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long row = static_cast<long>(blockIdx.x) * 4 + wave;
  const long total = static_cast<long>(s.batch) * s.heads * s.time;
  if (row >= total) return;
  const int t = static_cast<int>(row % s.time);
  const long plane = row / s.time;
  const int h = static_cast<int>(plane % s.heads), b = static_cast<int>(plane / s.heads);
  const long kv_plane = static_cast<long>(b) * s.kv_heads + h / s.rep;
  const TI* kh = k + kv_plane * s.time * s.dim;
  const TI* vh = v + kv_plane * s.time * s.dim;
  const int D = s.dim;
  for (int d = lane; d < D; d += 64) {
    q_lds[wave][d] = dev_load<TI>(q, row * D + d);
    g_lds[wave][d] = dev_load<TI>(gy, row * D + d);
  }
  const float row_lse = lse[row], dr = delta[row];
  bool bad = !(dev_finite(row_lse) && dev_finite(dr));
  constexpr int ND = MAXD / 64;
  float acc[ND];
#pragma unroll
  for (int i = 0; i < ND; ++i) acc[i] = 0.0f;
  const int j_begin = first_key(s, t), j_end = t + 1;
  for (int j0 = j_begin; j0 < j_end; j0 += 64) {
    const int j = j0 + lane;
    float coef = 0.0f;
    if (j < j_end) {
      const TI* kr = kh + static_cast<long>(j) * D;
      const TI* vr = vh + static_cast<long>(j) * D;
      float dot = 0.0f, dp = 0.0f;
      for (int d = 0; d < D; ++d) {
        dot += q_lds[wave][d] * dev_load<TI>(kr, d);
        dp += g_lds[wave][d] * dev_load<TI>(vr, d);
      }
      float sc = dot * s.scale;
      float p = expf(sc - row_lse);
      bad |= !(dev_finite(sc) && dev_finite(p));
      coef = s.scale * (p * (dp - dr));
    }
    c_lds[wave][lane] = coef;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const int nk = min(64, j_end - j0);
#pragma unroll
    for (int i = 0; i < ND; ++i) {
      const int d = i * 64 + lane;
      if (d < D) {
        float a = acc[i];
        for (int jj = 0; jj < nk; ++jj) a += c_lds[wave][jj] * dev_load<TI>(kh, static_cast<long>(j0 + jj) * D + d);
        acc[i] = a;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
#pragma unroll
  for (int i = 0; i < ND; ++i) {
    const int d = i * 64 + lane;
    if (d < D) {
      bad |= !dev_finite(acc[i]);
      dev_store<TO>(gq, row * D + d, acc[i]);
    }
  }
  if (bad) dev_raise_fault(fault, tag);
}

// dK, dV: one wave per key row of a KV head; walks the query heads of the
// group in ascending order and, within a head, queries in ascending order.
template <typename TI, typename TO>
__global__ __launch_bounds__(SD_THREADS) void sdpa_bwd_dkv_rows_kernel(
    const TI* __restrict__ q, const TI* __restrict__ k, const TI* __restrict__ v, const float* __restrict__ lse,
    const float* __restrict__ delta, const TI* __restrict__ gy, TO* __restrict__ gk, TO* __restrict__ gv, SdpaShape s,
    OmxFaultWord* fault, unsigned long long tag) {
  __shared__ float k_lds[4][MAXD];
  __shared__ float v_lds[4][MAXD];
  __shared__ float c_lds[4][64];
  __shared__ float p_lds[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long row = static_cast<long>(blockIdx.x) * 4 + wave;  // (b*Hkv + g)*T + j
  const long total = static_cast<long>(s.batch) * s.kv_heads * s.time;
  if (row >= total) return;
  const int j = static_cast<int>(row % s.time);
  const long kv_plane = row / s.time;
  const int g = static_cast<int>(kv_plane % s.kv_heads), b = static_cast<int>(kv_plane / s.kv_heads);
  const int D = s.dim;
  for (int d = lane; d < D; d += 64) {
    k_lds[wave][d] = dev_load<TI>(k, row * D + d);
    v_lds[wave][d] = dev_load<TI>(v, row * D + d);
  }
  constexpr int ND = MAXD / 64;
  float acck[ND], accv[ND];
#pragma unroll
  for (int i = 0; i < ND; ++i) acck[i] = accv[i] = 0.0f;
  bool bad = false;
  const int t_end = last_query(s, j) + 1;
  for (int r = 0; r < s.rep; ++r) {
    const long q_plane = static_cast<long>(b) * s.heads + static_cast<long>(g) * s.rep + r;
    const TI* qh = q + q_plane * s.time * D;
    const TI* gh = gy + q_plane * s.time * D;
    const float* lse_h = lse + q_plane * s.time;
    const float* del_h = delta + q_plane * s.time;
    for (int t0 = j; t0 < t_end; t0 += 64) {
      const int t = t0 + lane;
      float coef = 0.0f, p = 0.0f;
      if (t < t_end) {
        const TI* qr = qh + static_cast<long>(t) * D;
        const TI* gr = gh + static_cast<long>(t) * D;
        float dot = 0.0f, dp = 0.0f;
        for (int d = 0; d < D; ++d) {
          dot += dev_load<TI>(qr, d) * k_lds[wave][d];
          dp += dev_load<TI>(gr, d) * v_lds[wave][d];
        }
        float sc = dot * s.scale;
        p = expf(sc - lse_h[t]);
        bad |= !(dev_finite(sc) && dev_finite(p));
        coef = s.scale * (p * (dp - del_h[t]));
      }
      c_lds[wave][lane] = coef;
      p_lds[wave][lane] = p;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      const int nq = min(64, t_end - t0);
#pragma unroll
      for (int i = 0; i < ND; ++i) {
        const int d = i * 64 + lane;
        if (d < D) {
          float ak = acck[i], av = accv[i];
          for (int tt = 0; tt < nq; ++tt) {
            ak += c_lds[wave][tt] * dev_load<TI>(qh, static_cast<long>(t0 + tt) * D + d);
            av += p_lds[wave][tt] * dev_load<TI>(gh, static_cast<long>(t0 + tt) * D + d);
          }
          acck[i] = ak;
          accv[i] = av;
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
#pragma unroll
  for (int i = 0; i < ND; ++i) {
    const int d = i * 64 + lane;
    if (d < D) {
      bad |= !(dev_finite(acck[i]) && dev_finite(accv[i]));
      dev_store<TO>(gk, row * D + d, acck[i]);
      dev_store<TO>(gv, row * D + d, accv[i]);
    }
  }
  if (bad) dev_raise_fault(fault, tag);
}

// ---------------------------------------------------------------- tiled f32 kernels
// The f32 tier at head dims 16 / 32 / 64 / 128: 64 query rows x 64 key rows per step, tiles staged
// in LDS (row pitch D + 4 floats, so that 16-byte reads of 16 consecutive rows fall in distinct
// banks), 256 threads as a 16 x 16 grid. Thread (ty, tx) owns the scores of query rows ty + 16 i
// and key rows tx + 16 c, and of the row-by-D results the rows ty + 16 i at columns
// VW tx + 16 VW cc. Same formulas as the row kernels above; sums run in tile order.
constexpr int ST_THREADS = 256;
constexpr int ST_WP = 68;  // pitch of the 64 x 64 weight tile

template <int D>
struct StCols {
  static constexpr int DC = D / 16;            // result columns per thread
  static constexpr int VW = DC >= 4 ? 4 : DC;  // in chunks of this many
  static constexpr int NCH = DC / VW;
};

// 64 rows of D floats starting at row r0 of a [rows, D] plane; rows past `rows` read as zeros.
template <int D>
__device__ __forceinline__ void st_load_tile(float* __restrict__ lds, const float* __restrict__ g, int r0, int rows) {
  constexpr int V4 = D / 4, P = D + 4;
  for (int idx = threadIdx.x; idx < 64 * V4; idx += ST_THREADS) {
    const int r = idx / V4, c4 = idx - r * V4;
    float4 val = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (r0 + r < rows) val = *reinterpret_cast<const float4*>(g + static_cast<long>(r0 + r) * D + 4 * c4);
    *reinterpret_cast<float4*>(lds + r * P + 4 * c4) = val;
  }
}

// s[i][c] = A[ty + 16 i] . B[tx + 16 c] over D.
template <int D>
__device__ __forceinline__ void st_dot(const float* __restrict__ A, const float* __restrict__ B, int ty, int tx,
                                       float (&s)[4][4]) {
  constexpr int P = D + 4;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int c = 0; c < 4; ++c) s[i][c] = 0.0f;
#pragma unroll 4
  for (int d = 0; d < D; d += 4) {
    float4 a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = *reinterpret_cast<const float4*>(A + (ty + 16 * i) * P + d);
#pragma unroll
    for (int c = 0; c < 4; ++c) b[c] = *reinterpret_cast<const float4*>(B + (tx + 16 * c) * P + d);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        float acc = s[i][c];
        acc = fmaf(a[i].x, b[c].x, acc);
        acc = fmaf(a[i].y, b[c].y, acc);
        acc = fmaf(a[i].z, b[c].z, acc);
        acc = fmaf(a[i].w, b[c].w, acc);
        s[i][c] = acc;
      }
  }
}

// acc[i][..] += sum over k of W[ty + 16 i][k] M[k][columns of this thread]; W is a 64 x 64 tile of
// pitch ST_WP, M a 64 x D tile.
template <int D>
__device__ __forceinline__ void st_accumulate(const float* __restrict__ W, const float* __restrict__ M, int ty, int tx,
                                              float (&acc)[4][StCols<D>::DC]) {
  constexpr int P = D + 4, VW = StCols<D>::VW, NCH = StCols<D>::NCH;
#pragma unroll 2
  for (int k = 0; k < 64; k += 4) {
    float4 w4[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w4[i] = *reinterpret_cast<const float4*>(W + (ty + 16 * i) * ST_WP + k);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      float m[NCH * VW];
#pragma unroll
      for (int cc = 0; cc < NCH; ++cc) {
        const float* src = M + (k + kk) * P + VW * tx + 16 * VW * cc;
        if constexpr (VW == 4) {
          const float4 v = *reinterpret_cast<const float4*>(src);
          m[4 * cc] = v.x; m[4 * cc + 1] = v.y; m[4 * cc + 2] = v.z; m[4 * cc + 3] = v.w;
        } else if constexpr (VW == 2) {
          const float2 v = *reinterpret_cast<const float2*>(src);
          m[0] = v.x; m[1] = v.y;
        } else {
          m[0] = src[0];
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float wv = kk == 0 ? w4[i].x : kk == 1 ? w4[i].y : kk == 2 ? w4[i].z : w4[i].w;
#pragma unroll
        for (int e = 0; e < NCH * VW; ++e) acc[i][e] = fmaf(wv, m[e], acc[i][e]);
      }
    }
  }
}

// Stores the thread's columns of row `row` of a [rows, D] plane; returns whether a value was non-finite.
template <int D>
__device__ __forceinline__ bool st_store_row(float* __restrict__ g, long row, int tx, const float (&v)[StCols<D>::DC],
                                             float scale) {
  constexpr int VW = StCols<D>::VW, NCH = StCols<D>::NCH;
  bool bad = false;
#pragma unroll
  for (int cc = 0; cc < NCH; ++cc) {
    float* dst = g + row * D + VW * tx + 16 * VW * cc;
#pragma unroll
    for (int e = 0; e < VW; ++e) {
      const float o = v[VW * cc + e] * scale;
      bad |= !dev_finite(o);
      dst[e] = o;
    }
  }
  return bad;
}

// The largest / the sum of a value over the 16 threads that share a query row.
__device__ __forceinline__ float st_row_max(float v) {
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}
__device__ __forceinline__ float st_row_sum(float v) {
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Forward: one workgroup per 64 query rows of a head.
template <int D>
__global__ __launch_bounds__(ST_THREADS) void sdpa_tiled_fwd_kernel(const float* __restrict__ q,
                                                                    const float* __restrict__ k,
                                                                    const float* __restrict__ v,
                                                                    float* __restrict__ out, float* __restrict__ lse,
                                                                    SdpaShape s, OmxFaultWord* fault,
                                                                    unsigned long long tag) {
  constexpr int P = D + 4, DC = StCols<D>::DC;
  __shared__ __align__(16) float Qs[64 * P];
  __shared__ __align__(16) float Ks[64 * P];
  __shared__ __align__(16) float Vs[64 * P];
  __shared__ __align__(16) float Ws[64 * ST_WP];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int plane = blockIdx.y, h = plane % s.heads, b = plane / s.heads;
  const long kv_plane = static_cast<long>(b) * s.kv_heads + h / s.rep;
  const float* qh = q + static_cast<long>(plane) * s.time * D;
  const float* kh = k + kv_plane * s.time * D;
  const float* vh = v + kv_plane * s.time * D;
  const int t0 = blockIdx.x * 64;
  st_load_tile<D>(Qs, qh, t0, s.time);
  float o[4][DC], mx[4], sum[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    mx[i] = -INFINITY;
    sum[i] = 0.0f;
#pragma unroll
    for (int e = 0; e < DC; ++e) o[i][e] = 0.0f;
  }
  bool bad = false;
  const int t_last = min(s.time, t0 + 64) - 1;
  const int kb_first = first_key(s, t0) / 64, kb_last = t_last / 64;
  for (int kb = kb_first; kb <= kb_last; ++kb) {
    __syncthreads();  // the previous step's reads of Ks, Vs and Ws are done
    st_load_tile<D>(Ks, kh, kb * 64, s.time);
    st_load_tile<D>(Vs, vh, kb * 64, s.time);
    __syncthreads();
    float sc[4][4];
    st_dot<D>(Qs, Ks, ty, tx, sc);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = t0 + ty + 16 * i, lo = first_key(s, t);
      float top = -INFINITY;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int j = kb * 64 + tx + 16 * c;
        const bool seen = t < s.time && j <= t && j >= lo;
        const float val = sc[i][c] * s.scale;
        bad |= seen && !dev_finite(val);
        sc[i][c] = seen ? val : -INFINITY;
        top = fmaxf(top, sc[i][c]);
      }
      top = st_row_max(top);
      const float new_max = fmaxf(mx[i], top);
      // A row that has seen no key yet keeps its empty state.
      const float rescale = new_max == -INFINITY ? 1.0f : expf(mx[i] - new_max);
      float part = 0.0f;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const float p = sc[i][c] == -INFINITY ? 0.0f : expf(sc[i][c] - new_max);
        part += p;
        Ws[(ty + 16 * i) * ST_WP + tx + 16 * c] = p;
      }
      part = st_row_sum(part);
      sum[i] = sum[i] * rescale + part;
      mx[i] = new_max;
#pragma unroll
      for (int e = 0; e < DC; ++e) o[i][e] *= rescale;
    }
    __syncthreads();
    st_accumulate<D>(Ws, Vs, ty, tx, o);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + ty + 16 * i;
    if (t < s.time) {
      bad |= !(dev_finite(sum[i]) && sum[i] > 0.0f);
      const long row = static_cast<long>(plane) * s.time + t;
      bad |= st_store_row<D>(out, row, tx, o[i], 1.0f / sum[i]);
      if (tx == 0) lse[row] = mx[i] + logf(sum[i]);
    }
  }
  if (bad) dev_raise_fault(fault, tag);
}

// The weights of one 64 x 64 step of the backward: p = e^(S - lse) and dS = scale p (dP - Dr) for
// the thread's 4 x 4 scores; `bad` gathers non-finite scores and probabilities.
struct StRows {
  float lse[4], dr[4];
};
__device__ __forceinline__ void st_backward_weights(const SdpaShape& s, int t0, int j0, int ty, int tx,
                                                    const StRows& rows, const float (&sc)[4][4],
                                                    const float (&dp)[4][4], float (&p)[4][4], float (&ds)[4][4],
                                                    bool& bad) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + ty + 16 * i, lo = first_key(s, t);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int j = j0 + tx + 16 * c;
      const bool seen = t < s.time && j <= t && j >= lo;
      const float val = sc[i][c] * s.scale;
      const float pr = seen ? expf(val - rows.lse[i]) : 0.0f;
      bad |= seen && !(dev_finite(val) && dev_finite(pr));
      p[i][c] = pr;
      ds[i][c] = seen ? s.scale * (pr * (dp[i][c] - rows.dr[i])) : 0.0f;
    }
  }
}

// dQ: one workgroup per 64 query rows of a head.
template <int D>
__global__ __launch_bounds__(ST_THREADS) void sdpa_tiled_dq_kernel(const float* __restrict__ q,
                                                                   const float* __restrict__ k,
                                                                   const float* __restrict__ v,
                                                                   const float* __restrict__ lse,
                                                                   const float* __restrict__ delta,
                                                                   const float* __restrict__ gy,
                                                                   float* __restrict__ gq, SdpaShape s,
                                                                   OmxFaultWord* fault, unsigned long long tag) {
  constexpr int P = D + 4, DC = StCols<D>::DC;
  __shared__ __align__(16) float Qs[64 * P];
  __shared__ __align__(16) float Gs[64 * P];
  __shared__ __align__(16) float Ks[64 * P];
  __shared__ __align__(16) float Vs[64 * P];
  __shared__ __align__(16) float Ws[64 * ST_WP];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int plane = blockIdx.y, h = plane % s.heads, b = plane / s.heads;
  const long kv_plane = static_cast<long>(b) * s.kv_heads + h / s.rep;
  const long row0 = static_cast<long>(plane) * s.time;
  const float* kh = k + kv_plane * s.time * D;
  const float* vh = v + kv_plane * s.time * D;
  const int t0 = blockIdx.x * 64;
  st_load_tile<D>(Qs, q + row0 * D, t0, s.time);
  st_load_tile<D>(Gs, gy + row0 * D, t0, s.time);
  bool bad = false;
  StRows rows;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + ty + 16 * i;
    rows.lse[i] = t < s.time ? lse[row0 + t] : 0.0f;
    rows.dr[i] = t < s.time ? delta[row0 + t] : 0.0f;
    bad |= !(dev_finite(rows.lse[i]) && dev_finite(rows.dr[i]));
  }
  float acc[4][DC];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < DC; ++e) acc[i][e] = 0.0f;
  const int t_last = min(s.time, t0 + 64) - 1;
  const int kb_first = first_key(s, t0) / 64, kb_last = t_last / 64;
  for (int kb = kb_first; kb <= kb_last; ++kb) {
    __syncthreads();
    st_load_tile<D>(Ks, kh, kb * 64, s.time);
    st_load_tile<D>(Vs, vh, kb * 64, s.time);
    __syncthreads();
    float sc[4][4], dp[4][4], p[4][4], ds[4][4];
    st_dot<D>(Qs, Ks, ty, tx, sc);
    st_dot<D>(Gs, Vs, ty, tx, dp);
    st_backward_weights(s, t0, kb * 64, ty, tx, rows, sc, dp, p, ds, bad);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int c = 0; c < 4; ++c) Ws[(ty + 16 * i) * ST_WP + tx + 16 * c] = ds[i][c];
    __syncthreads();
    st_accumulate<D>(Ws, Ks, ty, tx, acc);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + ty + 16 * i;
    if (t < s.time) bad |= st_store_row<D>(gq, row0 + t, tx, acc[i], 1.0f);
  }
  if (bad) dev_raise_fault(fault, tag);
}

// dK, dV: one workgroup per 64 key rows of a KV head; the query heads of the group in ascending
// order and, within a head, query blocks in ascending order.
template <int D>
__global__ __launch_bounds__(ST_THREADS) void sdpa_tiled_dkv_kernel(const float* __restrict__ q,
                                                                    const float* __restrict__ k,
                                                                    const float* __restrict__ v,
                                                                    const float* __restrict__ lse,
                                                                    const float* __restrict__ delta,
                                                                    const float* __restrict__ gy,
                                                                    float* __restrict__ gk, float* __restrict__ gv,
                                                                    SdpaShape s, OmxFaultWord* fault,
                                                                    unsigned long long tag) {
  constexpr int P = D + 4, DC = StCols<D>::DC;
  __shared__ __align__(16) float Qs[64 * P];
  __shared__ __align__(16) float Gs[64 * P];
  __shared__ __align__(16) float Ks[64 * P];
  __shared__ __align__(16) float Vs[64 * P];
  __shared__ __align__(16) float Wt[64 * ST_WP];  // [key][query]
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int kv_plane = blockIdx.y, g = kv_plane % s.kv_heads, b = kv_plane / s.kv_heads;
  const long kv_row0 = static_cast<long>(kv_plane) * s.time;
  const int j0 = blockIdx.x * 64;
  st_load_tile<D>(Ks, k + kv_row0 * D, j0, s.time);
  st_load_tile<D>(Vs, v + kv_row0 * D, j0, s.time);
  float acck[4][DC], accv[4][DC];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < DC; ++e) acck[i][e] = accv[i][e] = 0.0f;
  bool bad = false;
  const int j_last = min(s.time, j0 + 64) - 1;
  const int qb_last = last_query(s, j_last) / 64;
  for (int r = 0; r < s.rep; ++r) {
    const long row0 = (static_cast<long>(b) * s.heads + static_cast<long>(g) * s.rep + r) * s.time;
    for (int qb = blockIdx.x; qb <= qb_last; ++qb) {
      const int t0 = qb * 64;
      __syncthreads();  // the previous step's reads of Qs, Gs and Wt are done
      st_load_tile<D>(Qs, q + row0 * D, t0, s.time);
      st_load_tile<D>(Gs, gy + row0 * D, t0, s.time);
      StRows rows;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int t = t0 + ty + 16 * i;
        rows.lse[i] = t < s.time ? lse[row0 + t] : 0.0f;
        rows.dr[i] = t < s.time ? delta[row0 + t] : 0.0f;
      }
      __syncthreads();
      float sc[4][4], dp[4][4], p[4][4], ds[4][4];
      st_dot<D>(Qs, Ks, ty, tx, sc);
      st_dot<D>(Gs, Vs, ty, tx, dp);
      st_backward_weights(s, t0, j0, ty, tx, rows, sc, dp, p, ds, bad);
      // dV += P^T dO
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) Wt[(tx + 16 * c) * ST_WP + ty + 16 * i] = p[i][c];
      __syncthreads();
      st_accumulate<D>(Wt, Gs, ty, tx, accv);
      __syncthreads();
      // dK += dS^T Q
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) Wt[(tx + 16 * c) * ST_WP + ty + 16 * i] = ds[i][c];
      __syncthreads();
      st_accumulate<D>(Wt, Qs, ty, tx, acck);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int j = j0 + ty + 16 * i;
    if (j < s.time) {
      bad |= st_store_row<D>(gk, kv_row0 + j, tx, acck[i], 1.0f);
      bad |= st_store_row<D>(gv, kv_row0 + j, tx, accv[i], 1.0f);
    }
  }
  if (bad) dev_raise_fault(fault, tag);
}

// The tiled kernels put the (batch, head) plane in grid.y, which holds at most 65535: more planes
// than that (many short sequences) go to the row kernels, whose grids are one-dimensional.
bool sdpa_tiled_supports(uint64_t dim, uint64_t planes, std::initializer_list<int32_t> dtypes, std::initializer_list<const void*> ptrs) {
  if (dim != 16 && dim != 32 && dim != 64 && dim != 128) return false;
  if (planes > 65535) return false;
  for (int32_t d : dtypes)
    if (d != OMX_F32) return false;
  for (const void* p : ptrs)
    if (reinterpret_cast<uintptr_t>(p) & 15u) return false;
  return true;
}

int32_t check_shape(omx_ctx* ctx, const char* op, uint64_t batch, uint64_t heads, uint64_t kv_heads, uint64_t time,
                    uint64_t dim, uint64_t window, SdpaShape* s) {
  if (batch == 0 || heads == 0 || kv_heads == 0 || time == 0 || dim == 0)
    return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (kv_heads > heads || heads % kv_heads != 0)
    return omx_fail(ctx, OMX_SHAPE, "%s: heads %llu is not a multiple of kv heads %llu", op,
                    (unsigned long long)heads, (unsigned long long)kv_heads);
  if (dim > MAXD) return omx_fail(ctx, OMX_UNSUPPORTED_HEAD_DIM, "head_dim %llu limit %d", (unsigned long long)dim, MAXD);
  if (batch * heads * time > 0x7fffffffull || time > 0x3fffffffull)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: B*H*T does not fit in i32", op);
  s->batch = static_cast<int>(batch);
  s->heads = static_cast<int>(heads);
  s->kv_heads = static_cast<int>(kv_heads);
  s->time = static_cast<int>(time);
  s->dim = static_cast<int>(dim);
  // A window of at least T is every earlier key (attn.rs:745).
  s->window = (window == 0 || window >= time) ? 0 : static_cast<int>(window);
  s->rep = static_cast<int>(heads / kv_heads);
  s->scale = 1.0f / sqrtf(static_cast<float>(static_cast<uint32_t>(dim)));
  return OMX_OK;
}

}  // namespace

extern "C" {

int32_t omx_causal_sdpa_forward(omx_ctx* ctx, const void* q, const void* k, const void* v, int32_t operand_dtype,
                                void* out, int32_t out_dtype, void* lse, uint64_t batch, uint64_t heads,
                                uint64_t kv_heads, uint64_t time, uint64_t head_dim, uint64_t window) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "causal_sdpa_forward";
  if (!q || !k || !v || !out || !lse) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(operand_dtype) || !omx_valid_float_dtype(out_dtype))
    return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  SdpaShape s;
  int32_t rc = check_shape(ctx, op, batch, heads, kv_heads, time, head_dim, window, &s);
  if (rc != OMX_OK) return rc;
  unsigned long long tag = omx_tag(ctx, F_SDPA_FORWARD);
  if (omx_flash_sdpa_supports(head_dim, operand_dtype))
    return omx_flash_sdpa_forward(ctx, q, k, v, out, out_dtype, nullptr, static_cast<float*>(lse), batch, heads,
                                  kv_heads, time, head_dim, s.window, s.scale, tag, nullptr);
  if (ctx->sdpa_tiled && sdpa_tiled_supports(head_dim, batch * heads, {operand_dtype, out_dtype}, {q, k, v, out})) {
    dim3 tgrid(static_cast<unsigned>((time + 63) / 64), static_cast<unsigned>(batch * heads));
#define SDPA_TILED_FWD(D_)                                                                                      \
  hipLaunchKernelGGL((sdpa_tiled_fwd_kernel<D_>), tgrid, dim3(ST_THREADS), 0, ctx->stream,                      \
                     static_cast<const float*>(q), static_cast<const float*>(k), static_cast<const float*>(v),  \
                     static_cast<float*>(out), static_cast<float*>(lse), s, ctx->fault, tag)
    if (head_dim == 16) SDPA_TILED_FWD(16);
    else if (head_dim == 32) SDPA_TILED_FWD(32);
    else if (head_dim == 64) SDPA_TILED_FWD(64);
    else SDPA_TILED_FWD(128);
#undef SDPA_TILED_FWD
    OMX_LAUNCH_CHECK(ctx, "sdpa_tiled_fwd_kernel");
    return OMX_OK;
  }
  const long rows = static_cast<long>(batch) * heads * time;
  dim3 grid(static_cast<unsigned>((rows + 3) / 4)), block(SD_THREADS);
#define SDPA_FWD(TI, TO)                                                                                          \
  hipLaunchKernelGGL((sdpa_fwd_rows_kernel<TI, TO>), grid, block, 0, ctx->stream, static_cast<const TI*>(q),      \
                     static_cast<const TI*>(k), static_cast<const TI*>(v), static_cast<TO*>(out),                 \
                     static_cast<float*>(lse), s, ctx->fault, tag)
  if (operand_dtype == OMX_F32 && out_dtype == OMX_F32) SDPA_FWD(float, float);
  else if (operand_dtype == OMX_F32) SDPA_FWD(float, unsigned short);
  else if (out_dtype == OMX_F32) SDPA_FWD(unsigned short, float);
  else SDPA_FWD(unsigned short, unsigned short);
#undef SDPA_FWD
  OMX_LAUNCH_CHECK(ctx, "sdpa_fwd_rows_kernel");
  return OMX_OK;
}

int32_t omx_causal_sdpa_backward(omx_ctx* ctx, const void* q, const void* k, const void* v, const void* out,
                                 const void* lse, const void* gy, int32_t operand_dtype, int32_t out_dtype,
                                 int32_t gy_dtype, void* gq, void* gk, void* gv, int32_t grad_dtype, uint64_t batch,
                                 uint64_t heads, uint64_t kv_heads, uint64_t time, uint64_t head_dim,
                                 uint64_t window) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "causal_sdpa_backward";
  if (!q || !k || !v || !out || !lse || !gy || !gq || !gk || !gv)
    return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(operand_dtype) || !omx_valid_float_dtype(grad_dtype) ||
      !omx_valid_float_dtype(out_dtype) || !omx_valid_float_dtype(gy_dtype))
    return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  SdpaShape s;
  int32_t rc = check_shape(ctx, op, batch, heads, kv_heads, time, head_dim, window, &s);
  if (rc != OMX_OK) return rc;
  unsigned long long tag = omx_tag(ctx, F_SDPA_BACKWARD);
  const long rows = static_cast<long>(batch) * heads * time;
  const uint64_t n = static_cast<uint64_t>(rows) * head_dim;
  if (omx_flash_sdpa_supports(head_dim, operand_dtype)) {
    // The MFMA kernels read bf16: an f32 output goes in as bf16 + rounding residual (nothing of it
    // is lost to the row term dO . O), an f32 grad_output rounded to bf16.
    const void* out16 = out;
    const void* residual = nullptr;
    const void* gy16 = gy;
    if (out_dtype == OMX_F32 || gy_dtype == OMX_F32) {
      void* ws = nullptr;
      rc = omx_workspace(ctx, 3 * n * 2, &ws, 1);
      if (rc != OMX_OK) return rc;
      unsigned short* base = static_cast<unsigned short*>(ws);
      if (out_dtype == OMX_F32) {
        const unsigned blocks = static_cast<unsigned>(std::min<uint64_t>((n + 255) / 256, 65536));
        hipLaunchKernelGGL(sdpa_split_output_kernel, dim3(blocks), dim3(256), 0, ctx->stream,
                           static_cast<const float*>(out), base, base + n, static_cast<long>(n));
        OMX_LAUNCH_CHECK(ctx, "sdpa_split_output_kernel");
        out16 = base;
        residual = base + n;
      }
      if (gy_dtype == OMX_F32) {
        rc = omx_convert(ctx, gy, OMX_F32, base + 2 * n, OMX_BF16, n);
        if (rc != OMX_OK) return rc;
        gy16 = base + 2 * n;
      }
    }
    return omx_flash_sdpa_backward(ctx, q, k, v, out16, residual, static_cast<const float*>(lse), gy16, gq, gk, gv,
                                   grad_dtype, batch, heads, kv_heads, time, head_dim, s.window, s.scale, tag, nullptr);
  }
  const long kv_rows = static_cast<long>(batch) * kv_heads * time;
  void* ws = nullptr;
  rc = omx_workspace(ctx, rows * sizeof(float), &ws);
  if (rc != OMX_OK) return rc;
  float* delta = static_cast<float*>(ws);
  dim3 grid(static_cast<unsigned>((rows + 3) / 4)), kv_grid(static_cast<unsigned>((kv_rows + 3) / 4)), block(SD_THREADS);
  const float* lsef = static_cast<const float*>(lse);
  // The row term reads out and grad_output as they are stored; the two passes read grad_output in
  // the operands' storage type.
#define SDPA_DELTA(TOUT, TGY)                                                                                 \
  hipLaunchKernelGGL((sdpa_delta_kernel<TOUT, TGY>), grid, block, 0, ctx->stream, static_cast<const TOUT*>(out), \
                     static_cast<const TGY*>(gy), delta, rows, s.dim)
  if (out_dtype == OMX_F32 && gy_dtype == OMX_F32) SDPA_DELTA(float, float);
  else if (out_dtype == OMX_F32) SDPA_DELTA(float, unsigned short);
  else if (gy_dtype == OMX_F32) SDPA_DELTA(unsigned short, float);
  else SDPA_DELTA(unsigned short, unsigned short);
#undef SDPA_DELTA
  OMX_LAUNCH_CHECK(ctx, "sdpa_delta_kernel");
  if (gy_dtype != operand_dtype) {
    void* conv = nullptr;
    rc = omx_workspace(ctx, n * omx_dtype_size(operand_dtype), &conv, 1);
    if (rc != OMX_OK) return rc;
    rc = omx_convert(ctx, gy, gy_dtype, conv, operand_dtype, n);
    if (rc != OMX_OK) return rc;
    gy = conv;
  }
  if (ctx->sdpa_tiled && sdpa_tiled_supports(head_dim, batch * heads, {operand_dtype, grad_dtype}, {q, k, v, gy, gq, gk, gv})) {
    dim3 qgrid(static_cast<unsigned>((time + 63) / 64), static_cast<unsigned>(batch * heads));
    dim3 kgrid(static_cast<unsigned>((time + 63) / 64), static_cast<unsigned>(batch * kv_heads));
#define SDPA_TILED_BWD(D_)                                                                                          \
  do {                                                                                                              \
    hipLaunchKernelGGL((sdpa_tiled_dq_kernel<D_>), qgrid, dim3(ST_THREADS), 0, ctx->stream,                         \
                       static_cast<const float*>(q), static_cast<const float*>(k), static_cast<const float*>(v),    \
                       lsef, delta, static_cast<const float*>(gy), static_cast<float*>(gq), s, ctx->fault, tag);    \
    hipLaunchKernelGGL((sdpa_tiled_dkv_kernel<D_>), kgrid, dim3(ST_THREADS), 0, ctx->stream,                        \
                       static_cast<const float*>(q), static_cast<const float*>(k), static_cast<const float*>(v),    \
                       lsef, delta, static_cast<const float*>(gy), static_cast<float*>(gk), static_cast<float*>(gv), \
                       s, ctx->fault, tag);                                                                         \
  } while (0)
    if (head_dim == 16) SDPA_TILED_BWD(16);
    else if (head_dim == 32) SDPA_TILED_BWD(32);
    else if (head_dim == 64) SDPA_TILED_BWD(64);
    else SDPA_TILED_BWD(128);
#undef SDPA_TILED_BWD
    OMX_LAUNCH_CHECK(ctx, "sdpa tiled backward kernels");
    return OMX_OK;
  }
#define SDPA_BWD(TI, TO)                                                                                              \
  do {                                                                                                                \
    hipLaunchKernelGGL((sdpa_bwd_dq_rows_kernel<TI, TO>), grid, block, 0, ctx->stream, static_cast<const TI*>(q),     \
                       static_cast<const TI*>(k), static_cast<const TI*>(v), lsef, delta, static_cast<const TI*>(gy), \
                       static_cast<TO*>(gq), s, ctx->fault, tag);                                                     \
    hipLaunchKernelGGL((sdpa_bwd_dkv_rows_kernel<TI, TO>), kv_grid, block, 0, ctx->stream,                            \
                       static_cast<const TI*>(q), static_cast<const TI*>(k), static_cast<const TI*>(v), lsef, delta,  \
                       static_cast<const TI*>(gy), static_cast<TO*>(gk), static_cast<TO*>(gv), s, ctx->fault, tag);   \
  } while (0)
  if (operand_dtype == OMX_F32 && grad_dtype == OMX_F32) SDPA_BWD(float, float);
  else if (operand_dtype == OMX_F32) SDPA_BWD(float, unsigned short);
  else if (grad_dtype == OMX_F32) SDPA_BWD(unsigned short, float);
  else SDPA_BWD(unsigned short, unsigned short);
#undef SDPA_BWD
  OMX_LAUNCH_CHECK(ctx, "sdpa backward row kernels");
  return OMX_OK;
}

int32_t omx_causal_sdpa_backward_recompute(omx_ctx* ctx, const void* q, const void* k, const void* v, const void* gy,
                                           int32_t operand_dtype, int32_t gy_dtype, void* gq, void* gk, void* gv,
                                           int32_t grad_dtype, uint64_t batch, uint64_t heads, uint64_t kv_heads,
                                           uint64_t time, uint64_t head_dim, uint64_t window) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "causal_sdpa_backward_recompute";
  // The gradient's arguments are checked before the forward runs (backend.rs:1781-1792).
  if (!q || !k || !v || !gy || !gq || !gk || !gv) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(operand_dtype) || !omx_valid_float_dtype(grad_dtype) || !omx_valid_float_dtype(gy_dtype))
    return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  SdpaShape s;
  int32_t rc = check_shape(ctx, op, batch, heads, kv_heads, time, head_dim, window, &s);
  if (rc != OMX_OK) return rc;
  // The forward's output stays f32 (the unrounded O the row term needs) in the library's own scratch.
  const uint64_t rows = batch * heads * time;
  const uint64_t out_bytes = (rows * head_dim * 4 + 255) & ~255ull;
  void* ws = nullptr;
  rc = omx_workspace(ctx, out_bytes + rows * 4, &ws, 2);
  if (rc != OMX_OK) return rc;
  void* out = ws;
  void* lse = static_cast<char*>(ws) + out_bytes;
  rc = omx_causal_sdpa_forward(ctx, q, k, v, operand_dtype, out, OMX_F32, lse, batch, heads, kv_heads, time, head_dim,
                               window);
  if (rc != OMX_OK) return rc;
  return omx_causal_sdpa_backward(ctx, q, k, v, out, lse, gy, operand_dtype, OMX_F32, gy_dtype, gq, gk, gv, grad_dtype,
                                  batch, heads, kv_heads, time, head_dim, window);
}

// Time-major attention: the permute -> causal_sdpa -> permute of
// ojas-model/src/block.rs:186-199 (causal_attention) in one pass over [B, T, heads, D] tensors.
static int32_t check_attention(omx_ctx* ctx, const char* op, int32_t operand_dtype, uint64_t head_dim, uint64_t heads,
                               uint64_t kv_heads, uint64_t q_pitch, uint64_t kv_pitch, uint64_t out_pitch,
                               std::initializer_list<const void*> ptrs) {
  for (const void* p : ptrs) {
    if (!p) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
    if (reinterpret_cast<uintptr_t>(p) & 15u) return omx_fail(ctx, OMX_SHAPE, "%s: tensor not 16-byte aligned", op);
  }
  if (!omx_flash_sdpa_supports(head_dim, operand_dtype))
    return omx_fail(ctx, OMX_UNSUPPORTED, "%s: only bf16 operands with head_dim 64 (compose permute and causal_sdpa)",
                    op);
  if (q_pitch < heads * head_dim || out_pitch < heads * head_dim || kv_pitch < kv_heads * head_dim ||
      (q_pitch | kv_pitch | out_pitch) % 8 != 0)
    return omx_fail(ctx, OMX_SHAPE, "%s: row pitch below heads * head_dim or not a multiple of 8", op);
  return OMX_OK;
}

static int32_t attention_forward(omx_ctx* ctx, const char* op, const void* q, uint64_t q_pitch, const void* k,
                                 const void* v, uint64_t kv_pitch, int32_t operand_dtype, void* out,
                                 void* out_residual, uint64_t out_pitch, int32_t out_dtype, void* lse, uint64_t batch,
                                 uint64_t time, uint64_t heads, uint64_t kv_heads, uint64_t head_dim, uint64_t window) {
  OMX_REQUIRE_CTX(ctx);
  if (out_dtype != OMX_BF16) return omx_fail(ctx, OMX_DTYPE, "%s: output must be bf16", op);
  SdpaShape s;
  int32_t rc = check_shape(ctx, op, batch, heads, kv_heads, time, head_dim, window, &s);
  if (rc != OMX_OK) return rc;
  rc = check_attention(ctx, op, operand_dtype, head_dim, heads, kv_heads, q_pitch, kv_pitch, out_pitch,
                       {q, k, v, out, lse});
  if (rc != OMX_OK) return rc;
  if (reinterpret_cast<uintptr_t>(out_residual) & 15u)
    return omx_fail(ctx, OMX_SHAPE, "%s: tensor not 16-byte aligned", op);
  const long D = static_cast<long>(head_dim), T = static_cast<long>(time);
  const long strides[9] = {static_cast<long>(q_pitch),   D, T * static_cast<long>(q_pitch),
                           static_cast<long>(kv_pitch),  D, T * static_cast<long>(kv_pitch),
                           static_cast<long>(out_pitch), D, T * static_cast<long>(out_pitch)};
  return omx_flash_sdpa_forward(ctx, q, k, v, out, out_dtype, out_residual, static_cast<float*>(lse), batch, heads,
                                kv_heads, time, head_dim, s.window, s.scale, omx_tag(ctx, F_SDPA_FORWARD), strides);
}

static int32_t attention_backward(omx_ctx* ctx, const char* op, const void* q, uint64_t q_pitch, const void* k,
                                  const void* v, uint64_t kv_pitch, const void* out, const void* out_residual,
                                  const void* gy, uint64_t out_pitch, const void* lse, int32_t operand_dtype, void* gq,
                                  void* gk, void* gv, int32_t grad_dtype, uint64_t batch, uint64_t time, uint64_t heads,
                                  uint64_t kv_heads, uint64_t head_dim, uint64_t window) {
  OMX_REQUIRE_CTX(ctx);
  if (grad_dtype != OMX_BF16) return omx_fail(ctx, OMX_DTYPE, "%s: gradients must be bf16", op);
  SdpaShape s;
  int32_t rc = check_shape(ctx, op, batch, heads, kv_heads, time, head_dim, window, &s);
  if (rc != OMX_OK) return rc;
  rc = check_attention(ctx, op, operand_dtype, head_dim, heads, kv_heads, q_pitch, kv_pitch, out_pitch,
                       {q, k, v, out, gy, lse, gq, gk, gv});
  if (rc != OMX_OK) return rc;
  if (reinterpret_cast<uintptr_t>(out_residual) & 15u)
    return omx_fail(ctx, OMX_SHAPE, "%s: tensor not 16-byte aligned", op);
  const long D = static_cast<long>(head_dim), T = static_cast<long>(time);
  const long strides[9] = {static_cast<long>(q_pitch),   D, T * static_cast<long>(q_pitch),
                           static_cast<long>(kv_pitch),  D, T * static_cast<long>(kv_pitch),
                           static_cast<long>(out_pitch), D, T * static_cast<long>(out_pitch)};
  return omx_flash_sdpa_backward(ctx, q, k, v, out, out_residual, static_cast<const float*>(lse), gy, gq, gk, gv,
                                 grad_dtype, batch, heads, kv_heads, time, head_dim, s.window, s.scale,
                                 omx_tag(ctx, F_SDPA_BACKWARD), strides);
}

int32_t omx_causal_attention_forward(omx_ctx* ctx, const void* q, uint64_t q_pitch, const void* k, const void* v,
                                     uint64_t kv_pitch, int32_t operand_dtype, void* out, uint64_t out_pitch,
                                     int32_t out_dtype, void* lse, uint64_t batch, uint64_t time, uint64_t heads,
                                     uint64_t kv_heads, uint64_t head_dim, uint64_t window) {
  return attention_forward(ctx, "causal_attention_forward", q, q_pitch, k, v, kv_pitch, operand_dtype, out, nullptr,
                           out_pitch, out_dtype, lse, batch, time, heads, kv_heads, head_dim, window);
}

int32_t omx_causal_attention_backward(omx_ctx* ctx, const void* q, uint64_t q_pitch, const void* k, const void* v,
                                      uint64_t kv_pitch, const void* out, const void* gy, uint64_t out_pitch,
                                      const void* lse, int32_t operand_dtype, void* gq, void* gk, void* gv,
                                      int32_t grad_dtype, uint64_t batch, uint64_t time, uint64_t heads,
                                      uint64_t kv_heads, uint64_t head_dim, uint64_t window) {
  return attention_backward(ctx, "causal_attention_backward", q, q_pitch, k, v, kv_pitch, out, nullptr, gy, out_pitch,
                            lse, operand_dtype, gq, gk, gv, grad_dtype, batch, time, heads, kv_heads, head_dim, window);
}

int32_t omx_causal_attention_forward_saving(omx_ctx* ctx, const void* q, uint64_t q_pitch, const void* k,
                                            const void* v, uint64_t kv_pitch, int32_t operand_dtype, void* out,
                                            void* out_residual, uint64_t out_pitch, int32_t out_dtype, void* lse,
                                            uint64_t batch, uint64_t time, uint64_t heads, uint64_t kv_heads,
                                            uint64_t head_dim, uint64_t window) {
  const char* op = "causal_attention_forward_saving";
  if (ctx && !out_residual) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  return attention_forward(ctx, op, q, q_pitch, k, v, kv_pitch, operand_dtype, out, out_residual, out_pitch, out_dtype,
                           lse, batch, time, heads, kv_heads, head_dim, window);
}

int32_t omx_causal_attention_backward_saved(omx_ctx* ctx, const void* q, uint64_t q_pitch, const void* k,
                                            const void* v, uint64_t kv_pitch, const void* out,
                                            const void* out_residual, const void* gy, uint64_t out_pitch,
                                            const void* lse, int32_t operand_dtype, void* gq, void* gk, void* gv,
                                            int32_t grad_dtype, uint64_t batch, uint64_t time, uint64_t heads,
                                            uint64_t kv_heads, uint64_t head_dim, uint64_t window) {
  const char* op = "causal_attention_backward_saved";
  if (ctx && !out_residual) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  return attention_backward(ctx, op, q, q_pitch, k, v, kv_pitch, out, out_residual, gy, out_pitch, lse, operand_dtype,
                            gq, gk, gv, grad_dtype, batch, time, heads, kv_heads, head_dim, window);
}

}  // extern "C"
