// RMSNorm for row widths 256..2048 with 16-byte accesses, optionally fused with
// the residual add in front of it (forward) or behind it (backward).
//
// Reference semantics: ojas-cpu/src/norm.rs:24-204 (rms_norm_forward /
// _backward, trait backend.rs:1658-1672) and ojas-cpu/src/accum.rs:31-106
// (residual_add_forward). The fused forms are the two-op sequences of
// ojas-model/src/block.rs:247-249 (x = add(x, o); h = rms_norm(x)) and of the
// tape's gradient fan-in at a residual (ojas-autograd/src/tape.rs:2565-2591:
// grad_x = grad_from_add + grad_from_norm), with the same arithmetic per
// element as the separate kernels, so the results are the same bits.
//
// One wave owns a row; lane l owns columns 256 j + 4 l .. + 3 of chunk j, so a
// wave's loads are contiguous 1 KiB (f32) runs and the row stays in registers
// between the sum-of-squares pass and the scaling pass.
#include "omx_common.h"

namespace {

constexpr int RV_THREADS = 256;

template <typename TX, typename TA, typename TY, int NCH>
__global__ __launch_bounds__(RV_THREADS) void rms_fwd_vec_kernel(const TX* __restrict__ x, const TA* __restrict__ add,
                                                                 const float* __restrict__ w,
                                                                 float* __restrict__ sum_out, TY* __restrict__ y,
                                                                 size_t rows, int dim, float eps, OmxFaultWord* fault,
                                                                 unsigned long long tag) {
  const int lane = threadIdx.x & 63;
  const size_t row = static_cast<size_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const size_t base = row * dim;
  float xv[NCH][4];
  float ss = 0.0f;
  bool bad = false;
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const int c = j * 256 + lane * 4;
    if (c < dim) {
      dev_load4<TX>(x, base + c, xv[j]);
      if (add) {
        float av[4];
        dev_load4<TA>(add, base + c, av);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          xv[j][e] = xv[j][e] + av[e];
          bad |= !dev_finite(xv[j][e]);
        }
        dev_store4<float>(sum_out, base + c, xv[j]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) xv[j][e] = 0.0f;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) ss += xv[j][e] * xv[j][e];
  }
  ss = wave_sum(ss);
  const float denom = ss / static_cast<float>(dim) + eps;
  const float rstd = 1.0f / sqrtf(denom);
  bad |= !(dev_finite(denom) && denom > 0.0f && dev_finite(rstd));
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const int c = j * 256 + lane * 4;
    if (c < dim) {
      float wv[4], out[4];
      dev_load4<float>(w, c, wv);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        out[e] = xv[j][e] * rstd * wv[e];
        bad |= !dev_finite(out[e]);
      }
      dev_store4<TY>(y, base + c, out);
    }
  }
  if (bad) dev_raise_fault(fault, tag);
}

// Four elements as they sit in memory: the row waits in registers in this form between the passes
// (a bf16 operand at half the registers of its f32 values).
template <typename T>
struct Raw4 {
  float4 q;
  __device__ __forceinline__ void load(const T* p) { q = *reinterpret_cast<const float4*>(p); }
  __device__ __forceinline__ void clear() { q = make_float4(0.0f, 0.0f, 0.0f, 0.0f); }
  __device__ __forceinline__ void get(float (&v)[4]) const { v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w; }
};
template <>
struct Raw4<unsigned short> {
  uint2 q;
  __device__ __forceinline__ void load(const unsigned short* p) { q = *reinterpret_cast<const uint2*>(p); }
  __device__ __forceinline__ void clear() { q = make_uint2(0u, 0u); }
  __device__ __forceinline__ void get(float (&v)[4]) const {
    v[0] = __uint_as_float(q.x << 16); v[1] = __uint_as_float(q.x & 0xffff0000u);
    v[2] = __uint_as_float(q.y << 16); v[3] = __uint_as_float(q.y & 0xffff0000u);
  }
};

// gx = rms_norm_backward(x, w, gy) (+ add_in), optionally also stored as bf16;
// per-block partial column sums of gy * xhat for the weight gradient.
// Row bases are wave-uniform (scalar registers) and lane offsets 32 bits wide; all of a row's loads
// (the gradient to add included) are issued before the first reduction. FULL: dim == 256 NCH, no
// column guards. WIDE (rows above 1024 columns): the weight row is read again in each pass instead
// of waiting in registers and the lane's column sums wait in LDS, so that enough waves fit a SIMD
// to keep the loads in flight.
template <typename TX, typename TG, typename TO, int NCH, bool WIDE, bool FULL>
__global__ __launch_bounds__(RV_THREADS) void rms_bwd_vec_kernel(
    const TX* __restrict__ x, const float* __restrict__ w, const TG* __restrict__ gy, const float* __restrict__ add_in,
    TO* __restrict__ gx, unsigned short* __restrict__ gx16, float* __restrict__ partial, size_t rows, int dim,
    float eps, int rows_per_block, OmxFaultWord* fault, unsigned long long tag) {
  const bool want_w = partial != nullptr;  // a frozen weight: no column sums
  extern __shared__ float lds[];  // [4][dim]
  const unsigned lane = threadIdx.x & 63;
  const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const unsigned udim = FULL ? NCH * 256u : static_cast<unsigned>(dim);
  const float inv_dim = 1.0f / static_cast<float>(dim);
  constexpr int NW = WIDE ? 1 : NCH;
  float wv[NW][4], accw[NW][4];
  float* mine = lds + static_cast<size_t>(wave) * udim;
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const unsigned c = j * 256 + lane * 4;
    if constexpr (WIDE) {
      if (want_w && (FULL || c < udim)) *reinterpret_cast<float4*>(mine + c) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        wv[j][e] = 0.0f;
        accw[j][e] = 0.0f;
      }
      if (FULL || c < udim) dev_load4<float>(w, c, wv[j]);
    }
  }
  bool bad = false;
  const size_t first = static_cast<size_t>(blockIdx.x) * rows_per_block;
  const size_t last = min(rows, first + rows_per_block);
  for (size_t row = first + wave; row < last; row += 4) {
    const size_t base = row * udim;
    const TX* xr = x + base;
    const TG* gr = gy + base;
    // The weight row's address passes through an opaque scalar so its loads stay inside the loop.
    size_t wofs = 0;
    if constexpr (WIDE) asm volatile("" : "+s"(wofs));
    const float* wr = w + wofs;
    Raw4<TX> xq[NCH];
    Raw4<TG> gq[NCH];
    Raw4<float> aq[NCH];
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const unsigned c = j * 256 + lane * 4;
      if (FULL || c < udim) {
        xq[j].load(xr + c);
        gq[j].load(gr + c);
      } else {
        xq[j].clear();
        gq[j].clear();
      }
    }
    if (add_in) {
      const float* ar = add_in + base;
#pragma unroll
      for (int j = 0; j < NCH; ++j) {
        const unsigned c = j * 256 + lane * 4;
        if (FULL || c < udim) aq[j].load(ar + c);
        else aq[j].clear();
      }
    } else {
#pragma unroll
      for (int j = 0; j < NCH; ++j) aq[j].clear();
    }
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      float xv[4];
      xq[j].get(xv);
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += xv[e] * xv[e];
    }
    ss = wave_sum(ss);
    const float denom = ss * inv_dim + eps;
    const float rstd = 1.0f / sqrtf(denom);
    bad |= !(dev_finite(denom) && denom > 0.0f && dev_finite(rstd));
    float dot = 0.0f;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const unsigned c = j * 256 + lane * 4;
      float xv[4], gv[4], ww[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      xq[j].get(xv);
      gq[j].get(gv);
      if constexpr (WIDE) {
        if (FULL || c < udim) dev_load4<float>(wr, c, ww);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) dot += (gv[e] * (WIDE ? ww[e] : wv[WIDE ? 0 : j][e])) * (xv[e] * rstd);
    }
    dot = wave_sum(dot);
    const float mean = dot * inv_dim;
    TO* outr = gx + base;
    unsigned short* out16r = gx16 + (gx16 ? base : 0);
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const unsigned c = j * 256 + lane * 4;
      float xv[4], gv[4], ww[4] = {0.0f, 0.0f, 0.0f, 0.0f}, out[4], aw[4];
      xq[j].get(xv);
      gq[j].get(gv);
      if constexpr (WIDE) {
        if (FULL || c < udim) dev_load4<float>(wr, c, ww);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float xhat = xv[e] * rstd;
        out[e] = (gv[e] * (WIDE ? ww[e] : wv[WIDE ? 0 : j][e]) - xhat * mean) * rstd;
        aw[e] = gv[e] * xhat;
      }
      if constexpr (!WIDE) {
#pragma unroll
        for (int e = 0; e < 4; ++e) accw[j][e] += aw[e];
      }
      if (add_in) {
        float av[4];
        aq[j].get(av);
#pragma unroll
        for (int e = 0; e < 4; ++e) out[e] = av[e] + out[e];
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) bad |= !dev_finite(out[e]);
      if (FULL || c < udim) {
        if constexpr (WIDE) {
          if (want_w) {
            float4 a = *reinterpret_cast<const float4*>(mine + c);
            a.x += aw[0]; a.y += aw[1]; a.z += aw[2]; a.w += aw[3];
            *reinterpret_cast<float4*>(mine + c) = a;
          }
        }
        dev_store4<TO>(outr, c, out);
        if (gx16) dev_store4<unsigned short>(out16r, c, out);
      }
    }
  }
  if (want_w) {  // uniform over the grid
    if constexpr (!WIDE) {
#pragma unroll
      for (int j = 0; j < NCH; ++j) {
        const unsigned c = j * 256 + lane * 4;
        if (FULL || c < udim) dev_store4<float>(mine, c, accw[j]);
      }
    }
    __syncthreads();
    for (unsigned c = threadIdx.x; c < udim; c += RV_THREADS) {
      float s = ((lds[c] + lds[udim + c]) + lds[2 * udim + c]) + lds[3 * udim + c];
      partial[static_cast<size_t>(blockIdx.x) * udim + c] = s;
    }
  }
  if (bad) dev_raise_fault(fault, tag);
}

bool aligned16(std::initializer_list<const void*> ptrs) {
  uintptr_t bits = 0;
  for (const void* p : ptrs) bits |= reinterpret_cast<uintptr_t>(p);
  return (bits & 15u) == 0;
}

}  // namespace

bool omx_rms_vec_eligible(uint64_t dim, std::initializer_list<const void*> ptrs) {
  return dim % 4 == 0 && dim >= 256 && dim <= 2048 && aligned16(ptrs);
}

int32_t omx_rms_forward_vec(omx_ctx* ctx, const void* x, int32_t x_dtype, const void* add, int32_t add_dtype,
                            const float* w, float* sum_out, void* y, int32_t y_dtype, uint64_t rows, uint64_t dim,
                            float eps, unsigned long long tag) {
  dim3 grid(static_cast<unsigned>((rows + 3) / 4)), block(RV_THREADS);
  const int nch = static_cast<int>((dim + 255) / 256);
  typedef unsigned short h16;
  // Bytes: the row read (and the row added to it), the sum written when there is one, the normed row written.
  const auto width = [](int32_t dtype) { return dtype == OMX_BF16 ? 2.0 : 4.0; };
  OmxKernelTimer timer(ctx, OMX_K_RMS_FWD, static_cast<double>(rows) * static_cast<double>(dim) *
                                               (width(x_dtype) + (add ? width(add_dtype) + 4.0 : 0.0) + width(y_dtype)));
#define RV_FWD(TX, TA, TY, N)                                                                                      \
  omx_launch_timed(ctx, rms_fwd_vec_kernel<TX, TA, TY, N>, grid, block, 0, timer.start(), timer.stop(),            \
                   static_cast<const TX*>(x), static_cast<const TA*>(add), w, sum_out, static_cast<TY*>(y),        \
                   static_cast<size_t>(rows), static_cast<int>(dim), eps, ctx->fault, tag)
#define RV_FWD_N(TX, TA, TY)      \
  switch (nch) {                  \
    case 1: RV_FWD(TX, TA, TY, 1); break; \
    case 2: RV_FWD(TX, TA, TY, 2); break; \
    case 3: RV_FWD(TX, TA, TY, 3); break; \
    case 4: RV_FWD(TX, TA, TY, 4); break; \
    case 5: RV_FWD(TX, TA, TY, 5); break; \
    case 6: RV_FWD(TX, TA, TY, 6); break; \
    case 7: RV_FWD(TX, TA, TY, 7); break; \
    default: RV_FWD(TX, TA, TY, 8); break; \
  }
  const int key = (x_dtype == OMX_BF16 ? 4 : 0) | (add && add_dtype == OMX_BF16 ? 2 : 0) | (y_dtype == OMX_BF16 ? 1 : 0);
  switch (key) {
    case 0: RV_FWD_N(float, float, float) break;
    case 1: RV_FWD_N(float, float, h16) break;
    case 2: RV_FWD_N(float, h16, float) break;
    case 3: RV_FWD_N(float, h16, h16) break;
    case 4: RV_FWD_N(h16, float, float) break;
    case 5: RV_FWD_N(h16, float, h16) break;
    case 6: RV_FWD_N(h16, h16, float) break;
    default: RV_FWD_N(h16, h16, h16) break;
  }
#undef RV_FWD_N
#undef RV_FWD
  OMX_LAUNCH_CHECK(ctx, "rms_fwd_vec_kernel");
  return OMX_OK;
}

int32_t omx_rms_backward_vec(omx_ctx* ctx, const void* x, int32_t x_dtype, const float* w, const void* gy,
                             int32_t gy_dtype, const float* add_in, void* gx, int32_t gx_dtype, void* gx16, float* gw,
                             uint64_t rows, uint64_t dim, float eps, unsigned long long tag) {
  // The kernel's time does not depend on the rows a block takes between 2 and 16 per wave (the
  // loads of a row are all in flight at once); fewer blocks leave fewer partial rows to add.
  int rows_per_block = 8;
  while (rows_per_block < (dim > 1024 ? 16 : 32) && rows / rows_per_block > 512) rows_per_block *= 2;
  const uint64_t blocks = (rows + rows_per_block - 1) / rows_per_block;
  // A null gw: the weight is frozen, its gradient is not formed (no partial sums, no second launch).
  float *partial = nullptr, *scratch = nullptr;
  if (gw) {
    void* ws = nullptr;
    int32_t rc = omx_workspace(ctx, (blocks + OMX_COLUMN_SUM_GROUPS) * dim * sizeof(float), &ws);
    if (rc != OMX_OK) return rc;
    partial = static_cast<float*>(ws);
    scratch = partial + blocks * dim;
  }
  dim3 grid(static_cast<unsigned>(blocks)), block(RV_THREADS);
  const size_t smem = 4 * dim * sizeof(float);
  const int nch = static_cast<int>((dim + 255) / 256);
  const bool full = dim == static_cast<uint64_t>(nch) * 256;
  typedef unsigned short h16;
  // Bytes: the row and its gradient read (and the gradient added in), the input gradient written
  // (and its bf16 copy); the weight gradient's partial sums are the kernels' own traffic.
  const auto width = [](int32_t dtype) { return dtype == OMX_BF16 ? 2.0 : 4.0; };
  OmxKernelTimer timer(ctx, OMX_K_RMS_BWD,
                       static_cast<double>(rows) * static_cast<double>(dim) *
                           (width(x_dtype) + width(gy_dtype) + (add_in ? 4.0 : 0.0) + width(gx_dtype) + (gx16 ? 2.0 : 0.0)));
#define RV_BWD(TX, TG, TO, N)                                                                                        \
  do {                                                                                                               \
    if (full)                                                                                                        \
      omx_launch_timed(ctx, rms_bwd_vec_kernel<TX, TG, TO, N, (N > 4), true>, grid, block, smem, timer.start(),      \
                       gw ? nullptr : timer.stop(), static_cast<const TX*>(x), w, static_cast<const TG*>(gy), add_in,                    \
                       static_cast<TO*>(gx), static_cast<h16*>(gx16), partial, static_cast<size_t>(rows),            \
                       static_cast<int>(dim), eps, rows_per_block, ctx->fault, tag);                                 \
    else                                                                                                             \
      omx_launch_timed(ctx, rms_bwd_vec_kernel<TX, TG, TO, N, (N > 4), false>, grid, block, smem, timer.start(),     \
                       gw ? nullptr : timer.stop(), static_cast<const TX*>(x), w, static_cast<const TG*>(gy), add_in,                    \
                       static_cast<TO*>(gx), static_cast<h16*>(gx16), partial, static_cast<size_t>(rows),            \
                       static_cast<int>(dim), eps, rows_per_block, ctx->fault, tag);                                 \
  } while (0)
#define RV_BWD_N(TX, TG, TO)      \
  switch (nch) {                  \
    case 1: RV_BWD(TX, TG, TO, 1); break; \
    case 2: RV_BWD(TX, TG, TO, 2); break; \
    case 3: RV_BWD(TX, TG, TO, 3); break; \
    case 4: RV_BWD(TX, TG, TO, 4); break; \
    case 5: RV_BWD(TX, TG, TO, 5); break; \
    case 6: RV_BWD(TX, TG, TO, 6); break; \
    case 7: RV_BWD(TX, TG, TO, 7); break; \
    default: RV_BWD(TX, TG, TO, 8); break; \
  }
  const int key = (x_dtype == OMX_BF16 ? 4 : 0) | (gy_dtype == OMX_BF16 ? 2 : 0) | (gx_dtype == OMX_BF16 ? 1 : 0);
  switch (key) {
    case 0: RV_BWD_N(float, float, float) break;
    case 1: RV_BWD_N(float, float, h16) break;
    case 2: RV_BWD_N(float, h16, float) break;
    case 3: RV_BWD_N(float, h16, h16) break;
    case 4: RV_BWD_N(h16, float, float) break;
    case 5: RV_BWD_N(h16, float, h16) break;
    case 6: RV_BWD_N(h16, h16, float) break;
    default: RV_BWD_N(h16, h16, h16) break;
  }
#undef RV_BWD_N
#undef RV_BWD
  OMX_LAUNCH_CHECK(ctx, "rms_bwd_vec_kernel");
  if (!gw) return OMX_OK;
  return omx_column_sum(ctx, partial, gw, blocks, dim, tag, scratch, timer.stop());
}

extern "C" {

int32_t omx_residual_add_rms_norm_forward(omx_ctx* ctx, const void* x, int32_t x_dtype, const void* y, int32_t y_dtype,
                                          const void* w, void* sum_out, void* normed, int32_t normed_dtype,
                                          uint64_t rows, uint64_t dim, float eps) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "residual_add_rms_norm_forward";
  if (!x || !y || !w || !sum_out || !normed) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(x_dtype) || !omx_valid_float_dtype(y_dtype) || !omx_valid_float_dtype(normed_dtype))
    return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  if (rows == 0 || dim == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (!(eps == eps) || eps == INFINITY || eps == -INFINITY) return omx_fail(ctx, OMX_NON_FINITE, "%s", op);
  if (omx_rms_vec_eligible(dim, {x, y, w, sum_out, normed}))
    return omx_rms_forward_vec(ctx, x, x_dtype, y, y_dtype, static_cast<const float*>(w), static_cast<float*>(sum_out),
                               normed, normed_dtype, rows, dim, eps, omx_tag(ctx, F_RMS_FORWARD));
  int32_t rc = omx_residual_add(ctx, x, x_dtype, y, y_dtype, sum_out, OMX_F32, rows * dim);
  if (rc != OMX_OK) return rc;
  return omx_rms_norm_forward(ctx, sum_out, OMX_F32, w, normed, normed_dtype, rows, dim, eps);
}

int32_t omx_rms_norm_backward_residual(omx_ctx* ctx, const void* x, int32_t x_dtype, const void* w, const void* gy,
                                       int32_t gy_dtype, const void* residual_grad, void* gx, void* gx_bf16, void* gw,
                                       uint64_t rows, uint64_t dim, float eps) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "rms_norm_backward_residual";
  if (!x || !w || !gy || !residual_grad || !gx) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(x_dtype) || !omx_valid_float_dtype(gy_dtype))
    return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  if (rows == 0 || dim == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (!(eps == eps) || eps == INFINITY || eps == -INFINITY) return omx_fail(ctx, OMX_NON_FINITE, "%s", op);
  if (!gw && !omx_rms_vec_eligible(dim, {x, w, gy, residual_grad, gx, gx_bf16})) {
    // The separate kernels below always form the weight gradient: it goes to scratch.
    int32_t wrc = omx_workspace(ctx, dim * sizeof(float), &gw, 1);
    if (wrc != OMX_OK) return wrc;
  }
  if (omx_rms_vec_eligible(dim, {x, w, gy, residual_grad, gx, gx_bf16, gw}))
    return omx_rms_backward_vec(ctx, x, x_dtype, static_cast<const float*>(w), gy, gy_dtype,
                                static_cast<const float*>(residual_grad), gx, OMX_F32, gx_bf16,
                                static_cast<float*>(gw), rows, dim, eps, omx_tag(ctx, F_RMS_BACKWARD));
  // Other widths: the same three steps as separate kernels (gx is written, then added in place).
  int32_t rc = omx_rms_norm_backward(ctx, x, x_dtype, w, gy, gy_dtype, gx, OMX_F32, gw, rows, dim, eps);
  if (rc != OMX_OK) return rc;
  rc = omx_residual_add(ctx, residual_grad, OMX_F32, gx, OMX_F32, gx, OMX_F32, rows * dim);
  if (rc != OMX_OK) return rc;
  if (gx_bf16) return omx_to_bf16(ctx, gx, gx_bf16, rows * dim);
  return OMX_OK;
}

}  // extern "C"
