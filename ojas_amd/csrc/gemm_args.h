// Launch arguments shared by the GEMM kernels (gemm.hip, gemm_dma.hip).
#pragma once

#include "omx_common.h"

struct GemmArgs {
  const void* a;
  const void* b;
  void* c;
  long lda, ldb, ldc;
  int M, N, K;
  int c_bf16, accumulate;
  int a_vec, b_vec;  // 16-byte loads allowed (alignment of base and leading dimension)
  int c_vec;         // 4-column stores allowed (alignment of C and its row pitch)
  int tiles_m, tiles_n;
  int splits, ksteps_per_split;  // split-K: each split writes an f32 partial
  float* partial;                // [splits][M][N] when splits > 1
  int epi, epi_tanh;             // OMX_EPI_* (bf16 output, no split)
  const unsigned short* aux_in;
  unsigned short* aux_out;
  float epi_s1, epi_s2;  // OMX_EPI_AXPBY
  OmxFaultWord* fault;
  unsigned long long tag;
  // Strided batch: block (x, y) works on product y, whose operands start batch_* BYTES after
  // product y - 1's. batches == 1 for a single product.
  int batches;
  long batch_a, batch_b, batch_c;
};

// The arguments of product `product` of a strided batch.
__device__ __forceinline__ void gemm_select_batch(GemmArgs& g, int product) {
  if (g.batches > 1) {
    const long y = product;
    g.a = static_cast<const char*>(g.a) + y * g.batch_a;
    g.b = static_cast<const char*>(g.b) + y * g.batch_b;
    g.c = static_cast<char*>(g.c) + y * g.batch_c;
    // A split product of a batch keeps its partial sums behind the earlier products'.
    if (g.splits > 1) g.partial += y * g.splits * static_cast<long>(g.M) * g.N;
    // aux tensors are bf16 like the output they accompany: the same byte stride.
    if (g.aux_in) g.aux_in = reinterpret_cast<const unsigned short*>(reinterpret_cast<const char*>(g.aux_in) + y * g.batch_c);
    if (g.aux_out) g.aux_out = reinterpret_cast<unsigned short*>(reinterpret_cast<char*>(g.aux_out) + y * g.batch_c);
  }
}

// Stores four consecutive columns of one output row (row `grow`, columns
// gcol..gcol+3, clipped to N): a split-K partial, a bf16 result, or an f32
// result with optional accumulation. Returns true when a stored value is
// non-finite (partials are checked by the reduce kernel instead).
__device__ __forceinline__ bool gemm_store4(const GemmArgs& g, int split, int grow, int gcol, float x0, float x1,
                                            float x2, float x3) {
  float x[4] = {x0, x1, x2, x3};
  bool bad = false;
  if (g.splits > 1) {
    float* part = g.partial + static_cast<long>(split) * g.M * g.N + static_cast<long>(grow) * g.N + gcol;
    if ((g.N & 3) == 0 && gcol + 4 <= g.N) {
      *reinterpret_cast<float4*>(part) = make_float4(x0, x1, x2, x3);
    } else {
      for (int e = 0; e < 4 && gcol + e < g.N; ++e) part[e] = x[e];
    }
    return false;
  }
  const long off = static_cast<long>(grow) * g.ldc + gcol;
  const bool whole = g.c_vec != 0 && gcol + 4 <= g.N;
  if (g.c_bf16) {
    unsigned short* cp = static_cast<unsigned short*>(g.c) + off;
    if (whole) {
      uint2 w;
      w.x = dev_pack_bf16_pair(x0, x1);
      w.y = dev_pack_bf16_pair(x2, x3);
      *reinterpret_cast<uint2*>(cp) = w;
      bad = !(dev_finite(x0) && dev_finite(x1) && dev_finite(x2) && dev_finite(x3));
    } else {
      for (int e = 0; e < 4 && gcol + e < g.N; ++e) {
        cp[e] = dev_f32_to_bf16_bits(x[e]);
        bad |= !dev_finite(x[e]);
      }
    }
  } else {
    float* cp = static_cast<float*>(g.c) + off;
    if (whole) {
      if (g.accumulate) {
        const float4 old = *reinterpret_cast<const float4*>(cp);
        x[0] += old.x;
        x[1] += old.y;
        x[2] += old.z;
        x[3] += old.w;
      }
      *reinterpret_cast<float4*>(cp) = make_float4(x[0], x[1], x[2], x[3]);
      bad = !(dev_finite(x[0]) && dev_finite(x[1]) && dev_finite(x[2]) && dev_finite(x[3]));
    } else {
      for (int e = 0; e < 4 && gcol + e < g.N; ++e) {
        float y = g.accumulate ? x[e] + cp[e] : x[e];
        cp[e] = y;
        bad |= !dev_finite(y);
      }
    }
  }
  return bad;
}

// gemm_store4 with the optional activation of OmxGemmEpilogue applied first (bf16 outputs, no
// split). Kept apart from the plain store so the plain epilogue loops stay small enough to unroll.
// OMX_EPI_AXPBY on one element: `aux` as stored, `acc` the product's f32 accumulator.
__device__ __forceinline__ float gemm_axpby(const GemmArgs& g, float aux, float acc) {
  return dev_round_bf16(g.epi_s1 * aux) + dev_round_bf16(g.epi_s2 * dev_round_bf16(acc));
}

__device__ __forceinline__ bool gemm_store4_epi(const GemmArgs& g, int split, int grow, int gcol, float x0, float x1,
                                                float x2, float x3) {
  bool bad = false;
  const long off = static_cast<long>(grow) * g.ldc + gcol;
  const bool whole = g.c_vec != 0 && gcol + 4 <= g.N;
  {
    if (g.epi == OMX_EPI_GELU_FWD) {
      // The activation is taken of the value the pre-activation is stored as.
      const float u0 = dev_round_bf16(x0), u1 = dev_round_bf16(x1), u2 = dev_round_bf16(x2), u3 = dev_round_bf16(x3);
      const float a0 = g.epi_tanh ? dev_gelu_tanh_fast(u0) : dev_gelu_erf_fast(u0);
      const float a1 = g.epi_tanh ? dev_gelu_tanh_fast(u1) : dev_gelu_erf_fast(u1);
      const float a2 = g.epi_tanh ? dev_gelu_tanh_fast(u2) : dev_gelu_erf_fast(u2);
      const float a3 = g.epi_tanh ? dev_gelu_tanh_fast(u3) : dev_gelu_erf_fast(u3);
      unsigned short* ap = g.aux_out + off;
      if (whole) {
        uint2 w;
        w.x = dev_pack_bf16_pair(a0, a1);
        w.y = dev_pack_bf16_pair(a2, a3);
        *reinterpret_cast<uint2*>(ap) = w;
        bad = !(dev_finite(a0) && dev_finite(a1) && dev_finite(a2) && dev_finite(a3));
      } else {
        if (gcol + 0 < g.N) { ap[0] = dev_f32_to_bf16_bits(a0); bad |= !dev_finite(a0); }
        if (gcol + 1 < g.N) { ap[1] = dev_f32_to_bf16_bits(a1); bad |= !dev_finite(a1); }
        if (gcol + 2 < g.N) { ap[2] = dev_f32_to_bf16_bits(a2); bad |= !dev_finite(a2); }
        if (gcol + 3 < g.N) { ap[3] = dev_f32_to_bf16_bits(a3); bad |= !dev_finite(a3); }
      }
    } else if (g.epi == OMX_EPI_GELU_BWD || g.epi == OMX_EPI_AXPBY) {
      const unsigned short* ap = g.aux_in + off;
      float u0 = 0.0f, u1 = 0.0f, u2 = 0.0f, u3 = 0.0f;
      if (whole) {
        const uint2 w = *reinterpret_cast<const uint2*>(ap);
        u0 = __uint_as_float(w.x << 16);
        u1 = __uint_as_float(w.x & 0xffff0000u);
        u2 = __uint_as_float(w.y << 16);
        u3 = __uint_as_float(w.y & 0xffff0000u);
      } else {
        if (gcol + 0 < g.N) u0 = dev_bf16_bits_to_f32(ap[0]);
        if (gcol + 1 < g.N) u1 = dev_bf16_bits_to_f32(ap[1]);
        if (gcol + 2 < g.N) u2 = dev_bf16_bits_to_f32(ap[2]);
        if (gcol + 3 < g.N) u3 = dev_bf16_bits_to_f32(ap[3]);
      }
      if (g.epi == OMX_EPI_AXPBY) {
        x0 = gemm_axpby(g, u0, x0);
        x1 = gemm_axpby(g, u1, x1);
        x2 = gemm_axpby(g, u2, x2);
        x3 = gemm_axpby(g, u3, x3);
      } else {
        x0 = dev_round_bf16(x0) * (g.epi_tanh ? dev_gelu_tanh_grad_fast(u0) : dev_gelu_erf_grad_fast(u0));
        x1 = dev_round_bf16(x1) * (g.epi_tanh ? dev_gelu_tanh_grad_fast(u1) : dev_gelu_erf_grad_fast(u1));
        x2 = dev_round_bf16(x2) * (g.epi_tanh ? dev_gelu_tanh_grad_fast(u2) : dev_gelu_erf_grad_fast(u2));
        x3 = dev_round_bf16(x3) * (g.epi_tanh ? dev_gelu_tanh_grad_fast(u3) : dev_gelu_erf_grad_fast(u3));
      }
    }
  }
  return gemm_store4(g, split, grow, gcol, x0, x1, x2, x3) || bad;
}

// The activation epilogue for a 32-row block of a wave's tile that lies wholly inside the output
// (16-byte stores allowed): `staged` holds the block's f32 values, `pitch` floats per row,
// PPR 4-column pieces per row. One straight-line body per piece (the form of the activation is
// a template argument, the bounds are known), all of the backward's pre-activation loads issued
// ahead of the arithmetic. Returns true when a stored value is non-finite.
template <int EPI, bool TANH, int PPR>
__device__ __forceinline__ bool gemm_epilogue_block(const GemmArgs& g, const float* staged, int pitch, int grow0,
                                                    int gcol0, int lane) {
  constexpr int ITERS = 32 * PPR / 64;
  unsigned short* cbase = static_cast<unsigned short*>(g.c);
  // Non-finite values are found in the packed words that get stored: a bf16 is infinite or NaN
  // when its eight exponent bits are all set, and adding one at the exponent's lowest bit then
  // carries into the half's top bit. (GELU of a finite value is finite, so the forward tests the
  // pre-activation words only.)
  unsigned int flags = 0;
  auto note = [&](unsigned int w) { flags |= (w & 0x7F807F80u) + 0x00800080u; };
  long off[ITERS];
  uint2 aux[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int c = lane + it * 64, row = c / PPR, piece = c % PPR;
    off[it] = static_cast<long>(grow0 + row) * g.ldc + gcol0 + piece * 4;
    if constexpr (EPI != OMX_EPI_GELU_FWD) aux[it] = *reinterpret_cast<const uint2*>(g.aux_in + off[it]);
  }
  auto pack = [](float a, float b) {
    return dev_pack_bf16_pair(a, b);
  };
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int c = lane + it * 64, row = c / PPR, piece = c % PPR;
    const float4 val = *reinterpret_cast<const float4*>(staged + row * pitch + piece * 4);
    float x[4] = {val.x, val.y, val.z, val.w};
    if constexpr (EPI == OMX_EPI_GELU_FWD) {
      // The activation is taken of the value the pre-activation is stored as: one conversion per
      // pair gives both the stored word and, widened again, the activation's argument.
      const unsigned int w01 = pack(x[0], x[1]), w23 = pack(x[2], x[3]);
      const float u[4] = {__uint_as_float(w01 << 16), __uint_as_float(w01 & 0xffff0000u), __uint_as_float(w23 << 16),
                          __uint_as_float(w23 & 0xffff0000u)};
      float a[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) a[e] = TANH ? dev_gelu_tanh_fast(u[e]) : dev_gelu_erf_fast(u[e]);
      note(w01);
      note(w23);
      *reinterpret_cast<uint2*>(cbase + off[it]) = make_uint2(w01, w23);
      *reinterpret_cast<uint2*>(g.aux_out + off[it]) = make_uint2(pack(a[0], a[1]), pack(a[2], a[3]));
    } else {
      const float u[4] = {__uint_as_float(aux[it].x << 16), __uint_as_float(aux[it].x & 0xffff0000u),
                          __uint_as_float(aux[it].y << 16), __uint_as_float(aux[it].y & 0xffff0000u)};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if constexpr (EPI == OMX_EPI_AXPBY) x[e] = gemm_axpby(g, u[e], x[e]);
        else x[e] = dev_round_bf16(x[e]) * (TANH ? dev_gelu_tanh_grad_fast(u[e]) : dev_gelu_erf_grad_fast(u[e]));
      }
      const unsigned int w01 = pack(x[0], x[1]), w23 = pack(x[2], x[3]);
      note(w01);
      note(w23);
      *reinterpret_cast<uint2*>(cbase + off[it]) = make_uint2(w01, w23);
    }
  }
  return (flags & 0x80008000u) != 0;
}

// The plain store of a 32-row block that lies wholly inside the output, in the same straight-line
// form. KIND 0: f32 split-K partial; 1: bf16 result; 2: f32 result; 3: f32 result added to the
// stored one.
template <int KIND, int PPR>
__device__ __forceinline__ bool gemm_store_block(const GemmArgs& g, int split, const float* staged, int pitch,
                                                 int grow0, int gcol0, int lane) {
  constexpr int ITERS = 32 * PPR / 64;
  bool bad = false;
  const long ld = KIND == 0 ? g.N : g.ldc;
  float* fbase = KIND == 0 ? g.partial + static_cast<long>(split) * g.M * g.N : static_cast<float*>(g.c);
  unsigned short* hbase = static_cast<unsigned short*>(g.c);
  float4 old[ITERS];
  if constexpr (KIND == 3) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int c = lane + it * 64, row = c / PPR, piece = c % PPR;
      old[it] = *reinterpret_cast<const float4*>(fbase + static_cast<long>(grow0 + row) * ld + gcol0 + piece * 4);
    }
  }
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int c = lane + it * 64, row = c / PPR, piece = c % PPR;
    const long off = static_cast<long>(grow0 + row) * ld + gcol0 + piece * 4;
    float4 val = *reinterpret_cast<const float4*>(staged + row * pitch + piece * 4);
    if constexpr (KIND == 3) {
      val.x += old[it].x;
      val.y += old[it].y;
      val.z += old[it].z;
      val.w += old[it].w;
    }
    if constexpr (KIND == 1) {
      uint2 w;
      w.x = dev_pack_bf16_pair(val.x, val.y);
      w.y = dev_pack_bf16_pair(val.z, val.w);
      *reinterpret_cast<uint2*>(hbase + off) = w;
    } else {
      *reinterpret_cast<float4*>(fbase + off) = val;
    }
    // Partials are checked by the reduce kernel.
    if constexpr (KIND != 0) bad |= !(dev_finite(val.x) && dev_finite(val.y) && dev_finite(val.z) && dev_finite(val.w));
  }
  return bad;
}

// bf16 kernels with direct-to-LDS loads and a 256 x 256 (variant 9), 256 x 128 (variant 3) or
// 128 x 128 (variant 6) workgroup tile. Needs K % 64 == 0, 16-byte aligned
// operands, and row counts that are multiples of 8 for k-major operands.
bool omx_gemm_dma_eligible(const GemmArgs& g, bool a_km, bool b_km);
bool omx_gemm_w4_eligible(const GemmArgs& g, bool a_km, bool b_km, bool plain);
void omx_gemm_dma_tile(int variant, int* bm, int* bn);
int32_t omx_gemm_dma_launch(omx_ctx* ctx, const GemmArgs& g, bool a_km, bool b_km, int variant);

// bf16 kernel for outputs of at most 64 columns over at least 1024 rows of a k-contiguous A
// (K a multiple of 128, no accumulation): one pass over A, no split-K reduce.
bool omx_gemm_thin_eligible(const GemmArgs& g, bool a_km, bool b_km);
int32_t omx_gemm_thin_launch(omx_ctx* ctx, const GemmArgs& g, bool b_km);
