// MFMA GEMM for gfx950: C[M,N] (+)= A[M,K] . B[K,N], f32 accumulation.
//
// Serves BackendModule::linear_forward / linear_backward / linear_backward_input
// (ojas-core/src/backend.rs:1628-1656; CPU reference ojas-cpu/src/linalg.rs:69-210)
// and the Newton-Schulz products of muon_ns5_step (ojas-cpu/src/optim.rs:841-985).
//
// Two lanes share one kernel template:
//   bf16 storage -> v_mfma_f32_32x32x16_bf16 (8 k-values per lane per issue)
//   f32 storage  -> v_mfma_f32_32x32x2_f32   (1 k-value per lane per issue)
// Each product of two bf16 values is exact in f32, so the bf16 lane differs
// from the CPU Exact chain only in summation order (the Fast contract).
//
// Tiling: 128x128 output tile per 256-thread workgroup (4 waves, 2x2, each a
// 64x64 wave tile = 2x2 MFMA 32x32 blocks), K step of eight 16-byte chunks
// (64 bf16 / 32 f32), LDS double-buffered with the next K step prefetched into
// registers while the current one is multiplied. LDS rows are [row][k] with a
// 16-byte pad (144-byte pitch) so the 16-byte fragment reads of 32 lanes hit
// distinct banks. An operand whose K index is the slow one in memory
// ("k-major": gy and x in the weight gradient, W in the input gradient) is
// loaded with coalesced 16-byte reads along its fast index and transposed in
// registers on the way into LDS, so the fragment reads are the same for every
// operand layout.
#include <algorithm>
#include <cstdlib>

#include "gemm_args.h"
#include "omx_common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr int NT = 256;
constexpr int PITCH = 144;  // bytes per LDS row of a k-contiguous tile: 8 chunks of 16 B + pad

template <typename T>
union Chunk {
  u32x4 v;
  T e[16 / sizeof(T)];
};

// ---- operand with K contiguous: element (row, k) at p[row * ld + k]; LDS [row][k].
template <typename T, int ROWS>
__device__ __forceinline__ void load_kcontig(const T* __restrict__ p, long ld, int row0, int rows, int k0, int K,
                                             bool vec, u32x4* regs) {
  constexpr int KV = 16 / sizeof(T);
  const int tid = threadIdx.x;
#pragma unroll
  for (int i = 0; i < ROWS / 32; ++i) {
    int c = tid + NT * i;
    int row = c >> 3, kc = c & 7;
    int gr = row0 + row, gk = k0 + kc * KV;
    Chunk<T> ch;
    ch.v = u32x4{0u, 0u, 0u, 0u};
    if (gr < rows && gk < K) {
      const T* src = p + static_cast<long>(gr) * ld + gk;
      if (vec && gk + KV <= K) {
        ch.v = *reinterpret_cast<const u32x4*>(src);
      } else {
#pragma unroll
        for (int e = 0; e < KV; ++e)
          if (gk + e < K) ch.e[e] = src[e];
      }
    }
    regs[i] = ch.v;
  }
}
template <int ROWS>
__device__ __forceinline__ void store_kcontig(char* lds, const u32x4* regs) {
  const int tid = threadIdx.x;
#pragma unroll
  for (int i = 0; i < ROWS / 32; ++i) {
    int c = tid + NT * i;
    int row = c >> 3, kc = c & 7;
    *reinterpret_cast<u32x4*>(lds + row * PITCH + kc * 16) = regs[i];
  }
}

// ---- f32 operand with K as the slow index: element (row, k) at p[k * ld + row].
// 128 rows only. Each thread loads a 4 (k) x 4 (row) block with four 16-byte
// reads along the row index and stores it transposed into the [row][k] layout.
template <typename T>
__device__ __forceinline__ void load_kmajor(const T* __restrict__ p, long ld, int row0, int rows, int k0, int K,
                                            bool vec, u32x4* regs) {
  constexpr int KV = 16 / sizeof(T);
  constexpr int MPB = 128 / KV;
  const int tid = threadIdx.x;
  const int mb = tid % MPB, kb = tid / MPB;
  const int gr = row0 + mb * KV;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    int gk = k0 + kb * 4 + r;
    Chunk<T> ch;
    ch.v = u32x4{0u, 0u, 0u, 0u};
    if (gk < K && gr < rows) {
      const T* src = p + static_cast<long>(gk) * ld + gr;
      if (vec && gr + KV <= rows) {
        ch.v = *reinterpret_cast<const u32x4*>(src);
      } else {
#pragma unroll
        for (int e = 0; e < KV; ++e)
          if (gr + e < rows) ch.e[e] = src[e];
      }
    }
    regs[r] = ch.v;
  }
}
template <typename T>
__device__ __forceinline__ void store_kmajor(char* lds, const u32x4* regs) {
  constexpr int KV = 16 / sizeof(T);
  constexpr int MPB = 128 / KV;
  const int tid = threadIdx.x;
  const int mb = tid % MPB, kb = tid / MPB;
  Chunk<T> in[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) in[r].v = regs[r];
#pragma unroll
  for (int mi = 0; mi < KV; ++mi) {
    T out[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) out[r] = in[r].e[mi];
    char* dst = lds + (mb * KV + mi) * PITCH + kb * 4 * static_cast<int>(sizeof(T));
    if constexpr (sizeof(T) == 2) {
      u32x2 w;
      w.x = static_cast<unsigned int>(out[0]) | (static_cast<unsigned int>(out[1]) << 16);
      w.y = static_cast<unsigned int>(out[2]) | (static_cast<unsigned int>(out[3]) << 16);
      *reinterpret_cast<u32x2*>(dst) = w;
    } else {
      u32x4 w;
      w.x = __float_as_uint(out[0]);
      w.y = __float_as_uint(out[1]);
      w.z = __float_as_uint(out[2]);
      w.w = __float_as_uint(out[3]);
      *reinterpret_cast<u32x4*>(dst) = w;
    }
  }
}

// ---- bf16 operand with K as the slow index, kept in LDS as it lies in memory:
// [64 k][ROWS], pitch ROWS * 2 + 32 bytes (consecutive k rows shift by 8 banks,
// so the four k rows a 16-lane group touches in one transposing read fall on
// distinct banks). The copy in is plain 16-byte chunks; the MFMA fragment comes
// out of two ds_read_b64_tr_b16.
typedef short short4v __attribute__((ext_vector_type(4)));

template <int ROWS>
__device__ __forceinline__ void load_km16(const unsigned short* __restrict__ p, long ld, int row0, int rows, int k0,
                                          int K, bool vec, u32x4* regs) {
  constexpr int CPR = ROWS / 8;  // 16-byte chunks per k row
  const int tid = threadIdx.x;
#pragma unroll
  for (int i = 0; i < ROWS / 32; ++i) {
    int c = tid + NT * i;
    int kr = c / CPR, mc = c % CPR;
    int gk = k0 + kr, gr = row0 + mc * 8;
    Chunk<unsigned short> ch;
    ch.v = u32x4{0u, 0u, 0u, 0u};
    if (gk < K && gr < rows) {
      const unsigned short* src = p + static_cast<long>(gk) * ld + gr;
      if (vec && gr + 8 <= rows) {
        ch.v = *reinterpret_cast<const u32x4*>(src);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (gr + e < rows) ch.e[e] = src[e];
      }
    }
    regs[i] = ch.v;
  }
}
template <int ROWS>
__device__ __forceinline__ void store_km16(char* lds, const u32x4* regs) {
  constexpr int CPR = ROWS / 8;
  constexpr int PITCH_KM = ROWS * 2 + 32;
  const int tid = threadIdx.x;
#pragma unroll
  for (int i = 0; i < ROWS / 32; ++i) {
    int c = tid + NT * i;
    int kr = c / CPR, mc = c % CPR;
    *reinterpret_cast<u32x4*>(lds + kr * PITCH_KM + mc * 16) = regs[i];
  }
}
// Fragment of rows [row_base, row_base + 32) for k slab kk (16 k values): lane
// (i = lane%32, g = lane/32) receives k = 16kk + 8g + 0..7 of row row_base + i.
// A transposing read hands lane j of a 16-lane group element j%4 of the 8-byte
// words that lanes j/4, 4 + j/4, 8 + j/4, 12 + j/4 of the group point at; so
// lane s points at k row s/4 (+4 for the second read), row block 4(s%4).
template <int ROWS>
__device__ __forceinline__ u32x4 frag_km16(const char* tile, int row_base, int kk, int lane) {
  constexpr int PITCH_KM = ROWS * 2 + 32;
  const int s = lane & 15, half = (lane >> 4) & 1, g = lane >> 5;
  const char* p = tile + (kk * 16 + g * 8 + (s >> 2)) * PITCH_KM + (row_base + half * 16 + (s & 3) * 4) * 2;
  typedef short4v __attribute__((address_space(3))) * lds_ptr;
  short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
  short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 4 * PITCH_KM));
  u32x2 a = __builtin_bit_cast(u32x2, lo), b = __builtin_bit_cast(u32x2, hi);
  return u32x4{a.x, a.y, b.x, b.y};
}

template <typename T>
__device__ __forceinline__ void mma_step(const u32x4& af, const u32x4& bf, floatx16& acc) {
  if constexpr (sizeof(T) == 2) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, af), __builtin_bit_cast(bf16x8, bf),
                                                  acc, 0, 0, 0);
  } else {
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(af.x), __uint_as_float(bf.x), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(af.y), __uint_as_float(bf.y), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(af.z), __uint_as_float(bf.z), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(af.w), __uint_as_float(bf.w), acc, 0, 0, 0);
  }
}

template <typename T, bool KM, int ROWS>
constexpr int tile_bytes() {
  return (KM && sizeof(T) == 2) ? 64 * (ROWS * 2 + 32) : ROWS * PITCH;
}

// TM x TN MFMA 32x32 blocks per wave; the 4 waves sit 2 x 2, so the workgroup
// tile is (64 TM) x (64 TN).
template <typename T, bool A_KM, bool B_KM, int TM, int TN>
__global__ __launch_bounds__(NT) void gemm_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int KV = 16 / sizeof(T);
  constexpr int BK = 8 * KV;
  constexpr int BM = 64 * TM, BN = 64 * TN;
  constexpr bool A_TR = A_KM && sizeof(T) == 2, B_TR = B_KM && sizeof(T) == 2;
  constexpr int A_BYTES = tile_bytes<T, A_KM, BM>(), B_BYTES = tile_bytes<T, B_KM, BN>();
  constexpr int STAGE = A_BYTES + B_BYTES;
  static_assert(sizeof(T) == 2 || (TM == 2 && TN == 2), "the f32 lane uses 128x128 tiles");
  gemm_select_batch(g, blockIdx.y);
  const T* __restrict__ A = static_cast<const T*>(g.a);
  const T* __restrict__ B = static_cast<const T*>(g.b);

  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD one
  // contiguous run of tiles so neighbours share operand rows in its L2.
  const int total = g.tiles_m * g.tiles_n;
  const int split = blockIdx.x / total;
  int id = blockIdx.x - split * total;
  if (total % 8 == 0) id = (id & 7) * (total >> 3) + (id >> 3);
  // Within the run: walk M fastest inside bands of 8 tile rows.
  const int band = 8;
  int tiles_per_band = band * g.tiles_n;
  int band_id = id / tiles_per_band;
  int first_m = band_id * band;
  int band_rows = min(band, g.tiles_m - first_m);
  int in_band = id - band_id * tiles_per_band;
  const int tile_m = first_m + in_band % band_rows;
  const int tile_n = in_band / band_rows;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, lg = lane >> 5;

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  u32x4 ra[BM / 32], rb[BN / 32];
  const int ksteps_all = (g.K + BK - 1) / BK;
  const int ks_begin = split * g.ksteps_per_split;
  const int ks_end = min(ksteps_all, ks_begin + g.ksteps_per_split);
  auto load_tiles = [&](int ks) {
    int k0 = ks * BK;
    if constexpr (A_TR) load_km16<BM>(reinterpret_cast<const unsigned short*>(A), g.lda, m0, g.M, k0, g.K, g.a_vec, ra);
    else if constexpr (A_KM) load_kmajor<T>(A, g.lda, m0, g.M, k0, g.K, g.a_vec, ra);
    else load_kcontig<T, BM>(A, g.lda, m0, g.M, k0, g.K, g.a_vec, ra);
    if constexpr (B_TR) load_km16<BN>(reinterpret_cast<const unsigned short*>(B), g.ldb, n0, g.N, k0, g.K, g.b_vec, rb);
    else if constexpr (B_KM) load_kmajor<T>(B, g.ldb, n0, g.N, k0, g.K, g.b_vec, rb);
    else load_kcontig<T, BN>(B, g.ldb, n0, g.N, k0, g.K, g.b_vec, rb);
  };
  auto store_tiles = [&](int buf) {
    char* la = smem + buf * STAGE;
    char* lb = la + A_BYTES;
    if constexpr (A_TR) store_km16<BM>(la, ra);
    else if constexpr (A_KM) store_kmajor<T>(la, ra);
    else store_kcontig<BM>(la, ra);
    if constexpr (B_TR) store_km16<BN>(lb, rb);
    else if constexpr (B_KM) store_kmajor<T>(lb, rb);
    else store_kcontig<BN>(lb, rb);
  };

  load_tiles(ks_begin);
  store_tiles(0);
  __syncthreads();
  for (int ks = ks_begin; ks < ks_end; ++ks) {
    const int buf = (ks - ks_begin) & 1;
    if (ks + 1 < ks_end) load_tiles(ks + 1);
    const char* ta = smem + buf * STAGE;
    const char* tb = ta + A_BYTES;
    const char* la = ta + (wm * 32 * TM + l32) * PITCH + lg * 16;
    const char* lb = tb + (wn * 32 * TN + l32) * PITCH + lg * 16;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      u32x4 af[TM], bf[TN];
#pragma unroll
      for (int t = 0; t < TM; ++t) {
        if constexpr (A_TR) af[t] = frag_km16<BM>(ta, wm * 32 * TM + t * 32, kk, lane);
        else af[t] = *reinterpret_cast<const u32x4*>(la + t * 32 * PITCH + kk * 32);
      }
#pragma unroll
      for (int t = 0; t < TN; ++t) {
        if constexpr (B_TR) bf[t] = frag_km16<BN>(tb, wn * 32 * TN + t * 32, kk, lane);
        else bf[t] = *reinterpret_cast<const u32x4*>(lb + t * 32 * PITCH + kk * 32);
      }
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) mma_step<T>(af[tm], bf[tn], acc[tm][tn]);
    }
    if (ks + 1 < ks_end) store_tiles(buf ^ 1);
    __syncthreads();
  }

  // Accumulator register v of a 32x32 block holds row 8*(v/4) + 4*(lane/32) + v%4, column lane%32.
  // The tile is staged through LDS (free after the loop's last barrier) so that
  // global stores are whole 16-byte (f32) / 8-byte (bf16) pieces of a row.
  constexpr int CP = BN + 4;  // floats per staged row; the pad keeps 16-byte alignment
  static_assert(BM * CP * 4 <= 2 * STAGE, "the staged output tile must fit in the operand buffers");
  float* cs = reinterpret_cast<float*>(smem);
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const int col = (wn * TN + tn) * 32 + l32;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = (wm * TM + tm) * 32 + 8 * (v >> 2) + 4 * lg + (v & 3);
        cs[row * CP + col] = acc[tm][tn][v];
      }
    }
  __syncthreads();
  constexpr int CPR = BN / 4;  // 4-column pieces per row
  bool bad = false;
  for (int c = threadIdx.x; c < BM * CPR; c += NT) {
    const int row = c / CPR, cc = (c % CPR) * 4;
    const int grow = m0 + row, gcol = n0 + cc;
    if (grow >= g.M || gcol >= g.N) continue;
    const float4 val = *reinterpret_cast<const float4*>(cs + row * CP + cc);
    bad |= g.epi == OMX_EPI_NONE ? gemm_store4(g, split, grow, gcol, val.x, val.y, val.z, val.w)
                                 : gemm_store4_epi(g, split, grow, gcol, val.x, val.y, val.z, val.w);
  }
  if (bad) dev_raise_fault(g.fault, g.tag);
}

__global__ void splitk_reduce_kernel(GemmArgs g) {
  gemm_select_batch(g, blockIdx.y);
  const long total = static_cast<long>(g.M) * g.N;
  bool bad = false;
  for (long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
       i += static_cast<long>(gridDim.x) * blockDim.x) {
    const long row = i / g.N, col = i - row * g.N;
    const long off = row * g.ldc + col;
    float acc = g.accumulate ? static_cast<float*>(g.c)[off] : 0.0f;
    for (int s = 0; s < g.splits; ++s) acc += g.partial[static_cast<long>(s) * total + i];
    if (g.c_bf16) static_cast<unsigned short*>(g.c)[off] = dev_f32_to_bf16_bits(acc);
    else static_cast<float*>(g.c)[off] = acc;
    bad |= !dev_finite(acc);
  }
  if (bad) dev_raise_fault(g.fault, g.tag);
}

template <typename T, bool A_KM, bool B_KM, int TM, int TN>
int32_t launch_one(omx_ctx* ctx, const GemmArgs& g) {
  constexpr int BM = 64 * TM, BN = 64 * TN;
  constexpr int smem = 2 * (tile_bytes<T, A_KM, BM>() + tile_bytes<T, B_KM, BN>());
  auto kernel = &gemm_kernel<T, A_KM, B_KM, TM, TN>;
  // More than 64 KiB of dynamic LDS has to be granted per kernel (and per device: asked every time).
  OMX_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   smem));
  const int total = g.tiles_m * g.tiles_n * g.splits;
  omx_launch_timed(ctx, kernel, dim3(total, g.batches), dim3(NT), smem, ctx->timing_start,
                   g.splits > 1 ? nullptr : ctx->timing_stop, g);
  OMX_LAUNCH_CHECK(ctx, "gemm_kernel");
  return OMX_OK;
}

template <typename T, int TM, int TN>
int32_t launch(omx_ctx* ctx, const GemmArgs& g, bool a_km, bool b_km) {
  int32_t rc;
  if (!a_km && !b_km) rc = launch_one<T, false, false, TM, TN>(ctx, g);
  else if (!a_km && b_km) rc = launch_one<T, false, true, TM, TN>(ctx, g);
  else if (a_km && !b_km) rc = launch_one<T, true, false, TM, TN>(ctx, g);
  else rc = launch_one<T, true, true, TM, TN>(ctx, g);
  if (rc != OMX_OK) return rc;
  if (g.splits > 1) {
    long elems = static_cast<long>(g.M) * g.N;
    unsigned blocks = static_cast<unsigned>(std::min<long>((elems + 255) / 256, 4096));
    omx_launch_timed(ctx, splitk_reduce_kernel, dim3(blocks, g.batches), dim3(256), 0, nullptr, ctx->timing_stop, g);
    OMX_LAUNCH_CHECK(ctx, "splitk_reduce_kernel");
  }
  return OMX_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

// Internal entry shared by the linear ops, the fused loss and Muon.
int32_t omx_gemm_impl(omx_ctx* ctx, uint32_t fault_op, const void* a, uint64_t a_rs, uint64_t a_cs, const void* b,
                      uint64_t b_rs, uint64_t b_cs, int32_t operand_dtype, void* c, int32_t c_dtype, uint64_t ldc,
                      uint64_t m, uint64_t k, uint64_t n, int32_t accumulate, const OmxGemmEpilogue* epi,
                      const OmxGemmBatch* batch) {
  const char* op = omx_fault_name(fault_op);
  const uint64_t batches = batch ? batch->count : 1;
  if (batches == 0 || batches > 65535) return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: 1..65535 products per launch", op);
  if (epi && epi->mode != OMX_EPI_NONE && c_dtype != OMX_BF16)
    return omx_fail(ctx, OMX_DTYPE, "%s: a fused activation needs a bf16 output", op);
  if (!a || !b || !c) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(operand_dtype) || !omx_valid_float_dtype(c_dtype))
    return omx_fail(ctx, OMX_DTYPE, "%s: operands must be f32 or bf16", op);
  if (m == 0 || n == 0 || k == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (m > 0x7fffffffull || n > 0x7fffffffull || k > 0x7fffffffull)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: axis does not fit in i32", op);
  if (accumulate && c_dtype != OMX_F32) return omx_fail(ctx, OMX_DTYPE, "%s: accumulation needs an f32 output", op);
  bool a_km, b_km;
  long lda, ldb;
  if (a_cs == 1) {
    a_km = false;
    lda = static_cast<long>(a_rs);
  } else if (a_rs == 1) {
    a_km = true;
    lda = static_cast<long>(a_cs);
  } else {
    return omx_fail(ctx, OMX_SHAPE, "%s: operand A has no unit stride", op);
  }
  if (b_rs == 1) {
    b_km = false;
    ldb = static_cast<long>(b_cs);
  } else if (b_cs == 1) {
    b_km = true;
    ldb = static_cast<long>(b_rs);
  } else {
    return omx_fail(ctx, OMX_SHAPE, "%s: operand B has no unit stride", op);
  }
  const long kv = operand_dtype == OMX_BF16 ? 8 : 4;
  GemmArgs g;
  g.a = a;
  g.b = b;
  g.c = c;
  g.lda = lda;
  g.ldb = ldb;
  g.ldc = static_cast<long>(ldc);
  g.M = static_cast<int>(m);
  g.N = static_cast<int>(n);
  g.K = static_cast<int>(k);
  g.c_bf16 = c_dtype == OMX_BF16;
  g.accumulate = accumulate;
  g.a_vec = aligned16(a) && (lda % kv == 0);
  g.b_vec = aligned16(b) && (ldb % kv == 0);
  g.c_vec = aligned16(c) && (ldc % 4 == 0);
  g.batches = static_cast<int>(batches);
  g.batch_a = g.batch_b = g.batch_c = 0;
  if (batches > 1) {
    const uint64_t esz = operand_dtype == OMX_BF16 ? 2 : 4, csz = c_dtype == OMX_BF16 ? 2 : 4;
    g.batch_a = static_cast<long>(batch->stride_a * esz);
    g.batch_b = static_cast<long>(batch->stride_b * esz);
    g.batch_c = static_cast<long>(batch->stride_c * csz);
    if ((g.batch_a | g.batch_b | g.batch_c) & 15)
      return omx_fail(ctx, OMX_SHAPE, "%s: batch strides must be multiples of 16 bytes", op);
  }
  // Kernel choice. bf16 shapes whose output fills the chip with 256 x 256 (or
  // 256 x 128) tiles take the direct-to-LDS kernel; everything else (f32, odd
  // shapes, small outputs that need split-K) takes the 128 x 128 kernel.
  // A thin output over many rows (an adapter's rank, a gate's heads) is bound by reading A once: its
  // own kernel, which neither tiles the output nor splits K across launches.
  const bool thin = operand_dtype == OMX_BF16 && ctx->gemm_thin && !(epi && epi->mode != OMX_EPI_NONE) &&
                    omx_gemm_thin_eligible(g, a_km, b_km);
  int dma_variant = -1;
  if (!thin && operand_dtype == OMX_BF16 && omx_gemm_dma_eligible(g, a_km, b_km)) {
    const int mode = ctx->gemm_dma_mode;
    if (mode == 1 && ctx->gemm_forced_tiling >= 0) {
      dma_variant = ctx->gemm_forced_tiling;
    } else if (mode == 1) {
      // Three tilings, chosen by how many tiles the output makes per compute unit and how many K
      // steps a tile runs, not by a model's dimensions (measured over GPT-124M's shapes and over
      // d = 1024 / 2048 / 4096 with 8192 tokens; tests/test_gpu_gemm_kernels.py holds the choice
      // to within 10 % of the best forced tiling):
      //   3  256 x 128, 32-column steps, two workgroups per compute unit: one's first loads and
      //      store pass run under the other's products, so it is the form for short reductions
      //      and for outputs of a round or two of tiles. The default.
      //   6  128 x 128, four waves, three workgroups per compute unit: weight gradients (both
      //      operands k-major, K = tokens) whose output is under one tile per compute unit, with
      //      the reduction split (3 to 20 % ahead of 256 x 128 there), and input gradients whose
      //      256 x 128 tiles would leave compute units empty, over at least 32 steps (8192 x 768
      //      over K = 3072: 52 against 66 us).
      //   9  256 x 256, one wave per SIMD, one workgroup per compute unit: nothing hides its first
      //      loads and its store pass, so it takes long reductions whose tiles fill the chip
      //      (K = 8192, 8192 x 2048 outputs: 203 against 276 us for 256 x 128; the weight-gradient
      //      batches) and outputs of four rounds of tiles or more (the head's forward product). On
      //      K = 768 with a round or three of tiles it is ahead when timed alone and behind inside
      //      the training step (forward o 36.8 against 30.9 us).
      const bool unbatched = g.batches == 1;
      const bool plain = !(epi && epi->mode != OMX_EPI_NONE);
      const long outputs = static_cast<long>(g.M) * g.N;
      const long cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
      const long tiles256 = static_cast<long>((g.M + 255) / 256) * ((g.N + 255) / 256);
      const long tiles128 = static_cast<long>((g.M + 127) / 128) * ((g.N + 127) / 128);
      const long ksteps64 = g.K / 64;
      // How full the last round of 256 x 256 tiles is, one workgroup per compute unit.
      const long all256 = tiles256 * g.batches;
      const long rounds256 = (all256 + cus - 1) / cus;
      if (a_km && b_km && unbatched && ksteps64 >= 64 && tiles128 < cus) {
        dma_variant = 6;
      } else if (outputs * g.batches <= (1l << 20)) {
        dma_variant = -1;  // a handful of tiles: the register-staged kernel, which splits K freely
      } else if (a_km && b_km) {
        // Weight gradients (K = tokens). An unbatched product with a poor last round is cut by rows below.
        if (plain && ksteps64 >= 64 && all256 >= cus && (unbatched || all256 * 5 >= rounds256 * cus * 4)) dma_variant = 9;
        else if (plain && ksteps64 >= 128 && all256 * 8 >= cus) dma_variant = 9;  // with K split
        else dma_variant = 3;
        // 256 x 192 tiles where their rounds cost less: rounds of tiles x (4 or 3 units per K step + 18 per
        // tile), over the split counts the 256 x 256 tiling may take (a split pays 1000 / K of the product
        // for its partial sums). 12 products of 2304 x 768 are 324 tiles of 256 x 256 (two splits: three
        // rounds of half the length and a reduce pass) or 432 of 256 x 192 (two rounds, unsplit).
        if (dma_variant == 9 && !unbatched && g.N % 192 == 0) {
          const long all192 = static_cast<long>((g.M + 255) / 256) * (g.N / 192) * g.batches;
          double cost256 = 1e30;
          for (int s2 = 1; s2 <= 4 && ksteps64 / s2 >= 32; s2 *= 2) {
            const double c = static_cast<double>((all256 * s2 + cus - 1) / cus) * (4.0 * ksteps64 / s2 + 18.0) *
                             (s2 > 1 ? 1.0 + 1000.0 * s2 / static_cast<double>(g.K) : 1.0);
            if (c < cost256) cost256 = c;
          }
          const double cost192 = static_cast<double>((all192 + cus - 1) / cus) * (3.0 * ksteps64 + 18.0);
          if (cost192 < cost256) dma_variant = 10;
        }
      } else if (!a_km) {
        const long tiles256x128 = static_cast<long>((g.M + 255) / 256) * ((g.N + 127) / 128);
        if (unbatched && plain && tiles256 * 4 >= cus * 3) {
          // 256 x 256 or 256 x 192 tiles, by rounds of tiles x what a tile costs: 4 or 3 units per K step
          // and 18 outside the steps (first loads, store pass: about four and a half steps' worth).
          // 768 output columns are 3 x 256 or 4 x 192: 16384 rows make 192 tiles (a round three
          // quarters full) or 256 (a full one of tiles a quarter shorter).
          dma_variant = 9;
          if (g.N % 192 == 0) {
            const long tiles192 = static_cast<long>((g.M + 255) / 256) * (g.N / 192);
            const long cost256 = (tiles256 + cus - 1) / cus * (4 * ksteps64 + 18);
            const long cost192 = (tiles192 + cus - 1) / cus * (3 * ksteps64 + 18);
            if (cost192 < cost256) dma_variant = 10;
          }
        }
        else if (unbatched && plain && b_km && tiles256x128 < cus && ksteps64 >= 32) dma_variant = 6;
        else dma_variant = 3;
      } else {
        dma_variant = 3;
      }
    }
    else if (mode == 3) dma_variant = 3;
    else if (mode == 4) dma_variant = 6;
    else if (mode == 9) dma_variant = 9;
    else if (mode == 10) dma_variant = 10;
    if (dma_variant >= 9 && !omx_gemm_w4_eligible(g, a_km, b_km, !(epi && epi->mode != OMX_EPI_NONE))) dma_variant = 3;
  }
  // One 256 x 256 workgroup per compute unit: when the last round of tiles fills under 2/5 of the
  // chip (the head's weight gradient: 591 tiles on 256 units), the rows of the whole rounds go to
  // this tiling and the rest to a launch of their own, which picks a smaller tile (1181 -> 1034 us).
  if (dma_variant == 9 && ctx->gemm_dma_mode == 1 && ctx->gemm_row_split &&
      !ctx->gemm_in_row_split && batches == 1 && !(epi && epi->mode != OMX_EPI_NONE)) {
    const long cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
    const long tm = (g.M + 255) / 256, tn = (g.N + 255) / 256;
    const long rounds = tm * tn / cus, rest = tm * tn % cus;
    const long head_tm = rounds * cus / tn;
    if (rounds >= 1 && rounds <= 6 && rest > 0 && rest * 5 < cus * 2 && head_tm >= 1 && head_tm < tm) {
      const uint64_t m0 = static_cast<uint64_t>(head_tm) * 256;
      const uint64_t esz = 2, csz = c_dtype == OMX_BF16 ? 2 : 4;
      ctx->gemm_in_row_split = true;
      ctx->gemm_forced_tiling = dma_variant;
      int32_t rc = omx_gemm_impl(ctx, fault_op, a, a_rs, a_cs, b, b_rs, b_cs, operand_dtype, c, c_dtype, ldc, m0, k, n,
                                 accumulate, epi, nullptr);
      ctx->gemm_forced_tiling = -1;
      if (rc == OMX_OK)
        rc = omx_gemm_impl(ctx, fault_op, static_cast<const char*>(a) + m0 * a_rs * esz, a_rs, a_cs, b, b_rs, b_cs,
                           operand_dtype, static_cast<char*>(c) + m0 * ldc * csz, c_dtype, ldc, m - m0, k, n,
                           accumulate, epi, nullptr);
      ctx->gemm_in_row_split = false;
      return rc;
    }
  }
  int BM = 128, BN = 128;
  if (dma_variant >= 0) omx_gemm_dma_tile(dma_variant, &BM, &BN);
  g.tiles_m = (g.M + BM - 1) / BM;
  g.tiles_n = (g.N + BN - 1) / BN;
  if (static_cast<long>(g.tiles_m) * g.tiles_n > 0x7fffffffl)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: too many output tiles", op);
  // Few output tiles and a long reduction (the weight gradients: K = tokens):
  // split K so the grid fills the chip.
  {
    const int bk = operand_dtype == OMX_BF16 ? 64 : 32;
    const int ksteps = (g.K + bk - 1) / bk;
    const long tiles = static_cast<long>(g.tiles_m) * g.tiles_n;
    int splits = 1;
    // An f32 step is 64 MFMAs per wave (1.7 us): two of them already pay for a split.
    const int min_steps = operand_dtype == OMX_BF16 ? 8 : 2;
    // A strided batch splits on the register-staged kernel (thin outputs over a long reduction: 16
    // products of 16 tiles each leave three quarters of the chip's wave slots empty) and on the
    // 256 x 256 kernel when that fills its last round of tiles better (12 products of 768 x 768 are
    // 108 tiles: two splits; of 2304 x 768, 324 tiles: two splits make three rounds of half the length).
    const long all_tiles = tiles * g.batches;
    const bool may_split =
        !thin && (g.batches == 1 ? tiles < 256 : ((dma_variant < 0 && all_tiles < 512) || dma_variant >= 9));
    if (may_split && ksteps >= 4 * min_steps && !(epi && epi->mode != OMX_EPI_NONE)) {
      splits = static_cast<int>(((g.batches == 1 ? 512 : 1024) + all_tiles - 1) / all_tiles);
      if (splits > ksteps / min_steps) splits = ksteps / min_steps;
      if (splits < 1) splits = 1;
      if (dma_variant >= 0) {  // a power of two, so that a split stays on one XCD (see gemm_dma_kernel)
        int p2 = 1;
        while (p2 * 2 <= splits + splits / 4) p2 *= 2;  // 7..9 -> 8, 10..12 -> 8, 13..16 -> 16
        splits = p2;
        if (dma_variant >= 9) {
          // One workgroup per compute unit: what counts is how full the last round of workgroups is
          // (192 tiles split in two are 384 workgroups on 256 units, a round and a half; split in
          // four they are three full rounds of half the length). A split's partial sums cost 8 bytes
          // of traffic per output element against 2 K operations: at 4 TB/s and 1 PFLOP/s that is
          // 1000 / K of the product's time per split, which the fuller chip has to pay back.
          const long units = ctx->cu_count > 0 ? ctx->cu_count : 256;
          int best = 1;
          double best_fill = 0.0;
          for (int s2 = 1; s2 <= 4 && ksteps / s2 >= 4 * min_steps; s2 *= 2) {
            const long groups = all_tiles * s2;
            const double fill = static_cast<double>(groups) / static_cast<double>((groups + units - 1) / units * units);
            if (fill > best_fill * (1.0 + 1000.0 * s2 / static_cast<double>(g.K)) + 0.05) {
              best = s2;
              best_fill = fill;
            }
          }
          splits = best;
        }
      }
    }
    g.ksteps_per_split = (ksteps + splits - 1) / splits;
    if (dma_variant >= 9) g.ksteps_per_split += g.ksteps_per_split & 1;  // its K loop takes steps in pairs
    g.splits = (ksteps + g.ksteps_per_split - 1) / g.ksteps_per_split;
    g.partial = nullptr;
    if (g.splits > 1) {
      void* ws = nullptr;
      int32_t wrc = omx_workspace(ctx, static_cast<uint64_t>(g.splits) * batches * m * n * sizeof(float), &ws, 1);
      if (wrc != OMX_OK) return wrc;
      g.partial = static_cast<float*>(ws);
    }
  }
  g.epi = epi ? epi->mode : OMX_EPI_NONE;
  g.epi_tanh = epi ? epi->tanh_form : 0;
  g.aux_in = epi ? static_cast<const unsigned short*>(epi->aux_in) : nullptr;
  g.aux_out = epi ? static_cast<unsigned short*>(epi->aux_out) : nullptr;
  g.epi_s1 = epi ? epi->s1 : 0.0f;
  g.epi_s2 = epi ? epi->s2 : 0.0f;
  // The activation's side tensor is accessed with the output's vector width.
  if (epi && !((!epi->aux_in || aligned16(epi->aux_in)) && (!epi->aux_out || aligned16(epi->aux_out)))) g.c_vec = 0;
  g.fault = ctx->fault;
  g.tag = omx_tag(ctx, fault_op);
  omx_ctx::TimedLaunch timed{};
  if (ctx->profile_gemm) {
    auto take = [&](hipEvent_t* e) -> hipError_t {
      if (!ctx->event_pool.empty()) {
        *e = ctx->event_pool.back();
        ctx->event_pool.pop_back();
        return hipSuccess;
      }
      return hipEventCreate(e);
    };
    OMX_HIP(ctx, take(&timed.start));
    OMX_HIP(ctx, take(&timed.stop));
    timed.flops = 2.0 * static_cast<double>(m) * static_cast<double>(n) * static_cast<double>(k) * static_cast<double>(batches);
    // The kernels' own dispatch timestamps: an event recorded on the stream would be one more
    // packet before and after every product (1 ms per step over 150 products).
    ctx->timing_start = timed.start;
    ctx->timing_stop = timed.stop;
  }
  int32_t rc;
  if (thin) {
    rc = omx_gemm_thin_launch(ctx, g, b_km);
  } else if (dma_variant >= 0) {
    rc = omx_gemm_dma_launch(ctx, g, a_km, b_km, dma_variant);
    if (rc == OMX_OK && g.splits > 1) {
      long elems = static_cast<long>(g.M) * g.N;
      unsigned blocks = static_cast<unsigned>(std::min<long>((elems + 255) / 256, 4096));
      omx_launch_timed(ctx, splitk_reduce_kernel, dim3(blocks, g.batches), dim3(256), 0, nullptr, ctx->timing_stop, g);
      OMX_LAUNCH_CHECK(ctx, "splitk_reduce_kernel");
    }
  } else if (operand_dtype != OMX_BF16) {
    rc = launch<float, 2, 2>(ctx, g, a_km, b_km);
  } else {
    rc = launch<unsigned short, 2, 2>(ctx, g, a_km, b_km);
  }
  if (ctx->profile_gemm) {
    ctx->timing_start = ctx->timing_stop = nullptr;
    if (rc == OMX_OK) ctx->timed.push_back(timed);
  }
  return rc;
}

int32_t omx_timing_begin(omx_ctx* ctx, double flops, omx_ctx::TimedLaunch* timed) {
  *timed = omx_ctx::TimedLaunch{};
  if (!ctx->profile_gemm) return OMX_OK;
  auto take = [&](hipEvent_t* e) -> hipError_t {
    if (!ctx->event_pool.empty()) {
      *e = ctx->event_pool.back();
      ctx->event_pool.pop_back();
      return hipSuccess;
    }
    return hipEventCreate(e);
  };
  OMX_HIP(ctx, take(&timed->start));
  OMX_HIP(ctx, take(&timed->stop));
  timed->flops = flops;
  ctx->timing_start = timed->start;
  ctx->timing_stop = timed->stop;
  return OMX_OK;
}

void omx_timing_end(omx_ctx* ctx, bool launched, const omx_ctx::TimedLaunch& timed) {
  if (!ctx->profile_gemm) return;
  ctx->timing_start = ctx->timing_stop = nullptr;
  if (launched) ctx->timed.push_back(timed);
}

OmxKernelTimer::OmxKernelTimer(omx_ctx* c, int cls, double work) : ctx(c) {
  if (!(ctx->profile_classes >> cls & 1u)) return;
  hipEvent_t* both[2] = {&t.start, &t.stop};
  for (hipEvent_t* e : both) {
    if (!ctx->event_pool.empty()) {
      *e = ctx->event_pool.back();
      ctx->event_pool.pop_back();
    } else if (hipEventCreate(e) != hipSuccess) {
      (void)hipGetLastError();
      if (e == &t.stop) ctx->event_pool.push_back(t.start);
      return;  // this launch goes untimed
    }
  }
  t.flops = work;
  t.cls = cls;
  on = true;
}

OmxKernelTimer::~OmxKernelTimer() {
  if (on) ctx->timed.push_back(t);
}

extern "C" {

int32_t omx_set_option(omx_ctx* ctx, const char* name, int64_t value) {
  OMX_REQUIRE_CTX(ctx);
  if (name && strcmp(name, "gemm_thin") == 0) {
    ctx->gemm_thin = value != 0;
    return OMX_OK;
  }
  if (name && strcmp(name, "gemm_dma") == 0) {
    if (value != 0 && value != 1 && value != 3 && value != 4 && value != 9 && value != 10)
      return omx_fail(ctx, OMX_OUT_OF_RANGE, "set_option: gemm_dma takes 0, 1, 3, 4, 9 or 10");
    ctx->gemm_dma_mode = static_cast<int>(value);
    return OMX_OK;
  }
  if (name && strcmp(name, "gemm_row_split") == 0) {
    ctx->gemm_row_split = value != 0;
    return OMX_OK;
  }
  if (name && strcmp(name, "flash_schedule") == 0) {
    if (value < 0 || value > 2) return omx_fail(ctx, OMX_OUT_OF_RANGE, "set_option: flash_schedule takes 0..2");
    ctx->flash_schedule = static_cast<int>(value);
    return OMX_OK;
  }
  if (name && strcmp(name, "ce_fused") == 0) {
    if (value < 0 || value > 1) return omx_fail(ctx, OMX_OUT_OF_RANGE, "set_option: ce_fused takes 0..1");
    ctx->ce_fused = static_cast<int>(value);
    return OMX_OK;
  }
  if (name && strcmp(name, "sdpa_tiled") == 0) {
    if (value < 0 || value > 1) return omx_fail(ctx, OMX_OUT_OF_RANGE, "set_option: sdpa_tiled takes 0..1");
    ctx->sdpa_tiled = static_cast<int>(value);
    return OMX_OK;
  }
  if (name && strcmp(name, "muon_fused_sums") == 0) {
    if (value < 0 || value > 1) return omx_fail(ctx, OMX_OUT_OF_RANGE, "set_option: muon_fused_sums takes 0..1");
    ctx->muon_fused_sums = static_cast<int>(value);
    return OMX_OK;
  }
  if (name && strcmp(name, "adamw_trust") == 0) {
    if (value < 0 || value > 1) return omx_fail(ctx, OMX_OUT_OF_RANGE, "set_option: adamw_trust takes 0..1");
    ctx->adamw_trust = static_cast<int>(value);
    return OMX_OK;
  }
  if (name && strcmp(name, "kv_attention") == 0) {
    if (value < 0 || value > 1) return omx_fail(ctx, OMX_OUT_OF_RANGE, "set_option: kv_attention takes 0..1");
    ctx->kv_attention_mode = static_cast<int>(value);
    return OMX_OK;
  }
  return omx_fail(ctx, OMX_UNSUPPORTED, "set_option: unknown option %s", name ? name : "(null)");
}

int32_t omx_profile_gemm(omx_ctx* ctx, int32_t enable) {
  OMX_REQUIRE_CTX(ctx);
  ctx->profile_gemm = enable != 0;
  return OMX_OK;
}

int32_t omx_profile_kernels(omx_ctx* ctx, uint32_t class_mask) {
  OMX_REQUIRE_CTX(ctx);
  if (class_mask >> OMX_K_CLASSES) return omx_fail(ctx, OMX_OUT_OF_RANGE, "profile_kernels: classes 0..%d", OMX_K_CLASSES - 1);
  ctx->profile_gemm = (class_mask & 1u) != 0;
  ctx->profile_classes = class_mask & ~1u;
  return OMX_OK;
}

int32_t omx_profile_kernels_report(omx_ctx* ctx, int32_t cls, uint64_t* launches, double* total_ms, double* total_work) {
  OMX_REQUIRE_CTX(ctx);
  if (cls < 0 || cls >= OMX_K_CLASSES) return omx_fail(ctx, OMX_OUT_OF_RANGE, "profile_kernels_report: class %d", cls);
  OMX_HIP(ctx, hipStreamSynchronize(ctx->stream));
  double ms = 0.0, work = 0.0;
  uint64_t count = 0;
  std::vector<omx_ctx::TimedLaunch> rest;
  for (auto& t : ctx->timed) {
    if (t.cls != cls) {
      rest.push_back(t);
      continue;
    }
    float one = 0.0f;
    OMX_HIP(ctx, hipEventElapsedTime(&one, t.start, t.stop));
    ms += one;
    work += t.flops;
    ++count;
    ctx->event_pool.push_back(t.start);
    ctx->event_pool.push_back(t.stop);
  }
  ctx->timed.swap(rest);
  if (launches) *launches = count;
  if (total_ms) *total_ms = ms;
  if (total_work) *total_work = work;
  return OMX_OK;
}

int32_t omx_profile_gemm_report(omx_ctx* ctx, uint64_t* launches, double* total_ms, double* total_flops) {
  return omx_profile_kernels_report(ctx, OMX_K_GEMM, launches, total_ms, total_flops);
}

int32_t omx_gemm(omx_ctx* ctx, const void* a, uint64_t a_rs, uint64_t a_cs, const void* b, uint64_t b_rs,
                 uint64_t b_cs, int32_t operand_dtype, void* c, int32_t c_dtype, uint64_t m, uint64_t k,
                 uint64_t n, int32_t accumulate) {
  OMX_REQUIRE_CTX(ctx);
  return omx_gemm_impl(ctx, F_GEMM, a, a_rs, a_cs, b, b_rs, b_cs, operand_dtype, c, c_dtype, n, m, k, n, accumulate);
}

int32_t omx_gemm_pitched(omx_ctx* ctx, const void* a, uint64_t a_rs, uint64_t a_cs, const void* b, uint64_t b_rs,
                         uint64_t b_cs, int32_t operand_dtype, void* c, int32_t c_dtype, uint64_t ldc, uint64_t m,
                         uint64_t k, uint64_t n, int32_t accumulate) {
  OMX_REQUIRE_CTX(ctx);
  if (ldc < n) return omx_fail(ctx, OMX_SHAPE, "gemm: output pitch %llu is below its %llu columns", (unsigned long long)ldc,
                               (unsigned long long)n);
  return omx_gemm_impl(ctx, F_GEMM, a, a_rs, a_cs, b, b_rs, b_cs, operand_dtype, c, c_dtype, ldc, m, k, n, accumulate);
}

int32_t omx_gemm_strided_batch(omx_ctx* ctx, const void* a, uint64_t a_rs, uint64_t a_cs, const void* b,
                               uint64_t b_rs, uint64_t b_cs, int32_t operand_dtype, void* c, int32_t c_dtype,
                               uint64_t m, uint64_t k, uint64_t n, int32_t accumulate, uint64_t count,
                               uint64_t stride_a, uint64_t stride_b, uint64_t stride_c) {
  OMX_REQUIRE_CTX(ctx);
  const OmxGemmBatch batch{count, stride_a, stride_b, stride_c};
  return omx_gemm_impl(ctx, F_GEMM, a, a_rs, a_cs, b, b_rs, b_cs, operand_dtype, c, c_dtype, n, m, k, n, accumulate,
                       nullptr, &batch);
}

int32_t omx_gemm_pitched_strided_batch(omx_ctx* ctx, const void* a, uint64_t a_rs, uint64_t a_cs, const void* b,
                                       uint64_t b_rs, uint64_t b_cs, int32_t operand_dtype, void* c, int32_t c_dtype,
                                       uint64_t ldc, uint64_t m, uint64_t k, uint64_t n, int32_t accumulate,
                                       uint64_t count, uint64_t stride_a, uint64_t stride_b, uint64_t stride_c) {
  OMX_REQUIRE_CTX(ctx);
  if (ldc < n) return omx_fail(ctx, OMX_SHAPE, "gemm: output pitch %llu is below its %llu columns", (unsigned long long)ldc,
                               (unsigned long long)n);
  const OmxGemmBatch batch{count, stride_a, stride_b, stride_c};
  return omx_gemm_impl(ctx, F_GEMM, a, a_rs, a_cs, b, b_rs, b_cs, operand_dtype, c, c_dtype, ldc, m, k, n, accumulate,
                       nullptr, &batch);
}

}  // extern "C"
