// bf16 product with a thin output: C[M, N] = A.B with N <= 64 (a low-rank adapter's h = x A^T and
// gh = gy B, a gate's 12 logits per token). Same contract as gemm.hip (f32 accumulation; reference:
// ojas-cpu/src/linalg.rs:69-210).
//
// Such a product reads M x K of A for almost no arithmetic: it is bound by reading A once. On the
// tiled kernels its one column of tiles has to split K to fill the chip and needs a reduce launch
// for it. Here a workgroup owns 16 rows of A and its four waves a quarter of K each; both operands go
// from global memory straight into v_mfma_f32_16x16x32_bf16 fragments (a lane's eight k-contiguous
// values are one 16-byte load), every load of a wave's K range is in flight before its first
// product, and the four partial sums meet in LDS in wave order. B (N x K, a few tens of KiB) is
// re-read by every workgroup and stays in L2.
#include "gemm_tiles.h"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

constexpr int THIN_ROWS = 16;   // rows of A per workgroup
constexpr int THIN_WAVES = 4;   // K slices per workgroup
constexpr int THIN_CHUNK = 16;  // 32-column steps whose loads are in flight together
constexpr int THIN_MAX_N = 64;

// Eight k-consecutive values of B for output column n: one 16-byte load where k is contiguous,
// eight two-byte loads where n is.
template <bool B_KM>
__device__ __forceinline__ u32x4_t thin_b_frag(const unsigned short* __restrict__ b, long ldb, int n, int k) {
  if constexpr (!B_KM) {
    return *reinterpret_cast<const u32x4_t*>(b + static_cast<long>(n) * ldb + k);
  } else {
    const unsigned short* p = b + static_cast<long>(k) * ldb + n;
    u32x4_t r;
    r.x = p[0] | (static_cast<unsigned int>(p[ldb]) << 16);
    r.y = p[2 * ldb] | (static_cast<unsigned int>(p[3 * ldb]) << 16);
    r.z = p[4 * ldb] | (static_cast<unsigned int>(p[5 * ldb]) << 16);
    r.w = p[6 * ldb] | (static_cast<unsigned int>(p[7 * ldb]) << 16);
    return r;
  }
}

template <bool B_KM>
__global__ __launch_bounds__(THIN_WAVES * 64) void gemm_thin_kernel(GemmArgs g) {
  gemm_select_batch(g, blockIdx.y);
  __shared__ float red[THIN_WAVES][THIN_MAX_N / 16][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l16 = lane & 15, kc = (lane >> 4) * 8;
  const int row0 = blockIdx.x * THIN_ROWS;
  const int row = min(row0 + l16, g.M - 1);  // rows past M are read from the last one and never stored
  const unsigned short* a = static_cast<const unsigned short*>(g.a) + static_cast<long>(row) * g.lda;
  const unsigned short* b = static_cast<const unsigned short*>(g.b);
  const int nblocks = (g.N + 15) / 16;
  const int kslice = g.K / THIN_WAVES;  // a multiple of 32
  const int k_begin = wave * kslice;
  floatx4_t acc[THIN_MAX_N / 16];
#pragma unroll
  for (int nb = 0; nb < THIN_MAX_N / 16; ++nb) acc[nb] = floatx4_t{0.0f, 0.0f, 0.0f, 0.0f};
  for (int k0 = 0; k0 < kslice; k0 += 32 * THIN_CHUNK) {
    const int steps = min(THIN_CHUNK, (kslice - k0) / 32);
    u32x4_t xf[THIN_CHUNK];
#pragma unroll
    for (int s = 0; s < THIN_CHUNK; ++s)
      if (s < steps) xf[s] = *reinterpret_cast<const u32x4_t*>(a + k_begin + k0 + 32 * s + kc);
#pragma unroll
    for (int nb = 0; nb < THIN_MAX_N / 16; ++nb) {
      if (nb < nblocks) {
        const int n = min(nb * 16 + l16, g.N - 1);
        u32x4_t bf[THIN_CHUNK];
#pragma unroll
        for (int s = 0; s < THIN_CHUNK; ++s)
          if (s < steps) bf[s] = thin_b_frag<B_KM>(b, g.ldb, n, k_begin + k0 + 32 * s + kc);
#pragma unroll
        for (int s = 0; s < THIN_CHUNK; ++s)
          if (s < steps)
            acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, bf[s]),
                                                              __builtin_bit_cast(bf16x8_t, xf[s]), acc[nb], 0, 0, 0);
      }
    }
  }
  // acc[nb][v] is C[row l16][column nb * 16 + 4 * (lane / 16) + v] of this wave's K slice.
#pragma unroll
  for (int nb = 0; nb < THIN_MAX_N / 16; ++nb)
    if (nb < nblocks)
#pragma unroll
      for (int v = 0; v < 4; ++v) red[wave][nb][v][lane] = acc[nb][v];
  __syncthreads();
  // Wave w adds up column blocks w, w + 4, ...: the slices in order 0, 1, 2, 3.
  bool bad = false;
  for (int nb = wave; nb < nblocks; nb += THIN_WAVES) {
    float x[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) x[v] = ((red[0][nb][v][lane] + red[1][nb][v][lane]) + red[2][nb][v][lane]) + red[3][nb][v][lane];
    if (row0 + l16 < g.M) bad |= gemm_store4(g, 0, row0 + l16, nb * 16 + (lane >> 4) * 4, x[0], x[1], x[2], x[3]);
  }
  if (bad) dev_raise_fault(g.fault, g.tag);
}

}  // namespace

bool omx_gemm_thin_eligible(const GemmArgs& g, bool a_km, bool b_km) {
  if (a_km || g.N > THIN_MAX_N || g.K % (32 * THIN_WAVES) != 0 || !g.a_vec) return false;
  if (!b_km && !g.b_vec) return false;
  if (g.accumulate || g.M < 1024) return false;  // few rows: the tiled kernels' split-K has more waves
  return true;
}

int32_t omx_gemm_thin_launch(omx_ctx* ctx, const GemmArgs& g, bool b_km) {
  dim3 grid(static_cast<unsigned>((g.M + THIN_ROWS - 1) / THIN_ROWS), static_cast<unsigned>(g.batches));
  if (b_km) omx_launch_timed(ctx, gemm_thin_kernel<true>, grid, dim3(THIN_WAVES * 64), 0, ctx->timing_start, ctx->timing_stop, g);
  else omx_launch_timed(ctx, gemm_thin_kernel<false>, grid, dim3(THIN_WAVES * 64), 0, ctx->timing_start, ctx->timing_stop, g);
  OMX_LAUNCH_CHECK(ctx, "gemm_thin_kernel");
  return OMX_OK;
}
