// bf16 MFMA GEMM with direct-to-LDS loads (global_load_lds_dwordx4) and a large
// workgroup tile, for shapes whose output has enough tiles to fill the chip.
//
// Same contract as gemm.hip (C[M,N] (+)= A.B, f32 accumulation, every operand
// layout; reference: ojas-cpu/src/linalg.rs:69-210), different data movement:
//   * 512 threads (8 waves); tile 256 x 128 (waves 4 x 2, each 64 x 64) or 256 x 256 (waves
//     2 x 4, each 128 x 64; half the L2-to-LDS traffic per FLOP).
//   * Variant 3, the default: K steps of 32 columns, three stages in 72 KiB and at most 128
//     VGPRs, so two workgroups share a compute unit and one's output stores, first loads and
//     barrier waits overlap the other's products. Its weakness: a k-contiguous operand row
//     contributes half a 128-byte cache line per step, each line is requested twice, far enough
//     apart that the second request misses L1 again, and the load path then delivers 65 GB/s
//     per compute unit instead of 107 GB/s (measured with the loads alone).
//   * Variant 0 (256 x 256, two stages): K steps of 64 columns, whole cache lines, one workgroup per
//     compute unit. Load latency (about 0.6 us) is then exposed; it wins on long reductions with
//     large outputs only.
//   * operand tiles go from global memory straight into LDS: no staging
//     registers and no LDS store instructions. A wave-wide load writes 64
//     consecutive 16-byte slots, so the LDS tile is unpadded and bank conflicts
//     are avoided by choosing WHICH chunk each lane fetches (an XOR swizzle):
//       k-contiguous operand, [row][BK/8 chunks]: slot s of row r holds chunk s ^ ((r >> 2) & 3)
//         for 64-byte rows and s ^ ((r >> 1) & 7) for 128-byte rows;
//       k-major operand, [k][ROWS/8 chunks]:   slot s of k row kr holds chunk s ^ 4(kr & 3).
//     LDS has 64 four-byte banks: a 16-byte read serves 16 lanes per clock, i.e. rows r..r+15 of
//     one chunk column, whose 64-byte rows repeat banks every 4 rows (128-byte rows: every 2),
//     so the XOR must separate rows r, r+4, r+8, r+12 (r, r+2, ..., r+14); a transposing 8-byte read serves 32 lanes per clock, four k rows of
//     64 bytes each, which the XOR moves 64 bytes apart. Both measured conflict-free
//     (4.0 and 1.9 clocks per wave read with 16 waves; 7.1 and 3.0 with a 2-way conflict).
//   * NST LDS stages: the loads of K steps ks+1 .. ks+NST-1 are in flight while step ks is
//     multiplied; one counted vmcnt wait + barrier per step.
// Rows past M (or N) are fetched from a clamped valid address and never stored.
#include "gemm_tiles.h"

int32_t omx_gemm_dma_launch_nn(omx_ctx* ctx, const GemmArgs& g, int variant);
int32_t omx_gemm_dma_launch_nt(omx_ctx* ctx, const GemmArgs& g, int variant);
int32_t omx_gemm_dma_launch_tn(omx_ctx* ctx, const GemmArgs& g, int variant);
int32_t omx_gemm_dma_launch_tt(omx_ctx* ctx, const GemmArgs& g, int variant);

bool omx_gemm_dma_eligible(const GemmArgs& g, bool a_km, bool b_km) {
  if (g.K % 64 != 0 || !g.a_vec || !g.b_vec) return false;
  if (g.lda >= (1l << 22) || g.ldb >= (1l << 22)) return false;  // a tile's lane offsets are 32 bits of bytes
  if (a_km && g.M % 8 != 0) return false;
  if (b_km && g.N % 8 != 0) return false;
  return true;
}

// The one-wave-per-SIMD kernel (variants 9 and 10) also needs a k-major B with a k-major A, an even
// number of 64-column K steps, and a store pass without an activation.
bool omx_gemm_w4_eligible(const GemmArgs& g, bool a_km, bool b_km, bool plain) {
  return plain && (!a_km || b_km) && g.K % 128 == 0;
}

void omx_gemm_dma_tile(int variant, int* bm, int* bn) {
  *bm = variant == 6 ? 128 : 256;
  *bn = variant == 9 ? 256 : variant == 10 ? 192 : 128;
}


// One translation unit per operand layout holds the kernels (gemm_dma_impl.h).
int32_t omx_gemm_dma_launch(omx_ctx* ctx, const GemmArgs& g, bool a_km, bool b_km, int variant) {
  if (!a_km && !b_km) return omx_gemm_dma_launch_nn(ctx, g, variant);
  if (!a_km && b_km) return omx_gemm_dma_launch_nt(ctx, g, variant);
  if (a_km && !b_km) return omx_gemm_dma_launch_tn(ctx, g, variant);
  return omx_gemm_dma_launch_tt(ctx, g, variant);
}
