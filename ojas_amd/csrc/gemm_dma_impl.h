// The direct-to-LDS bf16 GEMM kernels and their launcher, as templates on the operand layout.
// One translation unit per layout includes this file (they compile side by side); gemm_dma.hip
// holds the description of the kernels and chooses among the four.
#pragma once
#include "gemm_tiles.h"
#include "gemm_w4_impl.h"

namespace {

// EPI: the store pass this instantiation is compiled for (OMX_EPI_*), or OMX_EPI_ANY for the one
// that chooses at run time. A kernel of its own per store pass keeps each one's code (a few KiB of
// straight-line stores) and registers out of the others.
constexpr int OMX_EPI_ANY = -1;
template <bool A_KM, bool B_KM, int WGM, int WGN, int TM, int TN, int DBK, int NST, int EPI = OMX_EPI_ANY>
__global__ __launch_bounds__(WGM* WGN * 64, dma_waves_per_simd(WGM* WGN, NST*(WGM* TM + WGN * TN) * 32 * DBK * 2)) void
gemm_dma_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32;
  constexpr int A_BYTES = BM * DBK * 2, B_BYTES = BN * DBK * 2, STAGE = A_BYTES + B_BYTES;
  constexpr int NW = WGM * WGN;           // waves per workgroup
  constexpr int LPS = STAGE / 1024 / NW;  // loads per wave per step
  constexpr int KK = DBK / 16;            // MFMA K slabs per step
  static_assert(NW == 4 || NW == 8, "four or eight waves");
  // Six waves share 16 + 24 loads unevenly; with two stages every wait is for all of a wave's loads.
  static_assert(STAGE % (1024 * NW) == 0 || NST == 2, "counted waits need the same number of loads in every wave");

  // Workgroups go to the 8 XCDs round-robin by blockIdx.x, and each XCD has its own L2. Without
  // split-K an XCD takes a contiguous eighth of the tiles; with it, blockIdx.x % splits is the
  // split, so (for the power-of-two split counts the host picks) all tiles of one K chunk run on
  // the same XCD, side by side, and that chunk of both operands is fetched into one L2 once
  // instead of into all eight.
  // In a strided batch (grid.y = products, never split) an XCD takes a contiguous eighth of the
  // (product, tile) pairs instead of an eighth of every product's tiles, so a product's operands
  // are fetched into one or two L2s instead of all eight.
  const int total = g.tiles_m * g.tiles_n;
  int split = 0, id = blockIdx.x, product = blockIdx.y;
  if (g.batches > 1 && g.splits == 1 && ((total * g.batches) & 7) == 0) {
    const int linear = blockIdx.y * total + blockIdx.x;
    const int r = (linear & 7) * ((total * g.batches) >> 3) + (linear >> 3);
    product = r / total;
    id = r - product * total;
  } else if (g.splits > 1) {
    split = blockIdx.x % g.splits;
    id = blockIdx.x / g.splits;
  } else if (total % 8 == 0) {
    id = (id & 7) * (total >> 3) + (id >> 3);
  }
  const int band = 4;
  const int tiles_per_band = band * g.tiles_n;
  const int band_id = id / tiles_per_band;
  const int first_m = band_id * band;
  const int band_rows = min(band, g.tiles_m - first_m);
  const int in_band = id - band_id * tiles_per_band;
  const int tile_m = first_m + in_band % band_rows;
  const int tile_n = in_band / band_rows;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  gemm_select_batch(g, product);
  const unsigned short* __restrict__ A = static_cast<const unsigned short*>(g.a);
  const unsigned short* __restrict__ B = static_cast<const unsigned short*>(g.b);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WGN, wn = wave % WGN;
  const int l32 = lane & 31, lg = lane >> 5;

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // g.ksteps_per_split counts 64-wide K blocks.
  constexpr int SPB = 64 / DBK;  // pipeline steps per block
  const int ks_begin = SPB * split * g.ksteps_per_split;
  const int ks_end = min(g.K / DBK, ks_begin + SPB * g.ksteps_per_split);
  // Everything a K step needs is computed here, once per tile: the loads' global addresses and
  // the fragments' LDS offsets. Inside the loop the stage is a compile-time constant (the loop
  // body is unrolled over the stages), so a step is loads, LDS reads and MFMAs and little else.
  // (scalar base + lane offsets where every wave issues the same number of loads of each operand)
  constexpr bool EVEN_LOADS = (BM * DBK * 2 / 1024) % NW == 0 && (BN * DBK * 2 / 1024) % NW == 0;
  std::conditional_t<EVEN_LOADS, TileLoadsOff<A_KM, BM, DBK, NW>, TileLoads<A_KM, BM, DBK, NW>> la;
  std::conditional_t<EVEN_LOADS, TileLoadsOff<B_KM, BN, DBK, NW>, TileLoads<B_KM, BN, DBK, NW>> lb;
  la.init(A, g.lda, m0, g.M, ks_begin * DBK, wave, lane);
  lb.init(B, g.ldb, n0, g.N, ks_begin * DBK, wave, lane);
  const unsigned lds0 = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<uintptr_t>(smem)));
  int a_off[TM][KK], b_off[TN][KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
    for (int t = 0; t < TM; ++t) a_off[t][kk] = frag_offset<A_KM, BM, DBK>((wm * TM + t) * 32, kk, lane);
#pragma unroll
    for (int t = 0; t < TN; ++t) b_off[t][kk] = A_BYTES + frag_offset<B_KM, BN, DBK>((wn * TN + t) * 32, kk, lane);
  }
  // Waits until at most `groups` of this wave's per-step load groups are still in flight.
  auto wait_groups = [&](int groups) {
    static_assert(2 * LPS < 64, "vmcnt is six bits");
    if (groups >= 2) __builtin_amdgcn_s_waitcnt(vmcnt_only(2 * LPS));
    else if (groups == 1) __builtin_amdgcn_s_waitcnt(vmcnt_only(LPS));
    else __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
  };

#pragma unroll
  for (int i = 0; i < NST - 1; ++i)
    if (ks_begin + i < ks_end) {
      la.issue(lds0 + i * STAGE, wave);
      lb.issue(lds0 + i * STAGE + A_BYTES, wave);
    }
  wait_groups(min(NST - 2, ks_end - ks_begin - 1));
  __syncthreads();
  // The fragments of the next 16-column slab are read while the current slab is multiplied; the
  // first slab of the next step is read right after the barrier that publishes its stage, ahead
  // of the last slab's products, so neither the LDS latency nor the barrier drains the MFMA pipe.
  // Two sets of fragment registers that take turns (a step has an even number of slabs, so slab 0 of every step
  // finds its fragments in set 0): no copies, and no wait for the next slab's fragments before this slab's
  // products have been issued.
  static_assert(KK % 2 == 0, "the fragment sets alternate by slab");
  u32x4 af[2][TM], bf[2][TN];
  auto read_frags = [&](const char* stage, int kk, u32x4(&a)[TM], u32x4(&b)[TN]) {
#pragma unroll
    for (int t = 0; t < TM; ++t) a[t] = frag_at<A_KM, BM>(stage + a_off[t][kk]);
#pragma unroll
    for (int t = 0; t < TN; ++t) b[t] = frag_at<B_KM, BN>(stage + b_off[t][kk]);
  };
  read_frags(smem, 0, af[0], bf[0]);
  // One K step: the loads of step ks + NST - 1, then the slabs of stage `stage` (fragments one slab
  // ahead), the wait + barrier before the last slab's products, and the first slab of `next`.
  auto k_step = [&](int ks, unsigned fill_stage, const char* stage, const char* next) {
    if (ks + NST - 1 < ks_end) {
      la.issue(lds0 + fill_stage * STAGE, wave);
      lb.issue(lds0 + fill_stage * STAGE + A_BYTES, wave);
    }
    static_for<0, KK>([&](auto kk_index) {
      constexpr int kk = decltype(kk_index)::value, cur = kk % 2, nxt = cur ^ 1;
      if constexpr (kk + 1 < KK) {
        read_frags(stage, kk + 1, af[nxt], bf[nxt]);
      } else {
        // Step ks + 1 must have landed (this wave's share, then everyone's); later steps may
        // still be in flight. Every wave has its last fragments of this stage in registers by
        // now, so the barrier also releases the stage for the loads of step ks + NST.
        wait_groups(min(NST - 2, ks_end - ks - 2));
        __syncthreads();
        if (ks + 1 < ks_end) read_frags(next, 0, af[nxt], bf[nxt]);
      }
      // Keeps the reads above the products: the scheduler would otherwise sink them to their
      // first use to save registers, which puts the LDS latency back in front of every slab.
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
          acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, af[cur][tm]),
                                                                __builtin_bit_cast(bf16x8, bf[cur][tn]), acc[tm][tn], 0,
                                                                0, 0);
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  if constexpr (TM * TN <= 4) {
    // Unrolled over the stages, so every LDS address is the precomputed offset plus a constant.
    for (int ks = ks_begin; ks < ks_end;) {
#pragma unroll
      for (int st = 0; st < NST; ++st) {  // step ks lives in stage st
        k_step(ks, (st + NST - 1) % NST, smem + st * STAGE, smem + ((st + 1) % NST) * STAGE);
        if (++ks >= ks_end) break;
      }
    }
  } else {
    // With 256 accumulator registers per lane the unrolled form runs out of registers; the stage is
    // a loop variable here, at the price of one address add per fragment read.
    int st = 0;
#pragma unroll 1
    for (int ks = ks_begin; ks < ks_end; ++ks) {
      const int nx = st + 1 == NST ? 0 : st + 1;
      k_step(ks, st == 0 ? NST - 1 : st - 1, smem + st * STAGE, smem + nx * STAGE);
      st = nx;
    }
  }
  __syncthreads();  // the staging below reuses the stages

  // Epilogue: each wave stages 32 rows of its tile at a time through its own
  // LDS region and writes whole 4-column pieces.
  constexpr int CPW = TN * 32 + 4;
  static_assert(NW * 32 * CPW * 4 <= NST * STAGE, "staging fits");
  float* cs = reinterpret_cast<float*>(smem) + wave * (32 * CPW);
  bool bad = false;
  // The row block is a compile-time index (the body is too long for the unroller to take on its
  // own, and a run-time index would move the accumulators to scratch memory).
  static_for<0, TM>([&](auto tm_index) {
    constexpr int tm = decltype(tm_index)::value;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int v = 0; v < 16; ++v) cs[(8 * (v >> 2) + 4 * lg + (v & 3)) * CPW + tn * 32 + l32] = acc[tm][tn][v];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    constexpr int PPR = TN * 8;  // 4-column pieces per row
    // A block that lies wholly inside the output takes a straight-line store loop (compiled for
    // the two forms the dispatcher picks by itself); edge blocks and the other forms go piece by piece.
    constexpr bool kFastStores = (DBK == 32 && TM * TN <= 4) || NW == 6;
    const int grow0 = m0 + (wm * TM + tm) * 32, gcol0 = n0 + wn * TN * 32;
    bool stored = false;
    if constexpr (kFastStores) {
      const bool interior = grow0 + 32 <= g.M && gcol0 + TN * 32 <= g.N;
      if constexpr (EPI == OMX_EPI_ANY || EPI == OMX_EPI_NONE) {
        if (interior && g.epi == OMX_EPI_NONE && (g.splits > 1 ? (g.N & 3) == 0 : g.c_vec != 0)) {
          if (g.splits > 1) bad |= gemm_store_block<0, PPR>(g, split, cs, CPW, grow0, gcol0, lane);
          else if (g.c_bf16) bad |= gemm_store_block<1, PPR>(g, split, cs, CPW, grow0, gcol0, lane);
          else if (!g.accumulate) bad |= gemm_store_block<2, PPR>(g, split, cs, CPW, grow0, gcol0, lane);
          else bad |= gemm_store_block<3, PPR>(g, split, cs, CPW, grow0, gcol0, lane);
          stored = true;
        }
      }
      if constexpr (EPI == OMX_EPI_ANY) {
        if (!stored && interior && g.epi != OMX_EPI_NONE && g.c_vec != 0) {
          if (g.epi == OMX_EPI_GELU_FWD) {
            bad |= g.epi_tanh ? gemm_epilogue_block<OMX_EPI_GELU_FWD, true, PPR>(g, cs, CPW, grow0, gcol0, lane)
                              : gemm_epilogue_block<OMX_EPI_GELU_FWD, false, PPR>(g, cs, CPW, grow0, gcol0, lane);
          } else if (g.epi == OMX_EPI_AXPBY) {
            bad |= gemm_epilogue_block<OMX_EPI_AXPBY, false, PPR>(g, cs, CPW, grow0, gcol0, lane);
          } else {
            bad |= g.epi_tanh ? gemm_epilogue_block<OMX_EPI_GELU_BWD, true, PPR>(g, cs, CPW, grow0, gcol0, lane)
                              : gemm_epilogue_block<OMX_EPI_GELU_BWD, false, PPR>(g, cs, CPW, grow0, gcol0, lane);
          }
          stored = true;
        }
      } else if constexpr (EPI == OMX_EPI_AXPBY) {
        if (interior && g.c_vec != 0) {
          bad |= gemm_epilogue_block<OMX_EPI_AXPBY, false, PPR>(g, cs, CPW, grow0, gcol0, lane);
          stored = true;
        }
      } else if constexpr (EPI != OMX_EPI_NONE) {
        if (interior && g.c_vec != 0) {
          bad |= g.epi_tanh ? gemm_epilogue_block<EPI, true, PPR>(g, cs, CPW, grow0, gcol0, lane)
                            : gemm_epilogue_block<EPI, false, PPR>(g, cs, CPW, grow0, gcol0, lane);
          stored = true;
        }
      }
    }
    if (!stored) {
#pragma unroll 1
      for (int c = lane; c < 32 * PPR; c += 64) {
        const int row = c / PPR, piece = c % PPR;
        const int grow = grow0 + row, gcol = gcol0 + piece * 4;
        if (grow < g.M && gcol < g.N) {
          const float4 val = *reinterpret_cast<const float4*>(cs + row * CPW + piece * 4);
          bad |= g.epi == OMX_EPI_NONE ? gemm_store4(g, split, grow, gcol, val.x, val.y, val.z, val.w)
                                       : gemm_store4_epi(g, split, grow, gcol, val.x, val.y, val.z, val.w);
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  });
  if (bad) dev_raise_fault(g.fault, g.tag);
}

template <bool A_KM, bool B_KM, int WGM, int WGN, int TM, int TN, int DBK, int NST>
int32_t launch_dma(omx_ctx* ctx, const GemmArgs& g) {
  constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32;
  constexpr int smem = NST * (BM + BN) * DBK * 2;
  auto kernel = &gemm_dma_kernel<A_KM, B_KM, WGM, WGN, TM, TN, DBK, NST>;
  // The two tiles the dispatcher picks by itself have a kernel per store pass.
  if constexpr (DBK == 32 && TM * TN <= 4 && NST == 3) {
    kernel = g.epi == OMX_EPI_GELU_FWD   ? &gemm_dma_kernel<A_KM, B_KM, WGM, WGN, TM, TN, DBK, NST, OMX_EPI_GELU_FWD>
             : g.epi == OMX_EPI_GELU_BWD ? &gemm_dma_kernel<A_KM, B_KM, WGM, WGN, TM, TN, DBK, NST, OMX_EPI_GELU_BWD>
             : g.epi == OMX_EPI_AXPBY    ? &gemm_dma_kernel<A_KM, B_KM, WGM, WGN, TM, TN, DBK, NST, OMX_EPI_AXPBY>
                                         : &gemm_dma_kernel<A_KM, B_KM, WGM, WGN, TM, TN, DBK, NST, OMX_EPI_NONE>;
  }
  OMX_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   smem));
  omx_launch_timed(ctx, kernel, dim3(g.tiles_m * g.tiles_n * g.splits, g.batches), dim3(WGM * WGN * 64), smem,
                   ctx->timing_start, g.splits > 1 ? nullptr : ctx->timing_stop, g);
  OMX_LAUNCH_CHECK(ctx, "gemm_dma_kernel");
  return OMX_OK;
}

// The tilings the dispatcher chooses among: 9 and 10: 256 x 256 and 256 x 192, one wave per SIMD, one
// workgroup per compute unit (gemm_w4_impl.h); 3: 256 x 128 in 32-column steps (three stages, two workgroups per
// compute unit); 6: 128 x 128 with four waves (three per compute unit).
template <bool A_KM, bool B_KM>
int32_t launch_variant(omx_ctx* ctx, const GemmArgs& g, int variant) {
  if (variant == 9 || variant == 10) {
    // (the caller has asked omx_gemm_w4_eligible: a k-major A comes with a k-major B and 256 x 256 tiles)
    if constexpr (!A_KM || B_KM) {
      return variant == 10 ? launch_w4<A_KM, B_KM, 3>(ctx, g) : launch_w4<A_KM, B_KM, 4>(ctx, g);
    }
    return omx_fail(ctx, OMX_SHAPE, "gemm: no one-wave-per-SIMD kernel for this operand layout");
  }
  if (variant == 6) return launch_dma<A_KM, B_KM, 2, 2, 2, 2, 32, 3>(ctx, g);
  return launch_dma<A_KM, B_KM, 4, 2, 2, 2, 32, 3>(ctx, g);
}

}  // namespace
