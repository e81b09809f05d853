// The bf16 GEMM in its alternating form: a 256 x 256 output tile per workgroup, one workgroup per
// compute unit, eight waves of 128 x 64 in two groups of four (one wave of each group on every
// SIMD) that take turns: while one group's waves issue their matrix products for half a K step
// from fragments already in registers, the other group's waves read their next fragments out of
// LDS and start global -> LDS loads. A barrier closes every turn, so the two groups stay half a
// step apart for the whole tile: the matrix pipe of a SIMD always has one wave issuing products
// back to back, with no memory instruction of its own in between, and the LDS reads, the load
// issue and every wait of the other wave are hidden behind them.
//
//   K steps of 64 columns (whole 128-byte lines of a k-contiguous operand), two LDS stages of
//   64 KiB; step j lives in stage j % 2. A step is consumed in two halves of 16 products
//   (v_mfma_f32_32x32x16_bf16, 512 clocks of the matrix pipe) each, and a half is what one set of
//   loads can refill:
//     A k-contiguous (a load covers 8 rows x 64 columns): half 0 is the wave's row blocks 0-1 over
//       the whole step against all of B, half 1 its row blocks 2-3 against the same B fragments,
//       which stay in registers. Part 0 of a stage = B and the A rows of half 0, part 1 = the A
//       rows of half 1.
//     A k-major (a load covers 2 K rows x 256 rows): half h is K slabs 2h, 2h+1 of every block.
//       Part h = K rows 32h .. 32h+31 of A, and of B when B is k-major too (a k-contiguous B is
//       refilled whole with part 1).
//
//   turn      group 0 (waves 0-3, tile rows 0-127)       group 1 (waves 4-7, tile rows 128-255)
//   S0(j)     read half 0 of step j; start part 1 of      start part 1 of step j+1; products of
//             step j+1                                    half 1 of step j-1
//   S1(j)     products of half 0                          read half 0 of step j
//   S2(j)     read half 1 of step j; start part 0 of      start part 0 of step j+2; products of
//             step j+2                                    half 0
//   S3(j)     products of half 1                          read half 1
//
//   Both groups have read part 0 of step j by the end of S1(j) and part 1 by the end of S3(j), and
//   each part is refilled in the turn after that, for the step two ahead: every load has six turns
//   (one and a half steps, about 1.6 us) to land, where refilling a stage only once all of it has
//   been read would leave four. That matters because a compute unit's load path takes about
//   0.5 us to stream a step's 64 KiB on top of about 0.6 us of latency: four turns (1.05 us at
//   full matrix rate) cannot hide that, six can. Each wave waits for its own loads of a part
//   before the barrier that precedes the part's first read (a counted vmcnt: the loads issued
//   since may stay in flight), and that barrier publishes them to the other waves.
//
// The operand tiles, their swizzle and the fragment reads are those of gemm_dma_kernel
// (gemm_tiles.h); the store pass is its staged one (a wave's 32-row blocks through its own LDS
// region), which group 0 runs while group 1 still multiplies its last half step.
#pragma once
#include "gemm_tiles.h"

namespace {

constexpr int PP_BM = 256, PP_BN = 256, PP_BK = 64;
constexpr int PP_A_BYTES = PP_BM * PP_BK * 2, PP_B_BYTES = PP_BN * PP_BK * 2, PP_STAGE = PP_A_BYTES + PP_B_BYTES;
constexpr int PP_SMEM = 2 * PP_STAGE;

// s_waitcnt operand that waits for lgkmcnt == 0 only (vmcnt and expcnt at their maxima).
constexpr int lgkmcnt_zero() { return 0xC07F; }

template <bool A_KM, bool B_KM, int EPI>
__global__ __launch_bounds__(512, 2) void gemm_pp_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int TM = 4, TN = 2, NW = 8;
  // Tile order: as gemm_dma_kernel (an XCD takes a contiguous eighth of the tiles; with split-K
  // the splits of one K chunk share an XCD; bands of four tile rows).
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
  const int m0 = tile_m * PP_BM, n0 = tile_n * PP_BN;
  gemm_select_batch(g, product);
  const unsigned short* __restrict__ A = static_cast<const unsigned short*>(g.a);
  const unsigned short* __restrict__ B = static_cast<const unsigned short*>(g.b);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave >> 2, wn = wave & 3;
  const int l32 = lane & 31, lg = lane >> 5;

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // g.ksteps_per_split counts 64-wide K blocks.
  const int ks_begin = split * g.ksteps_per_split;
  const int ks_end = min(g.K / PP_BK, ks_begin + g.ksteps_per_split);
  const int steps = ks_end - ks_begin;
  TileLoads<A_KM, PP_BM, PP_BK, NW> la;
  TileLoads<B_KM, PP_BN, PP_BK, NW> lb;
  la.init(A, g.lda, m0, g.M, ks_begin * PP_BK, wave, lane);
  lb.init(B, g.ldb, n0, g.N, ks_begin * PP_BK, wave, lane);
  const unsigned lds0 = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<uintptr_t>(smem)));
  const int a_first = frag_offset<A_KM, PP_BM, PP_BK>(wm * 128, 0, lane);
  const int b_first = PP_A_BYTES + frag_offset<B_KM, PP_BN, PP_BK>(wn * 64, 0, lane);

  // The loads of one part of a step into `stage`.
  constexpr bool BY_ROWS = !A_KM;
  constexpr int N0 = BY_ROWS ? 6 : (B_KM ? 4 : 2), N1 = 8 - N0;  // loads per wave in part 0 / part 1
  auto issue_part = [&](int stage, auto part_index) {
    constexpr int part = decltype(part_index)::value;
    const unsigned ta = lds0 + stage * PP_STAGE, tb = ta + PP_A_BYTES;
    if constexpr (BY_ROWS) {
      // A load i of wave w fills rows 8 (w + 8 i) ..: i = 0, 2 are the row blocks of half 0.
      if constexpr (part == 0) {
        lb.template issue_some<0xFu>(tb, wave);
        la.template issue_some<0x5u>(ta, wave);
      } else {
        la.template issue_some<0xAu>(ta, wave);
      }
    } else {
      // A load i of wave w fills K rows 2 (w + 8 i), +1: i = 0, 1 are K rows 0-31.
      if constexpr (part == 0) {
        la.template issue_some<0x3u>(ta, wave);
        if constexpr (B_KM) lb.template issue_some<0x3u>(tb, wave);
      } else {
        la.template issue_some<0xCu>(ta, wave);
        if constexpr (B_KM) lb.template issue_some<0xCu>(tb, wave);
        else lb.template issue_some<0xFu>(tb, wave);
      }
    }
  };
  // Waits until at most `n` of this wave's loads (the most recently issued) are in flight.
  constexpr int NO_WAIT = 64;
  auto wait_loads = [&](int n) {
    if (n >= NO_WAIT) return;
    if (n >= 8) __builtin_amdgcn_s_waitcnt(vmcnt_only(8));
    else if (n >= 6) __builtin_amdgcn_s_waitcnt(vmcnt_only(6));
    else if (n >= 4) __builtin_amdgcn_s_waitcnt(vmcnt_only(4));
    else if (n >= 2) __builtin_amdgcn_s_waitcnt(vmcnt_only(2));
    else __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
  };
  // Fragments: by rows, 2 row blocks x 4 slabs of A and (read with half 0, kept for half 1)
  // 2 column blocks x 4 slabs of B; by K, 4 row blocks x 2 slabs of A and 2 x 2 of B.
  constexpr int FA_T = BY_ROWS ? 2 : 4, FA_K = BY_ROWS ? 4 : 2, FB_K = BY_ROWS ? 4 : 2;
  u32x4 fa[FA_T][FA_K], fb[TN][FB_K];
  auto read_half = [&](int stage, auto half_index) {
    constexpr int half = decltype(half_index)::value;
    const char* base = smem + stage * PP_STAGE;
    static_for<0, FA_K>([&](auto k_index) {
      constexpr int k = decltype(k_index)::value;
      constexpr int kk = BY_ROWS ? k : 2 * half + k;
      static_for<0, FA_T>([&](auto t_index) {
        constexpr int t = decltype(t_index)::value;
        constexpr int block = BY_ROWS ? 2 * half + t : t;
        fa[t][k] = frag_at<A_KM, PP_BM>(base + frag_from_first<A_KM, PP_BM, PP_BK, block, kk>(a_first));
      });
      if constexpr (!BY_ROWS || half == 0) {
        static_for<0, TN>([&](auto t_index) {
          constexpr int t = decltype(t_index)::value;
          fb[t][k] = frag_at<B_KM, PP_BN>(base + frag_from_first<B_KM, PP_BN, PP_BK, t, kk>(b_first));
        });
      }
    });
  };
  // Ends a reading turn: the fragments are in registers (their part of the stage may be refilled
  // once the barrier has passed) and at most `in_flight` of this wave's loads are outstanding.
  auto end_read_turn = [&](int in_flight) {
    __builtin_amdgcn_sched_barrier(0);
    wait_loads(in_flight);
    __builtin_amdgcn_s_waitcnt(lgkmcnt_zero());
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  auto end_product_turn = [&](int in_flight) {
    wait_loads(in_flight);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  auto products = [&](auto half_index) {
    constexpr int half = decltype(half_index)::value;
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int k = 0; k < FA_K; ++k)
#pragma unroll
      for (int t = 0; t < FA_T; ++t)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
          floatx16& c = acc[BY_ROWS ? 2 * half + t : t][tn];
          c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa[t][k]),
                                                      __builtin_bit_cast(bf16x8, fb[tn][k]), c, 0, 0, 0);
        }
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_sched_barrier(0);
  };
  const std::integral_constant<int, 0> H0{};
  const std::integral_constant<int, 1> H1{};
  // What may stay in flight at the barrier that ends S1(j) (part 1 of step j is read next: behind
  // it come both parts of step j + 1) and at the one that ends S3(j) (part 0 of step j + 1 is read
  // next: behind it come its part 1 and part 0 of step j + 2).
  auto after_s1 = [&](int j) { return j + 1 < steps ? N0 + N1 : 0; };
  auto after_s3 = [&](int j) { return (j + 1 < steps ? N1 : 0) + (j + 2 < steps ? N0 : 0); };

  // Both stages' first loads, then part 0 of step 0 published.
  issue_part(0, H0);
  issue_part(0, H1);
  if (steps > 1) {
    issue_part(1, H0);
    issue_part(1, H1);
  }
  wait_loads(N1 + (steps > 1 ? N0 + N1 : 0));
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);

  if (wm == 0) {
#pragma unroll 1
    for (int j = 0; j < steps; ++j) {
      const int stage = j & 1;
      // S0
      read_half(stage, H0);
      if (j >= 1 && j + 1 < steps) issue_part(stage ^ 1, H1);
      end_read_turn(NO_WAIT);
      // S1
      products(H0);
      end_product_turn(after_s1(j));
      // S2
      read_half(stage, H1);
      if (j + 2 < steps) issue_part(stage, H0);
      end_read_turn(NO_WAIT);
      // S3
      products(H1);
      end_product_turn(after_s3(j));
    }
  } else {
    __builtin_amdgcn_s_barrier();  // S0(0): nothing to multiply yet
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll 1
    for (int j = 0; j < steps; ++j) {
      const int stage = j & 1;
      // S1
      read_half(stage, H0);
      end_read_turn(after_s1(j));
      // S2
      if (j + 2 < steps) issue_part(stage, H0);
      products(H0);
      end_product_turn(NO_WAIT);
      // S3
      read_half(stage, H1);
      end_read_turn(after_s3(j));
      // S0(j + 1)
      if (j + 2 < steps) issue_part(stage, H1);
      products(H1);
      if (j + 1 < steps) end_product_turn(NO_WAIT);
    }
  }

  // Store pass: each wave stages 32 rows of its tile at a time through its own LDS region and
  // writes whole 4-column pieces. No workgroup barrier: group 0 gets here a turn before group 1,
  // whose last turn reads no LDS.
  constexpr int CPW = TN * 32 + 4;
  static_assert(NW * 32 * CPW * 4 <= PP_SMEM, "staging fits");
  float* cs = reinterpret_cast<float*>(smem) + wave * (32 * CPW);
  bool bad = false;
  static_for<0, TM>([&](auto tm_index) {
    constexpr int tm = decltype(tm_index)::value;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int v = 0; v < 16; ++v) cs[(8 * (v >> 2) + 4 * lg + (v & 3)) * CPW + tn * 32 + l32] = acc[tm][tn][v];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    constexpr int PPR = TN * 8;  // 4-column pieces per row
    const int grow0 = m0 + (wm * TM + tm) * 32, gcol0 = n0 + wn * TN * 32;
    const bool interior = grow0 + 32 <= g.M && gcol0 + TN * 32 <= g.N;
    bool stored = false;
    if constexpr (EPI == OMX_EPI_NONE) {
      if (interior && (g.splits > 1 ? (g.N & 3) == 0 : g.c_vec != 0)) {
        if (g.splits > 1) bad |= gemm_store_block<0, PPR>(g, split, cs, CPW, grow0, gcol0, lane);
        else if (g.c_bf16) bad |= gemm_store_block<1, PPR>(g, split, cs, CPW, grow0, gcol0, lane);
        else if (!g.accumulate) bad |= gemm_store_block<2, PPR>(g, split, cs, CPW, grow0, gcol0, lane);
        else bad |= gemm_store_block<3, PPR>(g, split, cs, CPW, grow0, gcol0, lane);
        stored = true;
      }
    } else if constexpr (EPI == OMX_EPI_AXPBY) {
      if (interior && g.c_vec != 0) {
        bad |= gemm_epilogue_block<OMX_EPI_AXPBY, false, PPR>(g, cs, CPW, grow0, gcol0, lane);
        stored = true;
      }
    } else {
      if (interior && g.c_vec != 0) {
        bad |= g.epi_tanh ? gemm_epilogue_block<EPI, true, PPR>(g, cs, CPW, grow0, gcol0, lane)
                          : gemm_epilogue_block<EPI, false, PPR>(g, cs, CPW, grow0, gcol0, lane);
        stored = true;
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

template <bool A_KM, bool B_KM>
int32_t launch_pp(omx_ctx* ctx, const GemmArgs& g) {
  auto kernel = g.epi == OMX_EPI_GELU_FWD   ? &gemm_pp_kernel<A_KM, B_KM, OMX_EPI_GELU_FWD>
                : g.epi == OMX_EPI_GELU_BWD ? &gemm_pp_kernel<A_KM, B_KM, OMX_EPI_GELU_BWD>
                : g.epi == OMX_EPI_AXPBY    ? &gemm_pp_kernel<A_KM, B_KM, OMX_EPI_AXPBY>
                                            : &gemm_pp_kernel<A_KM, B_KM, OMX_EPI_NONE>;
  OMX_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   PP_SMEM));
  omx_launch_timed(ctx, kernel, dim3(g.tiles_m * g.tiles_n * g.splits, g.batches), dim3(512), PP_SMEM, ctx->timing_start,
                   g.splits > 1 ? nullptr : ctx->timing_stop, g);
  OMX_LAUNCH_CHECK(ctx, "gemm_pp_kernel");
  return OMX_OK;
}

}  // namespace
