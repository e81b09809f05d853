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

// ---------------------------------------------------------------------------------------------
// Persistent form of the kernel above for unsplit products: a workgroup walks a list of tiles
// (workgroup w of G takes tiles w, w + G, ...) and the global -> LDS pipeline runs straight
// across tile boundaries: the loads of the next tile's first steps are issued during the current
// tile's last steps, so no tile after a workgroup's first pays the load latency up front. That
// needs an epilogue that leaves the LDS stages alone: the accumulators go to memory straight from
// registers. For bf16 outputs two neighbouring lanes (columns c, c + 1) swap one value each, so
// that every lane holds two consecutive columns of one row and stores them as one 4-byte word;
// no barrier is involved, a wave finishes its part of a tile on its own and moves on.
// Where a workgroup is in its list of tiles. Tiles are numbered within bands of `band_rows` tile
// rows (a band holds band_rows x tiles_n tiles, column-major inside the band, so the tiles that
// run side by side share a few row panels and column panels); bands follow each other through
// a product and products through a strided batch. Stepping to the workgroup's next tile is a few
// additions and compares: no division runs inside the K loop.
struct TileCursor {
  int band, product, in_band;
  __device__ __forceinline__ void advance(int stride, int band_tiles, int bands_per_product) {
    in_band += stride;
    while (in_band >= band_tiles) {
      in_band -= band_tiles;
      if (++band == bands_per_product) {
        band = 0;
        ++product;
      }
    }
  }
  __device__ __forceinline__ void coords(int band_rows, int bm, int bn, int* m0, int* n0) const {
    int row, col;
    if (band_rows == 4) {
      row = in_band & 3;
      col = in_band >> 2;
    } else if (band_rows == 2) {
      row = in_band & 1;
      col = in_band >> 1;
    } else if (band_rows == 3) {
      col = (in_band * 43691) >> 17;  // in_band / 3 for in_band < 2^16
      row = in_band - 3 * col;
    } else {
      row = 0;
      col = in_band;
    }
    *m0 = (band * band_rows + row) * bm;
    *n0 = col * bn;
  }
};

__device__ __forceinline__ unsigned int pack_bf16_pair(float a, float b) {
  return dev_pack_bf16_pair(a, b);
}
// The value lane ^ 1 holds in `x`.
__device__ __forceinline__ float from_neighbour(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, true));
}

// One 32 x 32 accumulator block that lies wholly inside the output (4-byte aligned words for bf16),
// rows grow0.., columns gcol0.., from registers to memory.
// Lane (j = lane % 32, lg = lane / 32) holds column j of rows 8 (v / 4) + 4 lg + v % 4.
// (Every register index is a compile-time constant: static_for, not a loop the unroller may decline.)
template <int EPI>
__device__ __forceinline__ bool store_block_direct(const GemmArgs& g, char* cbase, const unsigned short* aux_in,
                                                   unsigned short* aux_out, const floatx16& acc, int grow0, int gcol0,
                                                   int l32, int lg) {
  bool bad = false;
  if (g.c_bf16) {
    // Even lanes end up with (row r: columns j, j + 1), odd lanes with (row r + 1: columns j - 1, j).
    const bool odd = (l32 & 1) != 0;
    unsigned short* c16 = reinterpret_cast<unsigned short*>(cbase);
    // Element offset of this lane's first word: row grow0 + 4 lg + odd, column gcol0 + (j & ~1).
    const long first = static_cast<long>(grow0 + 4 * lg + (odd ? 1 : 0)) * g.ldc + gcol0 + (l32 & ~1);
    static_for<0, 8>([&](auto p_index) {
      constexpr int v = 2 * decltype(p_index)::value;  // registers v, v + 1: rows r, r + 1
      const float lo = acc[v], hi = acc[v + 1];
      const float got = from_neighbour(odd ? lo : hi);
      float x0 = odd ? got : lo, x1 = odd ? hi : got;
      const long off = first + static_cast<long>(8 * (v >> 2) + (v & 3)) * g.ldc;
      if constexpr (EPI == OMX_EPI_GELU_FWD) {
        const float u0 = dev_round_bf16(x0), u1 = dev_round_bf16(x1);
        const float a0 = g.epi_tanh ? dev_gelu_tanh_fast(u0) : dev_gelu_erf_fast(u0);
        const float a1 = g.epi_tanh ? dev_gelu_tanh_fast(u1) : dev_gelu_erf_fast(u1);
        bad |= !(dev_finite(a0) && dev_finite(a1));
        *reinterpret_cast<unsigned int*>(aux_out + off) = pack_bf16_pair(a0, a1);
      } else if constexpr (EPI == OMX_EPI_GELU_BWD) {
        const unsigned int w = *reinterpret_cast<const unsigned int*>(aux_in + off);
        const float u0 = __uint_as_float(w << 16), u1 = __uint_as_float(w & 0xffff0000u);
        x0 = dev_round_bf16(x0) * (g.epi_tanh ? dev_gelu_tanh_grad_fast(u0) : dev_gelu_erf_grad_fast(u0));
        x1 = dev_round_bf16(x1) * (g.epi_tanh ? dev_gelu_tanh_grad_fast(u1) : dev_gelu_erf_grad_fast(u1));
      } else if constexpr (EPI == OMX_EPI_AXPBY) {
        const unsigned int w = *reinterpret_cast<const unsigned int*>(aux_in + off);
        x0 = gemm_axpby(g, __uint_as_float(w << 16), x0);
        x1 = gemm_axpby(g, __uint_as_float(w & 0xffff0000u), x1);
      }
      bad |= !(dev_finite(x0) && dev_finite(x1));
      *reinterpret_cast<unsigned int*>(c16 + off) = pack_bf16_pair(x0, x1);
    });
    return bad;
  }
  float* c32 = reinterpret_cast<float*>(cbase);
  const long first = static_cast<long>(grow0 + 4 * lg) * g.ldc + gcol0 + l32;
  static_for<0, 16>([&](auto v_index) {
    constexpr int v = decltype(v_index)::value;
    const long off = first + static_cast<long>(8 * (v >> 2) + (v & 3)) * g.ldc;
    const float x = g.accumulate ? acc[v] + c32[off] : acc[v];
    bad |= !dev_finite(x);
    c32[off] = x;
  });
  return bad;
}

template <bool A_KM, bool B_KM, int WGM, int WGN, int TM, int TN, int DBK, int NST, int EPI>
__global__ __launch_bounds__(WGM* WGN * 64,
                             dma_waves_per_simd(WGM* WGN, (NST * 1024 + 256) * (WGM * TM + WGN * TN) * 32 * DBK * 2 / 1024)) void
gemm_dma_persistent_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32;
  constexpr int A_BYTES = BM * DBK * 2, B_BYTES = BN * DBK * 2, STAGE = A_BYTES + B_BYTES;
  constexpr int NW = WGM * WGN;
  constexpr int LPS = STAGE / 1024 / NW;
  constexpr int KK = DBK / 16;
  static_assert(STAGE % (1024 * NW) == 0 && NST == 3 && TM * TN <= 4, "the persistent form");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WGN, wn = wave % WGN;
  // g.band_rows divides tiles_m; the host also guarantees whole tiles and at least two K steps.
  const int band_rows = g.band_rows;
  const int band_tiles = band_rows * g.tiles_n, bands_per_product = g.tiles_m / band_rows;
  const int total = g.tiles_m * g.tiles_n * g.batches;
  const int G = gridDim.x;
  const int ksteps = g.K / DBK;
  const int my_tiles = (total - static_cast<int>(blockIdx.x) + G - 1) / G;
  const int total_steps = my_tiles * ksteps;  // the host keeps this within an int
  // Workgroups go to the 8 XCDs round-robin by index and each XCD has its own L2: an XCD takes a
  // contiguous eighth of the numbered tiles when they split evenly (G is then a multiple of 8).
  const bool by_xcd = (total & 7) == 0;
  const int first = by_xcd ? (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3) : blockIdx.x;
  const int stride = by_xcd ? G >> 3 : G;
  TileCursor load_at;
  load_at.product = first / (band_tiles * bands_per_product);
  {
    const int in_product = first - load_at.product * band_tiles * bands_per_product;
    load_at.band = in_product / band_tiles;
    load_at.in_band = in_product - load_at.band * band_tiles;
  }
  TileCursor store_at = load_at;

  const unsigned lds_wave = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<uintptr_t>(smem))) + wave * 1024;
  // One fragment offset per operand in registers; the others follow from it with one operation
  // each (see frag_from_first), which leaves the registers for the accumulators.
  const int a_first = frag_offset<A_KM, BM, DBK>(wm * TM * 32, 0, lane);
  // LDS layout: the NST stages of A, then the NST stages of B, so that every fragment address is one
  // of four registers (first offset of A and of B, each with and without the slab bit) plus an
  // immediate below 64 KiB.
  constexpr int B_REGION = NST * A_BYTES;
  const int b_first = B_REGION + frag_offset<B_KM, BN, DBK>(wn * TN * 32, 0, lane);
  TileLoadsScalarBase<A_KM, BM, DBK, NW> la;
  TileLoadsScalarBase<B_KM, BN, DBK, NW> lb;
  unsigned* park_a = reinterpret_cast<unsigned*>(smem + NST * STAGE);
  unsigned* park_b = park_a + decltype(la)::PARK_BYTES / 4;
  la.init_lanes(park_a, g.lda, wave, lane);
  lb.init_lanes(park_b, g.ldb, wave, lane);
  // Moving the load cursor to a tile is scalar work only.
  auto aim_loads = [&]() {
    int m0, n0;
    load_at.coords(band_rows, BM, BN, &m0, &n0);
    la.aim(static_cast<const char*>(g.a) + load_at.product * g.batch_a, g.lda, m0);
    lb.aim(static_cast<const char*>(g.b) + load_at.product * g.batch_b, g.ldb, n0);
  };
  auto issue_stage = [&](auto stage_index) {
    constexpr int stage = decltype(stage_index)::value;
    unsigned off_a[decltype(la)::N], off_b[decltype(lb)::N];
    la.fetch(park_a, off_a);
    lb.fetch(park_b, off_b);
    la.template issue<stage * A_BYTES>(off_a, lds_wave);
    lb.template issue<B_REGION + stage * B_BYTES>(off_b, lds_wave);
  };
  auto issue_stage_at = [&](int stage) {  // the stage as a run-time value
    unsigned off_a[decltype(la)::N], off_b[decltype(lb)::N];
    la.fetch(park_a, off_a);
    lb.fetch(park_b, off_b);
    la.template issue_at<0>(off_a, lds_wave, stage * A_BYTES);
    lb.template issue_at<B_REGION>(off_b, lds_wave, stage * B_BYTES);
  };
  // A wave's memory operations complete in the order issued, stores included, and one counter
  // covers them all. `after_stores` > 0: this wave's stores of the previous tile were issued after
  // the loads being waited for, so they may stay in flight as well (up to 32 store
  // instructions for a bf16 tile; more than that, or the counter's range, waits for some of them).
  const bool many_stores = !g.c_bf16 || EPI == OMX_EPI_GELU_FWD;
  int after_stores = 0;
  auto wait_loads = [&](bool newer_group) {
    if (after_stores > 0) {
      if (many_stores) __builtin_amdgcn_s_waitcnt(vmcnt_only(63));
      else if (newer_group) __builtin_amdgcn_s_waitcnt(vmcnt_only(LPS + 32));
      else __builtin_amdgcn_s_waitcnt(vmcnt_only(32));
    } else {
      if (newer_group) __builtin_amdgcn_s_waitcnt(vmcnt_only(LPS));
      else __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
    }
  };
  aim_loads();
  issue_stage(std::integral_constant<int, 0>{});
  if (ksteps == 1) {  // not reached: the host requires two steps; keeps the cursor logic below simple
    return;
  }
  issue_stage(std::integral_constant<int, 1>{});
  wait_loads(true);  // step 0 has landed
  __syncthreads();

  floatx16 acc[TM][TN];
  auto clear = [&]() {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
  };
  clear();
  u32x4 af[TM], bf[TN];
  auto read_frags = [&](int stage, auto kk_index, u32x4(&a)[TM], u32x4(&b)[TN]) {
    constexpr int kk = decltype(kk_index)::value;
    static_for<0, TM>([&](auto t) {
      a[t] = frag_at<A_KM, BM>(smem + stage * A_BYTES + frag_from_first<A_KM, BM, DBK, decltype(t)::value, kk>(a_first));
    });
    static_for<0, TN>([&](auto t) {
      b[t] = frag_at<B_KM, BN>(smem + stage * B_BYTES + frag_from_first<B_KM, BN, DBK, decltype(t)::value, kk>(b_first));
    });
  };
  read_frags(0, std::integral_constant<int, 0>{}, af, bf);
  int gs = 0;  // steps multiplied so far, over all of this workgroup's tiles
  bool preissued = false;  // the loads the tile's first step would issue are already on their way
  // One K step of the tile at hand, multiplied out of stage S: first the loads of the step two
  // ahead (the next tile's, from the tile's last two steps on) into the stage step gs - 1 left.
  auto k_step = [&](auto stage_index, int ks) {
    constexpr int S = decltype(stage_index)::value;
    constexpr int stage = S, next = (S + 1) % NST;
    const bool more = gs + 2 < total_steps;
    if (more && !(ks == 0 && preissued)) {
      if (ks + 2 == ksteps) {
        load_at.advance(stride, band_tiles, bands_per_product);
        aim_loads();
      }
      issue_stage(std::integral_constant<int, (S + NST - 1) % NST>{});
    }
    static_for<0, KK>([&](auto kk_index) {
      constexpr int kk = decltype(kk_index)::value;
      u32x4 an[TM], bn[TN];
#pragma unroll
      for (int t = 0; t < TM; ++t) an[t] = af[t];
#pragma unroll
      for (int t = 0; t < TN; ++t) bn[t] = bf[t];
      if constexpr (kk + 1 < KK) {
        read_frags(stage, std::integral_constant<int, kk + 1>{}, an, bn);
      } else {
        // Step gs + 1 must have landed; the step issued above may still be in flight.
        wait_loads(more);
        __syncthreads();
        if (gs + 1 < total_steps) read_frags(next, std::integral_constant<int, 0>{}, an, bn);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
          acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, af[tm]),
                                                                __builtin_bit_cast(bf16x8, bf[tn]), acc[tm][tn], 0, 0,
                                                                0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < TM; ++t) af[t] = an[t];
#pragma unroll
      for (int t = 0; t < TN; ++t) bf[t] = bn[t];
    });
    ++gs;
    after_stores -= after_stores > 0;
  };
  int st = 0;  // the stage the tile's first step lives in: the stages keep rotating across tiles
  // One tile's steps, unrolled over the stages from a compile-time starting stage, so every LDS
  // address is a precomputed offset plus a constant.
  auto run_tile = [&](auto first_stage) {
    constexpr int S0 = decltype(first_stage)::value;
    for (int ks = 0; ks < ksteps;) {
      bool done = false;
      static_for<0, NST>([&](auto i_index) {
        if (done) return;
        k_step(std::integral_constant<int, (S0 + decltype(i_index)::value) % NST>{}, ks);
        if (++ks >= ksteps) done = true;
      });
    }
  };
  while (gs < total_steps) {
    // The accumulators are zero here and stored before the next pass: nothing but the prefetched
    // fragments crosses the three copies of the step loop.
    if (st == 0) run_tile(std::integral_constant<int, 0>{});
    else if (st == 1) run_tile(std::integral_constant<int, 1>{});
    else run_tile(std::integral_constant<int, 2>{});
    st = (st + ksteps) % NST;
    // The loads the next tile's first step would issue go out ahead of this tile's stores, so
    // that the next two steps can wait for their loads without waiting for the stores.
    preissued = false;
    if (gs + 2 < total_steps) {
      if (2 == ksteps) {
        load_at.advance(stride, band_tiles, bands_per_product);
        aim_loads();
      }
      issue_stage_at((st + NST - 1) % NST);
      preissued = true;
    }
    int m0, n0;
    store_at.coords(band_rows, BM, BN, &m0, &n0);
    char* cbase = static_cast<char*>(g.c) + store_at.product * g.batch_c;
    // aux tensors are bf16 like the output they accompany: the same byte stride between products.
    const unsigned short* aux_in = g.aux_in;
    unsigned short* aux_out = g.aux_out;
    if (aux_in) aux_in = reinterpret_cast<const unsigned short*>(reinterpret_cast<const char*>(aux_in) + store_at.product * g.batch_c);
    if (aux_out) aux_out = reinterpret_cast<unsigned short*>(reinterpret_cast<char*>(aux_out) + store_at.product * g.batch_c);
    bool bad = false;
    static_for<0, TM>([&](auto tm_index) {
      constexpr int tm = decltype(tm_index)::value;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
        bad |= store_block_direct<EPI>(g, cbase, aux_in, aux_out, acc[tm][tn], m0 + (wm * TM + tm) * 32,
                                       n0 + (wn * TN + tn) * 32, threadIdx.x & 31, (threadIdx.x >> 5) & 1);
    });
    if (bad) dev_raise_fault(g.fault, g.tag);
    clear();
    after_stores = 2;
    store_at.advance(stride, band_tiles, bands_per_product);
  }
}

// The persistent form pays for its longer code and parked offsets from 64 K steps on (K >= 2048).
constexpr int kPersistentMinSteps = 64;

template <bool A_KM, bool B_KM, int WGM, int WGN, int TM, int TN, int DBK, int NST>
int32_t launch_dma(omx_ctx* ctx, const GemmArgs& g) {
  constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32;
  constexpr int smem = NST * (BM + BN) * DBK * 2;
  if constexpr (NST == 3 && TM * TN <= 4 && ((BM + BN) * DBK * 2) % (1024 * WGM * WGN) == 0) {
    // Tiles wholly inside both operands (the persistent form never clamps a row).
    const long tiles_all = static_cast<long>(g.tiles_m) * g.tiles_n * g.batches;
    if (g.splits == 1 && g.M % BM == 0 && g.N % BN == 0 && g.K / DBK >= kPersistentMinSteps &&
        (!g.c_bf16 || g.c_vec) &&
        g.tiles_n * 4 < 65536 && tiles_all * (g.K / DBK) < (1l << 30)) {
      GemmArgs gp = g;
      gp.band_rows = g.tiles_m % 4 == 0 ? 4 : g.tiles_m % 3 == 0 ? 3 : g.tiles_m % 2 == 0 ? 2 : 1;
      auto pk = g.epi == OMX_EPI_GELU_FWD   ? &gemm_dma_persistent_kernel<A_KM, B_KM, WGM, WGN, TM, TN, DBK, NST, OMX_EPI_GELU_FWD>
                : g.epi == OMX_EPI_GELU_BWD ? &gemm_dma_persistent_kernel<A_KM, B_KM, WGM, WGN, TM, TN, DBK, NST, OMX_EPI_GELU_BWD>
                : g.epi == OMX_EPI_AXPBY    ? &gemm_dma_persistent_kernel<A_KM, B_KM, WGM, WGN, TM, TN, DBK, NST, OMX_EPI_AXPBY>
                                            : &gemm_dma_persistent_kernel<A_KM, B_KM, WGM, WGN, TM, TN, DBK, NST, OMX_EPI_NONE>;
      // The stages, then the parked load offsets: one word per thread and load.
      constexpr int psmem = smem + (BM + BN) * DBK * 2 / 1024 * 64 * 4;
      OMX_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void*>(pk), hipFuncAttributeMaxDynamicSharedMemorySize, psmem));
      // As many workgroups as fit the chip at once (LDS-limited), a multiple of the 8 XCDs.
      const int per_cu = 160 * 1024 / psmem < 16 / (WGM * WGN) ? 160 * 1024 / psmem : 16 / (WGM * WGN);
      const long slots = static_cast<long>(ctx->cu_count > 0 ? ctx->cu_count : 256) * per_cu;
      const long total = static_cast<long>(g.tiles_m) * g.tiles_n * g.batches;
      const unsigned grid = static_cast<unsigned>(total < slots ? total : slots);
      omx_launch_timed(ctx, pk, dim3(grid), dim3(WGM * WGN * 64), psmem, ctx->timing_start, ctx->timing_stop, gp);
      OMX_LAUNCH_CHECK(ctx, "gemm_dma_persistent_kernel");
      return OMX_OK;
    }
  }
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
