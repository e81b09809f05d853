// The bf16 GEMM with one wave per SIMD: a 256 x 256 output tile per workgroup, one workgroup per
// compute unit, four waves of 128 x 128 each (16 accumulator blocks of 32 x 32: 256 of the wave's
// 512 registers); with TN = 3 the tile is 256 x 192 and a wave's part 128 x 96 (768 output columns
// are four such tiles: 16384 rows then make 256 tiles, one per compute unit, where 256 x 256 tiles
// make 192). A wave interleaves its own LDS reads and global -> LDS loads between its own
// matrix products, in an order fixed in the source: per product a wave reads two thirds of the
// fragment bytes that eight waves of 128 x 64 read, and no other wave on the SIMD takes issue
// slots from the products.
//
//   K steps of 64 columns, two LDS stages per operand (A0 A1 B0 B1, 32 KiB each). A step is 64
//   products per wave in two halves of 32, and a stage is refilled in two parts, each as soon as
//   every wave has read it:
//     A k-contiguous (a load covers 8 rows x 64 columns): half 0 is the wave's row blocks 0-1 over
//       the step's four K slabs against all of B, half 1 its row blocks 2-3 against the same B
//       fragments, which stay in registers. Part 0 = B and the A rows of half 0 (12 loads per
//       wave), part 1 = the A rows of half 1 (4 loads).
//     A and B k-major (a load covers 2 K rows x 256 rows): half h is K slabs 2h, 2h + 1 of every
//       block; part h = K rows 32h .. 32h + 31 of both operands (8 loads per wave).
//   During half 1 of step j the wave reads part 0 of step j + 1, during half 0 part 1 of step j.
//   Two barriers per step: B0, after the first 8 products of half 0, says that every wave has read
//   part 0 of this step, and publishes part 1; part 0 of step j + 2 is loaded behind it. B1,
//   between the halves, says that part 1 has been read and publishes part 0 of step j + 1; part 1
//   of step j + 2 is loaded behind it. Every load has more than a step to land.
//   The K loop holds one copy of the step per stage and nothing else: the last steps skip their
//   loads by scalar branches, and the step count is even (K a multiple of 128, an even number of
//   steps per split). With further copies of the step, or a branch around the second one, the
//   compiler permutes the 256 accumulator registers between the copies through scratch memory.
#pragma once
#include "gemm_tiles.h"

namespace {

constexpr int W4_BM = 256, W4_BK = 64;  // the tile is 256 rows by 64 TN columns (TN = 4, or 3: 192 columns)
constexpr int W4_OPERAND = W4_BM * W4_BK * 2;  // one stage of one operand
constexpr int W4_SMEM = 4 * W4_OPERAND;
constexpr int W4_B0 = 2 * W4_OPERAND;  // LDS byte offset of B's first stage

// Loads of one operand: a wave-uniform base address (the tile's first element at the current K
// step) and a 32-bit byte offset per lane and load, so a K step advances one scalar.
// The chunk swizzle of a k-major tile row (kr) of ROWS columns: 16-byte chunks moved by multiples of 64 bytes so that
// the four K rows a transposing read touches per clock fall into different banks (rows of 512 bytes all start in
// bank 0: four shifts; rows of 384 bytes alternate between banks 0 and 32: one shift for every second pair).
template <int ROWS>
__device__ __forceinline__ int w4_km_swizzle(int kr) {
  return ROWS == 256 ? (kr & 3) * 4 : ((kr >> 1) & 1) * 4;
}

template <bool KM, int ROWS>
struct W4Loads {
  static constexpr int N = ROWS / 32;  // ROWS / 8 loads of 1 KiB per step, four waves
  unsigned off[N];
  const char* base;
  long step;
  __device__ __forceinline__ void init(const unsigned short* __restrict__ p, long ld, int row0, int rows, int k0,
                                       int wave, int lane) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int q = wave + 4 * i;
      if constexpr (!KM) {
        const int r = q * 8 + (lane >> 3);
        const int kc = (lane & 7) ^ ((r >> 1) & 7);
        int gr = row0 + r;
        gr = gr < rows ? gr : rows - 1;
        off[i] = static_cast<unsigned>(gr - row0) * static_cast<unsigned>(ld * 2) + kc * 16;
      } else {
        constexpr int CPR = ROWS / 8;  // 16-byte chunks per K row
        const int idx = q * 64 + lane;
        const int kr = idx / CPR, slot = idx % CPR;
        const int mc = slot ^ w4_km_swizzle<ROWS>(kr);
        int gm = mc * 8;
        gm = row0 + gm + 8 <= rows ? gm : 0;
        off[i] = static_cast<unsigned>(kr) * static_cast<unsigned>(ld * 2) + gm * 2;
      }
    }
    base = reinterpret_cast<const char*>(p) +
           (KM ? static_cast<long>(k0) * ld + row0 : static_cast<long>(row0) * ld + k0) * 2;
    step = (KM ? W4_BK * ld : W4_BK) * 2;
  }
  // Load I of this wave into LDS byte `lds_wave` + LDS_IMM.
  template <int I, int LDS_IMM>
  __device__ __forceinline__ void issue(unsigned lds_wave) const {
    asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off[I]), "s"(base),
                 "s"(lds_wave), "n"(LDS_IMM)
                 : "memory", "scc");
  }
};

// Fragment addresses of one operand tile of ROWS rows: four registers holding LDS byte addresses in stage 0; the
// block, the K slab and the stage are immediates of the read. `tile` is the tile's LDS address, `row_base` the first
// of the wave's rows in it.
template <bool KM, int ROWS>
struct W4Frags {
  unsigned b[4];
  __device__ __forceinline__ void init(unsigned tile, int row_base, int lane) {
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      if constexpr (!KM) {
        // [row][8 chunks of 16 bytes], chunk c of row r in slot c ^ ((r >> 1) & 7); x is the K slab.
        const int r = row_base + (lane & 31);
        const int kc = x * 2 + (lane >> 5);
        b[x] = tile + r * (W4_BK * 2) + ((kc ^ ((r >> 1) & 7)) << 4);
      } else {
        // [K row][ROWS / 8 chunks]; x is the 32-column block; the first of the two transposing reads.
        const int s16 = lane & 15, half = (lane >> 4) & 1, g = lane >> 5;
        const int kr = g * 8 + (s16 >> 2);
        const int col = row_base + x * 32 + half * 16 + (s16 & 3) * 4;
        b[x] = tile + kr * (ROWS * 2) + (((col >> 3) ^ w4_km_swizzle<ROWS>(kr)) << 4) + (col & 7) * 2;
      }
      // Held as it is: re-derived from its parts, a read would pay an addition for what the
      // instruction's offset field carries for nothing.
      asm volatile("" : "+v"(b[x]));
    }
  }
  template <int T, int KK, int STAGE>
  __device__ __forceinline__ u32x4 read() const {
    if constexpr (!KM) {
      typedef const u32x4 __attribute__((address_space(3))) * lds_ptr;
      return *reinterpret_cast<lds_ptr>(static_cast<uintptr_t>(b[KK] + (T * 32 * W4_BK * 2 + STAGE * W4_OPERAND)));
    } else {
      typedef short4v __attribute__((address_space(3))) * lds_ptr;
      const unsigned p = b[T] + (KK * 16 * ROWS * 2 + STAGE * W4_OPERAND);
      short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_ptr>(static_cast<uintptr_t>(p)));
      short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_ptr>(static_cast<uintptr_t>(p + 4 * ROWS * 2)));
      u32x2 x = __builtin_bit_cast(u32x2, lo), y = __builtin_bit_cast(u32x2, hi);
      return u32x4{x.x, x.y, y.x, y.y};
    }
  }
};

template <bool A_KM, bool B_KM, int TN>
__global__ __launch_bounds__(256, 1) void gemm_w4_kernel(GemmArgs g) {
  static_assert(!A_KM || B_KM, "a k-major A goes with a k-major B");
  static_assert(TN == 4 || TN == 3, "256 x 256 or 256 x 192 tiles");
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int TM = 4, NW = 4, W4_BN = TN * 64;
  // Tile order: as gemm_dma_kernel.
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
  // (the divisions above run on the vector unit: back to scalars, which the loads' bases need)
  const int m0 = __builtin_amdgcn_readfirstlane(tile_m * W4_BM), n0 = __builtin_amdgcn_readfirstlane(tile_n * W4_BN);
  product = __builtin_amdgcn_readfirstlane(product);
  split = __builtin_amdgcn_readfirstlane(split);
  gemm_select_batch(g, product);
  const unsigned short* __restrict__ A = static_cast<const unsigned short*>(g.a);
  const unsigned short* __restrict__ B = static_cast<const unsigned short*>(g.b);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave >> 1, wn = wave & 1;  // the wave's 128 rows and 32 TN columns of the tile
  const int l32 = lane & 31, lg = lane >> 5;

  floatx16 acc[TM][TN];
  // Cleared once the first loads are on their way (256 register writes).
  auto clear_acc = [&]() {
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
    __builtin_amdgcn_sched_barrier(0);
  };

  const int ks_begin = split * g.ksteps_per_split;
  const int ks_end = min(g.K / W4_BK, ks_begin + g.ksteps_per_split);
  const int steps = ks_end - ks_begin;
  W4Loads<A_KM, W4_BM> la;
  W4Loads<B_KM, W4_BN> lb;
  la.init(A, g.lda, m0, g.M, ks_begin * W4_BK, wave, lane);
  lb.init(B, g.ldb, n0, g.N, ks_begin * W4_BK, wave, lane);
  const unsigned lds_wave =
      __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<uintptr_t>(smem))) + wave * 1024;
  // Waits until at most YES (if `which`) or NO of this wave's loads, the most recently issued, are in flight.
  auto wait_loads = [&](bool which, auto yes_count, auto no_count) {
    if (which) __builtin_amdgcn_s_waitcnt(vmcnt_only(decltype(yes_count)::value));
    else __builtin_amdgcn_s_waitcnt(vmcnt_only(decltype(no_count)::value));
  };
  auto publish = [&](bool which, auto yes_count, auto no_count) {
    __builtin_amdgcn_sched_barrier(0);
    wait_loads(which, yes_count, no_count);
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt == 0: this wave's fragment reads have returned
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };

  // The products are taken with the operands exchanged: a lane then holds, for ONE output row (block
  // row l32), four consecutive columns per register quad (8 (v / 4) + 4 lg + v % 4), which the
  // store pass packs and stages 8 or 16 bytes at a time.
  auto product_of = [&](floatx16& c, const u32x4& a, const u32x4& b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, b), __builtin_bit_cast(bf16x8, a), c, 0, 0, 0);
  };
  const unsigned lds0 = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<uintptr_t>(smem)));
  const std::integral_constant<int, 0> S0{};
  const std::integral_constant<int, 1> S1{};
  if constexpr (!A_KM) {
    W4Frags<false, W4_BM> ra;
    W4Frags<B_KM, W4_BN> rb;
    ra.init(lds0, wm * 128, lane);
    rb.init(lds0 + W4_B0, wn * TN * 32, lane);

    // Part 0 of a stage: all of B (2 TN loads per wave) and A's loads 0, 1, 4, 5 (rows 0-63 and 128-191 of the
    // tile); part 1: A's loads 2, 3, 6, 7. `n` counts the part's loads.
    constexpr int NB = 2 * TN, NP0 = NB + 4, NSTEP = NP0 + 4;
    constexpr int SL = 2 * TN, HL = 4 * SL;  // products per K slab of a half, per half
    typedef std::integral_constant<int, 0> C0;
    typedef std::integral_constant<int, 4> C4;
    typedef std::integral_constant<int, NSTEP> CSTEP;
    typedef std::integral_constant<int, 4 + NP0> C4P0;
    auto issue_p0 = [&](auto stage_index, auto n_index) {
      constexpr int stage = decltype(stage_index)::value, n = decltype(n_index)::value;
      if constexpr (n < NB) {
        lb.template issue<n, W4_B0 + stage * W4_OPERAND + NW * n * 1024>(lds_wave);
      } else {
        constexpr int i = n == NB ? 0 : n == NB + 1 ? 1 : n == NB + 2 ? 4 : 5;
        la.template issue<i, stage * W4_OPERAND + NW * i * 1024>(lds_wave);
      }
    };
    auto issue_p1 = [&](auto stage_index, auto n_index) {
      constexpr int stage = decltype(stage_index)::value, n = decltype(n_index)::value;
      constexpr int i = n == 0 ? 2 : n == 1 ? 3 : n == 2 ? 6 : 7;
      la.template issue<i, stage * W4_OPERAND + NW * i * 1024>(lds_wave);
    };
    // fa0[t][k]: row blocks 0-1, fa1[t][k]: row blocks 2-3, fb[u][k]: column blocks, K slab k.
    u32x4 fa0[2][4], fa1[2][4], fb[TN][4];
    // Fragment n (0 .. TN + 1) of K slab k of part 0 of a stage: TN of B, two of A.
    auto read_p0 = [&](auto stage_index, auto k_index, auto n_index) {
      constexpr int stage = decltype(stage_index)::value, k = decltype(k_index)::value, n = decltype(n_index)::value;
      if constexpr (n < TN) fb[n][k] = rb.template read<n, k, stage>();
      else fa0[n - TN][k] = ra.template read<n - TN, k, stage>();
    };
    // Fragment n (0..7) of part 1 of a stage: K slab n / 2, row block 2 + n % 2.
    auto read_p1 = [&](auto stage_index, auto n_index) {
      constexpr int stage = decltype(stage_index)::value, n = decltype(n_index)::value;
      fa1[n % 2][n / 2] = ra.template read<2 + n % 2, n / 2, stage>();
    };
    // Both stages' loads, part 0 of step 0 published, its fragments read.
    static_for<0, NP0>([&](auto n_index) { issue_p0(S0, n_index); });
    static_for<0, 4>([&](auto n_index) { issue_p1(S0, n_index); });
    la.base += la.step;
    lb.base += lb.step;
    if (steps > 1) {
      static_for<0, NP0>([&](auto n_index) { issue_p0(S1, n_index); });
      static_for<0, 4>([&](auto n_index) { issue_p1(S1, n_index); });
      la.base += la.step;
      lb.base += lb.step;
    }
    clear_acc();
    wait_loads(steps > 1, std::integral_constant<int, 4 + NSTEP>{}, C4{});
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, 4>([&](auto k_index) {
      static_for<0, TN + 2>([&](auto n_index) { read_p0(S0, k_index, n_index); });
    });
    __builtin_amdgcn_sched_barrier(0);

    // One K step out of stage STAGE. `next`: another step follows; `loads`: two more follow (the
    // loads of the second start here). The fragment reads "of the next step" also run in the last
    // step, on stale data nobody uses. The K loop holds one copy of this per stage and nothing
    // else, so the accumulators stay where they are.
    // Part 0's load i goes out after product P0_AT(i) of half 0: spread over the products behind B0.
    auto step = [&](auto stage_index, bool next, bool loads) {
      constexpr int STAGE = decltype(stage_index)::value;
      const std::integral_constant<int, STAGE> HERE{};
      const std::integral_constant<int, STAGE ^ 1> THERE{};
      // Half 0.
      static_for<0, HL>([&](auto n_index) {
        constexpr int n = decltype(n_index)::value, k = n / SL, t = (n % SL) / TN, u = n % TN;
        product_of(acc[t][u], fa0[t][k], fb[u][k]);
        if constexpr (n == SL - 1) {
          // B0. In flight behind part 1 of this step: both parts of the next.
          publish(next, CSTEP{}, C0{});
        } else {
          if constexpr (n >= SL) {
            // load i after product SL + i (HL - SL) / NP0 (TN = 4: every second product)
            constexpr int lo = ((n - SL) * NP0 + (HL - SL) - 1) / (HL - SL);  // first i with its place >= n
            if constexpr (lo < NP0 && SL + lo * (HL - SL) / NP0 == n) {
              if (loads) issue_p0(HERE, std::integral_constant<int, lo>{});
            }
          }
          if constexpr (n > SL && n < SL + 17 && (n - SL) % 2 == 1) read_p1(HERE, std::integral_constant<int, (n - SL - 1) / 2>{});
          __builtin_amdgcn_sched_barrier(0);
        }
      });
      if (loads) lb.base += lb.step;
      // B1. In flight behind part 0 of the next step: its part 1 and part 0 of the one after.
      publish(loads, C4P0{}, C4{});
      // Half 1.
      static_for<0, HL>([&](auto n_index) {
        constexpr int n = decltype(n_index)::value, k = n / SL, t = (n % SL) / TN, u = n % TN;
        product_of(acc[2 + t][u], fa1[t][k], fb[u][k]);
        if constexpr (n < 8 && n % 2 == 0) {
          if (loads) issue_p1(HERE, std::integral_constant<int, n / 2>{});
        }
        // The next step's fragments of slab k - 1 go where this step's have just been used.
        if constexpr (n >= SL && n % SL < TN + 2)
          read_p0(THERE, std::integral_constant<int, n / SL - 1>{}, std::integral_constant<int, n % SL>{});
        __builtin_amdgcn_sched_barrier(0);
      });
      if (loads) la.base += la.step;
      static_for<0, TN + 2>([&](auto n_index) { read_p0(THERE, std::integral_constant<int, 3>{}, n_index); });
      __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll 1
    for (int j = 0; j < steps; j += 2) {  // the host keeps the step count even
      step(S0, true, j + 2 < steps);
      step(S1, j + 2 < steps, j + 3 < steps);
    }
  } else {
    W4Frags<true, W4_BM> ra;
    W4Frags<true, W4_BN> rb;
    ra.init(lds0, wm * 128, lane);
    rb.init(lds0 + W4_B0, wn * TN * 32, lane);
    // Part h of a stage: this wave's loads 4h .. 4h + 3 of A, then TN h .. TN h + TN - 1 of B.
    constexpr int NPART = 4 + TN, NF = 2 * NPART;  // loads per part and wave; fragments per half
    constexpr int SLAB = 4 * TN, HL = 2 * SLAB;   // products per K slab, per half
    typedef std::integral_constant<int, 0> C0;
    typedef std::integral_constant<int, NPART> C1P;
    typedef std::integral_constant<int, 2 * NPART> C2P;
    typedef std::integral_constant<int, 3 * NPART> C3P;
    auto issue_part = [&](auto stage_index, auto h_index, auto n_index) {
      constexpr int stage = decltype(stage_index)::value, h = decltype(h_index)::value, n = decltype(n_index)::value;
      if constexpr (n < 4) {
        constexpr int i = 4 * h + n;
        la.template issue<i, stage * W4_OPERAND + NW * i * 1024>(lds_wave);
      } else {
        constexpr int i = TN * h + (n - 4);
        lb.template issue<i, W4_B0 + stage * W4_OPERAND + NW * i * 1024>(lds_wave);
      }
    };
    // fa[h][t][s]: row block t, K slab 2h + s; fb[h][u][s] likewise.
    u32x4 fa[2][4][2], fb[2][TN][2];
    // Fragment n (0 .. NF - 1) of half h of a stage: eight of A, then 2 TN of B.
    auto read_half = [&](auto stage_index, auto h_index, auto n_index) {
      constexpr int stage = decltype(stage_index)::value, h = decltype(h_index)::value, n = decltype(n_index)::value;
      if constexpr (n < 8) fa[h][n / 2][n % 2] = ra.template read<n / 2, 2 * h + n % 2, stage>();
      else fb[h][(n - 8) / 2][n % 2] = rb.template read<(n - 8) / 2, 2 * h + n % 2, stage>();
    };
    const std::integral_constant<int, 0> H0{};
    const std::integral_constant<int, 1> H1{};

    static_for<0, NPART>([&](auto n_index) { issue_part(S0, H0, n_index); });
    static_for<0, NPART>([&](auto n_index) { issue_part(S0, H1, n_index); });
    la.base += la.step;
    lb.base += lb.step;
    if (steps > 1) {
      static_for<0, NPART>([&](auto n_index) { issue_part(S1, H0, n_index); });
      static_for<0, NPART>([&](auto n_index) { issue_part(S1, H1, n_index); });
      la.base += la.step;
      lb.base += lb.step;
    }
    clear_acc();
    wait_loads(steps > 1, C3P{}, C1P{});
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NF>([&](auto n_index) { read_half(S0, H0, n_index); });
    __builtin_amdgcn_sched_barrier(0);

    auto step = [&](auto stage_index, bool next, bool loads) {
      constexpr int STAGE = decltype(stage_index)::value;
      const std::integral_constant<int, STAGE> HERE{};
      const std::integral_constant<int, STAGE ^ 1> THERE{};
      // Half 0.
      static_for<0, HL>([&](auto n_index) {
        constexpr int n = decltype(n_index)::value, sl = n / SLAB, t = (n % SLAB) / TN, u = n % TN;
        product_of(acc[t][u], fa[0][t][sl], fb[0][u][sl]);
        if constexpr (n == 7) {
          // B0. In flight behind part 1 of this step: both parts of the next.
          publish(next, C2P{}, C0{});
        } else {
          if constexpr (n >= 8 && n < 8 + NF) {
            if constexpr (n % 2 == 0 && (n - 8) / 2 < NPART) {
              if (loads) issue_part(HERE, H0, std::integral_constant<int, (n - 8) / 2>{});
            }
            read_half(HERE, H1, std::integral_constant<int, n - 8>{});
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      });
      // B1. In flight behind part 0 of the next step: its part 1 and part 0 of the one after.
      publish(loads, C2P{}, C1P{});
      // Half 1.
      static_for<0, HL>([&](auto n_index) {
        constexpr int n = decltype(n_index)::value, sl = n / SLAB, t = (n % SLAB) / TN, u = n % TN;
        product_of(acc[t][u], fa[1][t][sl], fb[1][u][sl]);
        if constexpr (n < NF) {
          if constexpr (n % 2 == 0 && n / 2 < NPART) {
            if (loads) issue_part(HERE, H1, std::integral_constant<int, n / 2>{});
          }
          read_half(THERE, H0, n_index);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      if (loads) {
        la.base += la.step;
        lb.base += lb.step;
      }
      __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll 1
    for (int j = 0; j < steps; j += 2) {  // the host keeps the step count even
      step(S0, true, j + 2 < steps);
      step(S1, j + 2 < steps, j + 3 < steps);
    }
  }
  // Every wave has read its last fragments before the stages are reused for the store pass.
  __builtin_amdgcn_s_waitcnt(vmcnt_only(0) & 0xC07F);
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);

  // Store pass: each wave stages 32 rows of its tile at a time through its own LDS region and
  // writes whole pieces of rows.
  constexpr int CPW = TN * 32 + 4;
  static_assert(NW * 32 * CPW * 4 <= W4_SMEM, "staging fits");
  float* cs = reinterpret_cast<float*>(smem) + wave * (32 * CPW);
  bool bad = false;
  constexpr int PPR = TN * 8;  // 4-column pieces per row
  const int gcol0 = n0 + wn * TN * 32;
  const bool packed = g.splits == 1 && g.c_bf16 && g.c_vec != 0 && (g.ldc & 7) == 0 &&
                      (reinterpret_cast<uintptr_t>(g.c) & 15) == 0;
  constexpr int HP = TN * 32 * 2 + 16;  // bytes per staged bf16 row
  char* hs = reinterpret_cast<char*>(cs);
  unsigned flags = 0;  // bit 15 or 31 set: a stored bf16 has an all-ones exponent
  static_for<0, TM>([&](auto tm_index) {
    constexpr int tm = decltype(tm_index)::value;
    const int grow0 = m0 + (wm * TM + tm) * 32;
    const bool interior = grow0 + 32 <= g.M && gcol0 + TN * 32 <= g.N;
    if (packed && interior) {
      // bf16: rounded in registers, staged 8 bytes at a time, stored 16 bytes per lane (a wave
      // instruction writes four rows of 64 TN bytes; with TN = 3 four lanes in 16 sit out).
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const floatx16& c = acc[tm][tn];
          uint2 w;
          w.x = dev_pack_bf16_pair(c[4 * q], c[4 * q + 1]);
          w.y = dev_pack_bf16_pair(c[4 * q + 2], c[4 * q + 3]);
          flags |= ((w.x & 0x7F807F80u) + 0x00800080u) | ((w.y & 0x7F807F80u) + 0x00800080u);
          *reinterpret_cast<uint2*>(hs + l32 * HP + (tn * 32 + 8 * q + 4 * lg) * 2) = w;
        }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      unsigned short* crow = static_cast<unsigned short*>(g.c) + static_cast<long>(grow0 + (lane >> 4)) * g.ldc + gcol0 +
                             (lane & 15) * 8;
      const long four_rows = 4 * g.ldc;
      if ((lane & 15) < TN * 4) {
#pragma unroll
        for (int it = 0; it < 8; ++it) {
          const uint4 v = *reinterpret_cast<const uint4*>(hs + (it * 4 + (lane >> 4)) * HP + (lane & 15) * 16);
          *reinterpret_cast<uint4*>(crow + it * four_rows) = v;
        }
      }
    } else {
      // f32 results, split-K partials, ragged edges: staged as f32 rows.
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const floatx16& c = acc[tm][tn];
          *reinterpret_cast<float4*>(cs + l32 * CPW + tn * 32 + 8 * q + 4 * lg) =
              make_float4(c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3]);
        }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      if (interior && (g.splits > 1 ? (g.N & 3) == 0 : g.c_vec != 0)) {
        if (g.splits > 1) bad |= gemm_store_block<0, PPR>(g, split, cs, CPW, grow0, gcol0, lane);
        else if (g.c_bf16) bad |= gemm_store_block<1, PPR>(g, split, cs, CPW, grow0, gcol0, lane);
        else if (!g.accumulate) bad |= gemm_store_block<2, PPR>(g, split, cs, CPW, grow0, gcol0, lane);
        else bad |= gemm_store_block<3, PPR>(g, split, cs, CPW, grow0, gcol0, lane);
      } else {
#pragma unroll 1
        for (int c = lane; c < 32 * PPR; c += 64) {
          const int row = c / PPR, piece = c % PPR;
          const int grow = grow0 + row, gcol = gcol0 + piece * 4;
          if (grow < g.M && gcol < g.N) {
            const float4 val = *reinterpret_cast<const float4*>(cs + row * CPW + piece * 4);
            bad |= gemm_store4(g, split, grow, gcol, val.x, val.y, val.z, val.w);
          }
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  });
  bad |= (flags & 0x80008000u) != 0;
  if (bad) dev_raise_fault(g.fault, g.tag);
}

template <bool A_KM, bool B_KM, int TN>
int32_t launch_w4(omx_ctx* ctx, const GemmArgs& g) {
  auto kernel = &gemm_w4_kernel<A_KM, B_KM, TN>;
  OMX_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   W4_SMEM));
  omx_launch_timed(ctx, kernel, dim3(g.tiles_m * g.tiles_n * g.splits, g.batches), dim3(256), W4_SMEM, ctx->timing_start,
                   g.splits > 1 ? nullptr : ctx->timing_stop, g);
  OMX_LAUNCH_CHECK(ctx, "gemm_w4_kernel");
  return OMX_OK;
}

}  // namespace
