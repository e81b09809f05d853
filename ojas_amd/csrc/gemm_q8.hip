// Dequant-fused bf16 MFMA GEMM over a frozen weight stored as symmetric int8 codes in groups of
// 32 consecutive input columns with one f32 scale per group (value = code * scale; the
// reference's per-channel form ojas-cpu/src/quant_sparse.rs:284-346 applied per group).
//
//   forward        y[n, o]  = sum_k x[n, k]  * W[o, k]   (+ add[n, o])     ojas-model/src/lora.rs:332-344 `base`
//   input gradient gx[n, k] = sum_o gy[n, o] * W[o, k]   (+ add[n, k])
// The weight is frozen, so there is no weight gradient.
//
// Data movement, per workgroup (512 threads, tile 256 x 128, 32-column K steps):
//   * the activation operand goes global -> LDS directly, three stages, as in gemm_dma.hip;
//   * the codes never exist as bf16 in HBM: waves 0..3 each fetch 1 KiB of codes per step
//     (global -> LDS directly, 16 codes per lane) plus the lane's group scale, three steps ahead;
//     the wave that fetched them reads its own 16 bytes back, widens them
//     (fma(byte ^ 0x80, scale, -128 scale) is code * scale rounded once, then round-to-nearest-even
//     to bf16) and writes them into the swizzled bf16 tile the MFMA fragments are read from.
//     Fetch and widening stay inside one wave, so the only synchronisation they add is the
//     step's barrier, which already publishes the activation tile.
//   * 48 KiB activation stages + 16 KiB of widened weights (two buffers) + 15 KiB of raw codes and
//     scales = 79 KiB: two workgroups share a compute unit.
// HBM traffic per product: the activation once per column band, the codes once per row band at
// ONE byte per weight, the scales at one eighth of that.
#include "gemm_tiles.h"

typedef __bf16 bf16x2q __attribute__((ext_vector_type(2)));
typedef float floatx2q __attribute__((ext_vector_type(2)));

namespace {

struct Q8Args {
  const unsigned short* a;  // [M][K] bf16, K contiguous
  long lda;
  const signed char* codes;  // [nout][kin]
  const float* scales;       // [nout][kin / 32]
  long kin;
  unsigned short* c;  // [M][N] bf16, or f32 when c_f32 (the pointer is then a float*)
  long ldc;
  int c_f32;
  const unsigned short* add;  // optional [M][N] bf16 with C's pitch, added before the rounding
  int M, N, K;
  int tiles_m, tiles_n;
  int packed;  // the weight is in the blocked layout of omx_pack_i8_group
  // Optional low-rank term added in the accumulators: C[m, n] += sum_p lr_h[m][off + p] * lr_w[n][p],
  // p < lr_rank (a multiple of 16), off = (n / lr_block_cols) * lr_rank when lr_block_cols > 0.
  const unsigned short* lr_h;  // [M][lr_pitch] bf16
  const unsigned short* lr_w;  // [N][lr_w_pitch] bf16
  long lr_pitch, lr_w_pitch;
  int lr_rank, lr_block_cols;
  OmxFaultWord* fault;
  unsigned long long tag;
};

// Blocked weight layout (omx_pack_i8_group): the [n_out, k_in] codes are cut into blocks of 8 output
// rows x 4 groups (128 input columns), stored block after block in row-major block order; inside a
// block the group index runs slowest: [group % 4][row % 8][32 codes]. A forward step (32 rows, one
// group) then reads four runs of 256 contiguous bytes instead of 32 pieces of 32 bytes, and an
// input-gradient step (8 rows, 128 columns per load) reads whole 1 KiB blocks. The scales are
// blocked the same way, [group % 4][row % 8] floats per block.
__device__ __forceinline__ long q8_packed_code_offset(long row, long group, long kin) {
  return ((row >> 3) * (kin >> 7) + (group >> 2)) * 1024 + (group & 3) * 256 + (row & 7) * 32;
}
__device__ __forceinline__ long q8_packed_scale_index(long row, long group, long kin) {
  return ((row >> 3) * (kin >> 7) + (group >> 2)) * 32 + (group & 3) * 8 + (row & 7);
}

constexpr int QBM = 256, QBN = 128, QBK = 32, QNW = 8;
constexpr int Q_A_STAGE = QBM * QBK * 2;            // 16 KiB
constexpr int Q_B16 = QBN * QBK * 2;                // 8 KiB
constexpr int Q_OFF_B16 = 3 * Q_A_STAGE;            // two widened-weight buffers
constexpr int Q_OFF_RAW = Q_OFF_B16 + 2 * Q_B16;    // [3 slots][4 waves][1 KiB] codes
constexpr int Q_OFF_SCL = Q_OFF_RAW + 3 * 4 * 1024; // [3 slots][4 waves][256 B] scales
constexpr int Q_SMEM = Q_OFF_SCL + 3 * 4 * 256;     // 79 KiB

__device__ __forceinline__ unsigned int q8_pack2(float a, float b) {
  floatx2q f = {a, b};
  return __builtin_bit_cast(unsigned int, __builtin_convertvector(f, bf16x2q));
}

// Waits until at most `newer` of this wave's loads are outstanding (a wave-uniform count).
__device__ __forceinline__ void q8_wait_newer(int newer) {
  if (newer >= 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
  else if (newer == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
  else if (newer == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// B_KM false: forward (the weight tile is [out row][32 k], k contiguous in memory).
// B_KM true: input gradient (the weight tile is [32 reduction rows = out][128 columns = k]).
template <bool B_KM>
__global__ __launch_bounds__(512, 4) void gemm_q8_kernel(Q8Args g) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int TM = 2, TN = 2, WGN = 2, KK = QBK / 16;
  const int total = g.tiles_m * g.tiles_n;
  int id = blockIdx.x;
  // An XCD (workgroups go round-robin by index) takes a contiguous eighth of the tiles.
  if (total % 8 == 0) id = (id & 7) * (total >> 3) + (id >> 3);
  const int band = 4;
  const int tiles_per_band = band * g.tiles_n;
  const int band_id = id / tiles_per_band;
  const int first_m = band_id * band;
  const int band_rows = min(band, g.tiles_m - first_m);
  const int in_band = id - band_id * tiles_per_band;
  const int tile_m = first_m + in_band % band_rows;
  const int tile_n = in_band / band_rows;
  const int m0 = tile_m * QBM, n0 = tile_n * QBN;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WGN, wn = wave % WGN;
  const int l32 = lane & 31, lg = lane >> 5;
  const bool feeds_b = wave < 4;  // wave-uniform: this wave fetches and widens a quarter of the weight tile

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  const int steps = g.K / QBK;
  TileLoadsOff<false, QBM, QBK, QNW> la;  // a scalar base that advances by the step and fixed lane offsets
  la.init(g.a, g.lda, m0, g.M, 0, wave, lane);
  const unsigned lds0 = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<uintptr_t>(smem)));

  // This lane's 16 codes of a step, its scale, and where their 16 bf16 go in the widened tile. The
  // loads take a scalar base, which advances by the step, and a lane offset in bytes that never
  // changes (the host keeps the weight under 2 GiB), so no vector instruction forms an address in the K loop.
  unsigned code_off, scale_off;
  long code_step, scale_step;  // bytes
  int w_off0, w_off1;  // byte offsets of the two 16-byte chunks inside a widened buffer
  const long groups = g.kin / 32;
  if constexpr (!B_KM) {
    const int r = wave * 32 + (lane >> 1), h = lane & 1;  // tile row (output feature), half of its 32 codes
    int gr = n0 + r;
    gr = gr < g.N ? gr : g.N - 1;
    if (g.packed) {
      code_off = static_cast<unsigned>(q8_packed_code_offset(gr, 0, g.kin) + h * 16);
      scale_off = static_cast<unsigned>(q8_packed_scale_index(gr, 0, g.kin) * 4);
      code_step = 256;
      scale_step = 8 * 4;
    } else {
      code_off = static_cast<unsigned>(static_cast<long>(gr) * g.kin + h * 16);
      scale_off = static_cast<unsigned>(static_cast<long>(gr) * groups * 4);
      code_step = QBK;
      scale_step = 4;
    }
    const int x = (r >> 2) & 3;
    w_off0 = r * 64 + (((2 * h) ^ x) << 4);
    w_off1 = r * 64 + (((2 * h + 1) ^ x) << 4);
  } else {
    const int kr = wave * 8 + (lane >> 3), j = lane & 7;  // reduction row of the step, 16-column piece
    int gc = n0 + j * 16;
    gc = gc + 16 <= g.N ? gc : 0;
    if (g.packed) {
      code_off = static_cast<unsigned>(q8_packed_code_offset(kr, gc / 32, g.kin) + (j & 1) * 16);
      scale_off = static_cast<unsigned>(q8_packed_scale_index(kr, gc / 32, g.kin) * 4);
    } else {
      code_off = static_cast<unsigned>(static_cast<long>(kr) * g.kin + gc);
      scale_off = static_cast<unsigned>((static_cast<long>(kr) * groups + gc / 32) * 4);
    }
    code_step = QBK * g.kin;
    scale_step = QBK * groups * 4;
    const int x = (kr & 3) * 4;
    w_off0 = kr * 256 + (((2 * j) ^ x) << 4);
    w_off1 = kr * 256 + (((2 * j + 1) ^ x) << 4);
  }
  const unsigned raw_lds = lds0 + Q_OFF_RAW + wave * 1024;  // + slot * 4096
  const unsigned scl_lds = lds0 + Q_OFF_SCL + wave * 256;   // + slot * 1024
  const char* code_base = reinterpret_cast<const char*>(g.codes);
  const char* scale_base = reinterpret_cast<const char*>(g.scales);
  auto issue_raw = [&](int slot) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(code_off), "s"(code_base),
                 "s"(raw_lds + slot * 4096)
                 : "memory");
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(scale_off), "s"(scale_base),
                 "s"(scl_lds + slot * 1024)
                 : "memory");
    code_base += code_step;
    scale_base += scale_step;
  };
  // Reads this lane's own 16 codes and scale back from slot `slot` and writes 16 bf16 into `dst`.
  auto widen = [&](int slot, char* dst) {
    const u32x4 cw = *reinterpret_cast<const u32x4*>(smem + Q_OFF_RAW + slot * 4096 + wave * 1024 + lane * 16);
    const float sc = *reinterpret_cast<const float*>(smem + Q_OFF_SCL + slot * 1024 + wave * 256 + lane * 4);
    const float nb = -128.0f * sc;
    const unsigned int w[4] = {cw.x ^ 0x80808080u, cw.y ^ 0x80808080u, cw.z ^ 0x80808080u, cw.w ^ 0x80808080u};
    unsigned int o[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float f0 = __builtin_fmaf(static_cast<float>(w[i] & 0xffu), sc, nb);
      const float f1 = __builtin_fmaf(static_cast<float>((w[i] >> 8) & 0xffu), sc, nb);
      const float f2 = __builtin_fmaf(static_cast<float>((w[i] >> 16) & 0xffu), sc, nb);
      const float f3 = __builtin_fmaf(static_cast<float>(w[i] >> 24), sc, nb);
      o[2 * i] = q8_pack2(f0, f1);
      o[2 * i + 1] = q8_pack2(f2, f3);
    }
    *reinterpret_cast<u32x4*>(dst + w_off0) = u32x4{o[0], o[1], o[2], o[3]};
    *reinterpret_cast<u32x4*>(dst + w_off1) = u32x4{o[4], o[5], o[6], o[7]};
  };

  int a_off[TM][KK], b_off[TN][KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
    for (int t = 0; t < TM; ++t) a_off[t][kk] = frag_offset<false, QBM, QBK>((wm * TM + t) * 32, kk, lane);
#pragma unroll
    for (int t = 0; t < TN; ++t) b_off[t][kk] = Q_OFF_B16 + frag_offset<B_KM, QBN, QBK>((wn * TN + t) * 32, kk, lane);
  }

  // Issue order: raw(0), raw(1), raw(2), A(0), A(1); then per step raw(s + 3), A(s + 2). A wave's
  // loads complete in order, so the wait for A(s + 1) at the end of step s also covers raw(s + 2).
  const int raw_loads = feeds_b ? 2 : 0;
  if (feeds_b) {
#pragma unroll
    for (int i = 0; i < 3; ++i)
      if (i < steps) issue_raw(i);
  }
  la.issue(lds0, wave);
  if (steps > 1) la.issue(lds0 + Q_A_STAGE, wave);
  q8_wait_newer(steps > 1 ? 2 : 0);  // A(0) and every raw slot issued before it
  if (feeds_b) widen(0, smem + Q_OFF_B16);
  __syncthreads();

  // Two sets of fragment registers that take turns (an even number of slabs per step: slab 0 always finds its
  // fragments in set 0): no copies, no wait for the next slab's fragments before this slab's products are issued.
  static_assert(KK % 2 == 0, "the fragment sets alternate by slab");
  u32x4 af[2][TM], bf[2][TN];
  auto read_frags = [&](const char* a_stage, const char* b_buf, int kk, u32x4(&a)[TM], u32x4(&b)[TN]) {
#pragma unroll
    for (int t = 0; t < TM; ++t) a[t] = frag_at<false, QBM>(a_stage + a_off[t][kk]);
#pragma unroll
    for (int t = 0; t < TN; ++t) b[t] = frag_at<B_KM, QBN>(b_buf + b_off[t][kk]);
  };
  read_frags(smem, smem, 0, af[0], bf[0]);
  // Step ks reads activation stage sa = ks % 3 and widened buffer sb = ks % 2.
  auto k_step = [&](int ks, int sa, int sb, int raw_slot_next, int raw_slot_fill) {
    const char* a_stage = smem + sa * Q_A_STAGE;
    const char* a_next = smem + ((sa + 1) % 3) * Q_A_STAGE;
    const char* b_buf = smem + sb * Q_B16;
    char* b_next = smem + (sb ^ 1) * Q_B16;
    // The weights of step ks + 1 (landed: they were issued before A(ks), which the previous
    // step's wait covered) are widened into the buffer step ks - 1 read, released by its barrier.
    if (feeds_b && ks + 1 < steps) widen(raw_slot_next, b_next + Q_OFF_B16);
    int newer = 0;
    if (ks + 3 < steps) {
      if (feeds_b) issue_raw(raw_slot_fill);
      newer += raw_loads;
    }
    if (ks + 2 < steps) {
      la.issue(lds0 + ((sa + 2) % 3) * Q_A_STAGE, wave);
      newer += 2;
    }
    static_for<0, KK>([&](auto kk_index) {
      constexpr int kk = decltype(kk_index)::value, cur = kk % 2, nxt = cur ^ 1;
      if constexpr (kk + 1 < KK) {
        read_frags(a_stage, b_buf, kk + 1, af[nxt], bf[nxt]);
      } else {
        q8_wait_newer(newer);  // A(ks + 1) has landed (this wave's share, then everyone's)
        __syncthreads();
        if (ks + 1 < steps) read_frags(a_next, b_next, 0, af[nxt], bf[nxt]);
      }
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
  // Unrolled over the six (stage, buffer) combinations so every LDS address is a precomputed
  // offset plus a constant.
  for (int ks = 0; ks < steps;) {
    bool done = false;
    static_for<0, 6>([&](auto idx) {
      constexpr int i = decltype(idx)::value;
      if (done) return;
      // raw(j) lives in slot j % 3: step ks widens raw(ks + 1) and refills the slot of raw(ks).
      k_step(ks, i % 3, i % 2, (i + 1) % 3, i % 3);
      if (++ks >= steps) done = true;
    });
  }
  // The low-rank term: lr_rank / 16 more MFMA slabs whose fragments come straight from global
  // memory (16 bytes per lane and fragment; every load of the main loop has landed by now).
  if (g.lr_rank > 0) {
    const int h_off = g.lr_block_cols > 0 ? (n0 / g.lr_block_cols) * g.lr_rank : 0;
    for (int p = 0; p < g.lr_rank; p += 16) {
      u32x4 ta[TM], tb[TN];
#pragma unroll
      for (int t = 0; t < TM; ++t) {
        int row = m0 + (wm * TM + t) * 32 + l32;
        row = row < g.M ? row : g.M - 1;
        ta[t] = *reinterpret_cast<const u32x4*>(g.lr_h + static_cast<long>(row) * g.lr_pitch + h_off + p + lg * 8);
      }
#pragma unroll
      for (int t = 0; t < TN; ++t) {
        int col = n0 + (wn * TN + t) * 32 + l32;
        col = col < g.N ? col : g.N - 1;
        tb[t] = *reinterpret_cast<const u32x4*>(g.lr_w + static_cast<long>(col) * g.lr_w_pitch + p + lg * 8);
      }
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
          acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ta[tm]),
                                                                __builtin_bit_cast(bf16x8, tb[tn]), acc[tm][tn], 0, 0,
                                                                0);
    }
  }
  __syncthreads();  // the staging below reuses the stages

  // Epilogue: each wave stages 32 rows of its tile at a time through its own LDS region and
  // writes whole 4-column pieces as bf16.
  constexpr int CPW = TN * 32 + 4;
  static_assert(QNW * 32 * CPW * 4 <= Q_SMEM, "staging fits");
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
    constexpr int ITERS = 32 * PPR / 64;
    const int grow0 = m0 + (wm * TM + tm) * 32, gcol0 = n0 + wn * TN * 32;
    const bool interior = grow0 + 32 <= g.M && gcol0 + TN * 32 <= g.N;
    if (interior) {
      uint2 addv[ITERS];
      if (g.add) {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          const int c = lane + it * 64, row = c / PPR, piece = c % PPR;
          addv[it] = *reinterpret_cast<const uint2*>(g.add + static_cast<long>(grow0 + row) * g.ldc + gcol0 + piece * 4);
        }
      }
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int c = lane + it * 64, row = c / PPR, piece = c % PPR;
        float4 val = *reinterpret_cast<const float4*>(cs + row * CPW + piece * 4);
        if (g.add) {
          val.x += __uint_as_float(addv[it].x << 16);
          val.y += __uint_as_float(addv[it].x & 0xffff0000u);
          val.z += __uint_as_float(addv[it].y << 16);
          val.w += __uint_as_float(addv[it].y & 0xffff0000u);
        }
        bad |= !(dev_finite(val.x) && dev_finite(val.y) && dev_finite(val.z) && dev_finite(val.w));
        const long at = static_cast<long>(grow0 + row) * g.ldc + gcol0 + piece * 4;
        if (g.c_f32) *reinterpret_cast<float4*>(reinterpret_cast<float*>(g.c) + at) = val;
        else *reinterpret_cast<uint2*>(g.c + at) = make_uint2(q8_pack2(val.x, val.y), q8_pack2(val.z, val.w));
      }
    } else {
#pragma unroll 1
      for (int c = lane; c < 32 * PPR; c += 64) {
        const int row = c / PPR, piece = c % PPR;
        const int grow = grow0 + row, gcol = gcol0 + piece * 4;
        if (grow >= g.M) continue;
        for (int e = 0; e < 4 && gcol + e < g.N; ++e) {
          const long off = static_cast<long>(grow) * g.ldc + gcol + e;
          float v = cs[row * CPW + piece * 4 + e];
          if (g.add) v += dev_bf16_bits_to_f32(g.add[off]);
          bad |= !dev_finite(v);
          if (g.c_f32) reinterpret_cast<float*>(g.c)[off] = v;
          else g.c[off] = dev_f32_to_bf16_bits(v);
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  });
  if (bad) dev_raise_fault(g.fault, g.tag);
}

// One thread per 16 codes: row-major -> blocked (or back).
__global__ void q8_pack_kernel(const signed char* __restrict__ src, const float* __restrict__ src_scales,
                               signed char* __restrict__ dst, float* __restrict__ dst_scales, long nout, long kin,
                               int unpack) {
  const long pieces = nout * (kin / 16);
  const long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= pieces) return;
  const long row = i / (kin / 16), p = i % (kin / 16), group = p >> 1;
  const long rm = row * kin + p * 16, bl = q8_packed_code_offset(row, group, kin) + (p & 1) * 16;
  const uint4 v = *reinterpret_cast<const uint4*>(src + (unpack ? bl : rm));
  *reinterpret_cast<uint4*>(dst + (unpack ? rm : bl)) = v;
  if ((p & 1) == 0) {
    const long srm = row * (kin / 32) + group, sbl = q8_packed_scale_index(row, group, kin);
    dst_scales[unpack ? srm : sbl] = src_scales[unpack ? sbl : srm];
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <bool B_KM>
int32_t launch_q8(omx_ctx* ctx, const Q8Args& g, double flops) {
  auto kernel = &gemm_q8_kernel<B_KM>;
  OMX_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   Q_SMEM));
  omx_ctx::TimedLaunch timed{};
  int32_t rc = omx_timing_begin(ctx, flops, &timed);
  if (rc != OMX_OK) return rc;
  omx_launch_timed(ctx, kernel, dim3(g.tiles_m * g.tiles_n), dim3(512), Q_SMEM, ctx->timing_start, ctx->timing_stop, g);
  hipError_t err = hipGetLastError();
  omx_timing_end(ctx, err == hipSuccess, timed);
  if (err != hipSuccess) return omx_hip_fail(ctx, err, "gemm_q8_kernel");
  return OMX_OK;
}

int32_t check_q8(omx_ctx* ctx, const char* op, const void* act, const void* codes, const void* scales, const void* out,
                 const void* add, uint64_t rows, uint64_t kin, uint64_t nout, uint64_t group, int32_t dtype,
                 int32_t layout) {
  if (!act || !codes || !scales || !out) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (dtype != OMX_BF16) return omx_fail(ctx, OMX_DTYPE, "%s: activations must be bf16", op);
  if (rows == 0 || kin == 0 || nout == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (group != 32) return omx_fail(ctx, OMX_UNSUPPORTED, "%s: group size %llu (only 32)", op, (unsigned long long)group);
  if (kin % 32 != 0) return omx_fail(ctx, OMX_SHAPE, "%s: k_in %llu is not a multiple of the group", op, (unsigned long long)kin);
  if (layout != OMX_I8_ROW_MAJOR && layout != OMX_I8_BLOCKED)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: weight layout %d", op, layout);
  if (layout == OMX_I8_BLOCKED && (kin % 128 != 0 || nout % 8 != 0))
    return omx_fail(ctx, OMX_SHAPE, "%s: the blocked layout needs k_in %% 128 == 0 and n_out %% 8 == 0", op);
  if (rows > 0x7fffffffull || kin > 0x7fffffffull || nout > 0x7fffffffull)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: axis does not fit in i32", op);
  // The kernel's loads address a lane's bytes with 32 bits beside a 64-bit base.
  if (kin >= (1ull << 22) || nout * kin >= (1ull << 31))
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: a weight of 2 GiB or more, or k_in of 4 Mi or more", op);
  if (!aligned16(act) || !aligned16(codes) || !aligned16(out) || (add && !aligned16(add)) ||
      (reinterpret_cast<uintptr_t>(scales) & 3u))
    return omx_fail(ctx, OMX_SHAPE, "%s: operands must be 16-byte aligned", op);
  return OMX_OK;
}

// Validates and installs the optional low-rank term of an entry point (`cols`: the product's output columns).
int32_t set_low_rank(omx_ctx* ctx, const char* op, Q8Args* g, const omx_low_rank* lr, uint64_t cols) {
  g->lr_h = nullptr;
  g->lr_w = nullptr;
  g->lr_pitch = 0;
  g->lr_w_pitch = 0;
  g->lr_rank = 0;
  g->lr_block_cols = 0;
  if (!lr || lr->rank == 0) return OMX_OK;
  if (!lr->h || !lr->w) return omx_fail(ctx, OMX_PLACEMENT, "%s: low-rank term with a null pointer", op);
  if (lr->rank % 16 != 0 || lr->rank > 1024)
    return omx_fail(ctx, OMX_SHAPE, "%s: low-rank width %llu is not a multiple of 16 up to 1024", op,
                    (unsigned long long)lr->rank);
  if (lr->block_cols != 0 && (lr->block_cols % QBN != 0 || cols % lr->block_cols != 0))
    return omx_fail(ctx, OMX_SHAPE, "%s: low-rank column blocks of %llu do not tile %llu columns in steps of %d", op,
                    (unsigned long long)lr->block_cols, (unsigned long long)cols, QBN);
  const uint64_t blocks = lr->block_cols ? cols / lr->block_cols : 1;
  if (lr->h_pitch % 8 != 0 || lr->h_pitch < blocks * lr->rank || lr->w_pitch % 8 != 0 || lr->w_pitch < lr->rank ||
      !aligned16(lr->h) || !aligned16(lr->w))
    return omx_fail(ctx, OMX_SHAPE, "%s: low-rank operands must be 16-byte aligned with a pitch that holds them", op);
  g->lr_h = static_cast<const unsigned short*>(lr->h);
  g->lr_w = static_cast<const unsigned short*>(lr->w);
  g->lr_pitch = static_cast<long>(lr->h_pitch);
  g->lr_w_pitch = static_cast<long>(lr->w_pitch);
  g->lr_rank = static_cast<int>(lr->rank);
  g->lr_block_cols = static_cast<int>(lr->block_cols);
  return OMX_OK;
}

}  // namespace

extern "C" {

int32_t omx_linear_i8_group_forward(omx_ctx* ctx, const void* x, int32_t x_dtype, const void* codes_i8,
                                    const void* scales_f32, uint64_t group, int32_t layout, const void* add,
                                    const omx_low_rank* low_rank, void* y, int32_t y_dtype, uint64_t rows,
                                    uint64_t kin, uint64_t nout) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "linear_i8_group_forward";
  int32_t rc = check_q8(ctx, op, x, codes_i8, scales_f32, y, add, rows, kin, nout, group, x_dtype, layout);
  if (rc != OMX_OK) return rc;
  if (!omx_valid_float_dtype(y_dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: the output must be f32 or bf16", op);
  if (nout % 4 != 0) return omx_fail(ctx, OMX_SHAPE, "%s: n_out %llu is not a multiple of 4", op, (unsigned long long)nout);
  Q8Args g{};
  g.a = static_cast<const unsigned short*>(x);
  g.lda = static_cast<long>(kin);
  g.codes = static_cast<const signed char*>(codes_i8);
  g.scales = static_cast<const float*>(scales_f32);
  g.kin = static_cast<long>(kin);
  g.c = static_cast<unsigned short*>(y);
  g.c_f32 = y_dtype == OMX_F32;
  g.ldc = static_cast<long>(nout);
  g.add = static_cast<const unsigned short*>(add);
  g.M = static_cast<int>(rows);
  g.N = static_cast<int>(nout);
  g.K = static_cast<int>(kin);
  g.tiles_m = (g.M + QBM - 1) / QBM;
  g.tiles_n = (g.N + QBN - 1) / QBN;
  g.packed = layout == OMX_I8_BLOCKED;
  g.fault = ctx->fault;
  rc = set_low_rank(ctx, op, &g, low_rank, nout);
  if (rc != OMX_OK) return rc;
  g.tag = omx_tag(ctx, F_LINEAR_FORWARD);
  return launch_q8<false>(ctx, g, 2.0 * rows * kin * nout);
}

int32_t omx_linear_i8_group_backward_input(omx_ctx* ctx, const void* codes_i8, const void* scales_f32, uint64_t group,
                                           int32_t layout, const void* gy, int32_t gy_dtype, const void* add,
                                           const omx_low_rank* low_rank, void* gx, uint64_t rows, uint64_t kin,
                                           uint64_t nout) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "linear_i8_group_backward_input";
  int32_t rc = check_q8(ctx, op, gy, codes_i8, scales_f32, gx, add, rows, kin, nout, group, gy_dtype, layout);
  if (rc != OMX_OK) return rc;
  if (nout % 32 != 0)
    return omx_fail(ctx, OMX_SHAPE, "%s: n_out %llu is not a multiple of 32", op, (unsigned long long)nout);
  Q8Args g{};
  g.a = static_cast<const unsigned short*>(gy);
  g.lda = static_cast<long>(nout);
  g.codes = static_cast<const signed char*>(codes_i8);
  g.scales = static_cast<const float*>(scales_f32);
  g.kin = static_cast<long>(kin);
  g.c = static_cast<unsigned short*>(gx);
  g.ldc = static_cast<long>(kin);
  g.add = static_cast<const unsigned short*>(add);
  g.M = static_cast<int>(rows);
  g.N = static_cast<int>(kin);
  g.K = static_cast<int>(nout);
  g.tiles_m = (g.M + QBM - 1) / QBM;
  g.tiles_n = (g.N + QBN - 1) / QBN;
  g.packed = layout == OMX_I8_BLOCKED;
  g.fault = ctx->fault;
  rc = set_low_rank(ctx, op, &g, low_rank, kin);
  if (rc != OMX_OK) return rc;
  g.tag = omx_tag(ctx, F_LINEAR_BACKWARD);
  return launch_q8<true>(ctx, g, 2.0 * rows * kin * nout);
}

int32_t omx_pack_i8_group(omx_ctx* ctx, const void* codes_i8, const void* scales_f32, void* blocked_codes,
                          void* blocked_scales, uint64_t nout, uint64_t kin, uint64_t group, int32_t unpack) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "pack_i8_group";
  if (!codes_i8 || !scales_f32 || !blocked_codes || !blocked_scales)
    return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (group != 32) return omx_fail(ctx, OMX_UNSUPPORTED, "%s: group size %llu (only 32)", op, (unsigned long long)group);
  if (nout == 0 || kin == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (kin % 128 != 0 || nout % 8 != 0)
    return omx_fail(ctx, OMX_SHAPE, "%s: the blocked layout needs k_in %% 128 == 0 and n_out %% 8 == 0", op);
  if (!aligned16(codes_i8) || !aligned16(blocked_codes) || codes_i8 == blocked_codes || scales_f32 == blocked_scales)
    return omx_fail(ctx, OMX_SHAPE, "%s: codes must be 16-byte aligned and the copy out of place", op);
  const long pieces = static_cast<long>(nout) * static_cast<long>(kin / 16);
  // unpack: the first pair is the blocked form and the second receives the row-major one.
  const signed char* src = static_cast<const signed char*>(unpack ? blocked_codes : codes_i8);
  const float* src_s = static_cast<const float*>(unpack ? blocked_scales : scales_f32);
  signed char* dst = static_cast<signed char*>(unpack ? const_cast<void*>(codes_i8) : blocked_codes);
  float* dst_s = static_cast<float*>(unpack ? const_cast<void*>(scales_f32) : blocked_scales);
  hipLaunchKernelGGL(q8_pack_kernel, dim3(static_cast<unsigned>((pieces + 255) / 256)), dim3(256), 0, ctx->stream, src,
                     src_s, dst, dst_s, static_cast<long>(nout), static_cast<long>(kin), unpack);
  OMX_LAUNCH_CHECK(ctx, "q8_pack_kernel");
  return OMX_OK;
}

}  // extern "C"
