// bf16 MFMA flash attention for head_dim 64 and 128: causal forward, and the backward
// as two passes (dK/dV per key block, dQ per query block) that recompute the
// probabilities from the saved log-sum-exp, so no T x T matrix exists and no
// atomics are needed (the sums of one output never leave one wavefront).
//
// Reference semantics: ojas-cpu/src/attn.rs:176-227 (forward rows), :519-597
// (backward from saved output and lse); the blocked CPU kernel
// ojas-cpu/src/attn/flash.rs:1-41 is the Fast-tier precedent for this shape of
// algorithm (online softmax, delta = sum P dP).
//
// Mapping onto v_mfma_f32_32x32x16_bf16 (A: lane (i = l%32, g = l/32) holds
// A[i][8g..8g+7]; B: lane (j, g) holds B[8g..8g+7][j]; D: lane (j, g), register
// v holds D[8(v/4) + 4g + v%4][j]):
//   * scores are formed transposed, S^T = K . Q^T (forward, dQ pass), or plain,
//     S = Q . K^T (dK/dV pass), so that the index a softmax statistic belongs to
//     (the query in the first case, nothing per-lane in the second) is the
//     lane's column and every row reduction stays inside a lane plus one
//     exchange with lane l^32;
//   * an accumulator tile is reused directly as the B operand of the next
//     product (P^T for O^T = V^T P^T, P / dS for dV^T, dK^T, dS^T for dQ^T):
//     registers 8c..8c+7 of a lane are k-slab c, holding rows
//     16c + {4g..4g+3, 8+4g..8+4g+3}; the A operand stored transposed in LDS
//     keeps its k index in the matching order (bits 2 and 3 of the index
//     swapped), so one 16-byte LDS read fetches exactly those rows.
#include "omx_common.h"
#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

namespace {

// Head dims 64 and 128 (template argument D of everything below).
constexpr int fpitch(int D) { return D * 2 + 16; }      // bytes per LDS row: D bf16 + 16 pad
constexpr int ftile(int D) { return 64 * fpitch(D); }   // a 64-row tile
constexpr int FT = 256;                                 // threads per block (4 waves of 32 rows)
constexpr float LOG2E = 1.4426950408889634f;

// Element strides of one tensor: between rows (time steps), heads and batches.
struct FlashStrides {
  long rs, hs, bs;
};
struct FlashShape {
  int batch, heads, kv_heads, time, window, rep;
  // One 128-row block per workgroup instead of a mirrored pair, heaviest blocks first (query side:
  // forward and dQ; key side: dK/dV). Chosen by the host when the pairs would leave workgroup
  // places empty (few planes) or, on the key side, need a half-empty second round.
  int q_single, kv_single;
  float scale;
  FlashStrides q, kv, o;  // q and grad_q; k, v and their gradients; out and grad_out
};


__device__ __forceinline__ unsigned int pack2(float a, float b) {
  floatx2 f = {a, b};
  return __builtin_bit_cast(unsigned int, __builtin_convertvector(f, bf16x2));
}
__device__ __forceinline__ u32x4 pack8(const floatx16& acc, int c) {
  u32x4 r;
  r.x = pack2(acc[8 * c + 0], acc[8 * c + 1]);
  r.y = pack2(acc[8 * c + 2], acc[8 * c + 3]);
  r.z = pack2(acc[8 * c + 4], acc[8 * c + 5]);
  r.w = pack2(acc[8 * c + 6], acc[8 * c + 7]);
  return r;
}
// acc + both bf16 halves of w (v_dot2c_f32_bf16 against a pair of ones).
__device__ __forceinline__ float sum_pairs(unsigned int w, float acc) {
  typedef __bf16 bf16_pair __attribute__((ext_vector_type(2)));
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16_pair, w), __builtin_bit_cast(bf16_pair, 0x3F803F80u),
                                         acc, false);
}
// acc + the products of the two bf16 halves of a and b (v_dot2c_f32_bf16; a product of two bf16
// values is exact in f32).
__device__ __forceinline__ float dot_pairs(unsigned int a, unsigned int b, float acc) {
  typedef __bf16 bf16_pair __attribute__((ext_vector_type(2)));
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16_pair, a), __builtin_bit_cast(bf16_pair, b), acc, false);
}
__device__ __forceinline__ floatx16 mfma(const u32x4& a, const u32x4& b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                 0, 0);
}
// max(a, b, c) in one instruction. fmaxf first quiets each accumulator value (a v_max_f32 of the
// value with itself) because the compiler cannot know an MFMA result is canonical; this does not.
// NaNs are skipped, as by fmaxf.
__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ floatx16 zero16() {
  floatx16 z;
#pragma unroll
  for (int v = 0; v < 16; ++v) z[v] = 0.0f;
  return z;
}

// A 64-row x D-column bf16 tile starting at row `row0` of a [time, D] plane: D / 32 16-byte
// chunks per thread. Thread t moves chunk t % (D/8) of rows t / (D/8) + i * (2048 / D); rows at or
// past `time` read as zeros.
template <int D>
__device__ __forceinline__ void tile_load(const unsigned short* __restrict__ plane, long rs, int row0, int time,
                                          u32x4 (&r)[D / 32]) {
  constexpr int CPR = D / 8, RPP = FT / CPR;
  const int t = threadIdx.x;
  const int row = row0 + t / CPR, kc = t % CPR;
#pragma unroll
  for (int i = 0; i < D / 32; ++i) {
    r[i] = u32x4{0u, 0u, 0u, 0u};
    if (row + i * RPP < time)
      r[i] = *reinterpret_cast<const u32x4*>(plane + static_cast<long>(row + i * RPP) * rs + kc * 8);
  }
}
// [row][d] form.
template <int D>
__device__ __forceinline__ void tile_store_rows(char* lds, const u32x4 (&r)[D / 32]) {
  constexpr int CPR = D / 8, RPP = FT / CPR;
  const int t = threadIdx.x;
  const int row = t / CPR, kc = t % CPR;
#pragma unroll
  for (int i = 0; i < D / 32; ++i) *reinterpret_cast<u32x4*>(lds + (row + i * RPP) * fpitch(D) + kc * 16) = r[i];
}
// The same loads with the per-thread part of the address formed once. A tile that ends inside the
// sequence is fetched from a wave-uniform base (plane + row0 rows) plus the thread's fixed 32-bit byte
// offset: no address arithmetic and no bounds test per load. Only the last, ragged tile takes the
// checked path. The host refuses row strides for which the offset would not fit.
template <int D>
struct TileFetch {
  static constexpr int CPR = D / 8, RPP = FT / CPR;
  unsigned off;  // bytes from a tile's first element to this thread's first chunk
  long rs;
  int time;
  __device__ __forceinline__ TileFetch(long row_stride, int t_end) : rs(row_stride), time(t_end) {
    const int t = threadIdx.x;
    off = static_cast<unsigned>((t / CPR) * row_stride + (t % CPR) * 8) * 2u;
  }
  __device__ __forceinline__ void load(const unsigned short* __restrict__ plane, int row0, u32x4 (&r)[D / 32]) const {
    if (row0 + 64 <= time) {
      const char* base = reinterpret_cast<const char*>(plane + static_cast<long>(row0) * rs);
#pragma unroll
      for (int i = 0; i < D / 32; ++i) r[i] = *reinterpret_cast<const u32x4*>(base + static_cast<long>(i * RPP) * rs * 2 + off);
    } else {
      tile_load<D>(plane, rs, row0, time, r);
    }
  }
};
constexpr long FLASH_MAX_ROW_STRIDE = 1L << 24;  // elements: 31 rows of it, in bytes, stay below 2^32

// The wave's index as a scalar, so that what depends on it (which tiles the wave takes, which of
// them the diagonal cuts) is decided by scalar branches.
__device__ __forceinline__ int wave_index() { return __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6)); }

// x combined with the value lane ^ 32 holds: v_permlane32_swap exchanges the upper half of one
// register with the lower half of another, so swapping x with a copy of itself leaves (x of the lower
// lane, x of the upper lane) in the register pair of both lanes. One VALU instruction, no LDS round trip.
__device__ __forceinline__ float halves_max(float x) {
  const unsigned int u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  float m;
  asm("v_max_f32 %0, %1, %2" : "=v"(m) : "v"(__uint_as_float(r[0])), "v"(__uint_as_float(r[1])));
  return m;
}
__device__ __forceinline__ float halves_sum(float x) {
  const unsigned int u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// A operand from a [row][d] tile: rows sub*32 + lane%32, d-slab kk.
template <int D>
__device__ __forceinline__ u32x4 frag_rows(const char* lds, int sub, int kk, int l32, int lg) {
  return *reinterpret_cast<const u32x4*>(lds + (sub * 32 + l32) * fpitch(D) + kk * 32 + lg * 16);
}
// A operand of a product whose K index is the tile's ROW (O^T = V^T P^T, dV^T = dO^T P,
// dK^T = Q^T dS, dQ^T = K^T dS^T), read straight from the [row][d] tile with the transposing LDS
// read: a 16-lane group fetches a 4-row x 16-column block (8 bytes per lane) and each lane gets
// one column's 4 rows. Lane (i = lane % 32, g = lane / 32) ends up with column d = mt*32 + i and
// rows sub*32 + 16c + {4g..4g+3, 8+4g..8+4g+3}: the order in which an accumulator tile, reused as
// the B operand, holds its rows.
typedef short short4v __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
template <int D>
__device__ __forceinline__ u32x4 frag_tr(const char* lds, int mt, int sub, int c, int lane) {
  constexpr int FPITCH = fpitch(D);
  const int s = lane & 15, half = (lane >> 4) & 1, g = lane >> 5;
  const char* p = lds + (sub * 32 + c * 16 + 4 * g + (s >> 2)) * FPITCH + (mt * 32 + half * 16 + (s & 3) * 4) * 2;
  typedef short4v __attribute__((address_space(3))) * lds_ptr;
  const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
  const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 8 * FPITCH));
  const u32x2 a = __builtin_bit_cast(u32x2, lo), b = __builtin_bit_cast(u32x2, hi);
  return u32x4{a.x, a.y, b.x, b.y};
}
// B operand held in registers: the lane's own row of a [time, D] plane.
template <int D>
__device__ __forceinline__ void row_frags(const unsigned short* __restrict__ plane, long rs, int row, int time, int lg,
                                          u32x4 (&f)[D / 16]) {
#pragma unroll
  for (int kk = 0; kk < D / 16; ++kk) {
    f[kk] = u32x4{0u, 0u, 0u, 0u};
    if (row < time) f[kk] = *reinterpret_cast<const u32x4*>(plane + static_cast<long>(row) * rs + kk * 16 + lg * 8);
  }
}
// Row index (within a 32-row sub-tile) that accumulator register v of this lane holds.
__device__ __forceinline__ int acc_row(int v, int lg) { return 8 * (v >> 2) + 4 * lg + (v & 3); }

// Stores transposed accumulators (d x rows) as rows of a [time, D] plane.
template <int D, typename TO>
__device__ __forceinline__ bool store_transposed_acc(TO* __restrict__ plane, long rs, int row, int time, int lg,
                                                     const floatx16 (&acc)[D / 32], float mul) {
  bool bad = false;
  if (row >= time) return false;
#pragma unroll
  for (int mt = 0; mt < D / 32; ++mt)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const int d = mt * 32 + 8 * q4 + 4 * lg;
      float x0 = acc[mt][4 * q4 + 0] * mul, x1 = acc[mt][4 * q4 + 1] * mul, x2 = acc[mt][4 * q4 + 2] * mul,
            x3 = acc[mt][4 * q4 + 3] * mul;
      bad |= !(dev_finite(x0) && dev_finite(x1) && dev_finite(x2) && dev_finite(x3));
      if constexpr (sizeof(TO) == 2) {
        uint2 w;
        w.x = pack2(x0, x1);
        w.y = pack2(x2, x3);
        *reinterpret_cast<uint2*>(plane + static_cast<long>(row) * rs + d) = w;
      } else {
        *reinterpret_cast<float4*>(plane + static_cast<long>(row) * rs + d) = make_float4(x0, x1, x2, x3);
      }
    }
  return bad;
}

// The bf16 store of the output together with what the rounding dropped: residual = x - bf16(x),
// itself rounded to bf16, so that bf16(x) + residual carries 16 bits of x's mantissa.
template <int D>
__device__ __forceinline__ bool store_transposed_acc_split(unsigned short* __restrict__ plane,
                                                           unsigned short* __restrict__ resid, long rs, int row,
                                                           int time, int lg, const floatx16 (&acc)[D / 32], float mul) {
  bool bad = false;
  if (row >= time) return false;
#pragma unroll
  for (int mt = 0; mt < D / 32; ++mt)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const int d = mt * 32 + 8 * q4 + 4 * lg;
      const float x0 = acc[mt][4 * q4 + 0] * mul, x1 = acc[mt][4 * q4 + 1] * mul, x2 = acc[mt][4 * q4 + 2] * mul,
                  x3 = acc[mt][4 * q4 + 3] * mul;
      bad |= !(dev_finite(x0) && dev_finite(x1) && dev_finite(x2) && dev_finite(x3));
      uint2 w, r;
      w.x = pack2(x0, x1);
      w.y = pack2(x2, x3);
      r.x = pack2(x0 - __uint_as_float(w.x << 16), x1 - __uint_as_float(w.x & 0xffff0000u));
      r.y = pack2(x2 - __uint_as_float(w.y << 16), x3 - __uint_as_float(w.y & 0xffff0000u));
      *reinterpret_cast<uint2*>(plane + static_cast<long>(row) * rs + d) = w;
      *reinterpret_cast<uint2*>(resid + static_cast<long>(row) * rs + d) = r;
    }
  return bad;
}

// Workgroup -> (pair of row blocks, plane). Workgroups go to the 8 XCDs round-robin by their
// linear index and every XCD has its own L2, so the `pairs` workgroups of one plane (one head's
// K and V, or Q and dO) are given indices that are equal modulo 8: they run on one XCD, side by
// side, and the plane's tiles are fetched into one L2 instead of into several.
__device__ __forceinline__ void flash_block_of(int pairs, int planes, int* pair, long* plane) {
  const int id = blockIdx.x;
  if ((planes & 7) == 0) {
    *plane = (id & 7) + 8 * (id / (8 * pairs));
    *pair = (id >> 3) % pairs;
  } else {
    *pair = id % pairs;
    *plane = id / pairs;
  }
}

// ------------------------------------------------------------------ forward
// One 32-query x 64-key tile of one wave: scores, online softmax, weights times values.
//   NSUB      32-key halves of the tile that hold a visible key (the second half of a tile whose
//             first key is the wave's first query is hidden from all 32 rows and is left out);
//   MASK_SUB  the half the causal diagonal cuts (its keys start at the wave's first query), or -1;
//   GENERAL   the tile crosses the sequence end or a window edge: every element is tested.
// `m` is the running maximum of the raw scores; the scale joins inside the fma. `lsum` sums the
// weights as computed, `wsum` their bf16 copies (this lane's half of the keys).
template <int D, int NSUB, int MASK_SUB, bool GENERAL>
__device__ __forceinline__ void flash_fwd_tile(const char* k_rows, const char* v_rows, const u32x4 (&qf)[D / 16],
                                               floatx16 (&o)[D / 32], float& m, float& lsum, float& wsum,
                                               float scale_log2, int key0, int q_row, int T, int window, int lane) {
  constexpr int KK = D / 16, MT = D / 32;
  const int l32 = lane & 31, lg = lane >> 5;
  floatx16 sc[NSUB];
  // The SIMD serves its oldest wave first, and matrix and vector instructions of different waves
  // barely overlap (measured: three waves of 16 MFMAs + 160 FMAs take 0.88 of the sum of both alone).
  // A wave in its vector phase therefore holds up the others' products for the whole phase; raised
  // priority for the two short product phases keeps the matrix units fed (7 % on the forward pass).
  __builtin_amdgcn_s_setprio(2);
#pragma unroll
  for (int sub = 0; sub < NSUB; ++sub) {
    sc[sub] = zero16();
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) sc[sub] = mfma(frag_rows<D>(k_rows, sub, kk, l32, lg), qf[kk], sc[sub]);
  }
  __builtin_amdgcn_s_setprio(0);
  if constexpr (GENERAL) {
#pragma unroll
    for (int sub = 0; sub < NSUB; ++sub)
#pragma unroll
      for (int vv = 0; vv < 16; ++vv) {
        const int key = key0 + sub * 32 + acc_row(vv, lg);
        const bool masked = key > q_row || key >= T || (window > 0 && key + window <= q_row);
        sc[sub][vv] = masked ? -INFINITY : sc[sub][vv];
      }
  } else if constexpr (MASK_SUB >= 0) {
    // Key 4 lg + acc_row(v, 0) of the half against query l32 of the wave: a constant against one
    // value that never changes (kept opaque: hoisted out of the tile loop, the sixteen compare
    // results would occupy 32 scalar registers for the whole kernel).
    int tri = l32 - 4 * lg;
    asm volatile("" : "+v"(tri));
#pragma unroll
    for (int vv = 0; vv < 16; ++vv) sc[MASK_SUB][vv] = acc_row(vv, 0) > tri ? -INFINITY : sc[MASK_SUB][vv];
  }
  // Two chains, so that neither waits on the other's result.
  float tmax, tmax2;
  if constexpr (NSUB == 2) {
    tmax = fmaxf(sc[0][0], sc[1][0]);
    tmax2 = fmaxf(sc[0][1], sc[1][1]);
#pragma unroll
    for (int vv = 2; vv < 16; vv += 2) {
      tmax = max3(tmax, sc[0][vv], sc[1][vv]);
      tmax2 = max3(tmax2, sc[0][vv + 1], sc[1][vv + 1]);
    }
  } else {
    tmax = fmaxf(sc[0][0], sc[0][1]);
    tmax2 = fmaxf(sc[0][2], sc[0][3]);
#pragma unroll
    for (int vv = 4; vv < 16; vv += 4) {
      tmax = max3(tmax, sc[0][vv], sc[0][vv + 1]);
      tmax2 = max3(tmax2, sc[0][vv + 2], sc[0][vv + 3]);
    }
  }
  tmax = halves_max(fmaxf(tmax, tmax2));
  // The reference point of the exponents moves only when a row's maximum grew by more than 8
  // binary orders (always on a row's first tile, where m is -inf): below that the weights of
  // this tile are at most 2^8, well inside f32 and bf16, and the accumulators need no rescaling.
  // The quotient at the end and the log-sum-exp use the same reference, so both stay exact.
  const bool grow = (tmax - m) * scale_log2 > 8.0f;
  const float new_m = grow ? tmax : m;
  const float m_safe = new_m == -INFINITY ? 0.0f : new_m;
  const float neg_m = -m_safe * scale_log2;
  float psum = 0.0f;
#pragma unroll
  for (int sub = 0; sub < NSUB; ++sub)
#pragma unroll
    for (int vv = 0; vv < 16; ++vv) {
      float p = __builtin_amdgcn_exp2f(fmaf(sc[sub][vv], scale_log2, neg_m));
      sc[sub][vv] = p;
      psum += p;
    }
  psum = halves_sum(psum);
  if (__any(grow)) {
    // Some row's reference moved: rescale what is accumulated so far (by exactly 1 in the
    // rows that keep theirs).
    const float alpha = __builtin_amdgcn_exp2f(fmaf(m, scale_log2, neg_m));
    lsum *= alpha;
    wsum *= alpha;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int vv = 0; vv < 16; ++vv) o[mt][vv] *= alpha;
  }
  lsum += psum;
  m = new_m;
  __builtin_amdgcn_s_setprio(2);
#pragma unroll
  for (int sub = 0; sub < NSUB; ++sub)
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const u32x4 pb = pack8(sc[sub], c);
      wsum = sum_pairs(pb.x, sum_pairs(pb.y, sum_pairs(pb.z, sum_pairs(pb.w, wsum))));
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) o[mt] = mfma(frag_tr<D>(v_rows, mt, sub, c, lane), pb, o[mt]);
    }
  __builtin_amdgcn_s_setprio(0);
}

// WIN: the sliding-window form (every tile tested element by element), compiled apart so that the
// plain causal kernel carries neither its code nor its registers.
template <int D, typename TO, bool WIN>
__global__ __launch_bounds__(FT, D == 64 ? 3 : 2) void flash_fwd_kernel(const unsigned short* __restrict__ q,
                                                       const unsigned short* __restrict__ k,
                                                       const unsigned short* __restrict__ v, TO* __restrict__ out,
                                                       unsigned short* __restrict__ resid, float* __restrict__ lse,
                                                       FlashShape s, OmxFaultWord* fault, unsigned long long tag) {
  constexpr int KK = D / 16, MT = D / 32, NL = D / 32;  // d slabs, d blocks of the output, loads per thread and tile
  // Two key / value tile pairs: the next tile is stored while this one is multiplied, so a tile
  // costs one barrier.
  __shared__ __attribute__((aligned(16))) char smem[4 * ftile(D)];
  const int lane = threadIdx.x & 63, wave = wave_index(), l32 = lane & 31, lg = lane >> 5;
  const int T = s.time;
  const TileFetch<D> fetch(s.kv.rs, T);
  // Query block j sees j / 2 + 1 key tiles (causal): a workgroup takes a late block and then
  // its mirror image from the front, so every workgroup does the same amount of work and the
  // grid ends without a tail of half-empty compute units.
  const int q_blocks = (T + 127) / 128;
  int pair;
  long plane;
  if (s.q_single) {  // block rank (0 = the last, heaviest block) in the high part of the index
    pair = static_cast<int>(blockIdx.x) / (s.batch * s.heads);
    plane = static_cast<int>(blockIdx.x) % (s.batch * s.heads);
  } else {
    flash_block_of((q_blocks + 1) / 2, s.batch * s.heads, &pair, &plane);
  }
  for (int pass = 0; pass < (s.q_single ? 1 : 2); ++pass) {
    const int qb = pass == 0 ? q_blocks - 1 - pair : pair;
    if (pass == 1 && qb >= q_blocks - 1 - pair) break;
    const int h = static_cast<int>(plane % s.heads), b = static_cast<int>(plane / s.heads);
    const int kvh = h / s.rep;
    const unsigned short* qp = q + b * s.q.bs + h * s.q.hs;
    const unsigned short* kp = k + b * s.kv.bs + kvh * s.kv.hs;
    const unsigned short* vp = v + b * s.kv.bs + kvh * s.kv.hs;
    const int wave_q0 = qb * 128 + wave * 32;
    const int q_row = wave_q0 + l32;
    u32x4 qf[KK];
    row_frags<D>(qp, s.q.rs, q_row, T, lg, qf);
    floatx16 o[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) o[mt] = zero16();
    // `lsum` sums the weights as computed (the log-sum-exp, from which the backward pass rebuilds
    // them); `wsum` sums the bf16 copies the matrix units multiply into V (this lane's half of
    // the keys), and the output is divided by that: the output is then an exact weighted mean of
    // value rows, so a component shared by all of them passes through unchanged, and
    // dO . out cancels it against dP = dO . V in the backward pass. Divided by lsum it would
    // come through scaled by (sum of rounded weights) / (sum of weights).
    float m = -INFINITY, lsum = 0.0f, wsum = 0.0f;
    const float scale_log2 = s.scale * LOG2E;
    const int block_q0 = qb * 128, block_q1 = min(T - 1, qb * 128 + 127);
    const int kt_first = s.window > 0 ? max(0, block_q0 + 1 - s.window) / 64 : 0;
    const int kt_last = block_q1 / 64;
    // The next tile's global loads are in flight while the current one is multiplied.
    u32x4 rk[NL], rv[NL];
    fetch.load(kp, kt_first * 64, rk);
    fetch.load(vp, kt_first * 64, rv);
    __syncthreads();  // the previous pass's reads of the first pair are done
    tile_store_rows<D>(smem, rk);
    tile_store_rows<D>(smem + ftile(D), rv);
    if (kt_first < kt_last) {
      fetch.load(kp, kt_first * 64 + 64, rk);
      fetch.load(vp, kt_first * 64 + 64, rv);
    }
    // One step of the tile pipeline, taken by every wave for every tile of the block: wait for tile
    // kt's pair, store tile kt + 1 into the other pair, start the loads of tile kt + 2.
    const char* k_rows;
    const char* v_rows;
    auto advance = [&](int kt) {
      const int cur = (kt - kt_first) & 1;
      k_rows = smem + cur * 2 * ftile(D);
      v_rows = k_rows + ftile(D);
      __syncthreads();  // this pair is complete, and every wave is done with the other one
      if (kt < kt_last) {
        char* next = smem + (cur ^ 1) * 2 * ftile(D);
        tile_store_rows<D>(next, rk);
        tile_store_rows<D>(next + ftile(D), rv);
        if (kt + 1 < kt_last) {
          fetch.load(kp, kt * 64 + 128, rk);
          fetch.load(vp, kt * 64 + 128, rv);
        }
      }
    };
    int kt = kt_first;
    if constexpr (WIN) {
      for (; kt <= kt_last; ++kt) {
        advance(kt);
        const int key0 = kt * 64;
        if (key0 <= wave_q0 + 31 && key0 + 63 + s.window > wave_q0)
          flash_fwd_tile<D, 2, -1, true>(k_rows, v_rows, qf, o, m, lsum, wsum, scale_log2, key0, q_row, T, s.window, lane);
      }
    } else if (wave_q0 < T) {  // (a wave whose rows all lie past the sequence end only keeps the barriers)
      // The wave's first query is a multiple of 32 and a tile's first key a multiple of 64, so the
      // diagonal cuts exactly one 32 x 32 half of one tile, the wave's last: the first half of the tile
      // that starts at the wave's first query (whose second half no row sees), or the second half of
      // the tile that starts 32 keys earlier. The tiles before it need no mask, and their loop holds
      // nothing else: one body, so the accumulators stay in the registers the matrix units update.
      const int diag_kt = wave_q0 / 64;
      for (; kt < diag_kt; ++kt) {
        advance(kt);
        flash_fwd_tile<D, 2, -1, false>(k_rows, v_rows, qf, o, m, lsum, wsum, scale_log2, kt * 64, q_row, T, 0, lane);
      }
      advance(kt);
      const int key0 = kt * 64;
      if (D > 64 || key0 + 63 >= T)  // (at head_dim 128 the two cut-tile forms cost registers the kernel does not have)
        flash_fwd_tile<D, 2, -1, true>(k_rows, v_rows, qf, o, m, lsum, wsum, scale_log2, key0, q_row, T, 0, lane);
      else if (key0 == wave_q0)
        flash_fwd_tile<D, 1, 0, false>(k_rows, v_rows, qf, o, m, lsum, wsum, scale_log2, key0, q_row, T, 0, lane);
      else
        flash_fwd_tile<D, 2, 1, false>(k_rows, v_rows, qf, o, m, lsum, wsum, scale_log2, key0, q_row, T, 0, lane);
      ++kt;
    }
    for (; kt <= kt_last; ++kt) advance(kt);  // tiles of the block's later waves (same barrier count for all)
    wsum = halves_sum(wsum);
    bool bad = false;
    if (q_row < T) {
      bad |= !(dev_finite(lsum) && lsum > 0.0f && wsum > 0.0f);
      if (lg == 0) lse[plane * T + q_row] = m * s.scale + logf(lsum);
    }
    const long o_off = b * s.o.bs + h * s.o.hs;
    if constexpr (sizeof(TO) == 2) {
      if (resid) bad |= store_transposed_acc_split<D>(out + o_off, resid + o_off, s.o.rs, q_row, T, lg, o, 1.0f / wsum);
      else bad |= store_transposed_acc<D, TO>(out + o_off, s.o.rs, q_row, T, lg, o, 1.0f / wsum);
    } else {
      bad |= store_transposed_acc<D, TO>(out + o_off, s.o.rs, q_row, T, lg, o, 1.0f / wsum);
    }
    if (bad) dev_raise_fault(fault, tag);
  }  // pass
}

// ------------------------------------------------------------------ backward: dK, dV
// One 64-query x 32-key tile of one wave in the dK/dV pass. GENERAL: the tile crosses the diagonal,
// the sequence end or a window edge and every element is tested (as in the dQ pass, the cheaper
// forms of the cut tile would push the kernel past its registers).
template <int D, bool WANT_DK, bool WANT_DV, bool GENERAL>
__device__ __forceinline__ void flash_dkv_tile(const char* q_rows, const char* g_rows, const float* lse_s,
                                               const float* del_s, const u32x4 (&kf)[D / 16],
                                               const u32x4 (&vf)[WANT_DK ? D / 16 : 1], floatx16 (&dk)[WANT_DK ? D / 32 : 1],
                                               floatx16 (&dv)[WANT_DV ? D / 32 : 1], float scale_log2, int q0, int key_row,
                                               int T, int window, int lane) {
  constexpr int KK = D / 16, MT = D / 32;
  const int l32 = lane & 31, lg = lane >> 5;
#pragma unroll
  for (int sub = 0; sub < 2; ++sub) {
    floatx16 sc = zero16(), dp = zero16();
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      sc = mfma(frag_rows<D>(q_rows, sub, kk, l32, lg), kf[kk], sc);
      if constexpr (WANT_DK) dp = mfma(frag_rows<D>(g_rows, sub, kk, l32, lg), vf[kk], dp);
    }
    if constexpr (GENERAL) {
#pragma unroll
      for (int vv = 0; vv < 16; ++vv) {
        const int qi = q0 + sub * 32 + acc_row(vv, lg);
        const bool masked = key_row > qi || qi >= T || key_row >= T || (window > 0 && key_row + window <= qi);
        sc[vv] = masked ? -INFINITY : sc[vv];
      }
    }
    // P = 2^(s * scale * log2e - lse * log2e); dS / scale = P (dP - delta): the scale joins dK at the end.
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const float4 l4 = *reinterpret_cast<const float4*>(lse_s + sub * 32 + 8 * q4 + 4 * lg);
      const float lv[4] = {l4.x, l4.y, l4.z, l4.w};
      float dl[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      if constexpr (WANT_DK) {
        const float4 d4 = *reinterpret_cast<const float4*>(del_s + sub * 32 + 8 * q4 + 4 * lg);
        dl[0] = d4.x;
        dl[1] = d4.y;
        dl[2] = d4.z;
        dl[3] = d4.w;
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int vv = 4 * q4 + j;
        const float p = __builtin_amdgcn_exp2f(fmaf(sc[vv], scale_log2, -lv[j]));
        if constexpr (WANT_DK) dp[vv] = p * (dp[vv] - dl[j]);
        sc[vv] = p;
      }
    }
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      u32x4 pb = u32x4{0u, 0u, 0u, 0u}, dsb = u32x4{0u, 0u, 0u, 0u};
      if constexpr (WANT_DV) pb = pack8(sc, c);
      if constexpr (WANT_DK) dsb = pack8(dp, c);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if constexpr (WANT_DV) dv[mt] = mfma(frag_tr<D>(g_rows, mt, sub, c, lane), pb, dv[mt]);
        if constexpr (WANT_DK) dk[mt] = mfma(frag_tr<D>(q_rows, mt, sub, c, lane), dsb, dk[mt]);
      }
    }
  }
}

// One key block of one KV head: the loop over the query tiles that see it, accumulating dK
// (WANT_DK) and / or dV (WANT_DV) for the wave's 32 keys, then their stores. head_dim 64 runs it
// once for both. At head_dim 128 the two accumulator sets (128 registers), both key / value
// fragments (64) and the score tiles do not fit the 256 registers of two waves per SIMD, so the
// block is walked twice, once per gradient; the second walk recomputes the scores.
template <int D, typename TO, bool WANT_DK, bool WANT_DV, bool WIN>
__device__ __forceinline__ bool flash_dkv_block(const unsigned short* __restrict__ q,
                                                const unsigned short* __restrict__ k,
                                                const unsigned short* __restrict__ v, const float* __restrict__ lse,
                                                const float* __restrict__ delta, const unsigned short* __restrict__ gy,
                                                TO* __restrict__ gk, TO* __restrict__ gv, const FlashShape& s, char* smem,
                                                int kb, int b, int gidx) {
  constexpr int KK = D / 16, MT = D / 32, NL = D / 32;
  constexpr int SET = 2 * ftile(D) + 2 * 64 * 4;
  const int lane = threadIdx.x & 63, wave = wave_index(), l32 = lane & 31, lg = lane >> 5;
  const int T = s.time;
  const TileFetch<D> fetch_q(s.q.rs, T), fetch_g(s.o.rs, T);
  const long kv_off = b * s.kv.bs + gidx * s.kv.hs;
  const int wave_k0 = kb * 128 + wave * 32;
  const int key_row = wave_k0 + l32;
  u32x4 kf[KK], vf[WANT_DK ? KK : 1];
  row_frags<D>(k + kv_off, s.kv.rs, key_row, T, lg, kf);
  if constexpr (WANT_DK) row_frags<D>(v + kv_off, s.kv.rs, key_row, T, lg, vf);
  floatx16 dk[WANT_DK ? MT : 1], dv[WANT_DV ? MT : 1];
#pragma unroll
  for (int mt = 0; mt < (WANT_DK ? MT : 1); ++mt) dk[mt] = zero16();
#pragma unroll
  for (int mt = 0; mt < (WANT_DV ? MT : 1); ++mt) dv[mt] = zero16();
  const float scale_log2 = s.scale * LOG2E;
  const int block_k0 = kb * 128, block_k1 = min(T - 1, kb * 128 + 127);
  const int qt_first = block_k0 / 64;
  const int qt_last = (s.window > 0 ? min(T - 1, block_k1 + s.window - 1) : T - 1) / 64;
  bool bad = false;
  // One flat sequence of (query head of the group, query tile), ascending, so the
  // next tile's global loads can be in flight while the current one is multiplied.
  const int nq = qt_last - qt_first + 1;
  const int steps = s.rep * nq;
  u32x4 rq[NL], rg[NL];
  float row_lse = 0.0f, row_del = 0.0f;
  // (head of the group, query tile) of the tile being fetched.
  int fetch_r = 0, fetch_qt = qt_first;
  auto fetch = [&]() {
    const int r = fetch_r, q0 = fetch_qt * 64;
    if (++fetch_qt > qt_last) {
      fetch_qt = qt_first;
      ++fetch_r;
    }
    const long q_plane = static_cast<long>(b) * s.heads + static_cast<long>(gidx) * s.rep + r;
    const long head = static_cast<long>(gidx) * s.rep + r;
    fetch_q.load(q + b * s.q.bs + head * s.q.hs, q0, rq);
    fetch_g.load(gy + b * s.o.bs + head * s.o.hs, q0, rg);
    row_lse = 0.0f;
    row_del = 0.0f;
    if (threadIdx.x < 64 && q0 + static_cast<int>(threadIdx.x) < T) {
      row_lse = lse[q_plane * T + q0 + threadIdx.x];
      row_del = delta[q_plane * T + q0 + threadIdx.x];
      bad |= !(dev_finite(row_lse) && dev_finite(row_del));
    }
  };
  auto store_set = [&](char* set) {
    tile_store_rows<D>(set, rq);
    tile_store_rows<D>(set + ftile(D), rg);
    if (threadIdx.x < 64) {
      float* stats = reinterpret_cast<float*>(set + 2 * ftile(D));
      stats[threadIdx.x] = row_lse * LOG2E;
      stats[64 + threadIdx.x] = row_del;
    }
  };
  fetch();
  __syncthreads();  // an earlier walk's reads of the first set are done
  store_set(smem);
  if (steps > 1) fetch();
  // One step of the tile pipeline, taken by every wave for every tile: wait for set idx, store the
  // next one into the other set, start the loads of the one after.
  int idx = 0;
  const char* q_rows;
  const char* g_rows;
  const float* lse_s;
  const float* del_s;
  auto advance = [&]() {
    q_rows = smem + (idx & 1) * SET;
    g_rows = q_rows + ftile(D);
    lse_s = reinterpret_cast<const float*>(q_rows + 2 * ftile(D));
    del_s = lse_s + 64;
    __syncthreads();  // this set is complete, and every wave is done with the other one
    if (idx + 1 < steps) {
      store_set(smem + ((idx & 1) ^ 1) * SET);
      if (idx + 2 < steps) fetch();
    }
    ++idx;
  };
  auto tile = [&](auto general, int q0) {
    flash_dkv_tile<D, WANT_DK, WANT_DV, decltype(general)::value>(q_rows, g_rows, lse_s, del_s, kf, vf, dk, dv, scale_log2, q0,
                                                                 key_row, T, s.window, lane);
  };
  for (int r = 0; r < s.rep; ++r) {
    int qt = qt_first;
    if constexpr (WIN) {
      for (; qt <= qt_last; ++qt) {
        advance();
        const int q0 = qt * 64;
        if (q0 + 63 >= wave_k0 && q0 < wave_k0 + 31 + s.window) tile(std::true_type{}, q0);
      }
    } else if (wave_k0 < T) {  // (a wave whose keys all lie past the sequence end only keeps the barriers)
      // The wave's first key is a multiple of 32 and a tile's first query a multiple of 64, so the
      // diagonal cuts one tile, the first the wave takes. The tiles after it need no mask until the
      // sequence ends inside one, or inside the wave's keys; their loop holds nothing else.
      const int diag_qt = wave_k0 / 64;
      for (; qt < diag_qt; ++qt) advance();  // tiles of the block's earlier waves
      advance();
      tile(std::true_type{}, qt * 64);
      ++qt;
      const int plain_last = wave_k0 + 31 >= T ? qt - 1 : (T / 64) - 1;  // the last tile that ends inside the sequence
      for (; qt <= min(plain_last, qt_last); ++qt) {
        advance();
        tile(std::false_type{}, qt * 64);
      }
      for (; qt <= qt_last; ++qt) {
        advance();
        tile(std::true_type{}, qt * 64);
      }
    }
    for (; qt <= qt_last; ++qt) advance();
  }
  if constexpr (WANT_DK) bad |= store_transposed_acc<D, TO>(gk + kv_off, s.kv.rs, key_row, T, lg, dk, s.scale);
  if constexpr (WANT_DV) bad |= store_transposed_acc<D, TO>(gv + kv_off, s.kv.rs, key_row, T, lg, dv, 1.0f);
  return bad;
}

template <int D, typename TO, bool WIN>
__global__ __launch_bounds__(FT, 2) void flash_bwd_dkv_kernel(
    const unsigned short* __restrict__ q, const unsigned short* __restrict__ k, const unsigned short* __restrict__ v,
    const float* __restrict__ lse, const float* __restrict__ delta, const unsigned short* __restrict__ gy,
    TO* __restrict__ gk, TO* __restrict__ gv, FlashShape s, OmxFaultWord* fault, unsigned long long tag) {
  // Two sets of (query tile, gradient tile, 64 log-sum-exp values, 64 row terms): the next set is
  // stored while this one is multiplied, so a tile costs one barrier.
  __shared__ __attribute__((aligned(16))) char smem[2 * (2 * ftile(D) + 2 * 64 * 4)];
  // Early key blocks are seen by the most queries: a workgroup takes one of them and then its
  // mirror image from the back (see the forward kernel).
  const int k_blocks = (s.time + 127) / 128;
  int pair;
  long kv_plane;
  if (s.kv_single) {  // block index (0 = the first, heaviest block) in the high part of the index
    pair = static_cast<int>(blockIdx.x) / (s.batch * s.kv_heads);
    kv_plane = static_cast<int>(blockIdx.x) % (s.batch * s.kv_heads);
  } else {
    flash_block_of((k_blocks + 1) / 2, s.batch * s.kv_heads, &pair, &kv_plane);
  }
  const int gidx = static_cast<int>(kv_plane % s.kv_heads), b = static_cast<int>(kv_plane / s.kv_heads);
  bool bad = false;
  for (int pass = 0; pass < (s.kv_single ? 1 : 2); ++pass) {
    const int kb = pass == 0 ? pair : k_blocks - 1 - pair;
    if (pass == 1 && kb <= pair) break;
    if constexpr (D == 64) {
      bad |= flash_dkv_block<D, TO, true, true, WIN>(q, k, v, lse, delta, gy, gk, gv, s, smem, kb, b, gidx);
    } else {
      bad |= flash_dkv_block<D, TO, false, true, WIN>(q, k, v, lse, delta, gy, gk, gv, s, smem, kb, b, gidx);
      bad |= flash_dkv_block<D, TO, true, false, WIN>(q, k, v, lse, delta, gy, gk, gv, s, smem, kb, b, gidx);
    }
  }
  if (bad) dev_raise_fault(fault, tag);
}

// ------------------------------------------------------------------ backward: the mean key row
// key_mean[b, kv head, :] = the mean of up to 64 of that head's key rows, evenly spaced in time, in
// f32. The dQ pass needs a vector close to what the key rows share, not the exact mean (what it
// does with it is exact for any vector), so a sample is enough. One workgroup per (batch, kv head);
// a lane reads 8 values of a row, 256 / (D / 8) rows go round at once.
template <int D>
__global__ __launch_bounds__(256) void flash_key_mean_kernel(const unsigned short* __restrict__ k,
                                                             float* __restrict__ key_mean, FlashShape s) {
  constexpr int LPR = D / 8, ROWS = 256 / LPR;
  __shared__ float part[ROWS][D];
  const int b = blockIdx.x / s.kv_heads, h = blockIdx.x % s.kv_heads;
  const unsigned short* kp = k + b * s.kv.bs + h * s.kv.hs;
  const int col = (threadIdx.x % LPR) * 8, first = threadIdx.x / LPR;
  const int samples = min(s.time, 64);
  float sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int i = first; i < samples; i += ROWS) {
    const long row = static_cast<long>(i) * s.time / samples;
    const u32x4 w = *reinterpret_cast<const u32x4*>(kp + row * s.kv.rs + col);
    const unsigned int ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      sum[2 * j] += __uint_as_float(ww[j] << 16);
      sum[2 * j + 1] += __uint_as_float(ww[j] & 0xffff0000u);
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) part[first][col + i] = sum[i];
  __syncthreads();
  if (threadIdx.x < D) {
    float total = 0.0f;
    for (int r = 0; r < ROWS; ++r) total += part[r][threadIdx.x];
    key_mean[static_cast<long>(blockIdx.x) * D + threadIdx.x] = total / static_cast<float>(samples);
  }
}

// ------------------------------------------------------------------ backward: dQ
// One 32-query x 64-key tile of one wave in the dQ pass. GENERAL: the tile crosses the diagonal,
// the sequence end or a window edge and every element is tested (the forward's cheaper forms of
// the cut tile cost registers this kernel does not have: with them it spills, and runs 11 % slower).
// dS / scale = P (dP - delta) goes into dQ^T through the matrix units, and `ds_sum` collects this
// lane's share of the row sum of its bf16 copy.
template <int D, bool GENERAL>
__device__ __forceinline__ void flash_dq_tile(const char* k_rows, const char* v_rows, const u32x4 (&qf)[D / 16],
                                              const u32x4 (&gf)[D / 16], floatx16 (&dq)[D / 32], float& ds_sum,
                                              float scale_log2, float neg_lse, float row_del, int key0, int q_row, int T,
                                              int window, int lane) {
  constexpr int KK = D / 16, MT = D / 32;
  const int l32 = lane & 31, lg = lane >> 5;
#pragma unroll
  for (int sub = 0; sub < 2; ++sub) {
    floatx16 sc = zero16(), dp = zero16();
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      sc = mfma(frag_rows<D>(k_rows, sub, kk, l32, lg), qf[kk], sc);
      dp = mfma(frag_rows<D>(v_rows, sub, kk, l32, lg), gf[kk], dp);
    }
    if constexpr (GENERAL) {
#pragma unroll
      for (int vv = 0; vv < 16; ++vv) {
        const int key = key0 + sub * 32 + acc_row(vv, lg);
        const bool masked = key > q_row || key >= T || q_row >= T || (window > 0 && key + window <= q_row);
        sc[vv] = masked ? -INFINITY : sc[vv];
      }
    }
#pragma unroll
    for (int vv = 0; vv < 16; ++vv) {
      const float p = __builtin_amdgcn_exp2f(fmaf(sc[vv], scale_log2, neg_lse));
      dp[vv] = p * (dp[vv] - row_del);  // dS / scale: the scale joins dQ at the end
    }
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const u32x4 dsb = pack8(dp, c);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) dq[mt] = mfma(frag_tr<D>(k_rows, mt, sub, c, lane), dsb, dq[mt]);
      ds_sum = sum_pairs(dsb.x, sum_pairs(dsb.y, sum_pairs(dsb.z, sum_pairs(dsb.w, ds_sum))));
    }
  }
}

template <int D, typename TO, bool WIN>
__global__ __launch_bounds__(FT, D == 64 ? 3 : 2) void flash_bwd_dq_kernel(
    const unsigned short* __restrict__ q, const unsigned short* __restrict__ k, const unsigned short* __restrict__ v,
    const unsigned short* __restrict__ out, const unsigned short* __restrict__ resid, const float* __restrict__ lse,
    float* __restrict__ delta, const float* __restrict__ key_mean, const unsigned short* __restrict__ gy,
    TO* __restrict__ gq, FlashShape s, OmxFaultWord* fault, unsigned long long tag) {
  constexpr int KK = D / 16, MT = D / 32, NL = D / 32;
  // Two key / value tile pairs, as in the forward: one barrier per tile.
  __shared__ __attribute__((aligned(16))) char smem[4 * ftile(D)];
  const int lane = threadIdx.x & 63, wave = wave_index(), l32 = lane & 31, lg = lane >> 5;
  const int T = s.time;
  const TileFetch<D> fetch(s.kv.rs, T);
  // A late query block, then its mirror image from the front (see the forward kernel).
  const int q_blocks = (T + 127) / 128;
  int pair;
  long plane;
  if (s.q_single) {  // block rank (0 = the last, heaviest block) in the high part of the index
    pair = static_cast<int>(blockIdx.x) / (s.batch * s.heads);
    plane = static_cast<int>(blockIdx.x) % (s.batch * s.heads);
  } else {
    flash_block_of((q_blocks + 1) / 2, s.batch * s.heads, &pair, &plane);
  }
  for (int pass = 0; pass < (s.q_single ? 1 : 2); ++pass) {
    const int qb = pass == 0 ? q_blocks - 1 - pair : pair;
    if (pass == 1 && qb >= q_blocks - 1 - pair) break;
    const int h = static_cast<int>(plane % s.heads), b = static_cast<int>(plane / s.heads);
    const int kvh = h / s.rep;
    const unsigned short* kp = k + b * s.kv.bs + kvh * s.kv.hs;
    const unsigned short* vp = v + b * s.kv.bs + kvh * s.kv.hs;
    const int wave_q0 = qb * 128 + wave * 32;
    const int q_row = wave_q0 + l32;
    u32x4 qf[KK], gf[KK];
    row_frags<D>(q + b * s.q.bs + h * s.q.hs, s.q.rs, q_row, T, lg, qf);
    row_frags<D>(gy + b * s.o.bs + h * s.o.hs, s.o.rs, q_row, T, lg, gf);
    // delta = dO . O of this lane's row: each half-wave holds half of the row's values. The
    // dK/dV pass, launched after this one, reads it back from `delta`. dS = P (dP - delta) sums to
    // zero along a row only as far as delta matches sum_j P dP: taken from the bf16 output alone it
    // is off by 2^-9 of |dO| |O|, which a component shared by all value rows (and by all key rows,
    // in dQ = dS K) turns into a multiple of the gradient itself. With the saved rounding residual
    // of the output the mismatch drops to 2^-17.
    float row_del = 0.0f;
    {
      auto dot_rows = [&](const unsigned short* plane) {
        u32x4 of[KK];
        row_frags<D>(plane + b * s.o.bs + h * s.o.hs, s.o.rs, q_row, T, lg, of);
        float sum = 0.0f;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          const unsigned int gw[4] = {gf[kk].x, gf[kk].y, gf[kk].z, gf[kk].w};
          const unsigned int ow[4] = {of[kk].x, of[kk].y, of[kk].z, of[kk].w};
#pragma unroll
          for (int w = 0; w < 4; ++w) sum = dot_pairs(gw[w], ow[w], sum);
        }
        return sum;
      };
      row_del = dot_rows(out);
      if (resid) row_del += dot_rows(resid);
      row_del = halves_sum(row_del);
    }
    float row_lse = 0.0f;
    bool bad = false;
    if (q_row < T) {
      row_lse = lse[plane * T + q_row];
      if (lg == 0) delta[plane * T + q_row] = row_del;
      bad |= !(dev_finite(row_lse) && dev_finite(row_del));
    }
    const float neg_lse = -row_lse * LOG2E;
    floatx16 dq[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) dq[mt] = zero16();
    // A row of dS sums to zero, so dQ = dS K does not see a vector added to every key row. The
    // bf16 copy of dS that the matrix units read sums to its rounding error instead, and that
    // error times a component shared by all key rows (a residual stream grows one) lands in dQ at
    // 2^-9 of the component, however small the part of K that varies. `ds_sum` collects this
    // lane's share of the row sum of the rounded dS; the end takes (row sum) x (mean key) off.
    float ds_sum = 0.0f;
    const float scale_log2 = s.scale * LOG2E;
    const int block_q0 = qb * 128, block_q1 = min(T - 1, qb * 128 + 127);
    const int kt_first = s.window > 0 ? max(0, block_q0 + 1 - s.window) / 64 : 0;
    const int kt_last = block_q1 / 64;
    u32x4 rk[NL], rv[NL];
    fetch.load(kp, kt_first * 64, rk);
    fetch.load(vp, kt_first * 64, rv);
    __syncthreads();  // the previous pass's reads of the first pair are done
    tile_store_rows<D>(smem, rk);
    tile_store_rows<D>(smem + ftile(D), rv);
    if (kt_first < kt_last) {
      fetch.load(kp, kt_first * 64 + 64, rk);
      fetch.load(vp, kt_first * 64 + 64, rv);
    }
    // The tile pipeline and the split into unmasked tiles, the wave's diagonal tile and the other
    // waves' tiles are the forward kernel's.
    const char* k_rows;
    const char* v_rows;
    auto advance = [&](int kt) {
      const int cur = (kt - kt_first) & 1;
      k_rows = smem + cur * 2 * ftile(D);
      v_rows = k_rows + ftile(D);
      __syncthreads();  // this pair is complete, and every wave is done with the other one
      if (kt < kt_last) {
        char* next = smem + (cur ^ 1) * 2 * ftile(D);
        tile_store_rows<D>(next, rk);
        tile_store_rows<D>(next + ftile(D), rv);
        if (kt + 1 < kt_last) {
          fetch.load(kp, kt * 64 + 128, rk);
          fetch.load(vp, kt * 64 + 128, rv);
        }
      }
    };
    int kt = kt_first;
    if constexpr (WIN) {
      for (; kt <= kt_last; ++kt) {
        advance(kt);
        const int key0 = kt * 64;
        if (key0 <= wave_q0 + 31 && key0 + 63 + s.window > wave_q0)
          flash_dq_tile<D, true>(k_rows, v_rows, qf, gf, dq, ds_sum, scale_log2, neg_lse, row_del, key0, q_row, T, s.window,
                                 lane);
      }
    } else if (wave_q0 < T) {
      const int diag_kt = wave_q0 / 64;
      for (; kt < diag_kt; ++kt) {
        advance(kt);
        flash_dq_tile<D, false>(k_rows, v_rows, qf, gf, dq, ds_sum, scale_log2, neg_lse, row_del, kt * 64, q_row, T, 0, lane);
      }
      advance(kt);
      flash_dq_tile<D, true>(k_rows, v_rows, qf, gf, dq, ds_sum, scale_log2, neg_lse, row_del, kt * 64, q_row, T, 0, lane);
      ++kt;
    }
    for (; kt <= kt_last; ++kt) advance(kt);  // tiles of the block's later waves (same barrier count for all)
    {
      const float* mean = key_mean + (static_cast<long>(b) * s.kv_heads + kvh) * D;
      const float row_sum = halves_sum(ds_sum);  // the two half-waves hold half the keys each
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const float4 m = *reinterpret_cast<const float4*>(mean + mt * 32 + 8 * q4 + 4 * lg);
          dq[mt][4 * q4 + 0] = fmaf(-row_sum, m.x, dq[mt][4 * q4 + 0]);
          dq[mt][4 * q4 + 1] = fmaf(-row_sum, m.y, dq[mt][4 * q4 + 1]);
          dq[mt][4 * q4 + 2] = fmaf(-row_sum, m.z, dq[mt][4 * q4 + 2]);
          dq[mt][4 * q4 + 3] = fmaf(-row_sum, m.w, dq[mt][4 * q4 + 3]);
        }
    }
    bad |= store_transposed_acc<D, TO>(gq + b * s.q.bs + h * s.q.hs, s.q.rs, q_row, T, lg, dq, s.scale);
    if (bad) dev_raise_fault(fault, tag);
  }  // pass
}

// `strides`: nine element strides (row, head, batch of q; of k / v; of out), or null for
// contiguous [batch, heads, time, dim] tensors.
FlashShape make_shape(uint64_t batch, uint64_t heads, uint64_t kv_heads, uint64_t time, uint64_t dim, uint64_t window,
                      float scale, const long* strides) {
  FlashShape s;
  const long T = static_cast<long>(time), FD = static_cast<long>(dim);
  s.q = {FD, T * FD, static_cast<long>(heads) * T * FD};
  s.kv = {FD, T * FD, static_cast<long>(kv_heads) * T * FD};
  s.o = s.q;
  if (strides) {
    s.q = {strides[0], strides[1], strides[2]};
    s.kv = {strides[3], strides[4], strides[5]};
    s.o = {strides[6], strides[7], strides[8]};
  }
  s.batch = static_cast<int>(batch);
  s.heads = static_cast<int>(heads);
  s.kv_heads = static_cast<int>(kv_heads);
  s.time = static_cast<int>(time);
  s.window = static_cast<int>(window);
  s.rep = static_cast<int>(heads / kv_heads);
  s.q_single = s.kv_single = 0;
  s.scale = scale;
  return s;
}

// Whether a pass takes one block per workgroup: when the mirrored pairs are no more than the chip's
// workgroup places (`per_cu` per compute unit), twice as many workgroups fill them, and where the
// pairs fill the places exactly the lighter blocks still help: a compute unit serves its oldest
// workgroup first, so equal workgroups that start together end one after another (30, 38 and 45 us
// measured for the three of a unit), and the light blocks of the second half fill that tail
// (forward 43.2 -> 42.1 us at 768 pairs). `also_rounds`: also when the pairs need more than one
// round, whose last would run part empty (the blocks go out heaviest first).
int flash_single(omx_ctx* ctx, unsigned pair_groups, int per_cu, bool also_rounds) {
  if (ctx->flash_schedule != 0) return ctx->flash_schedule == 1 ? 1 : 0;  // forced (tests cover both)
  const unsigned places = static_cast<unsigned>(ctx->cu_count > 0 ? ctx->cu_count : 256) * per_cu;
  if (pair_groups <= places) return 1;
  return also_rounds ? 1 : 0;
}

template <int D>
void launch_forward(omx_ctx* ctx, const unsigned short* q, const unsigned short* k, const unsigned short* v, void* out,
                    int32_t out_dtype, void* out_residual, float* lse, const FlashShape& shape, unsigned long long tag) {
  FlashShape s = shape;
  // Two 128-row query blocks per workgroup (see the kernel), or one when the pairs would not fill
  // the chip's workgroup places.
  const unsigned q_blocks = static_cast<unsigned>((s.time + 127) / 128), planes = static_cast<unsigned>(s.batch * s.heads);
  s.q_single = flash_single(ctx, (q_blocks + 1) / 2 * planes, D == 64 ? 3 : 2, false);
  dim3 grid((s.q_single ? q_blocks : (q_blocks + 1) / 2) * planes), block(FT);
  // Causal-counted work: half of the 4 B H T^2 D of the two full products.
  OmxKernelTimer timer(ctx, OMX_K_FLASH_FWD, 2.0 * s.batch * s.heads * static_cast<double>(s.time) * s.time * D);
  auto go = [&](auto kernel, auto* out_ptr, unsigned short* resid_ptr) {
    omx_launch_timed(ctx, kernel, grid, block, 0, timer.start(), timer.stop(), q, k, v, out_ptr, resid_ptr, lse, s,
                     ctx->fault, tag);
  };
  unsigned short* resid = static_cast<unsigned short*>(out_residual);
  if (out_dtype == OMX_BF16) {
    if (s.window > 0) go(flash_fwd_kernel<D, unsigned short, true>, static_cast<unsigned short*>(out), resid);
    else go(flash_fwd_kernel<D, unsigned short, false>, static_cast<unsigned short*>(out), resid);
  } else {
    if (s.window > 0) go(flash_fwd_kernel<D, float, true>, static_cast<float*>(out), static_cast<unsigned short*>(nullptr));
    else go(flash_fwd_kernel<D, float, false>, static_cast<float*>(out), static_cast<unsigned short*>(nullptr));
  }
}

template <int D>
void launch_backward(omx_ctx* ctx, const unsigned short* q, const unsigned short* k, const unsigned short* v,
                     const unsigned short* out, const unsigned short* resid, const float* lse, float* delta,
                     float* key_mean, const unsigned short* gy, void* gq, void* gk, void* gv, int32_t grad_dtype,
                     const FlashShape& shape, unsigned long long tag) {
  FlashShape s = shape;
  // Five causal-counted products (S and dP twice each way, dV, dQ, dK) of B H T^2 D each.
  OmxKernelTimer timer(ctx, OMX_K_FLASH_BWD, 5.0 * s.batch * s.heads * static_cast<double>(s.time) * s.time * D);
  omx_launch_timed(ctx, flash_key_mean_kernel<D>, dim3(static_cast<unsigned>(s.batch * s.kv_heads)), dim3(256), 0,
                   timer.start(), nullptr, k, key_mean, s);
  // dQ first: it also leaves delta = dO . O per row for the dK/dV pass.
  dim3 block(FT);
  const unsigned pairs = static_cast<unsigned>((s.time + 127) / 128 + 1) / 2;  // two 128-row blocks per workgroup
  const unsigned blocks = static_cast<unsigned>((s.time + 127) / 128);
  const unsigned kv_planes = static_cast<unsigned>(s.batch * s.kv_heads), q_planes = static_cast<unsigned>(s.batch * s.heads);
  s.q_single = flash_single(ctx, pairs * q_planes, D == 64 ? 3 : 2, false);
  s.kv_single = flash_single(ctx, pairs * kv_planes, 2, true);
  dim3 kv_grid((s.kv_single ? blocks : pairs) * kv_planes);
  dim3 q_grid((s.q_single ? blocks : pairs) * q_planes);
  auto go = [&](auto dq_kernel, auto dkv_kernel, auto* gq_ptr, auto* gk_ptr, auto* gv_ptr) {
    hipLaunchKernelGGL(dq_kernel, q_grid, block, 0, ctx->stream, q, k, v, out, resid, lse, delta, key_mean, gy, gq_ptr, s,
                       ctx->fault, tag);
    omx_launch_timed(ctx, dkv_kernel, kv_grid, block, 0, nullptr, timer.stop(), q, k, v, lse, delta, gy, gk_ptr, gv_ptr, s,
                     ctx->fault, tag);
  };
  if (grad_dtype == OMX_BF16) {
    typedef unsigned short T16;
    if (s.window > 0)
      go(flash_bwd_dq_kernel<D, T16, true>, flash_bwd_dkv_kernel<D, T16, true>, static_cast<T16*>(gq), static_cast<T16*>(gk),
         static_cast<T16*>(gv));
    else
      go(flash_bwd_dq_kernel<D, T16, false>, flash_bwd_dkv_kernel<D, T16, false>, static_cast<T16*>(gq),
         static_cast<T16*>(gk), static_cast<T16*>(gv));
  } else {
    if (s.window > 0)
      go(flash_bwd_dq_kernel<D, float, true>, flash_bwd_dkv_kernel<D, float, true>, static_cast<float*>(gq),
         static_cast<float*>(gk), static_cast<float*>(gv));
    else
      go(flash_bwd_dq_kernel<D, float, false>, flash_bwd_dkv_kernel<D, float, false>, static_cast<float*>(gq),
         static_cast<float*>(gk), static_cast<float*>(gv));
  }
}

// The tile loads add a thread's rows as a 32-bit byte offset to a scalar base.
int32_t check_row_strides(omx_ctx* ctx, const FlashShape& s) {
  for (long rs : {s.q.rs, s.kv.rs, s.o.rs})
    if (rs < 1 || rs > FLASH_MAX_ROW_STRIDE)
      return omx_fail(ctx, OMX_SHAPE, "flash attention: row stride %ld outside 1..%ld elements", rs, FLASH_MAX_ROW_STRIDE);
  return OMX_OK;
}

}  // namespace

bool omx_flash_sdpa_supports(uint64_t dim, int32_t operand_dtype) {
  return (dim == 64 || dim == 128) && operand_dtype == OMX_BF16;
}

int32_t omx_flash_sdpa_forward(omx_ctx* ctx, const void* q, const void* k, const void* v, void* out, int32_t out_dtype,
                               void* out_residual, float* lse, uint64_t batch, uint64_t heads, uint64_t kv_heads,
                               uint64_t time, uint64_t dim, uint64_t window, float scale, unsigned long long tag,
                               const long* strides) {
  if (dim != 64 && dim != 128)
    return omx_fail(ctx, OMX_UNSUPPORTED_HEAD_DIM, "head_dim %llu: the MFMA kernels take 64 and 128",
                    (unsigned long long)dim);
  FlashShape s = make_shape(batch, heads, kv_heads, time, dim, window, scale, strides);
  if (int32_t rc = check_row_strides(ctx, s); rc != OMX_OK) return rc;
  const unsigned short* qs = static_cast<const unsigned short*>(q);
  const unsigned short* ks = static_cast<const unsigned short*>(k);
  const unsigned short* vs = static_cast<const unsigned short*>(v);
  if (dim == 64) launch_forward<64>(ctx, qs, ks, vs, out, out_dtype, out_residual, lse, s, tag);
  else launch_forward<128>(ctx, qs, ks, vs, out, out_dtype, out_residual, lse, s, tag);
  OMX_LAUNCH_CHECK(ctx, "flash_fwd_kernel");
  return OMX_OK;
}

int32_t omx_flash_sdpa_backward(omx_ctx* ctx, const void* q, const void* k, const void* v, const void* out,
                                const void* out_residual, const float* lse, const void* gy, void* gq, void* gk,
                                void* gv, int32_t grad_dtype,
                                uint64_t batch, uint64_t heads, uint64_t kv_heads, uint64_t time, uint64_t dim,
                                uint64_t window, float scale, unsigned long long tag, const long* strides) {
  if (dim != 64 && dim != 128)
    return omx_fail(ctx, OMX_UNSUPPORTED_HEAD_DIM, "head_dim %llu: the MFMA kernels take 64 and 128",
                    (unsigned long long)dim);
  FlashShape s = make_shape(batch, heads, kv_heads, time, dim, window, scale, strides);
  if (int32_t rc = check_row_strides(ctx, s); rc != OMX_OK) return rc;
  const long rows = static_cast<long>(batch * heads * time);
  void* ws = nullptr;
  const long rows4 = (rows + 3) & ~3L;  // the mean key rows are read four values at a time
  int32_t rc = omx_workspace(ctx, (rows4 + static_cast<long>(batch * kv_heads * dim)) * sizeof(float), &ws);
  if (rc != OMX_OK) return rc;
  float* delta = static_cast<float*>(ws);
  float* key_mean = delta + rows4;
  const unsigned short* qs = static_cast<const unsigned short*>(q);
  const unsigned short* ks = static_cast<const unsigned short*>(k);
  const unsigned short* vs = static_cast<const unsigned short*>(v);
  const unsigned short* os = static_cast<const unsigned short*>(out);
  const unsigned short* rs = static_cast<const unsigned short*>(out_residual);
  const unsigned short* gs = static_cast<const unsigned short*>(gy);
  if (dim == 64) launch_backward<64>(ctx, qs, ks, vs, os, rs, lse, delta, key_mean, gs, gq, gk, gv, grad_dtype, s, tag);
  else launch_backward<128>(ctx, qs, ks, vs, os, rs, lse, delta, key_mean, gs, gq, gk, gv, grad_dtype, s, tag);
  OMX_LAUNCH_CHECK(ctx, "flash backward kernels");
  return OMX_OK;
}
