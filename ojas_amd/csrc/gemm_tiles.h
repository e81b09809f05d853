// Pieces shared by the direct-to-LDS GEMM kernels (gemm_dma.hip, gemm_q8.hip): the per-lane
// global -> LDS load state of an operand tile, the swizzled fragment offsets that go with it,
// and the counted-wait helper.
#pragma once

#include <type_traits>

#include "gemm_args.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef short short4v __attribute__((ext_vector_type(4)));

// Per-lane state of one operand's loads: the global address of each of this wave's loads for the
// current K step (advanced by one step after every issue) and nothing else, so a step costs one
// 64-bit add per load. ROWS x BK bf16 per step, one wave instruction per KiB.
template <bool KM, int ROWS, int BK, int NW>  // NW: waves per workgroup
struct TileLoads {
  static constexpr int TOTAL = ROWS * BK * 2 / 1024;  // loads per step
  static constexpr int N = (TOTAL + NW - 1) / NW;     // per wave; the last one only in waves < TOTAL % NW
  static constexpr bool EVEN = TOTAL % NW == 0;
  const unsigned short* src[N];
  long step;  // elements between consecutive K steps

  __device__ __forceinline__ void init(const unsigned short* __restrict__ p, long ld, int row0, int rows, int k0,
                                       int wave, int lane) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int q = EVEN || wave + NW * i < TOTAL ? wave + NW * i : 0;  // an unused slot gets a valid address
      if constexpr (!KM) {
        // [row][BK / 8 chunks of 16 bytes], swizzled as frag_offset reads them.
        constexpr int LPR = BK / 8;  // lanes (chunks) per row
        const int r = q * (64 / LPR) + lane / LPR;
        const int kc = (lane % LPR) ^ (BK == 32 ? (r >> 2) & 3 : (r >> 1) & 7);
        int gr = row0 + r;
        gr = gr < rows ? gr : rows - 1;
        src[i] = p + static_cast<long>(gr) * ld + k0 + kc * 8;
      } else {
        constexpr int CPR = ROWS / 8;
        const int idx = q * 64 + lane;
        const int kr = idx / CPR, slot = idx % CPR;
        const int mc = slot ^ ((kr & 3) * 4);
        int gm = row0 + mc * 8;
        gm = gm + 8 <= rows ? gm : 0;
        src[i] = p + static_cast<long>(k0 + kr) * ld + gm;
      }
    }
    step = KM ? BK * ld : BK;
  }
  // Starts this step's loads into the operand tile at LDS byte address `tile` and moves on.
  __device__ __forceinline__ void issue(unsigned tile, int wave) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (!EVEN && wave + NW * i >= TOTAL) break;  // wave-uniform
      // Written as assembly: the compiler cannot tell that this asynchronous LDS write targets a
      // stage that is NOT being read, and would otherwise make every LDS read wait for it
      // (vmcnt(0) right after the issue), which serialises the loads with the products.
      asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src[i]),
                   "s"(tile + (wave + NW * i) * 1024)
                   : "memory");
      src[i] += step;
    }
  }
  // The same for the loads named in MASK only (bit i: this wave's load i, which fills KiB
  // wave + NW i of the tile): a part of the tile is refilled as soon as it has been read.
  template <unsigned MASK>
  __device__ __forceinline__ void issue_some(unsigned tile, int wave) {
    static_assert(EVEN, "every wave holds every load slot");
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (!((MASK >> i) & 1u)) continue;
      asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src[i]),
                   "s"(tile + (wave + NW * i) * 1024)
                   : "memory");
      src[i] += step;
    }
  }
};

// TileLoads with a wave-uniform base address (the tile's first element at the current K step, a scalar pair) and a
// 32-bit byte offset per lane and load that never changes: a K step advances one scalar instead of every lane's
// pointer (the 64-bit vector additions would take issue slots from the matrix instructions). Rows past the end are
// clamped in the offset, so edge tiles take this form too. Needs 255 rows of the leading dimension to fit 32 bits
// of bytes, and the same number of loads in every wave.
template <bool KM, int ROWS, int BK, int NW>
struct TileLoadsOff {
  static constexpr int TOTAL = ROWS * BK * 2 / 1024;
  static constexpr int N = TOTAL / NW;
  static_assert(TOTAL % NW == 0, "the same number of loads in every wave");
  unsigned off[N];
  const char* base;
  long step;  // bytes between consecutive K steps

  __device__ __forceinline__ void init(const unsigned short* __restrict__ p, long ld, int row0, int rows, int k0,
                                       int wave, int lane) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int q = wave + NW * i;
      if constexpr (!KM) {
        constexpr int LPR = BK / 8;
        const int r = q * (64 / LPR) + lane / LPR;
        const int kc = (lane % LPR) ^ (BK == 32 ? (r >> 2) & 3 : (r >> 1) & 7);
        int gr = row0 + r;
        gr = gr < rows ? gr : rows - 1;
        off[i] = static_cast<unsigned>(gr - row0) * static_cast<unsigned>(ld * 2) + kc * 16;
      } else {
        constexpr int CPR = ROWS / 8;
        const int idx = q * 64 + lane;
        const int kr = idx / CPR, slot = idx % CPR;
        const int mc = slot ^ ((kr & 3) * 4);
        int gm = mc * 8;
        gm = row0 + gm + 8 <= rows ? gm : 0;
        off[i] = static_cast<unsigned>(kr) * static_cast<unsigned>(ld * 2) + gm * 2;
      }
    }
    const long first = KM ? static_cast<long>(k0) * ld + row0 : static_cast<long>(row0) * ld + k0;
    const unsigned long long addr = reinterpret_cast<unsigned long long>(p) + static_cast<unsigned long long>(first) * 2;
    // (tile coordinates come out of vector divisions: back to scalars)
    const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(addr));
    const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(addr >> 32));
    base = reinterpret_cast<const char*>((static_cast<unsigned long long>(hi) << 32) | lo);
    step = (KM ? BK * ld : BK) * 2;
  }
  __device__ __forceinline__ void issue(unsigned tile, int wave) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off[i]), "s"(base),
                   "s"(tile + (wave + NW * i) * 1024)
                   : "memory");
    }
    base += step;
  }
};

// The same loads with one scalar base address per operand and a 32-bit byte offset per lane and
// load, taken from the tile's first element: the offsets do not depend on the tile, so a
// workgroup that walks several tiles only moves the scalar base (no per-lane address is ever
// recomputed), and a K step advances one scalar instead of every lane's pointer. The per-lane
// offsets are parked in LDS (`park`: N x threads words) and fetched back at each issue, which
// keeps them out of the registers the accumulators and fragments need. For tiles that lie
// wholly inside the operand (no row is clamped).
template <bool KM, int ROWS, int BK, int NW>
struct TileLoadsScalarBase {
  static constexpr int TOTAL = ROWS * BK * 2 / 1024;
  static constexpr int N = TOTAL / NW;
  static_assert(TOTAL % NW == 0, "the same number of loads in every wave");
  static constexpr int PARK_BYTES = N * NW * 64 * 4;
  const char* base;  // wave-uniform: the tile's first element + the current K step's byte offset
  long step;         // bytes between consecutive K steps

  __device__ __forceinline__ void init_lanes(unsigned* park, long ld, int wave, int lane) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int q = wave + NW * i;
      unsigned off;
      if constexpr (!KM) {
        constexpr int LPR = BK / 8;
        const int r = q * (64 / LPR) + lane / LPR;
        const int kc = (lane % LPR) ^ (BK == 32 ? (r >> 2) & 3 : (r >> 1) & 7);
        off = static_cast<unsigned>(r) * static_cast<unsigned>(ld * 2) + kc * 16;
      } else {
        constexpr int CPR = ROWS / 8;
        const int idx = q * 64 + lane;
        const int kr = idx / CPR, slot = idx % CPR;
        const int mc = slot ^ ((kr & 3) * 4);
        off = static_cast<unsigned>(kr) * static_cast<unsigned>(ld * 2) + mc * 16;
      }
      park[i * NW * 64 + threadIdx.x] = off;
    }
    step = (KM ? BK * ld : BK) * 2;
  }
  // Tile rows row0.. of the operand at `origin`, from K step 0.
  __device__ __forceinline__ void aim(const void* origin, long ld, int row0) {
    base = static_cast<const char*>(origin) + (KM ? static_cast<long>(row0) : static_cast<long>(row0) * ld) * 2;
  }
  // `lds_wave`: the LDS address of this wave's first KiB of the stage area; TILE: the byte offset
  // of the operand's tile in it. M0 is formed from the one scalar and an immediate.
  // The parked offsets of this lane, fetched with one wait for all of them.
  __device__ __forceinline__ void fetch(const unsigned* park, unsigned (&off)[N]) const {
    // (the index is formed here for the same reason as in xor_here)
    unsigned slot;
    asm volatile("v_lshlrev_b32 %0, 2, %1" : "=v"(slot) : "v"(threadIdx.x));
#pragma unroll
    for (int i = 0; i < N; ++i)
      off[i] = *reinterpret_cast<const unsigned*>(reinterpret_cast<const char*>(park) + i * NW * 64 * 4 + slot);
  }
  template <int TILE>
  __device__ __forceinline__ void issue(const unsigned (&off)[N], unsigned lds_wave) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off[i]), "s"(base),
                   "s"(lds_wave), "n"(TILE + NW * i * 1024)
                   : "memory", "scc");
    }
    base += step;
  }
  // The same with the stage's byte offset in a scalar register.
  template <int TILE>
  __device__ __forceinline__ void issue_at(const unsigned (&off)[N], unsigned lds_wave, unsigned stage_bytes) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      asm volatile("s_add_u32 m0, %2, %3\n\ts_add_u32 m0, m0, %4\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off[i]),
                   "s"(base), "s"(lds_wave), "s"(stage_bytes), "n"(TILE + NW * i * 1024)
                   : "memory", "scc");
    }
    base += step;
  }
};

// Byte offset, inside an operand tile, of this lane's fragment for 32-row block `row_base / 32`
// and 16-column K slab kk (k-major operands: of its first transposing read; the second is four
// K rows further).
template <bool KM, int ROWS, int BK>
__device__ __forceinline__ int frag_offset(int row_base, int kk, int lane) {
  if constexpr (!KM) {
    const int l32 = lane & 31, g = lane >> 5;
    const int r = row_base + l32;
    const int kc = kk * 2 + g;
    return r * (BK * 2) + ((kc ^ (BK == 32 ? (r >> 2) & 3 : (r >> 1) & 7)) << 4);
  } else {
    const int s = lane & 15, half = (lane >> 4) & 1, g = lane >> 5;
    const int kr = kk * 16 + g * 8 + (s >> 2);
    const int col = row_base + half * 16 + (s & 3) * 4;
    const int slot = (col >> 3) ^ (((s >> 2) & 3) * 4);
    return kr * (ROWS * 2) + slot * 16 + (col & 7) * 2;
  }
}
// frag_offset(row_base + 32 t, kk, lane) from `first` = frag_offset(row_base, 0, lane), for a
// row_base that is a multiple of 64. k-contiguous tiles: a 32-row block further is 32 rows of
// bytes further (the swizzle repeats every 8 or 16 rows), and slab kk flips the chunk index's bits
// 1.., i.e. bits 5.. of the offset. k-major tiles: slab kk is 16 K rows further, and a 32-column
// block further flips bit 2 of the chunk slot (bit 6 of the offset).
// x ^ bits, computed where it is used: the assembly statement keeps the compiler from hoisting
// the result out of the K loop into a register of its own (the accumulators need them all).
template <int BITS>
__device__ __forceinline__ int xor_here(int x) {
  if constexpr (BITS == 0) return x;
  int r;
  asm volatile("v_xor_b32 %0, %1, %2" : "=v"(r) : "n"(BITS), "v"(x));
  return r;
}
template <bool KM, int ROWS, int BK, int T, int KKI>
__device__ __forceinline__ int frag_from_first(int first) {
  if constexpr (!KM) return xor_here<(KKI << 5)>(first) + T * 32 * BK * 2;
  else return xor_here<(T << 6)>(first) + KKI * 16 * ROWS * 2;
}
template <bool KM, int ROWS>
__device__ __forceinline__ u32x4 frag_at(const char* p) {
  if constexpr (!KM) {
    return *reinterpret_cast<const u32x4*>(p);
  } else {
    typedef short4v __attribute__((address_space(3))) * lds_ptr;
    short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
    short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 4 * ROWS * 2));
    u32x2 a = __builtin_bit_cast(u32x2, lo), b = __builtin_bit_cast(u32x2, hi);
    return u32x4{a.x, a.y, b.x, b.y};
  }
}

// s_waitcnt operand that waits for vmcnt <= n only (vmcnt is bits 3:0 and 15:14).
constexpr int vmcnt_only(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }

// Waves per SIMD the kernel is compiled for: as many workgroups per compute unit as its LDS (160
// KiB) allows, up to four waves per SIMD.
constexpr int dma_waves_per_simd(int waves, int lds_bytes) {
  const int by_lds = 160 * 1024 / lds_bytes, by_waves = 16 / waves;
  return (by_lds < by_waves ? by_lds : by_waves) * waves / 4;
}

// f(integral_constant<int, I>) for I = BEGIN .. END - 1.
template <int BEGIN, int END, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (BEGIN < END) {
    f(std::integral_constant<int, BEGIN>{});
    static_for<BEGIN + 1, END>(f);
  }
}

}  // namespace
