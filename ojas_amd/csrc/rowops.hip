// Row-wise bandwidth-bound kernels: RMSNorm forward/backward, embedding
// gather / scatter-add, argmax and top-k. One wave (64 lanes) owns one row;
// reductions are wavefront shuffles; every tensor is read from HBM once.
//
// Reference semantics:
//   rms_norm_*   ojas-cpu/src/norm.rs:24-204   (trait backend.rs:1658-1672)
//   embedding_*  ojas-cpu/src/pointwise.rs:77-215 (trait backend.rs:1610-1626)
//   argmax/topk  ojas-core/src/backend.rs:184-195,1514-1606
#include "omx_common.h"

namespace {

constexpr int ROW_THREADS = 256;  // 4 waves per block, one row per wave at a time

// ---------------------------------------------------------------- RMSNorm
// PER = ceil(dim / 64): lane l owns columns l, l + 64, ... so a wave's loads
// are contiguous 64-element runs and the row stays in registers between the
// sum-of-squares pass and the scaling pass.
template <typename TX, typename TY, int PER>
__global__ __launch_bounds__(ROW_THREADS) void rms_fwd_kernel(const TX* __restrict__ x, const float* __restrict__ w,
                                                              TY* __restrict__ y, size_t rows, int dim, float eps,
                                                              OmxFaultWord* fault, unsigned long long tag) {
  const int lane = threadIdx.x & 63;
  const size_t row = static_cast<size_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const TX* xr = x + row * dim;
  float xv[PER];
  float ss = 0.0f;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    int c = j * 64 + lane;
    xv[j] = c < dim ? dev_load<TX>(xr, c) : 0.0f;
    ss += xv[j] * xv[j];
  }
  ss = wave_sum(ss);
  float denom = ss / static_cast<float>(dim) + eps;
  float rstd = 1.0f / sqrtf(denom);
  bool bad = !(dev_finite(denom) && denom > 0.0f && dev_finite(rstd));
  TY* yr = y + row * dim;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    int c = j * 64 + lane;
    if (c < dim) {
      float v = xv[j] * rstd * w[c];
      bad |= !dev_finite(v);
      dev_store<TY>(yr, c, v);
    }
  }
  if (bad) dev_raise_fault(fault, tag);
}

// Backward: gx per row, and per-block partial column sums of g * xhat that a
// second kernel adds in ascending block order (no atomics, deterministic).
template <typename TX, typename TG, typename TO, int PER>
__global__ __launch_bounds__(ROW_THREADS) void rms_bwd_kernel(const TX* __restrict__ x, const float* __restrict__ w,
                                                              const TG* __restrict__ gy, TO* __restrict__ gx,
                                                              float* __restrict__ partial, size_t rows, int dim,
                                                              float eps, int rows_per_block, OmxFaultWord* fault,
                                                              unsigned long long tag) {
  extern __shared__ float lds[];  // [4][dim]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float inv_dim = 1.0f / static_cast<float>(dim);
  float wv[PER], accw[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    int c = j * 64 + lane;
    wv[j] = c < dim ? w[c] : 0.0f;
    accw[j] = 0.0f;
  }
  bool bad = false;
  const size_t first = static_cast<size_t>(blockIdx.x) * rows_per_block;
  const size_t last = min(rows, first + rows_per_block);
  for (size_t row = first + wave; row < last; row += 4) {
    const TX* xr = x + row * dim;
    const TG* gr = gy + row * dim;
    float xv[PER], gv[PER];
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      int c = j * 64 + lane;
      xv[j] = c < dim ? dev_load<TX>(xr, c) : 0.0f;
      gv[j] = c < dim ? dev_load<TG>(gr, c) : 0.0f;
      ss += xv[j] * xv[j];
    }
    ss = wave_sum(ss);
    float denom = ss * inv_dim + eps;
    float rstd = 1.0f / sqrtf(denom);
    bad |= !(dev_finite(denom) && denom > 0.0f && dev_finite(rstd));
    float dot = 0.0f;
#pragma unroll
    for (int j = 0; j < PER; ++j) dot += (gv[j] * wv[j]) * (xv[j] * rstd);
    dot = wave_sum(dot);
    float mean = dot * inv_dim;
    TO* gxr = gx + row * dim;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      int c = j * 64 + lane;
      float xhat = xv[j] * rstd;
      float v = (gv[j] * wv[j] - xhat * mean) * rstd;
      accw[j] += gv[j] * xhat;
      if (c < dim) {
        bad |= !dev_finite(v);
        dev_store<TO>(gxr, c, v);
      }
    }
  }
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    int c = j * 64 + lane;
    if (c < dim) lds[wave * dim + c] = accw[j];
  }
  __syncthreads();
  for (int c = threadIdx.x; c < dim; c += ROW_THREADS) {
    float s = ((lds[c] + lds[dim + c]) + lds[2 * dim + c]) + lds[3 * dim + c];
    partial[static_cast<size_t>(blockIdx.x) * dim + c] = s;
  }
  if (bad) dev_raise_fault(fault, tag);
}

// out[c] = sum over blocks of partial[b][c]: 64 columns per workgroup, four
// row groups that each add their strided share, then a fixed four-way sum.
__global__ __launch_bounds__(256) void column_sum_kernel(const float* __restrict__ partial, float* __restrict__ out,
                                                         int blocks, int dim, OmxFaultWord* fault,
                                                         unsigned long long tag) {
  __shared__ float red[4][64];
  const int lane = threadIdx.x & 63, group = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  float s = 0.0f;
  if (c < dim)
    for (int b = group; b < blocks; b += 4) s += partial[static_cast<size_t>(b) * dim + c];
  red[group][lane] = s;
  __syncthreads();
  if (group == 0 && c < dim) {
    float total = ((red[0][lane] + red[1][lane]) + red[2][lane]) + red[3][lane];
    out[c] = total;
    if (!dev_finite(total)) dev_raise_fault(fault, tag);
  }
}

// The same for a few hundred rows in one launch: 16 row groups of 64 columns (1024 threads), four
// loads in flight per thread, the groups added in a fixed order.
__global__ __launch_bounds__(1024) void column_sum_wide_kernel(const float* __restrict__ partial,
                                                               float* __restrict__ out, int blocks, int dim,
                                                               OmxFaultWord* fault, unsigned long long tag) {
  __shared__ float red[16][64];
  const int lane = threadIdx.x & 63, group = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
  if (c < dim) {
    const float* col = partial + c;
    int b = group;
    for (; b + 48 < blocks; b += 64) {
      s0 += col[static_cast<size_t>(b) * dim];
      s1 += col[static_cast<size_t>(b + 16) * dim];
      s2 += col[static_cast<size_t>(b + 32) * dim];
      s3 += col[static_cast<size_t>(b + 48) * dim];
    }
    for (; b < blocks; b += 16) s0 += col[static_cast<size_t>(b) * dim];
  }
  red[group][lane] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (group == 0 && c < dim) {
    float total = 0.0f;
#pragma unroll
    for (int g = 0; g < 16; ++g) total += red[g][lane];
    out[c] = total;
    if (!dev_finite(total)) dev_raise_fault(fault, tag);
  }
}

// Stage 1 of a tall column sum: block (x, g) adds rows [g * per_group, (g + 1) * per_group) of its
// 64 columns, four row groups in parallel, then a fixed four-way sum.
__global__ __launch_bounds__(256) void column_sum_groups_kernel(const float* __restrict__ partial,
                                                                float* __restrict__ scratch, int blocks, int dim,
                                                                int per_group) {
  __shared__ float red[4][64];
  const int lane = threadIdx.x & 63, group = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  const int first = blockIdx.y * per_group, last = min(blocks, first + per_group);
  float s = 0.0f;
  if (c < dim)
    for (int b = first + group; b < last; b += 4) s += partial[static_cast<size_t>(b) * dim + c];
  red[group][lane] = s;
  __syncthreads();
  if (group == 0 && c < dim)
    scratch[static_cast<size_t>(blockIdx.y) * dim + c] = ((red[0][lane] + red[1][lane]) + red[2][lane]) + red[3][lane];
}

// ---------------------------------------------------------------- embedding
template <typename TT, typename TO>
__global__ void embedding_fwd_kernel(const TT* __restrict__ table, const unsigned int* __restrict__ ids,
                                     TO* __restrict__ out, size_t tokens, size_t vocab, int dim, OmxFaultWord* fault,
                                     unsigned long long tag) {
  const int lane = threadIdx.x & 63;
  const size_t n = static_cast<size_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (n >= tokens) return;
  size_t id = ids[n];
  TO* dst = out + n * dim;
  if (id >= vocab) {
    // Refused id: the row is zero-filled and the call reports OutOfRange.
    for (int c = lane; c < dim; c += 64) dev_store<TO>(dst, c, 0.0f);
    if (lane == 0) dev_raise_range(fault, tag);
    return;
  }
  const TT* src = table + id * dim;
  if constexpr (sizeof(TT) == sizeof(TO)) {
    // Same storage: a bit copy (NaN payloads and -0 survive).
    for (int c = lane; c < dim; c += 64) dst[c] = src[c];
  } else {
    for (int c = lane; c < dim; c += 64) dev_store<TO>(dst, c, dev_load<TT>(src, c));
  }
}

__global__ void count_ids_kernel(const unsigned int* __restrict__ ids, unsigned int* __restrict__ counts,
                                 size_t tokens, size_t vocab, OmxFaultWord* fault, unsigned long long tag) {
  size_t n = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (n >= tokens) return;
  unsigned int id = ids[n];
  if (id >= vocab) {
    dev_raise_range(fault, tag);
    return;
  }
  atomicAdd(&counts[id], 1u);
}

// Exclusive scan of counts[vocab] into offsets[vocab + 1] and a copy into
// cursor[vocab]; one 1024-thread block walks the array in 1024-wide strips.
__global__ __launch_bounds__(1024) void scan_counts_kernel(const unsigned int* __restrict__ counts,
                                                           unsigned int* __restrict__ offsets,
                                                           unsigned int* __restrict__ cursor, size_t vocab) {
  __shared__ unsigned int wave_tot[16];
  __shared__ unsigned int carry;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (size_t base = 0; base < vocab; base += 1024) {
    size_t i = base + threadIdx.x;
    unsigned int v = i < vocab ? counts[i] : 0u;
    unsigned int incl = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      unsigned int t = __shfl_up(incl, off, 64);
      if (lane >= off) incl += t;
    }
    if (lane == 63) wave_tot[wave] = incl;
    __syncthreads();
    unsigned int before = carry;
    for (int wv = 0; wv < wave; ++wv) before += wave_tot[wv];
    unsigned int excl = before + incl - v;
    if (i < vocab) {
      offsets[i] = excl;
      cursor[i] = excl;
    }
    __syncthreads();
    if (threadIdx.x == 1023) carry = excl + v;
    __syncthreads();
  }
  if (threadIdx.x == 0) offsets[vocab] = carry;
}

// The same scan over many blocks, for tables of more than a few thousand rows (one block walks
// 50304 counts in 55 us): every block of 1024 counts leaves its total, then every block adds up the
// totals before it (at most SCAN_MAX_BLOCKS of them) and scans its own counts behind that.
constexpr int SCAN_MAX_BLOCKS = 1024;
__device__ __forceinline__ unsigned int scan_block_1024(unsigned int v, unsigned int* wave_tot, unsigned int* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  unsigned int incl = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    unsigned int t = __shfl_up(incl, off, 64);
    if (lane >= off) incl += t;
  }
  if (lane == 63) wave_tot[wave] = incl;
  __syncthreads();
  unsigned int before = 0, all = 0;
  for (int wv = 0; wv < 16; ++wv) {
    if (wv < wave) before += wave_tot[wv];
    all += wave_tot[wv];
  }
  *total = all;
  return before + incl - v;  // exclusive, within the block
}
__global__ __launch_bounds__(1024) void scan_totals_kernel(const unsigned int* __restrict__ counts,
                                                           unsigned int* __restrict__ totals, size_t vocab) {
  __shared__ unsigned int wave_tot[16];
  const size_t i = static_cast<size_t>(blockIdx.x) * 1024 + threadIdx.x;
  unsigned int total;
  scan_block_1024(i < vocab ? counts[i] : 0u, wave_tot, &total);
  if (threadIdx.x == 0) totals[blockIdx.x] = total;
}
__global__ __launch_bounds__(1024) void scan_blocks_kernel(const unsigned int* __restrict__ counts,
                                                           const unsigned int* __restrict__ totals,
                                                           unsigned int* __restrict__ offsets,
                                                           unsigned int* __restrict__ cursor, size_t vocab) {
  __shared__ unsigned int wave_tot[16];
  __shared__ unsigned int lead_tot[16];
  // The totals of the blocks before this one: thread t takes block t's.
  unsigned int mine = threadIdx.x < blockIdx.x ? totals[threadIdx.x] : 0u;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mine += __shfl_xor(mine, off, 64);
  if ((threadIdx.x & 63) == 0) lead_tot[threadIdx.x >> 6] = mine;
  __syncthreads();
  unsigned int lead = 0;
  for (int wv = 0; wv < 16; ++wv) lead += lead_tot[wv];
  const size_t i = static_cast<size_t>(blockIdx.x) * 1024 + threadIdx.x;
  const unsigned int v = i < vocab ? counts[i] : 0u;
  unsigned int total;
  const unsigned int excl = lead + scan_block_1024(v, wave_tot, &total);
  if (i < vocab) {
    offsets[i] = excl;
    cursor[i] = excl;
  }
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) offsets[vocab] = lead + total;
}

__global__ void fill_positions_kernel(const unsigned int* __restrict__ ids, unsigned int* __restrict__ cursor,
                                      unsigned int* __restrict__ positions, size_t tokens, size_t vocab) {
  size_t n = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (n >= tokens) return;
  unsigned int id = ids[n];
  if (id >= vocab) return;
  unsigned int slot = atomicAdd(&cursor[id], 1u);
  positions[slot] = static_cast<unsigned int>(n);
}

// fill_positions_kernel leaves a row's token positions in arrival order. The sums below must run
// in ascending token order (the order of the CPU scatter, pointwise.rs:196-207) to carry the same
// bits, so every row's segment is sorted first, out of place:
//   * up to 64 positions: one wave, a bitonic network over lane shuffles;
//   * longer segments (one id filling a large share of the batch) are queued and sorted by
//     sort_long_segments_kernel below.
__global__ __launch_bounds__(ROW_THREADS) void sort_short_segments_kernel(const unsigned int* __restrict__ offsets,
                                                                          const unsigned int* __restrict__ positions,
                                                                          unsigned int* __restrict__ sorted,
                                                                          unsigned int* __restrict__ long_count,
                                                                          unsigned int* __restrict__ long_rows,
                                                                          size_t vocab) {
  const int lane = threadIdx.x & 63;
  const size_t v = static_cast<size_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (v >= vocab) return;
  const unsigned int begin = offsets[v], end = offsets[v + 1], len = end - begin;
  if (len == 0) return;
  if (len > 64) {
    if (lane == 0) long_rows[atomicAdd(long_count, 1u)] = static_cast<unsigned int>(v);
    return;
  }
  unsigned int p = static_cast<unsigned int>(lane) < len ? positions[begin + lane] : 0xffffffffu;
#pragma unroll
  for (int k = 2; k <= 64; k <<= 1)
#pragma unroll
    for (int j = k >> 1; j > 0; j >>= 1) {
      const unsigned int other = __shfl_xor(p, j, 64);
      const bool ascending = (lane & k) == 0;
      const bool keep_min = ((lane & j) == 0) == ascending;
      p = keep_min ? min(p, other) : max(p, other);
    }
  if (static_cast<unsigned int>(lane) < len) sorted[begin + lane] = p;
}

// One 1024-thread block per queued row. Positions are distinct token indices, so a bitmap orders
// them: for each window of 32768 tokens the block marks the row's positions that fall into it
// (one word per thread), then writes the set bits out in order at a running offset. Linear in
// the segment's length per window, whatever the length.
__global__ __launch_bounds__(1024) void sort_long_segments_kernel(const unsigned int* __restrict__ offsets,
                                                                   const unsigned int* __restrict__ positions,
                                                                   unsigned int* __restrict__ sorted,
                                                                   const unsigned int* __restrict__ long_count,
                                                                   const unsigned int* __restrict__ long_rows,
                                                                   size_t tokens) {
  __shared__ unsigned int bitmap[1024];
  __shared__ unsigned int wave_tot[16];
  __shared__ unsigned int written;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const unsigned int rows = *long_count;
  for (unsigned int q = blockIdx.x; q < rows; q += gridDim.x) {
    const unsigned int v = long_rows[q];
    const unsigned int begin = offsets[v], end = offsets[v + 1];
    if (threadIdx.x == 0) written = 0;
    for (size_t base = 0; base < tokens; base += 32768) {
      bitmap[threadIdx.x] = 0;
      __syncthreads();
      if (written == end - begin) break;  // uniform: read after the barrier, written before the previous one
      for (unsigned int s = begin + threadIdx.x; s < end; s += 1024) {
        const size_t rel = static_cast<size_t>(positions[s]) - base;  // wraps far above the window when below it
        if (rel < 32768) atomicOr(&bitmap[rel >> 5], 1u << (rel & 31));
      }
      __syncthreads();
      unsigned int w = bitmap[threadIdx.x];
      const unsigned int c = __popc(w);
      unsigned int incl = c;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const unsigned int t = __shfl_up(incl, off, 64);
        if (lane >= off) incl += t;
      }
      if (lane == 63) wave_tot[wave] = incl;
      __syncthreads();
      unsigned int before = written;
      for (int wv = 0; wv < wave; ++wv) before += wave_tot[wv];
      unsigned int at = begin + before + incl - c;
      while (w) {
        const int bit = __ffs(w) - 1;
        sorted[at++] = static_cast<unsigned int>(base) + threadIdx.x * 32 + bit;
        w &= w - 1;
      }
      __syncthreads();
      if (threadIdx.x == 1023) written = before + incl;
      __syncthreads();
    }
    __syncthreads();
  }
}

// One wave per table row: zero it, or add its tokens' gradient rows in ascending token order
// (`sorted`: the row's positions, ascending), so the f32 sums carry the CPU scatter's bits.
// V = 4: a lane owns four consecutive columns (16-byte accesses; dim a multiple of 4, aligned rows).
// ADD: the row's sum, complete, is added to what `table_grad` holds (the bits of the scatter
// followed by accumulate_grad), and rows no token names are left alone.
template <typename TG, int V, bool ADD>
__global__ __launch_bounds__(ROW_THREADS) void embedding_bwd_kernel(const unsigned int* __restrict__ offsets,
                                                                    const unsigned int* __restrict__ sorted,
                                                                    const TG* __restrict__ grad,
                                                                    float* __restrict__ table_grad, size_t vocab,
                                                                    int dim, OmxFaultWord* fault,
                                                                    unsigned long long tag) {
  const int lane = threadIdx.x & 63;
  const size_t v = static_cast<size_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (v >= vocab) return;
  const unsigned int begin = offsets[v], end = offsets[v + 1];
  float* dst = table_grad + v * dim;
  if (begin == end) {
    if constexpr (ADD) return;
    if constexpr (V == 4) {
      for (int c = lane * 4; c < dim; c += 256) *reinterpret_cast<float4*>(dst + c) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    } else {
      for (int c = lane; c < dim; c += 64) dst[c] = 0.0f;
    }
    return;
  }
  bool bad = false;
  constexpr int CHUNKS = 8 / V;  // 8 columns per lane and pass
  for (int c0 = 0; c0 < dim; c0 += 64 * 8) {
    float acc[CHUNKS][V];
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j)
#pragma unroll
      for (int e = 0; e < V; ++e) acc[j][e] = 0.0f;
    for (unsigned int s = begin; s < end; ++s) {
      const TG* src = grad + static_cast<size_t>(sorted[s]) * dim;
#pragma unroll
      for (int j = 0; j < CHUNKS; ++j) {
        const int c = c0 + (j * 64 + lane) * V;
        if (c < dim) {
          if constexpr (V == 4) {
            float g[4];
            dev_load4<TG>(src, c, g);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[j][e] = acc[j][e] + g[e];
          } else {
            acc[j][0] = acc[j][0] + dev_load<TG>(src, c);
          }
        }
      }
    }
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
      const int c = c0 + (j * 64 + lane) * V;
      if (c < dim) {
#pragma unroll
        for (int e = 0; e < V; ++e) bad |= !dev_finite(acc[j][e]);
        if constexpr (ADD) {
          if constexpr (V == 4) {
            const float4 old = *reinterpret_cast<const float4*>(dst + c);
            acc[j][0] = old.x + acc[j][0];
            acc[j][1] = old.y + acc[j][1];
            acc[j][2] = old.z + acc[j][2];
            acc[j][3] = old.w + acc[j][3];
          } else {
            acc[j][0] = dst[c] + acc[j][0];
          }
        }
        if constexpr (V == 4) *reinterpret_cast<float4*>(dst + c) = make_float4(acc[j][0], acc[j][1], acc[j][2], acc[j][3]);
        else dst[c] = acc[j][0];
      }
    }
  }
  if (bad) dev_raise_fault(fault, tag);
}

// ---------------------------------------------------------------- argmax / top-k
// Order of rank_logits (backend.rs:184-195): value descending with +0 == -0,
// then column ascending. `before(a, b)`: a ranks ahead of b.
__device__ __forceinline__ float rank_key(float v) { return v == 0.0f ? 0.0f : v; }
__device__ __forceinline__ bool ranks_before(float va, unsigned int ia, float vb, unsigned int ib) {
  float ka = rank_key(va), kb = rank_key(vb);
  return ka > kb || (ka == kb && ia < ib);
}

__global__ void argmax_rows_kernel(const float* __restrict__ x, size_t rows, unsigned int cols,
                                   unsigned int* __restrict__ out, OmxFaultWord* fault, unsigned long long tag) {
  const int lane = threadIdx.x & 63;
  const size_t row = static_cast<size_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float* r = x + row * cols;
  // Ties go to the lowest column: strict > within a lane's ascending walk.
  float best = -INFINITY;
  unsigned int idx = 0xffffffffu;
  bool bad = false;
  for (unsigned int c = lane; c < cols; c += 64) {
    float v = r[c];
    bad |= !dev_finite(v);
    if (idx == 0xffffffffu || v > best) {
      best = v;
      idx = c;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    float ov = __shfl_xor(best, off, 64);
    unsigned int oi = __shfl_xor(idx, off, 64);
    if (oi != 0xffffffffu && (idx == 0xffffffffu || ov > best || (ov == best && oi < idx))) {
      best = ov;
      idx = oi;
    }
  }
  bad = __any(bad);
  if (lane == 0) {
    out[row] = idx;
    if (bad) dev_raise_fault(fault, tag);
  }
}

// k passes over the row; pass j picks the best element ranked after pass
// j-1's pick. NaN and +inf are refused, -inf sorts last.
__global__ void topk_rows_kernel(const float* __restrict__ x, size_t rows, unsigned int cols, unsigned int k,
                                 float* __restrict__ values, unsigned int* __restrict__ ids, OmxFaultWord* fault,
                                 unsigned long long tag) {
  const int lane = threadIdx.x & 63;
  const size_t row = static_cast<size_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float* r = x + row * cols;
  bool bad = false;
  float prev_v = 0.0f;
  unsigned int prev_i = 0;
  for (unsigned int j = 0; j < k; ++j) {
    float best = 0.0f;
    unsigned int idx = 0xffffffffu;
    for (unsigned int c = lane; c < cols; c += 64) {
      float v = r[c];
      if (j == 0) bad |= (v != v) || v == INFINITY;
      if (j > 0 && !ranks_before(prev_v, prev_i, v, c)) continue;
      if (idx == 0xffffffffu || ranks_before(v, c, best, idx)) {
        best = v;
        idx = c;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      float ov = __shfl_xor(best, off, 64);
      unsigned int oi = __shfl_xor(idx, off, 64);
      if (oi != 0xffffffffu && (idx == 0xffffffffu || ranks_before(ov, oi, best, idx))) {
        best = ov;
        idx = oi;
      }
    }
    prev_v = best;
    prev_i = idx;
    if (lane == 0) {
      values[row * k + j] = best;
      ids[row * k + j] = idx;
    }
  }
  bad = __any(bad);
  if (lane == 0 && bad) dev_raise_fault(fault, tag);
}

inline int per_for_dim(uint64_t dim) {
  const int options[] = {1, 2, 4, 8, 12, 16, 32, 64, 128};
  for (int p : options)
    if (static_cast<uint64_t>(p) * 64 >= dim) return p;
  return 0;
}

template <typename TX, typename TY>
int32_t launch_rms_fwd(omx_ctx* ctx, const void* x, const float* w, void* y, uint64_t rows, uint64_t dim, float eps,
                       unsigned long long tag) {
  dim3 grid(static_cast<unsigned>((rows + 3) / 4)), block(ROW_THREADS);
  int per = per_for_dim(dim);
#define RMS_FWD(P)                                                                                              \
  case P:                                                                                                       \
    hipLaunchKernelGGL((rms_fwd_kernel<TX, TY, P>), grid, block, 0, ctx->stream, static_cast<const TX*>(x), w, \
                       static_cast<TY*>(y), rows, static_cast<int>(dim), eps, ctx->fault, tag);                 \
    break;
  switch (per) {
    RMS_FWD(1) RMS_FWD(2) RMS_FWD(4) RMS_FWD(8) RMS_FWD(12) RMS_FWD(16) RMS_FWD(32) RMS_FWD(64) RMS_FWD(128)
    default:
      return omx_fail(ctx, OMX_UNSUPPORTED, "rms_norm_forward: dim %llu above 8192", (unsigned long long)dim);
  }
#undef RMS_FWD
  OMX_LAUNCH_CHECK(ctx, "rms_fwd_kernel");
  return OMX_OK;
}

template <typename TX, typename TG, typename TO>
int32_t launch_rms_bwd(omx_ctx* ctx, const void* x, const float* w, const void* gy, void* gx, float* gw,
                       uint64_t rows, uint64_t dim, float eps, unsigned long long tag) {
  // 32 rows per block, more when that would leave over 2048 partial rows to add.
  int rows_per_block = 32;
  while ((rows + rows_per_block - 1) / rows_per_block > 2048 && rows_per_block < (1 << 20)) rows_per_block *= 2;
  uint64_t blocks = (rows + rows_per_block - 1) / rows_per_block;
  void* partial = nullptr;
  int32_t rc = omx_workspace(ctx, (blocks + OMX_COLUMN_SUM_GROUPS) * dim * sizeof(float), &partial);
  if (rc != OMX_OK) return rc;
  // A narrow row leaves the column sum one or two workgroups: it then adds its rows in two stages.
  float* stage = static_cast<float*>(partial) + blocks * dim;
  dim3 grid(static_cast<unsigned>(blocks)), block(ROW_THREADS);
  size_t smem = 4 * dim * sizeof(float);
  int per = per_for_dim(dim);
#define RMS_BWD(P)                                                                                                  \
  case P:                                                                                                           \
    hipLaunchKernelGGL((rms_bwd_kernel<TX, TG, TO, P>), grid, block, smem, ctx->stream, static_cast<const TX*>(x), \
                       w, static_cast<const TG*>(gy), static_cast<TO*>(gx), static_cast<float*>(partial), rows,     \
                       static_cast<int>(dim), eps, rows_per_block, ctx->fault, tag);                                \
    break;
  switch (per) {
    RMS_BWD(1) RMS_BWD(2) RMS_BWD(4) RMS_BWD(8) RMS_BWD(12) RMS_BWD(16) RMS_BWD(32) RMS_BWD(64)
    default:
      return omx_fail(ctx, OMX_UNSUPPORTED, "rms_norm_backward: dim %llu above 4096", (unsigned long long)dim);
  }
#undef RMS_BWD
  OMX_LAUNCH_CHECK(ctx, "rms_bwd_kernel");
  return omx_column_sum(ctx, static_cast<const float*>(partial), gw, blocks, dim, tag, stage);
}

int32_t rms_forward_impl(omx_ctx* ctx, const char* op, uint32_t fault_op, const void* x, int32_t x_dtype,
                         const void* w, void* y, int32_t y_dtype, uint64_t rows, uint64_t dim, float eps) {
  unsigned long long tag = omx_tag(ctx, fault_op);
  (void)op;
  const float* wf = static_cast<const float*>(w);
  if (omx_rms_vec_eligible(dim, {x, w, y}))
    return omx_rms_forward_vec(ctx, x, x_dtype, nullptr, OMX_F32, wf, nullptr, y, y_dtype, rows, dim, eps, tag);
  if (x_dtype == OMX_F32 && y_dtype == OMX_F32) return launch_rms_fwd<float, float>(ctx, x, wf, y, rows, dim, eps, tag);
  if (x_dtype == OMX_F32) return launch_rms_fwd<float, unsigned short>(ctx, x, wf, y, rows, dim, eps, tag);
  if (y_dtype == OMX_F32) return launch_rms_fwd<unsigned short, float>(ctx, x, wf, y, rows, dim, eps, tag);
  return launch_rms_fwd<unsigned short, unsigned short>(ctx, x, wf, y, rows, dim, eps, tag);
}

int32_t rms_backward_impl(omx_ctx* ctx, uint32_t fault_op, const void* x, int32_t x_dtype, const void* w,
                          const void* gy, int32_t gy_dtype, void* gx, int32_t gx_dtype, void* gw, uint64_t rows,
                          uint64_t dim, float eps) {
  unsigned long long tag = omx_tag(ctx, fault_op);
  const float* wf = static_cast<const float*>(w);
  float* gwf = static_cast<float*>(gw);
  if (omx_rms_vec_eligible(dim, {x, w, gy, gx, gw}))
    return omx_rms_backward_vec(ctx, x, x_dtype, wf, gy, gy_dtype, nullptr, gx, gx_dtype, nullptr, gwf, rows, dim, eps,
                                tag);
  typedef unsigned short h16;
  const int key = (x_dtype == OMX_BF16 ? 4 : 0) | (gy_dtype == OMX_BF16 ? 2 : 0) | (gx_dtype == OMX_BF16 ? 1 : 0);
  switch (key) {
    case 0: return launch_rms_bwd<float, float, float>(ctx, x, wf, gy, gx, gwf, rows, dim, eps, tag);
    case 1: return launch_rms_bwd<float, float, h16>(ctx, x, wf, gy, gx, gwf, rows, dim, eps, tag);
    case 2: return launch_rms_bwd<float, h16, float>(ctx, x, wf, gy, gx, gwf, rows, dim, eps, tag);
    case 3: return launch_rms_bwd<float, h16, h16>(ctx, x, wf, gy, gx, gwf, rows, dim, eps, tag);
    case 4: return launch_rms_bwd<h16, float, float>(ctx, x, wf, gy, gx, gwf, rows, dim, eps, tag);
    case 5: return launch_rms_bwd<h16, float, h16>(ctx, x, wf, gy, gx, gwf, rows, dim, eps, tag);
    case 6: return launch_rms_bwd<h16, h16, float>(ctx, x, wf, gy, gx, gwf, rows, dim, eps, tag);
    default: return launch_rms_bwd<h16, h16, h16>(ctx, x, wf, gy, gx, gwf, rows, dim, eps, tag);
  }
}

bool finite_host(float v) { return v == v && v != INFINITY && v != -INFINITY; }

}  // namespace

int32_t omx_column_sum(omx_ctx* ctx, const float* partial, float* out, uint64_t blocks, uint64_t dim,
                       unsigned long long tag, float* scratch, hipEvent_t stop) {
  const unsigned col_blocks = static_cast<unsigned>((dim + 63) / 64);
  if (blocks > 4 * OMX_COLUMN_SUM_GROUPS && blocks <= OMX_COLUMN_SUM_WIDE_ROWS) {
    omx_launch_timed(ctx, column_sum_wide_kernel, dim3(col_blocks), dim3(1024), 0, nullptr, stop, partial, out,
                     static_cast<int>(blocks), static_cast<int>(dim), ctx->fault, tag);
    OMX_LAUNCH_CHECK(ctx, "column_sum_wide_kernel");
    return OMX_OK;
  }
  if (scratch && blocks > 4 * OMX_COLUMN_SUM_GROUPS) {
    // Stage 1: group g adds its contiguous share of the rows into scratch[g]; stage 2 adds the groups.
    const int per_group = static_cast<int>((blocks + OMX_COLUMN_SUM_GROUPS - 1) / OMX_COLUMN_SUM_GROUPS);
    hipLaunchKernelGGL(column_sum_groups_kernel, dim3(col_blocks, OMX_COLUMN_SUM_GROUPS), dim3(256), 0, ctx->stream,
                       partial, scratch, static_cast<int>(blocks), static_cast<int>(dim), per_group);
    OMX_LAUNCH_CHECK(ctx, "column_sum_groups_kernel");
    partial = scratch;
    blocks = OMX_COLUMN_SUM_GROUPS;
  }
  omx_launch_timed(ctx, column_sum_kernel, dim3(col_blocks), dim3(256), 0, nullptr, stop, partial, out,
                   static_cast<int>(blocks), static_cast<int>(dim), ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "column_sum_kernel");
  return OMX_OK;
}

extern "C" {

int32_t omx_rms_norm_forward(omx_ctx* ctx, const void* x, int32_t x_dtype, const void* w, void* y, int32_t y_dtype,
                             uint64_t rows, uint64_t dim, float eps) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "rms_norm_forward";
  if (!x || !w || !y) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(x_dtype) || !omx_valid_float_dtype(y_dtype))
    return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  if (rows == 0 || dim == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (!(eps == eps) || eps == INFINITY || eps == -INFINITY) return omx_fail(ctx, OMX_NON_FINITE, "%s", op);
  return rms_forward_impl(ctx, op, F_RMS_FORWARD, x, x_dtype, w, y, y_dtype, rows, dim, eps);
}

int32_t omx_rms_norm_backward(omx_ctx* ctx, const void* x, int32_t x_dtype, const void* w, const void* gy,
                              int32_t gy_dtype, void* gx, int32_t gx_dtype, void* gw, uint64_t rows, uint64_t dim,
                              float eps) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "rms_norm_backward";
  if (!x || !w || !gy || !gx || !gw) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(x_dtype) || !omx_valid_float_dtype(gy_dtype) || !omx_valid_float_dtype(gx_dtype))
    return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  if (rows == 0 || dim == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (!(eps == eps) || eps == INFINITY || eps == -INFINITY) return omx_fail(ctx, OMX_NON_FINITE, "%s", op);
  return rms_backward_impl(ctx, F_RMS_BACKWARD, x, x_dtype, w, gy, gy_dtype, gx, gx_dtype, gw, rows, dim, eps);
}

int32_t omx_rms_qk_norm_forward(omx_ctx* ctx, const void* q, const void* k, int32_t x_dtype, const void* q_weight,
                                const void* k_weight, void* q_out, void* k_out, int32_t y_dtype, uint64_t q_rows,
                                uint64_t k_rows, uint64_t dim, float eps) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "rms_qk_norm_forward";
  if (!q || !k || !q_weight || !k_weight || !q_out || !k_out)
    return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(x_dtype) || !omx_valid_float_dtype(y_dtype))
    return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  if (q_rows == 0 || k_rows == 0 || dim == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (!finite_host(eps)) return omx_fail(ctx, OMX_NON_FINITE, "%s", op);
  int32_t rc = rms_forward_impl(ctx, op, F_RMS_QK_FORWARD, q, x_dtype, q_weight, q_out, y_dtype, q_rows, dim, eps);
  if (rc != OMX_OK) return rc;
  return rms_forward_impl(ctx, op, F_RMS_QK_FORWARD, k, x_dtype, k_weight, k_out, y_dtype, k_rows, dim, eps);
}

int32_t omx_rms_qk_norm_backward(omx_ctx* ctx, const void* q, const void* k, int32_t x_dtype, const void* q_weight,
                                 const void* k_weight, const void* grad_q, const void* grad_k, int32_t gy_dtype,
                                 void* gq, void* gk, int32_t gx_dtype, void* gq_weight, void* gk_weight,
                                 uint64_t q_rows, uint64_t k_rows, uint64_t dim, float eps) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "rms_qk_norm_backward";
  if (!q || !k || !q_weight || !k_weight || !grad_q || !grad_k || !gq || !gk || !gq_weight || !gk_weight)
    return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(x_dtype) || !omx_valid_float_dtype(gy_dtype) || !omx_valid_float_dtype(gx_dtype))
    return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  if (q_rows == 0 || k_rows == 0 || dim == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (!finite_host(eps)) return omx_fail(ctx, OMX_NON_FINITE, "%s", op);
  int32_t rc = rms_backward_impl(ctx, F_RMS_QK_BACKWARD, q, x_dtype, q_weight, grad_q, gy_dtype, gq, gx_dtype,
                                 gq_weight, q_rows, dim, eps);
  if (rc != OMX_OK) return rc;
  return rms_backward_impl(ctx, F_RMS_QK_BACKWARD, k, x_dtype, k_weight, grad_k, gy_dtype, gk, gx_dtype, gk_weight,
                           k_rows, dim, eps);
}

int32_t omx_embedding_forward(omx_ctx* ctx, const void* table, int32_t table_dtype, const void* ids, void* out,
                              int32_t out_dtype, uint64_t tokens, uint64_t vocab, uint64_t dim) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "embedding_forward";
  if (!table || !ids || !out) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(table_dtype) || !omx_valid_float_dtype(out_dtype))
    return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  if (tokens == 0 || vocab == 0 || dim == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (dim > 0x7fffffffull) return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: dim does not fit in i32", op);
  unsigned long long tag = omx_tag(ctx, F_EMBEDDING_FORWARD);
  dim3 grid(static_cast<unsigned>((tokens + 3) / 4)), block(ROW_THREADS);
  const unsigned int* idp = static_cast<const unsigned int*>(ids);
#define EMB_FWD(TT, TO)                                                                                      \
  hipLaunchKernelGGL((embedding_fwd_kernel<TT, TO>), grid, block, 0, ctx->stream, static_cast<const TT*>(table), \
                     idp, static_cast<TO*>(out), tokens, vocab, static_cast<int>(dim), ctx->fault, tag)
  if (table_dtype == OMX_F32 && out_dtype == OMX_F32) EMB_FWD(float, float);
  else if (table_dtype == OMX_F32) EMB_FWD(float, unsigned short);
  else if (out_dtype == OMX_F32) EMB_FWD(unsigned short, float);
  else EMB_FWD(unsigned short, unsigned short);
#undef EMB_FWD
  OMX_LAUNCH_CHECK(ctx, "embedding_fwd_kernel");
  return OMX_OK;
}

static int32_t embedding_backward_impl(omx_ctx* ctx, const void* ids, const void* grad, int32_t grad_dtype,
                                       void* table_grad, uint64_t tokens, uint64_t vocab, uint64_t dim, bool add) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = add ? "embedding_backward_accumulate" : "embedding_backward";
  if (!ids || !grad || !table_grad) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (!omx_valid_float_dtype(grad_dtype)) return omx_fail(ctx, OMX_DTYPE, "%s: dtype must be f32 or bf16", op);
  if (tokens == 0 || vocab == 0 || dim == 0) return omx_fail(ctx, OMX_SHAPE, "%s: zero-sized axis", op);
  if (tokens > 0xfffffffeull || vocab > 0xfffffffeull || dim > 0x7fffffffull)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: axis does not fit in u32", op);
  // Workspace: counts[V], offsets[V+1], cursor[V], positions[N], sorted[N], the count of rows with
  // more than 64 tokens (one word, padded to four) and their list (at most N / 65 of them).
  const uint64_t scan_blocks = (vocab + 1023) / 1024;
  uint64_t words = vocab + (vocab + 1) + vocab + tokens + tokens + 4 + (tokens / 64 + 1) + scan_blocks + 4;
  void* ws = nullptr;
  int32_t rc = omx_workspace(ctx, words * 4, &ws);
  if (rc != OMX_OK) return rc;
  unsigned int* counts = static_cast<unsigned int*>(ws);
  unsigned int* offsets = counts + vocab;
  unsigned int* cursor = offsets + vocab + 1;
  unsigned int* positions = cursor + vocab;
  unsigned int* sorted = positions + tokens;
  unsigned int* long_count = sorted + tokens;
  unsigned int* long_rows = long_count + 4;
  unsigned int* scan_totals = long_rows + (tokens / 64 + 1);
  unsigned long long tag = omx_tag(ctx, F_EMBEDDING_BACKWARD);
  rc = omx_fill_zero(ctx, counts, vocab * 4);
  if (rc != OMX_OK) return rc;
  rc = omx_fill_zero(ctx, long_count, 16);
  if (rc != OMX_OK) return rc;
  const unsigned int* idp = static_cast<const unsigned int*>(ids);
  dim3 tgrid(static_cast<unsigned>((tokens + 255) / 256));
  // Bytes: every gradient row read once, every table row written once (rows no token names get
  // zeros); the adding form reads and writes at most one table row per token.
  const double table_rows = add ? 2.0 * static_cast<double>(tokens < vocab ? tokens : vocab) : static_cast<double>(vocab);
  OmxKernelTimer timer(ctx, OMX_K_EMBED_BWD,
                       static_cast<double>(dim) * (static_cast<double>(tokens) * (grad_dtype == OMX_BF16 ? 2.0 : 4.0) +
                                                   table_rows * 4.0));
  omx_launch_timed(ctx, count_ids_kernel, tgrid, dim3(256), 0, timer.start(), nullptr, idp, counts, tokens, vocab,
                   ctx->fault, tag);
  OMX_LAUNCH_CHECK(ctx, "count_ids_kernel");
  if (scan_blocks > 4 && scan_blocks <= SCAN_MAX_BLOCKS) {
    const dim3 sgrid(static_cast<unsigned>(scan_blocks));
    hipLaunchKernelGGL(scan_totals_kernel, sgrid, dim3(1024), 0, ctx->stream, counts, scan_totals, vocab);
    OMX_LAUNCH_CHECK(ctx, "scan_totals_kernel");
    hipLaunchKernelGGL(scan_blocks_kernel, sgrid, dim3(1024), 0, ctx->stream, counts, scan_totals, offsets, cursor, vocab);
    OMX_LAUNCH_CHECK(ctx, "scan_blocks_kernel");
  } else {
    hipLaunchKernelGGL(scan_counts_kernel, dim3(1), dim3(1024), 0, ctx->stream, counts, offsets, cursor, vocab);
    OMX_LAUNCH_CHECK(ctx, "scan_counts_kernel");
  }
  hipLaunchKernelGGL(fill_positions_kernel, tgrid, dim3(256), 0, ctx->stream, idp, cursor, positions, tokens, vocab);
  OMX_LAUNCH_CHECK(ctx, "fill_positions_kernel");
  dim3 vgrid(static_cast<unsigned>((vocab + 3) / 4));
  hipLaunchKernelGGL(sort_short_segments_kernel, vgrid, dim3(ROW_THREADS), 0, ctx->stream, offsets, positions, sorted,
                     long_count, long_rows, vocab);
  OMX_LAUNCH_CHECK(ctx, "sort_short_segments_kernel");
  hipLaunchKernelGGL(sort_long_segments_kernel, dim3(256), dim3(1024), 0, ctx->stream, offsets, positions, sorted,
                     long_count, long_rows, tokens);
  OMX_LAUNCH_CHECK(ctx, "sort_long_segments_kernel");
  const bool vec4 = dim % 4 == 0 && (reinterpret_cast<uintptr_t>(grad) & 15u) == 0 &&
                    (reinterpret_cast<uintptr_t>(table_grad) & 15u) == 0 && (grad_dtype == OMX_F32 || dim % 8 == 0);
#define EMB_BWD(TG_, V_)                                                                                         \
  do {                                                                                                          \
    if (add)                                                                                                    \
      omx_launch_timed(ctx, embedding_bwd_kernel<TG_, V_, true>, vgrid, dim3(ROW_THREADS), 0, nullptr,          \
                       timer.stop(), offsets, sorted, static_cast<const TG_*>(grad),                            \
                       static_cast<float*>(table_grad), vocab, static_cast<int>(dim), ctx->fault, tag);         \
    else                                                                                                        \
      omx_launch_timed(ctx, embedding_bwd_kernel<TG_, V_, false>, vgrid, dim3(ROW_THREADS), 0, nullptr,         \
                       timer.stop(), offsets, sorted, static_cast<const TG_*>(grad),                            \
                       static_cast<float*>(table_grad), vocab, static_cast<int>(dim), ctx->fault, tag);         \
  } while (0)
  if (grad_dtype == OMX_F32) {
    if (vec4) EMB_BWD(float, 4);
    else EMB_BWD(float, 1);
  } else {
    if (vec4) EMB_BWD(unsigned short, 4);
    else EMB_BWD(unsigned short, 1);
  }
#undef EMB_BWD
  OMX_LAUNCH_CHECK(ctx, "embedding_bwd_kernel");
  return OMX_OK;
}

int32_t omx_embedding_backward(omx_ctx* ctx, const void* ids, const void* grad, int32_t grad_dtype, void* table_grad,
                               uint64_t tokens, uint64_t vocab, uint64_t dim) {
  return embedding_backward_impl(ctx, ids, grad, grad_dtype, table_grad, tokens, vocab, dim, false);
}

int32_t omx_embedding_backward_accumulate(omx_ctx* ctx, const void* ids, const void* grad, int32_t grad_dtype,
                                          void* table_grad, uint64_t tokens, uint64_t vocab, uint64_t dim) {
  return embedding_backward_impl(ctx, ids, grad, grad_dtype, table_grad, tokens, vocab, dim, true);
}

int32_t omx_argmax_rows(omx_ctx* ctx, const void* x, uint64_t rows, uint64_t cols, void* out) {
  OMX_REQUIRE_CTX(ctx);
  if (!x || !out) return omx_fail(ctx, OMX_PLACEMENT, "argmax_rows: null device pointer");
  if (rows == 0 || cols == 0) return omx_fail(ctx, OMX_SHAPE, "argmax_rows: zero-sized axis");
  if (cols > 0xfffffffeull) return omx_fail(ctx, OMX_OUT_OF_RANGE, "argmax_rows: cols does not fit in u32");
  hipLaunchKernelGGL(argmax_rows_kernel, dim3(static_cast<unsigned>((rows + 3) / 4)), dim3(ROW_THREADS), 0,
                     ctx->stream, static_cast<const float*>(x), rows, static_cast<unsigned int>(cols),
                     static_cast<unsigned int*>(out), ctx->fault, omx_tag(ctx, F_ARGMAX));
  OMX_LAUNCH_CHECK(ctx, "argmax_rows_kernel");
  return OMX_OK;
}

int32_t omx_topk_rows(omx_ctx* ctx, const void* x, uint64_t rows, uint64_t cols, uint64_t k, void* values,
                      void* ids) {
  OMX_REQUIRE_CTX(ctx);
  if (!x || !values || !ids) return omx_fail(ctx, OMX_PLACEMENT, "topk_rows: null device pointer");
  if (rows == 0 || cols == 0) return omx_fail(ctx, OMX_SHAPE, "topk_rows: zero-sized axis");
  if (k == 0 || k > cols) return omx_fail(ctx, OMX_SHAPE, "topk_rows: k %llu outside 1..=%llu", (unsigned long long)k,
                                          (unsigned long long)cols);
  if (cols > 0xfffffffeull) return omx_fail(ctx, OMX_OUT_OF_RANGE, "topk_rows: cols does not fit in u32");
  hipLaunchKernelGGL(topk_rows_kernel, dim3(static_cast<unsigned>((rows + 3) / 4)), dim3(ROW_THREADS), 0, ctx->stream,
                     static_cast<const float*>(x), rows, static_cast<unsigned int>(cols), static_cast<unsigned int>(k),
                     static_cast<float*>(values), static_cast<unsigned int*>(ids), ctx->fault, omx_tag(ctx, F_TOPK));
  OMX_LAUNCH_CHECK(ctx, "topk_rows_kernel");
  return OMX_OK;
}

}  // extern "C"
