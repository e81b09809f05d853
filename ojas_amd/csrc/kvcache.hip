// KV-cache attention for decode (and prefill onto a non-empty cache) and the cache write.
//
// Reference: BackendModule::cached_attention_forward / kv_cache_write
// (ojas-core/src/backend.rs:2526-2565; validators ojas-core/src/shapes.rs:2758-2879; CPU
// ojas-cpu/src/kv.rs). Caches are time-major rings [B, Tcap, Hkv, D]: position j lives in slot
// j % Tcap. Query i of Tq sits at position p = kv_len - Tq + i and attends to positions
// first..=p (first = 0, or p + 1 - window); head h reads KV head h / (H / Hkv).
//
// The op is bound by reading the cache once. One wave per block walks a run of 64-key tiles for up
// to 8 query rows that share a KV head (the heads of a group and/or consecutive queries), so the
// keys and values of a group are read once for all of its query heads:
//   * the K and V tiles are loaded with 16-byte coalesced reads into LDS;
//   * scores: lane j owns key j and reads its row from LDS (row pitch dim + 4 floats, so the 16
//     lanes a clock serves hit 64 distinct banks); the query rows are LDS broadcasts;
//   * softmax statistics are kept online per row (running max and sum), exact rescaling;
//   * values: lane d owns output column d (+ 64, 128, 192), the key's weight comes from its lane
//     with a readlane.
// Each block writes one partial (unnormalised output, max, sum) per row; a second kernel merges a
// row's partials in ascending order, so the result does not depend on scheduling.
// Values read from the cache or the queries that are NaN or infinite, and scores that overflow,
// raise the deferred fault; slots no query reads are never touched.
#include <algorithm>

#include "omx_common.h"

namespace {

constexpr int KV_TILE = 64;  // keys per tile
constexpr int KV_ROWS = 8;   // query rows per block

struct KvArgs {
  const float* q;
  const void* k_cache;
  const void* v_cache;
  float* partial;  // [rows_total][nparts][dim + 2]
  float* out;
  int batch, tq, heads, kv_heads, dim, capacity, group;
  long kv_len, window, read_lo;
  int tiles_per_block, nparts;
  float scale;
  OmxFaultWord* fault;
  unsigned long long tag;
};

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// Copies tile rows [pos0, pos0 + 64) of one KV head of both caches into LDS, widened to f32; rows
// at or past kv_len become zeros. A lane's 16-byte pieces are chunk indices lane, lane + 64, ...
// of the tile's 64 * dim / 4; (key0, piece0) locates chunk `lane`. Loads are issued eight keys'
// worth at a time for each cache before any is used, so their latencies overlap.
// Returns whether a value read was not finite.
constexpr int KV_BATCH = 8;
template <typename T>
__device__ __forceinline__ bool load_tiles(const T* __restrict__ kc, const T* __restrict__ vc, float* __restrict__ kt,
                                           float* __restrict__ vt, const KvArgs& a, long base_b, int kvh, long pos0,
                                           int key0, int piece0) {
  bool bad = false;
  const int dim = a.dim, pieces = dim >> 2, kpitch = dim + 4;
  const int step_keys = 64 / pieces, step_pieces = 64 - step_keys * pieces;  // chunk index + 64
  const int slot0 = static_cast<int>(pos0 % a.capacity);
  const int live = static_cast<int>(min(static_cast<long>(KV_TILE), a.kv_len - pos0));
  int key = key0, piece = piece0;
  for (int done = 0; done < pieces; done += KV_BATCH) {  // a lane has `pieces` chunks per tile
    float kv[KV_BATCH][4], vv[KV_BATCH][4];
    int at_key[KV_BATCH], at_d[KV_BATCH];
#pragma unroll
    for (int i = 0; i < KV_BATCH; ++i) {
      at_key[i] = key;
      at_d[i] = piece << 2;
#pragma unroll
      for (int e = 0; e < 4; ++e) kv[i][e] = vv[i][e] = 0.0f;
      if (done + i < pieces && key < live) {
        int slot = slot0 + key;  // the positions of a tile wrap the ring at most once
        slot = slot >= a.capacity ? slot - a.capacity : slot;
        const size_t off = static_cast<size_t>(((base_b + slot) * a.kv_heads + kvh) * dim + at_d[i]);
        dev_load4(kc, off, kv[i]);
        dev_load4(vc, off, vv[i]);
      }
      key += step_keys;
      piece += step_pieces;
      if (piece >= pieces) {
        piece -= pieces;
        ++key;
      }
    }
#pragma unroll
    for (int i = 0; i < KV_BATCH; ++i) {
      if (done + i < pieces) {
        bad |= !(dev_finite(kv[i][0]) && dev_finite(kv[i][1]) && dev_finite(kv[i][2]) && dev_finite(kv[i][3]) &&
                 dev_finite(vv[i][0]) && dev_finite(vv[i][1]) && dev_finite(vv[i][2]) && dev_finite(vv[i][3]));
        *reinterpret_cast<float4*>(kt + at_key[i] * kpitch + at_d[i]) = float4{kv[i][0], kv[i][1], kv[i][2], kv[i][3]};
        *reinterpret_cast<float4*>(vt + at_key[i] * dim + at_d[i]) = float4{vv[i][0], vv[i][1], vv[i][2], vv[i][3]};
      }
    }
  }
  return bad;
}

template <typename T, int NPL>  // NPL: output columns per lane (dim <= 64 * NPL)
__global__ __launch_bounds__(64) void cached_attention_partial_kernel(KvArgs a) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int lane = threadIdx.x;
  const int part = blockIdx.x, chunk = blockIdx.y;
  const int b = blockIdx.z / a.kv_heads, kvh = blockIdx.z - b * a.kv_heads;
  const int dim = a.dim, kpitch = dim + 4;
  float* kt = lds;                        // [64][dim + 4]
  float* vt = kt + KV_TILE * kpitch;      // [64][dim]
  float* qs = vt + KV_TILE * dim;         // [KV_ROWS][dim]
  const int rows_all = a.tq * a.group;
  const int row0 = chunk * KV_ROWS;
  const int rows = min(KV_ROWS, rows_all - row0);
  bool bad = false;

  // Row r of this block: query i = (row0 + r) / group, head kvh * group + (row0 + r) % group.
  long p_of[KV_ROWS], first_of[KV_ROWS];
  long out_row[KV_ROWS];
#pragma unroll
  for (int r = 0; r < KV_ROWS; ++r) {
    const int rr = min(row0 + r, rows_all - 1);
    const int i = rr / a.group, h = kvh * a.group + (rr - i * a.group);
    p_of[r] = a.kv_len - a.tq + i;
    first_of[r] = a.window > 0 ? max(0l, p_of[r] + 1 - a.window) : 0l;
    out_row[r] = (static_cast<long>(b) * a.tq + i) * a.heads + h;
  }
  for (int c = lane; c < rows * dim; c += 64) {
    const int r = c / dim, d = c - r * dim;
    const float v = a.q[out_row[r] * dim + d];
    bad |= !dev_finite(v);
    qs[r * dim + d] = v;
  }

  float m[KV_ROWS], l[KV_ROWS], acc[KV_ROWS][NPL];
#pragma unroll
  for (int r = 0; r < KV_ROWS; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.0f;
#pragma unroll
    for (int n = 0; n < NPL; ++n) acc[r][n] = 0.0f;
  }

  const long base_b = static_cast<long>(b) * a.capacity;
  const int key0 = lane / (dim >> 2), piece0 = lane - key0 * (dim >> 2);
  const T* kc = static_cast<const T*>(a.k_cache);
  const T* vc = static_cast<const T*>(a.v_cache);
  for (int t = 0; t < a.tiles_per_block; ++t) {
    const long pos0 = a.read_lo + (static_cast<long>(part) * a.tiles_per_block + t) * KV_TILE;
    if (pos0 >= a.kv_len) break;
    __syncthreads();  // the previous tile has been consumed
    bad |= load_tiles<T>(kc, vc, kt, vt, a, base_b, kvh, pos0, key0, piece0);
    __syncthreads();

    // Scores of key `lane` against every row.
    float s[KV_ROWS];
#pragma unroll
    for (int r = 0; r < KV_ROWS; ++r) s[r] = 0.0f;
    const float* krow = kt + lane * kpitch;
    for (int d = 0; d < dim; d += 4) {
      const float4 kv = *reinterpret_cast<const float4*>(krow + d);
#pragma unroll
      for (int r = 0; r < KV_ROWS; ++r) {
        if (r < rows) {
          const float4 qv = *reinterpret_cast<const float4*>(qs + r * dim + d);
          s[r] = fmaf(qv.x, kv.x, s[r]);
          s[r] = fmaf(qv.y, kv.y, s[r]);
          s[r] = fmaf(qv.z, kv.z, s[r]);
          s[r] = fmaf(qv.w, kv.w, s[r]);
        }
      }
    }
    const long pos = pos0 + lane;
    float p[KV_ROWS];
#pragma unroll
    for (int r = 0; r < KV_ROWS; ++r) {
      p[r] = 0.0f;
      if (r < rows) {
        const bool seen = pos <= p_of[r] && pos >= first_of[r];
        const float sc = s[r] * a.scale;
        bad |= seen && !dev_finite(sc);
        const float masked = seen ? sc : -INFINITY;
        const float tile_max = wave_max(masked);
        const float m_new = fmaxf(m[r], tile_max);
        if (m_new > -INFINITY) {  // uniform across the wave
          const float corr = expf(m[r] - m_new);  // 0 when this is the row's first visible tile
          p[r] = expf(masked - m_new);            // 0 for a hidden key
          l[r] = l[r] * corr + wave_sum(p[r]);
#pragma unroll
          for (int n = 0; n < NPL; ++n) acc[r][n] *= corr;
          m[r] = m_new;
        }
      }
    }
    // Values: out[r][d] += p[r][key] * V[key][d].
    const int keys = static_cast<int>(min(static_cast<long>(KV_TILE), a.kv_len - pos0));
    for (int j = 0; j < keys; ++j) {
      float v[NPL];
#pragma unroll
      for (int n = 0; n < NPL; ++n) v[n] = (lane + 64 * n < dim) ? vt[j * dim + lane + 64 * n] : 0.0f;
#pragma unroll
      for (int r = 0; r < KV_ROWS; ++r) {
        if (r < rows) {
          const float w = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, p[r]), j));
#pragma unroll
          for (int n = 0; n < NPL; ++n) acc[r][n] = fmaf(w, v[n], acc[r][n]);
        }
      }
    }
  }

  const int width = dim + 2;
#pragma unroll
  for (int r = 0; r < KV_ROWS; ++r) {
    if (r < rows) {
      float* dst = a.partial + (out_row[r] * a.nparts + part) * width;
#pragma unroll
      for (int n = 0; n < NPL; ++n)
        if (lane + 64 * n < dim) dst[lane + 64 * n] = acc[r][n];
      if (lane == 0) {
        dst[dim] = m[r];
        dst[dim + 1] = l[r];
      }
    }
  }
  if (bad) dev_raise_fault(a.fault, a.tag);
}

// ---- the fast path: head_dim a power of two ----
// A key's row is read by LPK = dim / 4 adjacent lanes, 16 bytes each, so one load instruction
// covers 64 / LPK keys with whole cache lines and needs no LDS. A tile is 16 such rounds; all 32
// loads of a tile (K and V) are issued before the first is used. Scores are reduced across the LPK
// lanes with DPP adds (bpermutes above 16 lanes); each lane group keeps the output columns of its
// own keys and the groups are summed once, at the end of the block.
constexpr int KG_ROUNDS = 16;
constexpr int KG_ROWS = 4;  // query rows per block

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// Sum over the LPK adjacent lanes that hold one key; every one of them receives the total.
template <int LPK>
__device__ __forceinline__ float group_sum(float v) {
  if constexpr (LPK >= 2) v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
  if constexpr (LPK >= 4) v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
  if constexpr (LPK >= 8) v = dpp_add<0x141>(v);  // row_half_mirror
  if constexpr (LPK >= 16) v = dpp_add<0x140>(v); // row_mirror
  if constexpr (LPK >= 32) v += __shfl_xor(v, 16);
  if constexpr (LPK >= 64) v += __shfl_xor(v, 32);
  return v;
}
// Combines the 64 / LPK lane groups (lanes that differ in the bits at and above LPK).
template <int LPK, typename F>
__device__ __forceinline__ float across_groups(float v, F f) {
#pragma unroll
  for (int o = LPK; o < 64; o <<= 1) v = f(v, __shfl_xor(v, o));
  return v;
}

template <typename T, int LPK>
__global__ __launch_bounds__(64) void cached_attention_group_kernel(KvArgs a) {
  constexpr int G = 64 / LPK;               // keys per round
  constexpr int TILE = KG_ROUNDS * G;       // keys per tile
  constexpr float LOG2E = 1.4426950408889634f;
  const int lane = threadIdx.x;
  const int part = blockIdx.x, chunk = blockIdx.y;
  const int b = blockIdx.z / a.kv_heads, kvh = blockIdx.z - b * a.kv_heads;
  const int g = lane / LPK, d0 = (lane % LPK) * 4;
  constexpr int dim = LPK * 4;
  const int rows_all = a.tq * a.group;
  const int row0 = chunk * KG_ROWS;
  const int rows = min(KG_ROWS, rows_all - row0);
  bool bad = false;

  long p_of[KG_ROWS], first_of[KG_ROWS], out_row[KG_ROWS];
  float q[KG_ROWS][4];
#pragma unroll
  for (int r = 0; r < KG_ROWS; ++r) {
    const int rr = min(row0 + r, rows_all - 1);
    const int i = rr / a.group, h = kvh * a.group + (rr - i * a.group);
    p_of[r] = a.kv_len - a.tq + i;
    first_of[r] = a.window > 0 ? max(0l, p_of[r] + 1 - a.window) : 0l;
    out_row[r] = (static_cast<long>(b) * a.tq + i) * a.heads + h;
    const float4 qv = *reinterpret_cast<const float4*>(a.q + out_row[r] * dim + d0);
    q[r][0] = qv.x; q[r][1] = qv.y; q[r][2] = qv.z; q[r][3] = qv.w;
    bad |= !(dev_finite(qv.x) && dev_finite(qv.y) && dev_finite(qv.z) && dev_finite(qv.w));
  }
  // Scores are kept in the exp2 domain: s * scale * log2(e).
  const float scale2 = a.scale * LOG2E;
  float m[KG_ROWS], l[KG_ROWS], acc[KG_ROWS][4];
#pragma unroll
  for (int r = 0; r < KG_ROWS; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.0f;
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[r][e] = 0.0f;
  }

  const long base_b = static_cast<long>(b) * a.capacity;
  const T* kc = static_cast<const T*>(a.k_cache);
  const T* vc = static_cast<const T*>(a.v_cache);
  const long span_keys = static_cast<long>(a.tiles_per_block) * KV_TILE;  // the host counts 64-key tiles
  const long part_lo = a.read_lo + part * span_keys;
  const long part_hi = min(a.kv_len, part_lo + span_keys);
  for (long pos0 = part_lo; pos0 < part_hi; pos0 += TILE) {
    const int slot0 = static_cast<int>(pos0 % a.capacity);
    float kv[KG_ROUNDS][4], vv[KG_ROUNDS][4];
#pragma unroll
    for (int i = 0; i < KG_ROUNDS; ++i) {
      // Every lane loads, with no branch around the load, so that the compiler issues all 32
      // before it waits for the first: a key past the end of the part re-reads the tile's first
      // key (a slot this block reads anyway), and its weight below is exactly zero.
      const int key = (pos0 + i * G + g < part_hi) ? i * G + g : 0;
      int slot = slot0 + key;  // a tile wraps the ring at most once
      slot = slot >= a.capacity ? slot - a.capacity : slot;
      const size_t off = static_cast<size_t>(((base_b + slot) * a.kv_heads + kvh) * dim + d0);
      dev_load4(kc, off, kv[i]);
      dev_load4(vc, off, vv[i]);
    }
#pragma unroll
    for (int r = 0; r < KG_ROWS; ++r) {
      if (r < rows) {  // uniform
        float s[KG_ROUNDS];
        float tile_max = -INFINITY;
#pragma unroll
        for (int i = 0; i < KG_ROUNDS; ++i) {
          float dot = q[r][0] * kv[i][0];
          dot = fmaf(q[r][1], kv[i][1], dot);
          dot = fmaf(q[r][2], kv[i][2], dot);
          dot = fmaf(q[r][3], kv[i][3], dot);
          dot = group_sum<LPK>(dot);
          const long pos = pos0 + i * G + g;
          const bool seen = pos < part_hi && pos <= p_of[r] && pos >= first_of[r];
          const float sc = dot * scale2;
          bad |= seen && !dev_finite(sc);
          s[i] = seen ? sc : -INFINITY;
          tile_max = fmaxf(tile_max, s[i]);
        }
        tile_max = across_groups<LPK>(tile_max, [](float x, float y) { return fmaxf(x, y); });
        const float m_new = fmaxf(m[r], tile_max);
        if (m_new > -INFINITY) {  // uniform: the row sees a key in this tile or saw one before
          const float corr = __builtin_amdgcn_exp2f(m[r] - m_new);
          float sum = 0.0f;
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[r][e] *= corr;
#pragma unroll
          for (int i = 0; i < KG_ROUNDS; ++i) {
            const float p = __builtin_amdgcn_exp2f(s[i] - m_new);  // 0 for a hidden key
            sum += p;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[r][e] = fmaf(p, vv[i][e], acc[r][e]);
          }
          l[r] = l[r] * corr + sum;  // this lane group's keys only
          m[r] = m_new;
        }
      }
    }
#pragma unroll
    for (int i = 0; i < KG_ROUNDS; ++i)
      bad |= !(dev_finite(kv[i][0]) && dev_finite(kv[i][1]) && dev_finite(kv[i][2]) && dev_finite(kv[i][3]) &&
               dev_finite(vv[i][0]) && dev_finite(vv[i][1]) && dev_finite(vv[i][2]) && dev_finite(vv[i][3]));
  }

  const int width = dim + 2;
  constexpr float LN2 = 0.6931471805599453f;
#pragma unroll
  for (int r = 0; r < KG_ROWS; ++r) {
    if (r < rows) {
      const float total = across_groups<LPK>(l[r], [](float x, float y) { return x + y; });
      float* dst = a.partial + (out_row[r] * a.nparts + part) * width;
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[r][e] = across_groups<LPK>(acc[r][e], [](float x, float y) { return x + y; });
      if (g == 0) *reinterpret_cast<float4*>(dst + d0) = float4{acc[r][0], acc[r][1], acc[r][2], acc[r][3]};
      if (lane == 0) {
        dst[dim] = m[r] * LN2;  // the merge works in the natural-log domain
        dst[dim + 1] = total;
      }
    }
  }
  if (bad) dev_raise_fault(a.fault, a.tag);
}

// One wave per output row: merges the row's partials, lowest part first.
template <int NPL>
__global__ __launch_bounds__(64) void cached_attention_merge_kernel(KvArgs a, long rows_total) {
  const long row = blockIdx.x;
  if (row >= rows_total) return;
  const int lane = threadIdx.x, dim = a.dim, width = dim + 2;
  const float* src = a.partial + row * a.nparts * width;
  float top = -INFINITY;
  for (int s = 0; s < a.nparts; ++s) top = fmaxf(top, src[s * width + dim]);
  float total = 0.0f, acc[NPL];
#pragma unroll
  for (int n = 0; n < NPL; ++n) acc[n] = 0.0f;
  for (int s = 0; s < a.nparts; ++s) {
    const float ms = src[s * width + dim];
    if (ms == -INFINITY) continue;  // a part in which this row saw no key
    const float w = expf(ms - top);
    total = fmaf(src[s * width + dim + 1], w, total);
#pragma unroll
    for (int n = 0; n < NPL; ++n)
      if (lane + 64 * n < dim) acc[n] = fmaf(src[s * width + lane + 64 * n], w, acc[n]);
  }
  const bool ok = dev_finite(total) && total > 0.0f;
  const float inv = 1.0f / total;
#pragma unroll
  for (int n = 0; n < NPL; ++n)
    if (lane + 64 * n < dim) a.out[row * dim + lane + 64 * n] = acc[n] * inv;
  if (!ok) dev_raise_fault(a.fault, a.tag);
}

// All-or-nothing cache write: the first kernel scans src, the second copies unless the scan refused.
__global__ void kv_scan_kernel(const float* __restrict__ src, size_t n, unsigned int* __restrict__ refuse,
                               OmxFaultWord* fault, unsigned long long tag) {
  bool bad = false;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * blockDim.x)
    bad |= !dev_finite(src[i]);
  if (bad) {
    atomicOr(refuse, 1u);
    dev_raise_fault(fault, tag);
  }
}
template <typename T>
__global__ void kv_write_kernel(T* __restrict__ cache, const float* __restrict__ src, size_t batch, size_t capacity,
                                size_t step, size_t tn, size_t at, const unsigned int* __restrict__ refuse) {
  if (*refuse) return;
  const size_t n = batch * tn * step;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t e = i % step, row = i / step;
    const size_t j = row % tn, b = row / tn;
    dev_store(cache, (b * capacity + (at + j) % capacity) * step + e, src[i]);
  }
}

template <typename T, int LPK, int NPL>
int32_t launch_group(omx_ctx* ctx, const KvArgs& a, dim3 grid, long rows_total) {
  hipLaunchKernelGGL((cached_attention_group_kernel<T, LPK>), grid, dim3(64), 0, ctx->stream, a);
  OMX_LAUNCH_CHECK(ctx, "cached_attention_group_kernel");
  hipLaunchKernelGGL((cached_attention_merge_kernel<NPL>), dim3(static_cast<unsigned>(rows_total)), dim3(64), 0,
                     ctx->stream, a, rows_total);
  OMX_LAUNCH_CHECK(ctx, "cached_attention_merge_kernel");
  return OMX_OK;
}

template <typename T>
int32_t launch_attention(omx_ctx* ctx, const KvArgs& a, dim3 grid, size_t lds_bytes, long rows_total) {
  auto run = [&](auto kernel, auto merge) -> int32_t {
    if (lds_bytes > 64 * 1024)  // beyond the default limit: ask for it (cheap, and idempotent)
      OMX_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    hipLaunchKernelGGL(kernel, grid, dim3(64), lds_bytes, ctx->stream, a);
    OMX_LAUNCH_CHECK(ctx, "cached_attention_partial_kernel");
    hipLaunchKernelGGL(merge, dim3(static_cast<unsigned>(rows_total)), dim3(64), 0, ctx->stream, a, rows_total);
    OMX_LAUNCH_CHECK(ctx, "cached_attention_merge_kernel");
    return OMX_OK;
  };
  if (a.dim <= 64) return run(&cached_attention_partial_kernel<T, 1>, &cached_attention_merge_kernel<1>);
  if (a.dim <= 128) return run(&cached_attention_partial_kernel<T, 2>, &cached_attention_merge_kernel<2>);
  return run(&cached_attention_partial_kernel<T, 4>, &cached_attention_merge_kernel<4>);
}

}  // namespace

extern "C" {

int32_t omx_cached_attention_forward(omx_ctx* ctx, const void* q, const void* k_cache, const void* v_cache,
                                     int32_t cache_dtype, void* out, uint64_t batch, uint64_t tq, uint64_t heads,
                                     uint64_t kv_heads, uint64_t head_dim, uint64_t capacity, uint64_t kv_len,
                                     uint64_t window) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "cached_attention_forward";
  if (!q || !k_cache || !v_cache || !out) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (cache_dtype != OMX_F32 && cache_dtype != OMX_BF16) return omx_fail(ctx, OMX_DTYPE, "%s: cache dtype", op);
  if (batch == 0 || tq == 0 || heads == 0 || head_dim == 0 || capacity == 0 || kv_heads == 0)
    return omx_fail(ctx, OMX_SHAPE, "%s: zero dimension in q or cache", op);
  if (heads % kv_heads != 0)
    return omx_fail(ctx, OMX_SHAPE, "%s: %llu query heads over %llu kv heads", op, (unsigned long long)heads,
                    (unsigned long long)kv_heads);
  if (kv_len < tq)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: kv_len %llu is below the %llu new positions", op,
                    (unsigned long long)kv_len, (unsigned long long)tq);
  if (window >= kv_len) window = 0;  // a window that covers every position is no window
  uint64_t span = kv_len;
  if (window != 0 && tq + (window - 1) < kv_len) span = tq + (window - 1);
  if (span > capacity)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: the %llu positions read up to kv_len %llu exceed cache capacity %llu",
                    op, (unsigned long long)span, (unsigned long long)kv_len, (unsigned long long)capacity);
  if (head_dim % 4 != 0 || head_dim > 256)
    return omx_fail(ctx, OMX_UNSUPPORTED_HEAD_DIM, "%s: head_dim %llu (a multiple of 4 up to 256)", op,
                    (unsigned long long)head_dim);
  const uint64_t rows_total = batch * tq * heads;
  if (batch * kv_heads > 65535 || rows_total > 0x7fffffffull || capacity > 0x7fffffffull || kv_len > (1ull << 40))
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: extent too large", op);

  KvArgs a;
  a.q = static_cast<const float*>(q);
  a.k_cache = k_cache;
  a.v_cache = v_cache;
  a.out = static_cast<float*>(out);
  a.batch = static_cast<int>(batch);
  a.tq = static_cast<int>(tq);
  a.heads = static_cast<int>(heads);
  a.kv_heads = static_cast<int>(kv_heads);
  a.dim = static_cast<int>(head_dim);
  a.capacity = static_cast<int>(capacity);
  a.group = static_cast<int>(heads / kv_heads);
  a.kv_len = static_cast<long>(kv_len);
  a.window = static_cast<long>(window);
  a.read_lo = static_cast<long>(kv_len - span);
  a.scale = 1.0f / std::sqrt(static_cast<float>(head_dim));
  a.fault = ctx->fault;
  a.tag = omx_tag(ctx, F_CACHED_ATTENTION);

  // Power-of-two head dims take the lane-group kernel; others the LDS-tiled one. The option
  // "kv_attention" = 1 forces the LDS-tiled kernel (for tests and measurements).
  const bool grouped = (head_dim & (head_dim - 1)) == 0 && ctx->kv_attention_mode != 1;
  const uint64_t block_rows = grouped ? KG_ROWS : KV_ROWS;
  const uint64_t rows_per_group = tq * (heads / kv_heads);
  const uint64_t chunks = (rows_per_group + block_rows - 1) / block_rows;
  if (chunks > 65535) return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: too many query rows per KV head", op);
  const uint64_t tiles = (span + KV_TILE - 1) / KV_TILE;
  // Enough blocks to fill the chip several times over, but no more parts than tiles.
  uint64_t parts = (8ull * ctx->cu_count + batch * kv_heads * chunks - 1) / (batch * kv_heads * chunks);
  parts = std::max<uint64_t>(1, std::min<uint64_t>(parts, tiles));
  a.tiles_per_block = static_cast<int>((tiles + parts - 1) / parts);
  a.nparts = static_cast<int>((tiles + a.tiles_per_block - 1) / a.tiles_per_block);

  void* ws = nullptr;
  int32_t rc = omx_workspace(ctx, rows_total * a.nparts * (head_dim + 2) * sizeof(float), &ws);
  if (rc != OMX_OK) return rc;
  a.partial = static_cast<float*>(ws);
  const size_t lds_bytes = (KV_TILE * (head_dim + 4) + KV_TILE * head_dim + KV_ROWS * head_dim) * sizeof(float);
  dim3 grid(static_cast<unsigned>(a.nparts), static_cast<unsigned>(chunks), static_cast<unsigned>(batch * kv_heads));
  const long nrows = static_cast<long>(rows_total);
  if (grouped) {
    const bool f32 = cache_dtype == OMX_F32;
    switch (head_dim) {
#define OMX_KV_CASE(DIM, NPL)                                                                     \
  case DIM:                                                                                       \
    return f32 ? launch_group<float, DIM / 4, NPL>(ctx, a, grid, nrows)                           \
               : launch_group<unsigned short, DIM / 4, NPL>(ctx, a, grid, nrows);
      OMX_KV_CASE(4, 1)
      OMX_KV_CASE(8, 1)
      OMX_KV_CASE(16, 1)
      OMX_KV_CASE(32, 1)
      OMX_KV_CASE(64, 1)
      OMX_KV_CASE(128, 2)
      OMX_KV_CASE(256, 4)
#undef OMX_KV_CASE
      default:
        break;
    }
  }
  if (cache_dtype == OMX_F32) return launch_attention<float>(ctx, a, grid, lds_bytes, nrows);
  return launch_attention<unsigned short>(ctx, a, grid, lds_bytes, nrows);
}

int32_t omx_kv_cache_write(omx_ctx* ctx, void* cache, int32_t cache_dtype, const void* src, uint64_t batch,
                           uint64_t capacity, uint64_t kv_heads, uint64_t head_dim, uint64_t tn, uint64_t at) {
  OMX_REQUIRE_CTX(ctx);
  const char* op = "kv_cache_write";
  if (!cache || !src) return omx_fail(ctx, OMX_PLACEMENT, "%s: null device pointer", op);
  if (cache_dtype != OMX_F32 && cache_dtype != OMX_BF16) return omx_fail(ctx, OMX_DTYPE, "%s: cache dtype", op);
  if (batch == 0 || capacity == 0 || kv_heads == 0 || head_dim == 0 || tn == 0)
    return omx_fail(ctx, OMX_SHAPE, "%s: zero dimension in cache or src", op);
  if (at + tn < at)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: at %llu + %llu overflows", op, (unsigned long long)at,
                    (unsigned long long)tn);
  if (tn > capacity)
    return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: %llu positions exceed capacity %llu", op, (unsigned long long)tn,
                    (unsigned long long)capacity);
  void* ws = nullptr;
  int32_t rc = omx_workspace(ctx, 256, &ws);
  if (rc != OMX_OK) return rc;
  unsigned int* refuse = static_cast<unsigned int*>(ws);
  rc = omx_fill_zero(ctx, refuse, 4);
  if (rc != OMX_OK) return rc;
  const size_t step = kv_heads * head_dim, n = batch * tn * step;
  const unsigned blocks = static_cast<unsigned>(std::min<size_t>((n + 255) / 256, 8192));
  hipLaunchKernelGGL(kv_scan_kernel, dim3(blocks), dim3(256), 0, ctx->stream, static_cast<const float*>(src), n, refuse,
                     ctx->fault, omx_tag(ctx, F_KV_CACHE_WRITE));
  OMX_LAUNCH_CHECK(ctx, "kv_scan_kernel");
  if (cache_dtype == OMX_F32)
    hipLaunchKernelGGL((kv_write_kernel<float>), dim3(blocks), dim3(256), 0, ctx->stream, static_cast<float*>(cache),
                       static_cast<const float*>(src), batch, capacity, step, tn, at, refuse);
  else
    hipLaunchKernelGGL((kv_write_kernel<unsigned short>), dim3(blocks), dim3(256), 0, ctx->stream,
                       static_cast<unsigned short*>(cache), static_cast<const float*>(src), batch, capacity, step, tn,
                       at, refuse);
  OMX_LAUNCH_CHECK(ctx, "kv_write_kernel");
  return OMX_OK;
}

}  // extern "C"
