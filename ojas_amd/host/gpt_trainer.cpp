// Host-side training-step driver above the C ABI (see include/ojas_gpt.h).
//
// Orchestration only: every tensor operation is one omx_* call, in the order
// the reference's tape would replay the same graph (forward in program order,
// backward in reverse with gradient fan-in added later-consumer-first,
// ojas-autograd/src/tape.rs:2004-2466,2565-2591), then the step of
// ojas-model/src/trainer.rs:754-1046: clip_grad_norm (sync point), adamw_step,
// sync + one scalar readback.
//
// All buffers are allocated once at creation: parameters, gradients and AdamW
// moments live in flat f32 arenas (one clip pass and one AdamW pass cover every
// tensor), the bf16 tier keeps a bf16 mirror of the parameters that AdamW
// refreshes, and saved activations have one slot per layer.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "ojas_gpt.h"

namespace {

constexpr uint64_t kAlign = 64;  // elements; keeps every tensor 256-byte aligned in both arenas

struct Slot {
  uint64_t offset, len;
};

}  // namespace

struct ogpt {
  omx_ctx* ctx = nullptr;
  ogpt_config c{};
  uint64_t N = 0, P = 0;  // tokens per batch, padded parameter count
  std::vector<Slot> slots;
  int32_t AD = OMX_F32;  // activation / operand dtype
  uint64_t asz = 4;
  uint64_t steps = 0;
  // omx_adamw_step_bounded's flag word, and which ranges it has covered since they were last
  // written from outside: nothing, the tables and norms (hybrid steps), or every parameter.
  void* unbounded = nullptr;  // the word after the loss, so one readback fetches both
  enum Tracked { kNone = 0, kHybrid = 1, kFull = 2 };
  int tracked = kNone;
  uint32_t flag_seen = 1;  // the flag as the last step's readback saw it (valid while tracked != kNone)
  uint64_t device_bytes = 0;
  std::vector<void*> owned;

  float *p32 = nullptr, *g32 = nullptr, *m1 = nullptr, *m2 = nullptr;
  uint64_t adamw_end = 0;  // the tables and the norm weights are arena elements [0, adamw_end)
  void* p16 = nullptr;
  uint32_t *ids = nullptr, *targets = nullptr, *positions = nullptr;
  float* loss = nullptr;

  // Per-layer saved activations.
  struct Layer {
    float *x, *x1;                          // residual stream (f32)
    void *h1, *q, *k, *v, *a, *ap, *h2, *u, *g;  // AD
    void* apr = nullptr;  // rounding residual of ap (fused bf16 attention only)
    float* lse;
  };
  std::vector<Layer> layers;
  float* x_final = nullptr;  // residual stream after the last layer
  void* hf = nullptr;        // final norm output (AD)
  // Scratch.
  float *e_tok = nullptr, *e_pos = nullptr;
  void *t_a = nullptr, *t_b = nullptr;       // [N,d] AD
  void *gu = nullptr, *gg = nullptr;         // [N,mlp] AD
  void *gq = nullptr, *gk = nullptr, *gv = nullptr, *ga = nullptr;  // [N,d] AD
  void* gy16 = nullptr;                      // AD copy of a residual-stream gradient
  // bf16 tier with head_dim 64: q, k and v are column blocks of one [N, 3d] projection output
  // (the three weights are adjacent in the arena, so they are one [3d, d] matrix), attention
  // runs time-major on those blocks, and their gradients are the blocks of `gqkv`.
  bool fused_qkv = false;
  void* gqkv = nullptr;                      // [N,3d] AD
  // With the fused projection, the four weight gradients of every layer wait until the backward's
  // end: each layer's inputs (h1, ap, h2, g) and output gradients (below) sit at a fixed stride in
  // stacked buffers, the gradient arena holds the layers at a fixed stride too, and four strided-
  // batch products over the layers replace 4 x layers split-K products.
  bool deferred_dw = false;
  void *h1_all = nullptr, *ap_all = nullptr, *h2_all = nullptr, *g_all = nullptr;
  void *gu_all = nullptr, *gqkv_all = nullptr;  // [layers][N,mlp], [layers][N,3d] AD
  void *gyd_all = nullptr, *gyo_all = nullptr;  // residual-stream gradient copies feeding down / o: [layers][N,d] AD
  float *gres = nullptr, *gres1 = nullptr, *gt = nullptr, *gh = nullptr;  // [N,d] f32
  void* ghf = nullptr;                       // [N,d] AD

  // Parameter views.
  const void* w(uint64_t i) const {
    return AD == OMX_BF16 ? static_cast<const void*>(static_cast<const uint16_t*>(p16) + slots[i].offset)
                          : static_cast<const void*>(p32 + slots[i].offset);
  }
  const float* w32(uint64_t i) const { return p32 + slots[i].offset; }
  float* g(uint64_t i) const { return g32 + slots[i].offset; }
  uint64_t li(uint64_t l, uint64_t which) const { return 2 + l * 8 + which; }
  uint64_t nf() const { return 2 + static_cast<uint64_t>(c.layers) * 8; }
};

namespace {

#define TRY(expr)                    \
  do {                               \
    int32_t rc_ = (expr);            \
    if (rc_ != OMX_OK) return rc_;   \
  } while (0)

int32_t alloc(ogpt* t, uint64_t bytes, void** out) {
  TRY(omx_alloc(t->ctx, bytes, out));
  t->owned.push_back(*out);
  t->device_bytes += bytes;
  return OMX_OK;
}
template <typename T>
int32_t alloc_t(ogpt* t, uint64_t count, T** out) {
  void* p = nullptr;
  TRY(alloc(t, count * sizeof(T), &p));
  *out = static_cast<T*>(p);
  return OMX_OK;
}
int32_t alloc_act(ogpt* t, uint64_t count, void** out) { return alloc(t, count * t->asz, out); }

// AD copy of an f32 tensor: the f32 tier aliases it, the bf16 tier rounds it.
int32_t to_operand(ogpt* t, const float* src, void* scratch, uint64_t n, const void** out) {
  if (t->AD == OMX_F32) {
    *out = src;
    return OMX_OK;
  }
  TRY(omx_to_bf16(t->ctx, src, scratch, n));
  *out = scratch;
  return OMX_OK;
}

int32_t forward(ogpt* t) {
  omx_ctx* ctx = t->ctx;
  const ogpt_config& c = t->c;
  const uint64_t N = t->N, d = c.d_model, M = c.mlp, B = c.batch, T = c.ctx, H = c.heads, D = c.head_dim;
  const int32_t AD = t->AD;
  const float eps = 1e-6f;
  TRY(omx_embedding_forward(ctx, t->w32(0), OMX_F32, t->ids, t->e_tok, OMX_F32, N, c.vocab, d));
  TRY(omx_embedding_forward(ctx, t->w32(1), OMX_F32, t->positions, t->e_pos, OMX_F32, N, T, d));
  // Every residual add is fused with the norm that reads its sum: the sum (f32 residual stream)
  // and the normed operand leave one kernel.
  {
    float* x = t->layers.empty() ? t->x_final : t->layers[0].x;
    void* h = t->layers.empty() ? t->hf : t->layers[0].h1;
    const float* nw = t->w32(t->layers.empty() ? t->nf() : t->li(0, 0));
    TRY(omx_residual_add_rms_norm_forward(ctx, t->e_tok, OMX_F32, t->e_pos, OMX_F32, nw, x, h, AD, N, d, eps));
  }
  for (uint32_t l = 0; l < c.layers; ++l) {
    ogpt::Layer& A = t->layers[l];
    const bool last = l + 1 == c.layers;
    float* x_next = last ? t->x_final : t->layers[l + 1].x;
    void* h_next = last ? t->hf : t->layers[l + 1].h1;
    const float* next_norm = t->w32(last ? t->nf() : t->li(l + 1, 0));
    if (t->fused_qkv) {
      TRY(omx_linear_forward(ctx, A.h1, AD, t->w(t->li(l, 1)), AD, A.q, AD, N, d, 3 * d));
      // The output's rounding residual is kept for the backward's row term, as the reference keeps
      // its saved output unrounded (ojas-core/src/autocast.rs:177-186).
      TRY(omx_causal_attention_forward_saving(ctx, A.q, 3 * d, A.k, A.v, 3 * d, AD, A.ap, A.apr, d, AD, A.lse, B, T, H,
                                              H, D, 0));
    } else {
      TRY(omx_linear_forward(ctx, A.h1, AD, t->w(t->li(l, 1)), AD, t->t_a, AD, N, d, d));
      TRY(omx_permute_0213(ctx, t->t_a, A.q, AD, B, T, H, D));
      TRY(omx_linear_forward(ctx, A.h1, AD, t->w(t->li(l, 2)), AD, t->t_a, AD, N, d, d));
      TRY(omx_permute_0213(ctx, t->t_a, A.k, AD, B, T, H, D));
      TRY(omx_linear_forward(ctx, A.h1, AD, t->w(t->li(l, 3)), AD, t->t_a, AD, N, d, d));
      TRY(omx_permute_0213(ctx, t->t_a, A.v, AD, B, T, H, D));
      TRY(omx_causal_sdpa_forward(ctx, A.q, A.k, A.v, AD, A.a, AD, A.lse, B, H, H, T, D, 0));
      TRY(omx_permute_0213(ctx, A.a, A.ap, AD, B, H, T, D));
    }
    TRY(omx_linear_forward(ctx, A.ap, AD, t->w(t->li(l, 4)), AD, t->t_a, AD, N, d, d));
    TRY(omx_residual_add_rms_norm_forward(ctx, A.x, OMX_F32, t->t_a, AD, t->w32(t->li(l, 5)), A.x1, A.h2, AD, N, d,
                                          eps));
    if (AD == OMX_BF16) {
      // The activation rides in the up-projection's store pass.
      TRY(omx_linear_gelu_forward(ctx, A.h2, t->w(t->li(l, 6)), AD, A.u, A.g, N, d, M, c.gelu_tanh));
    } else {
      TRY(omx_linear_forward(ctx, A.h2, AD, t->w(t->li(l, 6)), AD, A.u, AD, N, d, M));
      TRY(omx_gelu_forward(ctx, A.u, A.g, AD, N * M, c.gelu_tanh));
    }
    TRY(omx_linear_forward(ctx, A.g, AD, t->w(t->li(l, 7)), AD, t->t_a, AD, N, M, d));
    TRY(omx_residual_add_rms_norm_forward(ctx, A.x1, OMX_F32, t->t_a, AD, next_norm, x_next, h_next, AD, N, d, eps));
  }
  return OMX_OK;
}

int32_t backward(ogpt* t) {
  omx_ctx* ctx = t->ctx;
  const ogpt_config& c = t->c;
  const uint64_t N = t->N, d = c.d_model, M = c.mlp, B = c.batch, T = c.ctx, H = c.heads, D = c.head_dim;
  const int32_t AD = t->AD;
  const float eps = 1e-6f;
  // Tied head: loss, grad of the final norm output, and the head's share of the table gradient.
  // One row block of the whole vocabulary at a time: no logits are recomputed. 16384 rows (the
  // whole GPT-124M batch, a 1.65 GB bf16 tile) measured 0.1 ms per step ahead of two blocks of 8192.
  const uint64_t chunk_rows = N < 16384 ? N : 16384;
  TRY(omx_linear_cross_entropy_mean(ctx, t->hf, t->w(0), AD, t->targets, N, d, c.vocab, 0, 0, chunk_rows, c.vocab,
                                    t->loss, t->ghf, AD, t->g(0)));
  TRY(omx_rms_norm_backward(ctx, t->x_final, OMX_F32, t->w32(t->nf()), t->ghf, AD, t->gres, OMX_F32, t->g(t->nf()), N, d,
                            eps));
  // `gy` is the residual-stream gradient as a GEMM operand: gres itself on the f32 tier, its bf16
  // copy (written by the kernel that produced gres) on the bf16 tier.
  const bool defer = t->deferred_dw;  // implies the bf16 tier with the fused projection
  // Layer l's slice of a stacked [layers][per_layer] operand buffer.
  auto slice = [&](void* all, uint64_t l, uint64_t per_layer) {
    return static_cast<void*>(static_cast<char*>(all) + l * per_layer * t->asz);
  };
  const void* gy = nullptr;
  TRY(to_operand(t, t->gres, defer ? slice(t->gyd_all, c.layers - 1, N * d) : t->gy16, N * d, &gy));
  void* copy16 = AD == OMX_BF16 ? t->gy16 : nullptr;
  for (uint32_t l = c.layers; l-- > 0;) {
    ogpt::Layer& A = t->layers[l];
    void* gu = defer ? slice(t->gu_all, l, N * M) : t->gu;
    void* gqkv = defer ? slice(t->gqkv_all, l, 3 * N * d) : t->gqkv;
    // Where the two norm backwards of this layer leave the bf16 copy of the gradient they produce:
    // the operand of this layer's o projection, and of the layer below's down projection.
    void* copy_o = defer ? slice(t->gyo_all, l, N * d) : copy16;
    void* copy_below = defer && l > 0 ? slice(t->gyd_all, l - 1, N * d) : copy16;
    // Weight gradients go to the arena now, or wait for the batched products after the loop.
    auto gw = [&](uint64_t which) { return defer ? nullptr : t->g(t->li(l, which)); };
    // x_next = x1 + down(gelu(up(norm2(x1))))
    if (AD == OMX_BF16) {
      // The activation's derivative rides in the input-gradient product's store pass.
      if (!defer) TRY(omx_linear_backward(ctx, A.g, nullptr, gy, AD, nullptr, AD, t->g(t->li(l, 7)), OMX_F32, N, M, d));
      TRY(omx_linear_backward_input_gelu(ctx, t->w(t->li(l, 7)), gy, AD, A.u, gu, N, M, d, c.gelu_tanh));
    } else {
      TRY(omx_linear_backward(ctx, A.g, t->w(t->li(l, 7)), gy, AD, t->gg, AD, t->g(t->li(l, 7)), OMX_F32, N, M, d));
      TRY(omx_gelu_backward(ctx, A.u, t->gg, gu, AD, N * M, c.gelu_tanh));
    }
    TRY(omx_linear_backward(ctx, A.h2, t->w(t->li(l, 6)), gu, AD, t->t_a, AD, gw(6), OMX_F32, N, d, M));
    // Fan-in at x1: the residual branch arrives first, then the norm branch.
    TRY(omx_rms_norm_backward_residual(ctx, A.x1, OMX_F32, t->w32(t->li(l, 5)), t->t_a, AD, t->gres, t->gres1, copy_o,
                                       t->g(t->li(l, 5)), N, d, eps));
    gy = AD == OMX_BF16 ? static_cast<const void*>(copy_o) : static_cast<const void*>(t->gres1);
    // x1 = x + o(attention)
    TRY(omx_linear_backward(ctx, A.ap, t->w(t->li(l, 4)), gy, AD, t->t_a, AD, gw(4), OMX_F32, N, d, d));
    if (t->fused_qkv) {
      char* gq = static_cast<char*>(gqkv);
      TRY(omx_causal_attention_backward_saved(ctx, A.q, 3 * d, A.k, A.v, 3 * d, A.ap, A.apr, t->t_a, d, A.lse, AD, gq,
                                        gq + d * t->asz, gq + 2 * d * t->asz, AD, B, T, H, H, D, 0));
      // One product for the three projections: the input gradient is their sum, formed in the
      // product's f32 accumulators.
      TRY(omx_linear_backward(ctx, A.h1, t->w(t->li(l, 1)), gqkv, AD, t->t_b, AD, gw(1), OMX_F32, N, d, 3 * d));
      TRY(omx_rms_norm_backward_residual(ctx, A.x, OMX_F32, t->w32(t->li(l, 0)), t->t_b, AD, t->gres1, t->gres,
                                         copy_below, t->g(t->li(l, 0)), N, d, eps));
      gy = AD == OMX_BF16 ? static_cast<const void*>(copy_below) : static_cast<const void*>(t->gres);
      continue;
    }
    TRY(omx_permute_0213(ctx, t->t_a, t->ga, AD, B, T, H, D));
    TRY(omx_causal_sdpa_backward(ctx, A.q, A.k, A.v, A.a, A.lse, t->ga, AD, AD, AD, t->gq, t->gk, t->gv, AD, B, H, H, T, D, 0));
    // h1 feeds q, k, v; their gradients arrive v first, then k, then q.
    TRY(omx_permute_0213(ctx, t->gv, t->t_a, AD, B, H, T, D));
    TRY(omx_linear_backward(ctx, A.h1, t->w(t->li(l, 3)), t->t_a, AD, t->t_b, AD, t->g(t->li(l, 3)), OMX_F32, N, d, d));
    TRY(omx_permute_0213(ctx, t->gk, t->t_a, AD, B, H, T, D));
    TRY(omx_linear_backward(ctx, A.h1, t->w(t->li(l, 2)), t->t_a, AD, t->ga, AD, t->g(t->li(l, 2)), OMX_F32, N, d, d));
    TRY(omx_residual_add(ctx, t->t_b, AD, t->ga, AD, t->gh, OMX_F32, N * d));
    TRY(omx_permute_0213(ctx, t->gq, t->t_a, AD, B, H, T, D));
    TRY(omx_linear_backward(ctx, A.h1, t->w(t->li(l, 1)), t->t_a, AD, t->ga, AD, t->g(t->li(l, 1)), OMX_F32, N, d, d));
    TRY(omx_residual_add(ctx, t->gh, OMX_F32, t->ga, AD, t->gh, OMX_F32, N * d));
    TRY(omx_rms_norm_backward_residual(ctx, A.x, OMX_F32, t->w32(t->li(l, 0)), t->gh, OMX_F32, t->gres1, t->gres, copy16,
                                       t->g(t->li(l, 0)), N, d, eps));
    gy = AD == OMX_BF16 ? static_cast<const void*>(t->gy16) : static_cast<const void*>(t->gres);
  }
  if (defer) {
    // gw[l](o, j) = sum_r gy[l][r, o] * x[l][r, j] for every layer l in one launch per weight:
    // 4 x layers long reductions with small outputs become four products with enough tiles to fill
    // the chip without splitting K.
    const uint64_t layers = c.layers, per_layer = t->slots[t->li(1, 1)].offset - t->slots[t->li(0, 1)].offset;
    struct Deferred {
      const void *gy, *x;
      uint64_t which, out, in;
    } products[4] = {{t->gyd_all, t->g_all, 7, d, M},
                     {t->gu_all, t->h2_all, 6, M, d},
                     {t->gyo_all, t->ap_all, 4, d, d},
                     {t->gqkv_all, t->h1_all, 1, 3 * d, d}};
    for (const Deferred& p : products)
      TRY(omx_gemm_strided_batch(ctx, p.gy, 1, p.out, p.x, p.in, 1, AD, t->g(t->li(0, p.which)), OMX_F32, p.out, N, p.in,
                                 0, layers, N * p.out, N * p.in, per_layer));
  }
  // x0 = tok[ids] + pos[positions]; the tied table adds the embedding's share to the head's.
  TRY(omx_embedding_backward(ctx, t->positions, t->gres, OMX_F32, t->g(1), N, T, d));
  // The tied table: the gather's gradient joins the head's where it lies, row by named row.
  TRY(omx_embedding_backward_accumulate(ctx, t->ids, t->gres, OMX_F32, t->g(0), N, c.vocab, d));
  return OMX_OK;
}

}  // namespace

extern "C" {

int32_t ogpt_create(omx_ctx* ctx, const ogpt_config* config, ogpt** out) {
  if (!ctx || !config || !out) return OMX_BACKEND;
  *out = nullptr;
  const ogpt_config& c = *config;
  if (c.d_model == 0 || c.heads == 0 || c.head_dim == 0 || c.mlp == 0 || c.ctx == 0 || c.vocab == 0 || c.batch == 0)
    return OMX_SHAPE;
  if (static_cast<uint64_t>(c.heads) * c.head_dim != c.d_model) return OMX_SHAPE;
  ogpt* t = new ogpt();
  t->ctx = ctx;
  t->c = c;
  t->N = static_cast<uint64_t>(c.batch) * c.ctx;
  t->AD = c.bf16 ? OMX_BF16 : OMX_F32;
  t->asz = c.bf16 ? 2 : 4;
  const uint64_t d = c.d_model, M = c.mlp, N = t->N;
  // Slots in the parameter order of the header; places in the arena: the two tables, then every
  // norm weight, then the layers' matrices (a layer's six together, layers at a fixed stride), so
  // that what AdamW owns under the hybrid step is one range and takes one launch.
  auto push = [&](uint64_t len) { t->slots.push_back({0, len}); };
  push(static_cast<uint64_t>(c.vocab) * d);
  push(static_cast<uint64_t>(c.ctx) * d);
  for (uint32_t l = 0; l < c.layers; ++l) {
    push(d);
    for (int i = 0; i < 4; ++i) push(d * d);
    push(d);
    push(M * d);
    push(d * M);
  }
  push(d);
  auto place = [&](uint64_t i) {
    t->slots[i].offset = t->P;
    t->P += (t->slots[i].len + kAlign - 1) / kAlign * kAlign;
  };
  place(0);
  place(1);
  for (uint64_t l = 0; l < c.layers; ++l) {
    place(t->li(l, 0));
    place(t->li(l, 5));
  }
  place(t->nf());
  t->adamw_end = t->P;  // [0, adamw_end): tables and norm weights
  for (uint64_t l = 0; l < c.layers; ++l)
    for (uint64_t w : {1, 2, 3, 4, 6, 7}) place(t->li(l, w));
  // wq, wk, wv sit back to back when d*d needs no padding.
  t->fused_qkv = c.bf16 && c.head_dim == 64 && (d * d) % kAlign == 0;
  auto fail = [&](int32_t rc) {
    ogpt_destroy(t);
    return rc;
  };
#define CREATE_TRY(expr)                 \
  do {                                   \
    int32_t rc_ = (expr);                \
    if (rc_ != OMX_OK) return fail(rc_); \
  } while (0)
  CREATE_TRY(alloc_t(t, t->P, &t->p32));
  CREATE_TRY(alloc_t(t, t->P, &t->g32));
  CREATE_TRY(alloc_t(t, t->P, &t->m1));
  CREATE_TRY(alloc_t(t, t->P, &t->m2));
  CREATE_TRY(omx_fill_zero(ctx, t->p32, t->P * 4));
  CREATE_TRY(omx_fill_zero(ctx, t->g32, t->P * 4));
  CREATE_TRY(omx_fill_zero(ctx, t->m1, t->P * 4));
  CREATE_TRY(omx_fill_zero(ctx, t->m2, t->P * 4));
  if (c.bf16) {
    CREATE_TRY(alloc(t, t->P * 2, &t->p16));
    CREATE_TRY(omx_fill_zero(ctx, t->p16, t->P * 2));
  }
  CREATE_TRY(alloc_t(t, N, &t->ids));
  CREATE_TRY(alloc_t(t, N, &t->targets));
  CREATE_TRY(alloc_t(t, N, &t->positions));
  {
    void* block = nullptr;
    CREATE_TRY(alloc(t, 256, &block));
    CREATE_TRY(omx_fill_zero(ctx, block, 256));
    t->loss = static_cast<float*>(block);
    t->unbounded = t->loss + 1;
  }
  {
    std::vector<uint32_t> pos(N);
    for (uint64_t i = 0; i < N; ++i) pos[i] = static_cast<uint32_t>(i % c.ctx);
    CREATE_TRY(omx_upload(ctx, t->positions, 0, pos.data(), N * 4));
  }
  t->layers.resize(c.layers);
  t->deferred_dw = t->fused_qkv && c.layers > 1;
  const uint64_t L = c.layers;
  if (t->deferred_dw) {
    CREATE_TRY(alloc_act(t, L * N * d, &t->h1_all));
    CREATE_TRY(alloc_act(t, L * N * d, &t->ap_all));
    CREATE_TRY(alloc_act(t, L * N * d, &t->h2_all));
    CREATE_TRY(alloc_act(t, L * N * M, &t->g_all));
    CREATE_TRY(alloc_act(t, L * N * M, &t->gu_all));
    CREATE_TRY(alloc_act(t, L * 3 * N * d, &t->gqkv_all));
    CREATE_TRY(alloc_act(t, L * N * d, &t->gyd_all));
    CREATE_TRY(alloc_act(t, L * N * d, &t->gyo_all));
  }
  uint64_t layer_index = 0;
  for (auto& A : t->layers) {
    const uint64_t l = layer_index++;
    auto slice = [&](void* all, uint64_t per_layer) { return static_cast<void*>(static_cast<char*>(all) + l * per_layer * t->asz); };
    CREATE_TRY(alloc_t(t, N * d, &A.x));
    CREATE_TRY(alloc_t(t, N * d, &A.x1));
    if (t->deferred_dw) {
      A.h1 = slice(t->h1_all, N * d);
      A.ap = slice(t->ap_all, N * d);
      A.h2 = slice(t->h2_all, N * d);
      A.g = slice(t->g_all, N * M);
    } else {
      CREATE_TRY(alloc_act(t, N * d, &A.h1));
      CREATE_TRY(alloc_act(t, N * d, &A.ap));
      CREATE_TRY(alloc_act(t, N * d, &A.h2));
      CREATE_TRY(alloc_act(t, N * M, &A.g));
    }
    if (t->fused_qkv) {
      CREATE_TRY(alloc_act(t, 3 * N * d, &A.q));
      A.k = static_cast<char*>(A.q) + d * t->asz;
      A.v = static_cast<char*>(A.q) + 2 * d * t->asz;
      A.a = nullptr;
      CREATE_TRY(alloc_act(t, N * d, &A.apr));
    } else {
      CREATE_TRY(alloc_act(t, N * d, &A.q));
      CREATE_TRY(alloc_act(t, N * d, &A.k));
      CREATE_TRY(alloc_act(t, N * d, &A.v));
      CREATE_TRY(alloc_act(t, N * d, &A.a));
    }
    CREATE_TRY(alloc_act(t, N * M, &A.u));
    CREATE_TRY(alloc_t(t, static_cast<uint64_t>(c.batch) * c.heads * c.ctx, &A.lse));
  }
  CREATE_TRY(alloc_t(t, N * d, &t->x_final));
  CREATE_TRY(alloc_act(t, N * d, &t->hf));
  CREATE_TRY(alloc_t(t, N * d, &t->e_tok));
  CREATE_TRY(alloc_t(t, N * d, &t->e_pos));
  CREATE_TRY(alloc_act(t, N * d, &t->t_a));
  CREATE_TRY(alloc_act(t, N * d, &t->t_b));
  if (!t->deferred_dw) CREATE_TRY(alloc_act(t, N * M, &t->gu));
  CREATE_TRY(alloc_act(t, N * M, &t->gg));
  if (t->fused_qkv) {
    if (!t->deferred_dw) CREATE_TRY(alloc_act(t, 3 * N * d, &t->gqkv));
  } else {
    CREATE_TRY(alloc_act(t, N * d, &t->gq));
    CREATE_TRY(alloc_act(t, N * d, &t->gk));
    CREATE_TRY(alloc_act(t, N * d, &t->gv));
  }
  CREATE_TRY(alloc_act(t, N * d, &t->ga));
  CREATE_TRY(alloc_act(t, N * d, &t->gy16));
  CREATE_TRY(alloc_act(t, N * d, &t->ghf));
  CREATE_TRY(alloc_t(t, N * d, &t->gres));
  CREATE_TRY(alloc_t(t, N * d, &t->gres1));
  CREATE_TRY(alloc_t(t, N * d, &t->gt));
  CREATE_TRY(alloc_t(t, N * d, &t->gh));
#undef CREATE_TRY
  *out = t;
  return OMX_OK;
}

void ogpt_destroy(ogpt* t) {
  if (!t) return;
  for (void* p : t->owned) omx_free(t->ctx, p);
  delete t;
}

uint64_t ogpt_param_count(ogpt* t) { return t ? t->slots.size() : 0; }
uint64_t ogpt_param_len(ogpt* t, uint64_t index) { return (t && index < t->slots.size()) ? t->slots[index].len : 0; }
uint64_t ogpt_steps(ogpt* t) { return t ? t->steps : 0; }
uint64_t ogpt_device_bytes(ogpt* t) { return t ? t->device_bytes : 0; }

int32_t ogpt_set_param(ogpt* t, uint64_t index, const float* host) {
  if (!t || index >= t->slots.size() || !host) return OMX_SHAPE;
  const Slot& s = t->slots[index];
  t->tracked = ogpt::kNone;
  TRY(omx_upload(t->ctx, t->p32, s.offset * 4, host, s.len * 4));
  if (t->p16) TRY(omx_to_bf16(t->ctx, t->p32 + s.offset, static_cast<uint16_t*>(t->p16) + s.offset, s.len));
  return OMX_OK;
}
int32_t ogpt_get_param(ogpt* t, uint64_t index, float* host) {
  if (!t || index >= t->slots.size() || !host) return OMX_SHAPE;
  const Slot& s = t->slots[index];
  return omx_download(t->ctx, host, t->p32, s.offset * 4, s.len * 4);
}
int32_t ogpt_get_grad(ogpt* t, uint64_t index, float* host) {
  if (!t || index >= t->slots.size() || !host) return OMX_SHAPE;
  const Slot& s = t->slots[index];
  return omx_download(t->ctx, host, t->g32, s.offset * 4, s.len * 4);
}

int32_t ogpt_get_state(ogpt* t, uint64_t index, uint32_t slot, float* host) {
  if (!t || index >= t->slots.size() || !host || slot > 1) return OMX_SHAPE;
  const Slot& s = t->slots[index];
  return omx_download(t->ctx, host, slot == 0 ? t->m1 : t->m2, s.offset * 4, s.len * 4);
}
int32_t ogpt_set_state(ogpt* t, uint64_t index, uint32_t slot, const float* host) {
  if (!t || index >= t->slots.size() || !host || slot > 1) return OMX_SHAPE;
  const Slot& s = t->slots[index];
  t->tracked = ogpt::kNone;  // the next AdamW pass checks its operands again
  return omx_upload(t->ctx, slot == 0 ? t->m1 : t->m2, s.offset * 4, host, s.len * 4);
}
int32_t ogpt_set_steps(ogpt* t, uint64_t steps) {
  if (!t) return OMX_BACKEND;
  t->steps = steps;
  return OMX_OK;
}

int32_t ogpt_init(ogpt* t, uint64_t seed) {
  if (!t) return OMX_BACKEND;
  std::mt19937_64 rng(seed);
  std::normal_distribution<float> normal(0.0f, 0.02f);
  std::vector<float> host;
  for (uint64_t i = 0; i < t->slots.size(); ++i) {
    const Slot& s = t->slots[i];
    host.resize(s.len);
    const bool is_norm = s.len == t->c.d_model;
    for (auto& v : host) v = is_norm ? 1.0f : normal(rng);
    TRY(ogpt_set_param(t, i, host.data()));
  }
  TRY(omx_fill_zero(t->ctx, t->m1, t->P * 4));
  TRY(omx_fill_zero(t->ctx, t->m2, t->P * 4));
  t->tracked = ogpt::kNone;
  t->steps = 0;
  return omx_sync(t->ctx);
}

int32_t ogpt_set_batch(ogpt* t, const uint32_t* ids, const uint32_t* targets) {
  if (!t || !ids || !targets) return OMX_BACKEND;
  TRY(omx_upload(t->ctx, t->ids, 0, ids, t->N * 4));
  TRY(omx_upload(t->ctx, t->targets, 0, targets, t->N * 4));
  return OMX_OK;
}

int32_t ogpt_loss_and_grads(ogpt* t, float* loss) {
  if (!t) return OMX_BACKEND;
  TRY(forward(t));
  TRY(backward(t));
  float l = 0.0f;
  TRY(omx_read_scalar_f32(t->ctx, t->loss, &l));
  if (loss) *loss = l;
  return OMX_OK;
}

// Whether this step's AdamW inputs are known to be below 2^60 (see omx_adamw_step_bounded): the
// flag of the previous steps, which came back with the last step's loss, and the gradient norm
// for the gradients. When they are not known to be, the flag starts afresh with this step.
static int32_t adamw_inputs_bounded(ogpt* t, int need, float norm, int32_t* bounded) {
  const bool flag_clear = t->tracked >= need && t->flag_seen == 0;
  if (!flag_clear) TRY(omx_fill_zero(t->ctx, t->unbounded, 4));
  *bounded = flag_clear && std::isfinite(norm) && norm < 0x1p60f;
  return OMX_OK;
}
// The step's one readback at its end (trainer.rs:1031-1046): the loss and, behind it, the flag.
static int32_t read_loss_and_flag(ogpt* t, float* loss) {
  struct {
    float loss;
    uint32_t flag;
  } back = {0.0f, 1u};
  TRY(omx_download(t->ctx, &back, t->loss, 0, sizeof(back)));
  t->flag_seen = back.flag;
  *loss = back.loss;
  return OMX_OK;
}

int32_t ogpt_step(ogpt* t, const omx_adamw_config* adamw, float grad_clip, float* loss, float* grad_norm) {
  if (!t || !adamw) return OMX_BACKEND;
  TRY(forward(t));
  TRY(backward(t));
  // Sync point 1: the global gradient norm is a host value (trainer.rs:821-824).
  void* grads[1] = {t->g32};
  uint64_t lens[1] = {t->P};
  float norm = 0.0f;
  TRY(omx_clip_grad_norm(t->ctx, grads, lens, 1, grad_clip > 0.0f ? grad_clip : INFINITY, &norm));
  // One AdamW pass over the arena covers every tensor; the bf16 mirror is refreshed in the same pass.
  int32_t bounded = 0;
  TRY(adamw_inputs_bounded(t, ogpt::kFull, norm, &bounded));
  t->tracked = ogpt::kNone;  // until the readback below has seen this step through
  TRY(omx_adamw_step_bounded(t->ctx, t->p32, t->g32, t->m1, t->m2, t->P, t->steps, adamw, t->p16, bounded,
                             t->unbounded));
  // Sync point 2: sync + the step's one readback.
  float l = 0.0f;
  TRY(read_loss_and_flag(t, &l));
  t->tracked = ogpt::kFull;
  t->steps += 1;
  if (loss) *loss = l;
  if (grad_norm) *grad_norm = norm;
  return OMX_OK;
}

// Trainer::apply with the hybrid groups (ojas-model/src/trainer.rs:858-876, :1004-1028): Muon-NS5
// on every 2-D hidden matrix, AdamW on the tables and the norm weights.
int32_t ogpt_step_hybrid(ogpt* t, const omx_muon_config* muon, const omx_adamw_config* adamw, float grad_clip,
                         float* loss, float* grad_norm) {
  if (!t || !muon || !adamw) return OMX_BACKEND;
  TRY(forward(t));
  TRY(backward(t));
  void* grads[1] = {t->g32};
  uint64_t lens[1] = {t->P};
  float norm = 0.0f;
  TRY(omx_clip_grad_norm(t->ctx, grads, lens, 1, grad_clip > 0.0f ? grad_clip : INFINITY, &norm));
  uint16_t* mirror = static_cast<uint16_t*>(t->p16);
  int32_t bounded = 0;
  TRY(adamw_inputs_bounded(t, ogpt::kHybrid, norm, &bounded));
  t->tracked = ogpt::kNone;  // until the readback at the end has seen this step through
  const uint64_t d = t->c.d_model, mlp = t->c.mlp;
  // Matrices of one shape go through Newton-Schulz together: three batched calls per step.
  struct Group {
    uint64_t rows, cols;
    std::vector<void*> p, m, p16;
    std::vector<const void*> g;
  };
  Group groups[3] = {{d, d, {}, {}, {}, {}}, {mlp, d, {}, {}, {}, {}}, {d, mlp, {}, {}, {}, {}}};
  auto add = [&](Group& grp, uint64_t slot) {
    const uint64_t at = t->slots[slot].offset;  // the AdamW first-moment arena holds Muon's momentum
    grp.p.push_back(t->p32 + at);
    grp.g.push_back(t->g32 + at);
    grp.m.push_back(t->m1 + at);
    grp.p16.push_back(mirror ? mirror + at : nullptr);
  };
  // The tables and every norm weight lie together at the front of the arena (padding between
  // them holds zeros in all four arenas and stays zero): one AdamW launch.
  TRY(omx_adamw_step_bounded(t->ctx, t->p32, t->g32, t->m1, t->m2, t->adamw_end, t->steps, adamw, mirror, bounded,
                             t->unbounded));
  for (uint64_t l = 0; l < t->c.layers; ++l) {
    for (uint64_t w = 1; w <= 4; ++w) add(groups[0], t->li(l, w));
    add(groups[1], t->li(l, 6));
    add(groups[2], t->li(l, 7));
  }
  for (Group& grp : groups)
    TRY(omx_muon_ns5_step_batched(t->ctx, grp.p.data(), grp.g.data(), grp.m.data(), mirror ? grp.p16.data() : nullptr,
                                  grp.p.size(), grp.rows, grp.cols, muon));
  float l = 0.0f;
  TRY(read_loss_and_flag(t, &l));
  t->tracked = ogpt::kHybrid;  // the matrices and their first-moment slots are Muon's from here on
  t->steps += 1;
  if (loss) *loss = l;
  if (grad_norm) *grad_norm = norm;
  return OMX_OK;
}

}  // extern "C"
