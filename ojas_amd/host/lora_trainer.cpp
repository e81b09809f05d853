// Host-side driver of a LoRA fine-tune step over a frozen int8 decoder (see include/ojas_lora.h).
//
// Orchestration only: every tensor operation is one omx_* call, in the order the reference's tape
// would replay the graph of ojas-model/src/lora.rs:292-344 on a Llama-shaped block (forward in
// program order, backward in reverse; ojas-autograd/src/tape.rs:2004-2466), then the step of
// ojas-model/src/trainer.rs:754-1046: clip_grad_norm, adamw_step on the trainable leaves,
// one loss readback.
//
// Layout choices:
//  * q, k, v share one fused projection [3d, d] and gate, up one [2 hidden, d], so a block has four
//    quantised products each way; the base matrices live in the blocked int8 layout
//    (omx_pack_i8_group) and are never widened in memory.
//  * The adapters live in one f32 arena, every A of every layer first ([Aq, Ak, Av, Ao] per layer,
//    so a layer's q, k, v down-projections are one [3r, d] matrix), then every B ([Bq, Bk, Bv, Bo]
//    per layer: the three up-projections stacked are the [3d, r] operand of the fused
//    projection's low-rank term). Gradients and both AdamW moments mirror that arena; one clip
//    pass and one AdamW pass cover every adapter.
//  * The second adapter product never exists as a tensor: it is added in the accumulators of the
//    quantised product (omx_low_rank), forward and backward.
#include <cstdlib>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <random>
#include <vector>

#include "ojas_lora.h"

namespace {

#define TRY(expr)                  \
  do {                             \
    int32_t rc_ = (expr);          \
    if (rc_ != OMX_OK) return rc_; \
  } while (0)

struct QMat {
  void* codes = nullptr;   // blocked int8 [n_out, k_in]
  void* scales = nullptr;  // blocked f32 [n_out, k_in / 32]
  uint64_t nout = 0, kin = 0;
};

}  // namespace

struct olora {
  omx_ctx* ctx = nullptr;
  olora_config c{};
  uint64_t N = 0, P = 0, rd = 0;  // tokens, adapter elements, rank * d_model
  uint64_t steps = 0;
  uint64_t device_bytes = 0;
  std::vector<void*> owned;

  // Frozen base.
  void* emb16 = nullptr;    // [V, d] bf16
  float* norms = nullptr;   // [2 L + 1][d]
  struct Layer {
    QMat qkv, o, gu, dn;
    float *x = nullptr, *x1 = nullptr;  // residual stream before / inside the block (f32)
    void *h1 = nullptr, *ha = nullptr, *qkv_out = nullptr, *ap = nullptr, *apr = nullptr;  // bf16
    void* gu_out = nullptr;  // [N, 2 hidden] f32: the gate | up projection's output, read again by the backward
    float* lse = nullptr;
  };
  std::vector<Layer> layers;
  void *stage_codes = nullptr, *stage_scales = nullptr;  // row-major staging of one sub-matrix
  // The operands of the adapters' weight gradients, every layer's at a fixed stride (bf16): the
  // layers' h1, ha and ap point into the first three; gy_o, gqkv_all and gh_all keep each layer's
  // output gradients of the o site and of q | k | v and their gh = gy B until the end of the
  // backward, where six strided-batch products over the layers form every dA and dB (a reduction
  // over the tokens with an output of rank x d fills the chip only with the layers side by side).
  void *h1_all = nullptr, *ha_all = nullptr, *ap_all = nullptr, *gy_o = nullptr, *gqkv_all = nullptr, *gh_all = nullptr;

  // Adapters.
  float *p32 = nullptr, *g32 = nullptr, *m1 = nullptr, *m2 = nullptr, *tmp_b = nullptr;
  void *p16 = nullptr, *beff16 = nullptr, *at16 = nullptr;  // bf16: mirror, scale * B, A^T per layer [d, 4r]

  // Batch and scalars.
  uint32_t *ids = nullptr, *targets = nullptr;
  float *loss = nullptr, *cos_t = nullptr, *sin_t = nullptr, *dummy_gw = nullptr;
  // Scratch.
  float *x_final = nullptr, *gres = nullptr, *gres1 = nullptr;
  void *t_f = nullptr, *qkv32 = nullptr;  // f32 scratch: a [N, d] product output, the q | k | v projection's [N, 3d]
  void *hf = nullptr, *h2 = nullptr, *m = nullptr, *t_a = nullptr, *t_b = nullptr, *gy16 = nullptr, *gm = nullptr,
       *ggu = nullptr, *ga = nullptr, *ghf = nullptr;

  // Arena offsets (elements). which: 0 q, 1 k, 2 v, 3 o.
  uint64_t a_off(uint64_t l, uint64_t which) const { return (l * 4 + which) * rd; }
  uint64_t b_off(uint64_t l, uint64_t which) const { return static_cast<uint64_t>(c.layers) * 4 * rd + (l * 4 + which) * rd; }
  // External index -> arena offset: layer * 8 + {Aq, Bq, Ak, Bk, Av, Bv, Ao, Bo}.
  uint64_t slot(uint64_t index) const {
    const uint64_t l = index / 8, k = index % 8, site = k / 2;
    return (k % 2 == 0) ? a_off(l, site) : b_off(l, site);
  }
  const uint16_t* a16(uint64_t l, uint64_t which) const { return static_cast<const uint16_t*>(p16) + a_off(l, which); }
  const uint16_t* b16(uint64_t l, uint64_t which) const {
    return static_cast<const uint16_t*>(beff16) + (l * 4 + which) * rd;
  }
  const uint16_t* at(uint64_t l) const { return static_cast<const uint16_t*>(at16) + l * 4 * rd; }
  const float* norm(uint64_t l, uint64_t which) const { return norms + (l * 2 + which) * c.d_model; }
  const float* final_norm() const { return norms + static_cast<uint64_t>(c.layers) * 2 * c.d_model; }
};

namespace {

int32_t alloc(olora* t, uint64_t bytes, void** out) {
  TRY(omx_alloc(t->ctx, bytes, out));
  t->owned.push_back(*out);
  t->device_bytes += bytes;
  return OMX_OK;
}
template <typename T>
int32_t alloc_t(olora* t, uint64_t count, T** out) {
  void* p = nullptr;
  TRY(alloc(t, count * sizeof(T), &p));
  *out = static_cast<T*>(p);
  return OMX_OK;
}
int32_t alloc16(olora* t, uint64_t count, void** out) { return alloc(t, count * 2, out); }

int32_t alloc_qmat(olora* t, QMat* q, uint64_t nout, uint64_t kin) {
  q->nout = nout;
  q->kin = kin;
  TRY(alloc(t, nout * kin, &q->codes));
  TRY(alloc(t, nout * (kin / 32) * 4, &q->scales));
  return OMX_OK;
}

uint16_t* off16(void* p, uint64_t elems) { return static_cast<uint16_t*>(p) + elems; }

// The operand copies the products read, rebuilt after any change of the f32 adapters:
// beff16 = bf16(scale * B) and at16[l] = [A_q; A_k; A_v; A_o]^T as bf16 [d, 4r].
int32_t refresh_operands(olora* t) {
  const uint64_t L = t->c.layers, rd = t->rd, r = t->c.rank, d = t->c.d_model;
  if (t->c.lora_scale != 1.0f) {
    TRY(omx_copy(t->ctx, t->tmp_b, t->p32 + L * 4 * rd, L * 4 * rd * 4));
    TRY(omx_scale_grad(t->ctx, t->tmp_b, t->c.lora_scale, L * 4 * rd));
    TRY(omx_to_bf16(t->ctx, t->tmp_b, t->beff16, L * 4 * rd));
  }
  // [L][4r][d] -> [L][d][4r]
  return omx_permute_0213(t->ctx, t->p16, t->at16, OMX_BF16, L, 4 * r, d, 1);
}

// The forward's products leave their outputs in f32: what follows each (the rotation, the residual
// add and norm, SwiGLU) reads them unrounded, so an activation is rounded to bf16 once, where it
// becomes the next product's operand.
int32_t q8_forward(olora* t, const void* x, const QMat& w, const omx_low_rank* lr, void* y_f32) {
  return omx_linear_i8_group_forward(t->ctx, x, OMX_BF16, w.codes, w.scales, 32, OMX_I8_BLOCKED, nullptr, lr, y_f32,
                                     OMX_F32, t->N, w.kin, w.nout);
}
int32_t q8_backward(olora* t, const QMat& w, const void* gy, const omx_low_rank* lr, void* gx) {
  return omx_linear_i8_group_backward_input(t->ctx, w.codes, w.scales, 32, OMX_I8_BLOCKED, gy, OMX_BF16, nullptr, lr, gx,
                                            t->N, w.kin, w.nout);
}

int32_t forward(olora* t) {
  omx_ctx* ctx = t->ctx;
  const olora_config& c = t->c;
  const uint64_t N = t->N, d = c.d_model, Hd = c.hidden, B = c.batch, T = c.seq, H = c.heads, D = c.head_dim, r = c.rank;
  const float eps = c.rms_eps;
  TRY(omx_embedding_forward(ctx, t->emb16, OMX_BF16, t->ids, t->layers[0].x, OMX_F32, N, c.vocab, d));
  TRY(omx_rms_norm_forward(ctx, t->layers[0].x, OMX_F32, t->norm(0, 0), t->layers[0].h1, OMX_BF16, N, d, eps));
  for (uint32_t l = 0; l < c.layers; ++l) {
    olora::Layer& A = t->layers[l];
    const bool last = l + 1 == c.layers;
    // h A^T for the three sites at once: [N, 3r] in the first columns of ha.
    TRY(omx_gemm_pitched(ctx, A.h1, d, 1, t->a16(l, 0), 1, d, OMX_BF16, A.ha, OMX_BF16, 4 * r, N, d, 3 * r, 0));
    omx_low_rank lr_qkv{A.ha, t->b16(l, 0), 4 * r, r, r, d};
    TRY(q8_forward(t, A.h1, A.qkv, &lr_qkv, t->qkv32));
    TRY(omx_rope_half_split_pitched(ctx, t->qkv32, OMX_F32, A.qkv_out, 3 * d, t->cos_t, t->sin_t, N, T, 2 * H, H, D));
    // The output's rounding residual is kept for the backward's row term, as the reference keeps
    // its saved output unrounded (ojas-core/src/autocast.rs:177-186).
    TRY(omx_causal_attention_forward_saving(ctx, A.qkv_out, 3 * d, off16(A.qkv_out, d), off16(A.qkv_out, 2 * d), 3 * d,
                                            OMX_BF16, A.ap, A.apr, d, OMX_BF16, A.lse, B, T, H, H, D, 0));
    TRY(omx_gemm_pitched(ctx, A.ap, d, 1, t->a16(l, 3), 1, d, OMX_BF16, off16(A.ha, 3 * r), OMX_BF16, 4 * r, N, d, r, 0));
    omx_low_rank lr_o{off16(A.ha, 3 * r), t->b16(l, 3), 4 * r, r, r, 0};
    TRY(q8_forward(t, A.ap, A.o, &lr_o, t->t_f));
    TRY(omx_residual_add_rms_norm_forward(ctx, A.x, OMX_F32, t->t_f, OMX_F32, t->norm(l, 1), A.x1, t->h2, OMX_BF16, N, d,
                                          eps));
    TRY(q8_forward(t, t->h2, A.gu, nullptr, A.gu_out));
    TRY(omx_swiglu_forward(ctx, A.gu_out, t->m, OMX_F32, N, Hd));
    TRY(q8_forward(t, t->m, A.dn, nullptr, t->t_f));
    float* x_next = last ? t->x_final : t->layers[l + 1].x;
    void* h_next = last ? t->hf : t->layers[l + 1].h1;
    const float* next_norm = last ? t->final_norm() : t->norm(l + 1, 0);
    TRY(omx_residual_add_rms_norm_forward(ctx, A.x1, OMX_F32, t->t_f, OMX_F32, next_norm, x_next, h_next, OMX_BF16, N, d,
                                          eps));
  }
  return OMX_OK;
}

int32_t backward(olora* t) {
  omx_ctx* ctx = t->ctx;
  const olora_config& c = t->c;
  const uint64_t N = t->N, d = c.d_model, Hd = c.hidden, B = c.batch, T = c.seq, H = c.heads, D = c.head_dim, r = c.rank;
  const float eps = c.rms_eps;
  const uint64_t chunk_rows = N < 16384 ? N : 16384;
  TRY(omx_linear_cross_entropy_mean(ctx, t->hf, t->emb16, OMX_BF16, t->targets, N, d, c.vocab, 0, 0, chunk_rows, c.vocab,
                                    t->loss, t->ghf, OMX_BF16, nullptr));
  TRY(omx_rms_norm_backward(ctx, t->x_final, OMX_F32, t->final_norm(), t->ghf, OMX_BF16, t->gres, OMX_F32, t->dummy_gw, N,
                            d, eps));
  TRY(omx_to_bf16(ctx, t->gres, t->gy16, N * d));
  for (uint32_t l = c.layers; l-- > 0;) {
    olora::Layer& A = t->layers[l];
    // x_next = x1 + down(silu(gate) * up)
    TRY(q8_backward(t, A.dn, t->gy16, nullptr, t->gm));
    TRY(omx_swiglu_backward(ctx, A.gu_out, t->gm, t->ggu, OMX_F32, N, Hd));
    TRY(q8_backward(t, A.gu, t->ggu, nullptr, t->t_a));
    // Fan-in at x1: the residual branch first, then the norm branch. The bf16 copy is this layer's
    // own: the o site's weight gradients read it after the loop.
    uint16_t* gy_mid = off16(t->gy_o, l * N * d);
    uint16_t* gqkv = off16(t->gqkv_all, l * N * 3 * d);
    uint16_t* gh = off16(t->gh_all, l * N * 4 * r);
    TRY(omx_rms_norm_backward_residual(ctx, A.x1, OMX_F32, t->norm(l, 1), t->t_a, OMX_BF16, t->gres, t->gres1, gy_mid,
                                       nullptr, N, d, eps));  // the norms are frozen: no weight gradient
    // x1 = x + lora_linear(ap; Wo, Ao, Bo). With gy the gradient of the site's output:
    //   gh = gy B_eff [N, r];  dB_eff = gy^T h;  dA = gh^T x;  gx = gy W + gh A.
    TRY(omx_gemm_pitched(ctx, gy_mid, d, 1, t->b16(l, 3), r, 1, OMX_BF16, off16(gh, 3 * r), OMX_BF16, 4 * r, N, d, r, 0));
    omx_low_rank lr_o{off16(gh, 3 * r), t->at(l) + 3 * r, 4 * r, 4 * r, r, 0};
    TRY(q8_backward(t, A.o, gy_mid, &lr_o, t->ga));
    char* gq = reinterpret_cast<char*>(gqkv);
    TRY(omx_causal_attention_backward_saved(ctx, A.qkv_out, 3 * d, off16(A.qkv_out, d), off16(A.qkv_out, 2 * d), 3 * d,
                                            A.ap, A.apr, t->ga, d, A.lse, OMX_BF16, gq, gq + d * 2, gq + 2 * d * 2,
                                            OMX_BF16, B, T, H, H, D, 0));
    TRY(omx_rope_half_split_inplace(ctx, gqkv, OMX_BF16, 3 * d, t->cos_t, t->sin_t, N, T, 2 * H, D, 1));
    // gh for q, k and v in one launch: column blocks of gqkv against B_q, B_k, B_v (adjacent in the
    // arena) into adjacent column blocks of gh.
    TRY(omx_gemm_pitched_strided_batch(ctx, gqkv, 3 * d, 1, t->b16(l, 0), r, 1, OMX_BF16, gh, OMX_BF16, 4 * r, N, d, r, 0,
                                       3, d, t->b_off(0, 1) - t->b_off(0, 0), r));
    omx_low_rank lr_qkv{gh, t->at(l), 4 * r, 4 * r, 3 * r, 0};
    TRY(q8_backward(t, A.qkv, gqkv, &lr_qkv, t->t_b));
    TRY(omx_rms_norm_backward_residual(ctx, A.x, OMX_F32, t->norm(l, 0), t->t_b, OMX_BF16, t->gres1, t->gres, t->gy16,
                                       nullptr, N, d, eps));
  }
  // The adapters' weight gradients, every layer's in one launch per site: dB_eff = gy^T h for q, k,
  // v and o; dA = gh^T x for [Aq; Ak; Av] (adjacent in the arena: one product) and for Ao.
  {
    const uint64_t L = c.layers, rd = t->rd;
    const uint64_t s_d = N * d, s_3d = N * 3 * d, s_4r = N * 4 * r, s_c = 4 * rd;
    for (uint64_t j = 0; j < 3; ++j)
      TRY(omx_gemm_strided_batch(ctx, off16(t->gqkv_all, j * d), 1, 3 * d, off16(t->ha_all, j * r), 4 * r, 1, OMX_BF16,
                                 t->g32 + t->b_off(0, j), OMX_F32, d, N, r, 0, L, s_3d, s_4r, s_c));
    TRY(omx_gemm_strided_batch(ctx, t->gy_o, 1, d, off16(t->ha_all, 3 * r), 4 * r, 1, OMX_BF16, t->g32 + t->b_off(0, 3),
                               OMX_F32, d, N, r, 0, L, s_d, s_4r, s_c));
    TRY(omx_gemm_strided_batch(ctx, t->gh_all, 1, 4 * r, t->h1_all, d, 1, OMX_BF16, t->g32 + t->a_off(0, 0), OMX_F32,
                               3 * r, N, d, 0, L, s_4r, s_d, s_c));
    TRY(omx_gemm_strided_batch(ctx, off16(t->gh_all, 3 * r), 1, 4 * r, t->ap_all, d, 1, OMX_BF16,
                               t->g32 + t->a_off(0, 3), OMX_F32, r, N, d, 0, L, s_4r, s_d, s_c));
  }
  // B reaches the graph as scale * B (lora.rs:309-323): its gradient carries the factor.
  if (c.lora_scale != 1.0f) {
    const uint64_t nb = static_cast<uint64_t>(c.layers) * 4 * t->rd;
    TRY(omx_scale_grad(ctx, t->g32 + nb, c.lora_scale, nb));
  }
  return OMX_OK;
}

// cos / sin [seq, head_dim] as ojas-model/src/block.rs:31-71: angles in f64, one rounding to f32,
// both halves of a row alike.
void rope_tables(uint64_t seq, uint64_t dim, double base, std::vector<float>* cos_out, std::vector<float>* sin_out) {
  const uint64_t half = dim / 2;
  cos_out->resize(seq * dim);
  sin_out->resize(seq * dim);
  for (uint64_t row = 0; row < seq; ++row)
    for (uint64_t i = 0; i < half; ++i) {
      const double inv = std::pow(base, -static_cast<double>(2 * i) / static_cast<double>(dim));
      const double angle = static_cast<double>(row) * inv;
      const float cv = static_cast<float>(std::cos(angle)), sv = static_cast<float>(std::sin(angle));
      (*cos_out)[row * dim + i] = cv;
      (*cos_out)[row * dim + half + i] = cv;
      (*sin_out)[row * dim + i] = sv;
      (*sin_out)[row * dim + half + i] = sv;
    }
}

// The fused matrix that holds base matrix `which` of a layer, and the row it starts at.
QMat* fused_of(olora::Layer& A, uint32_t which, const olora_config& c, uint64_t* row0, uint64_t* rows) {
  const uint64_t d = c.d_model, h = c.hidden;
  switch (which) {
    case 0: *row0 = 0; *rows = d; return &A.qkv;
    case 1: *row0 = d; *rows = d; return &A.qkv;
    case 2: *row0 = 2 * d; *rows = d; return &A.qkv;
    case 3: *row0 = 0; *rows = d; return &A.o;
    case 4: *row0 = 0; *rows = h; return &A.gu;
    case 5: *row0 = h; *rows = h; return &A.gu;
    case 6: *row0 = 0; *rows = d; return &A.dn;
    default: return nullptr;
  }
}

}  // namespace

extern "C" {

int32_t olora_create(omx_ctx* ctx, const olora_config* config, olora** out) {
  if (!ctx || !config || !out) return OMX_BACKEND;
  *out = nullptr;
  const olora_config& c = *config;
  if (c.layers == 0 || c.d_model == 0 || c.heads == 0 || c.head_dim == 0 || c.hidden == 0 || c.vocab == 0 ||
      c.batch == 0 || c.seq == 0 || c.rank == 0)
    return OMX_SHAPE;
  if (static_cast<uint64_t>(c.heads) * c.head_dim != c.d_model) return OMX_SHAPE;
  if (c.d_model % 128 != 0 || c.hidden % 128 != 0 || c.rank % 16 != 0) return OMX_SHAPE;
  if (c.head_dim != 64 && c.head_dim != 128) return OMX_UNSUPPORTED_HEAD_DIM;
  if (!std::isfinite(c.lora_scale) || c.lora_scale < 0.0f) return OMX_OUT_OF_RANGE;
  olora* t = new olora();
  t->ctx = ctx;
  t->c = c;
  t->N = static_cast<uint64_t>(c.batch) * c.seq;
  t->rd = static_cast<uint64_t>(c.rank) * c.d_model;
  const uint64_t L = c.layers, d = c.d_model, h = c.hidden, N = t->N, r = c.rank;
  t->P = L * 8 * t->rd;
  auto fail = [&](int32_t rc) {
    olora_destroy(t);
    return rc;
  };
#define CREATE_TRY(expr)                 \
  do {                                   \
    int32_t rc_ = (expr);                \
    if (rc_ != OMX_OK) return fail(rc_); \
  } while (0)
  CREATE_TRY(alloc16(t, static_cast<uint64_t>(c.vocab) * d, &t->emb16));
  CREATE_TRY(alloc_t(t, (2 * L + 1) * d, &t->norms));
  const uint64_t stage_elems = (h > d ? h : d) * d;
  CREATE_TRY(alloc(t, stage_elems, &t->stage_codes));
  CREATE_TRY(alloc(t, stage_elems / 32 * 4, &t->stage_scales));
  t->layers.resize(L);
  CREATE_TRY(alloc16(t, L * N * d, &t->h1_all));
  CREATE_TRY(alloc16(t, L * N * 4 * r, &t->ha_all));
  CREATE_TRY(alloc16(t, L * N * d, &t->ap_all));
  CREATE_TRY(alloc16(t, L * N * d, &t->gy_o));
  CREATE_TRY(alloc16(t, L * N * 3 * d, &t->gqkv_all));
  CREATE_TRY(alloc16(t, L * N * 4 * r, &t->gh_all));
  uint64_t layer_index = 0;
  for (auto& A : t->layers) {
    CREATE_TRY(alloc_qmat(t, &A.qkv, 3 * d, d));
    CREATE_TRY(alloc_qmat(t, &A.o, d, d));
    CREATE_TRY(alloc_qmat(t, &A.gu, 2 * h, d));
    CREATE_TRY(alloc_qmat(t, &A.dn, d, h));
    CREATE_TRY(alloc_t(t, N * d, &A.x));
    CREATE_TRY(alloc_t(t, N * d, &A.x1));
    A.h1 = off16(t->h1_all, layer_index * N * d);
    A.ha = off16(t->ha_all, layer_index * N * 4 * r);
    A.ap = off16(t->ap_all, layer_index * N * d);
    ++layer_index;
    CREATE_TRY(alloc16(t, N * 3 * d, &A.qkv_out));
    CREATE_TRY(alloc16(t, N * d, &A.apr));
    CREATE_TRY(alloc(t, N * 2 * h * 4, &A.gu_out));
    CREATE_TRY(alloc_t(t, static_cast<uint64_t>(c.batch) * c.heads * c.seq, &A.lse));
  }
  CREATE_TRY(alloc_t(t, t->P, &t->p32));
  CREATE_TRY(alloc_t(t, t->P, &t->g32));
  CREATE_TRY(alloc_t(t, t->P, &t->m1));
  CREATE_TRY(alloc_t(t, t->P, &t->m2));
  CREATE_TRY(alloc16(t, t->P, &t->p16));
  CREATE_TRY(alloc16(t, L * 4 * t->rd, &t->at16));
  if (c.lora_scale != 1.0f) {
    CREATE_TRY(alloc_t(t, L * 4 * t->rd, &t->tmp_b));
    CREATE_TRY(alloc16(t, L * 4 * t->rd, &t->beff16));
  } else {
    t->beff16 = off16(t->p16, L * 4 * t->rd);
  }
  for (float* arena : {t->p32, t->g32, t->m1, t->m2}) CREATE_TRY(omx_fill_zero(ctx, arena, t->P * 4));
  CREATE_TRY(omx_fill_zero(ctx, t->p16, t->P * 2));
  CREATE_TRY(alloc_t(t, N, &t->ids));
  CREATE_TRY(alloc_t(t, N, &t->targets));
  {
    void* block = nullptr;
    CREATE_TRY(alloc(t, 256, &block));
    CREATE_TRY(omx_fill_zero(ctx, block, 256));
    t->loss = static_cast<float*>(block);
  }
  {
    std::vector<float> cv, sv;
    rope_tables(c.seq, c.head_dim, c.rope_base, &cv, &sv);
    CREATE_TRY(alloc_t(t, cv.size(), &t->cos_t));
    CREATE_TRY(alloc_t(t, sv.size(), &t->sin_t));
    CREATE_TRY(omx_upload(ctx, t->cos_t, 0, cv.data(), cv.size() * 4));
    CREATE_TRY(omx_upload(ctx, t->sin_t, 0, sv.data(), sv.size() * 4));
  }
  CREATE_TRY(alloc_t(t, d, &t->dummy_gw));
  CREATE_TRY(alloc_t(t, N * d, &t->x_final));
  CREATE_TRY(alloc_t(t, N * d, &t->gres));
  CREATE_TRY(alloc_t(t, N * d, &t->gres1));
  CREATE_TRY(alloc16(t, N * d, &t->hf));
  CREATE_TRY(alloc16(t, N * d, &t->h2));
  CREATE_TRY(alloc16(t, N * h, &t->m));
  CREATE_TRY(alloc16(t, N * d, &t->t_a));
  CREATE_TRY(alloc(t, N * d * 4, &t->t_f));
  CREATE_TRY(alloc(t, N * 3 * d * 4, &t->qkv32));
  CREATE_TRY(alloc16(t, N * d, &t->t_b));
  CREATE_TRY(alloc16(t, N * d, &t->gy16));
  CREATE_TRY(alloc16(t, N * h, &t->gm));
  CREATE_TRY(alloc16(t, N * 2 * h, &t->ggu));
  CREATE_TRY(alloc16(t, N * d, &t->ga));
  CREATE_TRY(alloc16(t, N * d, &t->ghf));
  CREATE_TRY(refresh_operands(t));
#undef CREATE_TRY
  *out = t;
  return OMX_OK;
}

void olora_destroy(olora* t) {
  if (!t) return;
  for (void* p : t->owned) omx_free(t->ctx, p);
  delete t;
}

int32_t olora_set_embedding(olora* t, const float* host) {
  if (!t || !host) return OMX_BACKEND;
  const uint64_t n = static_cast<uint64_t>(t->c.vocab) * t->c.d_model;
  // Through an f32 staging allocation: the table is the one tensor that may exceed every scratch buffer.
  void* stage = nullptr;
  TRY(omx_alloc(t->ctx, n * 4, &stage));
  int32_t rc = omx_upload(t->ctx, stage, 0, host, n * 4);
  if (rc == OMX_OK) rc = omx_to_bf16(t->ctx, stage, t->emb16, n);
  if (rc == OMX_OK) rc = omx_sync(t->ctx);
  omx_free(t->ctx, stage);
  return rc;
}

int32_t olora_set_norm(olora* t, uint32_t layer, uint32_t which, const float* host) {
  if (!t || !host) return OMX_BACKEND;
  if (layer > t->c.layers || which > 1 || (layer == t->c.layers && which != 0)) return OMX_SHAPE;
  const uint64_t d = t->c.d_model;
  return omx_upload(t->ctx, t->norms, (static_cast<uint64_t>(layer) * 2 + which) * d * 4, host, d * 4);
}

int32_t olora_set_matrix(olora* t, uint32_t layer, uint32_t which, const int8_t* codes, const float* scales) {
  if (!t || !codes || !scales) return OMX_BACKEND;
  if (layer >= t->c.layers || which > 6) return OMX_SHAPE;
  uint64_t row0 = 0, rows = 0;
  QMat* q = fused_of(t->layers[layer], which, t->c, &row0, &rows);
  const uint64_t kin = q->kin;
  TRY(omx_upload(t->ctx, t->stage_codes, 0, codes, rows * kin));
  TRY(omx_upload(t->ctx, t->stage_scales, 0, scales, rows * (kin / 32) * 4));
  // Blocks hold 8 whole rows, so a sub-matrix that starts at a multiple of 8 rows is a contiguous
  // run of the fused matrix's blocked form.
  return omx_pack_i8_group(t->ctx, t->stage_codes, t->stage_scales, static_cast<char*>(q->codes) + row0 * kin,
                           static_cast<float*>(q->scales) + row0 * (kin / 32), rows, kin, 32, 0);
}

int32_t olora_init_base(olora* t, uint64_t seed, float std) {
  if (!t) return OMX_BACKEND;
  const uint64_t d = t->c.d_model;
  TRY(omx_init_normal(t->ctx, t->emb16, OMX_BF16, static_cast<uint64_t>(t->c.vocab) * d, seed, std));
  std::vector<float> ones((2 * static_cast<uint64_t>(t->c.layers) + 1) * d, 1.0f);
  TRY(omx_upload(t->ctx, t->norms, 0, ones.data(), ones.size() * 4));
  uint64_t stream = 1;
  for (auto& A : t->layers)
    for (uint32_t which = 0; which < 7; ++which) {
      uint64_t row0 = 0, rows = 0;
      QMat* q = fused_of(A, which, t->c, &row0, &rows);
      TRY(omx_init_normal_i8_group(t->ctx, t->stage_codes, t->stage_scales, rows, q->kin, 32, seed + 0x9e3779b97f4a7c15ull * stream++, std));
      TRY(omx_pack_i8_group(t->ctx, t->stage_codes, t->stage_scales, static_cast<char*>(q->codes) + row0 * q->kin,
                            static_cast<float*>(q->scales) + row0 * (q->kin / 32), rows, q->kin, 32, 0));
    }
  return omx_sync(t->ctx);
}

uint64_t olora_adapter_count(olora* t) { return t ? static_cast<uint64_t>(t->c.layers) * 8 : 0; }
uint64_t olora_adapter_len(olora* t, uint64_t index) { return (t && index < olora_adapter_count(t)) ? t->rd : 0; }
uint64_t olora_steps(olora* t) { return t ? t->steps : 0; }
uint64_t olora_device_bytes(olora* t) { return t ? t->device_bytes : 0; }

int32_t olora_set_adapter(olora* t, uint64_t index, const float* host) {
  if (!t || !host || index >= olora_adapter_count(t)) return OMX_SHAPE;
  const uint64_t at = t->slot(index);
  TRY(omx_upload(t->ctx, t->p32, at * 4, host, t->rd * 4));
  TRY(omx_to_bf16(t->ctx, t->p32 + at, off16(t->p16, at), t->rd));
  return refresh_operands(t);
}
int32_t olora_get_adapter(olora* t, uint64_t index, float* host) {
  if (!t || !host || index >= olora_adapter_count(t)) return OMX_SHAPE;
  return omx_download(t->ctx, host, t->p32, t->slot(index) * 4, t->rd * 4);
}
int32_t olora_get_grad(olora* t, uint64_t index, float* host) {
  if (!t || !host || index >= olora_adapter_count(t)) return OMX_SHAPE;
  return omx_download(t->ctx, host, t->g32, t->slot(index) * 4, t->rd * 4);
}

int32_t olora_init_adapters(olora* t, uint64_t seed, float std) {
  if (!t) return OMX_BACKEND;
  std::mt19937_64 rng(seed);
  std::normal_distribution<float> normal(0.0f, std);
  const uint64_t na = static_cast<uint64_t>(t->c.layers) * 4 * t->rd;
  std::vector<float> host(t->P, 0.0f);  // B = 0 (lora.rs:9-12)
  for (uint64_t i = 0; i < na; ++i) host[i] = normal(rng);
  TRY(omx_upload(t->ctx, t->p32, 0, host.data(), t->P * 4));
  TRY(omx_to_bf16(t->ctx, t->p32, t->p16, t->P));
  TRY(omx_fill_zero(t->ctx, t->m1, t->P * 4));
  TRY(omx_fill_zero(t->ctx, t->m2, t->P * 4));
  t->steps = 0;
  TRY(refresh_operands(t));
  return omx_sync(t->ctx);
}

int32_t olora_set_batch(olora* t, const uint32_t* ids, const uint32_t* targets) {
  if (!t || !ids || !targets) return OMX_BACKEND;
  TRY(omx_upload(t->ctx, t->ids, 0, ids, t->N * 4));
  TRY(omx_upload(t->ctx, t->targets, 0, targets, t->N * 4));
  return OMX_OK;
}

int32_t olora_loss_and_grads(olora* t, float* loss) {
  if (!t) return OMX_BACKEND;
  TRY(forward(t));
  TRY(backward(t));
  float l = 0.0f;
  TRY(omx_read_scalar_f32(t->ctx, t->loss, &l));
  if (loss) *loss = l;
  return OMX_OK;
}

int32_t olora_step(olora* t, const omx_adamw_config* adamw, float grad_clip, float* loss, float* grad_norm) {
  if (!t || !adamw) return OMX_BACKEND;
  TRY(forward(t));
  TRY(backward(t));
  // Sync point 1: the global gradient norm is a host value (trainer.rs:821-824).
  void* grads[1] = {t->g32};
  uint64_t lens[1] = {t->P};
  float norm = 0.0f;
  TRY(omx_clip_grad_norm(t->ctx, grads, lens, 1, grad_clip > 0.0f ? grad_clip : INFINITY, &norm));
  TRY(omx_adamw_step(t->ctx, t->p32, t->g32, t->m1, t->m2, t->P, t->steps, adamw, t->p16));
  TRY(refresh_operands(t));
  // Sync point 2: the step's one readback.
  float l = 0.0f;
  TRY(omx_read_scalar_f32(t->ctx, t->loss, &l));
  t->steps += 1;
  if (loss) *loss = l;
  if (grad_norm) *grad_norm = norm;
  return OMX_OK;
}

}  // extern "C"
