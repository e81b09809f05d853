// Host-side training-step driver for the nanolab GPT graph above the C ABI (see include/ojas_nanolab.h).
//
// Orchestration only: every tensor operation is one omx_* call, in the order the reference's tape
// replays the graph of ojas-model/src/block.rs:218-264 (forward in program order, backward in
// reverse with a value's consumers adding their gradients later one first,
// ojas-autograd/src/tape.rs:2004-2466,2565-2591), then Trainer::run's optimizer half
// (ojas-model/src/trainer.rs:858-876,1004-1046).
//
// All buffers are allocated at creation. Parameters, the step's gradient, the last micro-batch's
// gradient and the optimizer state live in flat f32 arenas in parameter order (one clip pass covers
// every tensor; adjacent AdamW parameters share a pass; matrices of one shape share a batched
// Newton-Schulz call); the bf16 tier keeps a bf16 mirror of the parameters that the optimizers
// refresh. The gate and up projections are adjacent in the arena, so on the bf16 tier they are one
// [2 hidden, n_embd] matrix whose product feeds the fused SwiGLU.
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <map>
#include <random>
#include <utility>
#include <vector>

#include "ojas_nanolab.h"

namespace {

constexpr uint64_t kAlign = 64;  // elements; keeps every tensor 256-byte aligned in both arenas
constexpr uint64_t kPerBlock = 14;
enum Which : uint64_t {
  NORM1 = 0, WQ, WK, WV, WO, QNORM, KNORM, GATE_W, GATE_B, LAMBDA, NORM2, FFN_GATE, FFN_UP, FFN_DOWN
};

struct Slot {
  uint64_t offset, len, rows, cols;  // cols == 0: a vector
};

}  // namespace

struct onano {
  omx_ctx* ctx = nullptr;
  onano_config c{};
  uint64_t N = 0, P = 0;
  uint64_t adam_end = 0;  // the arena's first adam_end elements are AdamW's (table and vectors)
  std::vector<Slot> slots;
  int32_t AD = OMX_F32;
  uint64_t asz = 4;
  bool flash = false;      // time-major MFMA attention (bf16, head_dim 64 or 128)
  bool fused_mlp = false;  // one gate | up product and the fused SwiGLU (bf16)
  // With MFMA attention the q, k and v projections are one product (their weights are adjacent in
  // the arena: one [(heads + 2 kv_heads) head_dim, n_embd] matrix), QK-norm, RoPE and the value blend
  // are one pass over its output, and attention reads q, k and v where that pass left them.
  bool fused_qkv = false;
  // bf16 tier, fused paths: the forward's product outputs (the q | k | v, o, gate | up and down
  // projections) and the attention output the gate reads stay f32, so every activation is rounded
  // to bf16 once, where it becomes a product's operand, and not a second time where a product
  // left it. `LD` is the dtype of those outputs, `lsz` its size.
  bool keep_f32 = false;
  int32_t LD = OMX_F32;
  uint64_t lsz = 4;
  uint64_t steps = 0;
  uint64_t device_bytes = 0;
  std::vector<void*> owned;

  float *p32 = nullptr, *acc = nullptr, *g32 = nullptr, *m1 = nullptr, *m2 = nullptr;
  float* gdst = nullptr;  // where the running backward writes: acc (a step's first micro-batch) or g32
  void* p16 = nullptr;
  uint32_t *ids = nullptr, *targets = nullptr;
  float *loss = nullptr, *loss_acc = nullptr;
  // omx_adamw_step_bounded's flag word (the word after the accumulated loss, so one readback
  // fetches both), whether it has covered AdamW's range since that was last written from outside,
  // and the flag as the last step's readback saw it.
  void* unbounded = nullptr;
  bool tracked = false;
  uint32_t flag_seen = 1;
  float *cos_t = nullptr, *sin_t = nullptr;

  struct Layer {
    float *x, *x1;  // residual stream entering the block and after attention (f32)
    void *h, *q_lin, *k_lin, *q, *k, *raw_v, *v, *ap, *apr, *y, *h2, *gu, *g_lin, *up, *g_act, *m;
    void *qp, *kp, *vp, *att;  // [B, heads, T, D] copies for the row kernels (no MFMA attention)
    void *qkv_lin, *qkv;       // fused projection output and what attention reads: [N, (heads + 2 kv_heads) D]
    float *lse, *gates;
  };
  std::vector<Layer> layers;
  float* x_final = nullptr;
  void* hf = nullptr;
  // Scratch.
  void *t_q = nullptr, *t_k = nullptr;   // [N, H D], [N, KV D] AD
  void *t_a = nullptr;                   // [N, max(d, H D)] AD
  void *t_f = nullptr;                   // [N, d] LD: the o and down projections' outputs on the forward
  float *ap32 = nullptr;                 // [N, H D] f32: the attention output and its rounding residual, summed (keep_f32)
  void *gm = nullptr, *ggu = nullptr, *g_gact = nullptr, *g_up = nullptr;  // MLP gradients AD
  void *gyy = nullptr, *gap = nullptr, *gq = nullptr, *gk = nullptr, *gv = nullptr, *g_raw_v = nullptr, *part_v0 = nullptr;
  void *g_v0 = nullptr;                  // [N, KV D] AD: what the later blocks' blends send to block 0's v
  void *g_qkv = nullptr, *g_qkv_lin = nullptr, *gqkv_all = nullptr;  // fused projection: gradients [N, P3] AD
  void* gz_all = nullptr;  // the gates' pre-activation gradients [layers][N, heads] AD (deferred weight gradients)
  float* v0_acc = nullptr;               // the same as g_v0 in f32 (fused projection)
  void *gqp = nullptr, *gkp = nullptr, *gvp = nullptr, *gap_p = nullptr;  // permuted gradients (row kernels)
  void *gy16 = nullptr, *ghf = nullptr;
  float *gres = nullptr, *gres1 = nullptr, *gh = nullptr;
  // bf16 tier with more than one block: the seven weight gradients of every block wait until the
  // backward's end. Each block's product inputs (h, y, h2, m) and output gradients sit at a fixed
  // stride in stacked buffers, the gradient arena holds the blocks at a fixed stride too, and seven
  // strided-batch products over the blocks replace 7 x layers split-K products: long reductions
  // (the step's tokens) with small outputs fill the chip only together.
  bool deferred_dw = false;
  void *h_all = nullptr, *y_all = nullptr, *h2_all = nullptr, *m_all = nullptr;
  void *gyd_all = nullptr, *ggu_all = nullptr, *gyo_all = nullptr, *gq_all = nullptr, *gk_all = nullptr, *gv_all = nullptr;

  const void* w(uint64_t i) const {
    return AD == OMX_BF16 ? static_cast<const void*>(static_cast<const uint16_t*>(p16) + slots[i].offset)
                          : static_cast<const void*>(p32 + slots[i].offset);
  }
  const float* w32(uint64_t i) const { return p32 + slots[i].offset; }
  float* g(uint64_t i) const { return gdst + slots[i].offset; }
  uint64_t li(uint64_t l, uint64_t which) const { return 1 + l * kPerBlock + which; }
  uint64_t nf() const { return 1 + static_cast<uint64_t>(c.layers) * kPerBlock; }
  bool is_muon(uint64_t i) const { return i != 0 && slots[i].cols != 0; }
  bool is_frozen(uint64_t i) const { return i == li(0, LAMBDA); }
};

namespace {

#define TRY(expr)                  \
  do {                             \
    int32_t rc_ = (expr);          \
    if (rc_ != OMX_OK) return rc_; \
  } while (0)

int32_t alloc(onano* t, uint64_t bytes, void** out) {
  TRY(omx_alloc(t->ctx, bytes, out));
  t->owned.push_back(*out);
  t->device_bytes += bytes;
  return OMX_OK;
}
template <typename T>
int32_t alloc_t(onano* t, uint64_t count, T** out) {
  void* p = nullptr;
  TRY(alloc(t, count * sizeof(T), &p));
  *out = static_cast<T*>(p);
  return OMX_OK;
}
int32_t alloc_act(onano* t, uint64_t count, void** out) { return alloc(t, count * t->asz, out); }

// AD copy of an f32 tensor: the f32 tier aliases it, the bf16 tier rounds it.
int32_t to_operand(onano* t, const float* src, void* scratch, uint64_t n, const void** out) {
  if (t->AD == OMX_F32) {
    *out = src;
    return OMX_OK;
  }
  TRY(omx_to_bf16(t->ctx, src, scratch, n));
  *out = scratch;
  return OMX_OK;
}

int32_t forward(onano* t) {
  omx_ctx* ctx = t->ctx;
  const onano_config& c = t->c;
  const uint64_t N = t->N, d = c.n_embd, B = c.batch, T = c.seq, H = c.heads, KV = c.kv_heads, D = c.head_dim,
                 Hd = c.hidden, W = c.window;
  const uint64_t qd = H * D, kd = KV * D;
  const int32_t AD = t->AD, LD = t->LD;
  const float eps = c.rms_eps;
  // x = tok_emb[ids], then norm1 of block 0 (or the final norm of a model without blocks).
  {
    float* x = t->layers.empty() ? t->x_final : t->layers[0].x;
    void* h = t->layers.empty() ? t->hf : t->layers[0].h;
    TRY(omx_embedding_forward(ctx, t->w32(0), OMX_F32, t->ids, x, OMX_F32, N, c.vocab, d));
    TRY(omx_rms_norm_forward(ctx, x, OMX_F32, t->w32(t->layers.empty() ? t->nf() : t->li(0, NORM1)), h, AD, N, d, eps));
  }
  for (uint32_t l = 0; l < c.layers; ++l) {
    onano::Layer& A = t->layers[l];
    const bool last = l + 1 == c.layers;
    float* x_next = last ? t->x_final : t->layers[l + 1].x;
    void* h_next = last ? t->hf : t->layers[l + 1].h;
    const float* next_norm = t->w32(last ? t->nf() : t->li(l + 1, NORM1));
    if (t->fused_qkv) {
      const uint64_t P3 = qd + 2 * kd;
      char* prepared = static_cast<char*>(A.qkv);
      TRY(omx_linear_forward(ctx, A.h, AD, t->w(t->li(l, WQ)), AD, A.qkv_lin, LD, N, d, P3));
      // Block 0 has no earlier value to blend with (block.rs:232-238).
      TRY(omx_qkv_prepare_forward(ctx, A.qkv_lin, LD, A.qkv, P3, t->w32(t->li(l, QNORM)), t->w32(t->li(l, KNORM)), t->cos_t,
                                  t->sin_t, l > 0 ? t->layers[0].qkv_lin : nullptr,
                                  l > 0 ? t->w32(t->li(l, LAMBDA)) : nullptr, N, T, H, KV, D, eps));
      TRY(omx_causal_attention_forward_saving(ctx, prepared, P3, prepared + qd * 2, prepared + (qd + kd) * 2, P3, AD, A.ap,
                                              A.apr, qd, AD, A.lse, B, T, H, KV, D, W));
    } else {
    TRY(omx_linear_forward(ctx, A.h, AD, t->w(t->li(l, WQ)), AD, A.q_lin, LD, N, d, qd));
    TRY(omx_linear_forward(ctx, A.h, AD, t->w(t->li(l, WK)), AD, A.k_lin, LD, N, d, kd));
    TRY(omx_linear_forward(ctx, A.h, AD, t->w(t->li(l, WV)), AD, A.raw_v, AD, N, d, kd));
    TRY(omx_rms_qk_norm_forward(ctx, A.q_lin, A.k_lin, LD, t->w32(t->li(l, QNORM)), t->w32(t->li(l, KNORM)), t->t_q,
                                t->t_k, AD, N * H, N * KV, D, eps));
    TRY(omx_rope_half_split_forward(ctx, t->t_q, t->cos_t, t->sin_t, A.q, AD, N * H, D, T, H));
    TRY(omx_rope_half_split_forward(ctx, t->t_k, t->cos_t, t->sin_t, A.k, AD, N * KV, D, T, KV));
    // Block 0 has no earlier value to blend with (block.rs:232-238).
    if (l > 0)
      TRY(omx_value_residual_blend_forward(ctx, A.raw_v, t->layers[0].raw_v, t->w32(t->li(l, LAMBDA)), A.v, AD, N * kd));
    if (t->flash) {
      // The output's rounding residual is kept for the backward's row term, as the reference keeps
      // its saved output unrounded (ojas-core/src/autocast.rs:177-186).
      TRY(omx_causal_attention_forward_saving(ctx, A.q, qd, A.k, A.v, kd, AD, A.ap, A.apr, qd, AD, A.lse, B, T, H, KV, D,
                                              W));
    } else {
      TRY(omx_permute_0213(ctx, A.q, A.qp, AD, B, T, H, D));
      TRY(omx_permute_0213(ctx, A.k, A.kp, AD, B, T, KV, D));
      TRY(omx_permute_0213(ctx, A.v, A.vp, AD, B, T, KV, D));
      TRY(omx_causal_sdpa_forward(ctx, A.qp, A.kp, A.vp, AD, A.att, AD, A.lse, B, H, KV, T, D, W));
      TRY(omx_permute_0213(ctx, A.att, A.ap, AD, B, H, T, D));
    }
    }
    // The row-kernel attention keeps no rounding residual: the gate then reads what was stored.
    const bool gate_f32 = t->keep_f32 && t->flash;
    const void* attn = A.ap;
    if (gate_f32) {  // the gate reads the attention output at 16 bits of mantissa: what was stored plus what that dropped
      TRY(omx_residual_add(ctx, A.ap, AD, A.apr, AD, t->ap32, OMX_F32, N * qd));
      attn = t->ap32;
    }
    TRY(omx_per_head_sigmoid_gate_forward(ctx, A.h, t->w(t->li(l, GATE_W)), AD, t->w32(t->li(l, GATE_B)), attn,
                                          gate_f32 ? OMX_F32 : AD, A.y, AD, A.gates, N, d, H, D));
    TRY(omx_linear_forward(ctx, A.y, AD, t->w(t->li(l, WO)), AD, t->t_f, LD, N, qd, d));
    TRY(omx_residual_add_rms_norm_forward(ctx, A.x, OMX_F32, t->t_f, LD, t->w32(t->li(l, NORM2)), A.x1, A.h2, AD, N, d,
                                          eps));
    if (t->fused_mlp) {
      TRY(omx_linear_forward(ctx, A.h2, AD, t->w(t->li(l, FFN_GATE)), AD, A.gu, LD, N, d, 2 * Hd));
      TRY(omx_swiglu_forward(ctx, A.gu, A.m, LD, N, Hd));
    } else {
      TRY(omx_linear_forward(ctx, A.h2, AD, t->w(t->li(l, FFN_GATE)), AD, A.g_lin, AD, N, d, Hd));
      TRY(omx_silu_forward(ctx, A.g_lin, A.g_act, AD, N * Hd));
      TRY(omx_linear_forward(ctx, A.h2, AD, t->w(t->li(l, FFN_UP)), AD, A.up, AD, N, d, Hd));
      TRY(omx_mul_forward(ctx, A.g_act, A.up, A.m, AD, N * Hd));
    }
    TRY(omx_linear_forward(ctx, A.m, AD, t->w(t->li(l, FFN_DOWN)), AD, t->t_f, LD, N, Hd, d));
    TRY(omx_residual_add_rms_norm_forward(ctx, A.x1, OMX_F32, t->t_f, LD, next_norm, x_next, h_next, AD, N, d, eps));
  }
  return OMX_OK;
}

int32_t backward(onano* t, float loss_seed) {
  omx_ctx* ctx = t->ctx;
  const onano_config& c = t->c;
  const uint64_t N = t->N, d = c.n_embd, B = c.batch, T = c.seq, H = c.heads, KV = c.kv_heads, D = c.head_dim,
                 Hd = c.hidden, W = c.window;
  const uint64_t qd = H * D, kd = KV * D;
  const int32_t AD = t->AD, LD = t->LD;
  const float eps = c.rms_eps;
  const uint64_t chunk_rows = N < 16384 ? N : 16384;
  TRY(omx_linear_cross_entropy_mean(ctx, t->hf, t->w(0), AD, t->targets, N, d, c.vocab, 0, 0, chunk_rows, c.vocab,
                                    t->loss, t->ghf, AD, t->g(0)));
  if (loss_seed != 1.0f) {
    // The backward starts from the micro-batch's weight: every gradient is linear in it.
    if (AD == OMX_F32) {
      TRY(omx_scale_grad(ctx, t->ghf, loss_seed, N * d));
    } else {
      TRY(omx_to_f32(ctx, t->ghf, t->gres1, N * d));
      TRY(omx_scale_grad(ctx, t->gres1, loss_seed, N * d));
      TRY(omx_to_bf16(ctx, t->gres1, t->ghf, N * d));
    }
    TRY(omx_scale_grad(ctx, t->g(0), loss_seed, static_cast<uint64_t>(c.vocab) * d));
  }
  TRY(omx_rms_norm_backward(ctx, t->x_final, OMX_F32, t->w32(t->nf()), t->ghf, AD, t->gres, OMX_F32, t->g(t->nf()), N, d,
                            eps));
  const bool defer = t->deferred_dw;  // implies the bf16 tier
  auto slice = [&](void* all, uint64_t l, uint64_t per_layer) {
    return static_cast<void*>(static_cast<char*>(all) + l * per_layer * t->asz);
  };
  const void* gy = nullptr;
  TRY(to_operand(t, t->gres, defer ? slice(t->gyd_all, c.layers - 1, N * d) : t->gy16, N * d, &gy));
  void* copy16 = AD == OMX_BF16 ? t->gy16 : nullptr;
  bool have_g_v0 = false;
  for (uint32_t l = c.layers; l-- > 0;) {
    onano::Layer& A = t->layers[l];
    // Where this block's output gradients go: scratch, or the block's slice of the stacked buffers.
    void* ggu = defer ? slice(t->ggu_all, l, 2 * N * Hd) : t->ggu;
    void* gq_lin = defer ? slice(t->gq_all, l, N * qd) : t->gq;
    void* gk_lin = defer ? slice(t->gk_all, l, N * kd) : t->gk;
    void* g_raw_v_out = defer ? slice(t->gv_all, l, N * kd) : t->g_raw_v;
    // Where the two norm backwards of this block leave the bf16 copy of the gradient they produce:
    // the operand of this block's o projection, and of the block below's down projection.
    void* copy_o = defer ? slice(t->gyo_all, l, N * d) : copy16;
    void* copy_below = defer && l > 0 ? slice(t->gyd_all, l - 1, N * d) : copy16;
    // Weight gradients go to the arena now, or wait for the batched products after the loop.
    auto gw = [&](uint64_t which) { return defer ? nullptr : t->g(t->li(l, which)); };
    // x_next = x1 + down(silu(gate(h2)) * up(h2))
    TRY(omx_linear_backward(ctx, A.m, t->w(t->li(l, FFN_DOWN)), gy, AD, t->gm, AD, gw(FFN_DOWN), OMX_F32, N, Hd, d));
    if (t->fused_mlp) {
      TRY(omx_swiglu_backward(ctx, A.gu, t->gm, ggu, LD, N, Hd));
      // One product for both projections: their input gradients add in its f32 accumulators.
      TRY(omx_linear_backward(ctx, A.h2, t->w(t->li(l, FFN_GATE)), ggu, AD, t->t_a, AD, gw(FFN_GATE), OMX_F32, N, d,
                              2 * Hd));
      TRY(omx_rms_norm_backward_residual(ctx, A.x1, OMX_F32, t->w32(t->li(l, NORM2)), t->t_a, AD, t->gres, t->gres1, copy_o,
                                         t->g(t->li(l, NORM2)), N, d, eps));
    } else {
      TRY(omx_mul_backward(ctx, A.g_act, A.up, t->gm, t->g_gact, t->g_up, AD, N * Hd));
      TRY(omx_linear_backward(ctx, A.h2, t->w(t->li(l, FFN_UP)), t->g_up, AD, t->t_a, AD, t->g(t->li(l, FFN_UP)), OMX_F32, N,
                              d, Hd));
      TRY(omx_silu_backward(ctx, A.g_lin, t->g_gact, t->gm, AD, N * Hd));  // gm is free again: the gradient of g_lin
      // gy16 is free here too: the down projection above was the last reader of the operand copy.
      TRY(omx_linear_backward(ctx, A.h2, t->w(t->li(l, FFN_GATE)), t->gm, AD, t->gy16, AD, t->g(t->li(l, FFN_GATE)), OMX_F32,
                              N, d, Hd));
      TRY(omx_residual_add(ctx, t->t_a, AD, t->gy16, AD, t->gh, OMX_F32, N * d));
      TRY(omx_rms_norm_backward_residual(ctx, A.x1, OMX_F32, t->w32(t->li(l, NORM2)), t->gh, OMX_F32, t->gres, t->gres1,
                                         copy16, t->g(t->li(l, NORM2)), N, d, eps));
    }
    gy = AD == OMX_BF16 ? static_cast<const void*>(t->fused_mlp ? copy_o : copy16) : static_cast<const void*>(t->gres1);
    // x1 = x + o(gate(h) * attention)
    // The gate's backward takes the attention output and the gradient of its own output in one
    // dtype: both f32 when the forward kept the output's dropped bits.
    const bool gate_f32 = t->keep_f32 && t->flash;
    const int32_t GD = gate_f32 ? OMX_F32 : AD;
    const void* attn = A.ap;
    if (gate_f32) {
      TRY(omx_residual_add(ctx, A.ap, AD, A.apr, AD, t->ap32, OMX_F32, N * qd));
      attn = t->ap32;
    }
    TRY(omx_linear_backward(ctx, A.y, t->w(t->li(l, WO)), gy, AD, t->gyy, GD, gw(WO), OMX_F32, N, qd, d));
    if (defer && t->gz_all)  // the gate's weight gradient waits for the batched product below
      TRY(omx_per_head_sigmoid_gate_backward_deferred(ctx, A.h, t->w(t->li(l, GATE_W)), AD, t->w32(t->li(l, GATE_B)), attn,
                                                      GD, t->gyy, GD, A.gates, t->fused_qkv ? nullptr : t->gh, OMX_F32,
                                                      slice(t->gz_all, l, N * H),
                                                      t->g(t->li(l, GATE_B)), t->gap, AD, N, d, H, D));
    else
      TRY(omx_per_head_sigmoid_gate_backward(ctx, A.h, t->w(t->li(l, GATE_W)), AD, t->w32(t->li(l, GATE_B)), attn, GD,
                                             t->gyy, GD, A.gates, t->gh, OMX_F32, t->g(t->li(l, GATE_W)),
                                             t->g(t->li(l, GATE_B)), t->gap, AD, N, d, H, D));
    if (t->fused_qkv) {
      const uint64_t P3 = qd + 2 * kd;
      char* prepared = static_cast<char*>(A.qkv);
      char* gp = static_cast<char*>(t->g_qkv);
      void* g_lin = defer ? slice(t->gqkv_all, l, N * P3) : t->g_qkv_lin;
      TRY(omx_causal_attention_backward_saved(ctx, prepared, P3, prepared + qd * 2, prepared + (qd + kd) * 2, P3, A.ap, A.apr,
                                              t->gap, qd, A.lse, AD, gp, gp + qd * 2, gp + (qd + kd) * 2, AD, B, T, H, KV, D,
                                              W));
      // Block 0's value also feeds every later block's blend: their shares collect in v0_acc (the
      // last block writes it, the others add) and join block 0's own gradient here.
      const bool blends = l > 0, last = l + 1 == c.layers;
      TRY(omx_qkv_prepare_backward(ctx, A.qkv_lin, LD, t->g_qkv, g_lin, P3, t->w32(t->li(l, QNORM)), t->w32(t->li(l, KNORM)),
                                   t->cos_t, t->sin_t, blends ? t->layers[0].qkv_lin : nullptr,
                                   blends ? t->w32(t->li(l, LAMBDA)) : nullptr, blends ? t->v0_acc : nullptr, last ? 1 : 0,
                                   !blends && c.layers > 1 ? t->v0_acc : nullptr, t->g(t->li(l, QNORM)),
                                   t->g(t->li(l, KNORM)), blends ? t->g(t->li(l, LAMBDA)) : nullptr, N, T, H, KV, D, eps));
      if (!blends) TRY(omx_fill_zero(ctx, t->g(t->li(0, LAMBDA)), 4));
      // One product for the three projections: their input gradients add in its f32 accumulators.
      TRY(omx_linear_backward(ctx, A.h, t->w(t->li(l, WQ)), g_lin, AD, t->t_a, AD, gw(WQ), OMX_F32, N, d, P3));
      if (defer && t->gz_all)  // the gate's input gradient, left out above, joins here in one pass
        TRY(omx_per_head_sigmoid_gate_input_grad_add(ctx, slice(t->gz_all, l, N * H), t->w(t->li(l, GATE_W)), AD, t->t_a,
                                                     AD, t->gh, N, d, H));
      else
        TRY(omx_residual_add(ctx, t->gh, OMX_F32, t->t_a, AD, t->gh, OMX_F32, N * d));
      TRY(omx_rms_norm_backward_residual(ctx, A.x, OMX_F32, t->w32(t->li(l, NORM1)), t->gh, OMX_F32, t->gres1, t->gres,
                                         copy_below, t->g(t->li(l, NORM1)), N, d, eps));
      gy = static_cast<const void*>(copy_below);
      continue;
    }
    if (t->flash) {
      TRY(omx_causal_attention_backward_saved(ctx, A.q, qd, A.k, A.v, kd, A.ap, A.apr, t->gap, qd, A.lse, AD, t->gq, t->gk,
                                              t->gv, AD, B, T, H, KV, D, W));
    } else {
      TRY(omx_permute_0213(ctx, t->gap, t->gap_p, AD, B, T, H, D));
      TRY(omx_causal_sdpa_backward(ctx, A.qp, A.kp, A.vp, A.att, A.lse, t->gap_p, AD, AD, AD, t->gqp, t->gkp, t->gvp, AD, B,
                                   H, KV, T, D, W));
      TRY(omx_permute_0213(ctx, t->gvp, t->gv, AD, B, KV, T, D));
      TRY(omx_permute_0213(ctx, t->gkp, t->gk, AD, B, KV, T, D));
      TRY(omx_permute_0213(ctx, t->gqp, t->gq, AD, B, H, T, D));
    }
    // The value: block 0's raw v also feeds every later block's blend.
    const void* g_raw_v = t->gv;
    if (l == 0) {
      if (have_g_v0) {
        TRY(omx_residual_add(ctx, t->g_v0, AD, t->gv, AD, g_raw_v_out, AD, N * kd));
        g_raw_v = g_raw_v_out;
      }
      TRY(omx_fill_zero(ctx, t->g(t->li(0, LAMBDA)), 4));
    } else {
      void* to_v0 = have_g_v0 ? t->part_v0 : t->g_v0;
      TRY(omx_value_residual_blend_backward(ctx, A.raw_v, t->layers[0].raw_v, t->w32(t->li(l, LAMBDA)), t->gv, g_raw_v_out,
                                            to_v0, AD, t->g(t->li(l, LAMBDA)), N * kd));
      if (have_g_v0) TRY(omx_residual_add(ctx, t->g_v0, AD, t->part_v0, AD, t->g_v0, AD, N * kd));
      have_g_v0 = true;
      g_raw_v = g_raw_v_out;
    }
    TRY(omx_rope_half_split_backward(ctx, t->gk, t->cos_t, t->sin_t, t->t_k, AD, N * KV, D, T, KV));
    TRY(omx_rope_half_split_backward(ctx, t->gq, t->cos_t, t->sin_t, t->t_q, AD, N * H, D, T, H));
    TRY(omx_rms_qk_norm_backward(ctx, A.q_lin, A.k_lin, LD, t->w32(t->li(l, QNORM)), t->w32(t->li(l, KNORM)), t->t_q, t->t_k,
                                 AD, gq_lin, gk_lin, AD, t->g(t->li(l, QNORM)), t->g(t->li(l, KNORM)), N * H, N * KV, D, eps));
    // h feeds the gate, v, k and q; their gradients arrive in that order (the later consumer first).
    struct Proj {
      uint64_t which, out;
      const void* gy;
    } projections[3] = {{WV, kd, g_raw_v}, {WK, kd, gk_lin}, {WQ, qd, gq_lin}};
    for (const Proj& p : projections) {
      TRY(omx_linear_backward(ctx, A.h, t->w(t->li(l, p.which)), p.gy, AD, t->t_a, AD, gw(p.which), OMX_F32, N, d, p.out));
      TRY(omx_residual_add(ctx, t->gh, OMX_F32, t->t_a, AD, t->gh, OMX_F32, N * d));
    }
    TRY(omx_rms_norm_backward_residual(ctx, A.x, OMX_F32, t->w32(t->li(l, NORM1)), t->gh, OMX_F32, t->gres1, t->gres,
                                       copy_below, t->g(t->li(l, NORM1)), N, d, eps));
    gy = AD == OMX_BF16 ? static_cast<const void*>(copy_below) : static_cast<const void*>(t->gres);
  }
  if (defer) {
    // gw[l](o, j) = sum_r gy[l][r, o] * x[l][r, j] for every block l, one launch per weight.
    const uint64_t layers = c.layers, per_layer = t->slots[t->li(1, WQ)].offset - t->slots[t->li(0, WQ)].offset;
    struct Deferred {
      const void *gy, *x;
      uint64_t which, out, in;
    } products[6] = {{t->gyd_all, t->m_all, FFN_DOWN, d, Hd}, {t->ggu_all, t->h2_all, FFN_GATE, 2 * Hd, d},
                     {t->gyo_all, t->y_all, WO, d, qd},       {t->gv_all, t->h_all, WV, kd, d},
                     {t->gk_all, t->h_all, WK, kd, d},        {t->gq_all, t->h_all, WQ, qd, d}};
    if (t->fused_qkv) products[3] = {t->gqkv_all, t->h_all, WQ, qd + 2 * kd, d};
    const int count = t->fused_qkv ? 4 : 6;
    for (int i = 0; i < count; ++i) {
      const Deferred& p = products[i];
      TRY(omx_gemm_strided_batch(ctx, p.gy, 1, p.out, p.x, p.in, 1, AD, t->g(t->li(0, p.which)), OMX_F32, p.out, N, p.in, 0,
                                 layers, N * p.out, N * p.in, per_layer));
    }
    // The gates' weight gradients: heads x d each over all tokens, every block in one launch.
    if (t->gz_all)
      TRY(omx_gemm_strided_batch(ctx, t->gz_all, 1, H, t->h_all, d, 1, AD, t->g(t->li(0, GATE_W)), OMX_F32, H, N, d, 0, layers,
                               N * H, N * d, per_layer));
  }
  // The tied table: the head's gradient first, then the embedding's rows.
  // The tied table: the gather's gradient joins the head's where it lies, row by named row.
  TRY(omx_embedding_backward_accumulate(ctx, t->ids, t->gres, OMX_F32, t->g(0), N, c.vocab, d));
  return OMX_OK;
}

int32_t micro_batch(onano* t, float loss_seed, float loss_scale, int32_t first) {
  t->gdst = first ? t->acc : t->g32;
  TRY(forward(t));
  TRY(backward(t, loss_seed));
  if (loss_scale != 1.0f) TRY(omx_scale_grad(t->ctx, t->loss, loss_scale, 1));
  if (first) {
    TRY(omx_copy(t->ctx, t->loss_acc, t->loss, 4));
  } else {
    TRY(omx_accumulate_grad(t->ctx, t->acc, t->g32, t->P));
    TRY(omx_accumulate_grad(t->ctx, t->loss_acc, t->loss, 1));
  }
  return OMX_OK;
}

}  // namespace

extern "C" {

int32_t onano_create(omx_ctx* ctx, const onano_config* config, onano** out) {
  if (!ctx || !config || !out) return OMX_BACKEND;
  *out = nullptr;
  const onano_config& c = *config;
  if (c.n_embd == 0 || c.heads == 0 || c.kv_heads == 0 || c.head_dim == 0 || c.hidden == 0 || c.vocab == 0 ||
      c.batch == 0 || c.seq == 0)
    return OMX_SHAPE;
  if (c.heads % c.kv_heads != 0 || c.head_dim % 2 != 0) return OMX_SHAPE;
  if ((static_cast<uint64_t>(c.n_embd) * c.hidden) % kAlign != 0) return OMX_SHAPE;
  onano* t = new onano();
  t->ctx = ctx;
  t->c = c;
  t->AD = c.bf16 ? OMX_BF16 : OMX_F32;
  t->asz = c.bf16 ? 2 : 4;
  t->N = static_cast<uint64_t>(c.batch) * c.seq;
  t->flash = c.bf16 && (c.head_dim == 64 || c.head_dim == 128);
  t->fused_mlp = c.bf16 && c.hidden % 8 == 0;
  t->deferred_dw = t->fused_mlp && c.layers > 1;
  // The three projections are one matrix only if nothing pads the arena between them.
  t->fused_qkv = t->flash && (static_cast<uint64_t>(c.heads) * c.head_dim * c.n_embd) % kAlign == 0 &&
                 (static_cast<uint64_t>(c.kv_heads) * c.head_dim * c.n_embd) % kAlign == 0;
  t->keep_f32 = c.bf16 && t->fused_mlp;
  t->LD = t->keep_f32 ? OMX_F32 : t->AD;
  t->lsz = t->keep_f32 ? 4 : t->asz;
  const uint64_t N = t->N, d = c.n_embd, H = c.heads, KV = c.kv_heads, D = c.head_dim, Hd = c.hidden;
  const uint64_t qd = H * D, kd = KV * D;
  // Arena order (the parameter indices keep the order of names.rs): the table, then every vector of
  // every block and the final norm side by side (one AdamW pass covers them), block 0's vr_lambda
  // last among them (no gradient reaches it and no optimizer touches it), then the matrices block
  // by block at a fixed stride.
  struct Shape {
    uint64_t rows, cols;
  };
  std::vector<Shape> shapes;
  shapes.push_back({c.vocab, d});
  for (uint32_t l = 0; l < c.layers; ++l) {
    const Shape block[kPerBlock] = {{d, 0}, {qd, d}, {kd, d}, {kd, d}, {d, qd}, {D, 0}, {D, 0}, {H, d}, {H, 0}, {1, 0},
                                    {d, 0}, {Hd, d}, {Hd, d}, {d, Hd}};
    shapes.insert(shapes.end(), block, block + kPerBlock);
  }
  shapes.push_back({d, 0});
  t->slots.resize(shapes.size());
  uint64_t at = 0;
  auto place = [&](uint64_t i) {
    const uint64_t len = shapes[i].cols ? shapes[i].rows * shapes[i].cols : shapes[i].rows;
    t->slots[i] = {at, len, shapes[i].rows, shapes[i].cols};
    at += (len + kAlign - 1) / kAlign * kAlign;
  };
  const uint64_t frozen = 1 + LAMBDA;
  place(0);
  for (uint64_t i = 1; i < shapes.size(); ++i)
    if (shapes[i].cols == 0 && i != frozen) place(i);
  t->adam_end = at;
  place(frozen);
  for (uint64_t i = 1; i < shapes.size(); ++i)
    if (shapes[i].cols != 0) place(i);
  t->P = at;
#define CREATE_TRY(expr)           \
  do {                             \
    int32_t rc_ = (expr);          \
    if (rc_ != OMX_OK) {           \
      onano_destroy(t);            \
      return rc_;                  \
    }                              \
  } while (0)
  float** arenas[5] = {&t->p32, &t->acc, &t->g32, &t->m1, &t->m2};
  for (float** a : arenas) {
    CREATE_TRY(alloc_t(t, t->P, a));
    CREATE_TRY(omx_fill_zero(ctx, *a, t->P * 4));
  }
  t->gdst = t->acc;
  if (c.bf16) {
    CREATE_TRY(alloc(t, t->P * 2, &t->p16));
    CREATE_TRY(omx_fill_zero(ctx, t->p16, t->P * 2));
  }
  CREATE_TRY(alloc_t(t, N, &t->ids));
  CREATE_TRY(alloc_t(t, N, &t->targets));
  {
    void* block = nullptr;
    CREATE_TRY(alloc(t, 256, &block));
    CREATE_TRY(omx_fill_zero(ctx, block, 256));
    t->loss = static_cast<float*>(block);
    t->loss_acc = t->loss + 16;
    t->unbounded = t->loss_acc + 1;
  }
  {
    // Rope::rows (ojas-model/src/block.rs:31-71): angles in f64, one rounding to f32, both halves
    // of a row equal.
    const uint64_t half = D / 2;
    std::vector<float> cs(c.seq * D), sn(c.seq * D);
    for (uint64_t p = 0; p < c.seq; ++p)
      for (uint64_t i = 0; i < half; ++i) {
        const double inv = std::pow(c.rope_base, -static_cast<double>(2 * i) / static_cast<double>(D));
        const double ang = static_cast<double>(p) * inv;
        cs[p * D + i] = cs[p * D + half + i] = static_cast<float>(std::cos(ang));
        sn[p * D + i] = sn[p * D + half + i] = static_cast<float>(std::sin(ang));
      }
    CREATE_TRY(alloc_t(t, c.seq * D, &t->cos_t));
    CREATE_TRY(alloc_t(t, c.seq * D, &t->sin_t));
    CREATE_TRY(omx_upload(ctx, t->cos_t, 0, cs.data(), cs.size() * 4));
    CREATE_TRY(omx_upload(ctx, t->sin_t, 0, sn.data(), sn.size() * 4));
  }
  t->layers.resize(c.layers);
  const uint64_t L = c.layers;
  if (t->deferred_dw) {
    CREATE_TRY(alloc_act(t, L * N * d, &t->h_all));
    CREATE_TRY(alloc_act(t, L * N * qd, &t->y_all));
    CREATE_TRY(alloc_act(t, L * N * d, &t->h2_all));
    CREATE_TRY(alloc_act(t, L * N * Hd, &t->m_all));
    CREATE_TRY(alloc_act(t, L * N * d, &t->gyd_all));
    CREATE_TRY(alloc_act(t, L * 2 * N * Hd, &t->ggu_all));
    CREATE_TRY(alloc_act(t, L * N * d, &t->gyo_all));
    // (a strided batch wants its products 16 bytes apart at least)
    if ((N * c.heads * t->asz) % 16 == 0) CREATE_TRY(alloc_act(t, L * N * c.heads, &t->gz_all));
    if (t->fused_qkv) {
      CREATE_TRY(alloc_act(t, L * N * (qd + 2 * kd), &t->gqkv_all));
    } else {
      CREATE_TRY(alloc_act(t, L * N * qd, &t->gq_all));
      CREATE_TRY(alloc_act(t, L * N * kd, &t->gk_all));
      CREATE_TRY(alloc_act(t, L * N * kd, &t->gv_all));
    }
  }
  uint32_t index = 0;
  for (auto& A : t->layers) {
    const uint64_t l = index;
    const bool first = index++ == 0;
    std::memset(&A, 0, sizeof(A));
    auto stacked = [&](void* all, uint64_t per_layer) { return static_cast<void*>(static_cast<char*>(all) + l * per_layer * t->asz); };
    CREATE_TRY(alloc_t(t, N * d, &A.x));
    CREATE_TRY(alloc_t(t, N * d, &A.x1));
    if (t->deferred_dw) {
      A.h = stacked(t->h_all, N * d);
      A.y = stacked(t->y_all, N * qd);
      A.h2 = stacked(t->h2_all, N * d);
      A.m = stacked(t->m_all, N * Hd);
    } else {
      CREATE_TRY(alloc_act(t, N * d, &A.h));
      CREATE_TRY(alloc_act(t, N * qd, &A.y));
      CREATE_TRY(alloc_act(t, N * d, &A.h2));
      CREATE_TRY(alloc_act(t, N * Hd, &A.m));
    }
    if (t->fused_qkv) {
      CREATE_TRY(alloc(t, N * (qd + 2 * kd) * t->lsz, &A.qkv_lin));
      CREATE_TRY(alloc_act(t, N * (qd + 2 * kd), &A.qkv));
    } else {
      CREATE_TRY(alloc(t, N * qd * t->lsz, &A.q_lin));
      CREATE_TRY(alloc(t, N * kd * t->lsz, &A.k_lin));
      CREATE_TRY(alloc_act(t, N * qd, &A.q));
      CREATE_TRY(alloc_act(t, N * kd, &A.k));
      CREATE_TRY(alloc_act(t, N * kd, &A.raw_v));
      if (first) A.v = A.raw_v;
      else CREATE_TRY(alloc_act(t, N * kd, &A.v));
    }
    CREATE_TRY(alloc_act(t, N * qd, &A.ap));
    if (t->fused_mlp) {
      CREATE_TRY(alloc(t, 2 * N * Hd * t->lsz, &A.gu));
    } else {
      CREATE_TRY(alloc_act(t, N * Hd, &A.g_lin));
      CREATE_TRY(alloc_act(t, N * Hd, &A.up));
      CREATE_TRY(alloc_act(t, N * Hd, &A.g_act));
    }
    if (t->flash) {
      CREATE_TRY(alloc_act(t, N * qd, &A.apr));
    } else {
      CREATE_TRY(alloc_act(t, N * qd, &A.qp));
      CREATE_TRY(alloc_act(t, N * kd, &A.kp));
      CREATE_TRY(alloc_act(t, N * kd, &A.vp));
      CREATE_TRY(alloc_act(t, N * qd, &A.att));
    }
    CREATE_TRY(alloc_t(t, static_cast<uint64_t>(c.batch) * H * c.seq, &A.lse));
    CREATE_TRY(alloc_t(t, N * H, &A.gates));
  }
  CREATE_TRY(alloc_t(t, N * d, &t->x_final));
  CREATE_TRY(alloc_act(t, N * d, &t->hf));
  CREATE_TRY(alloc_act(t, N * qd, &t->t_q));
  CREATE_TRY(alloc_act(t, N * kd, &t->t_k));
  CREATE_TRY(alloc_act(t, N * (d > qd ? d : qd), &t->t_a));
  CREATE_TRY(alloc(t, N * d * t->lsz, &t->t_f));
  if (t->keep_f32 && t->flash) CREATE_TRY(alloc_t(t, N * qd, &t->ap32));
  CREATE_TRY(alloc_act(t, N * Hd, &t->gm));
  if (t->fused_mlp) {
    if (!t->deferred_dw) CREATE_TRY(alloc_act(t, 2 * N * Hd, &t->ggu));
  } else {
    CREATE_TRY(alloc_act(t, N * Hd, &t->g_gact));
    CREATE_TRY(alloc_act(t, N * Hd, &t->g_up));
  }
  if (t->fused_qkv) {
    CREATE_TRY(alloc_act(t, N * (qd + 2 * kd), &t->g_qkv));
    if (!t->deferred_dw) CREATE_TRY(alloc_act(t, N * (qd + 2 * kd), &t->g_qkv_lin));
    CREATE_TRY(alloc_t(t, N * kd, &t->v0_acc));
  }
  CREATE_TRY(alloc(t, N * qd * (t->keep_f32 && t->flash ? 4 : t->asz), &t->gyy));
  CREATE_TRY(alloc_act(t, N * qd, &t->gap));
  CREATE_TRY(alloc_act(t, N * qd, &t->gq));
  CREATE_TRY(alloc_act(t, N * kd, &t->gk));
  CREATE_TRY(alloc_act(t, N * kd, &t->gv));
  CREATE_TRY(alloc_act(t, N * kd, &t->g_raw_v));
  CREATE_TRY(alloc_act(t, N * kd, &t->part_v0));
  CREATE_TRY(alloc_act(t, N * kd, &t->g_v0));
  if (!t->flash) {
    CREATE_TRY(alloc_act(t, N * qd, &t->gqp));
    CREATE_TRY(alloc_act(t, N * kd, &t->gkp));
    CREATE_TRY(alloc_act(t, N * kd, &t->gvp));
    CREATE_TRY(alloc_act(t, N * qd, &t->gap_p));
  }
  CREATE_TRY(alloc_act(t, N * d, &t->gy16));
  CREATE_TRY(alloc_act(t, N * d, &t->ghf));
  CREATE_TRY(alloc_t(t, N * d, &t->gres));
  CREATE_TRY(alloc_t(t, N * d, &t->gres1));
  CREATE_TRY(alloc_t(t, N * d, &t->gh));
#undef CREATE_TRY
  *out = t;
  return OMX_OK;
}

void onano_destroy(onano* t) {
  if (!t) return;
  for (void* p : t->owned) omx_free(t->ctx, p);
  delete t;
}

uint64_t onano_param_count(onano* t) { return t ? t->slots.size() : 0; }
uint64_t onano_param_len(onano* t, uint64_t index) { return (t && index < t->slots.size()) ? t->slots[index].len : 0; }
uint64_t onano_steps(onano* t) { return t ? t->steps : 0; }
uint64_t onano_device_bytes(onano* t) { return t ? t->device_bytes : 0; }

int32_t onano_set_steps(onano* t, uint64_t steps) {
  if (!t) return OMX_BACKEND;
  t->steps = steps;
  return OMX_OK;
}

int32_t onano_set_param(onano* t, uint64_t index, const float* host) {
  if (!t || index >= t->slots.size() || !host) return OMX_SHAPE;
  const Slot& s = t->slots[index];
  t->tracked = false;
  TRY(omx_upload(t->ctx, t->p32, s.offset * 4, host, s.len * 4));
  if (t->p16) TRY(omx_to_bf16(t->ctx, t->p32 + s.offset, static_cast<uint16_t*>(t->p16) + s.offset, s.len));
  return OMX_OK;
}
int32_t onano_get_param(onano* t, uint64_t index, float* host) {
  if (!t || index >= t->slots.size() || !host) return OMX_SHAPE;
  const Slot& s = t->slots[index];
  return omx_download(t->ctx, host, t->p32, s.offset * 4, s.len * 4);
}
int32_t onano_get_grad(onano* t, uint64_t index, float* host) {
  if (!t || index >= t->slots.size() || !host) return OMX_SHAPE;
  const Slot& s = t->slots[index];
  return omx_download(t->ctx, host, t->acc, s.offset * 4, s.len * 4);
}
int32_t onano_get_state(onano* t, uint64_t index, uint32_t slot, float* host) {
  if (!t || index >= t->slots.size() || !host || slot > 1) return OMX_SHAPE;
  const Slot& s = t->slots[index];
  return omx_download(t->ctx, host, slot == 0 ? t->m1 : t->m2, s.offset * 4, s.len * 4);
}
int32_t onano_set_state(onano* t, uint64_t index, uint32_t slot, const float* host) {
  if (!t || index >= t->slots.size() || !host || slot > 1) return OMX_SHAPE;
  const Slot& s = t->slots[index];
  t->tracked = false;
  return omx_upload(t->ctx, slot == 0 ? t->m1 : t->m2, s.offset * 4, host, s.len * 4);
}

int32_t onano_init(onano* t, uint64_t seed) {
  if (!t) return OMX_BACKEND;
  std::mt19937_64 rng(seed);
  std::normal_distribution<float> normal(0.0f, 0.02f);
  std::vector<float> host;
  for (uint64_t i = 0; i < t->slots.size(); ++i) {
    const Slot& s = t->slots[i];
    host.resize(s.len);
    const uint64_t which = (i == 0 || i == t->nf()) ? NORM1 : (i - 1) % kPerBlock;
    for (auto& v : host) {
      if (s.cols != 0) v = normal(rng);
      else if (i != 0 && which == GATE_B) v = 0.0f;
      else if (i != 0 && which == LAMBDA) v = 0.5f;
      else v = 1.0f;
    }
    TRY(onano_set_param(t, i, host.data()));
  }
  TRY(omx_fill_zero(t->ctx, t->m1, t->P * 4));
  TRY(omx_fill_zero(t->ctx, t->m2, t->P * 4));
  t->steps = 0;
  t->tracked = false;
  return omx_sync(t->ctx);
}

// ---------------------------------------------------------------------------------------------
// The reference's fresh init (ojas-model/src/init.rs:55-114): every parameter draws from its own
// SplitMix64 stream seeded with seed ^ fnv1a(name), through Box-Muller in f64, so a parameter's
// values depend on the seed and its name alone.
namespace {

// 64-bit FNV-1a (init.rs:15-29).
uint64_t fnv1a_64(const char* bytes, size_t n) {
  uint64_t h = 0xcbf29ce484222325ull;
  for (size_t i = 0; i < n; ++i) h = (h ^ static_cast<unsigned char>(bytes[i])) * 0x00000100000001b3ull;
  return h;
}

// SplitMix64 (ojas-kernels/src/rng.rs; CounterRng of ojas-data/src/rng.rs:10).
struct CounterStream {
  uint64_t state;
  uint64_t next() {
    state += 0x9e3779b97f4a7c15ull;
    uint64_t z = state;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
  }
};

// Standard normal values in pairs (init.rs:35-59): u1 in (0, 1], u2 in [0, 1) from the top 53 bits
// of two draws; the cosine branch is returned first, the sine branch kept for the next call.
struct NormalStream {
  CounterStream rng;
  bool has_spare = false;
  double spare = 0.0;
  double next() {
    if (has_spare) {
      has_spare = false;
      return spare;
    }
    constexpr double ulp53 = 1.0 / 9007199254740992.0;
    const double u1 = static_cast<double>((rng.next() >> 11) + 1) * ulp53;
    const double u2 = static_cast<double>(rng.next() >> 11) * ulp53;
    const double radius = std::sqrt(-2.0 * std::log(u1));
    const double angle = 6.283185307179586476925286766559 * u2;
    spare = radius * std::sin(angle);
    has_spare = true;
    return radius * std::cos(angle);
  }
};

const char* const kBlockNames[kPerBlock] = {
    "norm1.weight",        "mixer.q_proj.weight", "mixer.k_proj.weight", "mixer.v_proj.weight", "mixer.o_proj.weight",
    "mixer.q_norm.weight", "mixer.k_norm.weight", "mixer.gate.weight",   "mixer.gate.bias",     "mixer.vr_lambda",
    "norm2.weight",        "ffn.gate.weight",     "ffn.up.weight",       "ffn.down.weight"};
// The init rule of each row of the parameter table (ojas-model/src/names.rs:188-300): the output
// projections o_proj and ffn.down start at zero (:236-243, :290-296), norm weights at one, the
// gate's bias and vr_lambda at zero, every other matrix at N(0, 0.02).
const int kBlockInit[kPerBlock] = {ONANO_INIT_ONES,   ONANO_INIT_NORMAL, ONANO_INIT_NORMAL, ONANO_INIT_NORMAL, ONANO_INIT_ZEROS,
                                   ONANO_INIT_ONES,   ONANO_INIT_ONES,   ONANO_INIT_NORMAL, ONANO_INIT_ZEROS,  ONANO_INIT_ZEROS,
                                   ONANO_INIT_ONES,   ONANO_INIT_NORMAL, ONANO_INIT_NORMAL, ONANO_INIT_ZEROS};

}  // namespace

uint64_t onano_fnv1a(const char* bytes, uint64_t len) { return bytes || len == 0 ? fnv1a_64(bytes, len) : 0; }

int32_t onano_reference_init_values(const char* name, uint64_t len, int32_t init, float std_dev, uint64_t seed, float* out) {
  if (!name || (!out && len != 0)) return OMX_PLACEMENT;
  if (init == ONANO_INIT_ZEROS) {
    for (uint64_t i = 0; i < len; ++i) out[i] = 0.0f;
  } else if (init == ONANO_INIT_ONES) {
    for (uint64_t i = 0; i < len; ++i) out[i] = 1.0f;
  } else if (init == ONANO_INIT_NORMAL) {
    if (!(std::isfinite(std_dev) && std_dev > 0.0f)) return OMX_OUT_OF_RANGE;  // init.rs:101-106
    NormalStream normal{CounterStream{seed ^ fnv1a_64(name, std::strlen(name))}};
    const double sd = static_cast<double>(std_dev);  // the f32 constant widened, not the decimal 0.02
    for (uint64_t i = 0; i < len; ++i) out[i] = static_cast<float>(sd * normal.next());
  } else {
    return OMX_OUT_OF_RANGE;
  }
  return OMX_OK;
}

int32_t onano_param_name(onano* t, uint64_t index, char* out, uint64_t capacity) {
  if (!t || !out || index >= t->slots.size()) return OMX_SHAPE;
  char text[96];
  if (index == 0) std::snprintf(text, sizeof text, "tok_emb.weight");
  else if (index == t->nf()) std::snprintf(text, sizeof text, "norm_f.weight");
  else std::snprintf(text, sizeof text, "blocks.%llu.%s", static_cast<unsigned long long>((index - 1) / kPerBlock), kBlockNames[(index - 1) % kPerBlock]);
  if (std::strlen(text) + 1 > capacity) return OMX_CAPACITY_EXCEEDED;
  std::memcpy(out, text, std::strlen(text) + 1);
  return OMX_OK;
}

int32_t onano_init_reference(onano* t, uint64_t seed) {
  if (!t) return OMX_BACKEND;
  std::vector<float> host;
  char name[96];
  for (uint64_t i = 0; i < t->slots.size(); ++i) {
    const Slot& s = t->slots[i];
    host.resize(s.len);
    TRY(onano_param_name(t, i, name, sizeof name));
    const int32_t init = i == 0 ? ONANO_INIT_NORMAL : i == t->nf() ? ONANO_INIT_ONES : kBlockInit[(i - 1) % kPerBlock];
    TRY(onano_reference_init_values(name, s.len, init, 0.02f, seed, host.data()));
    TRY(onano_set_param(t, i, host.data()));
  }
  TRY(omx_fill_zero(t->ctx, t->m1, t->P * 4));
  TRY(omx_fill_zero(t->ctx, t->m2, t->P * 4));
  t->steps = 0;
  t->tracked = false;
  return omx_sync(t->ctx);
}

int32_t onano_micro_batch(onano* t, const uint32_t* ids, const uint32_t* targets, float loss_seed, float loss_scale,
                          int32_t first) {
  if (!t || !ids || !targets) return OMX_BACKEND;
  TRY(omx_upload(t->ctx, t->ids, 0, ids, t->N * 4));
  TRY(omx_upload(t->ctx, t->targets, 0, targets, t->N * 4));
  return micro_batch(t, loss_seed, loss_scale, first);
}

int32_t onano_micro_batch_resident(onano* t, float loss_seed, float loss_scale, int32_t first) {
  if (!t) return OMX_BACKEND;
  return micro_batch(t, loss_seed, loss_scale, first);
}

int32_t onano_loss(onano* t, float* loss) {
  if (!t || !loss) return OMX_BACKEND;
  return omx_read_scalar_f32(t->ctx, t->loss_acc, loss);
}

// Trainer::apply with the hybrid groups (ojas-model/src/trainer.rs:858-876, :1004-1028).
int32_t onano_apply(onano* t, const omx_muon_config* muon, const omx_adamw_config* adamw, float grad_clip, float* loss,
                    float* grad_norm) {
  if (!t || !muon || !adamw) return OMX_BACKEND;
  void* grads[1] = {t->acc};
  uint64_t lens[1] = {t->P};
  float norm = 0.0f;
  // Sync point 1: the global gradient norm is a host value (trainer.rs:821-824). The arena's
  // padding and block 0's vr_lambda hold zeros and add nothing to it.
  TRY(omx_clip_grad_norm(t->ctx, grads, lens, 1, grad_clip > 0.0f ? grad_clip : INFINITY, &norm));
  uint16_t* mirror = static_cast<uint16_t*>(t->p16);
  // AdamW: the table and every vector sit side by side at the arena's start. Its checking pass is
  // skipped when nothing in its range can overflow: the flag of the previous steps, which came back
  // with the last step's loss, vouches for the parameters and moments, the gradient norm for the
  // gradients. When they are not known to be bounded the flag starts afresh with this step.
  const bool flag_clear = t->tracked && t->flag_seen == 0;
  if (!flag_clear) TRY(omx_fill_zero(t->ctx, t->unbounded, 4));
  const int32_t bounded = flag_clear && std::isfinite(norm) && norm < 0x1p60f;
  t->tracked = false;  // until the readback below has seen this step through
  TRY(omx_adamw_step_bounded(t->ctx, t->p32, t->acc, t->m1, t->m2, t->adam_end, t->steps, adamw, mirror, bounded,
                             t->unbounded));
  const uint64_t count = t->slots.size();
  // Muon: matrices of one shape go through Newton-Schulz together.
  struct Group {
    std::vector<void*> p, m, p16;
    std::vector<const void*> g;
  };
  std::map<std::pair<uint64_t, uint64_t>, Group> groups;
  for (uint64_t i = 0; i < count; ++i) {
    if (!t->is_muon(i)) continue;
    const Slot& s = t->slots[i];
    Group& grp = groups[{s.rows, s.cols}];
    grp.p.push_back(t->p32 + s.offset);
    grp.g.push_back(t->acc + s.offset);
    grp.m.push_back(t->m1 + s.offset);
    grp.p16.push_back(mirror ? mirror + s.offset : nullptr);
  }
  for (auto& kv : groups) {
    Group& grp = kv.second;
    TRY(omx_muon_ns5_step_batched(t->ctx, grp.p.data(), grp.g.data(), grp.m.data(), mirror ? grp.p16.data() : nullptr,
                                  grp.p.size(), kv.first.first, kv.first.second, muon));
  }
  // Sync point 2: the step's one readback (trainer.rs:1031-1046).
  struct {
    float loss;
    uint32_t flag;
  } back = {0.0f, 1u};
  TRY(omx_download(t->ctx, &back, t->loss_acc, 0, sizeof(back)));
  t->flag_seen = back.flag;
  t->tracked = true;
  const float l = back.loss;
  t->steps += 1;
  if (loss) *loss = l;
  if (grad_norm) *grad_norm = norm;
  return OMX_OK;
}

}  // extern "C"
