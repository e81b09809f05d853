// CPU oracle: one GPT-2-shaped training step composed from the Exact ops.
//
// TEST INFRASTRUCTURE ONLY (parity checker and timed CPU baseline).
//
// The graph is the one the benchmark configurations describe, expressed in the
// reference's own Backend ops (every op below has a CPU Exact implementation,
// ojas-cpu/src/backend.rs:640-652,805-821,913-953,1071-1098,1833-1868):
//   x = embedding(tok, ids) + embedding(pos, positions)
//   per layer: rms_norm -> linear q,k,v -> permute [0,2,1,3] -> causal_sdpa ->
//              permute back -> linear o -> residual_add -> rms_norm ->
//              linear d->mlp -> gelu -> linear mlp->d -> residual_add
//   rms_norm -> tied head: linear_cross_entropy_mean(h, tok, targets)
// The backward pass chains the ops' own backward functions in reverse, with
// gradient fan-in added in the order the reference's tape visits consumers
// (ojas-autograd/src/tape.rs:2565-2591: later consumers first).
//
// Parity unpinned by the reference: no fixture holds this graph. The tests pin
// it with f64 central differences and with per-op parity.
#include <cstring>
#include <vector>

#include "ojas_exact.h"

namespace {

struct Layout {
  size_t d, mlp, heads, hd, layers, ctx, vocab, batch, n;
  // parameter indices
  size_t tok() const { return 0; }
  size_t pos() const { return 1; }
  size_t layer(size_t l, size_t which) const { return 2 + l * 8 + which; }  // n1,wq,wk,wv,wo,n2,w1,w2
  size_t final_norm() const { return 2 + layers * 8; }
  size_t count() const { return 3 + layers * 8; }
  size_t len(size_t i) const {
    if (i == 0) return vocab * d;
    if (i == 1) return ctx * d;
    if (i == final_norm()) return d;
    switch ((i - 2) % 8) {
      case 0:
      case 5:
        return d;
      case 1:
      case 2:
      case 3:
      case 4:
        return d * d;
      case 6:
        return mlp * d;
      default:
        return d * mlp;
    }
  }
};

Layout layout_of(const orc_gpt_config* c) {
  Layout L;
  L.d = c->d_model;
  L.mlp = c->mlp;
  L.heads = c->heads;
  L.hd = c->head_dim;
  L.layers = c->layers;
  L.ctx = c->ctx;
  L.vocab = c->vocab;
  L.batch = c->batch;
  L.n = static_cast<size_t>(c->batch) * c->ctx;
  return L;
}

struct LayerActs {
  std::vector<float> x, h1, q, k, v, a, lse, ap, x1, h2, u, g;
};

void add_into(std::vector<float>& acc, const std::vector<float>& g) {
  for (size_t i = 0; i < acc.size(); ++i) acc[i] = acc[i] + g[i];
}

#define ORC_TRY(expr)          \
  do {                         \
    int rc_ = (expr);          \
    if (rc_ != ORC_OK) return rc_; \
  } while (0)

}  // namespace

extern "C" {

size_t orc_gpt_param_count(const orc_gpt_config* c) { return layout_of(c).count(); }
size_t orc_gpt_param_len(const orc_gpt_config* c, size_t index) { return layout_of(c).len(index); }

int orc_gpt_loss_and_grads(const orc_gpt_config* c, float* const* params, const uint32_t* ids,
                           const uint32_t* targets, float* loss, float* const* grads) {
  const Layout L = layout_of(c);
  if (L.heads * L.hd != L.d) return ORC_SHAPE;
  const size_t N = L.n, d = L.d, T = L.ctx, B = L.batch, H = L.heads, D = L.hd, M = L.mlp;
  const float eps = 1e-6f;
  std::vector<uint32_t> positions(N);
  for (size_t i = 0; i < N; ++i) positions[i] = static_cast<uint32_t>(i % T);

  // ---- forward ----
  std::vector<float> e_tok(N * d), e_pos(N * d), x(N * d);
  ORC_TRY(orc_embedding_forward(params[L.tok()], ids, e_tok.data(), N, L.vocab, d));
  ORC_TRY(orc_embedding_forward(params[L.pos()], positions.data(), e_pos.data(), N, T, d));
  ORC_TRY(orc_residual_add(e_tok.data(), e_pos.data(), x.data(), N * d));
  std::vector<LayerActs> acts(L.layers);
  std::vector<float> tmp(N * d);
  for (size_t l = 0; l < L.layers; ++l) {
    LayerActs& A = acts[l];
    const float* n1 = params[L.layer(l, 0)];
    const float* wq = params[L.layer(l, 1)];
    const float* wk = params[L.layer(l, 2)];
    const float* wv = params[L.layer(l, 3)];
    const float* wo = params[L.layer(l, 4)];
    const float* n2 = params[L.layer(l, 5)];
    const float* w1 = params[L.layer(l, 6)];
    const float* w2 = params[L.layer(l, 7)];
    A.x = x;
    A.h1.resize(N * d);
    ORC_TRY(orc_rms_norm_forward(A.x.data(), n1, A.h1.data(), N, d, eps));
    A.q.resize(N * d);
    A.k.resize(N * d);
    A.v.resize(N * d);
    ORC_TRY(orc_linear_forward(A.h1.data(), wq, tmp.data(), N, d, d));
    orc_permute_0213(tmp.data(), A.q.data(), B, T, H, D);
    ORC_TRY(orc_linear_forward(A.h1.data(), wk, tmp.data(), N, d, d));
    orc_permute_0213(tmp.data(), A.k.data(), B, T, H, D);
    ORC_TRY(orc_linear_forward(A.h1.data(), wv, tmp.data(), N, d, d));
    orc_permute_0213(tmp.data(), A.v.data(), B, T, H, D);
    A.a.resize(N * d);
    A.lse.resize(B * H * T);
    ORC_TRY(orc_causal_sdpa_forward(A.q.data(), A.k.data(), A.v.data(), A.a.data(), A.lse.data(), B, H, H, T, D, 0));
    A.ap.resize(N * d);
    orc_permute_0213(A.a.data(), A.ap.data(), B, H, T, D);
    ORC_TRY(orc_linear_forward(A.ap.data(), wo, tmp.data(), N, d, d));
    A.x1.resize(N * d);
    ORC_TRY(orc_residual_add(A.x.data(), tmp.data(), A.x1.data(), N * d));
    A.h2.resize(N * d);
    ORC_TRY(orc_rms_norm_forward(A.x1.data(), n2, A.h2.data(), N, d, eps));
    A.u.resize(N * M);
    ORC_TRY(orc_linear_forward(A.h2.data(), w1, A.u.data(), N, d, M));
    A.g.resize(N * M);
    if (c->gelu_tanh) orc_gelu_tanh_forward_vec(A.u.data(), A.g.data(), N * M);
    else orc_gelu_erf_forward_vec(A.u.data(), A.g.data(), N * M);
    ORC_TRY(orc_linear_forward(A.g.data(), w2, tmp.data(), N, M, d));
    ORC_TRY(orc_residual_add(A.x1.data(), tmp.data(), x.data(), N * d));
  }
  std::vector<float> hf(N * d);
  ORC_TRY(orc_rms_norm_forward(x.data(), params[L.final_norm()], hf.data(), N, d, eps));
  if (!grads) return orc_linear_cross_entropy_mean(hf.data(), params[L.tok()], targets, N, d, L.vocab, 0, 0, loss,
                                                   nullptr, nullptr);

  // ---- backward ----
  std::vector<float> ghf(N * d), g_head(L.vocab * d);
  ORC_TRY(orc_linear_cross_entropy_mean(hf.data(), params[L.tok()], targets, N, d, L.vocab, 0, 0, loss, ghf.data(),
                                        g_head.data()));
  std::vector<float> gx(N * d);
  ORC_TRY(orc_rms_norm_backward(x.data(), params[L.final_norm()], ghf.data(), gx.data(), grads[L.final_norm()], N, d,
                                eps));
  std::vector<float> gt(N * d), gt2(N * d), gu(N * M), gg(N * M);
  std::vector<float> gq(N * d), gk(N * d), gv(N * d), ga(N * d), gh(N * d);
  for (size_t li = L.layers; li-- > 0;) {
    LayerActs& A = acts[li];
    const float* n1 = params[L.layer(li, 0)];
    const float* wq = params[L.layer(li, 1)];
    const float* wk = params[L.layer(li, 2)];
    const float* wv = params[L.layer(li, 3)];
    const float* wo = params[L.layer(li, 4)];
    const float* n2 = params[L.layer(li, 5)];
    const float* w1 = params[L.layer(li, 6)];
    const float* w2 = params[L.layer(li, 7)];
    // x2 = x1 + down(g): gx flows to both.
    ORC_TRY(orc_linear_backward(A.g.data(), w2, gx.data(), gg.data(), grads[L.layer(li, 7)], N, M, d));
    if (c->gelu_tanh) orc_gelu_tanh_backward_vec(A.u.data(), gg.data(), gu.data(), N * M);
    else orc_gelu_erf_backward_vec(A.u.data(), gg.data(), gu.data(), N * M);
    ORC_TRY(orc_linear_backward(A.h2.data(), w1, gu.data(), gh.data(), grads[L.layer(li, 6)], N, d, M));
    ORC_TRY(orc_rms_norm_backward(A.x1.data(), n2, gh.data(), gt.data(), grads[L.layer(li, 5)], N, d, eps));
    // grad of x1: the residual branch first, then the norm branch.
    std::vector<float> gx1 = gx;
    add_into(gx1, gt);
    // x1 = x + o(ap)
    ORC_TRY(orc_linear_backward(A.ap.data(), wo, gx1.data(), gt.data(), grads[L.layer(li, 4)], N, d, d));
    orc_permute_0213(gt.data(), ga.data(), B, T, H, D);  // [B,T,H,D] -> [B,H,T,D]
    ORC_TRY(orc_causal_sdpa_backward(A.q.data(), A.k.data(), A.v.data(), A.a.data(), A.lse.data(), ga.data(), gq.data(),
                                     gk.data(), gv.data(), B, H, H, T, D, 0));
    // h1 feeds q, k, v: later consumers first (v, k, q).
    orc_permute_0213(gv.data(), gt.data(), B, H, T, D);
    ORC_TRY(orc_linear_backward(A.h1.data(), wv, gt.data(), gh.data(), grads[L.layer(li, 3)], N, d, d));
    orc_permute_0213(gk.data(), gt.data(), B, H, T, D);
    ORC_TRY(orc_linear_backward(A.h1.data(), wk, gt.data(), gt2.data(), grads[L.layer(li, 2)], N, d, d));
    add_into(gh, gt2);
    orc_permute_0213(gq.data(), gt.data(), B, H, T, D);
    ORC_TRY(orc_linear_backward(A.h1.data(), wq, gt.data(), gt2.data(), grads[L.layer(li, 1)], N, d, d));
    add_into(gh, gt2);
    ORC_TRY(orc_rms_norm_backward(A.x.data(), n1, gh.data(), gt.data(), grads[L.layer(li, 0)], N, d, eps));
    gx = gx1;
    add_into(gx, gt);
  }
  // x = tok[ids] + pos[positions]; the tied table also receives the head's gradient.
  ORC_TRY(orc_embedding_backward(positions.data(), gx.data(), grads[L.pos()], N, T, d));
  ORC_TRY(orc_embedding_backward(ids, gx.data(), grads[L.tok()], N, L.vocab, d));
  for (size_t i = 0; i < L.vocab * d; ++i) grads[L.tok()][i] = g_head[i] + grads[L.tok()][i];
  return ORC_OK;
}

}  // extern "C"
