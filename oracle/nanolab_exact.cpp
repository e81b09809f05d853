// CPU oracle: loss and gradients of the nanolab GPT (the reference's own model
// graph) composed from the Exact ops.
//
// TEST INFRASTRUCTURE ONLY (parity checker).
//
// Graph: ojas-model/src/block.rs:218-264 (block_with), :343-420 (hidden,
// forward_logits, tied head); RoPE tables :31-71; parameter order
// ojas-model/src/names.rs:188-300 (tok_emb, then per block norm1, q_proj,
// k_proj, v_proj, o_proj, q_norm, k_norm, gate.weight, gate.bias, vr_lambda,
// norm2, ffn.gate, ffn.up, ffn.down, then norm_f).
//   x = embedding(tok, ids)
//   per block: h = rms(x); q,k,v = linear(h); q,k = rms over head_dim; rope;
//              v = blend(v, v0) for blocks >= 1 (v0 = block 0's raw v);
//              y = sdpa(permute q,k,v); y = gate(h, y); x = x + o_proj(y);
//              h2 = rms(x); x = x + down(silu(gate(h2)) * up(h2))
//   loss = linear_cross_entropy_mean(rms(x), tok, targets)
// The backward chains the ops' own backward functions in reverse; a value
// with several consumers adds their gradients later consumer first
// (ojas-autograd/src/tape.rs:2565-2591).
//
// Pinned by ojas-oracle/fixtures/tiny/{init,forward,grads_init}.safetensors
// (torch 2.13 logits, loss and every gradient at the seeded init).
//
// orc_nanolab_loss_and_grads_rounded runs the same graph with bf16 roundings
// (orc_round_bf16_vec, the integer rule of ojas-core/src/autocast.rs:66-101)
// placed where a bf16 tier places them; every operation itself stays Exact
// f32 arithmetic on the rounded values, as `Autocast<CpuBackend>` computes:
//   ORC_ROUND_OPERANDS  only what a matrix product reads: the operands `prep`
//                       rounds (autocast.rs:518-525) for linear_*, the gate,
//                       causal_sdpa_* and the fused head. Fewer roundings than
//                       any tier whose products take bf16 operands can have:
//                       its distance from the Exact result is that noise floor.
//   ORC_ROUND_AUTOCAST  the reference's own bf16 tier: the operands, the
//                       activation outputs `emit` rounds (:533-538: linear,
//                       attention and gate outputs, their input gradients) and
//                       the pointwise results `promote` rounds when their
//                       inputs are tagged (:540-546: SiLU, the product, RoPE's
//                       backward). Norms, residual adds (the stream is never
//                       tagged), the blend (lambda is a parameter) and the
//                       loss stay f32; weight gradients stay f32 (`keep_f32`).
// The saved attention output that the backward's row term reads is never
// rounded (:177-186, :1200-1236). With rounding 0 the function is
// orc_nanolab_loss_and_grads bit for bit.
#include <cmath>
#include <vector>

#include "ojas_exact.h"

namespace {

struct Dims {
  size_t L, d, H, KV, D, hidden, V, B, T, N, qw, kvw;
};
Dims dims_of(const orc_nanolab_config* c) {
  Dims s;
  s.L = c->layers;
  s.d = c->n_embd;
  s.H = c->n_head;
  s.KV = c->n_kv_head;
  s.D = c->head_dim;
  s.hidden = c->hidden;
  s.V = c->vocab;
  s.B = c->batch;
  s.T = c->seq;
  s.N = s.B * s.T;
  s.qw = s.H * s.D;
  s.kvw = s.KV * s.D;
  return s;
}
enum { P_NORM1, P_Q, P_K, P_V, P_O, P_QN, P_KN, P_GW, P_GB, P_LAMBDA, P_NORM2, P_FGATE, P_FUP, P_FDOWN, P_PER_BLOCK };
size_t pidx(size_t layer, int which) { return 1 + layer * P_PER_BLOCK + which; }
size_t plen(const Dims& s, size_t i) {
  if (i == 0) return s.V * s.d;
  if (i == 1 + s.L * P_PER_BLOCK) return s.d;
  switch ((i - 1) % P_PER_BLOCK) {
    case P_NORM1:
    case P_NORM2: return s.d;
    case P_Q: return s.qw * s.d;
    case P_K:
    case P_V: return s.kvw * s.d;
    case P_O: return s.d * s.qw;
    case P_QN:
    case P_KN: return s.D;
    case P_GW: return s.H * s.d;
    case P_GB: return s.H;
    case P_LAMBDA: return 1;
    case P_FGATE:
    case P_FUP: return s.hidden * s.d;
    default: return s.d * s.hidden;
  }
}

struct BlockActs {
  std::vector<float> x, h, q_lin, k_lin, raw_v, qn, kn, q, k, v, qp, kp, vp, a, lse, ap, y, x1, h2, g_lin, g_act, up, m;
};

void add_into(std::vector<float>& acc, const std::vector<float>& g) {
  for (size_t i = 0; i < acc.size(); ++i) acc[i] = acc[i] + g[i];
}

// Where a rounding sits: at a product's operand, or at an output the reference's Autocast emits.
enum RoundAt { AT_OPERAND, AT_OUTPUT };
struct Rounding {
  int mode;
  void operator()(std::vector<float>& v, RoundAt at) const {
    if (mode == ORC_ROUND_AUTOCAST || (mode == ORC_ROUND_OPERANDS && at == AT_OPERAND))
      orc_round_bf16_vec(v.data(), v.data(), v.size());
  }
  // A rounded copy for a product to read while the f32 value lives on (the residual stream's gradient).
  std::vector<float> copy(const std::vector<float>& v, RoundAt at) const {
    std::vector<float> out = v;
    (*this)(out, at);
    return out;
  }
};

#define ORC_TRY(expr)              \
  do {                             \
    int rc_ = (expr);              \
    if (rc_ != ORC_OK) return rc_; \
  } while (0)

}  // namespace

extern "C" {

size_t orc_nanolab_param_count(const orc_nanolab_config* c) { return 2 + static_cast<size_t>(c->layers) * P_PER_BLOCK; }
size_t orc_nanolab_param_len(const orc_nanolab_config* c, size_t index) { return plen(dims_of(c), index); }

// ojas-model/src/block.rs:31-71: angles in f64, one rounding to f32; both
// halves of a row hold the same values.
void orc_rope_tables(size_t seq, size_t head_dim, double base, float* cos, float* sin) {
  const size_t half = head_dim / 2;
  for (size_t row = 0; row < seq; ++row)
    for (size_t i = 0; i < half; ++i) {
      double inv = std::pow(base, -static_cast<double>(2 * i) / static_cast<double>(head_dim));
      double angle = static_cast<double>(row) * inv;
      float c = static_cast<float>(std::cos(angle)), s = static_cast<float>(std::sin(angle));
      cos[row * head_dim + i] = c;
      cos[row * head_dim + half + i] = c;
      sin[row * head_dim + i] = s;
      sin[row * head_dim + half + i] = s;
    }
}

static int nanolab_impl(int rounding, const orc_nanolab_config* c, float* const* params, const uint32_t* ids,
                        const uint32_t* targets, float* loss, float* logits, float* const* grads) {
  if (rounding != 0 && rounding != ORC_ROUND_OPERANDS && rounding != ORC_ROUND_AUTOCAST) return ORC_OUT_OF_RANGE;
  const Rounding R{rounding};
  const Dims s = dims_of(c);
  if (s.KV == 0 || s.H % s.KV != 0 || s.D % 2 != 0) return ORC_SHAPE;
  const size_t N = s.N, d = s.d, B = s.B, T = s.T, H = s.H, KV = s.KV, D = s.D, M = s.hidden;
  const float eps = c->rms_eps;
  const size_t final_norm = 1 + s.L * P_PER_BLOCK;
  std::vector<float> cos(T * D), sin(T * D);
  orc_rope_tables(T, D, c->rope_base, cos.data(), sin.data());

  // ---- forward ----
  std::vector<float> x(N * d), tmp(N * d);
  ORC_TRY(orc_embedding_forward(params[0], ids, x.data(), N, s.V, d));
  std::vector<BlockActs> acts(s.L);
  for (size_t l = 0; l < s.L; ++l) {
    BlockActs& A = acts[l];
    auto P = [&](int which) { return params[pidx(l, which)]; };
    A.x = x;
    A.h.resize(N * d);
    ORC_TRY(orc_rms_norm_forward(A.x.data(), P(P_NORM1), A.h.data(), N, d, eps));
    R(A.h, AT_OPERAND);  // read by the three projections and the gate
    A.q_lin.resize(N * s.qw);
    A.k_lin.resize(N * s.kvw);
    A.raw_v.resize(N * s.kvw);
    ORC_TRY(orc_linear_forward(A.h.data(), P(P_Q), A.q_lin.data(), N, d, s.qw));
    ORC_TRY(orc_linear_forward(A.h.data(), P(P_K), A.k_lin.data(), N, d, s.kvw));
    ORC_TRY(orc_linear_forward(A.h.data(), P(P_V), A.raw_v.data(), N, d, s.kvw));
    R(A.q_lin, AT_OUTPUT);
    R(A.k_lin, AT_OUTPUT);
    R(A.raw_v, AT_OUTPUT);
    A.qn.resize(N * s.qw);
    A.kn.resize(N * s.kvw);
    ORC_TRY(orc_rms_norm_forward(A.q_lin.data(), P(P_QN), A.qn.data(), N * H, D, eps));
    ORC_TRY(orc_rms_norm_forward(A.k_lin.data(), P(P_KN), A.kn.data(), N * KV, D, eps));
    A.q.resize(N * s.qw);
    A.k.resize(N * s.kvw);
    ORC_TRY(orc_rope_forward(A.qn.data(), cos.data(), sin.data(), A.q.data(), N * H, D, T, H));
    ORC_TRY(orc_rope_forward(A.kn.data(), cos.data(), sin.data(), A.k.data(), N * KV, D, T, KV));
    A.v.resize(N * s.kvw);
    if (l == 0) A.v = A.raw_v;
    else ORC_TRY(orc_value_residual_forward(A.raw_v.data(), acts[0].raw_v.data(), P(P_LAMBDA)[0], A.v.data(), N * s.kvw));
    R(A.q, AT_OPERAND);
    R(A.k, AT_OPERAND);
    R(A.v, AT_OPERAND);
    A.qp.resize(N * s.qw);
    A.kp.resize(N * s.kvw);
    A.vp.resize(N * s.kvw);
    orc_permute_0213(A.q.data(), A.qp.data(), B, T, H, D);
    orc_permute_0213(A.k.data(), A.kp.data(), B, T, KV, D);
    orc_permute_0213(A.v.data(), A.vp.data(), B, T, KV, D);
    A.a.resize(N * s.qw);
    A.lse.resize(B * H * T);
    ORC_TRY(orc_causal_sdpa_forward(A.qp.data(), A.kp.data(), A.vp.data(), A.a.data(), A.lse.data(), B, H, KV, T, D,
                                    c->window));
    A.ap.resize(N * s.qw);
    orc_permute_0213(A.a.data(), A.ap.data(), B, H, T, D);
    R(A.ap, AT_OUTPUT);  // what the gate reads; A.a, which the backward's row term reads, stays as it is
    A.y.resize(N * s.qw);
    ORC_TRY(orc_gate_forward(A.h.data(), P(P_GW), P(P_GB), A.ap.data(), A.y.data(), N, d, H, D));
    R(A.y, AT_OPERAND);
    ORC_TRY(orc_linear_forward(A.y.data(), P(P_O), tmp.data(), N, s.qw, d));
    R(tmp, AT_OUTPUT);
    A.x1.resize(N * d);
    ORC_TRY(orc_residual_add(A.x.data(), tmp.data(), A.x1.data(), N * d));
    A.h2.resize(N * d);
    ORC_TRY(orc_rms_norm_forward(A.x1.data(), P(P_NORM2), A.h2.data(), N, d, eps));
    R(A.h2, AT_OPERAND);
    A.g_lin.resize(N * M);
    A.g_act.resize(N * M);
    A.up.resize(N * M);
    A.m.resize(N * M);
    ORC_TRY(orc_linear_forward(A.h2.data(), P(P_FGATE), A.g_lin.data(), N, d, M));
    R(A.g_lin, AT_OUTPUT);
    orc_silu_forward_vec(A.g_lin.data(), A.g_act.data(), N * M);
    R(A.g_act, AT_OUTPUT);
    ORC_TRY(orc_linear_forward(A.h2.data(), P(P_FUP), A.up.data(), N, d, M));
    R(A.up, AT_OUTPUT);
    ORC_TRY(orc_mul_forward(A.g_act.data(), A.up.data(), A.m.data(), N * M));
    R(A.m, AT_OPERAND);
    ORC_TRY(orc_linear_forward(A.m.data(), P(P_FDOWN), tmp.data(), N, M, d));
    R(tmp, AT_OUTPUT);
    ORC_TRY(orc_residual_add(A.x1.data(), tmp.data(), x.data(), N * d));
  }
  std::vector<float> hf(N * d);
  ORC_TRY(orc_rms_norm_forward(x.data(), params[final_norm], hf.data(), N, d, eps));
  R(hf, AT_OPERAND);
  if (logits) ORC_TRY(orc_linear_forward(hf.data(), params[0], logits, N, d, s.V));
  if (!grads)
    return orc_linear_cross_entropy_mean(hf.data(), params[0], targets, N, d, s.V, 0, 0, loss, nullptr, nullptr);

  // ---- backward ----
  std::vector<float> ghf(N * d), g_head(s.V * d);
  ORC_TRY(orc_linear_cross_entropy_mean(hf.data(), params[0], targets, N, d, s.V, 0, 0, loss, ghf.data(),
                                        g_head.data()));
  R(ghf, AT_OUTPUT);
  std::vector<float> gx(N * d);
  ORC_TRY(orc_rms_norm_backward(x.data(), params[final_norm], ghf.data(), gx.data(), grads[final_norm], N, d, eps));
  std::vector<float> g_v0(N * s.kvw, 0.0f);  // gradient of block 0's raw v from the later blocks' blends
  bool g_v0_live = false;
  std::vector<float> gm(N * M), g_gact(N * M), g_up(N * M), g_glin(N * M), gh2(N * d), gh2b(N * d), gt(N * d);
  std::vector<float> gy(N * s.qw), gap(N * s.qw), ga(N * s.qw), gqp(N * s.qw), gkp(N * s.kvw), gvp(N * s.kvw);
  std::vector<float> gq(N * s.qw), gk(N * s.kvw), gv(N * s.kvw), gqn(N * s.qw), gkn(N * s.kvw), gq_lin(N * s.qw),
      gk_lin(N * s.kvw), g_raw_v(N * s.kvw), g_v0_part(N * s.kvw), gh(N * d), gh_part(N * d);
  for (size_t l = s.L; l-- > 0;) {
    BlockActs& A = acts[l];
    auto P = [&](int which) { return params[pidx(l, which)]; };
    auto G = [&](int which) { return grads[pidx(l, which)]; };
    // x2 = x1 + down(m)
    {
      const std::vector<float> gx_op = R.copy(gx, AT_OPERAND);
      ORC_TRY(orc_linear_backward(A.m.data(), P(P_FDOWN), gx_op.data(), gm.data(), G(P_FDOWN), N, M, d));
    }
    R(gm, AT_OUTPUT);
    ORC_TRY(orc_mul_backward(A.g_act.data(), A.up.data(), gm.data(), g_gact.data(), g_up.data(), N * M));
    R(g_gact, AT_OUTPUT);
    R(g_up, AT_OPERAND);
    // h2 feeds ffn.gate then ffn.up: the later consumer (up) first.
    ORC_TRY(orc_linear_backward(A.h2.data(), P(P_FUP), g_up.data(), gh2.data(), G(P_FUP), N, d, M));
    R(gh2, AT_OUTPUT);
    orc_silu_backward_vec(A.g_lin.data(), g_gact.data(), g_glin.data(), N * M);
    R(g_glin, AT_OPERAND);
    ORC_TRY(orc_linear_backward(A.h2.data(), P(P_FGATE), g_glin.data(), gh2b.data(), G(P_FGATE), N, d, M));
    R(gh2b, AT_OUTPUT);
    add_into(gh2, gh2b);
    ORC_TRY(orc_rms_norm_backward(A.x1.data(), P(P_NORM2), gh2.data(), gt.data(), G(P_NORM2), N, d, eps));
    std::vector<float> gx1 = gx;  // the residual branch first, then the norm branch
    add_into(gx1, gt);
    // x1 = x + o_proj(y)
    {
      const std::vector<float> gx1_op = R.copy(gx1, AT_OPERAND);
      ORC_TRY(orc_linear_backward(A.y.data(), P(P_O), gx1_op.data(), gy.data(), G(P_O), N, s.qw, d));
    }
    R(gy, AT_OPERAND);  // emitted by the product, read by the gate's backward
    // h feeds q, k, v and (last) the gate: the gate's gradient comes first.
    ORC_TRY(orc_gate_backward(A.h.data(), P(P_GW), P(P_GB), A.ap.data(), gy.data(), gh.data(), G(P_GW), G(P_GB),
                              gap.data(), N, d, H, D));
    R(gh, AT_OUTPUT);
    R(gap, AT_OPERAND);
    orc_permute_0213(gap.data(), ga.data(), B, T, H, D);
    ORC_TRY(orc_causal_sdpa_backward(A.qp.data(), A.kp.data(), A.vp.data(), A.a.data(), A.lse.data(), ga.data(),
                                     gqp.data(), gkp.data(), gvp.data(), B, H, KV, T, D, c->window));
    orc_permute_0213(gvp.data(), gv.data(), B, KV, T, D);
    orc_permute_0213(gkp.data(), gk.data(), B, KV, T, D);
    orc_permute_0213(gqp.data(), gq.data(), B, H, T, D);
    R(gq, AT_OUTPUT);
    R(gk, AT_OUTPUT);
    R(gv, AT_OUTPUT);
    if (l == 0) {
      // Block 0's raw v: the later blocks' blends were visited first, its own attention last.
      if (g_v0_live) {
        g_raw_v = g_v0;
        add_into(g_raw_v, gv);
      } else {
        g_raw_v = gv;
      }
      grads[pidx(0, P_LAMBDA)][0] = 0.0f;
    } else {
      float gl = 0.0f;
      ORC_TRY(orc_value_residual_backward(A.raw_v.data(), acts[0].raw_v.data(), gv.data(), P(P_LAMBDA)[0],
                                          g_raw_v.data(), g_v0_part.data(), &gl, N * s.kvw));
      G(P_LAMBDA)[0] = gl;
      if (g_v0_live) add_into(g_v0, g_v0_part);
      else g_v0 = g_v0_part;
      g_v0_live = true;
    }
    ORC_TRY(orc_rope_backward(gk.data(), cos.data(), sin.data(), gkn.data(), N * KV, D, T, KV));
    ORC_TRY(orc_rope_backward(gq.data(), cos.data(), sin.data(), gqn.data(), N * H, D, T, H));
    R(gkn, AT_OUTPUT);
    R(gqn, AT_OUTPUT);
    ORC_TRY(orc_rms_norm_backward(A.k_lin.data(), P(P_KN), gkn.data(), gk_lin.data(), G(P_KN), N * KV, D, eps));
    ORC_TRY(orc_rms_norm_backward(A.q_lin.data(), P(P_QN), gqn.data(), gq_lin.data(), G(P_QN), N * H, D, eps));
    R(gq_lin, AT_OPERAND);
    R(gk_lin, AT_OPERAND);
    R(g_raw_v, AT_OPERAND);
    ORC_TRY(orc_linear_backward(A.h.data(), P(P_V), g_raw_v.data(), gh_part.data(), G(P_V), N, d, s.kvw));
    R(gh_part, AT_OUTPUT);
    add_into(gh, gh_part);
    ORC_TRY(orc_linear_backward(A.h.data(), P(P_K), gk_lin.data(), gh_part.data(), G(P_K), N, d, s.kvw));
    R(gh_part, AT_OUTPUT);
    add_into(gh, gh_part);
    ORC_TRY(orc_linear_backward(A.h.data(), P(P_Q), gq_lin.data(), gh_part.data(), G(P_Q), N, d, s.qw));
    R(gh_part, AT_OUTPUT);
    add_into(gh, gh_part);
    ORC_TRY(orc_rms_norm_backward(A.x.data(), P(P_NORM1), gh.data(), gt.data(), G(P_NORM1), N, d, eps));
    gx = gx1;
    add_into(gx, gt);
  }
  // The tied table: the head's gradient first, then the embedding's rows.
  ORC_TRY(orc_embedding_backward(ids, gx.data(), grads[0], N, s.V, d));
  for (size_t i = 0; i < s.V * d; ++i) grads[0][i] = g_head[i] + grads[0][i];
  return ORC_OK;
}

int orc_nanolab_loss_and_grads(const orc_nanolab_config* c, float* const* params, const uint32_t* ids,
                               const uint32_t* targets, float* loss, float* logits, float* const* grads) {
  return nanolab_impl(0, c, params, ids, targets, loss, logits, grads);
}

int orc_nanolab_loss_and_grads_rounded(int rounding, const orc_nanolab_config* c, float* const* params,
                                       const uint32_t* ids, const uint32_t* targets, float* loss, float* const* grads) {
  return nanolab_impl(rounding, c, params, ids, targets, loss, nullptr, grads);
}

}  // extern "C"
