// CPU oracle: group-wise symmetric int8 weights and one LoRA fine-tune step over a frozen decoder.
//
// TEST INFRASTRUCTURE ONLY (parity checker and timed CPU baseline).
//
// Weight format. The reference ships a symmetric int8 format per OUTPUT CHANNEL
// (ojas-cpu/src/quant_sparse.rs:284-346: scale = abs_max / 127, or 1 for a row of zeros;
// code = round(v * 127 / abs_max) clamped to [-127, 127]; value = code * scale) and an affine
// group format with bf16 parameters (ojas-core/src/quant.rs:13-22). The format of this path,
// symmetric int8 in groups of 32 consecutive input columns with one f32 scale per group, is the
// first rule applied to a group of a row instead of the whole row; with group == k_in it IS the
// reference's per-channel form, which tests/test_oracle_lora.py checks.
// PARITY UNPINNED by the reference for group < k_in: no fixture holds this format. It is pinned by
// its closed form (dequantise, then the digest-pinned Exact GEMM), by brute force on tiny inputs
// and by a known-answer table of codes and scales.
//
// Graph (the adapter of ojas-model/src/lora.rs:292-344 on the q, k, v and o projections of a
// Llama-shaped block; every op is one of the Exact ops of ojas_exact.cpp):
//   x = embedding(tok, ids)
//   per layer: h = rms_norm(x, n1)
//              q,k,v = lora_linear(h, W, A, scale * B)   (base = linear(x, W); delta =
//                      linear(linear(x, A), B_eff); add(base, delta), lora.rs:332-344)
//              q,k = rope_half_split(q), rope_half_split(k); a = causal_sdpa(q, k, v)
//              x1 = x + lora_linear(a, Wo, Ao, scale * Bo)
//              h2 = rms_norm(x1, n2); m = silu(linear(h2, Wg)) * linear(h2, Wu)
//              x = x1 + linear(m, Wd)
//   loss = linear_cross_entropy_mean(rms_norm(x, nf), tok, targets)      (tied head)
// Only A and B receive gradients (the base is Graph::frozen, lora.rs:4-8).
#include <cmath>
#include <cstring>
#include <vector>

#include "ojas_exact.h"

namespace {

#define ORC_TRY(expr)              \
  do {                             \
    int rc_ = (expr);              \
    if (rc_ != ORC_OK) return rc_; \
  } while (0)

void add_into(std::vector<float>& acc, const std::vector<float>& g) {
  for (size_t i = 0; i < acc.size(); ++i) acc[i] = acc[i] + g[i];
}

struct Site {
  std::vector<float> h;      // x A^T  [N, r]
  std::vector<float> b_eff;  // scale * B  [out, r]
};

// lora.rs:332-344.
int lora_forward(const float* x, const float* w, const float* a, const float* b, float scale, size_t N, size_t in,
                 size_t out, size_t r, Site& s, std::vector<float>& y) {
  std::vector<float> delta(N * out);
  y.resize(N * out);
  ORC_TRY(orc_linear_forward(x, w, y.data(), N, in, out));
  s.h.resize(N * r);
  ORC_TRY(orc_linear_forward(x, a, s.h.data(), N, in, r));
  s.b_eff.resize(out * r);
  for (size_t i = 0; i < out * r; ++i) s.b_eff[i] = scale == 1.0f ? b[i] : b[i] * scale;  // lora.rs:309-323
  ORC_TRY(orc_linear_forward(s.h.data(), s.b_eff.data(), delta.data(), N, r, out));
  return orc_residual_add(y.data(), delta.data(), y.data(), N * out);
}

// gx = gy W + (gy B_eff) A; gB = scale * gy^T h; gA = (gy B_eff)^T x. x's two consumers are
// visited later-first (the adapter's down projection, then the base), as the tape does.
int lora_backward(const float* x, const float* w, const float* a, float scale, const Site& s, const float* gy, size_t N,
                  size_t in, size_t out, size_t r, float* ga, float* gb, std::vector<float>& gx) {
  std::vector<float> gh(N * r), gb_eff(out * r), gx_base(N * in);
  ORC_TRY(orc_linear_backward(s.h.data(), s.b_eff.data(), gy, gh.data(), gb_eff.data(), N, r, out));
  for (size_t i = 0; i < out * r; ++i) gb[i] = scale == 1.0f ? gb_eff[i] : gb_eff[i] * scale;
  gx.resize(N * in);
  ORC_TRY(orc_linear_backward(x, a, gh.data(), gx.data(), ga, N, in, r));
  ORC_TRY(orc_linear_backward(x, w, gy, gx_base.data(), nullptr, N, in, out));
  add_into(gx, gx_base);
  return ORC_OK;
}

struct Acts {
  std::vector<float> x, h, q_lin, k_lin, v_lin, q, k, qp, kp, vp, a, lse, ap, x1, h2, g_lin, g_act, up, m;
  Site sq, sk, sv, so;
};

}  // namespace

extern "C" {

// quant_sparse.rs:306-326 applied to groups of `group` consecutive columns of a row.
int orc_quantize_i8_group(const float* w, int8_t* codes, float* scales, size_t rows, size_t cols, size_t group) {
  if (group == 0 || cols % group != 0) return ORC_SHAPE;
  const size_t gpr = cols / group;
  for (size_t i = 0; i < rows * cols; ++i)
    if (!std::isfinite(w[i])) return ORC_NON_FINITE;
  for (size_t r = 0; r < rows; ++r)
    for (size_t g = 0; g < gpr; ++g) {
      const float* v = w + r * cols + g * group;
      float abs_max = 0.0f;
      for (size_t i = 0; i < group; ++i) abs_max = std::fmax(abs_max, std::fabs(v[i]));
      scales[r * gpr + g] = abs_max > 0.0f ? abs_max / 127.0f : 1.0f;
      const float inv = abs_max > 0.0f ? 127.0f / abs_max : 0.0f;
      for (size_t i = 0; i < group; ++i) {
        float q = std::round(v[i] * inv);  // half away from zero, as f32::round
        q = q < -127.0f ? -127.0f : (q > 127.0f ? 127.0f : q);
        codes[r * cols + g * group + i] = static_cast<int8_t>(q);
      }
    }
  return ORC_OK;
}

// quant_sparse.rs:335-344: value = (code as f32) * scale.
int orc_dequant_i8_group(const int8_t* codes, const float* scales, float* w, size_t rows, size_t cols, size_t group) {
  if (group == 0 || cols % group != 0) return ORC_SHAPE;
  const size_t gpr = cols / group;
  for (size_t r = 0; r < rows; ++r)
    for (size_t c = 0; c < cols; ++c)
      w[r * cols + c] = static_cast<float>(codes[r * cols + c]) * scales[r * gpr + c / group];
  return ORC_OK;
}

// y = x W^T with W given as codes and scales: dequantise, then the Exact linear.
int orc_linear_i8_group_forward(const float* x, const int8_t* codes, const float* scales, float* y, size_t rows,
                                size_t kin, size_t nout, size_t group) {
  std::vector<float> w(nout * kin);
  ORC_TRY(orc_dequant_i8_group(codes, scales, w.data(), nout, kin, group));
  return orc_linear_forward(x, w.data(), y, rows, kin, nout);
}
// gx = gy W.
int orc_linear_i8_group_backward_input(const int8_t* codes, const float* scales, const float* gy, float* gx,
                                       size_t rows, size_t kin, size_t nout, size_t group) {
  std::vector<float> w(nout * kin);
  ORC_TRY(orc_dequant_i8_group(codes, scales, w.data(), nout, kin, group));
  return orc_linear_backward(nullptr, w.data(), gy, gx, nullptr, rows, kin, nout);
}

// frozen: tok [V,d]; per layer n1 [d], wq, wk, wv, wo [d,d], n2 [d], wgate, wup [hidden,d], wdown [d,hidden];
// final norm [d]  (2 + 9 * layers tensors, already dequantised).
// adapters / grads: per layer Aq [r,d], Bq [d,r], Ak, Bk, Av, Bv, Ao, Bo  (8 * layers tensors).
size_t orc_lora_frozen_count(const orc_lora_config* c) { return 2 + 9 * static_cast<size_t>(c->layers); }
size_t orc_lora_adapter_count(const orc_lora_config* c) { return 8 * static_cast<size_t>(c->layers); }

int orc_lora_loss_and_grads(const orc_lora_config* c, const float* const* frozen, const float* const* adapters,
                            const uint32_t* ids, const uint32_t* targets, float* loss, float* const* grads) {
  const size_t L = c->layers, d = c->d_model, H = c->heads, D = c->head_dim, M = c->hidden, V = c->vocab, B = c->batch,
               T = c->seq, r = c->rank, N = B * T;
  if (H * D != d || D % 2 != 0 || r == 0) return ORC_SHAPE;
  const float eps = c->rms_eps, scale = c->lora_scale;
  std::vector<float> cos(T * D), sin(T * D);
  orc_rope_tables(T, D, c->rope_base, cos.data(), sin.data());
  auto F = [&](size_t l, size_t which) { return frozen[1 + l * 9 + which]; };
  auto A_ = [&](size_t l, size_t which) { return adapters[l * 8 + which]; };
  const float* nf = frozen[1 + L * 9];

  std::vector<float> x(N * d), tmp;
  ORC_TRY(orc_embedding_forward(frozen[0], ids, x.data(), N, V, d));
  std::vector<Acts> acts(L);
  for (size_t l = 0; l < L; ++l) {
    Acts& a = acts[l];
    a.x = x;
    a.h.resize(N * d);
    ORC_TRY(orc_rms_norm_forward(a.x.data(), F(l, 0), a.h.data(), N, d, eps));
    ORC_TRY(lora_forward(a.h.data(), F(l, 1), A_(l, 0), A_(l, 1), scale, N, d, d, r, a.sq, a.q_lin));
    ORC_TRY(lora_forward(a.h.data(), F(l, 2), A_(l, 2), A_(l, 3), scale, N, d, d, r, a.sk, a.k_lin));
    ORC_TRY(lora_forward(a.h.data(), F(l, 3), A_(l, 4), A_(l, 5), scale, N, d, d, r, a.sv, a.v_lin));
    a.q.resize(N * d);
    a.k.resize(N * d);
    ORC_TRY(orc_rope_forward(a.q_lin.data(), cos.data(), sin.data(), a.q.data(), N * H, D, T, H));
    ORC_TRY(orc_rope_forward(a.k_lin.data(), cos.data(), sin.data(), a.k.data(), N * H, D, T, H));
    a.qp.resize(N * d);
    a.kp.resize(N * d);
    a.vp.resize(N * d);
    orc_permute_0213(a.q.data(), a.qp.data(), B, T, H, D);
    orc_permute_0213(a.k.data(), a.kp.data(), B, T, H, D);
    orc_permute_0213(a.v_lin.data(), a.vp.data(), B, T, H, D);
    a.a.resize(N * d);
    a.lse.resize(B * H * T);
    ORC_TRY(orc_causal_sdpa_forward(a.qp.data(), a.kp.data(), a.vp.data(), a.a.data(), a.lse.data(), B, H, H, T, D, 0));
    a.ap.resize(N * d);
    orc_permute_0213(a.a.data(), a.ap.data(), B, H, T, D);
    ORC_TRY(lora_forward(a.ap.data(), F(l, 4), A_(l, 6), A_(l, 7), scale, N, d, d, r, a.so, tmp));
    a.x1.resize(N * d);
    ORC_TRY(orc_residual_add(a.x.data(), tmp.data(), a.x1.data(), N * d));
    a.h2.resize(N * d);
    ORC_TRY(orc_rms_norm_forward(a.x1.data(), F(l, 5), a.h2.data(), N, d, eps));
    a.g_lin.resize(N * M);
    a.g_act.resize(N * M);
    a.up.resize(N * M);
    a.m.resize(N * M);
    ORC_TRY(orc_linear_forward(a.h2.data(), F(l, 6), a.g_lin.data(), N, d, M));
    orc_silu_forward_vec(a.g_lin.data(), a.g_act.data(), N * M);
    ORC_TRY(orc_linear_forward(a.h2.data(), F(l, 7), a.up.data(), N, d, M));
    ORC_TRY(orc_mul_forward(a.g_act.data(), a.up.data(), a.m.data(), N * M));
    tmp.resize(N * d);
    ORC_TRY(orc_linear_forward(a.m.data(), F(l, 8), tmp.data(), N, M, d));
    ORC_TRY(orc_residual_add(a.x1.data(), tmp.data(), x.data(), N * d));
  }
  std::vector<float> hf(N * d);
  ORC_TRY(orc_rms_norm_forward(x.data(), nf, hf.data(), N, d, eps));
  if (!grads) return orc_linear_cross_entropy_mean(hf.data(), frozen[0], targets, N, d, V, 0, 0, loss, nullptr, nullptr);

  std::vector<float> ghf(N * d), gx(N * d), gt(N * d), scratch_w(d);
  ORC_TRY(orc_linear_cross_entropy_mean(hf.data(), frozen[0], targets, N, d, V, 0, 0, loss, ghf.data(), nullptr));
  ORC_TRY(orc_rms_norm_backward(x.data(), nf, ghf.data(), gx.data(), scratch_w.data(), N, d, eps));
  std::vector<float> gm(N * M), g_gact(N * M), g_up(N * M), g_glin(N * M), gh2(N * d), gh2b(N * d);
  std::vector<float> gap, ga(N * d), gqp(N * d), gkp(N * d), gvp(N * d), gq(N * d), gk(N * d), gv(N * d), gq_lin(N * d),
      gk_lin(N * d), gh, gh_part;
  for (size_t l = L; l-- > 0;) {
    Acts& a = acts[l];
    auto G = [&](size_t which) { return grads[l * 8 + which]; };
    ORC_TRY(orc_linear_backward(nullptr, F(l, 8), gx.data(), gm.data(), nullptr, N, M, d));
    ORC_TRY(orc_mul_backward(a.g_act.data(), a.up.data(), gm.data(), g_gact.data(), g_up.data(), N * M));
    ORC_TRY(orc_linear_backward(nullptr, F(l, 7), g_up.data(), gh2.data(), nullptr, N, d, M));
    orc_silu_backward_vec(a.g_lin.data(), g_gact.data(), g_glin.data(), N * M);
    ORC_TRY(orc_linear_backward(nullptr, F(l, 6), g_glin.data(), gh2b.data(), nullptr, N, d, M));
    add_into(gh2, gh2b);
    ORC_TRY(orc_rms_norm_backward(a.x1.data(), F(l, 5), gh2.data(), gt.data(), scratch_w.data(), N, d, eps));
    std::vector<float> gx1 = gx;
    add_into(gx1, gt);
    ORC_TRY(lora_backward(a.ap.data(), F(l, 4), A_(l, 6), scale, a.so, gx1.data(), N, d, d, r, G(6), G(7), gap));
    orc_permute_0213(gap.data(), ga.data(), B, T, H, D);
    ORC_TRY(orc_causal_sdpa_backward(a.qp.data(), a.kp.data(), a.vp.data(), a.a.data(), a.lse.data(), ga.data(),
                                     gqp.data(), gkp.data(), gvp.data(), B, H, H, T, D, 0));
    orc_permute_0213(gvp.data(), gv.data(), B, H, T, D);
    orc_permute_0213(gkp.data(), gk.data(), B, H, T, D);
    orc_permute_0213(gqp.data(), gq.data(), B, H, T, D);
    ORC_TRY(orc_rope_backward(gk.data(), cos.data(), sin.data(), gk_lin.data(), N * H, D, T, H));
    ORC_TRY(orc_rope_backward(gq.data(), cos.data(), sin.data(), gq_lin.data(), N * H, D, T, H));
    ORC_TRY(lora_backward(a.h.data(), F(l, 3), A_(l, 4), scale, a.sv, gv.data(), N, d, d, r, G(4), G(5), gh));
    ORC_TRY(lora_backward(a.h.data(), F(l, 2), A_(l, 2), scale, a.sk, gk_lin.data(), N, d, d, r, G(2), G(3), gh_part));
    add_into(gh, gh_part);
    ORC_TRY(lora_backward(a.h.data(), F(l, 1), A_(l, 0), scale, a.sq, gq_lin.data(), N, d, d, r, G(0), G(1), gh_part));
    add_into(gh, gh_part);
    ORC_TRY(orc_rms_norm_backward(a.x.data(), F(l, 0), gh.data(), gt.data(), scratch_w.data(), N, d, eps));
    gx = gx1;
    add_into(gx, gt);
  }
  return ORC_OK;
}

}  // extern "C"
