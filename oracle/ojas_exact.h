/* CPU oracle for the nanolab-GPT training-step ops: a restatement of the
 * reference's `Numerics::Exact` arithmetic (ojas-cpu, ojas-core) in plain C++.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing in the product library links or loads
 * this; only the parity tests, the smoke check and the CPU-baseline leg of
 * the benchmark call it, and only as the checker / the timed CPU baseline.
 *
 * Every function cites the reference file:line whose arithmetic it restates.
 * Return value: 0 on success, otherwise one of the ORC_* codes below (same
 * numbering as the device library's error codes).
 *
 * Pinning status (which reference vectors hold each function) is listed in
 * the table at the top of ojas_exact.cpp.
 */
#ifndef OJAS_EXACT_H
#define OJAS_EXACT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  ORC_OK = 0,
  ORC_SHAPE = 1,
  ORC_DTYPE = 2,
  ORC_OUT_OF_RANGE = 3,
  ORC_NON_FINITE = 4,
};

/* Worker threads for the row/tile-parallel loops (outputs are split, never a
 * reduction: ojas-cpu/src/lib.rs:9-16). Bits do not depend on the count. */
void orc_set_threads(int threads);
int orc_get_threads(void);

/* ---- input generators and digests (ojas-test-support/src/rng.rs:4-40,
 *      ojas-cpu/tests/exact_golden.rs:43-52) ---- */
uint64_t orc_splitmix_next(uint64_t* state);
void orc_splitmix_vec(uint64_t* state, float* out, size_t n, float scale);
uint64_t orc_splitmix_below(uint64_t* state, uint64_t n);
uint64_t orc_fnv_f32(const float* values, size_t n);

/* ---- exact scalar math (ojas-core/src/exp_exact.rs, erf_exact.rs,
 *      gelu_tanh.rs, autocast.rs:66-101) ---- */
float orc_exp_exact(float x);
float orc_log_sum_exp_exact(float max, float sum);
float orc_log1p_exact(float x);
double orc_erf_f64(double z);
float orc_gelu_erf(float x);
float orc_gelu_erf_backward(float x, float dy);
float orc_gelu_tanh(float x);
float orc_gelu_tanh_backward(float x, float dy);
float orc_sigmoid_exact(float x);
uint16_t orc_f32_to_bf16(float x);
float orc_round_bf16(float x);
void orc_exp_exact_vec(const float* x, float* y, size_t n);
void orc_round_bf16_vec(const float* x, float* y, size_t n);
void orc_to_bf16_vec(const float* x, uint16_t* y, size_t n);
void orc_bf16_to_f32_vec(const uint16_t* x, float* y, size_t n);

/* ---- host scalar formation (ojas-core/src/backend.rs:244-477) ---- */
double orc_pow_u64(double base, uint64_t exp);
int orc_clip_scale(float max_norm, float total_norm, float* coef);
/* words: decay, 1-b1, b2, 1-b2, step_size, sqrt(bc2), eps as f64;
 * flags[0] = decays, flags[1] = lerp_low (f64), flags[2] = lerp_low (f32). */
int orc_adamw_scalars(double lr, double beta1, double beta2, double eps, double weight_decay,
                      uint64_t step_before, double words[7], int32_t flags[3]);

/* ---- matmul class (ojas-cpu/src/linalg.rs:69-210, gemm.rs:1-41) ---- */
int orc_linear_forward(const float* x, const float* w, float* y, size_t rows, size_t kin,
                       size_t nout);
int orc_linear_backward(const float* x, const float* w, const float* gy, float* gx, float* gw,
                        size_t rows, size_t kin, size_t nout);
/* C[m,n] = A[m,k] * B[k,n] with element strides, ascending-k chain from +0.0;
 * `accumulate` continues the chain from the stored C (gemm.rs:365-388). */
int orc_gemm(const float* a, size_t a_rs, size_t a_cs, const float* b, size_t b_rs, size_t b_cs,
             float* c, size_t m, size_t k, size_t n, int accumulate);

/* ---- attention (ojas-cpu/src/attn.rs:47-124,176-227,437-597) ----
 * q,out,gy,gq: [B,H,T,D]; k,v,gk,gv: [B,Hkv,T,D]; lse: [B,H,T].
 * window = 0 means every earlier key. */
int orc_causal_sdpa_forward(const float* q, const float* k, const float* v, float* out, float* lse,
                            size_t batch, size_t heads, size_t kv_heads, size_t time, size_t dim,
                            size_t window);
int orc_causal_sdpa_backward(const float* q, const float* k, const float* v, const float* out,
                             const float* lse, const float* gy, float* gq, float* gk, float* gv,
                             size_t batch, size_t heads, size_t kv_heads, size_t time, size_t dim,
                             size_t window);

/* ---- KV-cache attention (ojas-cpu/src/kv.rs; trait ojas-core/src/backend.rs:2526-2565) ----
 * q, out: [B,Tq,H,D]; caches: [B,Tcap,Hkv,D] rings (position j in slot j % Tcap).
 * window = 0 means every earlier position. */
int orc_cached_attention_forward(const float* q, const float* k_cache, const float* v_cache, float* out,
                                 size_t batch, size_t tq, size_t heads, size_t kv_heads, size_t dim,
                                 size_t capacity, size_t kv_len, size_t window);
int orc_kv_cache_write(float* cache, const float* src, size_t batch, size_t capacity, size_t kv_heads, size_t dim,
                       size_t tn, size_t at);

/* ---- norms and RoPE (ojas-cpu/src/norm.rs) ---- */
int orc_rms_norm_forward(const float* x, const float* w, float* y, size_t rows, size_t dim,
                         float eps);
int orc_rms_norm_backward(const float* x, const float* w, const float* gy, float* gx, float* gw,
                          size_t rows, size_t dim, float eps);
/* TimeDim layout: x is [.., time, heads, dim] rows, cos/sin [time, dim].
 * heads = 0 selects the Same layout (tables shaped like x). */
int orc_rope_forward(const float* x, const float* cos, const float* sin, float* y, size_t rows,
                     size_t dim, size_t time, size_t heads);
int orc_rope_backward(const float* gy, const float* cos, const float* sin, float* gx, size_t rows,
                      size_t dim, size_t time, size_t heads);

/* ---- loss (ojas-cpu/src/pointwise.rs:2167-2486, fused_ce.rs) ----
 * has_ignore = 0 disables ignore_index. */
int orc_cross_entropy_mean_forward(const float* logits, const uint32_t* targets, size_t rows,
                                   size_t vocab, int has_ignore, uint32_t ignore, float* loss);
int orc_cross_entropy_mean_backward(const float* logits, const uint32_t* targets, size_t rows,
                                    size_t vocab, int has_ignore, uint32_t ignore, float* grad);
/* Composed path the fused op equals bit for bit under Exact
 * (ojas-cpu/tests/framework_ce.rs:1-10). gx / gw may be NULL. */
int orc_linear_cross_entropy_mean(const float* x, const float* w, const uint32_t* targets,
                                  size_t rows, size_t dim, size_t vocab, int has_ignore,
                                  uint32_t ignore, float* loss, float* gx, float* gw);

/* ---- embedding (ojas-cpu/src/pointwise.rs:77-100,186-215) ---- */
int orc_embedding_forward(const float* table, const uint32_t* ids, float* out, size_t tokens,
                          size_t vocab, size_t dim);
int orc_embedding_backward(const uint32_t* ids, const float* grad, float* table_grad, size_t tokens,
                           size_t vocab, size_t dim);

/* ---- optimizers (ojas-cpu/src/optim.rs) ---- */
/* exact != 0: f64 element math (optim.rs:186-257); else the Fast f32
 * contract (optim.rs:302-395). Nothing is written on a non-finite value. */
int orc_adamw_step(float* p, const float* g, float* m, float* v, size_t n, uint64_t step_before,
                   double lr, double beta1, double beta2, double eps, double weight_decay,
                   int exact);
int orc_muon_ns5_step(float* p, const float* g, float* m, size_t rows, size_t cols, double lr,
                      double momentum, double weight_decay, int nesterov, int bf16);
/* Global L2 norm (f64 ascending sum of squares) over `count` gradients;
 * scales them in place when the clip coefficient is below 1. */
int orc_clip_grad_norm(float* const* grads, const size_t* lens, size_t count, float max_norm,
                       float* norm);

/* ---- elementwise and layout ---- */
int orc_residual_add(const float* x, const float* y, float* out, size_t n);
int orc_accumulate_grad(float* acc, const float* g, size_t n);
int orc_scale_grad(float* g, float s, size_t n);
void orc_gelu_erf_forward_vec(const float* x, float* y, size_t n);
void orc_gelu_erf_backward_vec(const float* x, const float* gy, float* gx, size_t n);
void orc_gelu_tanh_forward_vec(const float* x, float* y, size_t n);
void orc_gelu_tanh_backward_vec(const float* x, const float* gy, float* gx, size_t n);
/* ---- graph-B pointwise ops (ojas-cpu/src/pointwise.rs:346-366,515-546,
 *      579-620,770-905,1395-1470,1678-1781,1853-1894,2031-2148) ---- */
void orc_silu_forward_vec(const float* x, float* y, size_t n);
void orc_silu_backward_vec(const float* x, const float* gy, float* gx, size_t n);
int orc_mul_forward(const float* a, const float* b, float* out, size_t n);
int orc_mul_backward(const float* a, const float* b, const float* gy, float* ga, float* gb, size_t n);
/* x [rows, din], w [heads, din], bias [heads], attn / y [rows, heads, head_dim]. */
int orc_gate_values(const float* x, const float* w, const float* bias, float* gates, size_t rows,
                    size_t din, size_t heads);
int orc_gate_forward(const float* x, const float* w, const float* bias, const float* attn, float* y,
                     size_t rows, size_t din, size_t heads, size_t head_dim);
int orc_gate_backward(const float* x, const float* w, const float* bias, const float* attn,
                      const float* gy, float* gx, float* gw, float* gb, float* gattn, size_t rows,
                      size_t din, size_t heads, size_t head_dim);
int orc_value_residual_forward(const float* v, const float* v0, float lambda, float* out, size_t n);
int orc_value_residual_backward(const float* v, const float* v0, const float* gy, float lambda,
                                float* gv, float* gv0, float* glambda, size_t n);
/* [d0,d1,d2,d3] -> [d0,d2,d1,d3], bit-preserving (layout.rs:82-118). */
void orc_permute_0213(const float* x, float* y, size_t d0, size_t d1, size_t d2, size_t d3);
/* Ties go to the lowest column; NaN or +inf is ORC_NON_FINITE
 * (ojas-core/src/backend.rs:184-195,1514-1606). */
int orc_argmax_rows(const float* x, size_t rows, size_t cols, uint32_t* out);
int orc_topk_rows(const float* x, size_t rows, size_t cols, size_t k, uint32_t* idx, float* val);

/* ---- GPT-2-shaped training step composed from the ops above ----
 * (embedding x2, residual_add, rms_norm, linear, permute, causal_sdpa, gelu,
 *  cross-entropy, AdamW). Parameter order and sizes: see orc_gpt_param_count /
 * orc_gpt_param_len. gelu: 0 = erf, 1 = tanh. */
typedef struct {
  uint32_t layers, d_model, heads, head_dim, mlp, ctx, vocab, batch, gelu_tanh;
} orc_gpt_config;
size_t orc_gpt_param_count(const orc_gpt_config* c);
size_t orc_gpt_param_len(const orc_gpt_config* c, size_t index);
/* Forward + backward: writes loss and one gradient per parameter. */
int orc_gpt_loss_and_grads(const orc_gpt_config* c, float* const* params, const uint32_t* ids,
                           const uint32_t* targets, float* loss, float* const* grads);

/* ---- nanolab GPT (the reference's model graph, ojas-model/src/block.rs:218-420) ----
 * Parameter order as ojas-model/src/names.rs:188-300. window = 0: full causal. */
typedef struct {
  uint32_t layers, n_embd, n_head, n_kv_head, head_dim, hidden, vocab, batch, seq, window;
  float rms_eps;
  double rope_base;
} orc_nanolab_config;
size_t orc_nanolab_param_count(const orc_nanolab_config* c);
size_t orc_nanolab_param_len(const orc_nanolab_config* c, size_t index);
/* cos / sin [seq, head_dim] (ojas-model/src/block.rs:31-71). */
void orc_rope_tables(size_t seq, size_t head_dim, double base, float* cos, float* sin);
/* logits ([batch*seq, vocab]) and grads may be NULL. */
int orc_nanolab_loss_and_grads(const orc_nanolab_config* c, float* const* params, const uint32_t* ids,
                               const uint32_t* targets, float* loss, float* logits, float* const* grads);
/* The same graph with bf16 roundings placed as a bf16 tier places them (nanolab_exact.cpp): at the
 * products' operands only, or at every point the reference's Autocast rounds; 0 = none. */
enum { ORC_ROUND_OPERANDS = 1, ORC_ROUND_AUTOCAST = 2 };
int orc_nanolab_loss_and_grads_rounded(int rounding, const orc_nanolab_config* c, float* const* params,
                                       const uint32_t* ids, const uint32_t* targets, float* loss, float* const* grads);

/* ---- symmetric int8 weights in groups along the input axis, and the LoRA step over a frozen
 * decoder (oracle/lora_exact.cpp; ojas-cpu/src/quant_sparse.rs:284-346 applied per group,
 * ojas-model/src/lora.rs:292-344) ---- */
int orc_quantize_i8_group(const float* w, int8_t* codes, float* scales, size_t rows, size_t cols, size_t group);
int orc_dequant_i8_group(const int8_t* codes, const float* scales, float* w, size_t rows, size_t cols, size_t group);
int orc_linear_i8_group_forward(const float* x, const int8_t* codes, const float* scales, float* y, size_t rows,
                                size_t kin, size_t nout, size_t group);
int orc_linear_i8_group_backward_input(const int8_t* codes, const float* scales, const float* gy, float* gx,
                                       size_t rows, size_t kin, size_t nout, size_t group);
typedef struct {
  uint32_t layers, d_model, heads, head_dim, hidden, vocab, batch, seq, rank;
  float rms_eps, lora_scale;
  double rope_base;
} orc_lora_config;
size_t orc_lora_frozen_count(const orc_lora_config* c);
size_t orc_lora_adapter_count(const orc_lora_config* c);
/* frozen: dequantised f32 tensors; grads (one per adapter tensor) may be NULL for the loss alone. */
int orc_lora_loss_and_grads(const orc_lora_config* c, const float* const* frozen, const float* const* adapters,
                            const uint32_t* ids, const uint32_t* targets, float* loss, float* const* grads);

#ifdef __cplusplus
}
#endif
#endif
