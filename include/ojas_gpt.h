/* ojas_gpt.h: host-side training-step driver above the C ABI of
 * ojas_mi355x.h. It plays the part of the reference's generic callers
 * (`Tape<B>` + `Trainer<B>`, ojas-autograd/src/tape.rs:1499-2466,
 * ojas-model/src/trainer.rs:754-1046) for the GPT-2-shaped graph the benchmark
 * configurations describe, composed only of Backend ops:
 *   embedding x2 -> residual_add -> L x { rms_norm, linear q/k/v, permute,
 *   causal_sdpa, permute, linear o, residual_add, rms_norm, linear, gelu,
 *   linear, residual_add } -> rms_norm -> linear_cross_entropy_mean (tied head)
 * followed by clip_grad_norm and adamw_step, with the reference's two sync
 * points per step (the clip norm and the loss readback). It contains no
 * arithmetic of its own besides host scalars.
 */
#ifndef OJAS_GPT_H
#define OJAS_GPT_H

#include <stdint.h>

#include "ojas_mi355x.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ogpt ogpt;

typedef struct {
  uint32_t layers, d_model, heads, head_dim, mlp, ctx, vocab, batch;
  uint32_t gelu_tanh; /* 0: erf GELU, 1: tanh GELU */
  uint32_t bf16;      /* 0: f32 tier; 1: bf16 operands/activations, f32 master weights, residual stream and grads of weights */
} ogpt_config;

int32_t ogpt_create(omx_ctx* ctx, const ogpt_config* config, ogpt** out);
void ogpt_destroy(ogpt* t);

/* Parameters in order: tok[V,d], pos[ctx,d], per layer {norm1[d], wq, wk, wv, wo [d,d], norm2[d],
 * w1[mlp,d], w2[d,mlp]}, final norm[d]. */
uint64_t ogpt_param_count(ogpt* t);
uint64_t ogpt_param_len(ogpt* t, uint64_t index);
int32_t ogpt_set_param(ogpt* t, uint64_t index, const float* host);
int32_t ogpt_get_param(ogpt* t, uint64_t index, float* host);
int32_t ogpt_get_grad(ogpt* t, uint64_t index, float* host);
/* Optimizer state, for a run that resumes (TrainState, ojas-model/src/trainer.rs:300-330): slot 0 is
 * AdamW's first moment or, under ogpt_step_hybrid, a matrix's Muon momentum; slot 1 AdamW's second
 * moment; ogpt_set_steps sets the count that AdamW's bias correction starts from. */
int32_t ogpt_get_state(ogpt* t, uint64_t index, uint32_t slot, float* host);
int32_t ogpt_set_state(ogpt* t, uint64_t index, uint32_t slot, const float* host);
int32_t ogpt_set_steps(ogpt* t, uint64_t steps);
/* N(0, 0.02) matrices and tables from a seeded generator, norm weights 1, moments 0. */
int32_t ogpt_init(ogpt* t, uint64_t seed);

/* Uploads one batch of token ids and targets ([batch, ctx] each); it stays resident. */
int32_t ogpt_set_batch(ogpt* t, const uint32_t* ids, const uint32_t* targets);
/* Forward + backward on the resident batch; returns the loss (one sync). */
int32_t ogpt_loss_and_grads(ogpt* t, float* loss);
/* One optimizer step on the resident batch (Trainer::run with one micro-batch):
 * gradients, clip_grad_norm(grad_clip; <= 0 disables clipping but still
 * measures the norm), adamw_step on every parameter, loss readback. */
int32_t ogpt_step(ogpt* t, const omx_adamw_config* adamw, float grad_clip, float* loss, float* grad_norm);
/* The same step with the reference trainer's hybrid groups (ojas-model/src/trainer.rs:858-876,
 * ojas-cpu/src/train.rs:20-62): muon_ns5_step on every 2-D hidden matrix (wq, wk, wv, wo, w1, w2 of
 * each layer, each its own matrix), adamw_step on the two tables and the norm weights. Muon's
 * momentum lives where AdamW's first moment would. */
int32_t ogpt_step_hybrid(ogpt* t, const omx_muon_config* muon, const omx_adamw_config* adamw, float grad_clip,
                         float* loss, float* grad_norm);
/* Optimizer steps taken so far. */
uint64_t ogpt_steps(ogpt* t);
/* Bytes of device memory the trainer holds. */
uint64_t ogpt_device_bytes(ogpt* t);

#ifdef __cplusplus
}
#endif
#endif
