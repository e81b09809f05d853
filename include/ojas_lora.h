/* ojas_lora.h: host-side driver of one LoRA fine-tune step over a frozen, int8-quantised
 * Llama-shaped decoder, above the C ABI of ojas_mi355x.h.
 *
 * It plays the part of the reference's callers for this workload: `Tape<B>` over the graph of
 * ojas-model/src/lora.rs:292-344 (lora_linear on the q, k, v and o projections of a frozen base,
 * `Graph::frozen` for everything else) and the step of ojas-model/src/trainer.rs:754-1046
 * (clip_grad_norm, adamw_step on the trainable leaves only, one loss readback). Per block:
 *   rms_norm -> lora_linear q | k | v (one fused projection) -> rope_half_split on q and k ->
 *   causal attention -> lora_linear o -> residual -> rms_norm -> linear gate | up (fused) ->
 *   silu * up -> linear down -> residual;   then rms_norm -> linear_cross_entropy_mean (tied table).
 * The base matrices are symmetric int8 in groups of 32 input columns with f32 scales and are
 * used through omx_linear_i8_group_forward / _backward_input; the table and the norm weights are
 * frozen too. bf16 activations, f32 residual stream, f32 master adapters with bf16 operand copies.
 * It contains no arithmetic of its own besides host scalars.
 */
#ifndef OJAS_LORA_H
#define OJAS_LORA_H

#include <stdint.h>

#include "ojas_mi355x.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct olora olora;

typedef struct {
  uint32_t layers, d_model, heads, head_dim, hidden, vocab, batch, seq, rank;
  float rms_eps;
  float lora_scale; /* alpha / rank (LoraConfig::scaling, lora.rs:128-140) */
  double rope_base;
} olora_config;

/* d_model % 128 == 0, hidden % 128 == 0, head_dim 64 or 128, rank % 16 == 0. */
int32_t olora_create(omx_ctx* ctx, const olora_config* config, olora** out);
void olora_destroy(olora* t);

/* ---- the frozen base ---- */
/* The token table [vocab, d_model] (also the head); kept as bf16. */
int32_t olora_set_embedding(olora* t, const float* host);
/* Norm weights [d_model]: which 0 = the block's first norm, 1 = its second; layer == layers: the final norm. */
int32_t olora_set_norm(olora* t, uint32_t layer, uint32_t which, const float* host);
/* A base matrix as row-major codes [n_out, k_in] and scales [n_out, k_in / 32].
 * which: 0 wq, 1 wk, 2 wv, 3 wo ([d, d]); 4 wgate, 5 wup ([hidden, d]); 6 wdown ([d, hidden]). */
int32_t olora_set_matrix(olora* t, uint32_t layer, uint32_t which, const int8_t* codes, const float* scales);
/* A synthetic base made on the device: every matrix N(0, std) from a counter-based generator,
 * quantised per group; table N(0, std) rounded to bf16; norm weights 1. */
int32_t olora_init_base(olora* t, uint64_t seed, float std);

/* ---- the adapters: index = layer * 8 + {0 Aq, 1 Bq, 2 Ak, 3 Bk, 4 Av, 5 Bv, 6 Ao, 7 Bo};
 *      A is [rank, d_model], B is [d_model, rank] ---- */
uint64_t olora_adapter_count(olora* t);
uint64_t olora_adapter_len(olora* t, uint64_t index);
int32_t olora_set_adapter(olora* t, uint64_t index, const float* host);
int32_t olora_get_adapter(olora* t, uint64_t index, float* host);
int32_t olora_get_grad(olora* t, uint64_t index, float* host);
/* A ~ N(0, std), B = 0, moments 0, step count 0. */
int32_t olora_init_adapters(olora* t, uint64_t seed, float std);

/* Uploads one batch of token ids and targets ([batch, seq] each); it stays resident. */
int32_t olora_set_batch(olora* t, const uint32_t* ids, const uint32_t* targets);
/* Forward + backward on the resident batch; returns the loss (one sync). */
int32_t olora_loss_and_grads(olora* t, float* loss);
/* One optimizer step: gradients, clip_grad_norm (grad_clip <= 0 only measures), adamw_step on the
 * adapters, loss readback. */
int32_t olora_step(olora* t, const omx_adamw_config* adamw, float grad_clip, float* loss, float* grad_norm);
uint64_t olora_steps(olora* t);
uint64_t olora_device_bytes(olora* t);

#ifdef __cplusplus
}
#endif
#endif
