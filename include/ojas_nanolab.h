/* ojas_nanolab.h: host-side driver of one training step of the nanolab GPT graph (the reference's own
 * model: RMSNorm, q / k / v projections, per-head QK-norm, RoPE, value residual, causal attention
 * with grouped heads and an optional window, per-head sigmoid gate, o projection, SwiGLU, tied
 * head), above the C ABI of ojas_mi355x.h.
 *
 * It plays the part of the reference's callers for this model: `Tape<B>` over the graph of
 * ojas-model/src/block.rs:218-264 (`block_with`) and :343-420 (`hidden`, the tied head) with the
 * backward rules and gradient fan-in of ojas-autograd/src/tape.rs:2004-2466,2565-2591, and
 * `Trainer::run` of ojas-model/src/trainer.rs:754-1046: micro-batches whose backward starts from
 * their weight, gradients summed with accumulate_grad, one clip_grad_norm, muon_ns5_step on the
 * matrices other than the table and adamw_step on the table and the vectors, one loss readback.
 * Activations and operand copies are bf16 when `bf16` is set (f32 residual stream, f32 master
 * weights, gradients and optimizer state), f32 otherwise. It contains no arithmetic of its own
 * besides host scalars.
 */
#ifndef OJAS_NANOLAB_H
#define OJAS_NANOLAB_H

#include <stdint.h>

#include "ojas_mi355x.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct onano onano;

/* ojas_model::ModelSpec (ojas-model/src/spec.rs:45-70) plus the batch shape. window 0 = full causal.
 * bf16 != 0: bf16 operands with every activation rounded once (the forward's product outputs
 * and the attention output the gate reads stay f32 where the fused paths run: that is the
 * whole difference between 2e-2 and 2.5e-2 against the Exact gradients at two or three blocks). */
typedef struct {
  uint32_t layers, n_embd, heads, kv_heads, head_dim, hidden, vocab, batch, seq, window, bf16;
  float rms_eps;
  double rope_base;
} onano_config;

/* heads % kv_heads == 0, head_dim even, n_embd * hidden % 64 == 0. */
int32_t onano_create(omx_ctx* ctx, const onano_config* config, onano** out);
void onano_destroy(onano* t);

/* Parameters in the order of ojas-model/src/names.rs:188-300: tok_emb.weight, then per block
 * norm1.weight, mixer.{q,k,v,o}_proj.weight, mixer.{q,k}_norm.weight, mixer.gate.{weight,bias},
 * mixer.vr_lambda, norm2.weight, ffn.{gate,up,down}.weight, then norm_f.weight. */
uint64_t onano_param_count(onano* t);
uint64_t onano_param_len(onano* t, uint64_t index);
int32_t onano_set_param(onano* t, uint64_t index, const float* host);
int32_t onano_get_param(onano* t, uint64_t index, float* host);
/* The gradient accumulated over the step's micro-batches so far (clipped once onano_apply has run). */
int32_t onano_get_grad(onano* t, uint64_t index, float* host);
/* Optimizer state: slot 0 is Muon's momentum or AdamW's first moment, slot 1 AdamW's second moment
 * (zeros for a Muon parameter); the number of steps taken (TrainState, trainer.rs:300-330). */
int32_t onano_get_state(onano* t, uint64_t index, uint32_t slot, float* host);
int32_t onano_set_state(onano* t, uint64_t index, uint32_t slot, const float* host);
int32_t onano_set_steps(onano* t, uint64_t steps);
uint64_t onano_steps(onano* t);
/* N(0, 0.02) matrices and table, norm weights 1, gate bias 0, vr_lambda 0.5 from a seeded host
 * generator (synthetic weights for benchmarks; the reference's init streams are not restated). */
int32_t onano_init(onano* t, uint64_t seed);

/* The reference's fresh init, `init_params` (ojas-model/src/init.rs:67-114): parameter `name` draws
 * from SplitMix64(seed ^ fnv1a(name)) through Box-Muller in f64 (:35-59), `(std * z) as f32` with
 * std the f32 0.02 widened to f64; norm weights exactly one; o_proj, ffn.down, the gate's bias and
 * vr_lambda exactly zero (ojas-model/src/names.rs:188-300). Optimizer state and the step count are
 * cleared. The logarithm, sine and cosine are the C library's, as the reference's are Rust std's. */
int32_t onano_init_reference(onano* t, uint64_t seed);
/* Row `index` of the parameter table's name (names.rs:188-300), NUL-terminated. */
int32_t onano_param_name(onano* t, uint64_t index, char* out, uint64_t capacity);
/* `init_param` (init.rs:75-112) for one parameter on the host: no device involved. A std that is
 * not positive and finite is OMX_OUT_OF_RANGE (:101-106). */
enum { ONANO_INIT_ZEROS = 0, ONANO_INIT_ONES = 1, ONANO_INIT_NORMAL = 2 };
int32_t onano_reference_init_values(const char* name, uint64_t len, int32_t init, float std_dev, uint64_t seed, float* out);
/* 64-bit FNV-1a of `len` bytes (init.rs:15-29). */
uint64_t onano_fnv1a(const char* bytes, uint64_t len);

/* One micro-batch ([batch, seq] ids and targets): forward and backward with the backward started
 * from `loss_seed` (Tape::backward_seeded, trainer.rs:1089-1119). first != 0 starts a step (the
 * accumulated gradient and loss are replaced), otherwise they are added to. `loss_scale` multiplies
 * the micro-batch's loss before it is added (1 = as it is). */
int32_t onano_micro_batch(onano* t, const uint32_t* ids, const uint32_t* targets, float loss_seed, float loss_scale,
                          int32_t first);
/* The same on the ids and targets uploaded last (they stay resident): a benchmark's steady state. */
int32_t onano_micro_batch_resident(onano* t, float loss_seed, float loss_scale, int32_t first);
/* The accumulated loss (one sync). */
int32_t onano_loss(onano* t, float* loss);
/* The optimizer half of the step on the accumulated gradient: clip_grad_norm (grad_clip <= 0 only
 * measures), Muon on the 2-D parameters other than the table, AdamW on the rest (block 0's
 * vr_lambda, which no gradient reaches, is left alone), the loss readback. */
int32_t onano_apply(onano* t, const omx_muon_config* muon, const omx_adamw_config* adamw, float grad_clip, float* loss,
                    float* grad_norm);
uint64_t onano_device_bytes(onano* t);

#ifdef __cplusplus
}
#endif
#endif
