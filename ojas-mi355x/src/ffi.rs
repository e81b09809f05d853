//! `extern "C"` declarations for `libojas_mi355x.so`: one per entry point of include/ojas_mi355x.h.
//! Written by gen_ffi.py from that header; edit the header and run the script, not this file.
#![allow(non_camel_case_types, clippy::too_many_arguments)]

use std::os::raw::{c_char, c_int, c_void};

#[repr(C)]
pub struct OmxCtx {
    _private: [u8; 0],
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct OmxLowRank {
    pub h: *const c_void,
    pub w: *const c_void,
    pub h_pitch: u64,
    pub w_pitch: u64,
    pub rank: u64,
    pub block_cols: u64,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct OmxAdamwConfig {
    pub lr: f64,
    pub beta1: f64,
    pub beta2: f64,
    pub eps: f64,
    pub weight_decay: f64,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct OmxMuonConfig {
    pub lr: f64,
    pub momentum: f64,
    pub weight_decay: f64,
    pub nesterov: i32,
    pub ns5_bf16: i32,
}

pub const OMX_OK: i32 = 0;
pub const OMX_SHAPE: i32 = 1;
pub const OMX_DTYPE: i32 = 2;
pub const OMX_OUT_OF_RANGE: i32 = 3;
pub const OMX_NON_FINITE: i32 = 4;
pub const OMX_UNSUPPORTED_HEAD_DIM: i32 = 5;
pub const OMX_CAPACITY_EXCEEDED: i32 = 6;
pub const OMX_POISONED: i32 = 7;
pub const OMX_DEVICE_LOST: i32 = 8;
pub const OMX_WAIT_TIMEOUT: i32 = 9;
pub const OMX_BACKEND: i32 = 10;
pub const OMX_UNSUPPORTED: i32 = 11;
pub const OMX_PLACEMENT: i32 = 12;
pub const OMX_F32: i32 = 0;
pub const OMX_BF16: i32 = 1;
pub const OMX_U32: i32 = 2;
pub const OMX_I8_ROW_MAJOR: i32 = 0;
pub const OMX_I8_BLOCKED: i32 = 1;

extern "C" {
    pub fn omx_open(device: i32, budget_bytes: u64, out: *mut *mut OmxCtx) -> i32;
    pub fn omx_close(ctx: *mut OmxCtx);
    pub fn omx_last_error(ctx: *mut OmxCtx, buf: *mut c_char, cap: usize) -> usize;
    pub fn omx_device_name(ctx: *mut OmxCtx, buf: *mut c_char, cap: usize) -> usize;
    pub fn omx_alloc(ctx: *mut OmxCtx, bytes: u64, out: *mut *mut c_void) -> i32;
    pub fn omx_free(ctx: *mut OmxCtx, ptr: *mut c_void) -> i32;
    pub fn omx_budget_live(ctx: *mut OmxCtx) -> u64;
    pub fn omx_budget_peak(ctx: *mut OmxCtx) -> u64;
    pub fn omx_budget_limit(ctx: *mut OmxCtx) -> u64;
    pub fn omx_budget_pooled(ctx: *mut OmxCtx) -> u64;
    pub fn omx_budget_reset_peak(ctx: *mut OmxCtx);
    pub fn omx_upload(ctx: *mut OmxCtx, dst: *mut c_void, dst_offset: u64, host_src: *const c_void, bytes: u64) -> i32;
    pub fn omx_download(ctx: *mut OmxCtx, host_dst: *mut c_void, src: *const c_void, src_offset: u64, bytes: u64) -> i32;
    pub fn omx_copy(ctx: *mut OmxCtx, dst: *mut c_void, src: *const c_void, bytes: u64) -> i32;
    pub fn omx_fill_zero(ctx: *mut OmxCtx, dst: *mut c_void, bytes: u64) -> i32;
    pub fn omx_sync(ctx: *mut OmxCtx) -> i32;
    pub fn omx_stream(ctx: *mut OmxCtx) -> *mut c_void;
    pub fn omx_cast_bf16(ctx: *mut OmxCtx, x_f32: *const c_void, y_f32: *mut c_void, n: u64) -> i32;
    pub fn omx_to_bf16(ctx: *mut OmxCtx, x_f32: *const c_void, y_bf16: *mut c_void, n: u64) -> i32;
    pub fn omx_to_f32(ctx: *mut OmxCtx, x_bf16: *const c_void, y_f32: *mut c_void, n: u64) -> i32;
    pub fn omx_linear_forward(ctx: *mut OmxCtx, x: *const c_void, x_dtype: i32, w: *const c_void, w_dtype: i32, y: *mut c_void, y_dtype: i32, rows: u64, in_features: u64, out_features: u64) -> i32;
    pub fn omx_linear_backward(ctx: *mut OmxCtx, x: *const c_void, w: *const c_void, gy: *const c_void, operand_dtype: i32, gx: *mut c_void, gx_dtype: i32, gw: *mut c_void, gw_dtype: i32, rows: u64, in_features: u64, out_features: u64) -> i32;
    pub fn omx_gemm(ctx: *mut OmxCtx, a: *const c_void, a_rs: u64, a_cs: u64, b: *const c_void, b_rs: u64, b_cs: u64, operand_dtype: i32, c: *mut c_void, c_dtype: i32, m: u64, k: u64, n: u64, accumulate: i32) -> i32;
    pub fn omx_gemm_pitched(ctx: *mut OmxCtx, a: *const c_void, a_rs: u64, a_cs: u64, b: *const c_void, b_rs: u64, b_cs: u64, operand_dtype: i32, c: *mut c_void, c_dtype: i32, ldc: u64, m: u64, k: u64, n: u64, accumulate: i32) -> i32;
    pub fn omx_gemm_strided_batch(ctx: *mut OmxCtx, a: *const c_void, a_rs: u64, a_cs: u64, b: *const c_void, b_rs: u64, b_cs: u64, operand_dtype: i32, c: *mut c_void, c_dtype: i32, m: u64, k: u64, n: u64, accumulate: i32, count: u64, stride_a: u64, stride_b: u64, stride_c: u64) -> i32;
    pub fn omx_gemm_pitched_strided_batch(ctx: *mut OmxCtx, a: *const c_void, a_rs: u64, a_cs: u64, b: *const c_void, b_rs: u64, b_cs: u64, operand_dtype: i32, c: *mut c_void, c_dtype: i32, ldc: u64, m: u64, k: u64, n: u64, accumulate: i32, count: u64, stride_a: u64, stride_b: u64, stride_c: u64) -> i32;
    pub fn omx_linear_i8_group_forward(ctx: *mut OmxCtx, x: *const c_void, x_dtype: i32, codes_i8: *const c_void, scales_f32: *const c_void, group: u64, layout: i32, add: *const c_void, low_rank: *const OmxLowRank, y: *mut c_void, y_dtype: i32, rows: u64, k_in: u64, n_out: u64) -> i32;
    pub fn omx_linear_i8_group_backward_input(ctx: *mut OmxCtx, codes_i8: *const c_void, scales_f32: *const c_void, group: u64, layout: i32, gy: *const c_void, gy_dtype: i32, add: *const c_void, low_rank: *const OmxLowRank, gx: *mut c_void, rows: u64, k_in: u64, n_out: u64) -> i32;
    pub fn omx_pack_i8_group(ctx: *mut OmxCtx, codes_i8: *const c_void, scales_f32: *const c_void, blocked_codes: *mut c_void, blocked_scales: *mut c_void, n_out: u64, k_in: u64, group: u64, unpack: i32) -> i32;
    pub fn omx_causal_sdpa_forward(ctx: *mut OmxCtx, q: *const c_void, k: *const c_void, v: *const c_void, operand_dtype: i32, out: *mut c_void, out_dtype: i32, lse: *mut c_void, batch: u64, heads: u64, kv_heads: u64, time: u64, head_dim: u64, window: u64) -> i32;
    pub fn omx_causal_sdpa_backward(ctx: *mut OmxCtx, q: *const c_void, k: *const c_void, v: *const c_void, out: *const c_void, lse: *const c_void, gy: *const c_void, operand_dtype: i32, out_dtype: i32, gy_dtype: i32, gq: *mut c_void, gk: *mut c_void, gv: *mut c_void, grad_dtype: i32, batch: u64, heads: u64, kv_heads: u64, time: u64, head_dim: u64, window: u64) -> i32;
    pub fn omx_causal_sdpa_backward_recompute(ctx: *mut OmxCtx, q: *const c_void, k: *const c_void, v: *const c_void, gy: *const c_void, operand_dtype: i32, gy_dtype: i32, gq: *mut c_void, gk: *mut c_void, gv: *mut c_void, grad_dtype: i32, batch: u64, heads: u64, kv_heads: u64, time: u64, head_dim: u64, window: u64) -> i32;
    pub fn omx_linear_gelu_forward(ctx: *mut OmxCtx, x: *const c_void, w: *const c_void, operand_dtype: i32, u: *mut c_void, act: *mut c_void, rows: u64, in_features: u64, out_features: u64, tanh_form: i32) -> i32;
    pub fn omx_linear_backward_input_gelu(ctx: *mut OmxCtx, w: *const c_void, gy: *const c_void, operand_dtype: i32, u: *const c_void, gu: *mut c_void, rows: u64, in_features: u64, out_features: u64, tanh_form: i32) -> i32;
    pub fn omx_causal_attention_forward(ctx: *mut OmxCtx, q: *const c_void, q_pitch: u64, k: *const c_void, v: *const c_void, kv_pitch: u64, operand_dtype: i32, out: *mut c_void, out_pitch: u64, out_dtype: i32, lse: *mut c_void, batch: u64, time: u64, heads: u64, kv_heads: u64, head_dim: u64, window: u64) -> i32;
    pub fn omx_causal_attention_backward(ctx: *mut OmxCtx, q: *const c_void, q_pitch: u64, k: *const c_void, v: *const c_void, kv_pitch: u64, out: *const c_void, gy: *const c_void, out_pitch: u64, lse: *const c_void, operand_dtype: i32, gq: *mut c_void, gk: *mut c_void, gv: *mut c_void, grad_dtype: i32, batch: u64, time: u64, heads: u64, kv_heads: u64, head_dim: u64, window: u64) -> i32;
    pub fn omx_causal_attention_forward_saving(ctx: *mut OmxCtx, q: *const c_void, q_pitch: u64, k: *const c_void, v: *const c_void, kv_pitch: u64, operand_dtype: i32, out: *mut c_void, out_residual: *mut c_void, out_pitch: u64, out_dtype: i32, lse: *mut c_void, batch: u64, time: u64, heads: u64, kv_heads: u64, head_dim: u64, window: u64) -> i32;
    pub fn omx_causal_attention_backward_saved(ctx: *mut OmxCtx, q: *const c_void, q_pitch: u64, k: *const c_void, v: *const c_void, kv_pitch: u64, out: *const c_void, out_residual: *const c_void, gy: *const c_void, out_pitch: u64, lse: *const c_void, operand_dtype: i32, gq: *mut c_void, gk: *mut c_void, gv: *mut c_void, grad_dtype: i32, batch: u64, time: u64, heads: u64, kv_heads: u64, head_dim: u64, window: u64) -> i32;
    pub fn omx_rms_norm_forward(ctx: *mut OmxCtx, x: *const c_void, x_dtype: i32, w_f32: *const c_void, y: *mut c_void, y_dtype: i32, rows: u64, dim: u64, eps: f32) -> i32;
    pub fn omx_rms_norm_backward(ctx: *mut OmxCtx, x: *const c_void, x_dtype: i32, w_f32: *const c_void, gy: *const c_void, gy_dtype: i32, gx: *mut c_void, gx_dtype: i32, gw_f32: *mut c_void, rows: u64, dim: u64, eps: f32) -> i32;
    pub fn omx_residual_add_rms_norm_forward(ctx: *mut OmxCtx, x: *const c_void, x_dtype: i32, y: *const c_void, y_dtype: i32, w_f32: *const c_void, sum_f32: *mut c_void, normed: *mut c_void, normed_dtype: i32, rows: u64, dim: u64, eps: f32) -> i32;
    pub fn omx_rms_norm_backward_residual(ctx: *mut OmxCtx, x: *const c_void, x_dtype: i32, w_f32: *const c_void, gy: *const c_void, gy_dtype: i32, residual_grad_f32: *const c_void, gx_f32: *mut c_void, gx_bf16: *mut c_void, gw_f32: *mut c_void, rows: u64, dim: u64, eps: f32) -> i32;
    pub fn omx_cross_entropy_mean_forward(ctx: *mut OmxCtx, logits: *const c_void, logits_dtype: i32, targets_u32: *const c_void, rows: u64, vocab: u64, has_ignore: i32, ignore_index: u32, loss_f32: *mut c_void) -> i32;
    pub fn omx_cross_entropy_mean_forward_static(ctx: *mut OmxCtx, logits: *const c_void, logits_dtype: i32, targets_u32: *const c_void, rows: u64, vocab: u64, has_ignore: i32, ignore_index: u32, loss_f32: *mut c_void) -> i32;
    pub fn omx_cross_entropy_mean_backward(ctx: *mut OmxCtx, logits: *const c_void, logits_dtype: i32, targets_u32: *const c_void, rows: u64, vocab: u64, has_ignore: i32, ignore_index: u32, grad: *mut c_void, grad_dtype: i32) -> i32;
    pub fn omx_linear_cross_entropy_mean(ctx: *mut OmxCtx, x: *const c_void, w: *const c_void, operand_dtype: i32, targets_u32: *const c_void, rows: u64, dim: u64, vocab: u64, has_ignore: i32, ignore_index: u32, chunk_rows: u64, chunk_cols: u64, loss_f32: *mut c_void, gx: *mut c_void, gx_dtype: i32, gw_f32: *mut c_void) -> i32;
    pub fn omx_embedding_forward(ctx: *mut OmxCtx, table: *const c_void, table_dtype: i32, ids_u32: *const c_void, out: *mut c_void, out_dtype: i32, tokens: u64, vocab: u64, dim: u64) -> i32;
    pub fn omx_embedding_backward(ctx: *mut OmxCtx, ids_u32: *const c_void, grad: *const c_void, grad_dtype: i32, table_grad_f32: *mut c_void, tokens: u64, vocab: u64, dim: u64) -> i32;
    pub fn omx_embedding_backward_accumulate(ctx: *mut OmxCtx, ids_u32: *const c_void, grad: *const c_void, grad_dtype: i32, table_grad_f32: *mut c_void, tokens: u64, vocab: u64, dim: u64) -> i32;
    pub fn omx_adamw_step(ctx: *mut OmxCtx, param_f32: *mut c_void, grad_f32: *const c_void, moment1_f32: *mut c_void, moment2_f32: *mut c_void, n: u64, step: u64, config: *const OmxAdamwConfig, param_bf16: *mut c_void) -> i32;
    pub fn omx_adamw_step_bounded(ctx: *mut OmxCtx, param_f32: *mut c_void, grad_f32: *const c_void, moment1_f32: *mut c_void, moment2_f32: *mut c_void, n: u64, step: u64, config: *const OmxAdamwConfig, param_bf16: *mut c_void, inputs_bounded: i32, unbounded_flag: *mut c_void) -> i32;
    pub fn omx_muon_ns5_step(ctx: *mut OmxCtx, param_f32: *mut c_void, grad_f32: *const c_void, momentum_f32: *mut c_void, rows: u64, cols: u64, config: *const OmxMuonConfig, param_bf16: *mut c_void) -> i32;
    pub fn omx_muon_ns5_step_batched(ctx: *mut OmxCtx, params_f32: *const *mut c_void, grads_f32: *const *const c_void, momenta_f32: *const *mut c_void, params_bf16: *const *mut c_void, count: u64, rows: u64, cols: u64, config: *const OmxMuonConfig) -> i32;
    pub fn omx_muon_scratch_bytes(rows: u64, cols: u64) -> u64;
    pub fn omx_clip_grad_norm(ctx: *mut OmxCtx, grads_f32: *const *mut c_void, lens: *const u64, count: u64, max_norm: f32, norm_out: *mut f32) -> i32;
    pub fn omx_residual_add(ctx: *mut OmxCtx, x: *const c_void, x_dtype: i32, y: *const c_void, y_dtype: i32, out: *mut c_void, out_dtype: i32, n: u64) -> i32;
    pub fn omx_accumulate_grad(ctx: *mut OmxCtx, acc_f32: *mut c_void, grad_f32: *const c_void, n: u64) -> i32;
    pub fn omx_scale_grad(ctx: *mut OmxCtx, grad_f32: *mut c_void, scale: f32, n: u64) -> i32;
    pub fn omx_gelu_forward(ctx: *mut OmxCtx, x: *const c_void, y: *mut c_void, dtype: i32, n: u64, tanh_form: i32) -> i32;
    pub fn omx_gelu_backward(ctx: *mut OmxCtx, x: *const c_void, gy: *const c_void, gx: *mut c_void, dtype: i32, n: u64, tanh_form: i32) -> i32;
    pub fn omx_cached_attention_forward(ctx: *mut OmxCtx, q: *const c_void, k_cache: *const c_void, v_cache: *const c_void, cache_dtype: i32, out: *mut c_void, batch: u64, tq: u64, heads: u64, kv_heads: u64, head_dim: u64, capacity: u64, kv_len: u64, window: u64) -> i32;
    pub fn omx_kv_cache_write(ctx: *mut OmxCtx, cache: *mut c_void, cache_dtype: i32, src: *const c_void, batch: u64, capacity: u64, kv_heads: u64, head_dim: u64, tn: u64, at: u64) -> i32;
    pub fn omx_token_windows(ctx: *mut OmxCtx, tokens: *const c_void, bytes_per_token: i32, n_tokens: u64, starts: *const u64, batch: u64, seq_len: u64, x: *mut c_void, y: *mut c_void) -> i32;
    pub fn omx_permute_0213(ctx: *mut OmxCtx, x: *const c_void, y: *mut c_void, dtype: i32, d0: u64, d1: u64, d2: u64, d3: u64) -> i32;
    pub fn omx_silu_forward(ctx: *mut OmxCtx, x: *const c_void, y: *mut c_void, dtype: i32, n: u64) -> i32;
    pub fn omx_silu_backward(ctx: *mut OmxCtx, x: *const c_void, gy: *const c_void, gx: *mut c_void, dtype: i32, n: u64) -> i32;
    pub fn omx_mul_forward(ctx: *mut OmxCtx, a: *const c_void, b: *const c_void, out: *mut c_void, dtype: i32, n: u64) -> i32;
    pub fn omx_mul_backward(ctx: *mut OmxCtx, a: *const c_void, b: *const c_void, gy: *const c_void, ga: *mut c_void, gb: *mut c_void, dtype: i32, n: u64) -> i32;
    pub fn omx_rope_half_split_forward(ctx: *mut OmxCtx, x: *const c_void, cos_f32: *const c_void, sin_f32: *const c_void, y: *mut c_void, dtype: i32, rows: u64, dim: u64, time: u64, heads: u64) -> i32;
    pub fn omx_rope_half_split_backward(ctx: *mut OmxCtx, gy: *const c_void, cos_f32: *const c_void, sin_f32: *const c_void, gx: *mut c_void, dtype: i32, rows: u64, dim: u64, time: u64, heads: u64) -> i32;
    pub fn omx_rope_half_split_inplace(ctx: *mut OmxCtx, x: *mut c_void, dtype: i32, pitch: u64, cos_f32: *const c_void, sin_f32: *const c_void, tokens: u64, time: u64, heads: u64, dim: u64, backward: i32) -> i32;
    pub fn omx_rope_half_split_pitched(ctx: *mut OmxCtx, x: *const c_void, x_dtype: i32, out_bf16: *mut c_void, pitch: u64, cos_f32: *const c_void, sin_f32: *const c_void, tokens: u64, time: u64, heads: u64, plain_heads: u64, dim: u64) -> i32;
    pub fn omx_swiglu_forward(ctx: *mut OmxCtx, gate_up: *const c_void, out: *mut c_void, dtype: i32, rows: u64, hidden: u64) -> i32;
    pub fn omx_swiglu_backward(ctx: *mut OmxCtx, gate_up: *const c_void, gy: *const c_void, g_gate_up: *mut c_void, dtype: i32, rows: u64, hidden: u64) -> i32;
    pub fn omx_init_normal(ctx: *mut OmxCtx, dst: *mut c_void, dtype: i32, n: u64, seed: u64, std: f32) -> i32;
    pub fn omx_init_normal_i8_group(ctx: *mut OmxCtx, codes_i8: *mut c_void, scales_f32: *mut c_void, n_out: u64, k_in: u64, group: u64, seed: u64, std: f32) -> i32;
    pub fn omx_rms_qk_norm_forward(ctx: *mut OmxCtx, q: *const c_void, k: *const c_void, x_dtype: i32, q_weight_f32: *const c_void, k_weight_f32: *const c_void, q_out: *mut c_void, k_out: *mut c_void, y_dtype: i32, q_rows: u64, k_rows: u64, dim: u64, eps: f32) -> i32;
    pub fn omx_rms_qk_norm_backward(ctx: *mut OmxCtx, q: *const c_void, k: *const c_void, x_dtype: i32, q_weight_f32: *const c_void, k_weight_f32: *const c_void, grad_q: *const c_void, grad_k: *const c_void, gy_dtype: i32, gq: *mut c_void, gk: *mut c_void, gx_dtype: i32, gq_weight_f32: *mut c_void, gk_weight_f32: *mut c_void, q_rows: u64, k_rows: u64, dim: u64, eps: f32) -> i32;
    pub fn omx_per_head_sigmoid_gate_forward(ctx: *mut OmxCtx, input: *const c_void, weight: *const c_void, operand_dtype: i32, bias_f32: *const c_void, attn: *const c_void, attn_dtype: i32, y: *mut c_void, y_dtype: i32, gates_f32: *mut c_void, rows: u64, d_model: u64, heads: u64, head_dim: u64) -> i32;
    pub fn omx_per_head_sigmoid_gate_backward(ctx: *mut OmxCtx, input: *const c_void, weight: *const c_void, operand_dtype: i32, bias_f32: *const c_void, attn: *const c_void, attn_dtype: i32, gy: *const c_void, gy_dtype: i32, gates_f32: *const c_void, g_input: *mut c_void, g_input_dtype: i32, g_weight_f32: *mut c_void, g_bias_f32: *mut c_void, g_attn: *mut c_void, g_attn_dtype: i32, rows: u64, d_model: u64, heads: u64, head_dim: u64) -> i32;
    pub fn omx_per_head_sigmoid_gate_backward_deferred(ctx: *mut OmxCtx, input: *const c_void, weight: *const c_void, operand_dtype: i32, bias_f32: *const c_void, attn: *const c_void, attn_dtype: i32, gy: *const c_void, gy_dtype: i32, gates_f32: *const c_void, g_input: *mut c_void, g_input_dtype: i32, gz: *mut c_void, g_bias_f32: *mut c_void, g_attn: *mut c_void, g_attn_dtype: i32, rows: u64, d_model: u64, heads: u64, head_dim: u64) -> i32;
    pub fn omx_per_head_sigmoid_gate_input_grad_add(ctx: *mut OmxCtx, gz: *const c_void, weight: *const c_void, operand_dtype: i32, add_in: *const c_void, add_dtype: i32, out_f32: *mut c_void, rows: u64, d_model: u64, heads: u64) -> i32;
    pub fn omx_value_residual_blend_forward(ctx: *mut OmxCtx, value: *const c_void, value0: *const c_void, lambda_f32: *const c_void, out: *mut c_void, dtype: i32, n: u64) -> i32;
    pub fn omx_value_residual_blend_backward(ctx: *mut OmxCtx, value: *const c_void, value0: *const c_void, lambda_f32: *const c_void, gy: *const c_void, g_value: *mut c_void, g_value0: *mut c_void, dtype: i32, g_lambda_f32: *mut c_void, n: u64) -> i32;
    pub fn omx_qkv_prepare_forward(ctx: *mut OmxCtx, qkv_lin: *const c_void, lin_dtype: i32, qkv_out: *mut c_void, pitch: u64, q_weight_f32: *const c_void, k_weight_f32: *const c_void, cos_f32: *const c_void, sin_f32: *const c_void, value0: *const c_void, lambda_f32: *const c_void, tokens: u64, time: u64, heads: u64, kv_heads: u64, head_dim: u64, eps: f32) -> i32;
    pub fn omx_qkv_prepare_backward(ctx: *mut OmxCtx, qkv_lin: *const c_void, lin_dtype: i32, g_qkv: *const c_void, g_qkv_lin: *mut c_void, pitch: u64, q_weight_f32: *const c_void, k_weight_f32: *const c_void, cos_f32: *const c_void, sin_f32: *const c_void, value0: *const c_void, lambda_f32: *const c_void, value0_grad_f32: *mut c_void, value0_grad_first: i32, add_value_grad_f32: *const c_void, g_q_weight_f32: *mut c_void, g_k_weight_f32: *mut c_void, g_lambda_f32: *mut c_void, tokens: u64, time: u64, heads: u64, kv_heads: u64, head_dim: u64, eps: f32) -> i32;
    pub fn omx_argmax_rows(ctx: *mut OmxCtx, x_f32: *const c_void, rows: u64, cols: u64, out_u32: *mut c_void) -> i32;
    pub fn omx_topk_rows(ctx: *mut OmxCtx, x_f32: *const c_void, rows: u64, cols: u64, k: u64, values_f32: *mut c_void, ids_u32: *mut c_void) -> i32;
    pub fn omx_read_scalar_f32(ctx: *mut OmxCtx, src: *const c_void, out: *mut f32) -> i32;
    pub fn omx_set_option(ctx: *mut OmxCtx, name: *const c_char, value: i64) -> i32;
    pub fn omx_profile_gemm(ctx: *mut OmxCtx, enable: i32) -> i32;
    pub fn omx_profile_gemm_report(ctx: *mut OmxCtx, launches: *mut u64, total_ms: *mut f64, total_flops: *mut f64) -> i32;
    pub fn omx_profile_kernels(ctx: *mut OmxCtx, class_mask: u32) -> i32;
    pub fn omx_profile_kernels_report(ctx: *mut OmxCtx, kernel_class: i32, launches: *mut u64, total_ms: *mut f64, total_work: *mut f64) -> i32;
    pub fn omx_unsupported(ctx: *mut OmxCtx, op: *const c_char) -> i32;
}
