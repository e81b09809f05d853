/* ojas_mi355x.h: C ABI of the MI355X (gfx950) backend for the nanolab-GPT
 * training-step op set of ojas.
 *
 * The reference has no per-op C ABI: its boundary is the Rust trait
 * `ojas_core::Backend` (ojas-core/src/backend.rs:2634, method list :2655-2767).
 * Each entry point below is what a Rust crate implementing that trait binds
 * for one trait method; the comment on each names the method it serves.
 *
 * Conventions
 *  - Every function returns 0 (OMX_OK) or an omx_status that maps 1:1 onto an
 *    `OjasError` variant (ojas-core/src/error.rs:18-105). The text of the last
 *    error of a context is read with omx_last_error.
 *  - All tensor pointers are DEVICE pointers obtained from omx_alloc (or any
 *    hipMalloc'd memory of the context's device), contiguous row-major. A view
 *    with a byte offset is passed as pointer + offset by the caller.
 *  - Outputs are caller-allocated and fully overwritten. Nothing is freed that
 *    the library did not allocate.
 *  - dtype arguments are omx_dtype values. Matmul-class operands may be
 *    OMX_F32 or OMX_BF16 storage (the reference's bf16 operand slots,
 *    backend.rs:1003-1031); bf16 storage runs on the bf16 MFMA lane with f32
 *    accumulation, f32 storage on the f32 MFMA lane.
 *  - Non-finite detection is deferred (the contract of a device backend,
 *    ojas-wgpu/src/backend.rs:35-73): an op that meets a NaN/Inf returns
 *    OMX_OK, raises its bit in the context's device fault word, and the next
 *    omx_sync / omx_download / omx_clip_grad_norm / omx_read_scalar_f32
 *    returns OMX_NON_FINITE naming the first faulting op. Optimizer steps
 *    decide on the device and write nothing when any value is non-finite.
 *  - A context owns one HIP stream and is not thread-safe.
 */
#ifndef OJAS_MI355X_H
#define OJAS_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct omx_ctx omx_ctx;

/* OjasError variants, ojas-core/src/error.rs:18-105. */
typedef enum {
  OMX_OK = 0,
  OMX_SHAPE = 1,
  OMX_DTYPE = 2,
  OMX_OUT_OF_RANGE = 3,
  OMX_NON_FINITE = 4,
  OMX_UNSUPPORTED_HEAD_DIM = 5,
  OMX_CAPACITY_EXCEEDED = 6,
  OMX_POISONED = 7,
  OMX_DEVICE_LOST = 8,
  OMX_WAIT_TIMEOUT = 9,
  OMX_BACKEND = 10,
  OMX_UNSUPPORTED = 11,
  OMX_PLACEMENT = 12
} omx_status;

/* ojas-core/src/dtype.rs:5 (the three the GPT op set uses). */
typedef enum { OMX_F32 = 0, OMX_BF16 = 1, OMX_U32 = 2 } omx_dtype;

/* ---- context, residency, faults: BackendCore::{upload,download,sync}
 *      (backend.rs:908-973), Budget (ojas-core/src/budget.rs:19-316) ---- */

/* Opens device `device` with a byte budget for omx_alloc (0 = unlimited).
 * Failure kinds follow ojas-hip/src/lib.rs:106-122 (no device ->
 * OMX_DEVICE_LOST, out of memory -> OMX_CAPACITY_EXCEEDED, a device that is
 * not gfx950 -> OMX_UNSUPPORTED). */
int32_t omx_open(int32_t device, uint64_t budget_bytes, omx_ctx** out);
void omx_close(omx_ctx* ctx);
/* Copies the last error text (NUL-terminated) and returns its length. */
size_t omx_last_error(omx_ctx* ctx, char* buf, size_t cap);
/* Name of the device's architecture, e.g. "gfx950". */
size_t omx_device_name(omx_ctx* ctx, char* buf, size_t cap);

/* Budget: charge before allocating, refuse rather than clamp. */
int32_t omx_alloc(omx_ctx* ctx, uint64_t bytes, void** out);
int32_t omx_free(omx_ctx* ctx, void* ptr);
uint64_t omx_budget_live(omx_ctx* ctx);
uint64_t omx_budget_peak(omx_ctx* ctx);
uint64_t omx_budget_limit(omx_ctx* ctx);
/* Bytes of freed blocks the context keeps parked for reuse (at most 4 GiB, blocks of at most
 * 256 MiB; returned to the driver when an allocation fails and at close). The limit and `live`
 * count what callers hold; parked blocks are on top of that. */
uint64_t omx_budget_pooled(omx_ctx* ctx);
void omx_budget_reset_peak(omx_ctx* ctx);

int32_t omx_upload(omx_ctx* ctx, void* dst, uint64_t dst_offset, const void* host_src,
                   uint64_t bytes);
/* Waits for submitted work, reports a deferred fault, then copies. */
int32_t omx_download(omx_ctx* ctx, void* host_dst, const void* src, uint64_t src_offset,
                     uint64_t bytes);
int32_t omx_copy(omx_ctx* ctx, void* dst, const void* src, uint64_t bytes);
int32_t omx_fill_zero(omx_ctx* ctx, void* dst, uint64_t bytes);
/* Waits for all submitted work; reports and clears a deferred fault. */
int32_t omx_sync(omx_ctx* ctx);
/* The context's HIP stream (hipStream_t), for callers that time with events. */
void* omx_stream(omx_ctx* ctx);

/* ---- casts: BackendCore::{cast_bf16,to_bf16,to_f32} (backend.rs:975-1090),
 *      rounding rule ojas-core/src/autocast.rs:66-101 ---- */
int32_t omx_cast_bf16(omx_ctx* ctx, const void* x_f32, void* y_f32, uint64_t n);
int32_t omx_to_bf16(omx_ctx* ctx, const void* x_f32, void* y_bf16, uint64_t n);
int32_t omx_to_f32(omx_ctx* ctx, const void* x_bf16, void* y_f32, uint64_t n);

/* ---- BackendModule::linear_forward (backend.rs:1628):
 *      y[rows,out] = x[rows,in] . W[out,in]^T ---- */
int32_t omx_linear_forward(omx_ctx* ctx, const void* x, int32_t x_dtype, const void* w,
                           int32_t w_dtype, void* y, int32_t y_dtype, uint64_t rows,
                           uint64_t in_features, uint64_t out_features);
/* BackendModule::linear_backward (backend.rs:1631): gx = gy.W, gw = gy^T.x.
 * gx or gw may be NULL (linear_backward_input, backend.rs:1643-1656). */
int32_t omx_linear_backward(omx_ctx* ctx, const void* x, const void* w, const void* gy,
                            int32_t operand_dtype, void* gx, int32_t gx_dtype, void* gw,
                            int32_t gw_dtype, uint64_t rows, uint64_t in_features,
                            uint64_t out_features);
/* General product behind the three above and the Newton-Schulz products:
 * C[m,n] (+)= A.B with A(i,p) at a[i*a_rs + p*a_cs], B(p,j) at b[p*b_rs + j*b_cs]
 * (element strides; one stride of each operand must be 1). */
int32_t omx_gemm(omx_ctx* ctx, const void* a, uint64_t a_rs, uint64_t a_cs, const void* b,
                 uint64_t b_rs, uint64_t b_cs, int32_t operand_dtype, void* c, int32_t c_dtype,
                 uint64_t m, uint64_t k, uint64_t n, int32_t accumulate);

/* omx_gemm whose output rows are `ldc` elements apart (ldc >= n), so the product can be a column
 * block of a wider tensor. No counterpart in the trait. */
int32_t omx_gemm_pitched(omx_ctx* ctx, const void* a, uint64_t a_rs, uint64_t a_cs, const void* b,
                         uint64_t b_rs, uint64_t b_cs, int32_t operand_dtype, void* c, int32_t c_dtype,
                         uint64_t ldc, uint64_t m, uint64_t k, uint64_t n, int32_t accumulate);

/* `count` products of omx_gemm's form in one launch: product i reads its operands stride_a /
 * stride_b ELEMENTS after product i - 1's and writes stride_c elements after its output (strides
 * in multiples of 16 bytes; 1..65535 products). No counterpart in the trait, whose linear ops
 * take one product per call (backend.rs:1628-1656): a caller that keeps the same-shaped layers of
 * a model at a fixed stride uses it for their weight gradients, whose long reductions with small
 * outputs fill the chip only together. */
int32_t omx_gemm_strided_batch(omx_ctx* ctx, const void* a, uint64_t a_rs, uint64_t a_cs, const void* b,
                               uint64_t b_rs, uint64_t b_cs, int32_t operand_dtype, void* c,
                               int32_t c_dtype, uint64_t m, uint64_t k, uint64_t n, int32_t accumulate,
                               uint64_t count, uint64_t stride_a, uint64_t stride_b, uint64_t stride_c);
/* omx_gemm_strided_batch with omx_gemm_pitched's output pitch: product i writes the n columns that
 * start stride_c elements after product i - 1's, in rows `ldc` elements apart, so the products can
 * be adjacent column blocks of one tensor (stride_c = n). No counterpart in the trait. */
int32_t omx_gemm_pitched_strided_batch(omx_ctx* ctx, const void* a, uint64_t a_rs, uint64_t a_cs,
                                       const void* b, uint64_t b_rs, uint64_t b_cs,
                                       int32_t operand_dtype, void* c, int32_t c_dtype,
                                       uint64_t ldc, uint64_t m, uint64_t k, uint64_t n,
                                       int32_t accumulate, uint64_t count, uint64_t stride_a,
                                       uint64_t stride_b, uint64_t stride_c);

/* A frozen linear layer whose weight is stored as symmetric int8 codes [n_out, k_in] with one f32
 * scale per `group` consecutive input columns [n_out, k_in / group] (value = code * scale: the
 * per-channel form of ojas-cpu/src/quant_sparse.rs:284-346 applied to groups; group must be 32).
 * The codes are widened inside the product, on their way from HBM to the matrix units; no bf16
 * copy of the weight exists in memory. In the reference a quantised base reaches the graph as
 * dequantise -> linear_forward (ojas-autograd/src/tape.rs:1514-1518, backend.rs:2586); these two
 * entry points serve that pair of calls for a frozen base, forward and input gradient (a frozen
 * weight has no gradient, ojas-model/src/lora.rs:4-8).
 * x, gy, gx, add: bf16; the forward's y is bf16 or f32 (`y_dtype`: f32 keeps the product unrounded
 * for a pointwise op that follows, so the activation is rounded once, as the next product's
 * operand). `add` (optional, the output's shape) is added to the product before the rounding: the
 * place of the adapter's term in lora_linear (lora.rs:332-344).
 * forward needs k_in % 32 == 0 and n_out % 4 == 0; the input gradient k_in % 32 == 0 and n_out % 32 == 0.
 * `layout`: OMX_I8_ROW_MAJOR (codes [n_out, k_in], scales [n_out, k_in / 32]) or OMX_I8_BLOCKED, the
 * form omx_pack_i8_group writes (same bytes, reordered so that both products read whole cache
 * lines: blocks of 8 rows x 4 groups, [group % 4][row % 8][32 codes] inside a block, the scales
 * likewise; needs k_in % 128 == 0 and n_out % 8 == 0).
 * `low_rank` (optional): the adapter's second product, formed in the same accumulators instead of
 * as a tensor of its own (lora_up + add of lora.rs:326-344): out[n, c] += sum_p h[n][off + p] *
 * w[c][p] for p < rank, with h bf16 [rows, h_pitch] and w bf16 [output columns, w_pitch] (pitches:
 * elements between rows, multiples of 8, so either may be a column block of a wider tensor); rank
 * is a multiple of 16. block_cols > 0: column c reads h at
 * off = (c / block_cols) * rank, so one h [rows, 3 rank] serves a fused q / k / v projection
 * whose three up matrices are stacked in w (block_cols = d; a multiple of 128). For the forward,
 * h = x A^T and w = scale * B; for the input gradient, h = gy (scale * B) and w = A^T.
 * A weight of 2 GiB or more (n_out * k_in >= 2^31) or k_in >= 2^22 is refused with
 * OMX_OUT_OF_RANGE: the kernel addresses a lane's bytes with 32 bits beside a 64-bit base. */
enum { OMX_I8_ROW_MAJOR = 0, OMX_I8_BLOCKED = 1 };
typedef struct {
  const void* h;
  const void* w;
  uint64_t h_pitch, w_pitch, rank, block_cols;
} omx_low_rank;
int32_t omx_linear_i8_group_forward(omx_ctx* ctx, const void* x, int32_t x_dtype, const void* codes_i8,
                                    const void* scales_f32, uint64_t group, int32_t layout,
                                    const void* add, const omx_low_rank* low_rank, void* y,
                                    int32_t y_dtype, uint64_t rows, uint64_t k_in, uint64_t n_out);
int32_t omx_linear_i8_group_backward_input(omx_ctx* ctx, const void* codes_i8, const void* scales_f32,
                                           uint64_t group, int32_t layout, const void* gy,
                                           int32_t gy_dtype, const void* add,
                                           const omx_low_rank* low_rank, void* gx, uint64_t rows,
                                           uint64_t k_in, uint64_t n_out);
/* Reorders row-major codes and scales into the blocked layout (unpack = 0), or a blocked pair back
 * into row-major (unpack = 1: `codes_i8` / `scales_f32` are then the outputs). Out of place. A
 * load-time step of this library's own; the reference keeps quantised weights as plain tensors
 * (ojas-core/src/quant.rs:13-22). */
int32_t omx_pack_i8_group(omx_ctx* ctx, const void* codes_i8, const void* scales_f32, void* blocked_codes,
                          void* blocked_scales, uint64_t n_out, uint64_t k_in, uint64_t group,
                          int32_t unpack);

/* ---- BackendModule::causal_sdpa_forward / _backward (backend.rs:1729-1792).
 *      q,out,gy,gq: [B,H,T,D]; k,v,gk,gv: [B,Hkv,T,D]; lse: [B,H,T] f32.
 *      window = 0: every earlier key. scale = 1/sqrt(D) (backend.rs:159). ---- */
int32_t omx_causal_sdpa_forward(omx_ctx* ctx, const void* q, const void* k, const void* v,
                                int32_t operand_dtype, void* out, int32_t out_dtype, void* lse,
                                uint64_t batch, uint64_t heads, uint64_t kv_heads, uint64_t time,
                                uint64_t head_dim, uint64_t window);
/* out / gy may be stored as f32 or bf16 independently of the operands (the forward writes either;
 * the reference's tensors here are always f32). With bf16 operands an f32 `out` is read in full:
 * the row term dO . O sees the unrounded output. */
int32_t omx_causal_sdpa_backward(omx_ctx* ctx, const void* q, const void* k, const void* v,
                                 const void* out, const void* lse, const void* gy,
                                 int32_t operand_dtype, int32_t out_dtype, int32_t gy_dtype, void* gq,
                                 void* gk, void* gv, int32_t grad_dtype, uint64_t batch,
                                 uint64_t heads, uint64_t kv_heads, uint64_t time, uint64_t head_dim,
                                 uint64_t window);
/* BackendModule::causal_sdpa_backward_recompute (backend.rs:1781-1792): the backward for a caller
 * that kept neither output nor lse (Autocast routes a bf16-tagged saved output here,
 * ojas-core/src/autocast.rs:1200-1233). The forward runs again into the library's scratch with an
 * f32 output, then the backward reads it; gradient arguments are checked before that forward. */
int32_t omx_causal_sdpa_backward_recompute(omx_ctx* ctx, const void* q, const void* k, const void* v,
                                           const void* gy, int32_t operand_dtype, int32_t gy_dtype,
                                           void* gq, void* gk, void* gv, int32_t grad_dtype,
                                           uint64_t batch, uint64_t heads, uint64_t kv_heads,
                                           uint64_t time, uint64_t head_dim, uint64_t window);

/* linear_forward then gelu_{erf,tanh}_forward (backend.rs:1628-1656,1175-1220), the
 * activation applied while the product is stored: u = x W^T and act = gelu(u),
 * both bf16 [rows, out_features]; same bits as the two separate calls. The
 * reverse pair: gu = linear_backward(w, gy).grad_input * gelu'(u), i.e.
 * gelu_backward(u, gy W) in the product's store pass (gy [rows, out_features],
 * w [out_features, in_features], u / gu [rows, in_features]). bf16 only. */
int32_t omx_linear_gelu_forward(omx_ctx* ctx, const void* x, const void* w, int32_t operand_dtype,
                                void* u, void* act, uint64_t rows, uint64_t in_features,
                                uint64_t out_features, int32_t tanh_form);
int32_t omx_linear_backward_input_gelu(omx_ctx* ctx, const void* w, const void* gy,
                                       int32_t operand_dtype, const void* u, void* gu,
                                       uint64_t rows, uint64_t in_features, uint64_t out_features,
                                       int32_t tanh_form);

/* ---- causal_attention (ojas-model/src/block.rs:186-199): permute [0,2,1,3],
 *      causal_sdpa, permute back, done in one pass over time-major tensors.
 *      q / out / gy / gq are [batch, time, heads, head_dim], k / v / gk / gv
 *      [batch, time, kv_heads, head_dim]; a token's heads are contiguous and
 *      token rows are `*_pitch` elements apart (a multiple of 8, at least
 *      heads * head_dim), so q, k and v may be column blocks of one projection
 *      output. gq uses q_pitch, gk / gv use kv_pitch. lse is [batch, heads, time]
 *      f32. bf16 with head_dim 64 or 128; other shapes return Unsupported and the
 *      caller composes omx_permute_0213 with omx_causal_sdpa_*. ---- */
int32_t omx_causal_attention_forward(omx_ctx* ctx, const void* q, uint64_t q_pitch, const void* k,
                                     const void* v, uint64_t kv_pitch, int32_t operand_dtype,
                                     void* out, uint64_t out_pitch, int32_t out_dtype, void* lse,
                                     uint64_t batch, uint64_t time, uint64_t heads,
                                     uint64_t kv_heads, uint64_t head_dim, uint64_t window);
int32_t omx_causal_attention_backward(omx_ctx* ctx, const void* q, uint64_t q_pitch, const void* k,
                                      const void* v, uint64_t kv_pitch, const void* out,
                                      const void* gy, uint64_t out_pitch, const void* lse,
                                      int32_t operand_dtype, void* gq, void* gk, void* gv,
                                      int32_t grad_dtype, uint64_t batch, uint64_t time,
                                      uint64_t heads, uint64_t kv_heads, uint64_t head_dim,
                                      uint64_t window);

/* The same pair with the output's rounding residual kept for the backward pass:
 * out_residual = bf16(x - bf16(x)) for every output value x, laid out like out (same pitch).
 * The backward's row term delta = sum(gy * out) then matches sum_j P dP to 2^-17 instead of 2^-9,
 * which matters when the value rows (and key rows) share a large common component: the mismatch
 * times that component lands in gq and gk. The reference's bf16 tier never rounds the saved
 * output for the same reason ("the backward's dO . O must cancel the softmax row sum",
 * ojas-core/src/autocast.rs:177-186); with bf16 storage the residual is what keeps it. */
int32_t omx_causal_attention_forward_saving(omx_ctx* ctx, const void* q, uint64_t q_pitch,
                                            const void* k, const void* v, uint64_t kv_pitch,
                                            int32_t operand_dtype, void* out, void* out_residual,
                                            uint64_t out_pitch, int32_t out_dtype, void* lse,
                                            uint64_t batch, uint64_t time, uint64_t heads,
                                            uint64_t kv_heads, uint64_t head_dim, uint64_t window);
int32_t omx_causal_attention_backward_saved(omx_ctx* ctx, const void* q, uint64_t q_pitch,
                                            const void* k, const void* v, uint64_t kv_pitch,
                                            const void* out, const void* out_residual,
                                            const void* gy, uint64_t out_pitch, const void* lse,
                                            int32_t operand_dtype, void* gq, void* gk, void* gv,
                                            int32_t grad_dtype, uint64_t batch, uint64_t time,
                                            uint64_t heads, uint64_t kv_heads, uint64_t head_dim,
                                            uint64_t window);

/* ---- BackendModule::rms_norm_forward / _backward (backend.rs:1658-1672) ---- */
int32_t omx_rms_norm_forward(omx_ctx* ctx, const void* x, int32_t x_dtype, const void* w_f32,
                             void* y, int32_t y_dtype, uint64_t rows, uint64_t dim, float eps);
int32_t omx_rms_norm_backward(omx_ctx* ctx, const void* x, int32_t x_dtype, const void* w_f32,
                              const void* gy, int32_t gy_dtype, void* gx, int32_t gx_dtype,
                              void* gw_f32, uint64_t rows, uint64_t dim, float eps);

/* Two-op sequences of the block in one pass over HBM, same bits as the separate calls:
 *   sum = residual_add_forward(x, y); normed = rms_norm_forward(sum, w)
 *     (ojas-model/src/block.rs:247-249; sum is f32);
 *   gx = residual_grad + rms_norm_backward(x, w, gy).gx, the gradient fan-in at
 *     a residual (ojas-autograd/src/tape.rs:2565-2591); gx is f32, gx_bf16
 *     (may be null) receives the same values rounded to bf16; gw_f32 may be null for a
 *     frozen weight, whose gradient is then not formed. */
int32_t omx_residual_add_rms_norm_forward(omx_ctx* ctx, const void* x, int32_t x_dtype,
                                          const void* y, int32_t y_dtype, const void* w_f32,
                                          void* sum_f32, void* normed, int32_t normed_dtype,
                                          uint64_t rows, uint64_t dim, float eps);
int32_t omx_rms_norm_backward_residual(omx_ctx* ctx, const void* x, int32_t x_dtype,
                                       const void* w_f32, const void* gy, int32_t gy_dtype,
                                       const void* residual_grad_f32, void* gx_f32, void* gx_bf16,
                                       void* gw_f32, uint64_t rows, uint64_t dim, float eps);

/* ---- BackendModule::cross_entropy_mean_forward / _backward
 *      (backend.rs:2451-2466). loss is one f32 on the device. ---- */
int32_t omx_cross_entropy_mean_forward(omx_ctx* ctx, const void* logits, int32_t logits_dtype,
                                       const void* targets_u32, uint64_t rows, uint64_t vocab,
                                       int32_t has_ignore, uint32_t ignore_index, void* loss_f32);
/* omx_cross_entropy_mean_forward for callers that cannot allocate (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc). No counterpart in the reference. Same
 * arguments and result; the row state and the valid counter live in a file-scope device array
 * (786,688 bytes per device, held until the process ends) instead of the context's workspace,
 * so the call makes no hipMalloc / hipFree and grows nothing; the array's device address is looked
 * up by omx_open, so the call itself is kernel launches on the context's stream and nothing else.
 * At most 65536 rows: more is
 * OMX_CAPACITY_EXCEEDED and nothing runs. Every call on a device shares that array: calls that
 * overlap on one device (two contexts, two streams) race; calls on one context are stream-ordered
 * and safe. */
int32_t omx_cross_entropy_mean_forward_static(omx_ctx* ctx, const void* logits, int32_t logits_dtype,
                                              const void* targets_u32, uint64_t rows, uint64_t vocab,
                                              int32_t has_ignore, uint32_t ignore_index,
                                              void* loss_f32);
int32_t omx_cross_entropy_mean_backward(omx_ctx* ctx, const void* logits, int32_t logits_dtype,
                                        const void* targets_u32, uint64_t rows, uint64_t vocab,
                                        int32_t has_ignore, uint32_t ignore_index, void* grad,
                                        int32_t grad_dtype);
/* BackendModule::linear_cross_entropy_mean (backend.rs:2493-2524): mean CE of
 * x.W^T without an [N,V] logits tensor; at most chunk_rows x chunk_cols logits
 * exist at once (CeChunk, backend.rs:3081). gx / gw may be NULL (CeGrads). */
int32_t omx_linear_cross_entropy_mean(omx_ctx* ctx, const void* x, const void* w,
                                      int32_t operand_dtype, const void* targets_u32, uint64_t rows,
                                      uint64_t dim, uint64_t vocab, int32_t has_ignore,
                                      uint32_t ignore_index, uint64_t chunk_rows,
                                      uint64_t chunk_cols, void* loss_f32, void* gx,
                                      int32_t gx_dtype, void* gw_f32);

/* ---- BackendModule::embedding_forward / _backward (backend.rs:1610-1626).
 *      The gather is a bit copy; the scatter-add sums each table row's tokens
 *      in ascending token order (ojas-cpu/src/pointwise.rs:171-215). ---- */
int32_t omx_embedding_forward(omx_ctx* ctx, const void* table, int32_t table_dtype,
                              const void* ids_u32, void* out, int32_t out_dtype, uint64_t tokens,
                              uint64_t vocab, uint64_t dim);
int32_t omx_embedding_backward(omx_ctx* ctx, const void* ids_u32, const void* grad,
                               int32_t grad_dtype, void* table_grad_f32, uint64_t tokens,
                               uint64_t vocab, uint64_t dim);
/* embedding_backward followed by accumulate_grad onto `table_grad_f32` (backend.rs:1620-1626, then
 * the tape's sum of the gradients of a value used twice, as a tied table is,
 * ojas-autograd/src/tape.rs:2551-2585) in one pass:
 * each named row's sum is formed as above, then added to what the row holds; rows no token names
 * are neither read nor written. The bits are those of the two ops in sequence. */
int32_t omx_embedding_backward_accumulate(omx_ctx* ctx, const void* ids_u32, const void* grad,
                                          int32_t grad_dtype, void* table_grad_f32,
                                          uint64_t tokens, uint64_t vocab, uint64_t dim);

/* ---- optimizers ---- */
/* ojas_core::AdamWConfig (backend.rs:494-517). */
typedef struct {
  double lr, beta1, beta2, eps, weight_decay;
} omx_adamw_config;
/* BackendModule::adamw_step (backend.rs:2468-2478): `step` is the count before
 * this update. The scalars are formed in f64 on the host
 * (AdamWScalars, backend.rs:371-477) and the element math is f32 (the Fast
 * contract, ojas-cpu/src/optim.rs:302-395). param_bf16, when not NULL, also
 * receives the updated parameter rounded to bf16 (the copy the next step's
 * bf16 matmuls read). */
int32_t omx_adamw_step(omx_ctx* ctx, void* param_f32, const void* grad_f32, void* moment1_f32,
                       void* moment2_f32, uint64_t n, uint64_t step, const omx_adamw_config* config,
                       void* param_bf16);
/* The same update for a caller that owns the tensors between calls (a trainer's arenas). The
 * reference's all-or-nothing rule (nothing is written when any result is non-finite,
 * ojas-cpu/src/optim.rs:302-395) costs a checking pass over all four tensors before the writing
 * one. That pass has nothing to find when every input is below 2^60 in magnitude and the scalars
 * are moderate (step size <= 2^20, |1 - lr wd| <= 2, eps >= 2^-40): no result can overflow. So:
 * `unbounded_flag` (device u32, never cleared here) is OR-ed with 1 when a parameter or moment
 * that stays in memory after the call reaches 2^60 or is not finite: the inputs when the update
 * is refused or checked, the outputs when it is written. `inputs_bounded` != 0 is the caller's
 * word that param, both moments (a zero flag since they were last written from outside) and grad
 * (a finite gradient norm below 2^60) are all below 2^60; the checking pass is then skipped.
 * Results are bit for bit those of omx_adamw_step. No counterpart in the reference, whose backend
 * calls are stateless. `omx_set_option("adamw_trust", 0)` makes every call check. */
int32_t omx_adamw_step_bounded(omx_ctx* ctx, void* param_f32, const void* grad_f32,
                               void* moment1_f32, void* moment2_f32, uint64_t n, uint64_t step,
                               const omx_adamw_config* config, void* param_bf16,
                               int32_t inputs_bounded, void* unbounded_flag);
/* ojas_core::MuonNs5Config (backend.rs:548-570). */
typedef struct {
  double lr, momentum, weight_decay;
  int32_t nesterov;
  int32_t ns5_bf16;
} omx_muon_config;
/* BackendModule::muon_ns5_step (backend.rs:2480-2491). */
int32_t omx_muon_ns5_step(omx_ctx* ctx, void* param_f32, const void* grad_f32, void* momentum_f32,
                          uint64_t rows, uint64_t cols, const omx_muon_config* config,
                          void* param_bf16);
/* The same step for `count` tensors of one shape in one set of launches (no counterpart in
 * the reference, whose trainer calls muon_ns5_step once per tensor, trainer.rs:1004-1028): the
 * arithmetic per tensor is that of omx_muon_ns5_step, the Newton-Schulz products run as strided
 * batches. The arrays hold `count` device pointers (params_bf16 may be null, or hold nulls).
 * All or nothing for the whole batch: a non-finite value in any tensor leaves all of them
 * unchanged. Scratch: count * omx_muon_scratch_bytes(rows, cols), at most 64 tensors at a time. */
int32_t omx_muon_ns5_step_batched(omx_ctx* ctx, void* const* params_f32, const void* const* grads_f32,
                                  void* const* momenta_f32, void* const* params_bf16, uint64_t count,
                                  uint64_t rows, uint64_t cols, const omx_muon_config* config);
/* Bytes of device scratch omx_muon_ns5_step takes from the budget
 * (BackendCore::optimizer_scratch_bytes, backend.rs:938-961). */
uint64_t omx_muon_scratch_bytes(uint64_t rows, uint64_t cols);
/* BackendFloat::clip_grad_norm (backend.rs:1466-1471): global L2 norm with an
 * f64 sum of squares, returned on the host; scales in place when the clip
 * coefficient (clip_scale, backend.rs:277-303) is below 1. A sync point. */
int32_t omx_clip_grad_norm(omx_ctx* ctx, void* const* grads_f32, const uint64_t* lens,
                           uint64_t count, float max_norm, float* norm_out);

/* ---- elementwise and layout ---- */
/* BackendFloat::residual_add_forward (backend.rs:1165-1173): out = x + y, one
 * rounding per element. The operands may differ in storage (an f32 residual
 * stream plus a bf16 branch output). */
int32_t omx_residual_add(omx_ctx* ctx, const void* x, int32_t x_dtype, const void* y, int32_t y_dtype,
                         void* out, int32_t out_dtype, uint64_t n);
/* BackendFloat::accumulate_grad / scale_grad (backend.rs:1473-1510). */
int32_t omx_accumulate_grad(omx_ctx* ctx, void* acc_f32, const void* grad_f32, uint64_t n);
int32_t omx_scale_grad(omx_ctx* ctx, void* grad_f32, float scale, uint64_t n);
/* BackendFloat::gelu_erf_* / gelu_tanh_* (backend.rs:1175-1220). tanh_form
 * selects the tanh approximation. */
int32_t omx_gelu_forward(omx_ctx* ctx, const void* x, void* y, int32_t dtype, uint64_t n,
                         int32_t tanh_form);
int32_t omx_gelu_backward(omx_ctx* ctx, const void* x, const void* gy, void* gx, int32_t dtype,
                          uint64_t n, int32_t tanh_form);
/* ---- KV-cache attention and cache write (the step after the path: decode) ----
 * BackendModule::cached_attention_forward (backend.rs:2526-2555; validator
 * ojas-core/src/shapes.rs:2758-2826; CPU ojas-cpu/src/kv.rs:103-256): q [batch, tq, heads, head_dim]
 * f32 against caches [batch, capacity, kv_heads, head_dim], time-major rings in which position j
 * lives in slot j % capacity. Query i sits at position p = kv_len - tq + i and attends to positions
 * 0..=p, or with a window (0 = none) to p + 1 - window..=p; head h reads KV head
 * h / (heads / kv_heads). out is f32 [batch, tq, heads, head_dim]. kv_len < tq, or a read the ring
 * no longer holds, is OutOfRange. Slots that no query reads are never touched; a NaN or infinity in
 * one that is read raises the deferred NonFinite. cache_dtype OMX_F32 is the trait's contract;
 * OMX_BF16 caches (half the bytes to read) are this library's addition, widened exactly.
 * head_dim: a multiple of 4 up to 256, else UnsupportedHeadDim. */
int32_t omx_cached_attention_forward(omx_ctx* ctx, const void* q, const void* k_cache,
                                     const void* v_cache, int32_t cache_dtype, void* out,
                                     uint64_t batch, uint64_t tq, uint64_t heads, uint64_t kv_heads,
                                     uint64_t head_dim, uint64_t capacity, uint64_t kv_len,
                                     uint64_t window);
/* BackendModule::kv_cache_write (backend.rs:2557-2565; validator shapes.rs:2834-2879; CPU
 * ojas-cpu/src/kv.rs:258-292): src f32 [batch, tn, kv_heads, head_dim] goes to positions
 * at..at + tn of the ring, position j to slot j % capacity (tn <= capacity). All or nothing: a NaN
 * or infinity in src leaves the cache unchanged and raises the deferred NonFinite. A bf16 cache
 * receives the values rounded to nearest even. */
int32_t omx_kv_cache_write(omx_ctx* ctx, void* cache, int32_t cache_dtype, const void* src,
                           uint64_t batch, uint64_t capacity, uint64_t kv_heads, uint64_t head_dim,
                           uint64_t tn, uint64_t at);
/* The batch that BatchSampler::next_batch reads (ojas-data/src/sampler.rs:262-275), built on the
 * device from a token bin resident in HBM: x[b, t] = tokens[starts[b] + t],
 * y[b, t] = tokens[starts[b] + t + 1], u32 [batch, seq_len]. `tokens` is the bin's little-endian
 * token words on the device (bytes_per_token 2 or 4, n_tokens of them); `starts` is a HOST array
 * of `batch` window starts (odata_sampler_next_starts, ojas_data.h). A window that does not lie
 * inside the bin is OutOfRange and nothing is written. */
int32_t omx_token_windows(omx_ctx* ctx, const void* tokens, int32_t bytes_per_token,
                          uint64_t n_tokens, const uint64_t* starts, uint64_t batch,
                          uint64_t seq_len, void* x, void* y);
/* BackendFloat::permute with axes [0,2,1,3] (backend.rs:1115-1134; the one
 * permutation the model uses, ojas-model/src/block.rs:25,195-199):
 * [d0,d1,d2,d3] -> [d0,d2,d1,d3]. */
int32_t omx_permute_0213(omx_ctx* ctx, const void* x, void* y, int32_t dtype, uint64_t d0,
                         uint64_t d1, uint64_t d2, uint64_t d3);

/* ---- ops of the nanolab block (graph B) ---- */
/* BackendFloat::silu_forward / silu_backward (backend.rs:1151-1153; CPU
 * ojas-cpu/src/pointwise.rs:346-366,515-546): y = x sigmoid(x). */
int32_t omx_silu_forward(omx_ctx* ctx, const void* x, void* y, int32_t dtype, uint64_t n);
int32_t omx_silu_backward(omx_ctx* ctx, const void* x, const void* gy, void* gx, int32_t dtype,
                          uint64_t n);
/* BackendFloat::mul_forward / mul_backward (backend.rs:1155-1163): out = a b;
 * ga = gy b, gb = gy a. */
int32_t omx_mul_forward(omx_ctx* ctx, const void* a, const void* b, void* out, int32_t dtype,
                        uint64_t n);
int32_t omx_mul_backward(omx_ctx* ctx, const void* a, const void* b, const void* gy, void* ga,
                         void* gb, int32_t dtype, uint64_t n);
/* BackendModule::rope_half_split_forward / _backward (backend.rs:1674-1686; CPU
 * ojas-cpu/src/norm.rs:271-312). x is [rows, dim] with dim even; cos / sin are
 * f32. heads > 0: tables are [time, dim] and row r uses table row
 * (r / heads) % time (x is [.., time, heads, dim]). heads == 0: tables are
 * shaped like x. The backward takes grad_output in x's place. */
int32_t omx_rope_half_split_forward(omx_ctx* ctx, const void* x, const void* cos_f32,
                                    const void* sin_f32, void* y, int32_t dtype, uint64_t rows,
                                    uint64_t dim, uint64_t time, uint64_t heads);
int32_t omx_rope_half_split_backward(omx_ctx* ctx, const void* gy, const void* cos_f32,
                                     const void* sin_f32, void* gx, int32_t dtype, uint64_t rows,
                                     uint64_t dim, uint64_t time, uint64_t heads);
/* rope_half_split_forward / _backward (backend.rs:1674-1686) applied IN PLACE to the first
 * heads * dim columns of every row of a bf16 [tokens, pitch] tensor: the q and k column blocks
 * of a fused q | k | v projection output (heads = query heads + key heads), which the attention
 * entry points above then read where they lie. cos / sin are f32 [time, dim]; row r uses table
 * row r % time. backward != 0 rotates by the opposite angle (the op's gradient). dim % 16 == 0. */
int32_t omx_rope_half_split_inplace(omx_ctx* ctx, void* x, int32_t dtype, uint64_t pitch,
                                    const void* cos_f32, const void* sin_f32, uint64_t tokens,
                                    uint64_t time, uint64_t heads, uint64_t dim, int32_t backward);
/* The forward of the same out of place, from a projection output kept in f32 (or bf16) to the
 * bf16 tensor attention reads: the first `heads` heads of every token row are rotated, the
 * `plain_heads` that follow (the value heads) are converted as they are; both tensors share the
 * pitch. One rounding per value where the in-place form on a bf16 output makes two. */
int32_t omx_rope_half_split_pitched(omx_ctx* ctx, const void* x, int32_t x_dtype, void* out_bf16,
                                    uint64_t pitch, const void* cos_f32, const void* sin_f32,
                                    uint64_t tokens, uint64_t time, uint64_t heads,
                                    uint64_t plain_heads, uint64_t dim);
/* silu_forward then mul_forward (backend.rs:1151-1163; ojas-model/src/block.rs:248-262) on a fused
 * gate | up projection output: gate_up is [rows, 2 hidden] with the gate columns first, of
 * `dtype` (bf16, or f32: the product's output kept unrounded, so that the activation is rounded
 * once, as the next product's operand); out[r, c] = silu(gate[r, c]) * up[r, c], bf16. The backward
 * writes the gradient of gate_up (bf16, same layout) from gy [rows, hidden] bf16 (mul_backward
 * then silu_backward). hidden % 8 == 0. */
int32_t omx_swiglu_forward(omx_ctx* ctx, const void* gate_up, void* out, int32_t dtype, uint64_t rows,
                           uint64_t hidden);
int32_t omx_swiglu_backward(omx_ctx* ctx, const void* gate_up, const void* gy, void* g_gate_up,
                            int32_t dtype, uint64_t rows, uint64_t hidden);
/* Synthetic weights made on the device (no counterpart in the reference, whose init runs on the
 * host, ojas-model/src/init.rs:67-114): element i is N(0, std) from a counter-based generator of
 * (seed, i). omx_init_normal_i8_group draws row-major [n_out, k_in] values and stores them
 * quantised, codes and one scale per group of 32 (the rule of quant_sparse.rs:306-326 per group). */
int32_t omx_init_normal(omx_ctx* ctx, void* dst, int32_t dtype, uint64_t n, uint64_t seed, float std);
int32_t omx_init_normal_i8_group(omx_ctx* ctx, void* codes_i8, void* scales_f32, uint64_t n_out,
                                 uint64_t k_in, uint64_t group, uint64_t seed, float std);
/* BackendModule::rms_qk_norm_forward / _backward (backend.rs:1688-1708; CPU
 * ojas-cpu/src/backend.rs:1011-1040): RMSNorm over the last axis of q and of k,
 * each with its own weight. Both pairs are validated before either runs. */
int32_t omx_rms_qk_norm_forward(omx_ctx* ctx, const void* q, const void* k, int32_t x_dtype,
                                const void* q_weight_f32, const void* k_weight_f32, void* q_out,
                                void* k_out, int32_t y_dtype, uint64_t q_rows, uint64_t k_rows,
                                uint64_t dim, float eps);
int32_t omx_rms_qk_norm_backward(omx_ctx* ctx, const void* q, const void* k, int32_t x_dtype,
                                 const void* q_weight_f32, const void* k_weight_f32,
                                 const void* grad_q, const void* grad_k, int32_t gy_dtype, void* gq,
                                 void* gk, int32_t gx_dtype, void* gq_weight_f32,
                                 void* gk_weight_f32, uint64_t q_rows, uint64_t k_rows, uint64_t dim,
                                 float eps);
/* BackendModule::per_head_sigmoid_gate_forward[_saving] / _backward[_saved]
 * (backend.rs:1860-1905; CPU ojas-cpu/src/pointwise.rs:1395-1470,1678-1781,
 * 1853-1894): gates[r, h] = sigmoid(bias[h] + input[r, :] . weight[h, :]),
 * y[r, h, :] = attn[r, h, :] gates[r, h]. input [rows, d_model] and weight
 * [heads, d_model] share operand_dtype; bias is f32. `gates_f32` [rows, heads]
 * may be null: the forward then keeps nothing, and the backward recomputes the
 * gates instead of reading saved ones. */
int32_t omx_per_head_sigmoid_gate_forward(omx_ctx* ctx, const void* input, const void* weight,
                                          int32_t operand_dtype, const void* bias_f32,
                                          const void* attn, int32_t attn_dtype, void* y,
                                          int32_t y_dtype, void* gates_f32, uint64_t rows,
                                          uint64_t d_model, uint64_t heads, uint64_t head_dim);
int32_t omx_per_head_sigmoid_gate_backward(omx_ctx* ctx, const void* input, const void* weight,
                                           int32_t operand_dtype, const void* bias_f32,
                                           const void* attn, int32_t attn_dtype, const void* gy,
                                           int32_t gy_dtype, const void* gates_f32, void* g_input,
                                           int32_t g_input_dtype, void* g_weight_f32,
                                           void* g_bias_f32, void* g_attn, int32_t g_attn_dtype,
                                           uint64_t rows, uint64_t d_model, uint64_t heads,
                                           uint64_t head_dim);
/* per_head_sigmoid_gate_backward (backend.rs:1883-1905) without its weight gradient: `gz`
 * [rows, heads] in operand_dtype receives the gradient of the gate's pre-activation, from which
 * the caller forms grad_weight[h, i] = sum_r gz[r, h] input[r, i] itself. For a caller that
 * keeps the layers of a model at a fixed stride and adds up every layer's weight gradient in
 * one omx_gemm_strided_batch at the end of its backward (a 12 x d output over all tokens fills
 * the chip only with the layers side by side). Every other result is the bits of
 * omx_per_head_sigmoid_gate_backward. `g_input` may be null: the caller then takes the input
 * gradient from gz too (omx_per_head_sigmoid_gate_input_grad_add). */
int32_t omx_per_head_sigmoid_gate_backward_deferred(
    omx_ctx* ctx, const void* input, const void* weight, int32_t operand_dtype, const void* bias_f32,
    const void* attn, int32_t attn_dtype, const void* gy, int32_t gy_dtype, const void* gates_f32,
    void* g_input, int32_t g_input_dtype, void* gz, void* g_bias_f32, void* g_attn,
    int32_t g_attn_dtype, uint64_t rows, uint64_t d_model, uint64_t heads, uint64_t head_dim);
/* out_f32[r, i] = add_in[r, i] + sum_h gz[r, h] weight[h, i]: the grad_input of
 * per_head_sigmoid_gate_backward (backend.rs:1883-1905) from the gz that the deferred form hands
 * back, added to another gradient of the same input (residual_add_forward, backend.rs:1165-1173)
 * in one pass, for a caller that passed a null g_input to the deferred form. `out` may not be
 * `add_in`. */
int32_t omx_per_head_sigmoid_gate_input_grad_add(omx_ctx* ctx, const void* gz, const void* weight,
                                                 int32_t operand_dtype, const void* add_in,
                                                 int32_t add_dtype, void* out_f32, uint64_t rows,
                                                 uint64_t d_model, uint64_t heads);
/* BackendModule::value_residual_blend_forward / _backward (backend.rs:1907-1920;
 * CPU ojas-cpu/src/pointwise.rs:2031-2148): out = (1 - s) v + s v0 with
 * s = sigmoid(lambda); lambda and grad_lambda are one f32 each on the device. */
int32_t omx_value_residual_blend_forward(omx_ctx* ctx, const void* value, const void* value0,
                                         const void* lambda_f32, void* out, int32_t dtype,
                                         uint64_t n);
int32_t omx_value_residual_blend_backward(omx_ctx* ctx, const void* value, const void* value0,
                                          const void* lambda_f32, const void* gy, void* g_value,
                                          void* g_value0, int32_t dtype, void* g_lambda_f32,
                                          uint64_t n);

/* rms_qk_norm_forward, rope_half_split_forward and value_residual_blend_forward (backend.rs:1674-1699,
 * 1907-1920; the sequence of ojas-model/src/block.rs:225-240) in one pass over a fused q | k | v
 * projection output: [tokens, pitch] of `lin_dtype` (bf16, or f32: the product's output kept
 * unrounded, so q, k and v reach attention with one rounding) whose token rows hold the query heads,
 * then the key heads, then the value heads; the prepared tensor and both gradients are bf16. q and k heads are normed (weights f32 [head_dim]) and rotated (cos / sin f32
 * [time, head_dim], row r uses table row r % time); the normed row is not rounded to bf16 in
 * between, where the separate calls round. The value heads are blended with those of `value0`
 * (block 0's projection output: same layout, pitch and dtype; lambda f32 [1]), or copied when value0 is
 * NULL. head_dim 64 or 128. The backward takes the gradient of the prepared tensor in the same
 * layout and writes that of the projection output; what the blend sends to block 0's value is
 * written to (value0_grad_first != 0) or added to value0_grad_f32 [tokens, kv_heads * head_dim];
 * add_value_grad_f32 (same shape; the block without a blend) is added to the value's gradient.
 * No counterpart in the trait: a fusion of three of its calls. */
int32_t omx_qkv_prepare_forward(omx_ctx* ctx, const void* qkv_lin, int32_t lin_dtype, void* qkv_out, uint64_t pitch,
                                const void* q_weight_f32, const void* k_weight_f32, const void* cos_f32,
                                const void* sin_f32, const void* value0, const void* lambda_f32,
                                uint64_t tokens, uint64_t time, uint64_t heads, uint64_t kv_heads,
                                uint64_t head_dim, float eps);
int32_t omx_qkv_prepare_backward(omx_ctx* ctx, const void* qkv_lin, int32_t lin_dtype, const void* g_qkv, void* g_qkv_lin,
                                 uint64_t pitch, const void* q_weight_f32, const void* k_weight_f32,
                                 const void* cos_f32, const void* sin_f32, const void* value0,
                                 const void* lambda_f32, void* value0_grad_f32, int32_t value0_grad_first,
                                 const void* add_value_grad_f32, void* g_q_weight_f32, void* g_k_weight_f32,
                                 void* g_lambda_f32, uint64_t tokens, uint64_t time, uint64_t heads,
                                 uint64_t kv_heads, uint64_t head_dim, float eps);

/* ---- BackendInt::argmax_rows / topk_rows (backend.rs:1514-1606) ---- */
int32_t omx_argmax_rows(omx_ctx* ctx, const void* x_f32, uint64_t rows, uint64_t cols,
                        void* out_u32);
int32_t omx_topk_rows(omx_ctx* ctx, const void* x_f32, uint64_t rows, uint64_t cols, uint64_t k,
                      void* values_f32, void* ids_u32);

/* Reads one f32 from the device after a sync (the step's single readback,
 * ojas-model/src/trainer.rs:1031-1046). */
int32_t omx_read_scalar_f32(omx_ctx* ctx, const void* src, float* out);

/* Tuning knobs (no counterpart in the reference). "gemm_dma": 0 = register-staged 128x128 GEMM
 * kernel only, 1 = choose a tiling by the output's tiles per compute unit and the K steps per
 * tile (default), 3 / 4 / 9 / 10 = force the 256x128 (32-column steps) / 128x128 four-wave /
 * 256x256 / 256x192 one-wave-per-SIMD direct-to-LDS kernel wherever the operands are eligible
 * (tests and measurements). "flash_schedule": 0 = the bf16 attention kernels choose
 * between one 128-row block per workgroup and a mirrored pair by how the pairs fill the chip
 * (default), 1 / 2 = always one block / always the pair (the parity tests run both).
 * "gemm_thin": 0 = bf16 products with at most 64 output columns over 1024 rows or
 * more go through the tiled kernels and their split-K reduce instead of the one-pass kernel for
 * thin outputs (default 1). "gemm_row_split": 0 = a product on 256x256 tiles whose last round
 * of tiles fills under 2/5 of the compute units is not cut into two launches by rows (default 1:
 * the rows of the whole rounds keep the tiling, the rest choose their own). "kv_attention": 0 = choose by head_dim (default), 1 = always the
 * LDS-tiled kernel. "ce_fused": 0 = the fused linear-cross-entropy always takes its separate
 * statistics and gradient kernels (default 1: one kernel when a tile holds the whole
 * vocabulary). "adamw_trust": 0 = omx_adamw_step_bounded always runs its checking pass
 * (default 1). "muon_fused_sums": 0 = the bf16 Newton-Schulz iteration forms b A + c A^2 and
 * a X + B X in kernels of their own instead of in the products' store passes (default 1; the
 * same bits either way). "sdpa_tiled": 0 = f32 attention always takes the one-wave-per-row
 * kernels (default 1: LDS-tiled kernels at head_dim 16 / 32 / 64 / 128 with 16-byte aligned
 * f32 tensors). Results are within the same tolerances under every setting. */
int32_t omx_set_option(omx_ctx* ctx, const char* name, int64_t value);

/* Benchmark instrumentation (no counterpart in the reference, whose benches
 * time whole ops from the host, bench/README.md:59): while enabled, every
 * GEMM product's kernels carry a pair of HIP events on their dispatches (the
 * begin timestamp of its first kernel, the end timestamp of its last: the
 * MFMA kernel, or the split-K reduce after it), on the context's stream. The
 * report waits for the stream, sums the products' durations and their
 * 2*M*N*K FLOPs, and clears the record. */
int32_t omx_profile_gemm(omx_ctx* ctx, int32_t enable);
int32_t omx_profile_gemm_report(omx_ctx* ctx, uint64_t* launches, double* total_ms,
                                double* total_flops);
/* The same for the other kernel classes of the step (same standing: benchmark
 * instrumentation with no counterpart in the reference). `class_mask` has one
 * bit per class: 0 the GEMM products (as omx_profile_gemm), 1 flash attention
 * forward, 2 flash attention backward (mean key row, dQ, dK / dV kernels as one
 * launch), 3 the fused cross-entropy row kernel, 4 AdamW (checking pass, when
 * it runs, and update), 5 RMSNorm forward and 6 backward (with the weight
 * gradient's column sum) for row widths 256..2048, 7 embedding backward (count,
 * scan, fill, sort and accumulate kernels as one launch). A launch's work is
 * its algorithmic FLOPs (classes 0..2: 2 B H T^2 D forward and 5 B H T^2 D
 * backward, causal-counted) or its algorithmic bytes (classes 3..7: every
 * operand read once and every result written once). The report sums one class
 * and clears its record. */
int32_t omx_profile_kernels(omx_ctx* ctx, uint32_t class_mask);
int32_t omx_profile_kernels_report(omx_ctx* ctx, int32_t kernel_class, uint64_t* launches,
                                   double* total_ms, double* total_work);

/* Every Backend method outside the GPT op set answers through this: sets the
 * error text to the op's name and returns OMX_UNSUPPORTED
 * (unsupported_op, backend.rs:792-797). */
int32_t omx_unsupported(omx_ctx* ctx, const char* op);

#ifdef __cplusplus
}
#endif
#endif
