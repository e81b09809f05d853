// Context, budget, residency and deferred-fault plumbing of libojas_mi355x.
//
// Mirrors what a device backend owns below ojas_core::Backend: placement
// (upload/download, backend.rs:908-973), budget charging that refuses rather
// than clamps (ojas-core/src/budget.rs:257-316), and the deferred non-finite
// contract of a device backend (ojas-wgpu/src/backend.rs:35-73).
#include "omx_common.h"

static const char* kFaultNames[F_COUNT] = {
    "linear_forward",
    "linear_backward",
    "gemm",
    "causal_sdpa_forward",
    "causal_sdpa_backward",
    "rms_norm_forward",
    "rms_norm_backward",
    "cross_entropy_mean_forward",
    "cross_entropy_mean_backward",
    "linear_cross_entropy_mean",
    "embedding_forward",
    "embedding_backward",
    "adamw_step",
    "muon_ns5_step",
    "clip_grad_norm",
    "residual_add_forward",
    "accumulate_grad",
    "scale_grad",
    "gelu_forward",
    "gelu_backward",
    "argmax_rows",
    "topk_rows",
    "silu_forward",
    "silu_backward",
    "mul_forward",
    "mul_backward",
    "rope_half_split_forward",
    "rope_half_split_backward",
    "rms_qk_norm_forward",
    "rms_qk_norm_backward",
    "per_head_sigmoid_gate_forward",
    "per_head_sigmoid_gate_backward",
    "value_residual_blend_forward",
    "value_residual_blend_backward",
    "cached_attention_forward",
    "kv_cache_write",
};

const char* omx_fault_name(uint32_t op) { return op < F_COUNT ? kFaultNames[op] : "unknown"; }

int32_t omx_fail(omx_ctx* ctx, omx_status code, const char* fmt, ...) {
  if (ctx) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    ctx->last_error = buf;
  }
  return code;
}

// HIP status mapping follows ojas-hip/src/lib.rs:106-122: 2 is out of memory,
// 3/4/35/100/101 mean no usable device, anything else is a launch failure.
int32_t omx_hip_fail(omx_ctx* ctx, hipError_t err, const char* what) {
  int code = static_cast<int>(err);
  omx_status st = OMX_BACKEND;
  if (code == 2) st = OMX_CAPACITY_EXCEEDED;
  else if (code == 3 || code == 4 || code == 35 || code == 100 || code == 101) st = OMX_DEVICE_LOST;
  return omx_fail(ctx, st, "hip: %s failed: %s (%d)", what, hipGetErrorString(err), code);
}

static int32_t reset_fault(omx_ctx* ctx) {
  ctx->fault_host->mask = 0;
  ctx->fault_host->first = ~0ull;
  OMX_HIP(ctx, hipMemcpyAsync(ctx->fault, ctx->fault_host, sizeof(OmxFaultWord), hipMemcpyHostToDevice,
                              ctx->stream));
  OMX_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return OMX_OK;
}

extern "C" {

int32_t omx_open(int32_t device, uint64_t budget_bytes, omx_ctx** out) {
  if (!out) return OMX_BACKEND;
  *out = nullptr;
  int count = 0;
  hipError_t err = hipGetDeviceCount(&count);
  if (err != hipSuccess || count <= 0 || device < 0 || device >= count) return OMX_DEVICE_LOST;
  omx_ctx* ctx = new omx_ctx();
  ctx->device = device;
  ctx->budget_limit = budget_bytes;
  if (hipSetDevice(device) != hipSuccess) {
    delete ctx;
    return OMX_DEVICE_LOST;
  }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) != hipSuccess) {
    delete ctx;
    return OMX_DEVICE_LOST;
  }
  ctx->arch = prop.gcnArchName;
  ctx->cu_count = prop.multiProcessorCount;
  if (ctx->arch.rfind("gfx950", 0) != 0) {
    // The kernels are built for gfx950 only; any other device cannot run them.
    delete ctx;
    return OMX_UNSUPPORTED;
  }
  if (hipStreamCreate(&ctx->stream) != hipSuccess || hipMalloc(&ctx->fault, sizeof(OmxFaultWord)) != hipSuccess ||
      hipHostMalloc(&ctx->fault_host, sizeof(OmxFaultWord)) != hipSuccess) {
    delete ctx;
    return OMX_BACKEND;
  }
  if (reset_fault(ctx) != OMX_OK) {
    delete ctx;
    return OMX_BACKEND;
  }
  ctx->ce_static_scratch = omx_ce_static_scratch_address();
  *out = ctx;
  return OMX_OK;
}

void omx_close(omx_ctx* ctx) {
  if (!ctx) return;
  (void)hipSetDevice(ctx->device);
  (void)hipStreamSynchronize(ctx->stream);
  for (auto& kv : ctx->allocations) (void)hipFree(kv.first);
  for (auto& kv : ctx->pool) (void)hipFree(kv.second);
  if (ctx->fault) (void)hipFree(ctx->fault);
  if (ctx->fault_host) (void)hipHostFree(ctx->fault_host);
  if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
  delete ctx;
}

size_t omx_last_error(omx_ctx* ctx, char* buf, size_t cap) {
  if (!ctx) return 0;
  if (buf && cap) {
    size_t n = ctx->last_error.size() < cap - 1 ? ctx->last_error.size() : cap - 1;
    memcpy(buf, ctx->last_error.data(), n);
    buf[n] = 0;
  }
  return ctx->last_error.size();
}

size_t omx_device_name(omx_ctx* ctx, char* buf, size_t cap) {
  if (!ctx) return 0;
  if (buf && cap) {
    size_t n = ctx->arch.size() < cap - 1 ? ctx->arch.size() : cap - 1;
    memcpy(buf, ctx->arch.data(), n);
    buf[n] = 0;
  }
  return ctx->arch.size();
}

}  // extern "C"

// Returns every parked block to the device (waits for the stream first).
void omx_release_pool(omx_ctx* ctx) {
  if (ctx->pool.empty()) return;
  (void)hipStreamSynchronize(ctx->stream);
  for (auto& kv : ctx->pool) (void)hipFree(kv.second);
  ctx->pool.clear();
  ctx->pooled_bytes = 0;
}

extern "C" {

int32_t omx_alloc(omx_ctx* ctx, uint64_t bytes, void** out) {
  OMX_REQUIRE_CTX(ctx);
  if (!out) return omx_fail(ctx, OMX_BACKEND, "omx_alloc: null out");
  *out = nullptr;
  if (bytes == 0) return omx_fail(ctx, OMX_SHAPE, "omx_alloc: zero bytes");
  // Charge before allocating; refuse, never clamp (budget.rs:257-316).
  if (ctx->budget_limit && (bytes > ctx->budget_limit || ctx->budget_live > ctx->budget_limit - bytes))
    return omx_fail(ctx, OMX_CAPACITY_EXCEEDED, "requested %llu cap %llu live %llu", (unsigned long long)bytes,
                    (unsigned long long)ctx->budget_limit, (unsigned long long)ctx->budget_live);
  void* p = nullptr;
  auto pooled = ctx->pool.find(bytes);
  if (pooled != ctx->pool.end()) {
    // A block of this size freed earlier: every use of it is on this context's stream, so work
    // launched from here on is ordered after whatever still reads it.
    p = pooled->second;
    ctx->pool.erase(pooled);
    ctx->pooled_bytes -= bytes;
  } else {
    hipError_t err = hipMalloc(&p, bytes);
    if (err != hipSuccess && !ctx->pool.empty()) {
      // Out of device memory with blocks parked in the pool: give them back and try once more.
      (void)hipGetLastError();
      omx_release_pool(ctx);
      err = hipMalloc(&p, bytes);
    }
    if (err != hipSuccess) return omx_hip_fail(ctx, err, "hipMalloc");
  }
  ctx->allocations[p] = bytes;
  ctx->budget_live += bytes;
  if (ctx->budget_live > ctx->budget_peak) ctx->budget_peak = ctx->budget_live;
  *out = p;
  return OMX_OK;
}

int32_t omx_free(omx_ctx* ctx, void* ptr) {
  OMX_REQUIRE_CTX(ctx);
  if (!ptr) return OMX_OK;
  auto it = ctx->allocations.find(ptr);
  if (it == ctx->allocations.end()) return omx_fail(ctx, OMX_PLACEMENT, "omx_free: pointer not from this context");
  const uint64_t bytes = it->second;
  ctx->budget_live -= bytes;
  ctx->allocations.erase(it);
  // Freeing for real would wait for the stream (work that still reads the buffer is on it) and for
  // the whole device (hipFree). Blocks of moderate size are parked instead and handed out again by
  // omx_alloc to a request of the same size; reuse is safe without a wait because the next user's
  // work goes onto the same stream. The pool is not charged to the budget: the budget counts what
  // callers hold.
  constexpr uint64_t kMaxBlock = 256ull << 20, kMaxPool = 4ull << 30;
  if (bytes <= kMaxBlock && ctx->pooled_bytes + bytes <= kMaxPool) {
    ctx->pool.emplace(bytes, ptr);
    ctx->pooled_bytes += bytes;
    return OMX_OK;
  }
  OMX_HIP(ctx, hipStreamSynchronize(ctx->stream));
  OMX_HIP(ctx, hipFree(ptr));
  return OMX_OK;
}

uint64_t omx_budget_live(omx_ctx* ctx) { return ctx ? ctx->budget_live : 0; }
uint64_t omx_budget_peak(omx_ctx* ctx) { return ctx ? ctx->budget_peak : 0; }
uint64_t omx_budget_limit(omx_ctx* ctx) { return ctx ? ctx->budget_limit : 0; }
uint64_t omx_budget_pooled(omx_ctx* ctx) { return ctx ? ctx->pooled_bytes : 0; }
void omx_budget_reset_peak(omx_ctx* ctx) {
  if (ctx) ctx->budget_peak = ctx->budget_live;
}

int32_t omx_upload(omx_ctx* ctx, void* dst, uint64_t dst_offset, const void* host_src, uint64_t bytes) {
  OMX_REQUIRE_CTX(ctx);
  if (!dst || !host_src) return omx_fail(ctx, OMX_PLACEMENT, "upload: null pointer");
  if (bytes == 0) return OMX_OK;
  // Pageable source: the copy is staged, so the call returns once the source
  // has been read and the caller may reuse it.
  OMX_HIP(ctx, hipMemcpyAsync(static_cast<char*>(dst) + dst_offset, host_src, bytes, hipMemcpyHostToDevice,
                              ctx->stream));
  OMX_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return OMX_OK;
}

int32_t omx_sync(omx_ctx* ctx) {
  OMX_REQUIRE_CTX(ctx);
  OMX_HIP(ctx, hipMemcpyAsync(ctx->fault_host, ctx->fault, sizeof(OmxFaultWord), hipMemcpyDeviceToHost,
                              ctx->stream));
  OMX_HIP(ctx, hipStreamSynchronize(ctx->stream));
  if (ctx->fault_host->mask != 0) {
    uint32_t op = static_cast<uint32_t>(ctx->fault_host->first & 0x7full);
    bool range = (ctx->fault_host->first & 0x80ull) != 0;
    int32_t rc = reset_fault(ctx);
    if (rc != OMX_OK) return rc;
    if (range) return omx_fail(ctx, OMX_OUT_OF_RANGE, "%s: index outside its table", omx_fault_name(op));
    return omx_fail(ctx, OMX_NON_FINITE, "%s", omx_fault_name(op));
  }
  return OMX_OK;
}

int32_t omx_download(omx_ctx* ctx, void* host_dst, const void* src, uint64_t src_offset, uint64_t bytes) {
  OMX_REQUIRE_CTX(ctx);
  if (!host_dst || !src) return omx_fail(ctx, OMX_PLACEMENT, "download: null pointer");
  int32_t rc = omx_sync(ctx);
  if (rc != OMX_OK) return rc;
  if (bytes == 0) return OMX_OK;
  OMX_HIP(ctx, hipMemcpyAsync(host_dst, static_cast<const char*>(src) + src_offset, bytes, hipMemcpyDeviceToHost,
                              ctx->stream));
  OMX_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return OMX_OK;
}

int32_t omx_copy(omx_ctx* ctx, void* dst, const void* src, uint64_t bytes) {
  OMX_REQUIRE_CTX(ctx);
  if (bytes == 0) return OMX_OK;
  OMX_HIP(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
  return OMX_OK;
}

int32_t omx_read_scalar_f32(omx_ctx* ctx, const void* src, float* out) {
  return omx_download(ctx, out, src, 0, sizeof(float));
}

void* omx_stream(omx_ctx* ctx) { return ctx ? static_cast<void*>(ctx->stream) : nullptr; }

int32_t omx_unsupported(omx_ctx* ctx, const char* op) {
  return omx_fail(ctx, OMX_UNSUPPORTED, "%s", op ? op : "unknown op");
}

}  // extern "C"

int32_t omx_workspace(omx_ctx* ctx, uint64_t bytes, void** out, int slot) {
  if (bytes <= ctx->workspace_bytes[slot]) {
    *out = ctx->workspace[slot];
    return OMX_OK;
  }
  if (ctx->workspace[slot]) {
    // An outgrown workspace goes back to the driver, not into the pool: its size (a multiple of
    // 1 MiB that only this slot ever asked for) would match no later request and stay parked.
    auto it = ctx->allocations.find(ctx->workspace[slot]);
    if (it != ctx->allocations.end()) {
      ctx->budget_live -= it->second;
      ctx->allocations.erase(it);
    }
    OMX_HIP(ctx, hipStreamSynchronize(ctx->stream));
    OMX_HIP(ctx, hipFree(ctx->workspace[slot]));
    ctx->workspace[slot] = nullptr;
    ctx->workspace_bytes[slot] = 0;
  }
  uint64_t rounded = (bytes + (1ull << 20) - 1) & ~((1ull << 20) - 1);
  int32_t rc = omx_alloc(ctx, rounded, &ctx->workspace[slot]);
  if (rc != OMX_OK) return rc;
  ctx->workspace_bytes[slot] = rounded;
  *out = ctx->workspace[slot];
  return OMX_OK;
}
