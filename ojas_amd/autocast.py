"""`ojas_core::Autocast<B>` (ojas-core/src/autocast.rs) over `MiBackend`: the reference's bf16 compute
tier as a wrapper around any backend. Inside a region, matmul-class ops round their untagged f32
operands to bf16 (`prep`, :518-525) and their activation outputs (`emit`, :533-538), into rounded
f32 copies that carry the storage compute tag; pointwise ops round their output only when the
operands that gate it are already tagged (`promote`, :540-546); norms, embeddings, the loss and
the optimizers stay f32 (`pass`). Weight gradients stay f32 (`keep_f32`). Outside a region every
call goes straight to the inner backend.

Only the methods the nanolab graph and its trainer call are wrapped; anything else falls through to
the inner backend untouched (the reference wraps the whole trait).
"""
from contextlib import contextmanager

from .backend import F32, DeviceTensor, MiBackend


class Autocast:
    def __init__(self, inner: MiBackend):
        self.inner = inner
        self._depth = 0

    @contextmanager
    def region(self, enabled: bool = True):
        """`autocast_region(AutocastMode::Bf16)` (:626-660); `enabled=False` is `AutocastMode::Off`."""
        self._depth += 1 if enabled else 0
        try:
            yield self
        finally:
            self._depth -= 1 if enabled else 0

    @property
    def on(self) -> bool:
        return self._depth > 0

    def __getattr__(self, name):
        # `pass`: upload, download, zeros, embedding_*, rms_norm_*, rms_qk_norm_*, clip_grad_norm, ...
        return getattr(self.inner, name)

    # ---- the three rules ----
    def _round_new(self, t: DeviceTensor) -> DeviceTensor:
        r = self.inner.cast_bf16(t)
        r.compute_bf16 = True
        return r

    def _prep(self, t: DeviceTensor) -> DeviceTensor:
        if not self.on or t.dtype != F32 or t.compute_bf16:
            return t
        return self._round_new(t)

    def _emit(self, t: DeviceTensor) -> DeviceTensor:
        if not self.on or t.dtype != F32 or t.compute_bf16:
            return t
        return self._round_new(t)

    def _promote(self, tagged: bool, t: DeviceTensor) -> DeviceTensor:
        return self._emit(t) if self.on and tagged else t

    @staticmethod
    def _wrote(t: DeviceTensor):
        t.compute_bf16 = False

    # ---- data movement: carries the tag (:703-707) ----
    def permute(self, x, axes):
        out = self.inner.permute(x, axes)
        out.compute_bf16 = x.compute_bf16
        return out

    # ---- matmul class ----
    def linear_forward(self, x, w, out_dtype=None):
        return self._emit(self.inner.linear_forward(self._prep(x), self._prep(w), out_dtype))

    def linear_backward(self, x, w, gy, *args, **kwargs):
        gx, gw = self.inner.linear_backward(self._prep(x), self._prep(w), self._prep(gy), *args, **kwargs)
        return (self._emit(gx) if gx is not None else None), gw  # the weight gradient stays f32 (:1066-1078)

    def causal_sdpa_forward(self, q, k, v, window=None, out_dtype=None):
        out, lse = self.inner.causal_sdpa_forward(self._prep(q), self._prep(k), self._prep(v), window, out_dtype)
        return self._emit(out), lse  # the log-sum-exp stays f32, unrounded (:1183-1198)

    def causal_sdpa_backward(self, q, k, v, out, lse, gy, window=None, grad_dtype=F32):
        """:1200-1236: an emitted (rounded) output is not used, because the backward's dO . O must
        cancel the softmax row sum; the f32 output is recomputed from the same rounded operands."""
        q, k, v, gy = self._prep(q), self._prep(k), self._prep(v), self._prep(gy)
        if out.compute_bf16:
            grads = self.inner.causal_sdpa_backward_recompute(q, k, v, gy, window, grad_dtype)
        else:
            grads = self.inner.causal_sdpa_backward(q, k, v, out, lse, gy, window, grad_dtype)
        return tuple(self._emit(g) for g in grads)

    def causal_sdpa_backward_recompute(self, q, k, v, gy, window=None, grad_dtype=F32):
        """:1238-1262: the inner backend's own recompute sees the operands the pair above would."""
        grads = self.inner.causal_sdpa_backward_recompute(self._prep(q), self._prep(k), self._prep(v),
                                                          self._prep(gy), window, grad_dtype)
        return tuple(self._emit(g) for g in grads)

    def per_head_sigmoid_gate_forward_saving(self, x, w, b, attn, *args, **kwargs):
        out, scales = self.inner.per_head_sigmoid_gate_forward_saving(self._prep(x), self._prep(w), b,
                                                                      self._prep(attn), *args, **kwargs)
        return self._emit(out), scales

    def per_head_sigmoid_gate_backward_saved(self, x, w, b, attn, gy, scales, *args, **kwargs):
        """:1406-1432: the weight goes in as it is; its gradient and the bias's stay f32."""
        gx, gw, gb, gattn = self.inner.per_head_sigmoid_gate_backward_saved(self._prep(x), w, b, self._prep(attn),
                                                                            self._prep(gy), scales, *args, **kwargs)
        return self._emit(gx), gw, gb, self._emit(gattn)

    def linear_cross_entropy_mean(self, x, w, targets, *args, **kwargs):
        loss, gx, gw = self.inner.linear_cross_entropy_mean(self._prep(x), self._prep(w), targets, *args, **kwargs)
        return loss, (self._emit(gx) if gx is not None else None), gw

    # ---- pointwise: rounded only when the gating operands are tagged ----
    def silu_forward(self, x):
        return self._promote(x.compute_bf16, self.inner.silu_forward(x))

    def silu_backward(self, x, gy):
        return self._promote(x.compute_bf16 and gy.compute_bf16, self.inner.silu_backward(x, gy))

    def mul_forward(self, a, b):
        return self._promote(a.compute_bf16 and b.compute_bf16, self.inner.mul_forward(a, b))

    def mul_backward(self, a, b, gy):
        tagged = a.compute_bf16 and b.compute_bf16 and gy.compute_bf16
        ga, gb = self.inner.mul_backward(a, b, gy)
        return self._promote(tagged, ga), self._promote(tagged, gb)

    def residual_add_forward(self, x, y, *args, **kwargs):
        return self._promote(x.compute_bf16 and y.compute_bf16, self.inner.residual_add_forward(x, y, *args, **kwargs))

    def rope_half_split_forward(self, x, cos, sin):
        return self._promote(x.compute_bf16, self.inner.rope_half_split_forward(x, cos, sin))

    def rope_half_split_backward(self, gy, cos, sin):
        return self._promote(gy.compute_bf16, self.inner.rope_half_split_backward(gy, cos, sin))

    def value_residual_blend_forward(self, value, value0, lam):
        tagged = value.compute_bf16 and value0.compute_bf16 and lam.compute_bf16
        return self._promote(tagged, self.inner.value_residual_blend_forward(value, value0, lam))

    def value_residual_blend_backward(self, value, value0, lam, gy):
        tagged = value.compute_bf16 and value0.compute_bf16 and lam.compute_bf16 and gy.compute_bf16
        return tuple(self._promote(tagged, g) for g in self.inner.value_residual_blend_backward(value, value0, lam, gy))

    # ---- writers: what they write is f32 again (:1009-1027, :1928-1956) ----
    def accumulate_grad(self, acc, grad):
        self.inner.accumulate_grad(acc, grad)
        self._wrote(acc)

    def scale_grad(self, grad, scale):
        self.inner.scale_grad(grad, scale)
        self._wrote(grad)

    def adamw_step(self, param, grad, m1, m2, *args, **kwargs):
        self.inner.adamw_step(param, grad, m1, m2, *args, **kwargs)
        for t in (param, m1, m2):
            self._wrote(t)

    def muon_ns5_step(self, param, grad, momentum, *args, **kwargs):
        self.inner.muon_ns5_step(param, grad, momentum, *args, **kwargs)
        for t in (param, momentum):
            self._wrote(t)
