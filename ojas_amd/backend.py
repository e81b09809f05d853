"""`MiBackend`: the host-side mirror of ojas's `Backend` trait over the C ABI.

The reference's boundary is the Rust trait `ojas_core::Backend`
(ojas-core/src/backend.rs:2634; method list :2655-2767). This module binds
`libojas_mi355x.so` with ctypes and exposes the same method names, argument
meaning and error behaviour for the GPT op set; every other trait method
raises `OjasError(UNSUPPORTED)` (backend.rs:792-797). It holds no arithmetic:
each method validates nothing itself and forwards to one C entry point.

There is no CPU fallback: constructing `MiBackend` without the built library
or without a gfx950 device raises.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path
from typing import Optional, Sequence, Tuple

import numpy as np

from . import shapes

LIB_PATH = Path(__file__).resolve().parent / "libojas_mi355x.so"

F32, BF16, U32 = 0, 1, 2
I8 = 3  # int8 weight codes: a host-side tag only (the entry points that take codes take no dtype for them)
_NP_OF = {F32: np.float32, BF16: np.uint16, U32: np.uint32, I8: np.int8}
_SIZE_OF = {F32: 4, BF16: 2, U32: 4, I8: 1}

(OK, SHAPE, DTYPE, OUT_OF_RANGE, NON_FINITE, UNSUPPORTED_HEAD_DIM, CAPACITY_EXCEEDED, POISONED, DEVICE_LOST,
 WAIT_TIMEOUT, BACKEND, UNSUPPORTED, PLACEMENT) = range(13)
_STATUS_NAMES = ["Ok", "Shape", "Dtype", "OutOfRange", "NonFinite", "UnsupportedHeadDim", "CapacityExceeded",
                 "Poisoned", "DeviceLost", "WaitTimeout", "Backend", "Unsupported", "Placement"]


class OjasError(RuntimeError):
    """One `OjasError` variant (ojas-core/src/error.rs:18-105): `code` + detail text."""

    def __init__(self, code: int, detail: str = ""):
        name = _STATUS_NAMES[code] if 0 <= code < len(_STATUS_NAMES) else str(code)
        super().__init__(f"{name}: {detail}")
        self.code = code
        self.variant = name
        self.detail = detail


class AdamWConfig(C.Structure):
    """ojas_core::AdamWConfig (backend.rs:494-517)."""
    _fields_ = [("lr", C.c_double), ("beta1", C.c_double), ("beta2", C.c_double), ("eps", C.c_double),
                ("weight_decay", C.c_double)]

    @classmethod
    def nanolab(cls, lr: float, weight_decay: float) -> "AdamWConfig":
        return cls(lr, 0.9, 0.95, 1e-8, weight_decay)


class MuonNs5Config(C.Structure):
    """ojas_core::MuonNs5Config (backend.rs:548-570)."""
    _fields_ = [("lr", C.c_double), ("momentum", C.c_double), ("weight_decay", C.c_double), ("nesterov", C.c_int32),
                ("ns5_bf16", C.c_int32)]

    @classmethod
    def nanolab_default(cls) -> "MuonNs5Config":
        return cls(0.025, 0.99, 0.1, 1, 0)


class LowRank(C.Structure):
    """omx_low_rank: the adapter's second product, added in a quantised product's accumulators."""
    _fields_ = [("h", C.c_void_p), ("w", C.c_void_p), ("h_pitch", C.c_uint64), ("w_pitch", C.c_uint64),
                ("rank", C.c_uint64), ("block_cols", C.c_uint64)]


def load_library() -> C.CDLL:
    if not LIB_PATH.exists():
        raise OjasError(BACKEND, f"{LIB_PATH} is not built; run __graft_entry__.build()")
    lib = C.CDLL(str(LIB_PATH))
    lib.omx_last_error.restype = C.c_size_t
    lib.omx_device_name.restype = C.c_size_t
    for name in ("omx_budget_live", "omx_budget_peak", "omx_budget_limit", "omx_budget_pooled", "omx_muon_scratch_bytes"):
        if hasattr(lib, name):
            getattr(lib, name).restype = C.c_uint64
    lib.omx_stream.restype = C.c_void_p
    return lib


class DeviceTensor:
    """A contiguous device tensor: pointer, shape, dtype. Frees itself on drop
    (the role of `Arc<dyn DeviceBuffer>` + `Reservation`, tensor.rs:146-163)."""

    def __init__(self, backend: "MiBackend", ptr: int, shape: Tuple[int, ...], dtype: int, owns: bool = True):
        self.backend, self.ptr, self.shape, self.dtype, self._owns = backend, ptr, tuple(shape), dtype, owns
        # The storage compute tag of an f32 tensor (tensor.rs COMPUTE_BF16): True when its values are
        # known to be bf16-exact, so a second rounding would only clone. Set by `Autocast`.
        self.compute_bf16 = False

    @property
    def numel(self) -> int:
        return int(np.prod(self.shape)) if self.shape else 1

    @property
    def nbytes(self) -> int:
        return self.numel * _SIZE_OF[self.dtype]

    def reshape(self, *shape) -> "DeviceTensor":
        """Zero-copy view (tensor.rs:1555-1605); the view does not own the memory."""
        shape = tuple(shape[0]) if len(shape) == 1 and isinstance(shape[0], (tuple, list)) else tuple(shape)
        if int(np.prod(shape)) != self.numel:
            raise OjasError(SHAPE, f"reshape {self.shape} -> {shape}")
        view = DeviceTensor(self.backend, self.ptr, shape, self.dtype, owns=False)
        view._base = self
        view.compute_bf16 = self.compute_bf16
        return view

    def __del__(self):
        if getattr(self, "_owns", False) and self.ptr and self.backend is not None and self.backend._ctx:
            self.backend._lib.omx_free(self.backend._ctx, C.c_void_p(self.ptr))
            self.ptr = 0


class MiBackend:
    """`impl Backend for MiBackend`: BackendId::Hip, Numerics::Fast, bf16 operands accepted."""

    id = "hip"
    numerics = "fast"
    bf16_operands = True

    def __init__(self, device: int = 0, budget_bytes: int = 0):
        self._lib = load_library()
        ctx = C.c_void_p()
        rc = self._lib.omx_open(C.c_int32(device), C.c_uint64(budget_bytes), C.byref(ctx))
        self._ctx = ctx if rc == OK else None
        if rc != OK:
            raise OjasError(rc, "omx_open failed (no gfx950 device or runtime error)")

    def close(self):
        if self._ctx:
            self._lib.omx_close(self._ctx)
            self._ctx = None

    # ---- plumbing ----
    def _check(self, rc: int):
        if rc != OK:
            buf = C.create_string_buffer(512)
            self._lib.omx_last_error(self._ctx, buf, C.c_size_t(512))
            raise OjasError(rc, buf.value.decode("utf-8", "replace"))

    def device_name(self) -> str:
        buf = C.create_string_buffer(128)
        self._lib.omx_device_name(self._ctx, buf, C.c_size_t(128))
        return buf.value.decode()

    def stream(self) -> int:
        return int(self._lib.omx_stream(self._ctx) or 0)

    def budget(self):
        return {"live": int(self._lib.omx_budget_live(self._ctx)), "peak": int(self._lib.omx_budget_peak(self._ctx)),
                "limit": int(self._lib.omx_budget_limit(self._ctx)),
                "pooled": int(self._lib.omx_budget_pooled(self._ctx))}

    def empty(self, shape, dtype: int = F32) -> DeviceTensor:
        shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        n = int(np.prod(shape)) if shape else 1
        ptr = C.c_void_p()
        self._check(self._lib.omx_alloc(self._ctx, C.c_uint64(max(n, 1) * _SIZE_OF[dtype]), C.byref(ptr)))
        return DeviceTensor(self, ptr.value, shape, dtype)

    def zeros(self, shape, dtype: int = F32) -> DeviceTensor:
        t = self.empty(shape, dtype)
        self._check(self._lib.omx_fill_zero(self._ctx, C.c_void_p(t.ptr), C.c_uint64(t.nbytes)))
        return t

    def upload(self, host: np.ndarray, dtype: Optional[int] = None) -> DeviceTensor:
        """BackendCore::upload (backend.rs:917-936). float32 -> F32, uint32 -> U32,
        uint16 -> BF16 bits; `dtype=BF16` on a float32 array rounds on the device."""
        host = np.ascontiguousarray(host)
        if host.dtype == np.float32:
            src_dtype = F32
        elif host.dtype == np.uint32:
            src_dtype = U32
        elif host.dtype == np.uint16:
            src_dtype = BF16
        elif host.dtype == np.int8:
            src_dtype = I8
        else:
            raise OjasError(DTYPE, f"upload of {host.dtype}")
        t = self.empty(host.shape, src_dtype)
        if host.size:
            self._check(self._lib.omx_upload(self._ctx, C.c_void_p(t.ptr), C.c_uint64(0),
                                             host.ctypes.data_as(C.c_void_p), C.c_uint64(host.nbytes)))
        if dtype is not None and dtype != src_dtype:
            if src_dtype == F32 and dtype == BF16:
                return self.to_bf16(t)
            raise OjasError(DTYPE, "upload conversion")
        return t

    def download(self, t: DeviceTensor) -> np.ndarray:
        """BackendCore::download (backend.rs:938-961): syncs, reports deferred faults."""
        out = np.empty(t.shape, dtype=_NP_OF[t.dtype])
        self._check(self._lib.omx_download(self._ctx, out.ctypes.data_as(C.c_void_p), C.c_void_p(t.ptr),
                                           C.c_uint64(0), C.c_uint64(t.nbytes)))
        return out

    def download_f32(self, t: DeviceTensor) -> np.ndarray:
        """Downloads and widens bf16 storage exactly (bits << 16)."""
        a = self.download(t)
        if t.dtype == BF16:
            return (a.astype(np.uint32) << 16).view(np.float32)
        return a

    def set_option(self, name: str, value: int):
        """Tuning knobs of the library (`omx_set_option`); no counterpart in the reference."""
        self._check(self._lib.omx_set_option(self._ctx, name.encode(), C.c_int64(value)))

    def sync(self):
        """BackendCore::sync (backend.rs:963-973)."""
        self._check(self._lib.omx_sync(self._ctx))

    def _p(self, t: Optional[DeviceTensor]):
        return C.c_void_p(t.ptr) if t is not None else C.c_void_p(None)

    # ---- casts ----
    def cast_bf16(self, x: DeviceTensor) -> DeviceTensor:
        y = self.empty(x.shape, F32)
        self._check(self._lib.omx_cast_bf16(self._ctx, self._p(x), self._p(y), C.c_uint64(x.numel)))
        return y

    def to_bf16(self, x: DeviceTensor) -> DeviceTensor:
        y = self.empty(x.shape, BF16)
        self._check(self._lib.omx_to_bf16(self._ctx, self._p(x), self._p(y), C.c_uint64(x.numel)))
        return y

    def to_f32(self, x: DeviceTensor) -> DeviceTensor:
        y = self.empty(x.shape, F32)
        self._check(self._lib.omx_to_f32(self._ctx, self._p(x), self._p(y), C.c_uint64(x.numel)))
        return y

    # ---- matmul class ----
    def linear_forward(self, x: DeviceTensor, w: DeviceTensor, out_dtype: Optional[int] = None) -> DeviceTensor:
        rows = x.numel // x.shape[-1]
        kin, nout = x.shape[-1], w.shape[0]
        if w.shape[-1] != kin or len(w.shape) != 2:
            raise OjasError(SHAPE, f"linear_forward: input {x.shape} weight {w.shape}")
        od = F32 if out_dtype is None else out_dtype
        y = self.empty(x.shape[:-1] + (nout,), od)
        self._check(self._lib.omx_linear_forward(self._ctx, self._p(x), C.c_int32(x.dtype), self._p(w),
                                                 C.c_int32(w.dtype), self._p(y), C.c_int32(od), C.c_uint64(rows),
                                                 C.c_uint64(kin), C.c_uint64(nout)))
        return y

    def linear_backward(self, x, w, gy, gx_dtype=F32, need_gx=True, need_gw=True):
        rows = x.numel // x.shape[-1]
        kin, nout = x.shape[-1], w.shape[0]
        if not (x.dtype == w.dtype == gy.dtype):
            raise OjasError(DTYPE, "linear_backward: operands must share a dtype")
        gx = self.empty(x.shape, gx_dtype) if need_gx else None
        gw = self.empty(w.shape, F32) if need_gw else None
        self._check(self._lib.omx_linear_backward(self._ctx, self._p(x), self._p(w), self._p(gy), C.c_int32(x.dtype),
                                                  self._p(gx), C.c_int32(gx_dtype), self._p(gw), C.c_int32(F32),
                                                  C.c_uint64(rows), C.c_uint64(kin), C.c_uint64(nout)))
        return gx, gw

    def linear_backward_input(self, w, gy, in_features=None, gx_dtype=F32):
        rows = gy.numel // gy.shape[-1]
        kin, nout = w.shape[1], w.shape[0]
        gx = self.empty(gy.shape[:-1] + (kin,), gx_dtype)
        self._check(self._lib.omx_linear_backward(self._ctx, None, self._p(w), self._p(gy), C.c_int32(w.dtype),
                                                  self._p(gx), C.c_int32(gx_dtype), None, C.c_int32(F32),
                                                  C.c_uint64(rows), C.c_uint64(kin), C.c_uint64(nout)))
        return gx

    def rope_half_split_inplace(self, x, cos, sin, tokens, time, heads, dim, backward=False):
        """The rotary embedding applied in place to the first heads * dim columns of bf16 x [tokens, pitch]."""
        self._check(self._lib.omx_rope_half_split_inplace(
            self._ctx, self._p(x), C.c_int32(x.dtype), C.c_uint64(x.shape[-1]), self._p(cos), self._p(sin),
            C.c_uint64(tokens), C.c_uint64(time), C.c_uint64(heads), C.c_uint64(dim), C.c_int32(1 if backward else 0)))
        return x

    def rope_half_split_pitched(self, x, cos, sin, tokens, time, heads, plain_heads, dim):
        """The rotation out of place: x [tokens, pitch] f32 or bf16 -> bf16, `heads` rotated heads then
        `plain_heads` converted as they are (`omx_rope_half_split_pitched`)."""
        out = self.empty(x.shape, BF16)
        self._check(self._lib.omx_rope_half_split_pitched(
            self._ctx, self._p(x), C.c_int32(x.dtype), self._p(out), C.c_uint64(x.shape[-1]), self._p(cos), self._p(sin),
            C.c_uint64(tokens), C.c_uint64(time), C.c_uint64(heads), C.c_uint64(plain_heads), C.c_uint64(dim)))
        return out

    def swiglu_forward(self, gate_up):
        rows, two_h = gate_up.shape
        out = self.empty((rows, two_h // 2), BF16)
        self._check(self._lib.omx_swiglu_forward(self._ctx, self._p(gate_up), self._p(out), C.c_int32(gate_up.dtype),
                                                 C.c_uint64(rows), C.c_uint64(two_h // 2)))
        return out

    def swiglu_backward(self, gate_up, gy):
        rows, two_h = gate_up.shape
        g = self.empty(gate_up.shape, BF16)
        self._check(self._lib.omx_swiglu_backward(self._ctx, self._p(gate_up), self._p(gy), self._p(g),
                                                  C.c_int32(gate_up.dtype), C.c_uint64(rows), C.c_uint64(two_h // 2)))
        return g

    def pack_i8_group(self, codes, scales, group=32):
        """Row-major codes and scales -> the blocked layout (`omx_pack_i8_group`); same shapes."""
        nout, kin = codes.shape
        bc, bs = self.empty(codes.shape, I8), self.empty(scales.shape, F32)
        self._check(self._lib.omx_pack_i8_group(self._ctx, self._p(codes), self._p(scales), self._p(bc), self._p(bs),
                                                C.c_uint64(nout), C.c_uint64(kin), C.c_uint64(group), C.c_int32(0)))
        return bc, bs

    def unpack_i8_group(self, blocked_codes, blocked_scales, group=32):
        nout, kin = blocked_codes.shape
        c, s = self.empty(blocked_codes.shape, I8), self.empty(blocked_scales.shape, F32)
        self._check(self._lib.omx_pack_i8_group(self._ctx, self._p(c), self._p(s), self._p(blocked_codes),
                                                self._p(blocked_scales), C.c_uint64(nout), C.c_uint64(kin),
                                                C.c_uint64(group), C.c_int32(1)))
        return c, s

    @staticmethod
    def _low_rank(low_rank):
        """(h [rows, pitch] bf16, w [cols, rank] bf16, block_cols) -> a pointer to omx_low_rank, or None."""
        if low_rank is None:
            return None
        h, w, block_cols = low_rank
        return C.byref(LowRank(h.ptr, w.ptr, h.shape[-1], w.shape[-1], w.shape[-1], block_cols))

    def linear_i8_group_forward(self, x, codes, scales, add=None, group=32, blocked=False, low_rank=None,
                                out_dtype=BF16):
        """y = x W^T (+ add) for a frozen weight held as int8 codes [out, in] and f32 group scales
        [out, in / group] (value = code * scale); bf16 in, bf16 (or f32) out."""
        rows, kin, nout = x.numel // x.shape[-1], x.shape[-1], codes.shape[0]
        if codes.shape != (nout, kin) or scales.shape != (nout, kin // group) or codes.dtype != I8 or scales.dtype != F32:
            raise OjasError(SHAPE, f"linear_i8_group_forward: input {x.shape} codes {codes.shape} scales {scales.shape}")
        y = self.empty(x.shape[:-1] + (nout,), out_dtype)
        self._check(self._lib.omx_linear_i8_group_forward(
            self._ctx, self._p(x), C.c_int32(x.dtype), self._p(codes), self._p(scales), C.c_uint64(group),
            C.c_int32(1 if blocked else 0), self._p(add), self._low_rank(low_rank), self._p(y), C.c_int32(out_dtype),
            C.c_uint64(rows), C.c_uint64(kin), C.c_uint64(nout)))
        return y

    def linear_i8_group_backward_input(self, codes, scales, gy, add=None, group=32, blocked=False, low_rank=None):
        """gx = gy W (+ add) for the same weight form; there is no weight gradient (the base is frozen)."""
        nout, kin = codes.shape
        rows = gy.numel // gy.shape[-1]
        if gy.shape[-1] != nout or scales.shape != (nout, kin // group) or codes.dtype != I8 or scales.dtype != F32:
            raise OjasError(SHAPE, f"linear_i8_group_backward_input: gy {gy.shape} codes {codes.shape}")
        gx = self.empty(gy.shape[:-1] + (kin,), BF16)
        self._check(self._lib.omx_linear_i8_group_backward_input(
            self._ctx, self._p(codes), self._p(scales), C.c_uint64(group), C.c_int32(1 if blocked else 0), self._p(gy),
            C.c_int32(gy.dtype), self._p(add), self._low_rank(low_rank), self._p(gx), C.c_uint64(rows), C.c_uint64(kin), C.c_uint64(nout)))
        return gx

    def gemm(self, a: DeviceTensor, a_strides, b: DeviceTensor, b_strides, m, k, n, out_dtype=F32, c=None):
        """C[m,n] (+)= A.B with element strides (a_rs, a_cs), (b_rs, b_cs)."""
        acc = c is not None
        out = c if acc else self.empty((m, n), out_dtype)
        self._check(self._lib.omx_gemm(self._ctx, self._p(a), C.c_uint64(a_strides[0]), C.c_uint64(a_strides[1]),
                                       self._p(b), C.c_uint64(b_strides[0]), C.c_uint64(b_strides[1]),
                                       C.c_int32(a.dtype), self._p(out), C.c_int32(out.dtype), C.c_uint64(m),
                                       C.c_uint64(k), C.c_uint64(n), C.c_int32(1 if acc else 0)))
        return out

    def gemm_strided_batch(self, a: DeviceTensor, a_strides, b: DeviceTensor, b_strides, m, k, n, count,
                           batch_strides, out_dtype=F32):
        """`count` products of `gemm`'s form in one launch; `batch_strides` = element strides between
        consecutive products' A, B and C. Returns C [count, m, n] when the C stride is m * n."""
        sa, sb, sc = batch_strides
        if sc < m * n:
            raise OjasError(SHAPE, "gemm_strided_batch: outputs overlap")
        out = self.empty(((count - 1) * sc + m * n,), out_dtype)
        self._check(self._lib.omx_gemm_strided_batch(
            self._ctx, self._p(a), C.c_uint64(a_strides[0]), C.c_uint64(a_strides[1]), self._p(b),
            C.c_uint64(b_strides[0]), C.c_uint64(b_strides[1]), C.c_int32(a.dtype), self._p(out), C.c_int32(out_dtype),
            C.c_uint64(m), C.c_uint64(k), C.c_uint64(n), C.c_int32(0), C.c_uint64(count), C.c_uint64(sa),
            C.c_uint64(sb), C.c_uint64(sc)))
        return out

    def gemm_pitched_strided_batch(self, a: DeviceTensor, a_strides, b: DeviceTensor, b_strides, c: DeviceTensor, ldc,
                                   m, k, n, count, batch_strides):
        """`gemm_strided_batch` into column blocks of `c`, whose rows are `ldc` elements apart
        (`omx_gemm_pitched_strided_batch`); writes `c` in place."""
        sa, sb, sc = batch_strides
        self._check(self._lib.omx_gemm_pitched_strided_batch(
            self._ctx, self._p(a), C.c_uint64(a_strides[0]), C.c_uint64(a_strides[1]), self._p(b),
            C.c_uint64(b_strides[0]), C.c_uint64(b_strides[1]), C.c_int32(a.dtype), self._p(c), C.c_int32(c.dtype),
            C.c_uint64(ldc), C.c_uint64(m), C.c_uint64(k), C.c_uint64(n), C.c_int32(0), C.c_uint64(count),
            C.c_uint64(sa), C.c_uint64(sb), C.c_uint64(sc)))

    # ---- attention ----
    def causal_sdpa_forward(self, q, k, v, window: Optional[int] = None, out_dtype: Optional[int] = None):
        b, h, t, d = q.shape
        hkv = k.shape[1]
        if window == 0:
            raise OjasError(SHAPE, "sdpa window must be at least 1")
        od = F32 if out_dtype is None else out_dtype
        out = self.empty(q.shape, od)
        lse = self.empty((b, h, t), F32)
        self._check(self._lib.omx_causal_sdpa_forward(self._ctx, self._p(q), self._p(k), self._p(v),
                                                      C.c_int32(q.dtype), self._p(out), C.c_int32(od), self._p(lse),
                                                      C.c_uint64(b), C.c_uint64(h), C.c_uint64(hkv), C.c_uint64(t),
                                                      C.c_uint64(d), C.c_uint64(window or 0)))
        return out, lse

    def causal_sdpa_backward(self, q, k, v, out, lse, gy, window: Optional[int] = None, grad_dtype=F32):
        """`out` and `gy` are read in their own storage dtypes (f32 or bf16)."""
        b, h, t, d = q.shape
        hkv = k.shape[1]
        if window == 0:
            raise OjasError(SHAPE, "sdpa window must be at least 1")
        if not (q.dtype == k.dtype == v.dtype):
            raise OjasError(DTYPE, "causal_sdpa_backward: q, k, v must share a dtype")
        if out.shape != q.shape or gy.shape != q.shape or lse.dtype != F32:
            raise OjasError(SHAPE, f"causal_sdpa_backward: out {out.shape} / grad_output {gy.shape} against q {q.shape}")
        gq, gk, gv = self.empty(q.shape, grad_dtype), self.empty(k.shape, grad_dtype), self.empty(v.shape, grad_dtype)
        self._check(self._lib.omx_causal_sdpa_backward(self._ctx, self._p(q), self._p(k), self._p(v), self._p(out),
                                                       self._p(lse), self._p(gy), C.c_int32(q.dtype),
                                                       C.c_int32(out.dtype), C.c_int32(gy.dtype), self._p(gq),
                                                       self._p(gk), self._p(gv), C.c_int32(grad_dtype), C.c_uint64(b),
                                                       C.c_uint64(h), C.c_uint64(hkv), C.c_uint64(t), C.c_uint64(d),
                                                       C.c_uint64(window or 0)))
        return gq, gk, gv

    def causal_sdpa_backward_recompute(self, q, k, v, gy, window: Optional[int] = None, grad_dtype=F32):
        """BackendModule::causal_sdpa_backward_recompute (backend.rs:1781-1792), one call."""
        b, h, t, d = q.shape
        hkv = k.shape[1]
        if window == 0:
            raise OjasError(SHAPE, "sdpa window must be at least 1")
        if gy.shape != q.shape:
            raise OjasError(SHAPE, f"causal_sdpa_backward_recompute: grad_output {gy.shape} against q {q.shape}")
        gq, gk, gv = self.empty(q.shape, grad_dtype), self.empty(k.shape, grad_dtype), self.empty(v.shape, grad_dtype)
        self._check(self._lib.omx_causal_sdpa_backward_recompute(
            self._ctx, self._p(q), self._p(k), self._p(v), self._p(gy), C.c_int32(q.dtype), C.c_int32(gy.dtype),
            self._p(gq), self._p(gk), self._p(gv), C.c_int32(grad_dtype), C.c_uint64(b), C.c_uint64(h),
            C.c_uint64(hkv), C.c_uint64(t), C.c_uint64(d), C.c_uint64(window or 0)))
        return gq, gk, gv

    def linear_gelu_forward(self, x, w, tanh_form: bool = False):
        """`linear_forward` then `gelu_*_forward` in one kernel (bf16): returns (u, gelu(u))."""
        rows, nout = x.numel // x.shape[-1], w.shape[0]
        u, act = self.empty(x.shape[:-1] + (nout,), BF16), self.empty(x.shape[:-1] + (nout,), BF16)
        self._check(self._lib.omx_linear_gelu_forward(
            self._ctx, self._p(x), self._p(w), C.c_int32(x.dtype), self._p(u), self._p(act), C.c_uint64(rows),
            C.c_uint64(x.shape[-1]), C.c_uint64(nout), C.c_int32(1 if tanh_form else 0)))
        return u, act

    def linear_backward_input_gelu(self, w, gy, u, tanh_form: bool = False):
        """grad_input of `linear_backward(w, gy)` times gelu'(u) in one kernel (bf16)."""
        nout, nin = w.shape
        rows = gy.numel // nout
        if gy.shape[-1] != nout or u.numel != rows * nin or not (w.dtype == gy.dtype == u.dtype == BF16):
            raise BackendError(OMX_SHAPE, f"linear_backward_input_gelu: w {w.shape}, gy {gy.shape}, u {u.shape}")
        gu = self.empty(u.shape, BF16)
        self._check(self._lib.omx_linear_backward_input_gelu(
            self._ctx, self._p(w), self._p(gy), C.c_int32(gy.dtype), self._p(u), self._p(gu), C.c_uint64(rows),
            C.c_uint64(nin), C.c_uint64(nout), C.c_int32(1 if tanh_form else 0)))
        return gu

    def causal_attention_forward(self, q, k, v, window: Optional[int] = None, pitches=None, saving: bool = False):
        """`causal_attention` (ojas-model/src/block.rs:186-199) over time-major [B, T, heads, D]
        tensors. `pitches` = (q, kv) token-row pitches in elements when q / k / v are column
        blocks of a wider buffer; the output is contiguous. `saving=True` also returns the output's
        rounding residual (what the reference's f32 saved output keeps, autocast.rs:177-186) for
        `causal_attention_backward(..., residual=)`."""
        b, t, h, d = q.shape
        hkv = k.shape[2]
        qp, kvp = pitches if pitches else (h * d, hkv * d)
        out = self.empty((b, t, h, d), BF16)
        lse = self.empty((b, h, t), F32)
        tail = (C.c_uint64(h * d), C.c_int32(BF16), self._p(lse), C.c_uint64(b), C.c_uint64(t), C.c_uint64(h),
                C.c_uint64(hkv), C.c_uint64(d), C.c_uint64(window or 0))
        head = (self._ctx, self._p(q), C.c_uint64(qp), self._p(k), self._p(v), C.c_uint64(kvp), C.c_int32(q.dtype),
                self._p(out))
        if saving:
            residual = self.empty((b, t, h, d), BF16)
            self._check(self._lib.omx_causal_attention_forward_saving(*head, self._p(residual), *tail))
            return out, lse, residual
        self._check(self._lib.omx_causal_attention_forward(*head, *tail))
        return out, lse

    def causal_attention_backward(self, q, k, v, out, lse, gy, window: Optional[int] = None, pitches=None,
                                  grads=None, residual=None):
        """Backward of `causal_attention_forward`. `grads` = (gq, gk, gv) tensors to write (they use
        the operands' pitches); by default contiguous ones are allocated. `residual`: the third
        value of the saving forward."""
        b, t, h, d = q.shape
        hkv = k.shape[2]
        qp, kvp = pitches if pitches else (h * d, hkv * d)
        if grads is None:
            if pitches:
                raise OjasError(SHAPE, "causal_attention_backward: pass `grads` with pitched operands")
            grads = (self.empty(q.shape, BF16), self.empty(k.shape, BF16), self.empty(v.shape, BF16))
        gq, gk, gv = grads
        head = (self._ctx, self._p(q), C.c_uint64(qp), self._p(k), self._p(v), C.c_uint64(kvp), self._p(out))
        tail = (self._p(gy), C.c_uint64(h * d), self._p(lse), C.c_int32(q.dtype), self._p(gq), self._p(gk), self._p(gv),
                C.c_int32(BF16), C.c_uint64(b), C.c_uint64(t), C.c_uint64(h), C.c_uint64(hkv), C.c_uint64(d),
                C.c_uint64(window or 0))
        if residual is not None:
            if residual.shape != out.shape or residual.dtype != BF16:
                raise OjasError(SHAPE, "causal_attention_backward: residual must match the output")
            self._check(self._lib.omx_causal_attention_backward_saved(*head, self._p(residual), *tail))
        else:
            self._check(self._lib.omx_causal_attention_backward(*head, *tail))
        return gq, gk, gv

    # ---- norms ----
    def rms_norm_forward(self, x, w, eps: float = 1e-6, out_dtype: Optional[int] = None):
        dim = x.shape[-1]
        rows = x.numel // dim
        if w.shape != (dim,):
            raise OjasError(SHAPE, f"rms_norm_forward: weight {w.shape} for dim {dim}")
        od = x.dtype if out_dtype is None else out_dtype
        y = self.empty(x.shape, od)
        self._check(self._lib.omx_rms_norm_forward(self._ctx, self._p(x), C.c_int32(x.dtype), self._p(w), self._p(y),
                                                   C.c_int32(od), C.c_uint64(rows), C.c_uint64(dim), C.c_float(eps)))
        return y

    def rms_norm_backward(self, x, w, gy, eps: float = 1e-6):
        dim = x.shape[-1]
        rows = x.numel // dim
        gx = self.empty(x.shape, gy.dtype)
        gw = self.empty((dim,), F32)
        self._check(self._lib.omx_rms_norm_backward(self._ctx, self._p(x), C.c_int32(x.dtype), self._p(w),
                                                    self._p(gy), C.c_int32(gy.dtype), self._p(gx),
                                                    C.c_int32(gy.dtype), self._p(gw), C.c_uint64(rows),
                                                    C.c_uint64(dim), C.c_float(eps)))
        return gx, gw

    def residual_add_rms_norm_forward(self, x, y, w, eps: float = 1e-6, out_dtype: Optional[int] = None):
        """`residual_add_forward` then `rms_norm_forward` in one pass: returns (sum f32, normed)."""
        dim = x.shape[-1]
        od = y.dtype if out_dtype is None else out_dtype
        total, normed = self.empty(x.shape, F32), self.empty(x.shape, od)
        self._check(self._lib.omx_residual_add_rms_norm_forward(
            self._ctx, self._p(x), C.c_int32(x.dtype), self._p(y), C.c_int32(y.dtype), self._p(w), self._p(total),
            self._p(normed), C.c_int32(od), C.c_uint64(x.numel // dim), C.c_uint64(dim), C.c_float(eps)))
        return total, normed

    def rms_norm_backward_residual(self, x, w, gy, residual_grad, eps: float = 1e-6, want_bf16: bool = False,
                                   want_weight_grad: bool = True):
        """`rms_norm_backward` whose input gradient is added to `residual_grad` (f32):
        returns (gx f32, gx bf16 or None, gw; gw is None and not formed with `want_weight_grad=False`,
        for a frozen weight)."""
        dim = x.shape[-1]
        gx, gw = self.empty(x.shape, F32), (self.empty((dim,), F32) if want_weight_grad else None)
        gx16 = self.empty(x.shape, BF16) if want_bf16 else None
        self._check(self._lib.omx_rms_norm_backward_residual(
            self._ctx, self._p(x), C.c_int32(x.dtype), self._p(w), self._p(gy), C.c_int32(gy.dtype),
            self._p(residual_grad), self._p(gx), self._p(gx16), self._p(gw), C.c_uint64(x.numel // dim),
            C.c_uint64(dim), C.c_float(eps)))
        return gx, gx16, gw

    # ---- loss ----
    @staticmethod
    def _ign(ignore_index):
        return (C.c_int32(0), C.c_uint32(0)) if ignore_index is None else (C.c_int32(1), C.c_uint32(ignore_index))

    def cross_entropy_mean_forward(self, logits, targets, ignore_index=None):
        rows, vocab = logits.shape
        loss = self.empty((1,), F32)
        hi, iv = self._ign(ignore_index)
        self._check(self._lib.omx_cross_entropy_mean_forward(self._ctx, self._p(logits), C.c_int32(logits.dtype),
                                                             self._p(targets), C.c_uint64(rows), C.c_uint64(vocab),
                                                             hi, iv, self._p(loss)))
        return loss

    def cross_entropy_mean_forward_static(self, logits, targets, loss, ignore_index=None):
        """`cross_entropy_mean_forward` into a caller-allocated `loss`, through the entry point that
        allocates nothing (row state in a file-scope device array; at most 65536 rows)."""
        rows, vocab = logits.shape
        hi, iv = self._ign(ignore_index)
        self._check(self._lib.omx_cross_entropy_mean_forward_static(
            self._ctx, self._p(logits), C.c_int32(logits.dtype), self._p(targets), C.c_uint64(rows),
            C.c_uint64(vocab), hi, iv, self._p(loss)))
        return loss

    def cross_entropy_mean_backward(self, logits, targets, ignore_index=None, grad_dtype=F32):
        rows, vocab = logits.shape
        grad = self.empty(logits.shape, grad_dtype)
        hi, iv = self._ign(ignore_index)
        self._check(self._lib.omx_cross_entropy_mean_backward(self._ctx, self._p(logits), C.c_int32(logits.dtype),
                                                              self._p(targets), C.c_uint64(rows), C.c_uint64(vocab),
                                                              hi, iv, self._p(grad), C.c_int32(grad_dtype)))
        return grad

    def linear_cross_entropy_mean(self, x, w, targets, ignore_index=None, chunk=(1024, 8192), grads=(True, True),
                                  gx_dtype=F32):
        """Returns (loss, grad_input | None, grad_weight | None); `chunk` is CeChunk(rows, cols)."""
        rows, dim = x.shape
        vocab = w.shape[0]
        if x.dtype != w.dtype:
            raise OjasError(DTYPE, "linear_cross_entropy_mean: operands must share a dtype")
        loss = self.empty((1,), F32)
        gx = self.empty(x.shape, gx_dtype) if grads[0] else None
        gw = self.empty(w.shape, F32) if grads[1] else None
        hi, iv = self._ign(ignore_index)
        self._check(self._lib.omx_linear_cross_entropy_mean(
            self._ctx, self._p(x), self._p(w), C.c_int32(x.dtype), self._p(targets), C.c_uint64(rows),
            C.c_uint64(dim), C.c_uint64(vocab), hi, iv, C.c_uint64(chunk[0]), C.c_uint64(chunk[1]), self._p(loss),
            self._p(gx), C.c_int32(gx_dtype), self._p(gw)))
        return loss, gx, gw

    # ---- embedding ----
    def embedding_forward(self, table, ids, out_dtype: Optional[int] = None):
        vocab, dim = table.shape
        od = F32 if out_dtype is None else out_dtype
        out = self.empty(ids.shape + (dim,), od)
        self._check(self._lib.omx_embedding_forward(self._ctx, self._p(table), C.c_int32(table.dtype), self._p(ids),
                                                    self._p(out), C.c_int32(od), C.c_uint64(ids.numel),
                                                    C.c_uint64(vocab), C.c_uint64(dim)))
        return out

    def embedding_backward(self, ids, grad, vocab: int):
        dim = grad.shape[-1]
        out = self.empty((vocab, dim), F32)
        self._check(self._lib.omx_embedding_backward(self._ctx, self._p(ids), self._p(grad), C.c_int32(grad.dtype),
                                                     self._p(out), C.c_uint64(ids.numel), C.c_uint64(vocab),
                                                     C.c_uint64(dim)))
        return out

    def embedding_backward_accumulate(self, ids, grad, table_grad):
        """`embedding_backward` then `accumulate_grad` onto `table_grad` (f32 [vocab, dim]) in one
        pass over the rows the ids name (`omx_embedding_backward_accumulate`)."""
        vocab, dim = table_grad.shape
        if table_grad.dtype != F32 or grad.shape[-1] != dim:
            raise OjasError(SHAPE, f"embedding_backward_accumulate: grad {grad.shape} against table_grad {table_grad.shape}")
        self._check(self._lib.omx_embedding_backward_accumulate(
            self._ctx, self._p(ids), self._p(grad), C.c_int32(grad.dtype), self._p(table_grad), C.c_uint64(ids.numel),
            C.c_uint64(vocab), C.c_uint64(dim)))

    # ---- optimizers (in place) ----
    def adamw_step(self, param, grad, moment1, moment2, step: int, config: AdamWConfig, param_bf16=None):
        self._check(self._lib.omx_adamw_step(self._ctx, self._p(param), self._p(grad), self._p(moment1),
                                             self._p(moment2), C.c_uint64(param.numel), C.c_uint64(step),
                                             C.byref(config), self._p(param_bf16)))

    def adamw_step_bounded(self, param, grad, moment1, moment2, step: int, config: AdamWConfig, inputs_bounded: bool,
                           unbounded_flag: DeviceTensor, param_bf16=None):
        """`adamw_step` for a caller that tracks its tensors between calls: with `inputs_bounded`
        (every input below 2^60 in magnitude) the checking pass is skipped; `unbounded_flag` (one
        u32) is OR-ed with 1 when a stored parameter or moment reaches 2^60."""
        self._check(self._lib.omx_adamw_step_bounded(
            self._ctx, self._p(param), self._p(grad), self._p(moment1), self._p(moment2), C.c_uint64(param.numel),
            C.c_uint64(step), C.byref(config), self._p(param_bf16), C.c_int32(1 if inputs_bounded else 0),
            self._p(unbounded_flag)))

    def muon_ns5_step(self, param, grad, momentum, config: MuonNs5Config, param_bf16=None):
        rows, cols = param.shape
        self._check(self._lib.omx_muon_ns5_step(self._ctx, self._p(param), self._p(grad), self._p(momentum),
                                                C.c_uint64(rows), C.c_uint64(cols), C.byref(config),
                                                self._p(param_bf16)))

    def muon_ns5_step_batched(self, params, grads, momenta, config: MuonNs5Config, params_bf16=None):
        """`muon_ns5_step` on several tensors of one shape in one set of launches (in place)."""
        n = len(params)
        rows, cols = params[0].shape
        if any(p.shape != (rows, cols) for p in params) or len(grads) != n or len(momenta) != n:
            raise OjasError(SHAPE, "muon_ns5_step_batched: tensors of one shape, one gradient and momentum each")
        table = lambda ts: (C.c_void_p * n)(*[t.ptr for t in ts])
        mirrors = (C.c_void_p * n)(*[(t.ptr if t is not None else None) for t in params_bf16]) if params_bf16 else None
        self._check(self._lib.omx_muon_ns5_step_batched(self._ctx, table(params), table(grads), table(momenta), mirrors,
                                                        C.c_uint64(n), C.c_uint64(rows), C.c_uint64(cols),
                                                        C.byref(config)))

    def clip_grad_norm(self, grads: Sequence[DeviceTensor], max_norm: float) -> float:
        n = len(grads)
        ptrs = (C.c_void_p * max(n, 1))(*[g.ptr for g in grads])
        lens = (C.c_uint64 * max(n, 1))(*[g.numel for g in grads])
        norm = C.c_float()
        self._check(self._lib.omx_clip_grad_norm(self._ctx, ptrs, lens, C.c_uint64(n), C.c_float(max_norm),
                                                 C.byref(norm)))
        return float(norm.value)

    # ---- elementwise / layout ----
    def residual_add_forward(self, x, y, out_dtype: Optional[int] = None):
        if x.shape != y.shape:
            raise OjasError(SHAPE, "residual_add_forward: operands differ")
        od = x.dtype if out_dtype is None else out_dtype
        out = self.empty(x.shape, od)
        self._check(self._lib.omx_residual_add(self._ctx, self._p(x), C.c_int32(x.dtype), self._p(y),
                                               C.c_int32(y.dtype), self._p(out), C.c_int32(od), C.c_uint64(x.numel)))
        return out

    def accumulate_grad(self, acc, grad):
        self._check(self._lib.omx_accumulate_grad(self._ctx, self._p(acc), self._p(grad), C.c_uint64(acc.numel)))

    def scale_grad(self, grad, scale: float):
        self._check(self._lib.omx_scale_grad(self._ctx, self._p(grad), C.c_float(scale), C.c_uint64(grad.numel)))

    def _gelu(self, x, tanh_form):
        y = self.empty(x.shape, x.dtype)
        self._check(self._lib.omx_gelu_forward(self._ctx, self._p(x), self._p(y), C.c_int32(x.dtype),
                                               C.c_uint64(x.numel), C.c_int32(tanh_form)))
        return y

    def _gelu_bwd(self, x, gy, tanh_form):
        gx = self.empty(x.shape, x.dtype)
        self._check(self._lib.omx_gelu_backward(self._ctx, self._p(x), self._p(gy), self._p(gx), C.c_int32(x.dtype),
                                                C.c_uint64(x.numel), C.c_int32(tanh_form)))
        return gx

    def gelu_erf_forward(self, x):
        return self._gelu(x, 0)

    def gelu_erf_backward(self, x, gy):
        return self._gelu_bwd(x, gy, 0)

    def gelu_tanh_forward(self, x):
        return self._gelu(x, 1)

    def gelu_tanh_backward(self, x, gy):
        return self._gelu_bwd(x, gy, 1)

    def permute(self, x, axes):
        if list(axes) != [0, 2, 1, 3] or len(x.shape) != 4:
            raise OjasError(UNSUPPORTED, "permute: only axes [0,2,1,3] of a rank-4 tensor")
        d0, d1, d2, d3 = x.shape
        y = self.empty((d0, d2, d1, d3), x.dtype)
        self._check(self._lib.omx_permute_0213(self._ctx, self._p(x), self._p(y), C.c_int32(x.dtype), C.c_uint64(d0),
                                               C.c_uint64(d1), C.c_uint64(d2), C.c_uint64(d3)))
        return y

    # ---- ops of the nanolab block (backend.rs:1151-1163,1674-1708,1860-1920) ----
    def _same(self, op, *tensors):
        first = tensors[0]
        for t in tensors[1:]:
            if t.shape != first.shape:
                raise OjasError(SHAPE, f"{op}: shapes {first.shape} and {t.shape} differ")
            if t.dtype != first.dtype:
                raise OjasError(DTYPE, f"{op}: operands must share a dtype")

    def silu_forward(self, x):
        y = self.empty(x.shape, x.dtype)
        self._check(self._lib.omx_silu_forward(self._ctx, self._p(x), self._p(y), C.c_int32(x.dtype),
                                               C.c_uint64(x.numel)))
        return y

    def silu_backward(self, x, gy):
        self._same("silu_backward", x, gy)
        gx = self.empty(x.shape, x.dtype)
        self._check(self._lib.omx_silu_backward(self._ctx, self._p(x), self._p(gy), self._p(gx), C.c_int32(x.dtype),
                                                C.c_uint64(x.numel)))
        return gx

    def mul_forward(self, a, b):
        self._same("mul_forward", a, b)
        out = self.empty(a.shape, a.dtype)
        self._check(self._lib.omx_mul_forward(self._ctx, self._p(a), self._p(b), self._p(out), C.c_int32(a.dtype),
                                              C.c_uint64(a.numel)))
        return out

    def mul_backward(self, a, b, gy):
        self._same("mul_backward", a, b, gy)
        ga, gb = self.empty(a.shape, a.dtype), self.empty(a.shape, a.dtype)
        self._check(self._lib.omx_mul_backward(self._ctx, self._p(a), self._p(b), self._p(gy), self._p(ga),
                                               self._p(gb), C.c_int32(a.dtype), C.c_uint64(a.numel)))
        return ga, gb

    def _rope(self, fn, op, x, cos, sin):
        if cos.shape != sin.shape:
            raise OjasError(SHAPE, f"{op}: cos shape {cos.shape} != sin shape {sin.shape}")
        if cos.dtype != F32 or sin.dtype != F32:
            raise OjasError(DTYPE, f"{op}: cos and sin must be f32")
        dim = x.shape[-1]
        if dim % 2:
            raise OjasError(SHAPE, f"{op}: rope last dim {dim} is odd")
        rows = x.numel // dim
        if cos.shape == x.shape:
            time, heads = 0, 0
        elif len(x.shape) == 4 and cos.shape == (x.shape[1], dim):
            time, heads = x.shape[1], x.shape[2]
        else:
            raise OjasError(SHAPE, f"{op}: cos/sin shape {cos.shape} does not broadcast onto {x.shape}")
        y = self.empty(x.shape, x.dtype)
        self._check(fn(self._ctx, self._p(x), self._p(cos), self._p(sin), self._p(y), C.c_int32(x.dtype),
                       C.c_uint64(rows), C.c_uint64(dim), C.c_uint64(time), C.c_uint64(heads)))
        return y

    def rope_half_split_forward(self, x, cos, sin):
        return self._rope(self._lib.omx_rope_half_split_forward, "rope_half_split_forward", x, cos, sin)

    def rope_half_split_backward(self, grad_output, cos, sin):
        return self._rope(self._lib.omx_rope_half_split_backward, "rope_half_split_backward", grad_output, cos, sin)

    def rms_qk_norm_forward(self, q, k, q_weight, k_weight, eps: float = 1e-6, out_dtype: Optional[int] = None):
        dim = q.shape[-1]
        if k.shape[-1] != dim or q_weight.shape != (dim,) or k_weight.shape != (dim,) or q.dtype != k.dtype:
            raise OjasError(SHAPE, f"rms_qk_norm_forward: q {q.shape} k {k.shape} weights {q_weight.shape} "
                                   f"{k_weight.shape}")
        od = q.dtype if out_dtype is None else out_dtype
        qn, kn = self.empty(q.shape, od), self.empty(k.shape, od)
        self._check(self._lib.omx_rms_qk_norm_forward(
            self._ctx, self._p(q), self._p(k), C.c_int32(q.dtype), self._p(q_weight), self._p(k_weight), self._p(qn),
            self._p(kn), C.c_int32(od), C.c_uint64(q.numel // dim), C.c_uint64(k.numel // dim), C.c_uint64(dim),
            C.c_float(eps)))
        return qn, kn

    def rms_qk_norm_backward(self, q, k, q_weight, k_weight, grad_q, grad_k, eps: float = 1e-6):
        dim = q.shape[-1]
        if k.shape[-1] != dim or grad_q.shape != q.shape or grad_k.shape != k.shape or grad_q.dtype != grad_k.dtype:
            raise OjasError(SHAPE, "rms_qk_norm_backward: gradient shapes do not match q / k")
        gq, gk = self.empty(q.shape, grad_q.dtype), self.empty(k.shape, grad_q.dtype)
        gqw, gkw = self.empty((dim,), F32), self.empty((dim,), F32)
        self._check(self._lib.omx_rms_qk_norm_backward(
            self._ctx, self._p(q), self._p(k), C.c_int32(q.dtype), self._p(q_weight), self._p(k_weight),
            self._p(grad_q), self._p(grad_k), C.c_int32(grad_q.dtype), self._p(gq), self._p(gk),
            C.c_int32(grad_q.dtype), self._p(gqw), self._p(gkw), C.c_uint64(q.numel // dim),
            C.c_uint64(k.numel // dim), C.c_uint64(dim), C.c_float(eps)))
        return gq, gk, gqw, gkw

    def _gate_dims(self, op, x, w, b, attn):
        if len(w.shape) != 2:
            raise OjasError(SHAPE, f"{op}: gate weight must be [n_head, d_model]")
        heads, d_model = w.shape
        if x.shape[-1] != d_model:
            raise OjasError(SHAPE, f"{op}: gate weight in {d_model} != input dim {x.shape[-1]}")
        if b.shape != (heads,):
            raise OjasError(SHAPE, f"{op}: gate bias {b.shape} != [{heads}]")
        if len(attn.shape) != len(x.shape) + 1 or attn.shape[-2] != heads or attn.shape[:-2] != x.shape[:-1]:
            raise OjasError(SHAPE, f"{op}: gate attn {attn.shape} does not match input {x.shape}")
        if x.dtype != w.dtype or b.dtype != F32:
            raise OjasError(DTYPE, f"{op}: input and weight share a dtype; bias is f32")
        return x.numel // d_model, d_model, heads, attn.shape[-1]

    def per_head_sigmoid_gate_forward_saving(self, x, w, b, attn, out_dtype: Optional[int] = None, save=True):
        op = "per_head_sigmoid_gate_forward"
        rows, d_model, heads, dh = self._gate_dims(op, x, w, b, attn)
        od = attn.dtype if out_dtype is None else out_dtype
        y = self.empty(attn.shape, od)
        gates = self.empty((rows, heads), F32) if save else None
        self._check(self._lib.omx_per_head_sigmoid_gate_forward(
            self._ctx, self._p(x), self._p(w), C.c_int32(x.dtype), self._p(b), self._p(attn), C.c_int32(attn.dtype),
            self._p(y), C.c_int32(od), self._p(gates), C.c_uint64(rows), C.c_uint64(d_model), C.c_uint64(heads),
            C.c_uint64(dh)))
        return y, gates

    def per_head_sigmoid_gate_forward(self, x, w, b, attn, out_dtype: Optional[int] = None):
        return self.per_head_sigmoid_gate_forward_saving(x, w, b, attn, out_dtype, save=False)[0]

    def per_head_sigmoid_gate_backward_saved(self, x, w, b, attn, gy, scales, g_input_dtype: Optional[int] = None):
        op = "per_head_sigmoid_gate_backward"
        rows, d_model, heads, dh = self._gate_dims(op, x, w, b, attn)
        if gy.shape != attn.shape or gy.dtype != attn.dtype:
            raise OjasError(SHAPE, f"{op}: grad_output {gy.shape} != attn {attn.shape}")
        if scales is not None and (scales.shape != (rows, heads) or scales.dtype != F32):
            raise OjasError(SHAPE, f"{op}: gate scale length does not match rows * heads")
        gxd = x.dtype if g_input_dtype is None else g_input_dtype
        gx, gw = self.empty(x.shape, gxd), self.empty(w.shape, F32)
        gb, ga = self.empty((heads,), F32), self.empty(attn.shape, attn.dtype)
        self._check(self._lib.omx_per_head_sigmoid_gate_backward(
            self._ctx, self._p(x), self._p(w), C.c_int32(x.dtype), self._p(b), self._p(attn), C.c_int32(attn.dtype),
            self._p(gy), C.c_int32(gy.dtype), self._p(scales), self._p(gx), C.c_int32(gxd), self._p(gw), self._p(gb),
            self._p(ga), C.c_int32(attn.dtype), C.c_uint64(rows), C.c_uint64(d_model), C.c_uint64(heads),
            C.c_uint64(dh)))
        return gx, gw, gb, ga

    def per_head_sigmoid_gate_backward(self, x, w, b, attn, gy, g_input_dtype: Optional[int] = None):
        return self.per_head_sigmoid_gate_backward_saved(x, w, b, attn, gy, None, g_input_dtype)

    def per_head_sigmoid_gate_input_grad_add(self, gz, w, add_in):
        """add_in + gz w as f32 [rows, d_model]: the gate's input gradient from `gz`, joined to another
        gradient of the same input (`omx_per_head_sigmoid_gate_input_grad_add`)."""
        rows, heads = gz.shape
        d_model = w.shape[1]
        if w.shape[0] != heads or add_in.numel != rows * d_model or gz.dtype != w.dtype:
            raise OjasError(SHAPE, f"per_head_sigmoid_gate_input_grad_add: gz {gz.shape}, weight {w.shape}, "
                                   f"add_in {add_in.shape}")
        out = self.empty(add_in.shape, F32)
        self._check(self._lib.omx_per_head_sigmoid_gate_input_grad_add(
            self._ctx, self._p(gz), self._p(w), C.c_int32(w.dtype), self._p(add_in), C.c_int32(add_in.dtype),
            self._p(out), C.c_uint64(rows), C.c_uint64(d_model), C.c_uint64(heads)))
        return out

    def per_head_sigmoid_gate_backward_deferred(self, x, w, b, attn, gy, scales, g_input_dtype: Optional[int] = None,
                                                want_input_grad: bool = True):
        """`per_head_sigmoid_gate_backward_saved` without the weight gradient: returns (grad_input, gz
        [rows, heads] in the operands' dtype, grad_bias, grad_attn); grad_weight = gz^T input is the
        caller's (`omx_per_head_sigmoid_gate_backward_deferred`). `want_input_grad=False` leaves the
        input gradient to the caller as well (None comes back in its place)."""
        op = "per_head_sigmoid_gate_backward"
        rows, d_model, heads, dh = self._gate_dims(op, x, w, b, attn)
        if gy.shape != attn.shape or gy.dtype != attn.dtype:
            raise OjasError(SHAPE, f"{op}: grad_output {gy.shape} != attn {attn.shape}")
        if scales is not None and (scales.shape != (rows, heads) or scales.dtype != F32):
            raise OjasError(SHAPE, f"{op}: gate scale length does not match rows * heads")
        gxd = x.dtype if g_input_dtype is None else g_input_dtype
        gx = self.empty(x.shape, gxd) if want_input_grad else None
        gz = self.empty((rows, heads), x.dtype)
        gb, ga = self.empty((heads,), F32), self.empty(attn.shape, attn.dtype)
        self._check(self._lib.omx_per_head_sigmoid_gate_backward_deferred(
            self._ctx, self._p(x), self._p(w), C.c_int32(x.dtype), self._p(b), self._p(attn), C.c_int32(attn.dtype),
            self._p(gy), C.c_int32(gy.dtype), self._p(scales), self._p(gx), C.c_int32(gxd), self._p(gz), self._p(gb),
            self._p(ga), C.c_int32(attn.dtype), C.c_uint64(rows), C.c_uint64(d_model), C.c_uint64(heads),
            C.c_uint64(dh)))
        return gx, gz, gb, ga

    def qkv_prepare_forward(self, qkv_lin, q_weight, k_weight, cos, sin, heads, kv_heads, head_dim, value0=None, lam=None,
                            eps: float = 1e-6):
        """QK-norm, RoPE and the value blend over a fused q | k | v projection output (`omx_qkv_prepare_forward`):
        [batch, time, (heads + 2 kv_heads) head_dim], bf16 or f32; the result is bf16."""
        b, t, pitch = qkv_lin.shape
        if value0 is not None and value0.dtype != qkv_lin.dtype:
            raise OjasError(DTYPE, "qkv_prepare_forward: value0 has the projection output's dtype")
        out = self.empty(qkv_lin.shape, BF16)
        self._check(self._lib.omx_qkv_prepare_forward(
            self._ctx, self._p(qkv_lin), C.c_int32(qkv_lin.dtype), self._p(out), C.c_uint64(pitch), self._p(q_weight), self._p(k_weight),
            self._p(cos), self._p(sin), self._p(value0), self._p(lam), C.c_uint64(b * t), C.c_uint64(t), C.c_uint64(heads),
            C.c_uint64(kv_heads), C.c_uint64(head_dim), C.c_float(eps)))
        return out

    def qkv_prepare_backward(self, qkv_lin, g_qkv, q_weight, k_weight, cos, sin, heads, kv_heads, head_dim, value0=None,
                             lam=None, value0_grad=None, value0_grad_first=True, add_value_grad=None, eps: float = 1e-6):
        """Returns (g_qkv_lin, g_q_weight, g_k_weight, g_lambda or None); `value0_grad` (f32
        [batch, time, kv_heads head_dim]) is written or added to in place."""
        b, t, pitch = qkv_lin.shape
        if value0 is not None and value0.dtype != qkv_lin.dtype:
            raise OjasError(DTYPE, "qkv_prepare_backward: value0 has the projection output's dtype")
        g_lin = self.empty(qkv_lin.shape, BF16)
        gqw, gkw = self.empty((head_dim,), F32), self.empty((head_dim,), F32)
        g_lam = self.empty((1,), F32) if value0 is not None else None
        self._check(self._lib.omx_qkv_prepare_backward(
            self._ctx, self._p(qkv_lin), C.c_int32(qkv_lin.dtype), self._p(g_qkv), self._p(g_lin), C.c_uint64(pitch), self._p(q_weight),
            self._p(k_weight), self._p(cos), self._p(sin), self._p(value0), self._p(lam), self._p(value0_grad),
            C.c_int32(1 if value0_grad_first else 0), self._p(add_value_grad), self._p(gqw), self._p(gkw), self._p(g_lam),
            C.c_uint64(b * t), C.c_uint64(t), C.c_uint64(heads), C.c_uint64(kv_heads), C.c_uint64(head_dim), C.c_float(eps)))
        return g_lin, gqw, gkw, g_lam

    def value_residual_blend_forward(self, value, value0, lam):
        self._same("value_residual_blend_forward", value, value0)
        if lam.numel != 1 or lam.dtype != F32:
            raise OjasError(SHAPE, "value_residual_blend_forward: lambda must be one f32")
        out = self.empty(value.shape, value.dtype)
        self._check(self._lib.omx_value_residual_blend_forward(
            self._ctx, self._p(value), self._p(value0), self._p(lam), self._p(out), C.c_int32(value.dtype),
            C.c_uint64(value.numel)))
        return out

    def value_residual_blend_backward(self, value, value0, lam, gy):
        self._same("value_residual_blend_backward", value, value0, gy)
        if lam.numel != 1 or lam.dtype != F32:
            raise OjasError(SHAPE, "value_residual_blend_backward: lambda must be one f32")
        gv, gv0 = self.empty(value.shape, value.dtype), self.empty(value.shape, value.dtype)
        gl = self.empty((1,), F32)
        self._check(self._lib.omx_value_residual_blend_backward(
            self._ctx, self._p(value), self._p(value0), self._p(lam), self._p(gy), self._p(gv), self._p(gv0),
            C.c_int32(value.dtype), self._p(gl), C.c_uint64(value.numel)))
        return gv, gv0, gl

    # ---- integer ops ----
    # ---- decode: KV cache (backend.rs:2526-2565) ----
    def cached_attention_forward(self, q, k_cache, v_cache, kv_len: int, window: Optional[int] = None):
        """q f32 [B,Tq,H,D] against ring caches [B,Tcap,Hkv,D] (f32, or bf16 storage); f32 [B,Tq,H,D]."""
        if len(q.shape) != 4 or len(k_cache.shape) != 4 or k_cache.shape != v_cache.shape:
            raise OjasError(SHAPE, "cached_attention_forward: q and the caches are rank 4, k_cache == v_cache")
        b, tq, h, d = q.shape
        kb, cap, hkv, kd = k_cache.shape
        if kb != b or kd != d:
            raise OjasError(SHAPE, f"cached_attention_forward: q {q.shape} and cache {k_cache.shape} disagree")
        if window == 0:
            raise OjasError(SHAPE, "cached_attention_forward: attention window must be at least 1")
        if q.dtype != F32 or k_cache.dtype != v_cache.dtype:
            raise OjasError(DTYPE, "cached_attention_forward: q is f32 and the caches share a dtype")
        out = self.empty(q.shape, F32)
        self._check(self._lib.omx_cached_attention_forward(
            self._ctx, self._p(q), self._p(k_cache), self._p(v_cache), C.c_int32(k_cache.dtype), self._p(out),
            C.c_uint64(b), C.c_uint64(tq), C.c_uint64(h), C.c_uint64(hkv), C.c_uint64(d), C.c_uint64(cap),
            C.c_uint64(kv_len), C.c_uint64(window or 0)))
        return out

    def kv_cache_write(self, cache, src, at: int):
        """In place: src f32 [B,Tn,Hkv,D] to positions at..at+Tn of the ring `cache` [B,Tcap,Hkv,D]."""
        if len(cache.shape) != 4 or len(src.shape) != 4:
            raise OjasError(SHAPE, "kv_cache_write: cache and src are rank 4")
        b, cap, hkv, d = cache.shape
        sb, tn, sh, sd = src.shape
        if (sb, sh, sd) != (b, hkv, d):
            raise OjasError(SHAPE, f"kv_cache_write: src {src.shape} does not fit cache {cache.shape}")
        if src.dtype != F32:
            raise OjasError(DTYPE, "kv_cache_write: src is f32")
        self._check(self._lib.omx_kv_cache_write(self._ctx, self._p(cache), C.c_int32(cache.dtype), self._p(src),
                                                 C.c_uint64(b), C.c_uint64(cap), C.c_uint64(hkv), C.c_uint64(d),
                                                 C.c_uint64(tn), C.c_uint64(at)))

    def token_windows(self, tokens: DeviceTensor, starts, seq_len: int):
        """(x, y) u32 [batch, seq_len] from a bin resident on the device (`upload` of
        `TokenBin.read_raw`: U32 words, or u16 words uploaded as BF16-sized storage) and the host
        array of window starts `BatchSampler.next_starts` returns."""
        starts = np.ascontiguousarray(starts, np.uint64)
        batch = int(starts.size)
        x, y = self.empty((batch, seq_len), U32), self.empty((batch, seq_len), U32)
        self._check(self._lib.omx_token_windows(self._ctx, self._p(tokens), C.c_int32(_SIZE_OF[tokens.dtype]),
                                                C.c_uint64(tokens.numel), starts.ctypes.data_as(C.c_void_p),
                                                C.c_uint64(batch), C.c_uint64(seq_len), self._p(x), self._p(y)))
        return x, y

    def argmax_rows(self, x):
        rows, cols = x.shape
        out = self.empty((rows,), U32)
        self._check(self._lib.omx_argmax_rows(self._ctx, self._p(x), C.c_uint64(rows), C.c_uint64(cols), self._p(out)))
        return out

    def topk_rows(self, x, k: int):
        rows, cols = x.shape
        vals, ids = self.empty((rows, k), F32), self.empty((rows, k), U32)
        self._check(self._lib.omx_topk_rows(self._ctx, self._p(x), C.c_uint64(rows), C.c_uint64(cols), C.c_uint64(k),
                                            self._p(vals), self._p(ids)))
        return vals, ids

    def __getattr__(self, name):
        # Every other Backend method refuses by name (unsupported_op, backend.rs:792-797).
        if name.startswith("_"):
            raise AttributeError(name)

        def refuse(*_a, **_k):
            self._lib.omx_unsupported(self._ctx, name.encode())
            raise OjasError(UNSUPPORTED, name)

        return refuse


# ---- shape first (docs/shape-contract.md): every op runs its validator before placement, values,
# budget or launches. The table gives, per method, the validator call on the method's own
# arguments and how many leading arguments are tensor operands (checked for placement next).
class _Meta:
    """Shape and dtype of an operand the method does not take as a tensor (a table given by its
    vocabulary size)."""

    def __init__(self, shape, dtype):
        self.shape, self.dtype = tuple(shape), dtype


def _elementwise(op, n):
    return (lambda *a, **_k: shapes.elementwise_dims(op, *a[:n])), n


_VALIDATED = {
    "linear_forward": (lambda x, w, *_a, **_k: shapes.linear_forward_dims(x, w), 2),
    "linear_backward": (lambda x, w, gy, *_a, **_k: shapes.linear_backward_dims(x, w, gy), 3),
    "causal_sdpa_forward": (lambda q, k, v, window=None, *_a, **_k: shapes.causal_sdpa_forward_dims(q, k, v, window), 3),
    "causal_sdpa_backward": (lambda q, k, v, out, lse, gy, window=None, *_a, **_k:
                             shapes.causal_sdpa_backward_dims(q, k, v, out, lse, gy, window), 6),
    "rms_norm_forward": (lambda x, w, eps=1e-6, *_a, **_k: shapes.rms_norm_forward_dims(x, w, eps), 2),
    "rms_norm_backward": (lambda x, w, gy, eps=1e-6, *_a, **_k: shapes.rms_norm_backward_dims(x, w, gy, eps), 3),
    "rms_qk_norm_forward": (lambda q, k, qw, kw, eps=1e-6, *_a, **_k: shapes.rms_qk_norm_forward_dims(q, k, qw, kw, eps), 4),
    "rms_qk_norm_backward": (lambda q, k, qw, kw, gq, gk, eps=1e-6, *_a, **_k:
                             shapes.rms_qk_norm_backward_dims(q, k, qw, kw, gq, gk, eps), 6),
    "rope_half_split_forward": (lambda x, c, s: shapes.rope_half_split_forward_dims(x, c, s), 3),
    "rope_half_split_backward": (lambda g, c, s: shapes.rope_half_split_backward_dims(g, c, s), 3),
    "cross_entropy_mean_forward": (lambda l, t, *_a, **_k: shapes.cross_entropy_mean_forward_dims(l, t), 2),
    "cross_entropy_mean_backward": (lambda l, t, *_a, **_k: shapes.cross_entropy_mean_backward_dims(l, t), 2),
    "linear_cross_entropy_mean": (lambda x, w, t, ignore_index=None, chunk=(1024, 8192), *_a, **_k:
                                  shapes.linear_ce_dims(x, w, t, chunk), 3),
    "embedding_forward": (lambda table, ids, *_a, **_k: shapes.embedding_forward_dims(table, ids), 2),
    # The table itself is not an argument here: its vocabulary size stands in for it.
    "embedding_backward": (lambda ids, grad, vocab: shapes.embedding_backward_dims(
        _Meta((vocab, grad.shape[-1] if len(grad.shape) else 0), F32), ids, grad), 2),
    "adamw_step": (lambda p, g, m1, m2, *_a, **_k: shapes.adamw_step_dims(p, g, m1, m2), 4),
    "muon_ns5_step": (lambda p, g, m, *_a, **_k: shapes.muon_ns5_step_dims(p, g, m), 3),
    "residual_add_forward": _elementwise("residual_add_forward", 2),
    "accumulate_grad": _elementwise("accumulate_grad", 2),
    "scale_grad": (lambda g, *_a, **_k: shapes.scale_grad_dims(g), 1),
    "gelu_erf_forward": _elementwise("gelu_erf_forward", 1),
    "gelu_erf_backward": _elementwise("gelu_erf_backward", 2),
    "gelu_tanh_forward": _elementwise("gelu_tanh_forward", 1),
    "gelu_tanh_backward": _elementwise("gelu_tanh_backward", 2),
    "silu_forward": _elementwise("silu_forward", 1),
    "silu_backward": _elementwise("silu_backward", 2),
    "mul_forward": _elementwise("mul_forward", 2),
    "mul_backward": _elementwise("mul_backward", 3),
    "permute": (lambda x, axes: shapes.permute_dims(x, axes), 1),
    "per_head_sigmoid_gate_forward": (lambda x, w, b, a, *_a, **_k: shapes.per_head_sigmoid_gate_forward_dims(x, w, b, a), 4),
    "per_head_sigmoid_gate_forward_saving": (lambda x, w, b, a, *_a, **_k:
                                             shapes.per_head_sigmoid_gate_forward_dims(x, w, b, a), 4),
    "per_head_sigmoid_gate_backward": (lambda x, w, b, a, gy, *_a, **_k:
                                       shapes.per_head_sigmoid_gate_backward_dims(x, w, b, a, gy), 5),
    "per_head_sigmoid_gate_backward_saved": (lambda x, w, b, a, gy, *_a, **_k:
                                             shapes.per_head_sigmoid_gate_backward_dims(x, w, b, a, gy), 5),
    "per_head_sigmoid_gate_backward_deferred": (lambda x, w, b, a, gy, *_a, **_k:
                                                shapes.per_head_sigmoid_gate_backward_dims(x, w, b, a, gy), 5),
    "value_residual_blend_forward": (lambda v, v0, lam: shapes.value_residual_blend_forward_dims(v, v0, lam), 3),
    "value_residual_blend_backward": (lambda v, v0, lam, gy: shapes.value_residual_blend_backward_dims(v, v0, lam, gy), 4),
    "cached_attention_forward": (lambda q, kc, vc, kv_len, window=None: shapes.cached_attention_dims(q, kc, vc, kv_len, window), 3),
    "kv_cache_write": (lambda cache, src, at: shapes.kv_cache_write_dims(cache, src, at), 2),
    "argmax_rows": (lambda x: shapes.argmax_rows_dims(x), 1),
    "topk_rows": (lambda x, k: shapes.topk_rows_dims(x, k), 1),
}


def _shape_first(name, method, validator, operands):
    def checked(self, *args, **kwargs):
        try:
            validator(*args, **kwargs)
        except shapes.ShapeError as e:
            raise OjasError(e.code, f"{e.op}: {e.detail}") from None
        for t in args[:operands]:
            if t is not None and not isinstance(t, DeviceTensor):
                raise OjasError(PLACEMENT, f"{name}: operand is in host memory")
        return method(self, *args, **kwargs)

    checked.__name__, checked.__doc__ = name, method.__doc__
    return checked


def _clip_shape_first(method):
    def checked(self, grads, max_norm):
        try:
            shapes.clip_grad_norm_dims(list(grads))
        except shapes.ShapeError as e:
            raise OjasError(e.code, f"{e.op}: {e.detail}") from None
        if any(not isinstance(g, DeviceTensor) for g in grads):
            raise OjasError(PLACEMENT, "clip_grad_norm: operand is in host memory")
        return method(self, grads, max_norm)

    checked.__name__, checked.__doc__ = "clip_grad_norm", method.__doc__
    return checked


for _name, (_validator, _operands) in _VALIDATED.items():
    setattr(MiBackend, _name, _shape_first(_name, getattr(MiBackend, _name), _validator, _operands))
MiBackend.clip_grad_norm = _clip_shape_first(MiBackend.clip_grad_norm)
