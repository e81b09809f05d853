"""ctypes/numpy access to the CPU oracle (oracle/libojas_oracle.so).

Test infrastructure: the parity checker. Only tests, the smoke check and the
CPU-baseline leg of bench.py import this.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
LIB_PATH = ROOT / "oracle" / "libojas_oracle.so"

OK, SHAPE, DTYPE, OUT_OF_RANGE, NON_FINITE = 0, 1, 2, 3, 4


class OracleError(RuntimeError):
    def __init__(self, code: int, op: str):
        super().__init__(f"{op}: oracle error code {code}")
        self.code = code
        self.op = op


def build_oracle() -> None:
    subprocess.run(["make", "-C", str(ROOT / "oracle"), "-s"], check=True)


def _load() -> C.CDLL:
    if not LIB_PATH.exists():
        build_oracle()
    return C.CDLL(str(LIB_PATH))


_lib = _load()
_f = C.POINTER(C.c_float)
_u32 = C.POINTER(C.c_uint32)
_u16 = C.POINTER(C.c_uint16)
_sz = C.c_size_t


def _fp(a: np.ndarray):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(_f)


def _up(a: np.ndarray):
    assert a.dtype == np.uint32 and a.flags.c_contiguous
    return a.ctypes.data_as(_u32)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _check(code: int, op: str) -> None:
    if code != OK:
        raise OracleError(code, op)


_lib.orc_splitmix_next.restype = C.c_uint64
_lib.orc_splitmix_below.restype = C.c_uint64
_lib.orc_fnv_f32.restype = C.c_uint64
_lib.orc_exp_exact.restype = C.c_float
_lib.orc_exp_exact.argtypes = [C.c_float]
_lib.orc_log_sum_exp_exact.restype = C.c_float
_lib.orc_log_sum_exp_exact.argtypes = [C.c_float, C.c_float]
_lib.orc_log1p_exact.restype = C.c_float
_lib.orc_log1p_exact.argtypes = [C.c_float]
_lib.orc_erf_f64.restype = C.c_double
_lib.orc_erf_f64.argtypes = [C.c_double]
_lib.orc_sigmoid_exact.restype = C.c_float
_lib.orc_sigmoid_exact.argtypes = [C.c_float]
_lib.orc_pow_u64.restype = C.c_double
_lib.orc_pow_u64.argtypes = [C.c_double, C.c_uint64]
for _n in ("orc_gelu_erf", "orc_gelu_tanh", "orc_round_bf16"):
    getattr(_lib, _n).restype = C.c_float
    getattr(_lib, _n).argtypes = [C.c_float]
for _n in ("orc_gelu_erf_backward", "orc_gelu_tanh_backward"):
    getattr(_lib, _n).restype = C.c_float
    getattr(_lib, _n).argtypes = [C.c_float, C.c_float]
_lib.orc_f32_to_bf16.restype = C.c_uint16
_lib.orc_f32_to_bf16.argtypes = [C.c_float]


def set_threads(n: int) -> None:
    _lib.orc_set_threads(int(n))


def get_threads() -> int:
    return int(_lib.orc_get_threads())


class SplitMix64:
    """The reference's test generator (ojas-test-support/src/rng.rs:13-40)."""

    def __init__(self, seed: int):
        self.state = C.c_uint64(seed)

    def next_u64(self) -> int:
        return int(_lib.orc_splitmix_next(C.byref(self.state)))

    def below(self, n: int) -> int:
        return int(_lib.orc_splitmix_below(C.byref(self.state), C.c_uint64(n)))

    def vec(self, n: int, scale: float) -> np.ndarray:
        out = np.empty(n, dtype=np.float32)
        _lib.orc_splitmix_vec(C.byref(self.state), _fp(out), _sz(n), C.c_float(scale))
        return out


def fnv(values: np.ndarray) -> int:
    v = _f32(values).reshape(-1)
    return int(_lib.orc_fnv_f32(_fp(v), _sz(v.size)))


def exp_exact(x: float) -> float:
    return float(_lib.orc_exp_exact(C.c_float(x)))


def exp_exact_vec(x: np.ndarray) -> np.ndarray:
    x = _f32(x)
    y = np.empty_like(x)
    _lib.orc_exp_exact_vec(_fp(x), _fp(y), _sz(x.size))
    return y


def log_sum_exp_exact(m: float, s: float) -> float:
    return float(_lib.orc_log_sum_exp_exact(m, s))


def log1p_exact(x: float) -> float:
    return float(_lib.orc_log1p_exact(x))


def erf_f64(z: float) -> float:
    return float(_lib.orc_erf_f64(z))


def sigmoid_exact(x: float) -> float:
    return float(_lib.orc_sigmoid_exact(x))


def pow_u64(base: float, exp: int) -> float:
    return float(_lib.orc_pow_u64(base, exp))


def gelu_erf(x: float) -> float:
    return float(_lib.orc_gelu_erf(x))


def gelu_erf_backward(x: float, dy: float) -> float:
    return float(_lib.orc_gelu_erf_backward(x, dy))


def gelu_tanh(x: float) -> float:
    return float(_lib.orc_gelu_tanh(x))


def gelu_tanh_backward(x: float, dy: float) -> float:
    return float(_lib.orc_gelu_tanh_backward(x, dy))


def round_bf16(x: np.ndarray) -> np.ndarray:
    x = _f32(x)
    y = np.empty_like(x)
    _lib.orc_round_bf16_vec(_fp(x), _fp(y), _sz(x.size))
    return y


def to_bf16(x: np.ndarray) -> np.ndarray:
    x = _f32(x)
    y = np.empty(x.shape, dtype=np.uint16)
    _lib.orc_to_bf16_vec(_fp(x), y.ctypes.data_as(_u16), _sz(x.size))
    return y


def bf16_to_f32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.uint16)
    y = np.empty(x.shape, dtype=np.float32)
    _lib.orc_bf16_to_f32_vec(x.ctypes.data_as(_u16), _fp(y), _sz(x.size))
    return y


def clip_scale(max_norm: float, total_norm: float) -> float:
    out = C.c_float()
    _check(_lib.orc_clip_scale(C.c_float(max_norm), C.c_float(total_norm), C.byref(out)), "clip_grad_norm")
    return float(out.value)


def adamw_scalars(lr, beta1, beta2, eps, wd, step_before):
    words = (C.c_double * 7)()
    flags = (C.c_int32 * 3)()
    _check(
        _lib.orc_adamw_scalars(
            C.c_double(lr), C.c_double(beta1), C.c_double(beta2), C.c_double(eps), C.c_double(wd),
            C.c_uint64(step_before), words, flags),
        "adamw_step",
    )
    return list(words), list(flags)


def gemm(a: np.ndarray, b: np.ndarray, c: np.ndarray | None = None) -> np.ndarray:
    """C = A @ B (2-D, any strides) with the ascending-k chain; continues from `c` if given."""
    assert a.dtype == np.float32 and b.dtype == np.float32
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    acc = c is not None
    out = np.ascontiguousarray(c, dtype=np.float32).copy() if acc else np.empty((m, n), np.float32)
    es = 4
    _check(
        _lib.orc_gemm(
            a.ctypes.data_as(_f), _sz(a.strides[0] // es), _sz(a.strides[1] // es),
            b.ctypes.data_as(_f), _sz(b.strides[0] // es), _sz(b.strides[1] // es),
            _fp(out), _sz(m), _sz(k), _sz(n), C.c_int(1 if acc else 0)),
        "gemm",
    )
    return out


def linear_forward(x, w):
    x, w = _f32(x), _f32(w)
    rows, kin = x.shape
    nout = w.shape[0]
    y = np.empty((rows, nout), np.float32)
    _check(_lib.orc_linear_forward(_fp(x), _fp(w), _fp(y), _sz(rows), _sz(kin), _sz(nout)), "linear_forward")
    return y


def linear_backward(x, w, gy, need_gx=True, need_gw=True):
    x, w, gy = _f32(x), _f32(w), _f32(gy)
    rows, kin = x.shape
    nout = w.shape[0]
    gx = np.empty((rows, kin), np.float32) if need_gx else None
    gw = np.empty((nout, kin), np.float32) if need_gw else None
    _check(
        _lib.orc_linear_backward(_fp(x), _fp(w), _fp(gy), _fp(gx) if need_gx else None,
                                 _fp(gw) if need_gw else None, _sz(rows), _sz(kin), _sz(nout)),
        "linear_backward",
    )
    return gx, gw


def causal_sdpa_forward(q, k, v, window: int = 0):
    q, k, v = _f32(q), _f32(k), _f32(v)
    b, h, t, d = q.shape
    hkv = k.shape[1]
    out = np.empty_like(q)
    lse = np.empty((b, h, t), np.float32)
    _check(
        _lib.orc_causal_sdpa_forward(_fp(q), _fp(k), _fp(v), _fp(out), _fp(lse), _sz(b), _sz(h), _sz(hkv),
                                     _sz(t), _sz(d), _sz(window)),
        "causal_sdpa_forward",
    )
    return out, lse


def causal_sdpa_backward(q, k, v, out, lse, gy, window: int = 0):
    q, k, v, out, lse, gy = map(_f32, (q, k, v, out, lse, gy))
    b, h, t, d = q.shape
    hkv = k.shape[1]
    gq, gk, gv = np.empty_like(q), np.empty_like(k), np.empty_like(v)
    _check(
        _lib.orc_causal_sdpa_backward(_fp(q), _fp(k), _fp(v), _fp(out), _fp(lse), _fp(gy), _fp(gq), _fp(gk),
                                      _fp(gv), _sz(b), _sz(h), _sz(hkv), _sz(t), _sz(d), _sz(window)),
        "causal_sdpa_backward",
    )
    return gq, gk, gv


def rms_norm_forward(x, w, eps=1e-6):
    x, w = _f32(x), _f32(w)
    dim = x.shape[-1]
    rows = x.size // dim
    y = np.empty_like(x)
    _check(_lib.orc_rms_norm_forward(_fp(x), _fp(w), _fp(y), _sz(rows), _sz(dim), C.c_float(eps)), "rms_norm_forward")
    return y


def rms_norm_backward(x, w, gy, eps=1e-6):
    x, w, gy = _f32(x), _f32(w), _f32(gy)
    dim = x.shape[-1]
    rows = x.size // dim
    gx, gw = np.empty_like(x), np.empty_like(w)
    _check(
        _lib.orc_rms_norm_backward(_fp(x), _fp(w), _fp(gy), _fp(gx), _fp(gw), _sz(rows), _sz(dim), C.c_float(eps)),
        "rms_norm_backward",
    )
    return gx, gw


def _rope(fn, x, cos, sin, name):
    x, cos, sin = _f32(x), _f32(cos), _f32(sin)
    dim = x.shape[-1]
    rows = x.size // dim
    if cos.shape == x.shape:
        time, heads = 0, 0
    else:
        time, heads = x.shape[-3], x.shape[-2]
    y = np.empty_like(x)
    _check(fn(_fp(x), _fp(cos), _fp(sin), _fp(y), _sz(rows), _sz(dim), _sz(time), _sz(heads)), name)
    return y


def rope_forward(x, cos, sin):
    return _rope(_lib.orc_rope_forward, x, cos, sin, "rope_half_split_forward")


def rope_backward(gy, cos, sin):
    return _rope(_lib.orc_rope_backward, gy, cos, sin, "rope_half_split_backward")


def _ign(ignore):
    return (C.c_int(0), C.c_uint32(0)) if ignore is None else (C.c_int(1), C.c_uint32(ignore))


def cross_entropy_mean_forward(logits, targets, ignore=None) -> float:
    logits = _f32(logits)
    targets = np.ascontiguousarray(targets, dtype=np.uint32)
    rows, vocab = logits.shape
    loss = C.c_float()
    hi, iv = _ign(ignore)
    _check(
        _lib.orc_cross_entropy_mean_forward(_fp(logits), _up(targets), _sz(rows), _sz(vocab), hi, iv, C.byref(loss)),
        "cross_entropy_mean_forward",
    )
    return np.float32(loss.value)


def cross_entropy_mean_backward(logits, targets, ignore=None) -> np.ndarray:
    logits = _f32(logits)
    targets = np.ascontiguousarray(targets, dtype=np.uint32)
    rows, vocab = logits.shape
    grad = np.empty_like(logits)
    hi, iv = _ign(ignore)
    _check(
        _lib.orc_cross_entropy_mean_backward(_fp(logits), _up(targets), _sz(rows), _sz(vocab), hi, iv, _fp(grad)),
        "cross_entropy_mean_backward",
    )
    return grad


def linear_cross_entropy_mean(x, w, targets, ignore=None, need_gx=True, need_gw=True):
    x, w = _f32(x), _f32(w)
    targets = np.ascontiguousarray(targets, dtype=np.uint32)
    rows, dim = x.shape
    vocab = w.shape[0]
    loss = C.c_float()
    gx = np.empty_like(x) if need_gx else None
    gw = np.empty_like(w) if need_gw else None
    hi, iv = _ign(ignore)
    _check(
        _lib.orc_linear_cross_entropy_mean(_fp(x), _fp(w), _up(targets), _sz(rows), _sz(dim), _sz(vocab), hi, iv,
                                           C.byref(loss), _fp(gx) if need_gx else None,
                                           _fp(gw) if need_gw else None),
        "linear_cross_entropy_mean",
    )
    return np.float32(loss.value), gx, gw


def embedding_forward(table, ids):
    table = _f32(table)
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    vocab, dim = table.shape
    out = np.empty(ids.shape + (dim,), np.float32)
    _check(_lib.orc_embedding_forward(_fp(table), _up(ids), _fp(out), _sz(ids.size), _sz(vocab), _sz(dim)),
           "embedding_forward")
    return out


def embedding_backward(ids, grad, vocab):
    grad = _f32(grad)
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    dim = grad.shape[-1]
    out = np.empty((vocab, dim), np.float32)
    _check(_lib.orc_embedding_backward(_up(ids), _fp(grad), _fp(out), _sz(ids.size), _sz(vocab), _sz(dim)),
           "embedding_backward")
    return out


def adamw_step(p, g, m, v, step_before, lr, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.0, exact=True):
    """Returns updated copies (p, m, v)."""
    p, m, v = _f32(p).copy(), _f32(m).copy(), _f32(v).copy()
    g = _f32(g)
    _check(
        _lib.orc_adamw_step(_fp(p), _fp(g), _fp(m), _fp(v), _sz(p.size), C.c_uint64(step_before), C.c_double(lr),
                            C.c_double(beta1), C.c_double(beta2), C.c_double(eps), C.c_double(weight_decay),
                            C.c_int(1 if exact else 0)),
        "adamw_step",
    )
    return p, m, v


def muon_ns5_step(p, g, m, lr=0.025, momentum=0.99, weight_decay=0.1, nesterov=True, bf16=False):
    p, m = _f32(p).copy(), _f32(m).copy()
    g = _f32(g)
    rows, cols = p.shape
    _check(
        _lib.orc_muon_ns5_step(_fp(p), _fp(g), _fp(m), _sz(rows), _sz(cols), C.c_double(lr), C.c_double(momentum),
                               C.c_double(weight_decay), C.c_int(int(nesterov)), C.c_int(int(bf16))),
        "muon_ns5_step",
    )
    return p, m


def clip_grad_norm(grads, max_norm):
    """Returns (norm, clipped copies)."""
    gs = [_f32(g).copy() for g in grads]
    ptrs = (_f * len(gs))(*[_fp(g) for g in gs])
    lens = (_sz * len(gs))(*[g.size for g in gs])
    norm = C.c_float()
    _check(_lib.orc_clip_grad_norm(ptrs, lens, _sz(len(gs)), C.c_float(max_norm), C.byref(norm)), "clip_grad_norm")
    return np.float32(norm.value), gs


def residual_add(x, y):
    x, y = _f32(x), _f32(y)
    out = np.empty_like(x)
    _check(_lib.orc_residual_add(_fp(x), _fp(y), _fp(out), _sz(x.size)), "residual_add_forward")
    return out


def _vec1(fn, x):
    x = _f32(x)
    y = np.empty_like(x)
    fn(_fp(x), _fp(y), _sz(x.size))
    return y


def _vec2(fn, x, gy):
    x, gy = _f32(x), _f32(gy)
    y = np.empty_like(x)
    fn(_fp(x), _fp(gy), _fp(y), _sz(x.size))
    return y


def gelu_erf_forward(x):
    return _vec1(_lib.orc_gelu_erf_forward_vec, x)


def gelu_erf_backward_vec(x, gy):
    return _vec2(_lib.orc_gelu_erf_backward_vec, x, gy)


def gelu_tanh_forward(x):
    return _vec1(_lib.orc_gelu_tanh_forward_vec, x)


def gelu_tanh_backward_vec(x, gy):
    return _vec2(_lib.orc_gelu_tanh_backward_vec, x, gy)


def silu_forward(x):
    return _vec1(_lib.orc_silu_forward_vec, x)


def silu_backward(x, gy):
    return _vec2(_lib.orc_silu_backward_vec, x, gy)


def mul_forward(a, b):
    a, b = _f32(a), _f32(b)
    out = np.empty_like(a)
    _check(_lib.orc_mul_forward(_fp(a), _fp(b), _fp(out), _sz(a.size)), "mul_forward")
    return out


def mul_backward(a, b, gy):
    a, b, gy = _f32(a), _f32(b), _f32(gy)
    ga, gb = np.empty_like(a), np.empty_like(a)
    _check(_lib.orc_mul_backward(_fp(a), _fp(b), _fp(gy), _fp(ga), _fp(gb), _sz(a.size)), "mul_backward")
    return ga, gb


def _gate_dims(x, w, attn):
    din = x.shape[-1]
    heads, head_dim = attn.shape[-2], attn.shape[-1]
    assert w.shape == (heads, din) and attn.shape[:-2] == x.shape[:-1]
    return x.size // din, din, heads, head_dim


def gate_values(x, w, bias):
    x, w, bias = _f32(x), _f32(w), _f32(bias)
    rows, din, heads = x.size // x.shape[-1], x.shape[-1], w.shape[0]
    gates = np.empty((rows, heads), np.float32)
    _check(
        _lib.orc_gate_values(_fp(x), _fp(w), _fp(bias), _fp(gates), _sz(rows), _sz(din), _sz(heads)),
        "per_head_sigmoid_gate_forward",
    )
    return gates


def gate_forward(x, w, bias, attn):
    x, w, bias, attn = _f32(x), _f32(w), _f32(bias), _f32(attn)
    rows, din, heads, dh = _gate_dims(x, w, attn)
    y = np.empty_like(attn)
    _check(
        _lib.orc_gate_forward(_fp(x), _fp(w), _fp(bias), _fp(attn), _fp(y), _sz(rows), _sz(din), _sz(heads), _sz(dh)),
        "per_head_sigmoid_gate_forward",
    )
    return y


def gate_backward(x, w, bias, attn, gy):
    x, w, bias, attn, gy = _f32(x), _f32(w), _f32(bias), _f32(attn), _f32(gy)
    rows, din, heads, dh = _gate_dims(x, w, attn)
    gx, gw, gb, ga = np.empty_like(x), np.empty_like(w), np.empty_like(bias), np.empty_like(attn)
    _check(
        _lib.orc_gate_backward(
            _fp(x), _fp(w), _fp(bias), _fp(attn), _fp(gy), _fp(gx), _fp(gw), _fp(gb), _fp(ga),
            _sz(rows), _sz(din), _sz(heads), _sz(dh),
        ),
        "per_head_sigmoid_gate_backward",
    )
    return gx, gw, gb, ga


def value_residual_forward(v, v0, lam):
    v, v0 = _f32(v), _f32(v0)
    out = np.empty_like(v)
    _check(
        _lib.orc_value_residual_forward(_fp(v), _fp(v0), C.c_float(lam), _fp(out), _sz(v.size)),
        "value_residual_blend_forward",
    )
    return out


def value_residual_backward(v, v0, lam, gy):
    v, v0, gy = _f32(v), _f32(v0), _f32(gy)
    gv, gv0 = np.empty_like(v), np.empty_like(v)
    gl = C.c_float()
    _check(
        _lib.orc_value_residual_backward(
            _fp(v), _fp(v0), _fp(gy), C.c_float(lam), _fp(gv), _fp(gv0), C.byref(gl), _sz(v.size)
        ),
        "value_residual_blend_backward",
    )
    return gv, gv0, np.float32(gl.value)


def permute_0213(x):
    x = _f32(x)
    d0, d1, d2, d3 = x.shape
    y = np.empty((d0, d2, d1, d3), np.float32)
    _lib.orc_permute_0213(_fp(x), _fp(y), _sz(d0), _sz(d1), _sz(d2), _sz(d3))
    return y


def argmax_rows(x):
    x = _f32(x)
    rows, cols = x.shape
    out = np.empty(rows, np.uint32)
    _check(_lib.orc_argmax_rows(_fp(x), _sz(rows), _sz(cols), _up(out)), "argmax_rows")
    return out


def topk_rows(x, k):
    x = _f32(x)
    rows, cols = x.shape
    idx = np.empty((rows, k), np.uint32)
    val = np.empty((rows, k), np.float32)
    _check(_lib.orc_topk_rows(_fp(x), _sz(rows), _sz(cols), _sz(k), _up(idx), _fp(val)), "topk_rows")
    return val, idx


class GptConfig(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in
                ("layers", "d_model", "heads", "head_dim", "mlp", "ctx", "vocab", "batch", "gelu_tanh")]


if hasattr(_lib, "orc_gpt_param_count"):
    _lib.orc_gpt_param_count.restype = _sz
    _lib.orc_gpt_param_len.restype = _sz


def gpt_param_lens(cfg: GptConfig):
    n = int(_lib.orc_gpt_param_count(C.byref(cfg)))
    return [int(_lib.orc_gpt_param_len(C.byref(cfg), _sz(i))) for i in range(n)]


def gpt_loss_and_grads(cfg: GptConfig, params, ids, targets):
    params = [_f32(p).reshape(-1) for p in params]
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    targets = np.ascontiguousarray(targets, dtype=np.uint32)
    grads = [np.zeros_like(p) for p in params]
    pp = (_f * len(params))(*[_fp(p) for p in params])
    gp = (_f * len(grads))(*[_fp(g) for g in grads])
    loss = C.c_float()
    _check(_lib.orc_gpt_loss_and_grads(C.byref(cfg), pp, _up(ids), _up(targets), C.byref(loss), gp),
           "gpt_loss_and_grads")
    return np.float32(loss.value), grads


class NanolabConfig(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("layers", "n_embd", "n_head", "n_kv_head", "head_dim", "hidden", "vocab",
                                          "batch", "seq", "window")] + [("rms_eps", C.c_float),
                                                                        ("rope_base", C.c_double)]


_lib.orc_nanolab_param_count.restype = _sz
_lib.orc_nanolab_param_len.restype = _sz

# Parameter names in the order of ojas-model/src/names.rs:188-300.
NANOLAB_BLOCK_PARAMS = ("norm1.weight", "mixer.q_proj.weight", "mixer.k_proj.weight", "mixer.v_proj.weight",
                        "mixer.o_proj.weight", "mixer.q_norm.weight", "mixer.k_norm.weight", "mixer.gate.weight",
                        "mixer.gate.bias", "mixer.vr_lambda", "norm2.weight", "ffn.gate.weight", "ffn.up.weight",
                        "ffn.down.weight")


def nanolab_param_names(layers: int):
    names = ["tok_emb.weight"]
    for i in range(layers):
        names += [f"blocks.{i}.{n}" for n in NANOLAB_BLOCK_PARAMS]
    return names + ["norm_f.weight"]


def nanolab_param_lens(cfg: NanolabConfig):
    n = int(_lib.orc_nanolab_param_count(C.byref(cfg)))
    return [int(_lib.orc_nanolab_param_len(C.byref(cfg), _sz(i))) for i in range(n)]


def rope_tables(seq: int, head_dim: int, base: float = 10000.0):
    cos, sin = np.empty((seq, head_dim), np.float32), np.empty((seq, head_dim), np.float32)
    _lib.orc_rope_tables(_sz(seq), _sz(head_dim), C.c_double(base), _fp(cos), _fp(sin))
    return cos, sin


ROUND_OPERANDS, ROUND_AUTOCAST = 1, 2


def nanolab_loss_and_grads_rounded(cfg: NanolabConfig, params, ids, targets, rounding: int):
    """The nanolab graph with bf16 roundings placed as a bf16 tier places them (oracle/nanolab_exact.cpp):
    ROUND_OPERANDS = at the products' operands only, ROUND_AUTOCAST = wherever the reference's
    Autocast rounds; 0 = none (then equal to nanolab_loss_and_grads bit for bit). Returns (loss, grads)."""
    params = [_f32(p).reshape(-1) for p in params]
    assert [p.size for p in params] == nanolab_param_lens(cfg)
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    targets = np.ascontiguousarray(targets, dtype=np.uint32)
    grads = [np.zeros_like(p) for p in params]
    pp = (_f * len(params))(*[_fp(p) for p in params])
    gp = (_f * len(grads))(*[_fp(g) for g in grads])
    loss = C.c_float()
    _check(_lib.orc_nanolab_loss_and_grads_rounded(C.c_int(rounding), C.byref(cfg), pp, _up(ids), _up(targets),
                                                   C.byref(loss), gp), "nanolab_loss_and_grads_rounded")
    return np.float32(loss.value), grads


def nanolab_loss_and_grads(cfg: NanolabConfig, params, ids, targets, want_logits=False, want_grads=True):
    params = [_f32(p).reshape(-1) for p in params]
    assert [p.size for p in params] == nanolab_param_lens(cfg)
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    targets = np.ascontiguousarray(targets, dtype=np.uint32)
    grads = [np.zeros_like(p) for p in params]
    pp = (_f * len(params))(*[_fp(p) for p in params])
    gp = (_f * len(grads))(*[_fp(g) for g in grads]) if want_grads else None
    logits = np.empty((cfg.batch * cfg.seq, cfg.vocab), np.float32) if want_logits else None
    loss = C.c_float()
    _check(_lib.orc_nanolab_loss_and_grads(C.byref(cfg), pp, _up(ids), _up(targets), C.byref(loss),
                                           _fp(logits) if want_logits else None, gp), "nanolab_loss_and_grads")
    return np.float32(loss.value), logits, (grads if want_grads else None)


def cached_attention_forward(q, k_cache, v_cache, kv_len: int, window: int = 0):
    """q [B,Tq,H,D], caches [B,Tcap,Hkv,D] rings; returns [B,Tq,H,D]."""
    q, k_cache, v_cache = _f32(q), _f32(k_cache), _f32(v_cache)
    b, tq, h, d = q.shape
    _, cap, hkv, _ = k_cache.shape
    out = np.empty_like(q)
    _check(
        _lib.orc_cached_attention_forward(_fp(q), _fp(k_cache), _fp(v_cache), _fp(out), _sz(b), _sz(tq), _sz(h),
                                          _sz(hkv), _sz(d), _sz(cap), _sz(kv_len), _sz(window)),
        "cached_attention_forward",
    )
    return out


def kv_cache_write(cache, src, at: int):
    """Returns the updated copy of `cache` [B,Tcap,Hkv,D] after writing src [B,Tn,Hkv,D] at `at`."""
    cache, src = _f32(cache).copy(), _f32(src)
    b, cap, hkv, d = cache.shape
    _check(_lib.orc_kv_cache_write(_fp(cache), _fp(src), _sz(b), _sz(cap), _sz(hkv), _sz(d), _sz(src.shape[1]), _sz(at)),
           "kv_cache_write")
    return cache


# ---- symmetric int8 weights in groups, and the LoRA step (oracle/lora_exact.cpp) ----
_i8 = C.POINTER(C.c_int8)


def quantize_i8_group(w, group: int = 32):
    """w [rows, cols] -> (codes int8 [rows, cols], scales f32 [rows, cols // group])."""
    w = _f32(w)
    rows, cols = w.shape
    codes = np.empty((rows, cols), np.int8)
    scales = np.empty((rows, cols // group), np.float32)
    _check(_lib.orc_quantize_i8_group(_fp(w), codes.ctypes.data_as(_i8), _fp(scales), _sz(rows), _sz(cols), _sz(group)),
           "quantize_i8_group")
    return codes, scales


def dequant_i8_group(codes, scales, group: int = 32):
    codes = np.ascontiguousarray(codes, dtype=np.int8)
    scales = _f32(scales)
    rows, cols = codes.shape
    w = np.empty((rows, cols), np.float32)
    _check(_lib.orc_dequant_i8_group(codes.ctypes.data_as(_i8), _fp(scales), _fp(w), _sz(rows), _sz(cols), _sz(group)),
           "dequant_i8_group")
    return w


def linear_i8_group_forward(x, codes, scales, group: int = 32):
    x, codes, scales = _f32(x), np.ascontiguousarray(codes, dtype=np.int8), _f32(scales)
    rows, kin = x.shape
    nout = codes.shape[0]
    y = np.empty((rows, nout), np.float32)
    _check(_lib.orc_linear_i8_group_forward(_fp(x), codes.ctypes.data_as(_i8), _fp(scales), _fp(y), _sz(rows), _sz(kin),
                                            _sz(nout), _sz(group)), "linear_i8_group_forward")
    return y


def linear_i8_group_backward_input(codes, scales, gy, group: int = 32):
    gy, codes, scales = _f32(gy), np.ascontiguousarray(codes, dtype=np.int8), _f32(scales)
    rows, nout = gy.shape
    kin = codes.shape[1]
    gx = np.empty((rows, kin), np.float32)
    _check(_lib.orc_linear_i8_group_backward_input(codes.ctypes.data_as(_i8), _fp(scales), _fp(gy), _fp(gx), _sz(rows),
                                                   _sz(kin), _sz(nout), _sz(group)), "linear_i8_group_backward_input")
    return gx


class LoraConfig(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("layers", "d_model", "heads", "head_dim", "hidden", "vocab", "batch", "seq",
                                          "rank")] + [("rms_eps", C.c_float), ("lora_scale", C.c_float),
                                                      ("rope_base", C.c_double)]


_lib.orc_lora_frozen_count.restype = _sz
_lib.orc_lora_adapter_count.restype = _sz

LORA_FROZEN_PER_LAYER = ("norm1", "wq", "wk", "wv", "wo", "norm2", "wgate", "wup", "wdown")
LORA_ADAPTERS_PER_LAYER = ("Aq", "Bq", "Ak", "Bk", "Av", "Bv", "Ao", "Bo")


def lora_frozen_shapes(cfg: LoraConfig):
    d, m = cfg.d_model, cfg.hidden
    per = [(d,), (d, d), (d, d), (d, d), (d, d), (d,), (m, d), (m, d), (d, m)]
    return [(cfg.vocab, d)] + per * cfg.layers + [(d,)]


def lora_adapter_shapes(cfg: LoraConfig):
    d, r = cfg.d_model, cfg.rank
    return [(r, d), (d, r)] * 4 * cfg.layers


def lora_loss_and_grads(cfg: LoraConfig, frozen, adapters, ids, targets, want_grads=True):
    """frozen: dequantised f32 tensors in lora_frozen_shapes order; adapters in lora_adapter_shapes order."""
    frozen = [_f32(p).reshape(-1) for p in frozen]
    adapters = [_f32(p).reshape(-1) for p in adapters]
    assert [p.size for p in frozen] == [int(np.prod(s)) for s in lora_frozen_shapes(cfg)]
    assert [p.size for p in adapters] == [int(np.prod(s)) for s in lora_adapter_shapes(cfg)]
    ids = np.ascontiguousarray(ids, dtype=np.uint32).reshape(-1)
    targets = np.ascontiguousarray(targets, dtype=np.uint32).reshape(-1)
    grads = [np.zeros_like(p) for p in adapters]
    fp = (_f * len(frozen))(*[_fp(p) for p in frozen])
    ap = (_f * len(adapters))(*[_fp(p) for p in adapters])
    gp = (_f * len(grads))(*[_fp(g) for g in grads]) if want_grads else None
    loss = C.c_float()
    _check(_lib.orc_lora_loss_and_grads(C.byref(cfg), fp, ap, _up(ids), _up(targets), C.byref(loss), gp),
           "lora_loss_and_grads")
    return np.float32(loss.value), (grads if want_grads else None)
