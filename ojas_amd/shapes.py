"""Shape validators: one pure function per op, reading dtype and shape only.

The rule of the reference's `ojas_core::shapes` (ojas-core/src/shapes.rs, docs/shape-contract.md):
a backend calls the op's validator BEFORE it checks placement, looks at values, reserves budget or
launches anything, so a malformed call returns the same variant and op name on every backend,
whatever the budget holds and wherever the operands live. Check order inside every validator
(docs/shape-contract.md:27-33): each operand in argument order (dtype, else `Dtype`; no zero axis,
else `Shape "empty tensor"`), then the scalars the layout depends on (RMSNorm's eps, else
`NonFinite`), then ranks and cross-operand equalities in the op's documented order (else `Shape`),
then `OutOfRange` for what does not fit.

An operand is anything with `.shape` and `.dtype`: a `DeviceTensor` or a host numpy array (which the
backend refuses afterwards with `Placement`). Where the reference takes F32 only, bf16 storage is
accepted as well: it is this backend's opt-in storage type, and a u32 or int8 tensor in a float
slot is still `Dtype`. Each function cites the validator it follows.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import numpy as np

F32, BF16, U32, I8 = 0, 1, 2, 3
SHAPE, DTYPE, OUT_OF_RANGE, NON_FINITE = 1, 2, 3, 4
MAX_PERMUTE_RANK = 8
_NUMPY = {np.dtype(np.float32): F32, np.dtype(np.uint32): U32, np.dtype(np.int8): I8}


class ShapeError(Exception):
    """(code, op, detail): the backend turns it into its `OjasError`."""

    def __init__(self, code: int, op: str, detail: str = ""):
        super().__init__(f"{op}: {detail}")
        self.code, self.op, self.detail = code, op, detail


def dtype_of(t) -> int:
    d = t.dtype
    if isinstance(d, int):
        return d
    return _NUMPY.get(np.dtype(d), -1)


def shape_of(t) -> Tuple[int, ...]:
    return tuple(int(x) for x in t.shape)


def _refuse(op, detail):
    return ShapeError(SHAPE, op, detail)


def _operand(op, t, allowed) -> int:
    """shapes.rs:411-431 `operand`: dtype, then no zero axis; returns the element count."""
    if dtype_of(t) not in allowed:
        raise ShapeError(DTYPE, op, f"dtype {dtype_of(t)} where {allowed} is expected")
    s = shape_of(t)
    if 0 in s:
        raise _refuse(op, "empty tensor")
    return int(np.prod(s, dtype=np.int64)) if s else 1


def _float(op, t) -> int:
    return _operand(op, t, (F32, BF16))


def _u32(op, t) -> int:
    return _operand(op, t, (U32,))


def _same(op, a, b):
    if tuple(a) != tuple(b):
        raise _refuse(op, f"shape {list(a)} does not match {list(b)}")


def _same_shape(op, tensors) -> int:
    """shapes.rs:467-478 `same_shape`: every operand's dtype and axes first, then the equalities."""
    for t in tensors:
        _float(op, t)
    first = shape_of(tensors[0])
    for t in tensors[1:]:
        _same(op, first, shape_of(t))
    return int(np.prod(first, dtype=np.int64)) if first else 1


def _split_last(op, shape, rank0):
    if not shape:
        raise _refuse(op, rank0)
    return tuple(shape[:-1]), shape[-1]


def _rows(lead) -> int:
    return int(np.prod(lead, dtype=np.int64)) if lead else 1


# ---- integer ops: shapes.rs:503-547
def argmax_rows_dims(x):
    op = "argmax_rows"
    _float(op, x)
    s = shape_of(x)
    if len(s) != 2:
        raise _refuse(op, f"rank {len(s)} != 2 [rows, cols]")
    if s[0] >= 1 << 32 or s[1] >= 1 << 32:
        raise ShapeError(OUT_OF_RANGE, op, f"{list(s)} does not fit u32 ids")
    return s


def topk_rows_dims(x, k: int):
    op = "topk_rows"
    _float(op, x)
    s = shape_of(x)
    if len(s) != 2:
        raise _refuse(op, f"rank {len(s)} != 2 [rows, cols]")
    if k == 0 or k > s[1]:
        raise ShapeError(OUT_OF_RANGE, op, f"k = {k} is outside 1..={s[1]}")
    return s


# ---- embedding: shapes.rs:549-598 (table first, then ids: argument order)
def _table(op, table):
    s = shape_of(table)
    if len(s) != 2:
        raise _refuse(op, f"embedding table rank {len(s)} != 2 [vocab, dim]")
    return s


def embedding_forward_dims(table, ids):
    op = "embedding_forward"
    _float(op, table)
    tokens = _u32(op, ids)
    vocab, dim = _table(op, table)
    return vocab, dim, tokens, shape_of(ids) + (dim,)


def embedding_backward_dims(table, ids, grad_output):
    op = "embedding_backward"
    _float(op, table)
    tokens = _u32(op, ids)
    _float(op, grad_output)
    vocab, dim = _table(op, table)
    expect = shape_of(ids) + (dim,)
    if shape_of(grad_output) != expect:
        raise _refuse(op, f"embedding grad shape {list(shape_of(grad_output))} != {list(expect)}")
    return vocab, dim, tokens


# ---- linear: shapes.rs:600-659
def _linear(op, x, w):
    ws = shape_of(w)
    if len(ws) != 2:
        raise _refuse(op, f"weight rank {len(ws)} != 2 ([out, in])")
    lead, in_features = _split_last(op, shape_of(x), "input rank 0 has no in-features")
    if in_features != ws[1]:
        raise _refuse(op, f"input in-features {in_features} != weight in-features {ws[1]}")
    return _rows(lead), in_features, ws[0], lead + (ws[0],)


def linear_forward_dims(x, w):
    op = "linear_forward"
    for t in (x, w):
        _float(op, t)
    return _linear(op, x, w)


def linear_backward_dims(x, w, gy):
    op = "linear_backward"
    for t in (x, w, gy):
        _float(op, t)
    dims = _linear(op, x, w)
    if shape_of(gy) != dims[3]:
        raise _refuse(op, f"grad shape {list(shape_of(gy))} != forward shape {list(dims[3])}")
    return dims


# ---- RMSNorm: shapes.rs:661-775 (the gradient's shape before eps and the layout)
def _rms_layout(op, x, w, eps):
    if not math.isfinite(eps):
        raise ShapeError(NON_FINITE, op)
    lead, dim = _split_last(op, shape_of(x), "rms_norm input rank 0")
    if shape_of(w) != (dim,):
        raise _refuse(op, f"rms weight {list(shape_of(w))} != last dim {dim}")
    return _rows(lead), dim


def rms_norm_forward_dims(x, w, eps):
    op = "rms_norm_forward"
    for t in (x, w):
        _float(op, t)
    return _rms_layout(op, x, w, eps)


def rms_norm_backward_dims(x, w, gy, eps):
    op = "rms_norm_backward"
    for t in (x, w, gy):
        _float(op, t)
    _same(op, shape_of(x), shape_of(gy))
    return _rms_layout(op, x, w, eps)


def rms_qk_norm_forward_dims(q, k, qw, kw, eps):
    """The pair reports under `rms_norm_forward` (docs/shape-contract.md, decision 3); q first."""
    return rms_norm_forward_dims(q, qw, eps), rms_norm_forward_dims(k, kw, eps)


def rms_qk_norm_backward_dims(q, k, qw, kw, gq, gk, eps):
    return rms_norm_backward_dims(q, qw, gq, eps), rms_norm_backward_dims(k, kw, gk, eps)


# ---- RoPE: shapes.rs:777-827
def _rope(op, x, cos, sin):
    for t in (x, cos, sin):
        _float(op, t)
    xs, c, s = shape_of(x), shape_of(cos), shape_of(sin)
    if c != s:
        raise _refuse(op, f"cos shape {list(c)} != sin shape {list(s)}")
    lead, dim = _split_last(op, xs, "rope input rank 0")
    if dim % 2:
        raise _refuse(op, f"rope last dim {dim} is odd")
    if c == xs:
        return _rows(lead), dim, 0, 0
    if len(xs) == 4 and len(c) == 2 and c == (xs[1], dim):
        return _rows(lead), dim, xs[1], xs[2]
    raise _refuse(op, f"cos/sin shape {list(c)} does not broadcast onto {list(xs)}")


def rope_half_split_forward_dims(x, cos, sin):
    return _rope("rope_half_split_forward", x, cos, sin)


def rope_half_split_backward_dims(gy, cos, sin):
    return _rope("rope_half_split_backward", gy, cos, sin)


# ---- causal SDPA: shapes.rs:829-951 (the gradient's shape before any head-dim limit)
def _sdpa(op, q, k, v):
    qs, ks, vs = shape_of(q), shape_of(k), shape_of(v)
    if len(qs) != 4:
        raise _refuse(op, f"sdpa query rank {len(qs)} != 4 [B, H, T, D]")
    if ks != vs:
        raise _refuse(op, f"sdpa k {list(ks)} and v {list(vs)} differ")
    differ = _refuse(op, f"sdpa shapes q {list(qs)} k {list(ks)} v {list(vs)} differ")
    if len(ks) != 4:
        raise differ
    batch, heads, seq, dim = qs
    kb, kv_heads, kseq, kd = ks
    grouped = kv_heads != heads
    if (kb, kseq, kd) != (batch, seq, dim) or (grouped and (kv_heads == 0 or heads == 0 or kv_heads > heads or
                                                            heads % kv_heads)):
        raise differ
    return batch, heads, kv_heads, seq, dim


def _window(op, window):
    if window == 0 and window is not None:
        raise _refuse(op, "sdpa window must be at least 1")


def causal_sdpa_forward_dims(q, k, v, window: Optional[int]):
    op = "causal_sdpa_forward"
    for t in (q, k, v):
        _float(op, t)
    _window(op, window)
    return _sdpa(op, q, k, v)


def causal_sdpa_backward_dims(q, k, v, out, lse, gy, window: Optional[int]):
    op = "causal_sdpa_backward"
    for t in (q, k, v, out):
        _float(op, t)
    _operand(op, lse, (F32,))
    _float(op, gy)
    if shape_of(gy) != shape_of(q):
        raise _refuse(op, f"sdpa grad shape {list(shape_of(gy))} != query {list(shape_of(q))}")
    if shape_of(out) != shape_of(q):
        raise _refuse(op, f"sdpa output shape {list(shape_of(out))} != query {list(shape_of(q))}")
    if shape_of(lse) != shape_of(q)[:-1]:
        raise _refuse(op, f"sdpa lse shape {list(shape_of(lse))} != {list(shape_of(q)[:-1])}")
    _window(op, window)
    return _sdpa(op, q, k, v)


# ---- per-head gate and value residual: shapes.rs:953-1024, 1314-1346
def _gate(op, x, w, b, attn):
    ws = shape_of(w)
    if len(ws) != 2:
        raise _refuse(op, "gate weight must be [n_head, d_model]")
    heads, w_in = ws
    xs, a = shape_of(x), shape_of(attn)
    lead, d_model = _split_last(op, xs, "gate input rank 0")
    if w_in != d_model:
        raise _refuse(op, f"gate weight in {w_in} != input dim {d_model}")
    if shape_of(b) != (heads,):
        raise _refuse(op, f"gate bias {list(shape_of(b))} != [{heads}]")
    if len(a) != len(xs) + 1:
        raise _refuse(op, "gate attn rank must be input rank + 1")
    if a[-2] != heads:
        raise _refuse(op, "gate attn head axis != weight rows")
    if a[:-2] != lead:
        raise _refuse(op, "gate attn prefix does not match input prefix")
    return _rows(lead), d_model, heads, a[-1]


def per_head_sigmoid_gate_forward_dims(x, w, b, attn):
    op = "per_head_sigmoid_gate_forward"
    for t in (x, w, b, attn):
        _float(op, t)
    return _gate(op, x, w, b, attn)


def per_head_sigmoid_gate_backward_dims(x, w, b, attn, gy):
    op = "per_head_sigmoid_gate_backward"
    for t in (x, w, b, attn, gy):
        _float(op, t)
    _same(op, shape_of(attn), shape_of(gy))
    return _gate(op, x, w, b, attn)


def _scalar(t) -> bool:
    return all(d == 1 for d in shape_of(t))


def value_residual_blend_forward_dims(v, v0, lam):
    op = "value_residual_blend_forward"
    for t in (v, v0, lam):
        _float(op, t)
    if not _scalar(lam):
        raise _refuse(op, "expected a scalar tensor")
    _same(op, shape_of(v), shape_of(v0))
    return _rows(shape_of(v))


def value_residual_blend_backward_dims(v, v0, lam, gy):
    op = "value_residual_blend_backward"
    for t in (v, v0, lam, gy):
        _float(op, t)
    if not _scalar(lam):
        raise _refuse(op, "value residual lambda must be a scalar")
    _same(op, shape_of(v), shape_of(v0))
    _same(op, shape_of(v), shape_of(gy))
    return _rows(shape_of(v))


# ---- elementwise: shapes.rs:1348-1451, 1662-1690
def elementwise_dims(op: str, *tensors) -> int:
    """silu / mul / residual_add / gelu / accumulate_grad: `same_shape` under the op's name."""
    return _same_shape(op, tensors)


def scale_grad_dims(grad) -> int:
    return _float("scale_grad", grad)


# ---- permute: shapes.rs:2248-2296
def permute_dims(x, axes: Sequence[int]):
    op = "permute"
    _float(op, x)
    s = shape_of(x)
    if len(s) > MAX_PERMUTE_RANK:
        raise _refuse(op, f"rank {len(s)} exceeds {MAX_PERMUTE_RANK}")
    if len(axes) != len(s):
        raise _refuse(op, f"{len(axes)} permutation axes for a rank-{len(s)} tensor")
    seen = set()
    for a in axes:
        if a >= len(s) or a < 0:
            raise _refuse(op, f"axis {a} out of range for rank {len(s)}")
        if a in seen:
            raise _refuse(op, f"axis {a} repeated in {list(axes)}")
        seen.add(a)
    return tuple(s[a] for a in axes)


# ---- cross-entropy and its fusion with the head: shapes.rs:2309-2345, 2409-2446 (logits first)
def _ce(op, logits, targets):
    _float(op, logits)
    _u32(op, targets)
    prefix, vocab = _split_last(op, shape_of(logits), "cross-entropy logits rank 0")
    if shape_of(targets) != prefix:
        raise _refuse(op, f"targets {list(shape_of(targets))} != logits prefix {list(prefix)}")
    return _rows(prefix), vocab


def cross_entropy_mean_forward_dims(logits, targets):
    return _ce("cross_entropy_mean_forward", logits, targets)


def cross_entropy_mean_backward_dims(logits, targets):
    return _ce("cross_entropy_mean_backward", logits, targets)


def linear_ce_dims(x, w, targets, chunk: Tuple[int, int]):
    op = "linear_cross_entropy_mean"
    _float(op, x)
    _float(op, w)
    _u32(op, targets)
    xs, ws, ts = shape_of(x), shape_of(w), shape_of(targets)
    if (len(xs), len(ws), len(ts)) != (2, 2, 1):
        raise _refuse(op, f"expected input [N, d], weight [V, d], targets [N]; got {list(xs)}, {list(ws)}, {list(ts)}")
    if xs[1] != ws[1] or xs[0] != ts[0]:
        raise _refuse(op, f"input {list(xs)}, weight {list(ws)} and targets {list(ts)} disagree")
    if chunk[0] == 0 or chunk[1] == 0:
        raise _refuse(op, f"chunk {chunk} has a zero dimension")
    return xs[0], xs[1], ws[0]


# ---- optimizers and the clip: shapes.rs:2349-2396 (parameter first)
def clip_grad_norm_dims(grads) -> int:
    op = "clip_grad_norm"
    if not grads:
        raise _refuse(op, "empty tensor")
    return sum(_operand(op, g, (F32,)) for g in grads)


def adamw_step_dims(p, g, m1, m2) -> int:
    op = "adamw_step"
    for t in (p, g, m1, m2):
        _operand(op, t, (F32,))
    for t in (g, m1, m2):
        _same(op, shape_of(p), shape_of(t))
    return _rows(shape_of(p))


def muon_ns5_step_dims(p, g, m):
    op = "muon_ns5_step"
    for t in (p, g, m):
        _operand(op, t, (F32,))
    if len(shape_of(p)) != 2:
        raise _refuse(op, "muon parameter must be a matrix")
    _same(op, shape_of(p), shape_of(g))
    _same(op, shape_of(p), shape_of(m))
    return shape_of(p)


# ---- decoding: shapes.rs:2758-2879
def _rank4(op, name, t):
    s = shape_of(t)
    if len(s) != 4:
        raise _refuse(op, f"{name} rank {len(s)} != 4")
    return s


def cached_attention_dims(q, k_cache, v_cache, kv_len: int, window: Optional[int]):
    op = "cached_attention_forward"
    _float(op, q)
    batch, tq, heads, dim = _rank4(op, "q", q)
    _float(op, k_cache)
    k = _rank4(op, "k_cache", k_cache)
    _float(op, v_cache)
    v = _rank4(op, "v_cache", v_cache)
    if k != v:
        raise _refuse(op, f"k_cache {list(k)} != v_cache {list(v)}")
    kb, capacity, kv_heads, kd = k
    if kb != batch or kd != dim:
        raise _refuse(op, f"q {list(shape_of(q))} and cache {list(k)} disagree")
    if heads % kv_heads:
        raise _refuse(op, f"{heads} query heads over {kv_heads} kv heads")
    if window == 0 and window is not None:
        raise _refuse(op, "attention window must be at least 1")
    if kv_len < tq:
        raise ShapeError(OUT_OF_RANGE, op, f"kv_len {kv_len} is below the {tq} new positions")
    w = window if window is not None and window < kv_len else None
    span = min(kv_len, tq + w - 1) if w is not None else kv_len
    if span > capacity:
        raise ShapeError(OUT_OF_RANGE, op, f"the {span} positions read up to kv_len {kv_len} exceed cache capacity {capacity}")
    return batch, tq, capacity, heads, kv_heads, dim, w


def kv_cache_write_dims(cache, src, at: int):
    op = "kv_cache_write"
    _float(op, cache)
    batch, capacity, kv_heads, dim = _rank4(op, "cache", cache)
    _float(op, src)
    sb, tn, sh, sd = _rank4(op, "src", src)
    if (sb, sh, sd) != (batch, kv_heads, dim):
        raise _refuse(op, f"src {list(shape_of(src))} does not fit cache {list(shape_of(cache))}")
    if tn > capacity:
        raise ShapeError(OUT_OF_RANGE, op, f"{tn} positions exceed capacity {capacity}")
    return batch, tn, capacity, kv_heads, dim
