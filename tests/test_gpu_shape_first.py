"""Shape first (docs/shape-contract.md of the reference): every op runs its validator
(`ojas_amd/shapes.py`, restating ojas-core/src/shapes.rs) before it checks placement, looks at
values or device limits, or charges the budget. Modelled on ojas-wgpu/tests/shape_first.rs: each
malformed call below must return the validator's variant under the op's name, leave nothing
charged and record nothing (the next `sync` is clean), in three modes:

- (b) device operands and a budget that holds the operands and nothing else (the reference's modes
  (a) Budget 0 and (b) inputs-only cap are one here: this backend charges operands and outputs to
  one budget);
- (c) device operands with a NaN in a well-formed f32 operand;
- (d) host operands (the validator runs before placement).

An operand with a zero axis or of rank 0 cannot be uploaded as it is, so its case runs (d) only. The order inside a
validator is pinned by cases that are wrong in two ways at once (docs/shape-contract.md D5-D11).
"""
import numpy as np
import pytest

gpu = pytest.mark.gpu

SHAPE, DTYPE, OUT_OF_RANGE, NON_FINITE, CAPACITY, PLACEMENT = 1, 2, 3, 4, 6, 12
CAP = 8 << 20


def f(*shape):
    n = int(np.prod(shape)) if shape else 1
    return (0.25 + (np.arange(n) % 7) * 0.125).astype(np.float32).reshape(shape)


def u(*shape, value=0):
    return np.full(shape, value, np.uint32)


def cases():
    """(name, method, operands, extra args, nan operand index or None, expected code, expected op)."""
    c = []

    def add(name, method, operands, extra, nan, code, op=None):
        c.append((name, method, operands, extra, nan, code, op or method))

    # embedding: table first, then ids (D5); the id range is not the validator's (D11, D12)
    add("table rank 1", "embedding_forward", [f(4), u(2)], (), 0, SHAPE)
    add("table rank 3, id out of range", "embedding_forward", [f(2, 2, 2), u(2, value=9)], (), 0, SHAPE)
    add("f32 ids", "embedding_forward", [f(4, 2), f(2)], (), 0, DTYPE)
    add("u32 table", "embedding_forward", [u(4, 2), u(2)], (), None, DTYPE)
    add("u32 table and f32 ids: the table is named first", "embedding_forward", [u(4, 2), f(2)], (), None, DTYPE)
    add("zero ids", "embedding_forward", [f(4, 2), u(0)], (), None, SHAPE)
    add("u32 grad", "embedding_backward", [u(3), u(3, 2)], (4,), None, DTYPE)
    add("f32 ids", "embedding_backward", [f(3), f(3, 2)], (4,), 1, DTYPE)
    add("grad rows, id out of range", "embedding_backward", [u(3, value=9), f(2, 2)], (4,), 1, SHAPE)
    # linear
    add("weight rank 1", "linear_forward", [f(3, 4), f(4)], (), 0, SHAPE)
    add("in-features", "linear_forward", [f(3, 4), f(5, 3)], (), 0, SHAPE)
    add("u32 input", "linear_forward", [u(3, 4), f(5, 4)], (), 1, DTYPE)
    add("u32 weight and wrong in-features: dtype first", "linear_forward", [f(3, 4), u(5, 3)], (), 0, DTYPE)
    add("rank-0 input", "linear_forward", [f(), f(5, 1)], (), None, SHAPE)
    add("zero rows", "linear_forward", [f(0, 4), f(5, 4)], (), None, SHAPE)
    add("grad shape", "linear_backward", [f(3, 4), f(5, 4), f(3, 6)], (), 0, SHAPE)
    add("u32 grad", "linear_backward", [f(3, 4), f(5, 4), u(3, 5)], (), 0, DTYPE)
    add("weight rank 3", "linear_backward", [f(3, 4), f(5, 4, 1), f(3, 5)], (), 2, SHAPE)
    # RMSNorm: the gradient's shape before eps and the layout (D8)
    add("weight length", "rms_norm_forward", [f(3, 8), f(7)], (1e-6,), 0, SHAPE)
    add("eps inf", "rms_norm_forward", [f(3, 8), f(8)], (float("inf"),), 0, NON_FINITE)
    add("eps nan with a wrong weight: eps first", "rms_norm_forward", [f(3, 8), f(7)], (float("nan"),), 0, NON_FINITE)
    add("u32 weight and eps inf: dtype first", "rms_norm_forward", [f(3, 8), u(8)], (float("inf"),), 0, DTYPE)
    add("grad shape and eps inf: grad first", "rms_norm_backward", [f(3, 8), f(8), f(3, 7)], (float("inf"),), 0, SHAPE)
    add("weight length", "rms_norm_backward", [f(3, 8), f(9), f(3, 8)], (1e-6,), 2, SHAPE)
    add("k weight", "rms_qk_norm_forward", [f(2, 3, 8), f(2, 1, 8), f(8), f(4)], (1e-6,), 0, SHAPE, "rms_norm_forward")
    add("q weight and k dtype: q first", "rms_qk_norm_forward", [f(2, 3, 8), u(2, 1, 8), f(4), f(8)], (1e-6,), 0, SHAPE,
        "rms_norm_forward")
    add("grad k shape", "rms_qk_norm_backward", [f(2, 3, 8), f(2, 1, 8), f(8), f(8), f(2, 3, 8), f(2, 2, 8)], (1e-6,), 0,
        SHAPE, "rms_norm_backward")
    # RoPE
    add("odd dim", "rope_half_split_forward", [f(1, 2, 2, 5), f(2, 5), f(2, 5)], (), 0, SHAPE)
    add("cos != sin", "rope_half_split_forward", [f(1, 2, 2, 4), f(2, 4), f(3, 4)], (), 0, SHAPE)
    add("no broadcast", "rope_half_split_backward", [f(1, 2, 2, 4), f(3, 4), f(3, 4)], (), 0, SHAPE)
    add("u32 cos", "rope_half_split_backward", [f(1, 2, 2, 4), u(2, 4), f(2, 4)], (), 0, DTYPE)
    # causal SDPA: shapes before any head-dim limit (D9, D15)
    add("query rank 3", "causal_sdpa_forward", [f(2, 3, 4), f(2, 3, 4), f(2, 3, 4)], (), 0, SHAPE)
    add("k != v", "causal_sdpa_forward", [f(1, 2, 3, 4), f(1, 2, 3, 4), f(1, 1, 3, 4)], (), 0, SHAPE)
    add("head grouping 3 over 2", "causal_sdpa_forward", [f(1, 3, 3, 4), f(1, 2, 3, 4), f(1, 2, 3, 4)], (), 0, SHAPE)
    add("window 0", "causal_sdpa_forward", [f(1, 2, 3, 4), f(1, 2, 3, 4), f(1, 2, 3, 4)], (0,), 0, SHAPE)
    add("u32 v", "causal_sdpa_forward", [f(1, 2, 3, 4), f(1, 2, 3, 4), u(1, 2, 3, 4)], (), 0, DTYPE)
    add("head_dim 300 and k != v: the shape is named, not the limit", "causal_sdpa_forward",
        [f(1, 1, 2, 300), f(1, 1, 2, 300), f(1, 1, 3, 300)], (), 0, SHAPE)
    add("grad shape, head_dim 300", "causal_sdpa_backward",
        [f(1, 1, 2, 300), f(1, 1, 2, 300), f(1, 1, 2, 300), f(1, 1, 2, 300), f(1, 1, 2), f(1, 1, 2, 299)], (), 0, SHAPE)
    add("lse shape", "causal_sdpa_backward",
        [f(1, 2, 3, 4), f(1, 2, 3, 4), f(1, 2, 3, 4), f(1, 2, 3, 4), f(1, 2, 4), f(1, 2, 3, 4)], (), 0, SHAPE)
    add("output shape", "causal_sdpa_backward",
        [f(1, 2, 3, 4), f(1, 2, 3, 4), f(1, 2, 3, 4), f(1, 2, 3, 5), f(1, 2, 3), f(1, 2, 3, 4)], (), 0, SHAPE)
    add("u32 lse", "causal_sdpa_backward",
        [f(1, 2, 3, 4), f(1, 2, 3, 4), f(1, 2, 3, 4), f(1, 2, 3, 4), u(1, 2, 3), f(1, 2, 3, 4)], (), 0, DTYPE)
    # per-head gate (D10) and value residual
    add("bias length", "per_head_sigmoid_gate_forward", [f(2, 3, 8), f(2, 8), f(3), f(2, 3, 2, 4)], (), 0, SHAPE)
    add("weight in", "per_head_sigmoid_gate_forward", [f(2, 3, 8), f(2, 7), f(2), f(2, 3, 2, 4)], (), 0, SHAPE)
    add("attn rank", "per_head_sigmoid_gate_forward_saving", [f(2, 3, 8), f(2, 8), f(2), f(6, 2, 4)], (), 0, SHAPE,
        "per_head_sigmoid_gate_forward")
    add("grad shape and bias length: grad first", "per_head_sigmoid_gate_backward",
        [f(2, 3, 8), f(2, 8), f(3), f(2, 3, 2, 4), f(2, 3, 2, 5)], (), 0, SHAPE)
    add("attn heads", "per_head_sigmoid_gate_backward", [f(2, 3, 8), f(2, 8), f(2), f(2, 3, 3, 4), f(2, 3, 3, 4)], (), 0, SHAPE)
    add("lambda not a scalar", "value_residual_blend_forward", [f(2, 3), f(2, 3), f(2)], (), 0, SHAPE)
    add("value0 shape", "value_residual_blend_forward", [f(2, 3), f(3, 2), f(1)], (), 0, SHAPE)
    add("grad shape", "value_residual_blend_backward", [f(2, 3), f(2, 3), f(1), f(2, 4)], (), 0, SHAPE)
    # elementwise
    for op, n in (("silu_backward", 2), ("mul_forward", 2), ("mul_backward", 3), ("residual_add_forward", 2),
                  ("gelu_erf_backward", 2), ("gelu_tanh_backward", 2), ("accumulate_grad", 2)):
        add("shapes differ", op, [f(2, 3)] * (n - 1) + [f(3, 2)], (), 0, SHAPE)
        add("u32 operand", op, [f(2, 3)] * (n - 1) + [u(2, 3)], (), 0, DTYPE)
    for op in ("silu_forward", "gelu_erf_forward", "gelu_tanh_forward"):
        add("u32 input", op, [u(2, 3)], (), None, DTYPE)
        add("zero axis", op, [f(2, 0)], (), None, SHAPE)
    add("u32 grad", "scale_grad", [u(4)], (0.5,), None, DTYPE)
    add("axes count", "permute", [f(2, 3, 4, 5)], ([0, 2, 1],), 0, SHAPE)
    add("axis repeated", "permute", [f(2, 3, 4, 5)], ([0, 2, 2, 3],), 0, SHAPE)
    add("axis out of range", "permute", [f(2, 3, 4, 5)], ([0, 2, 1, 4],), 0, SHAPE)
    # cross-entropy: logits first, then targets (D6); target range is not the validator's
    add("targets shape", "cross_entropy_mean_forward", [f(4, 8), u(5)], (), 0, SHAPE)
    add("f32 targets", "cross_entropy_mean_forward", [f(4, 8), f(4)], (), 0, DTYPE)
    add("u32 logits and f32 targets: logits first", "cross_entropy_mean_backward", [u(4, 8), f(4)], (), None, DTYPE)
    add("targets shape, target out of range", "cross_entropy_mean_backward", [f(4, 8), u(3, value=99)], (), 0, SHAPE)
    add("model dim", "linear_cross_entropy_mean", [f(4, 8), f(16, 7), u(4)], (), 0, SHAPE)
    add("targets rank", "linear_cross_entropy_mean", [f(4, 8), f(16, 8), u(4, 1)], (), 0, SHAPE)
    add("chunk 0", "linear_cross_entropy_mean", [f(4, 8), f(16, 8), u(4)], (None, (0, 8)), 0, SHAPE)
    add("f32 targets", "linear_cross_entropy_mean", [f(4, 8), f(16, 8), f(4)], (), 0, DTYPE)
    # optimizers: the parameter first (D7); scalars are not the validator's
    add("moment shape", "adamw_step", [f(6), f(6), f(6), f(5)], (0, "adamw"), 1, SHAPE)
    add("u32 grad", "adamw_step", [f(6), u(6), f(6), f(6)], (0, "adamw"), 0, DTYPE)
    add("u32 param and grad shape: dtype of the param first", "adamw_step", [u(6), f(5), f(6), f(6)], (0, "adamw"), 1, DTYPE)
    add("vector parameter", "muon_ns5_step", [f(6), f(6), f(6)], ("muon",), 1, SHAPE)
    add("momentum shape", "muon_ns5_step", [f(2, 3), f(2, 3), f(3, 2)], ("muon",), 1, SHAPE)
    add("no gradients", "clip_grad_norm", [], (1.0,), None, SHAPE)
    add("u32 gradient", "clip_grad_norm", [f(4), u(4)], (1.0,), 0, DTYPE)
    # integer ops and decoding
    add("rank 1", "argmax_rows", [f(4)], (), 0, SHAPE)
    add("k above cols", "topk_rows", [f(2, 4)], (5,), 0, OUT_OF_RANGE)
    add("k 0", "topk_rows", [f(2, 4)], (0,), 0, OUT_OF_RANGE)
    add("k != v caches", "cached_attention_forward", [f(1, 1, 2, 4), f(1, 8, 1, 4), f(1, 8, 2, 4)], (3,), 0, SHAPE)
    add("kv_len below the new positions", "cached_attention_forward", [f(1, 3, 2, 4), f(1, 8, 1, 4), f(1, 8, 1, 4)], (2,), 0,
        OUT_OF_RANGE)
    add("kv_len above capacity", "cached_attention_forward", [f(1, 1, 2, 4), f(1, 8, 1, 4), f(1, 8, 1, 4)], (9,), 0, OUT_OF_RANGE)
    add("window 0", "cached_attention_forward", [f(1, 1, 2, 4), f(1, 8, 1, 4), f(1, 8, 1, 4)], (3, 0), 0, SHAPE)
    add("src heads", "kv_cache_write", [f(1, 8, 2, 4), f(1, 2, 1, 4)], (0,), 1, SHAPE)
    add("more positions than capacity", "kv_cache_write", [f(1, 2, 2, 4), f(1, 3, 2, 4)], (0,), 1, OUT_OF_RANGE)
    return c


CASES = cases()


@pytest.fixture(scope="module")
def be():
    from ojas_amd.backend import MiBackend

    backend = MiBackend(0, budget_bytes=CAP)
    yield backend
    backend.close()


def extras(extra):
    from ojas_amd.backend import AdamWConfig, MuonNs5Config

    swap = {"adamw": AdamWConfig.nanolab(1e-3, 0.1), "muon": MuonNs5Config.nanolab_default()}
    return tuple(swap.get(e, e) if isinstance(e, str) else e for e in extra)


def call(be, method, operands, extra):
    if method == "clip_grad_norm":
        return getattr(be, method)(list(operands), *extra)
    return getattr(be, method)(*operands, *extra)


def refused(be, method, operands, extra, code, op, mode):
    import gc

    from ojas_amd.backend import OjasError

    gc.collect()  # tensors of earlier cases are freed now, not during the call
    live = be.budget()["live"]
    with pytest.raises(OjasError) as e:
        call(be, method, operands, extras(extra))
    assert e.value.code == code, (mode, e.value.code, e.value.detail)
    assert e.value.detail.startswith(op + ":"), (mode, e.value.detail)
    assert be.budget()["live"] == live, mode  # nothing charged
    be.sync()  # nothing recorded


@gpu
@pytest.mark.parametrize("case", CASES, ids=[f"{c[1]}: {c[0]}" for c in CASES])
def test_malformed_call_is_refused_by_its_validator(be, case):
    from ojas_amd.backend import F32

    name, method, operands, extra, nan_at, code, op = case
    print(f"shape first: {method}: {name}", flush=True)
    # (d) host operands
    refused(be, method, operands, extra, code, op, "host operands")
    if any(0 in a.shape or a.ndim == 0 for a in operands):  # neither can be uploaded as it is
        return
    # (b) device operands, the budget holding them and nothing else
    device = [be.upload(a) for a in operands]
    room = be.budget()["limit"] - be.budget()["live"]
    filler = be.empty((room // 4,), F32) if room >= 4 else None
    assert be.budget()["limit"] - be.budget()["live"] < 256
    refused(be, method, device, extra, code, op, "full budget")
    del filler
    # (c) a NaN in a well-formed f32 operand
    if nan_at is not None:
        poisoned = list(device)
        poisoned[nan_at] = be.upload(np.full(operands[nan_at].shape, np.nan, np.float32))
        refused(be, method, poisoned, extra, code, op, "NaN operand")


@gpu
def test_well_formed_calls_meet_the_placement_check_and_the_budget_after_the_validator(be):
    """The same calls once they are well formed: host operands are `Placement`, a full budget is
    `CapacityExceeded`; so the refusals above came from the validators, not from these."""
    from ojas_amd.backend import F32, OjasError

    x, w = f(3, 4), f(5, 4)
    with pytest.raises(OjasError) as e:
        be.linear_forward(x, w)
    assert e.value.code == PLACEMENT
    dx, dw = be.upload(x), be.upload(w)
    room = be.budget()["limit"] - be.budget()["live"]
    filler = be.empty((room // 4,), F32)
    with pytest.raises(OjasError) as e:
        be.linear_forward(dx, dw)
    assert e.value.code == CAPACITY
    del filler
    assert be.download(be.linear_forward(dx, dw)).shape == (3, 5)


def test_validators_accept_what_the_ops_accept():
    """CPU-side: the validators' accepted shapes, and the order of their checks on host metadata."""
    from ojas_amd import shapes

    assert shapes.linear_forward_dims(f(2, 3, 4), f(5, 4)) == (6, 4, 5, (2, 3, 5))
    assert shapes.causal_sdpa_forward_dims(f(1, 4, 3, 8), f(1, 2, 3, 8), f(1, 2, 3, 8), None) == (1, 4, 2, 3, 8)
    assert shapes.rope_half_split_forward_dims(f(1, 2, 3, 4), f(2, 4), f(2, 4)) == (6, 4, 2, 3)
    assert shapes.rope_half_split_forward_dims(f(5, 4), f(5, 4), f(5, 4)) == (5, 4, 0, 0)
    assert shapes.embedding_forward_dims(f(9, 2), u(3, 5)) == (9, 2, 15, (3, 5, 2))
    assert shapes.cached_attention_dims(f(1, 1, 4, 8), f(1, 16, 2, 8), f(1, 16, 2, 8), 20, 4)[-1] == 4


@pytest.mark.parametrize("case", CASES, ids=[f"{c[1]}: {c[0]}" for c in CASES])
def test_validator_alone_names_the_variant_and_the_op(case):
    """CPU-side: the validator each method runs first, on the cases' host metadata."""
    from ojas_amd import shapes
    from ojas_amd.backend import _VALIDATED

    _, method, operands, extra, _, code, op = case
    with pytest.raises(shapes.ShapeError) as e:
        if method == "clip_grad_norm":
            shapes.clip_grad_norm_dims(list(operands))
        else:
            _VALIDATED[method][0](*operands, *extras(extra))
    assert (e.value.code, e.value.op) == (code, op), (e.value.code, e.value.op, e.value.detail)
