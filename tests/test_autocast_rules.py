"""The tag rules of `ojas_amd.autocast.Autocast` (ojas-core/src/autocast.rs) over a recording stand-in
for the device backend: which operands get rounded, which outputs come back tagged, and which calls
clear a tag. Host logic only; the numerics of the tier run on the GPU (tests/test_gpu_nanolab.py)."""
import pytest

from ojas_amd.autocast import Autocast
from ojas_amd.backend import BF16, F32


class T:
    def __init__(self, name, dtype=F32, tagged=False):
        self.name, self.dtype, self.shape, self.compute_bf16 = name, dtype, (2, 2), tagged


class Recorder:
    """Every method returns fresh untagged f32 tensors and logs (op, operand names)."""

    def __init__(self):
        self.calls = []

    def _log(self, op, *ts):
        self.calls.append((op, tuple(t.name for t in ts)))

    def cast_bf16(self, x):
        self._log("cast", x)
        return T(f"r({x.name})")

    def linear_forward(self, x, w, out_dtype=None):
        self._log("linear_forward", x, w)
        return T("y")

    def linear_backward(self, x, w, gy, **kw):
        self._log("linear_backward", x, w, gy)
        return T("gx"), T("gw")

    def causal_sdpa_forward(self, q, k, v, window=None, out_dtype=None):
        self._log("sdpa_forward", q, k, v)
        return T("att"), T("lse")

    def causal_sdpa_backward(self, q, k, v, out, lse, gy, window=None, grad_dtype=F32):
        self._log("sdpa_backward", q, k, v, out, lse, gy)
        return T("gq"), T("gk"), T("gv")

    def causal_sdpa_backward_recompute(self, q, k, v, gy, window=None, grad_dtype=F32):
        self._log("sdpa_backward_recompute", q, k, v, gy)
        return T("gq"), T("gk"), T("gv")

    def silu_forward(self, x):
        return T("silu")

    def mul_forward(self, a, b):
        return T("mul")

    def residual_add_forward(self, x, y):
        return T("sum")

    def rms_norm_forward(self, x, w, eps):
        self._log("rms_norm_forward", x, w)
        return T("h")

    def permute(self, x, axes):
        return T(f"p({x.name})")

    def accumulate_grad(self, acc, grad):
        self._log("accumulate_grad", acc, grad)

    def scale_grad(self, grad, scale):
        self._log("scale_grad", grad)

    def adamw_step(self, param, grad, m1, m2, step, cfg):
        self._log("adamw_step", param)

    def linear_cross_entropy_mean(self, x, w, targets):
        self._log("lce", x, w)
        return T("loss"), T("ghf"), T("ghead")


def ops(rec, name):
    return [c for c in rec.calls if c[0] == name]


def test_outside_a_region_every_call_goes_through_untouched():
    rec = Recorder()
    ac = Autocast(rec)
    y = ac.linear_forward(T("x"), T("w"))
    assert rec.calls == [("linear_forward", ("x", "w"))] and not y.compute_bf16
    with ac.region(enabled=False):  # AutocastMode::Off
        assert not ac.on
        ac.linear_forward(T("x"), T("w"))
    assert not ops(rec, "cast")


def test_matmul_class_rounds_untagged_operands_and_tags_its_output():
    rec = Recorder()
    ac = Autocast(rec)
    with ac.region():
        y = ac.linear_forward(T("x"), T("w"))
        assert [c[1][0] for c in ops(rec, "cast")] == ["x", "w", "y"]
        assert ops(rec, "linear_forward") == [("linear_forward", ("r(x)", "r(w)"))]
        assert y.compute_bf16 and y.name == "r(y)"
        rec.calls.clear()
        ac.linear_forward(y, T("w2"))  # a tagged operand is not rounded again
        assert [c[1][0] for c in ops(rec, "cast")] == ["w2", "y"]
    assert not ac.on


def test_bf16_storage_is_never_rounded():
    rec = Recorder()
    ac = Autocast(rec)
    with ac.region():
        ac.linear_forward(T("x", BF16), T("w", BF16))
    assert [c[1][0] for c in ops(rec, "cast")] == ["y"]


def test_weight_gradients_stay_f32():
    rec = Recorder()
    ac = Autocast(rec)
    with ac.region():
        gx, gw = ac.linear_backward(T("x"), T("w"), T("gy"))
        loss, ghf, ghead = ac.linear_cross_entropy_mean(T("hf"), T("emb"), T("t"))
    assert gx.compute_bf16 and not gw.compute_bf16
    assert ghf.compute_bf16 and not ghead.compute_bf16 and not loss.compute_bf16
    assert ops(rec, "lce") == [("lce", ("r(hf)", "r(emb)"))]


def test_pointwise_ops_follow_their_operands():
    ac = Autocast(Recorder())
    tagged, plain = T("a", tagged=True), T("b")
    with ac.region():
        assert ac.silu_forward(tagged).compute_bf16 and not ac.silu_forward(plain).compute_bf16
        assert ac.mul_forward(tagged, tagged).compute_bf16 and not ac.mul_forward(tagged, plain).compute_bf16
        assert ac.residual_add_forward(tagged, tagged).compute_bf16
        assert not ac.residual_add_forward(plain, tagged).compute_bf16
        assert ac.permute(tagged, [0, 2, 1, 3]).compute_bf16 and not ac.permute(plain, [0, 2, 1, 3]).compute_bf16
    assert not ac.silu_forward(tagged).compute_bf16  # outside: never rounded


def test_norms_pass_through_in_f32():
    rec = Recorder()
    ac = Autocast(rec)
    with ac.region():
        h = ac.rms_norm_forward(T("x", tagged=True), T("w"), 1e-6)
    assert not h.compute_bf16 and not ops(rec, "cast")


@pytest.mark.parametrize("out_tagged", [True, False])
def test_attention_backward_recomputes_a_rounded_output(out_tagged):
    """autocast.rs:1200-1236: the row term of the backward needs the unrounded output."""
    rec = Recorder()
    ac = Autocast(rec)
    q, k, v = (T(n, tagged=True) for n in "qkv")
    with ac.region():
        grads = ac.causal_sdpa_backward(q, k, v, T("saved", tagged=out_tagged), T("saved_lse"), T("gy", tagged=True))
    # A rounded output is not used at all: the inner backend's own recompute runs instead.
    assert not ops(rec, "sdpa_forward")
    if out_tagged:
        assert not ops(rec, "sdpa_backward")
        assert ops(rec, "sdpa_backward_recompute")[0][1] == ("q", "k", "v", "gy")
    else:
        assert not ops(rec, "sdpa_backward_recompute")
        assert ops(rec, "sdpa_backward")[0][1][3:5] == ("saved", "saved_lse")
    assert all(g.compute_bf16 for g in grads)


def test_attention_forward_keeps_the_log_sum_exp_in_f32():
    ac = Autocast(Recorder())
    with ac.region():
        out, lse = ac.causal_sdpa_forward(T("q"), T("k"), T("v"))
    assert out.compute_bf16 and not lse.compute_bf16


def test_writers_clear_the_tag():
    ac = Autocast(Recorder())
    acc, g, p = T("acc", tagged=True), T("g", tagged=True), T("p", tagged=True)
    ac.accumulate_grad(acc, T("other"))
    ac.scale_grad(g, 0.5)
    ac.adamw_step(p, T("grad"), T("m1"), T("m2"), 0, None)
    assert not acc.compute_bf16 and not g.compute_bf16 and not p.compute_bf16


def test_regions_nest():
    ac = Autocast(Recorder())
    with ac.region():
        with ac.region():
            assert ac.on
        assert ac.on
    assert not ac.on
