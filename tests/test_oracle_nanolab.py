"""The oracle's nanolab-GPT graph and bf16 Muon step against the reference's torch fixtures
(ojas-oracle/fixtures/tiny, gates of ojas-oracle/src/parity.rs:28-40 and
ojas-oracle/tests/ojas_cpu_parity.rs:100-160), plus f64 central differences for the gradient paths the
zero-initialised projections hide at the seeded init."""
import json
from pathlib import Path

import numpy as np
import pytest
from safetensors import safe_open

import oracle_api as orc

TINY = Path(__file__).parent / "golden" / "tiny"

FORWARD_LOSS_REL_TOL = 1e-5  # ojas-oracle/src/parity.rs:29
LOGITS_NORMWISE_REL_TOL = 1e-5  # :32
GRAD_NORMWISE_REL_TOL = 1e-4  # :35


def load(name):
    with safe_open(str(TINY / f"{name}.safetensors"), "np") as f:
        meta = {k: json.loads(v) for k, v in (f.metadata() or {}).items()}
        return {k: f.get_tensor(k) for k in f.keys()}, meta


def tiny_config(batch, seq):
    _, meta = load("init")
    spec = meta["ojas.spec"]
    return orc.NanolabConfig(layers=spec["n_layer"], n_embd=spec["n_embd"], n_head=spec["n_head"],
                             n_kv_head=spec["n_kv_head"], head_dim=spec["head_dim"], hidden=spec["hidden"],
                             vocab=spec["vocab"], batch=batch, seq=seq, window=0, rms_eps=spec["rms_eps"],
                             rope_base=spec["rope_base"])


def test_forward_loss_and_logits_match_the_torch_fixture():
    init, _ = load("init")
    fwd, meta = load("forward")
    ids, targets = fwd["x"].astype(np.uint32), fwd["y"].astype(np.uint32)
    cfg = tiny_config(*ids.shape)
    params = [init[n] for n in orc.nanolab_param_names(cfg.layers)]
    loss, logits, _ = orc.nanolab_loss_and_grads(cfg, params, ids, targets, want_logits=True, want_grads=False)
    want_loss = meta["ojas.oracle"]["loss"]
    assert abs(float(loss) - want_loss) <= FORWARD_LOSS_REL_TOL * abs(want_loss)
    want = fwd["logits"].reshape(-1, cfg.vocab).astype(np.float64)
    rel = np.linalg.norm(logits - want) / np.linalg.norm(want)
    assert rel <= LOGITS_NORMWISE_REL_TOL, rel


def test_gradients_at_the_init_match_the_torch_fixture():
    init, _ = load("init")
    fwd, _ = load("forward")
    want, meta = load("grads_init")
    info = meta["ojas.oracle"]
    ids, targets = fwd["x"].astype(np.uint32), fwd["y"].astype(np.uint32)
    cfg = tiny_config(*ids.shape)
    names = orc.nanolab_param_names(cfg.layers)
    loss, _, grads = orc.nanolab_loss_and_grads(cfg, [init[n] for n in names], ids, targets)
    assert abs(float(loss) - info["loss"]) <= FORWARD_LOSS_REL_TOL * info["loss"]
    seed = np.float32(info["loss_seed"])  # the fixture's backward starts from this instead of 1
    checked = 0
    for name, g in zip(names, grads):
        if name in info["no_grad"]:
            assert not np.any(g), name
            continue
        got = (g * seed).astype(np.float64)
        ref = want[name].reshape(-1).astype(np.float64)
        if name in info["zero_grad"]:
            assert not np.any(ref) and not np.any(got), f"{name}: torch's gradient is exactly zero"
            continue
        rel = np.linalg.norm(got - ref) / np.linalg.norm(ref)
        assert rel <= GRAD_NORMWISE_REL_TOL, (name, rel)
        checked += 1
    # o_proj and ffn.down of both blocks, norm_f, tok_emb: these hold the whole attention and
    # SwiGLU forward (RoPE, q/k norm, blend, gate, SiLU, product) in their values.
    assert checked == 6


def test_every_gradient_path_against_f64_central_differences():
    # At the init o_proj and ffn.down are zero, so most backward paths carry zeros. Random
    # projections make every path live; the check is directional: (L(p + h u) - L(p - h u)) / 2h
    # against <grad, u>, with the loss evaluated by the oracle and differenced in f64.
    r = orc.SplitMix64(2024)
    cfg = orc.NanolabConfig(layers=3, n_embd=32, n_head=4, n_kv_head=2, head_dim=8, hidden=48, vocab=64, batch=2,
                            seq=12, window=0, rms_eps=1e-6, rope_base=10000.0)
    names = orc.nanolab_param_names(cfg.layers)
    lens = orc.nanolab_param_lens(cfg)
    params = []
    for name, n in zip(names, lens):
        if name.endswith("norm.weight") or "norm" in name.split(".")[-2]:
            params.append(1.0 + r.vec(n, 0.2))
        elif name.endswith("vr_lambda"):
            params.append(r.vec(n, 1.0))
        elif name.endswith("gate.bias"):
            params.append(r.vec(n, 0.5))
        else:
            params.append(r.vec(n, 0.3))
    ids = np.array([r.below(cfg.vocab) for _ in range(cfg.batch * cfg.seq)], np.uint32).reshape(cfg.batch, cfg.seq)
    targets = np.array([r.below(cfg.vocab) for _ in range(cfg.batch * cfg.seq)], np.uint32).reshape(cfg.batch, cfg.seq)
    _, _, grads = orc.nanolab_loss_and_grads(cfg, params, ids, targets)
    assert not np.any(grads[names.index("blocks.0.mixer.vr_lambda")])
    h = 2e-3
    for i, name in enumerate(names):
        if name == "blocks.0.mixer.vr_lambda":
            continue
        # Half along the gradient (so the derivative is well above the f32 noise of the loss), half
        # a random direction (so a term dropped from the gradient cannot hide in its null space).
        u = r.vec(lens[i], 1.0)
        u = u / np.linalg.norm(u) + grads[i] / max(float(np.linalg.norm(grads[i])), 1e-30)
        u = (u / np.linalg.norm(u)).astype(np.float32)
        plus = [p.copy() for p in params]
        minus = [p.copy() for p in params]
        plus[i] = (params[i] + h * u).astype(np.float32)
        minus[i] = (params[i] - h * u).astype(np.float32)
        lp, _, _ = orc.nanolab_loss_and_grads(cfg, plus, ids, targets, want_grads=False)
        lm, _, _ = orc.nanolab_loss_and_grads(cfg, minus, ids, targets, want_grads=False)
        step = float(np.linalg.norm(plus[i].astype(np.float64) - minus[i]))
        numeric = (float(lp) - float(lm)) / step
        analytic = float(np.dot(grads[i].astype(np.float64), u))
        # f32 losses differ by ~1e-7 relative: the quotient is good to ~1e-4 absolute at this step.
        assert abs(numeric - analytic) <= 3e-4 + 2e-2 * abs(analytic), (name, numeric, analytic)


def test_window_and_grouped_heads_change_the_result_the_way_the_mask_says():
    # seq <= window is the full causal mask.
    r = orc.SplitMix64(77)
    base = dict(layers=1, n_embd=16, n_head=4, n_kv_head=2, head_dim=4, hidden=24, vocab=32, batch=1, seq=10,
                rms_eps=1e-6, rope_base=10000.0)
    cfg_full, cfg_wide, cfg_narrow = (orc.NanolabConfig(window=w, **base) for w in (0, 10, 3))
    lens = orc.nanolab_param_lens(cfg_full)
    params = [r.vec(n, 0.4) for n in lens]
    ids = np.array([r.below(32) for _ in range(10)], np.uint32).reshape(1, 10)
    full = orc.nanolab_loss_and_grads(cfg_full, params, ids, ids, want_grads=False)[0]
    wide = orc.nanolab_loss_and_grads(cfg_wide, params, ids, ids, want_grads=False)[0]
    narrow = orc.nanolab_loss_and_grads(cfg_narrow, params, ids, ids, want_grads=False)[0]
    assert full == wide and full != narrow


def test_rope_tables_have_matching_halves_and_unit_norm():
    cos, sin = orc.rope_tables(33, 16, 10000.0)
    assert np.array_equal(cos[:, :8], cos[:, 8:]) and np.array_equal(sin[:, :8], sin[:, 8:])
    assert np.all(cos[0] == 1.0) and np.all(sin[0] == 0.0)
    np.testing.assert_allclose(cos.astype(np.float64) ** 2 + sin.astype(np.float64) ** 2, 1.0, atol=2e-7)
    pos, i = 7, 3
    assert abs(cos[pos, i] - np.cos(pos * 10000.0 ** (-2 * i / 16))) < 1e-7


def test_bf16_muon_step_is_stock_nanolab_bit_for_bit():
    # ojas-oracle/tests/ojas_cpu_parity.rs:112-160: momentum and parameter bits equal torch's; the
    # f32 iteration is the contrast and must be off by more than 1% of the update.
    data, meta = load("muon_step_bf16")
    cases = meta["ojas.oracle"]["cases"]
    assert len(cases) == 4
    for i, case in enumerate(cases):
        p, g, m = (data[f"c{i}.{k}"] for k in ("p", "g", "m"))
        assert p.shape == (case["rows"], case["cols"])
        kw = dict(lr=case["lr"], momentum=case["momentum"], weight_decay=case["weight_decay"],
                  nesterov=case["nesterov"])
        p2, m2 = orc.muon_ns5_step(p.copy(), g, m.copy(), bf16=True, **kw)
        assert np.array_equal(m2.view(np.uint32), data[f"c{i}.m_after"].view(np.uint32)), f"case {i}: momentum"
        differ = int(np.count_nonzero(p2.view(np.uint32) != data[f"c{i}.p_after"].view(np.uint32)))
        assert differ == 0, f"case {i}: {differ} parameter values differ from torch's"
        p32, _ = orc.muon_ns5_step(p.copy(), g, m.copy(), bf16=False, **kw)
        want = data[f"c{i}.p_after"].astype(np.float64) - p
        rel32 = np.linalg.norm((p32.astype(np.float64) - p) - want) / np.linalg.norm(want)
        assert rel32 > 1e-2, f"case {i}: the f32 contrast is too close ({rel32:.2e}) to tell"


def test_trainer_steps_follow_the_torch_trace():
    """Micro-batch accumulation, the global clip, Muon-NS5 in f32 and AdamW, composed the way
    `Trainer::run` composes them, against the reference's torch trace: per-step mean loss within
    1e-4 nats, gradient norm 1e-4 relative, every parameter after step 5 within 1e-4 normwise
    (ojas-oracle/src/parity.rs:36-41, :468-470). Then the gradients at those parameters against
    `grads_step5` at the gradient gate. The loop goes on to step 40 and the whole loss curve is held to
    the reference's curve gates (2e-4 nats for the first ten steps, 2e-3 after; it must end a nat
    below ln V)."""
    import trace_fixture as tf

    trace = tf.Trace()
    init, _ = load("init")
    cfg = tiny_config(trace.batch, trace.seq)
    names = orc.nanolab_param_names(cfg.layers)
    frozen = {"blocks.0.mixer.vr_lambda"}
    params = {n: np.ascontiguousarray(init[n], np.float32) for n in names}
    state = {n: [np.zeros_like(params[n]), np.zeros_like(params[n])] for n in names}
    weight = np.float32(1.0 / trace.accum)
    losses, norms = [], []
    after_five = None
    for step in range(len(trace.mean_loss)):
        acc, loss_sum = None, np.float32(0)
        for micro in range(trace.accum):
            ids, targets = trace.micro(step, micro)
            loss, _, grads = orc.nanolab_loss_and_grads(cfg, [params[n].reshape(-1) for n in names], ids, targets)
            micro_tol = (tf.TRACE_LOSS_ABS_TOL if step < trace.steps else
                         tf.CURVE_EARLY_ABS_TOL if step < tf.CURVE_EARLY_STEPS else tf.CURVE_LATE_ABS_TOL)
            assert abs(float(loss) - trace.micro_loss[step * trace.accum + micro]) <= micro_tol, (step, micro)
            grads = [np.asarray(g, np.float32) * weight for g in grads]
            acc = grads if acc is None else [a + g for a, g in zip(acc, grads)]
            loss_sum = np.float32(loss_sum + np.float32(loss))
        live = [n for n in names if n not in frozen]
        norm, clipped = orc.clip_grad_norm([acc[names.index(n)] for n in live], trace.cfg["grad_clip"])
        mult = trace.lr_mult[step]
        for n, g in zip(live, clipped):
            shape = params[n].shape
            if tf.optimizer_of(n, shape) == "muon":
                p, m = orc.muon_ns5_step(params[n], g.reshape(shape), state[n][0], lr=trace.cfg["matrix_lr"] * mult,
                                         momentum=tf.MUON_MOMENTUM, weight_decay=tf.MUON_WEIGHT_DECAY, nesterov=True)
                params[n], state[n][0] = p, m
            else:
                p, m, v = orc.adamw_step(params[n].reshape(-1), g.reshape(-1), state[n][0].reshape(-1),
                                         state[n][1].reshape(-1), step, trace.cfg["lr"] * mult, trace.cfg["beta1"],
                                         trace.cfg["beta2"], trace.cfg["eps"], tf.ADAM_HYBRID_WEIGHT_DECAY)
                params[n], state[n] = p.reshape(shape), [m.reshape(shape), v.reshape(shape)]
        losses.append(float(loss_sum) / trace.accum)
        norms.append(float(norm))
        if step + 1 == trace.steps:
            after_five = {n: params[n].copy() for n in names}
    worst = tf.check_trace(trace, losses, norms, after_five, frozen)
    print(f"worst parameter distance after step {trace.steps}: {worst:.2e}")
    # All 40 steps of the curve, at the reference's curve gates (parity.rs:52-58).
    print(f"worst loss distance over 40 steps: {tf.check_curve(trace, losses, cfg.vocab):.2e}")

    want, gmeta = load("grads_step5")
    info = gmeta["ojas.oracle"]
    ids, targets = trace.micro(0, 0)
    at = {n: np.ascontiguousarray(trace.params_after[n], np.float32) for n in names}
    loss, _, grads = orc.nanolab_loss_and_grads(cfg, [at[n].reshape(-1) for n in names], ids, targets)
    assert abs(float(loss) - info["loss"]) <= FORWARD_LOSS_REL_TOL * abs(info["loss"])
    seed = np.float32(info["loss_seed"])
    for n, g in zip(names, grads):
        if n in info["no_grad"]:
            continue
        ref = want[n].reshape(-1).astype(np.float64)
        assert n not in info["zero_grad"], "after five steps no gradient is exactly zero"
        rel = np.linalg.norm(np.asarray(g, np.float64) * seed - ref) / np.linalg.norm(ref)
        assert rel <= GRAD_NORMWISE_REL_TOL, (n, rel)
