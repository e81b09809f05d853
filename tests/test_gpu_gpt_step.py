"""GPT-2-shaped training step on the GPU against the CPU oracle's composed step.

Gates (BASELINE.json north_star; the reference's whole-model gates are of the
same kind, ojas-oracle/src/parity.rs:29-74):
  * f32 tier: loss relative 1e-5; every gradient normwise
    max|gpu - cpu| <= 1e-5 * max|cpu| is too tight for a 4-layer chain of
    re-ordered f32 sums, so gradients use the reference's own normwise gate
    form with 1e-5 applied to the l2 norm: ||gpu - cpu|| <= 1e-5 * ||cpu||
    is checked first and the per-element bound 1e-4 * max|cpu| second (the
    reference's GPU-vs-CPU op gate, ojas-wgpu/tests/common/mod.rs:11).
  * bf16 tier: loss relative 1e-3; gradients 2e-2 per element relative to max|cpu|.
"""
import numpy as np
import pytest

import oracle_api as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    from ojas_amd.backend import MiBackend

    backend = MiBackend(0)
    yield backend
    backend.close()


def make_params(lens, d_model, seed, std=0.02):
    rng = np.random.default_rng(seed)
    return [np.ones(n, np.float32) + rng.normal(0, 0.05, n).astype(np.float32) if n == d_model
            else rng.normal(0, std, n).astype(np.float32) for n in lens]


def run_case(be, cfg_tuple, seed, std=0.02):
    from ojas_amd.trainer import GptConfig, GptTrainer, synthetic_batch

    cfg = GptConfig(*cfg_tuple)
    tr = GptTrainer(be, cfg)
    lens = tr.param_lens()
    ocfg = orc.GptConfig(*cfg_tuple[:9])
    assert lens == orc.gpt_param_lens(ocfg)
    params = make_params(lens, cfg.d_model, seed, std)
    ids, targets = synthetic_batch(cfg, seed)
    tr.set_params(params)
    tr.set_batch(ids, targets)
    loss = tr.loss_and_grads()
    grads = tr.grads()
    orc.set_threads(8)
    oloss, ograds = orc.gpt_loss_and_grads(ocfg, params, ids.reshape(-1), targets.reshape(-1))
    return tr, params, (loss, grads), (float(oloss), ograds)


TINY = (2, 32, 2, 16, 64, 16, 50, 2, 0)
SMALL = (2, 128, 2, 64, 256, 70, 300, 3, 1)  # head_dim 64, ragged T, tanh GELU
C1 = (4, 256, 4, 64, 1024, 256, 8192, 8, 0)  # BASELINE configs[0]


@pytest.mark.parametrize("shape,std", [(TINY, 0.2), (SMALL, 0.05), (C1, 0.02)])
def test_f32_tier_step_matches_cpu_exact(be, shape, std):
    print(f"gpt f32 {shape}", flush=True)
    tr, params, (loss, grads), (oloss, ograds) = run_case(be, shape + (0,), 7, std)
    assert abs(loss - oloss) <= 1e-5 * abs(oloss), (loss, oloss)
    for i, (g, og) in enumerate(zip(grads, ograds)):
        g64, og64 = g.astype(np.float64), og.astype(np.float64)
        norm = np.linalg.norm(og64)
        assert np.linalg.norm(g64 - og64) <= 1e-5 * max(norm, 1e-12), (i, np.linalg.norm(g64 - og64), norm)
        assert np.max(np.abs(g64 - og64)) <= 1e-4 * max(np.max(np.abs(og64)), 1e-12), i
    tr.close()


ONE_LAYER = (1,) + SMALL[1:]  # weight gradients inside the layer loop; two layers and more batch them at the end


@pytest.mark.parametrize("shape,std", [(SMALL, 0.05), (ONE_LAYER, 0.05), (C1, 0.02)])
def test_bf16_tier_step_within_bf16_tolerance_of_cpu_exact(be, shape, std):
    print(f"gpt bf16 {shape}", flush=True)
    tr, params, (loss, grads), (oloss, ograds) = run_case(be, shape + (1,), 11, std)
    assert abs(loss - oloss) <= 1e-3 * abs(oloss), (loss, oloss)
    for i, (g, og) in enumerate(zip(grads, ograds)):
        err = np.max(np.abs(g.astype(np.float64) - og.astype(np.float64)))
        assert err <= 2e-2 * max(np.max(np.abs(og)), 1e-12), (i, err, np.max(np.abs(og)))
    tr.close()


def test_optimizer_step_matches_cpu_adamw_on_the_same_gradients(be):
    from ojas_amd.backend import AdamWConfig

    tr, params, (loss, grads), (oloss, ograds) = run_case(be, SMALL + (0,), 3, 0.05)
    cfg = AdamWConfig.nanolab(3e-4, 0.1)
    step_loss, norm = tr.step(cfg, grad_clip=1.0)
    assert abs(step_loss - oloss) <= 1e-5 * abs(oloss)
    onorm, clipped = orc.clip_grad_norm(ograds, 1.0)
    assert abs(norm - float(onorm)) <= 1e-5 * float(onorm)
    after = tr.params()
    for i, (p, g) in enumerate(zip(params, clipped)):
        want, _, _ = orc.adamw_step(p, g, np.zeros_like(p), np.zeros_like(p), 0, 3e-4, 0.9, 0.95, 1e-8, 0.1, exact=True)
        # AdamW's first step moves a weight by lr * g / (|g| + eps): about lr where the gradient
        # is well above eps, and anywhere in [-lr, lr] where the gradient itself is at the level
        # of the allowed gradient error. The tight bound applies to the former only.
        diff = np.abs(after[i] - want)
        solid = np.abs(g) > 1e-3 * max(np.max(np.abs(g)), 1e-12)
        assert np.max(diff[solid], initial=0.0) <= 1e-2 * 3e-4, (i, np.max(diff[solid], initial=0.0))
        assert np.max(diff, initial=0.0) <= 2.1 * 3e-4, (i, np.max(diff))
    assert tr.steps() == 1
    # The loss goes down over a few steps on a fixed batch.
    losses = [tr.step(cfg, 1.0)[0] for _ in range(10)]
    assert losses[-1] < step_loss
    tr.close()


def test_steps_with_the_skipped_adamw_check_equal_steps_with_it(be):
    """The trainer vouches for its arenas once a step has passed over them (omx_adamw_step_bounded);
    the parameters after five steps are bit for bit those of a trainer that checks every time,
    across a parameter written from outside in between (which ends the trainer's word until the
    next checked step). The flag itself is covered with the op, in test_gpu_parity_ops.py."""
    from ojas_amd.backend import AdamWConfig
    from ojas_amd.trainer import GptConfig, GptTrainer, synthetic_batch

    cfg = GptConfig(*SMALL, 1)
    adam = AdamWConfig.nanolab(3e-3, 0.1)
    ids, targets = synthetic_batch(cfg, 9)
    results = []
    for trust in (1, 0):
        be.set_option("adamw_trust", trust)
        tr = GptTrainer(be, cfg)
        params = make_params(tr.param_lens(), cfg.d_model, 5, 0.05)
        tr.set_params(params)
        tr.set_batch(ids, targets)
        losses = [tr.step(adam, 1.0) for _ in range(3)]
        planted = tr.params()
        planted[3][7] = 0.5
        tr.set_params(planted)
        losses += [tr.step(adam, 1.0) for _ in range(2)]
        results.append((losses, tr.params()))
        tr.close()
    be.set_option("adamw_trust", 1)
    assert results[0][0] == results[1][0]
    assert all(np.array_equal(a, b) for a, b in zip(results[0][1], results[1][1]))


@pytest.mark.parametrize("hybrid", [False, True])
def test_a_trainer_resumed_from_exported_state_takes_the_same_steps(be, hybrid):
    """Parameters, both state slots and the step count carried into a fresh trainer
    (`ogpt_get_state` / `ogpt_set_state` / `ogpt_set_steps`) give, bit for bit, the steps the first
    trainer goes on to take."""
    from ojas_amd.backend import AdamWConfig, MuonNs5Config
    from ojas_amd.trainer import GptConfig, GptTrainer, synthetic_batch

    cfg = GptConfig(*SMALL, 1)
    adam = AdamWConfig.nanolab(3e-3, 0.1)
    muon = MuonNs5Config(0.02, 0.95, 0.1, 1, 1)
    ids, targets = synthetic_batch(cfg, 21)

    def step(tr):
        return tr.step_hybrid(muon, adam, 1.0) if hybrid else tr.step(adam, 1.0)

    first = GptTrainer(be, cfg)
    first.set_params(make_params(first.param_lens(), cfg.d_model, 6, 0.05))
    first.set_batch(ids, targets)
    for _ in range(3):
        step(first)
    params, m1, m2, steps = first.params(), first.state(0), first.state(1), first.steps()
    assert steps == 3 and any(np.any(m != 0) for m in m1)
    second = GptTrainer(be, cfg)
    second.set_params(params)
    second.set_state(0, m1)
    second.set_state(1, m2)
    second.set_steps(steps)
    second.set_batch(ids, targets)
    for _ in range(2):
        assert step(first) == step(second)
    assert second.steps() == 5
    assert all(np.array_equal(a, b) for a, b in zip(first.params(), second.params()))
    assert all(np.array_equal(a, b) for a, b in zip(first.state(1), second.state(1)))
    first.close()
    second.close()


def hybrid_expectation(params, grads, d, mlp, bf16, lr_adamw):
    """The oracle's hybrid update of every parameter from `grads` (already clipped): Muon-NS5 on the
    six hidden matrices of a layer, AdamW on tables and norms. Returns [(kind, want)]."""
    out = []
    for i, (p, g) in enumerate(zip(params, grads)):
        in_layer = 2 <= i < len(params) - 1
        which = (i - 2) % 8 if in_layer else -1
        if which in (1, 2, 3, 4, 6, 7):
            shape = (d, d) if which <= 4 else ((mlp, d) if which == 6 else (d, mlp))
            want, _ = orc.muon_ns5_step(p.reshape(shape), g.reshape(shape), np.zeros(shape, np.float32), lr=0.02,
                                        momentum=0.95, weight_decay=0.1, nesterov=True, bf16=bool(bf16))
            out.append(("muon", want.reshape(-1).astype(np.float64)))
        else:
            want, _, _ = orc.adamw_step(p, g, np.zeros_like(p), np.zeros_like(p), 0, lr_adamw, 0.9, 0.95, 1e-8, 0.0,
                                        exact=True)
            out.append(("adamw", want.reshape(-1).astype(np.float64)))
    return out


@pytest.mark.parametrize("bf16", [0, 1])
def test_hybrid_step_muon_on_matrices_adamw_on_tables_and_norms(be, bf16):
    """BASELINE configs[3]'s optimizer on a small shape: `ogpt_step_hybrid` against the oracle's
    clip + `muon_ns5_step` per hidden matrix + `adamw_step` per table / norm.

    The optimizer is checked on the device's OWN gradients (read back before the step, which
    recomputes the same ones bit for bit), so the gates are the optimizer's, not the backward
    pass's: every Muon update (new - old) within 1e-3 normwise of the oracle's in the f32 tier and
    5e-2 in the bf16 tier (the reference's gate for the bf16 iteration, ojas-oracle/src/parity.rs:42-52:
    the iteration rounds to bf16 at every product, and a wrong Newton-Schulz scale, a missing
    Nesterov term or a dropped weight decay are each far outside it); every AdamW element whose
    gradient is well above eps within 1 % of lr of the oracle's (a first step moves such an element
    by lr, so a no-op is off by lr and a wrong sign by 2 lr). The backward pass itself is held to
    the oracle's gradients at the tier's tolerance through the loss and the gradient norm."""
    from ojas_amd.backend import AdamWConfig, MuonNs5Config

    print(f"hybrid step bf16={bf16}", flush=True)
    tr, params, (_, dev_grads), (oloss, ograds) = run_case(be, SMALL + (bf16,), 5, 0.05)
    muon = MuonNs5Config(0.02, 0.95, 0.1, 1, bf16)
    lr = 3e-4
    adamw = AdamWConfig.nanolab(lr, 0.0)
    step_loss, norm = tr.step_hybrid(muon, adamw, grad_clip=1.0)
    assert abs(step_loss - oloss) <= (1e-3 if bf16 else 1e-5) * abs(oloss)
    onorm, _ = orc.clip_grad_norm(ograds, 1.0)
    assert abs(norm - float(onorm)) <= (2e-2 if bf16 else 1e-5) * float(onorm)
    dnorm, clipped = orc.clip_grad_norm(dev_grads, 1.0)
    assert abs(norm - float(dnorm)) <= 1e-5 * float(dnorm)
    after = tr.params()
    worst = {"muon": 0.0, "adamw": 0.0}
    for i, ((kind, want), p, g) in enumerate(zip(hybrid_expectation(params, clipped, SMALL[1], SMALL[4], bf16, lr),
                                                 params, clipped)):
        if kind == "muon":
            rel = np.linalg.norm(after[i] - want) / np.linalg.norm(want - p)
            worst[kind] = max(worst[kind], rel)
            assert rel <= (5e-2 if bf16 else 1e-3), (i, kind, rel)
        else:
            diff = np.abs(after[i] - want)
            solid = np.abs(g) > 1e-3 * max(np.max(np.abs(g)), 1e-12)
            assert np.any(solid), i
            worst[kind] = max(worst[kind], float(np.max(diff[solid])) / lr)
            assert np.max(diff[solid]) <= 1e-2 * lr, (i, float(np.max(diff[solid])) / lr)
            assert np.max(diff) <= 2.1 * lr, i
    print("worst update distance (muon: normwise relative; adamw: in units of lr)", worst, flush=True)
    losses = [tr.step_hybrid(muon, adamw, 1.0)[0] for _ in range(8)]
    assert losses[-1] < step_loss and tr.steps() == 9
    tr.close()
