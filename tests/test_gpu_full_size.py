"""The benchmark configurations at their full sizes (BASELINE.json configs[1] and configs[2]).

The CPU oracle finishes one 1024-token sequence of the 124M-parameter model in seconds, not the
whole 16-sequence batch, so the full-size step is pinned in three links:

  1. one sequence through the full model equals the oracle (loss and all 148 gradients);
  2. the 16-sequence step equals the mean of its 16 single-sequence steps (the loss is a mean over
     tokens and sequences do not interact, so this is exact up to the order of f32 sums);
  3. the gradient of the 16-sequence step predicts the change of its own loss along the gradient
     direction (central difference), which a dropped or mis-scaled backward term fails;
  4. the bf16 tier of the 16-sequence step stays within the bf16 tolerance of the f32 tier.

The bf16 tier has no batch-mean identity to the same precision: a rounding to bf16 turns any
difference in an f32 sum's order into whole-ulp flips of a few outputs, and a few roundings later
two runs carry independent rounding noise of the tier's own size (measured: a duplicated sequence
as a batch of two differs from the single sequence by 0.3 to 1.5 % normwise, from 2.5e-5 at the
first product). Each configuration is deterministic run to run.

The attention configuration runs against the oracle directly, with the identities the
mathematics fixes: softmax rows sum to one (constant V comes back unchanged, the columns of dV
sum to the columns of dO) and sum(q * dq) = sum(k * dk) (both are sum(dS * S)).
"""
import numpy as np
import pytest

import oracle_api as orc

pytestmark = pytest.mark.gpu

GPT124M = (12, 768, 12, 64, 3072, 1024, 50304, 16, 0)  # configs[2]


@pytest.fixture(scope="module")
def be():
    from ojas_amd.backend import MiBackend

    backend = MiBackend(0)
    yield backend
    backend.close()


def shape(batch, bf16):
    return GPT124M[:7] + (batch, GPT124M[8], bf16)


@pytest.fixture(scope="module")
def world():
    """Parameters, the 16-sequence batch, and the oracle's step on sequence 0."""
    from ojas_amd.trainer import GptConfig, synthetic_batch

    cfg = GptConfig(*shape(16, 0))
    ocfg = orc.GptConfig(*shape(1, 0)[:9])
    rng = np.random.default_rng(20)
    params = [np.ones(n, np.float32) + rng.normal(0, 0.05, n).astype(np.float32) if n == cfg.d_model
              else rng.normal(0, 0.02, n).astype(np.float32) for n in orc.gpt_param_lens(ocfg)]
    ids, targets = synthetic_batch(cfg, 5)
    print("oracle: one 1024-token sequence through the 124M-shape model", flush=True)
    orc.set_threads(16)
    oloss, ograds = orc.gpt_loss_and_grads(ocfg, params, ids[0], targets[0])
    return params, ids, targets, float(oloss), ograds


def gpu_step(be, batch, bf16, params, ids, targets):
    from ojas_amd.trainer import GptConfig, GptTrainer

    tr = GptTrainer(be, GptConfig(*shape(batch, bf16)))
    tr.set_params(params)
    tr.set_batch(np.ascontiguousarray(ids), np.ascontiguousarray(targets))
    loss = tr.loss_and_grads()
    grads = tr.grads()
    return tr, loss, grads


def test_one_sequence_f32_tier_matches_the_oracle(be, world):
    params, ids, targets, oloss, ograds = world
    tr, loss, grads = gpu_step(be, 1, 0, params, ids[:1], targets[:1])
    tr.close()
    assert abs(loss - oloss) <= 1e-5 * abs(oloss), (loss, oloss)
    for i, (g, og) in enumerate(zip(grads, ograds)):
        d = g.astype(np.float64) - og
        assert np.linalg.norm(d) <= 1e-5 * max(np.linalg.norm(og), 1e-12), (i, np.linalg.norm(d), np.linalg.norm(og))
        assert np.max(np.abs(d)) <= 1e-4 * max(np.max(np.abs(og)), 1e-12), i


def check_bf16_gradients(grads, ref):
    """The bf16 tier's gradient gate, at this depth as for single ops: every element within 2e-2
    of its tensor's largest value (measured at most 1.6e-2, in the query and key projections;
    1.4e-2 elsewhere), and every tensor within 2e-2 normwise (measured 1.4e-2 and 1.1e-2). The
    query and key projections meet it because the attention backward takes its row term from the
    output plus its saved rounding residual; from the bf16 output alone they measured up to
    3.1e-2 per element and 2.1e-2 normwise from the sixth layer on, where the residual stream has
    grown a component common to all positions."""
    for i, (g, r) in enumerate(zip(grads, ref)):
        d = g.astype(np.float64) - r
        assert np.max(np.abs(d)) <= 2e-2 * np.max(np.abs(r)), (i, np.max(np.abs(d)), np.max(np.abs(r)))
        assert np.linalg.norm(d) <= 2e-2 * np.linalg.norm(r), (i, np.linalg.norm(d), np.linalg.norm(r))


def test_one_sequence_bf16_tier_matches_the_oracle(be, world):
    params, ids, targets, oloss, ograds = world
    tr, loss, grads = gpu_step(be, 1, 1, params, ids[:1], targets[:1])
    tr.close()
    assert abs(loss - oloss) <= 1e-3 * abs(oloss), (loss, oloss)
    check_bf16_gradients(grads, ograds)


@pytest.fixture(scope="module")
def full_f32(be, world):
    """The 16 x 1024 step on the f32 tier: loss and gradients."""
    params, ids, targets, _, _ = world
    tr, loss, grads = gpu_step(be, 16, 0, params, ids, targets)
    tr.close()
    return loss, grads


def test_full_batch_is_the_mean_of_its_sequences(be, world, full_f32):
    """Sequences share nothing but the weights: loss and gradients of the batch are the means of
    the single-sequence ones, up to the order of f32 sums. With the single-sequence test above
    this ties the f32 tier of the whole configuration to the oracle."""
    from ojas_amd.trainer import GptConfig, GptTrainer

    params, ids, targets, _, _ = world
    loss16, grads16 = full_f32
    one = GptTrainer(be, GptConfig(*shape(1, 0)))
    one.set_params(params)
    mean_loss = 0.0
    mean = [np.zeros(g.shape, np.float64) for g in grads16]
    for s in range(16):
        one.set_batch(np.ascontiguousarray(ids[s:s + 1]), np.ascontiguousarray(targets[s:s + 1]))
        mean_loss += one.loss_and_grads() / 16
        for acc, g in zip(mean, one.grads()):
            acc += g
    one.close()
    assert abs(loss16 - mean_loss) <= 1e-5 * abs(mean_loss), (loss16, mean_loss)
    for i, (g, m) in enumerate(zip(grads16, mean)):
        m /= 16
        assert np.linalg.norm(g - m) <= 1e-5 * max(np.linalg.norm(m), 1e-12), (i, np.linalg.norm(g - m), np.linalg.norm(m))


def test_full_batch_bf16_tier_within_tolerance_of_the_f32_tier(be, world, full_f32):
    """configs[2] as benchmarked (bf16 operands, f32 accumulation and master weights) against the
    f32 tier of the same step, which the tests above tie to the oracle within 1e-5. Loss within
    1e-3 (measured 3e-6); gradients at the gates of check_bf16_gradients."""
    params, ids, targets, _, _ = world
    loss32, grads32 = full_f32
    tr, loss, grads = gpu_step(be, 16, 1, params, ids, targets)
    tr.close()
    assert abs(loss - loss32) <= 1e-3 * abs(loss32), (loss, loss32)
    check_bf16_gradients(grads, grads32)


def test_loss_curves_of_the_two_tiers_stay_together(be, world):
    """AdamW (lr 3e-4, betas 0.9/0.95, weight decay 0.1, clip 1.0) on the fixed 16 x 1024 batch: the
    bf16 tier's loss follows the f32 tier's within 1e-2 nats over the first 12 steps (measured at
    most 2.8e-3 while the loss falls by 2.7 nats), and over 50 steps it keeps falling and ends far
    more than the reference's minimum drop of 1 nat below ln V (ojas-oracle/src/parity.rs:58)."""
    from ojas_amd.backend import AdamWConfig
    from ojas_amd.trainer import GptConfig, GptTrainer

    params, ids, targets, _, _ = world
    cfg = AdamWConfig.nanolab(3e-4, 0.1)
    curves = {}
    for bf16, steps in ((0, 12), (1, 50)):
        tr = GptTrainer(be, GptConfig(*shape(16, bf16)))
        tr.set_params(params)
        tr.set_batch(ids, targets)
        curves[bf16] = np.array([tr.step(cfg, 1.0)[0] for _ in range(steps)])
        tr.close()
    gap = np.abs(curves[1][:12] - curves[0])
    assert np.max(gap) <= 1e-2, gap
    assert np.all(np.diff(curves[0]) < 0) and np.all(np.diff(curves[1][:12]) < 0)
    assert curves[1][-1] < np.log(GPT124M[6]) - 1.0 and curves[1][-1] < curves[1][25] < curves[1][12]


def test_full_batch_gradient_predicts_the_loss_along_itself(be, world, full_f32):
    """L(p + e g) - L(p - e g) = 2 e |g|^2 + O(e^3): the f32-tier backward of the whole
    16 x 1024 step against its own forward. The cubic term is 4.5e-4 of the first-order one at
    this step size (it falls fourfold when the step halves)."""
    from ojas_amd.trainer import GptConfig, GptTrainer

    params, ids, targets, _, _ = world
    loss, grads = full_f32
    sq = sum(float(np.sum(g.astype(np.float64) ** 2)) for g in grads)
    eps = 0.005 / sq  # a first-order change of 0.005 each way on a loss of about 10.98
    tr = GptTrainer(be, GptConfig(*shape(16, 0)))
    tr.set_batch(ids, targets)
    losses = []
    for sign in (1.0, -1.0):
        tr.set_params([p + np.float32(sign * eps) * g for p, g in zip(params, grads)])
        losses.append(tr.loss_and_grads())
    tr.close()
    measured = losses[0] - losses[1]
    assert abs(measured - 2 * eps * sq) <= 2e-3 * 2 * eps * sq, (measured, 2 * eps * sq, loss)
    assert losses[1] < loss < losses[0]


def test_attention_configuration_at_full_size(be):
    """configs[1]: B=8, H=12, T=1024, head_dim 64, bf16 operands, f32 accumulation."""
    from ojas_amd.backend import BF16, F32

    b, h, t, d = 8, 12, 1024, 64
    r = orc.SplitMix64(77)
    mk = lambda: orc.round_bf16(r.vec(b * h * t * d, 1.0)).reshape(b, h, t, d)
    q, k, v, gy = mk(), mk(), mk(), mk()
    print("oracle: attention 8 x 12 x 1024 x 64 forward and backward", flush=True)
    orc.set_threads(16)
    oy, olse = orc.causal_sdpa_forward(q, k, v, 0)
    oy16 = orc.round_bf16(oy)
    ogq, ogk, ogv = orc.causal_sdpa_backward(q, k, v, oy16, olse, gy, 0)
    dq, dk, dv, dgy = (be.upload(a, BF16) for a in (q, k, v, gy))
    y, lse = be.causal_sdpa_forward(dq, dk, dv, None, out_dtype=F32)
    y, lse = be.download(y), be.download(lse)
    assert np.max(np.abs(y - oy)) <= 1e-2 * np.max(np.abs(oy))
    assert np.max(np.abs(lse - olse)) <= 1e-5 * np.max(np.abs(olse))
    gq, gk, gv = be.causal_sdpa_backward(dq, dk, dv, be.upload(oy16, BF16), be.upload(olse), dgy, None, grad_dtype=F32)
    gq, gk, gv = be.download(gq), be.download(gk), be.download(gv)
    for name, got, want in (("gq", gq, ogq), ("gk", gk, ogk), ("gv", gv, ogv)):
        assert np.max(np.abs(got - want)) <= 2e-2 * np.max(np.abs(want)), name
    # Rows of the softmax sum to one: the columns of dV sum to the columns of dO ...
    f64 = lambda a: a.astype(np.float64)
    want = f64(gy).sum(axis=2)
    assert np.max(np.abs(f64(gv).sum(axis=2) - want)) <= 2e-3 * np.max(np.abs(want))
    # ... and dS * S summed either way: sum(q dq) = sum(k dk), per head.
    lhs, rhs = (f64(q) * f64(gq)).sum(axis=(2, 3)), (f64(k) * f64(gk)).sum(axis=(2, 3))
    assert np.max(np.abs(lhs - rhs)) <= 2e-3 * np.max(np.abs(lhs)), (lhs.ravel()[:3], rhs.ravel()[:3])
    # A constant value row comes back unchanged from every position.
    const = np.broadcast_to(orc.round_bf16(r.vec(d, 1.0)), (b, h, t, d)).copy()
    yc, _ = be.causal_sdpa_forward(dq, dk, be.upload(const, BF16), None, out_dtype=F32)
    assert np.max(np.abs(be.download(yc) - const)) <= 2e-3 * np.max(np.abs(const))
