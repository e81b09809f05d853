"""The nanolab GPT graph on the GPU, op by op through the C ABI (`ojas_amd/nanolab.py`), against the
reference's torch fixtures at the gates it holds its own device backends to
(ojas-model/tests/oracle_parity.rs:60-92: GPU_GATES = Gates::EXACT for these quantities; constants
ojas-oracle/src/parity.rs:28-40), and against the CPU oracle on parameters that keep every gradient
path live."""
import json
from pathlib import Path

import numpy as np
import pytest
from safetensors import safe_open

import oracle_api as orc

pytestmark = pytest.mark.gpu

TINY = Path(__file__).parent / "golden" / "tiny"
FORWARD_LOSS_REL_TOL = 1e-5
LOGITS_NORMWISE_REL_TOL = 1e-5
GRAD_NORMWISE_REL_TOL = 1e-4


@pytest.fixture(scope="module")
def be():
    from ojas_amd.backend import MiBackend

    backend = MiBackend(0)
    yield backend
    backend.close()


def load(name):
    with safe_open(str(TINY / f"{name}.safetensors"), "np") as f:
        meta = {k: json.loads(v) for k, v in (f.metadata() or {}).items()}
        return {k: f.get_tensor(k) for k in f.keys()}, meta


def tiny_spec():
    from ojas_amd.nanolab import NanolabSpec

    _, meta = load("init")
    s = meta["ojas.spec"]
    return NanolabSpec(n_layer=s["n_layer"], n_embd=s["n_embd"], n_head=s["n_head"], n_kv_head=s["n_kv_head"],
                       head_dim=s["head_dim"], hidden=s["hidden"], vocab=s["vocab"], rms_eps=s["rms_eps"],
                       rope_base=s["rope_base"])


def run(be, spec, host_params, ids, targets, want_logits=False):
    from ojas_amd.nanolab import NanolabGraph

    shapes = spec.param_shapes()
    params = {n: be.upload(np.ascontiguousarray(host_params[n], np.float32).reshape(shapes[n]))
              for n in spec.param_names()}
    graph = NanolabGraph(be, spec, params)
    loss, logits, grads = graph.loss_and_grads(be.upload(ids.astype(np.uint32)), be.upload(targets.astype(np.uint32)),
                                               want_logits)
    return (float(be.download(loss)[0]), None if logits is None else be.download(logits),
            {n: be.download(g) for n, g in grads.items()})


def test_tiny_fixture_forward_and_gradients(be):
    print("nanolab tiny fixture on the device", flush=True)
    spec = tiny_spec()
    init, _ = load("init")
    fwd, fmeta = load("forward")
    want, gmeta = load("grads_init")
    info = gmeta["ojas.oracle"]
    loss, logits, grads = run(be, spec, init, fwd["x"], fwd["y"], want_logits=True)
    want_loss = fmeta["ojas.oracle"]["loss"]
    assert abs(loss - want_loss) <= FORWARD_LOSS_REL_TOL * abs(want_loss), (loss, want_loss)
    ref = fwd["logits"].reshape(-1, spec.vocab).astype(np.float64)
    rel = np.linalg.norm(logits.reshape(ref.shape) - ref) / np.linalg.norm(ref)
    assert rel <= LOGITS_NORMWISE_REL_TOL, rel
    seed = np.float32(info["loss_seed"])
    checked = 0
    for name in spec.param_names():
        got = grads[name].reshape(-1)
        if name in info["no_grad"]:
            assert not np.any(got), name
            continue
        ref = want[name].reshape(-1).astype(np.float64)
        if name in info["zero_grad"]:
            assert not np.any(ref) and not np.any(got), f"{name}: torch's gradient is exactly zero"
            continue
        rel = np.linalg.norm(got * seed - ref) / np.linalg.norm(ref)
        assert rel <= GRAD_NORMWISE_REL_TOL, (name, rel)
        checked += 1
    assert checked == 6


@pytest.mark.parametrize("kv_heads,window", [(4, None), (2, None), (1, 7)])
def test_every_gradient_against_the_oracle(be, kv_heads, window):
    """Random parameters (o_proj and ffn.down not zero), grouped heads and a window: loss 1e-5
    relative, every gradient 1e-4 normwise against CPU Exact, the reference's device gates."""
    from ojas_amd.nanolab import NanolabSpec

    print(f"nanolab vs oracle kv_heads={kv_heads} window={window}", flush=True)
    spec = NanolabSpec(n_layer=3, n_embd=64, n_head=4, n_kv_head=kv_heads, head_dim=16, hidden=96, vocab=128,
                       window=window)
    B, T = 2, 24
    r = orc.SplitMix64(4242 + kv_heads)
    shapes = spec.param_shapes()
    host = {}
    for name in spec.param_names():
        n = int(np.prod(shapes[name]))
        if "norm" in name:
            host[name] = 1.0 + r.vec(n, 0.2)
        elif name.endswith("vr_lambda"):
            host[name] = r.vec(n, 1.0)
        elif name.endswith("gate.bias"):
            host[name] = r.vec(n, 0.5)
        else:
            host[name] = r.vec(n, 0.25)
    ids = np.array([r.below(spec.vocab) for _ in range(B * T)], np.uint32).reshape(B, T)
    targets = np.array([r.below(spec.vocab) for _ in range(B * T)], np.uint32).reshape(B, T)
    loss, _, grads = run(be, spec, host, ids, targets)
    cfg = orc.NanolabConfig(layers=spec.n_layer, n_embd=spec.n_embd, n_head=spec.n_head, n_kv_head=spec.n_kv_head,
                            head_dim=spec.head_dim, hidden=spec.hidden, vocab=spec.vocab, batch=B, seq=T,
                            window=window or 0, rms_eps=spec.rms_eps, rope_base=spec.rope_base)
    names = spec.param_names()
    assert names == orc.nanolab_param_names(spec.n_layer)
    o_loss, _, o_grads = orc.nanolab_loss_and_grads(cfg, [host[n] for n in names], ids, targets)
    assert abs(loss - float(o_loss)) <= FORWARD_LOSS_REL_TOL * abs(float(o_loss)), (loss, o_loss)
    for name, ref in zip(names, o_grads):
        got = grads[name].reshape(-1).astype(np.float64)
        if name == "blocks.0.mixer.vr_lambda":
            assert not np.any(got) and not np.any(ref)
            continue
        rel = np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-30)
        assert rel <= GRAD_NORMWISE_REL_TOL, (name, rel)


def test_trainer_steps_follow_the_torch_trace(be):
    """`NanolabTrainer.run` on the device over the reference's torch trace: per-step mean loss within
    1e-4 nats for five steps and every parameter after step 5 within 1e-4 normwise
    (ojas-oracle/src/parity.rs:36-41, :468-470); then on to step 40 with the whole loss curve at the
    reference's curve gates (2e-4 nats for the first ten steps, 2e-3 after, ending a nat below ln V;
    parity.rs:52-58)."""
    import trace_fixture as tf
    from ojas_amd.nanolab import NanolabTrainer

    print("nanolab 40-step trace on the device", flush=True)
    trace = tf.Trace()
    spec = tiny_spec()
    init, _ = load("init")
    trainer = NanolabTrainer(be, spec, init, adam_lr=trace.cfg["lr"], matrix_lr=trace.cfg["matrix_lr"],
                             grad_clip=trace.cfg["grad_clip"])
    losses, norms = [], []
    after_five = None
    for step in range(len(trace.mean_loss)):
        report = trainer.run([trace.micro(step, m) for m in range(trace.accum)], trace.lr_mult[step])
        assert report.step == step + 1 and report.tokens == trace.accum * trace.batch * trace.seq
        losses.append(report.loss)
        norms.append(report.grad_norm)
        if step + 1 == trace.steps:
            after_five = trainer.download_params()
    worst = tf.check_trace(trace, losses, norms, after_five, {"blocks.0.mixer.vr_lambda"})
    print(f"worst parameter distance after step {trace.steps}: {worst:.2e}", flush=True)
    print(f"worst loss distance over 40 steps: {tf.check_curve(trace, losses, spec.vocab):.2e}", flush=True)


def test_autocast_tier_stays_within_the_reference_gap_of_the_f32_run(be):
    """`check_autocast_divergence` (ojas-oracle/src/parity.rs:615-690): the same 40 steps under
    `Autocast` (`ojas_amd/autocast.py`) stay, step by step, within max(2e-3, 2 x torch's own worst
    f32-to-bf16 gap) of this backend's f32 run, and still end a nat below ln V. torch's bf16 curve is
    printed beside ours for the record only: two bf16 runs are not comparable step by step."""
    import trace_fixture as tf
    from ojas_amd.nanolab import NanolabTrainer

    print("nanolab 40 steps, f32 and autocast", flush=True)
    trace = tf.Trace()
    spec = tiny_spec()
    init, _ = load("init")
    curves = {}
    for autocast in (False, True):
        trainer = NanolabTrainer(be, spec, init, adam_lr=trace.cfg["lr"], matrix_lr=trace.cfg["matrix_lr"],
                                 grad_clip=trace.cfg["grad_clip"], autocast=autocast)
        curves[autocast] = np.array([trainer.run([trace.micro(step, m) for m in range(trace.accum)],
                                                 trace.lr_mult[step]).loss for step in range(40)])
    torch_f32, torch_bf16 = tf.autocast_gap()
    bound = max(tf.CURVE_LATE_ABS_TOL, tf.AUTOCAST_GAP_FACTOR * float(np.max(np.abs(torch_bf16 - torch_f32))))
    gap = np.abs(curves[True] - curves[False])
    print(f"worst |autocast - f32| {gap.max():.2e} at step {int(gap.argmax()) + 1} (bound {bound:.2e}); "
          f"torch's own {np.max(np.abs(torch_bf16 - torch_f32)):.2e}; "
          f"|autocast - torch bf16| {np.max(np.abs(curves[True] - torch_bf16)):.2e}", flush=True)
    assert np.any(curves[True] != curves[False])  # the tier did round something
    assert np.all(gap <= bound), (int(gap.argmax()), float(gap.max()))
    assert curves[True][-1] <= np.log(spec.vocab) - tf.CURVE_MIN_DROP_NATS


def test_save_then_resume_continues_bit_for_bit(be, tmp_path):
    """`Trainer::save` / `resume_from` over the checkpoint directory (ojas-model/src/checkpoint.rs): three
    steps, a save, a resume into a fresh trainer and two more steps equal five uninterrupted steps bit for
    bit, as `g9_forty_steps_equal_twenty_saved_dropped_resumed_and_twenty_more`
    (ojas-model/tests/checkpoint.rs) demands of the CPU. A resume with another seed, config or tokenizer
    hash is refused."""
    import trace_fixture as tf
    from ojas_amd.io import IoError, SafeTensors, read_checkpoint
    from ojas_amd.nanolab import NanolabTrainer, TrainConfig, resume_checkpoint, save_checkpoint, spec_from_json

    print("nanolab save / resume", flush=True)
    trace = tf.Trace()
    init, _ = load("init")
    spec = spec_from_json(SafeTensors(TINY / "init.safetensors").metadata()["ojas.spec"])
    cfg = TrainConfig(seq_len=trace.seq, batch=trace.batch, accum=trace.accum, data_seed=1337, total_steps=40,
                      warmup_steps=4)
    batches = lambda step: [trace.micro(step, m) for m in range(trace.accum)]
    whole = NanolabTrainer(be, spec, init)
    for step in range(5):
        whole.run(batches(step), trace.lr_mult[step])
    first = NanolabTrainer(be, spec, init)
    for step in range(3):
        first.run(batches(step), trace.lr_mult[step])
    ckpt = tmp_path / "ckpt"
    save_checkpoint(first, ckpt, cfg, cursor=(0, 12), run="r1", tokenizer_hash=bytes(range(32)))
    assert sorted(p.name for p in ckpt.iterdir()) == ["model.safetensors", "optim.safetensors", "state.ojck"]
    state = read_checkpoint(ckpt / "state.ojck")
    assert (state.step, state.cursor, len(state.rng_state)) == (3, (0, 12), 16) and not any(state.sections())
    assert SafeTensors(ckpt / "model.safetensors").metadata()["ojas.step"] == "3"
    del first
    resumed, cursor, run = resume_checkpoint(be, ckpt, cfg, tokenizer_hash=bytes(range(32)))
    assert (resumed.step, cursor, run) == (3, (0, 12), "r1")
    for step in range(3, 5):
        resumed.run(batches(step), trace.lr_mult[step])
    a, b = whole.download_params(), resumed.download_params()
    for name in spec.param_names():
        assert np.array_equal(a[name].view(np.uint32), b[name].view(np.uint32)), name
    for other, what in ((dict(data_seed=7), "train config"), (dict(accum=4), "train config")):
        with pytest.raises(IoError, match=what):
            resume_checkpoint(be, ckpt, TrainConfig(**{**cfg.__dict__, **other}), tokenizer_hash=bytes(range(32)))
    with pytest.raises(IoError, match="tokenizer hash"):
        resume_checkpoint(be, ckpt, cfg)
