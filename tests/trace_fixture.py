"""The reference's 40-step torch trace of the tiny nanolab model (ojas-oracle/python/golden.py:319-386),
as data: the micro-batches it drew, the schedule multipliers it applied, the losses and gradient norms
it logged, and the parameters after step 5.

A step here is `Trainer::run` (ojas-model/src/trainer.rs:754-857): `accum` micro-batches with uniform
weights 1/accum seeded into the backward (:1104-1111), gradients summed (`accumulate_grad`, :973-978),
one global clip at `grad_clip`, then per parameter Muon-NS5 (matrices other than the embedding) or AdamW
(the embedding and every vector) at `initial_lr * multiplier` (:858-876, :1004-1028). Group constants:
ojas-cpu/src/train.rs:20-62.
"""
import json
from pathlib import Path

import numpy as np
from safetensors import safe_open

TINY = Path(__file__).parent / "golden" / "tiny"
TRACE_LOSS_ABS_TOL = 1e-4  # ojas-oracle/src/parity.rs:38
TRACE_PARAM_NORMWISE_REL_TOL = 1e-4  # :41
MUON_MOMENTUM = 0.99
MUON_WEIGHT_DECAY = 0.1
ADAM_HYBRID_WEIGHT_DECAY = 0.0


def load(name):
    with safe_open(str(TINY / f"{name}.safetensors"), "np") as f:
        meta = {k: json.loads(v) for k, v in (f.metadata() or {}).items()}
        return {k: f.get_tensor(k) for k in f.keys()}, meta


class Trace:
    def __init__(self):
        self.params_after, meta = load("trace_ns5_f32")
        info = meta["ojas.oracle"]
        self.cfg = info["config"]
        self.steps = info["params_after_step"]
        self.lr_mult = info["lr_mult"]
        self.mean_loss = info["mean_loss"]
        self.micro_loss = info["micro_loss"]
        self.grad_norm = info["grad_norm"]
        self.starts = json.loads((TINY / "batch_starts.json").read_text())
        assert self.starts["bin_format"] == "headerless-u16le" and self.starts["bin_header_bytes"] == 0
        self.tokens = np.fromfile(TINY / "tokens.bin", dtype="<u2")
        assert self.tokens.size == self.starts["bin_tokens"]
        self.accum, self.batch, self.seq = self.starts["accum"], self.starts["batch"], self.starts["seq_len"]
        assert (self.accum, self.batch, self.seq) == (self.cfg["grad_accum"], self.cfg["batch_size"],
                                                      self.cfg["block_size"])

    def micro(self, step, micro):
        """(ids, targets) u32 [batch, seq]: the windows at the dumped starts, targets one token on
        (ojas-oracle/python/batches.py:76-88)."""
        first = (step * self.accum + micro) * self.batch
        rows = [self.tokens[s:s + self.seq + 1] for s in self.starts["starts"][first:first + self.batch]]
        buf = np.stack(rows).astype(np.uint32)
        return np.ascontiguousarray(buf[:, :-1]), np.ascontiguousarray(buf[:, 1:])


def optimizer_of(name, shape):
    """`OptimGroup` by name (ojas-model/src/names.rs:188-300): "adamw" for the embedding and
    vectors, "muon" for every other matrix."""
    return "muon" if len(shape) == 2 and name != "tok_emb.weight" else "adamw"


# The 40-step curve (framework-design section 10; ojas-oracle/src/parity.rs:52-58): |loss - torch's| per step.
CURVE_EARLY_ABS_TOL = 2e-4  # steps 1 ..= CURVE_EARLY_STEPS
CURVE_EARLY_STEPS = 10
CURVE_LATE_ABS_TOL = 2e-3
CURVE_MIN_DROP_NATS = 1.0  # the curve must end this far below ln V
AUTOCAST_GAP_FACTOR = 2.0  # parity.rs:59-74


def check_curve(trace, losses, vocab):
    """The per-step mean losses of all 40 steps against the trace's (`parity.rs:52-58`)."""
    assert len(losses) == len(trace.mean_loss) == 40
    worst = 0.0
    for s, (got, want) in enumerate(zip(losses, trace.mean_loss)):
        tol = CURVE_EARLY_ABS_TOL if s < CURVE_EARLY_STEPS else CURVE_LATE_ABS_TOL
        assert abs(got - want) <= tol, (s, got, want)
        worst = max(worst, abs(got - want))
    assert losses[-1] <= np.log(vocab) - CURVE_MIN_DROP_NATS, losses[-1]
    return worst


def autocast_gap():
    """torch's own f32 and autocast-bf16 curves over the same 40 steps (`autocast_gap.json`)."""
    d = json.loads((TINY / "autocast_gap.json").read_text())
    return np.array(d["f32_mean_loss"]), np.array(d["bf16_mean_loss"])


def check_trace(trace, losses, norms, params, frozen):
    for s in range(trace.steps):
        assert abs(losses[s] - trace.mean_loss[s]) <= TRACE_LOSS_ABS_TOL, (s, losses[s], trace.mean_loss[s])
        assert abs(norms[s] - trace.grad_norm[s]) <= 1e-4 * trace.grad_norm[s], (s, norms[s], trace.grad_norm[s])
    worst = 0.0
    for name, want in trace.params_after.items():
        got = np.asarray(params[name], np.float64).reshape(-1)
        ref = want.reshape(-1).astype(np.float64)
        if name in frozen:
            assert np.array_equal(got, ref), name
            continue
        rel = np.linalg.norm(got - ref) / np.linalg.norm(ref)
        assert rel <= TRACE_PARAM_NORMWISE_REL_TOL, (name, rel)
        worst = max(worst, rel)
    return worst
