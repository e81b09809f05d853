"""The nanolab GPT graph over `MiBackend`: forward, loss and every gradient.

Host-side orchestration only, the role of `forward_loss` + `Tape::backward` for the reference's own
model graph (ojas-model/src/block.rs:218-264 `block_with`, :343-420 `hidden` / tied head;
ojas-autograd/src/tape.rs:2004-2466 backward rules, :2565-2591 gradient fan-in, later consumer
first). Every tensor operation is one `MiBackend` method, i.e. one C-ABI call; nothing is computed
here. Parameters come in the order of ojas-model/src/names.rs:188-300.
"""
from __future__ import annotations

import ctypes as C
import json
import math
from contextlib import nullcontext
from dataclasses import dataclass
from decimal import Decimal
from pathlib import Path
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from .autocast import Autocast
from .backend import F32, AdamWConfig, MiBackend, MuonNs5Config, DeviceTensor, OjasError, NON_FINITE, OUT_OF_RANGE

BLOCK_PARAMS = ("norm1.weight", "mixer.q_proj.weight", "mixer.k_proj.weight", "mixer.v_proj.weight",
                "mixer.o_proj.weight", "mixer.q_norm.weight", "mixer.k_norm.weight", "mixer.gate.weight",
                "mixer.gate.bias", "mixer.vr_lambda", "norm2.weight", "ffn.gate.weight", "ffn.up.weight",
                "ffn.down.weight")


@dataclass
class NanolabSpec:
    """`ojas_model::ModelSpec` (ojas-model/src/spec.rs): the fields the graph reads."""
    n_layer: int
    n_embd: int
    n_head: int
    n_kv_head: int
    head_dim: int
    hidden: int
    vocab: int
    rms_eps: float = 1e-6
    rope_base: float = 10000.0
    window: Optional[int] = None
    max_seq: int = 0  # only the spec's JSON needs it

    def param_names(self) -> List[str]:
        names = ["tok_emb.weight"]
        for i in range(self.n_layer):
            names += [f"blocks.{i}.{n}" for n in BLOCK_PARAMS]
        return names + ["norm_f.weight"]

    def param_shapes(self) -> Dict[str, tuple]:
        d, q, kv = self.n_embd, self.n_head * self.head_dim, self.n_kv_head * self.head_dim
        per = {"norm1.weight": (d,), "mixer.q_proj.weight": (q, d), "mixer.k_proj.weight": (kv, d),
               "mixer.v_proj.weight": (kv, d), "mixer.o_proj.weight": (d, q), "mixer.q_norm.weight": (self.head_dim,),
               "mixer.k_norm.weight": (self.head_dim,), "mixer.gate.weight": (self.n_head, d),
               "mixer.gate.bias": (self.n_head,), "mixer.vr_lambda": (1,), "norm2.weight": (d,),
               "ffn.gate.weight": (self.hidden, d), "ffn.up.weight": (self.hidden, d),
               "ffn.down.weight": (d, self.hidden)}
        shapes = {"tok_emb.weight": (self.vocab, d), "norm_f.weight": (d,)}
        for i in range(self.n_layer):
            for n, shp in per.items():
                shapes[f"blocks.{i}.{n}"] = shp
        return shapes


def rope_tables(spec: NanolabSpec, seq: int):
    """`Rope::rows` (ojas-model/src/block.rs:31-71): angles in f64, one rounding to f32, both
    halves of a row equal. Host arrays; upload them once."""
    half = spec.head_dim // 2
    inv = np.array([spec.rope_base ** (-(2 * i) / spec.head_dim) for i in range(half)], np.float64)
    ang = np.arange(seq, dtype=np.float64)[:, None] * inv[None, :]
    cos = np.concatenate([np.cos(ang), np.cos(ang)], axis=1).astype(np.float32)
    sin = np.concatenate([np.sin(ang), np.sin(ang)], axis=1).astype(np.float32)
    return cos, sin


class NanolabGraph:
    """Runs the graph on one backend. `params` maps names to f32 device tensors."""

    def __init__(self, be: MiBackend, spec: NanolabSpec, params: Dict[str, DeviceTensor]):
        self.be, self.spec, self.p = be, spec, params

    def _blk(self, i: int, name: str) -> DeviceTensor:
        return self.p[f"blocks.{i}.{name}"]

    def loss_and_grads(self, ids: DeviceTensor, targets: DeviceTensor, want_logits: bool = False,
                       loss_seed: float = 1.0):
        """Returns (loss [1] f32, logits or None, {name: gradient}). `ids`, `targets` are u32 [B, T].
        `loss_seed` is the gradient of the loss the backward starts from (`Tape::backward_seeded`)."""
        be, s = self.be, self.spec
        B, T = ids.shape
        N, d, H, KV, D = B * T, s.n_embd, s.n_head, s.n_kv_head, s.head_dim
        eps, win = s.rms_eps, s.window
        cos_h, sin_h = rope_tables(s, T)
        cos, sin = be.upload(cos_h), be.upload(sin_h)
        swap = [0, 2, 1, 3]

        # ---- forward (block.rs:218-264) ----
        x = be.embedding_forward(self.p["tok_emb.weight"], ids).reshape(N, d)
        acts = []
        v0 = None
        for i in range(s.n_layer):
            a = {"x": x}
            a["h"] = be.rms_norm_forward(x, self._blk(i, "norm1.weight"), eps)
            a["q_lin"] = be.linear_forward(a["h"], self._blk(i, "mixer.q_proj.weight")).reshape(B, T, H, D)
            a["k_lin"] = be.linear_forward(a["h"], self._blk(i, "mixer.k_proj.weight")).reshape(B, T, KV, D)
            a["raw_v"] = be.linear_forward(a["h"], self._blk(i, "mixer.v_proj.weight")).reshape(B, T, KV, D)
            qn, kn = be.rms_qk_norm_forward(a["q_lin"], a["k_lin"], self._blk(i, "mixer.q_norm.weight"),
                                            self._blk(i, "mixer.k_norm.weight"), eps)
            q = be.rope_half_split_forward(qn, cos, sin)
            k = be.rope_half_split_forward(kn, cos, sin)
            if v0 is None:
                v = a["raw_v"]
                v0 = a["raw_v"]
            else:
                v = be.value_residual_blend_forward(a["raw_v"], v0, self._blk(i, "mixer.vr_lambda"))
            a["qp"], a["kp"], a["vp"] = be.permute(q, swap), be.permute(k, swap), be.permute(v, swap)
            a["att"], a["lse"] = be.causal_sdpa_forward(a["qp"], a["kp"], a["vp"], win)
            a["ap"] = be.permute(a["att"], swap)  # [B, T, H, D]
            a["y"], a["scales"] = be.per_head_sigmoid_gate_forward_saving(
                a["h"].reshape(B, T, d), self._blk(i, "mixer.gate.weight"), self._blk(i, "mixer.gate.bias"), a["ap"])
            o = be.linear_forward(a["y"].reshape(N, H * D), self._blk(i, "mixer.o_proj.weight"))
            a["x1"] = be.residual_add_forward(x, o)
            a["h2"] = be.rms_norm_forward(a["x1"], self._blk(i, "norm2.weight"), eps)
            a["g_lin"] = be.linear_forward(a["h2"], self._blk(i, "ffn.gate.weight"))
            a["g_act"] = be.silu_forward(a["g_lin"])
            a["up"] = be.linear_forward(a["h2"], self._blk(i, "ffn.up.weight"))
            a["m"] = be.mul_forward(a["g_act"], a["up"])
            down = be.linear_forward(a["m"], self._blk(i, "ffn.down.weight"))
            x = be.residual_add_forward(a["x1"], down)
            acts.append(a)
        hf = be.rms_norm_forward(x, self.p["norm_f.weight"], eps)
        logits = be.linear_forward(hf, self.p["tok_emb.weight"]) if want_logits else None
        tflat = targets.reshape(N)
        loss, ghf, g_head = be.linear_cross_entropy_mean(hf, self.p["tok_emb.weight"], tflat)
        if loss_seed != 1.0:
            be.scale_grad(ghf, loss_seed)
            be.scale_grad(g_head, loss_seed)

        # ---- backward: reverse program order; a value's consumers add their gradients later one first ----
        grads: Dict[str, DeviceTensor] = {}
        gx, grads["norm_f.weight"] = be.rms_norm_backward(x, self.p["norm_f.weight"], ghf, eps)
        g_v0 = None  # gradient of block 0's raw v from the later blocks' blends
        for i in reversed(range(s.n_layer)):
            a = acts[i]
            gm, grads[f"blocks.{i}.ffn.down.weight"] = be.linear_backward(a["m"], self._blk(i, "ffn.down.weight"), gx)
            g_gact, g_up = be.mul_backward(a["g_act"], a["up"], gm)
            gh2, grads[f"blocks.{i}.ffn.up.weight"] = be.linear_backward(a["h2"], self._blk(i, "ffn.up.weight"), g_up)
            g_glin = be.silu_backward(a["g_lin"], g_gact)
            part, grads[f"blocks.{i}.ffn.gate.weight"] = be.linear_backward(a["h2"], self._blk(i, "ffn.gate.weight"),
                                                                           g_glin)
            gh2 = be.residual_add_forward(gh2, part)
            gt, grads[f"blocks.{i}.norm2.weight"] = be.rms_norm_backward(a["x1"], self._blk(i, "norm2.weight"), gh2, eps)
            gx1 = be.residual_add_forward(gx, gt)
            gy, grads[f"blocks.{i}.mixer.o_proj.weight"] = be.linear_backward(
                a["y"].reshape(N, H * D), self._blk(i, "mixer.o_proj.weight"), gx1)
            gh, grads[f"blocks.{i}.mixer.gate.weight"], grads[f"blocks.{i}.mixer.gate.bias"], gap = \
                be.per_head_sigmoid_gate_backward_saved(a["h"].reshape(B, T, d), self._blk(i, "mixer.gate.weight"),
                                                        self._blk(i, "mixer.gate.bias"), a["ap"],
                                                        gy.reshape(B, T, H, D), a["scales"])
            gh = gh.reshape(N, d)
            ga = be.permute(gap, swap)
            gqp, gkp, gvp = be.causal_sdpa_backward(a["qp"], a["kp"], a["vp"], a["att"], a["lse"], ga, win)
            gv, gk, gq = be.permute(gvp, swap), be.permute(gkp, swap), be.permute(gqp, swap)
            if i == 0:
                g_raw_v = gv if g_v0 is None else be.residual_add_forward(g_v0, gv)
                grads["blocks.0.mixer.vr_lambda"] = be.zeros((1,), F32)
            else:
                g_raw_v, part_v0, grads[f"blocks.{i}.mixer.vr_lambda"] = be.value_residual_blend_backward(
                    a["raw_v"], acts[0]["raw_v"], self._blk(i, "mixer.vr_lambda"), gv)
                g_v0 = part_v0 if g_v0 is None else be.residual_add_forward(g_v0, part_v0)
            gkn = be.rope_half_split_backward(gk, cos, sin)
            gqn = be.rope_half_split_backward(gq, cos, sin)
            gq_lin, gk_lin, grads[f"blocks.{i}.mixer.q_norm.weight"], grads[f"blocks.{i}.mixer.k_norm.weight"] = \
                be.rms_qk_norm_backward(a["q_lin"], a["k_lin"], self._blk(i, "mixer.q_norm.weight"),
                                        self._blk(i, "mixer.k_norm.weight"), gqn, gkn, eps)
            for name, g_out in (("v_proj", g_raw_v.reshape(N, KV * D)), ("k_proj", gk_lin.reshape(N, KV * D)),
                                ("q_proj", gq_lin.reshape(N, H * D))):
                part, grads[f"blocks.{i}.mixer.{name}.weight"] = be.linear_backward(
                    a["h"], self._blk(i, f"mixer.{name}.weight"), g_out)
                gh = be.residual_add_forward(gh, part)
            gt, grads[f"blocks.{i}.norm1.weight"] = be.rms_norm_backward(a["x"], self._blk(i, "norm1.weight"), gh, eps)
            gx = be.residual_add_forward(gx1, gt)
        # The tied table: the head's gradient first, then the embedding's rows.
        g_emb = be.embedding_backward(ids.reshape(N), gx, s.vocab)
        grads["tok_emb.weight"] = be.residual_add_forward(g_head, g_emb)
        return loss, logits, grads


# ojas-cpu/src/train.rs:20-62
MUON_MOMENTUM = 0.99
MUON_WEIGHT_DECAY = 0.1
ADAM_HYBRID_WEIGHT_DECAY = 0.0
FROZEN = ("blocks.0.mixer.vr_lambda",)  # block 0 has no earlier value to blend with: no gradient reaches it


@dataclass
class StepReport:
    """`ojas_model::StepReport` (ojas-model/src/trainer.rs:280-297)."""
    loss: float
    grad_norm: float
    lr_multiplier: float
    step: int
    tokens: int


class NanolabTrainer:
    """`Trainer::run` (ojas-model/src/trainer.rs:754-857) for the f32 tier: micro-batches weighted
    by their share of the step's valid targets and seeded into the backward (:1089-1119), gradients
    summed with `accumulate_grad` (:973-978), one `clip_grad_norm`, then per parameter `muon_ns5_step`
    (matrices other than the embedding) or `adamw_step` (the embedding and the vectors) at the group's
    peak rate times the schedule multiplier (:858-876, :1004-1028). The multiplier is the caller's:
    the schedule is host arithmetic outside this path."""

    def __init__(self, be: MiBackend, spec: NanolabSpec, host_params: Dict[str, np.ndarray], adam_lr: float = 6e-4,
                 matrix_lr: float = 0.025, grad_clip: float = 1.0, ns5_bf16: bool = False, autocast: bool = False):
        # `TrainConfig::precision` (trainer.rs:120-135): bf16 wraps the backend in `Autocast` and the
        # forward, the backward and the taking of the gradients run inside its region (:935-966);
        # accumulation, the clip and the optimizers run outside it, on f32 masters.
        self.autocast = autocast
        if autocast:
            be = Autocast(be)
        self.be, self.spec = be, spec
        self.adam_lr, self.matrix_lr, self.grad_clip, self.ns5_bf16 = adam_lr, matrix_lr, grad_clip, ns5_bf16
        shapes = spec.param_shapes()
        self.names = spec.param_names()
        self.params = {n: be.upload(np.ascontiguousarray(host_params[n], np.float32).reshape(shapes[n]))
                       for n in self.names}
        self.trainable = [n for n in self.names if n not in FROZEN]
        self.muon = {n for n in self.trainable if len(shapes[n]) == 2 and n != "tok_emb.weight"}
        self.state = {n: [be.zeros(shapes[n], F32)] if n in self.muon else [be.zeros(shapes[n], F32),
                                                                              be.zeros(shapes[n], F32)]
                      for n in self.trainable}
        self.graph = NanolabGraph(be, spec, self.params)
        self.step = 0

    def run(self, batches: Sequence, lr_multiplier: float, ignore_index: Optional[int] = None) -> StepReport:
        """`batches`: (ids, targets) u32 host arrays [B, T], one per micro-batch."""
        be = self.be
        counts = [int(np.count_nonzero(y != ignore_index)) if ignore_index is not None else int(y.size)
                  for _, y in batches]
        live = [c for c in counts if c > 0]
        if not batches:
            raise OjasError(OUT_OF_RANGE, "Trainer::step: 0 micro-batches")
        if not live:
            raise OjasError(NON_FINITE, "Trainer::step: no valid target")
        uniform = all(c == live[0] for c in live)
        total = sum(counts)
        acc, loss_sum = None, None
        for (ids, targets), count in zip(batches, counts):
            if count == 0:
                continue
            weight = float(np.float32(1.0 / len(live))) if uniform else float(np.float32(count / total))
            with (be.region() if self.autocast else nullcontext()):
                loss, _, grads = self.graph.loss_and_grads(be.upload(np.ascontiguousarray(ids, np.uint32)),
                                                           be.upload(np.ascontiguousarray(targets, np.uint32)),
                                                           loss_seed=weight)
            if acc is None:
                acc = {n: grads[n] for n in self.trainable}
            else:
                for n in self.trainable:
                    be.accumulate_grad(acc[n], grads[n])
            if not uniform and weight != 1.0:
                be.scale_grad(loss, weight)
            loss_sum = loss if loss_sum is None else be.residual_add_forward(loss_sum, loss)
        grad_norm = be.clip_grad_norm([acc[n] for n in self.trainable], self.grad_clip)
        for n in self.trainable:
            if n in self.muon:
                cfg = MuonNs5Config(self.matrix_lr * lr_multiplier, MUON_MOMENTUM, MUON_WEIGHT_DECAY, 1,
                                    int(self.ns5_bf16))
                be.muon_ns5_step(self.params[n], acc[n], self.state[n][0], cfg)
            else:
                cfg = AdamWConfig.nanolab(self.adam_lr * lr_multiplier, ADAM_HYBRID_WEIGHT_DECAY)
                be.adamw_step(self.params[n], acc[n], self.state[n][0], self.state[n][1], self.step, cfg)
        value = float(be.download(loss_sum)[0])
        if not math.isfinite(value):
            raise OjasError(NON_FINITE, "Trainer::step")
        self.step += 1
        return StepReport(loss=value / len(live) if uniform else value, grad_norm=grad_norm,
                          lr_multiplier=lr_multiplier, step=self.step, tokens=sum(int(x.size) for x, _ in batches))

    def download_params(self) -> Dict[str, np.ndarray]:
        return {n: self.be.download(t) for n, t in self.params.items()}


class OnanoConfig(C.Structure):
    """onano_config of include/ojas_nanolab.h."""
    _fields_ = [(n, C.c_uint32) for n in ("layers", "n_embd", "heads", "kv_heads", "head_dim", "hidden", "vocab", "batch",
                                          "seq", "window", "bf16")] + [("rms_eps", C.c_float), ("rope_base", C.c_double)]


NATIVE_LIB_PATH = Path(__file__).resolve().parent / "libojas_nanolab.so"


class NativeNanolabTrainer:
    """`Trainer::run` (ojas-model/src/trainer.rs:754-857) through the C++ step driver of
    include/ojas_nanolab.h: the same step as `NanolabTrainer`, with the graph's ~60 calls per block
    made from C++ over buffers allocated once, and bf16 storage of activations and operand copies
    when `bf16` is set. The schedule multiplier is the caller's."""

    def __init__(self, be: MiBackend, spec: NanolabSpec, batch: int, seq: int, host_params=None, adam_lr: float = 6e-4,
                 matrix_lr: float = 0.025, grad_clip: float = 1.0, ns5_bf16: bool = False, bf16: bool = False):
        if not NATIVE_LIB_PATH.exists():
            raise OjasError(10, f"{NATIVE_LIB_PATH} is not built; run __graft_entry__.build()")
        self._lib = C.CDLL(str(NATIVE_LIB_PATH))
        for name in ("onano_param_count", "onano_param_len", "onano_steps", "onano_device_bytes"):
            getattr(self._lib, name).restype = C.c_uint64
        self.be, self.spec, self.batch, self.seq = be, spec, batch, seq
        self.adam_lr, self.matrix_lr, self.grad_clip, self.ns5_bf16 = adam_lr, matrix_lr, grad_clip, ns5_bf16
        self.names = spec.param_names()
        cfg = OnanoConfig(spec.n_layer, spec.n_embd, spec.n_head, spec.n_kv_head, spec.head_dim, spec.hidden, spec.vocab,
                          batch, seq, spec.window or 0, int(bf16), spec.rms_eps, spec.rope_base)
        h = C.c_void_p()
        rc = self._lib.onano_create(be._ctx, C.byref(cfg), C.byref(h))
        self._h = h if rc == 0 else None
        be._check(rc)
        shapes = spec.param_shapes()
        lens = [int(self._lib.onano_param_len(self._h, C.c_uint64(i))) for i in range(len(self.names))]
        assert int(self._lib.onano_param_count(self._h)) == len(self.names)
        assert lens == [int(np.prod(shapes[n])) for n in self.names]
        self.lens = lens
        if host_params is not None:
            self.set_params(host_params)

    def close(self):
        if self._h:
            self._lib.onano_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    @property
    def step(self) -> int:
        return int(self._lib.onano_steps(self._h))

    def init(self, seed: int):
        self.be._check(self._lib.onano_init(self._h, C.c_uint64(seed)))

    def init_reference(self, seed: int):
        """`init_params` (ojas-model/src/init.rs:114): the reference's per-name streams."""
        self.be._check(self._lib.onano_init_reference(self._h, C.c_uint64(seed)))

    def native_param_names(self) -> List[str]:
        out = []
        buf = C.create_string_buffer(96)
        for i in range(len(self.names)):
            self.be._check(self._lib.onano_param_name(self._h, C.c_uint64(i), buf, C.c_uint64(96)))
            out.append(buf.value.decode())
        return out

    def set_params(self, host_params: Dict[str, np.ndarray]):
        for i, n in enumerate(self.names):
            a = np.ascontiguousarray(host_params[n], np.float32).reshape(-1)
            self.be._check(self._lib.onano_set_param(self._h, C.c_uint64(i), a.ctypes.data_as(C.c_void_p)))

    def _get(self, fn, *extra) -> Dict[str, np.ndarray]:
        out = {}
        for i, (n, length) in enumerate(zip(self.names, self.lens)):
            a = np.empty(length, np.float32)
            self.be._check(fn(self._h, C.c_uint64(i), *extra, a.ctypes.data_as(C.c_void_p)))
            out[n] = a
        return out

    def download_params(self) -> Dict[str, np.ndarray]:
        shapes = self.spec.param_shapes()
        return {n: a.reshape(shapes[n]) for n, a in self._get(self._lib.onano_get_param).items()}

    def grads(self) -> Dict[str, np.ndarray]:
        return self._get(self._lib.onano_get_grad)

    def state(self, slot: int) -> Dict[str, np.ndarray]:
        return self._get(self._lib.onano_get_state, C.c_uint32(slot))

    def loss_and_grads(self, ids, targets, loss_seed: float = 1.0):
        """One micro-batch on its own: (loss, {name: gradient})."""
        self._micro(ids, targets, loss_seed, 1.0, True)
        loss = C.c_float()
        self.be._check(self._lib.onano_loss(self._h, C.byref(loss)))
        return float(loss.value), self.grads()

    def _micro(self, ids, targets, seed, scale, first):
        ids = np.ascontiguousarray(ids, np.uint32).reshape(-1)
        targets = np.ascontiguousarray(targets, np.uint32).reshape(-1)
        if ids.size != self.batch * self.seq or targets.size != ids.size:
            raise OjasError(1, f"micro-batch: expected {self.batch} x {self.seq} ids and targets")
        self.be._check(self._lib.onano_micro_batch(self._h, ids.ctypes.data_as(C.c_void_p),
                                                   targets.ctypes.data_as(C.c_void_p), C.c_float(seed), C.c_float(scale),
                                                   C.c_int32(1 if first else 0)))

    def run(self, batches: Sequence, lr_multiplier: float) -> StepReport:
        """`batches`: (ids, targets) u32 host arrays [batch, seq], one per micro-batch; every target counts."""
        if not batches:
            raise OjasError(OUT_OF_RANGE, "Trainer::step: 0 micro-batches")
        weight = float(np.float32(1.0 / len(batches)))  # equal counts: the uniform weights of trainer.rs:1089-1119
        for k, (ids, targets) in enumerate(batches):
            self._micro(ids, targets, weight, 1.0, k == 0)
        return self.apply(lr_multiplier, len(batches))

    def run_resident(self, lr_multiplier: float) -> StepReport:
        """One step of one micro-batch on the ids and targets uploaded last."""
        self.be._check(self._lib.onano_micro_batch_resident(self._h, C.c_float(1.0), C.c_float(1.0), C.c_int32(1)))
        return self.apply(lr_multiplier, 1)

    def apply(self, lr_multiplier: float, micro_batches: int) -> StepReport:
        muon = MuonNs5Config(self.matrix_lr * lr_multiplier, MUON_MOMENTUM, MUON_WEIGHT_DECAY, 1, int(self.ns5_bf16))
        adamw = AdamWConfig.nanolab(self.adam_lr * lr_multiplier, ADAM_HYBRID_WEIGHT_DECAY)
        loss, norm = C.c_float(), C.c_float()
        self.be._check(self._lib.onano_apply(self._h, C.byref(muon), C.byref(adamw), C.c_float(self.grad_clip),
                                             C.byref(loss), C.byref(norm)))
        value = float(loss.value)
        if not math.isfinite(value):
            raise OjasError(NON_FINITE, "Trainer::step")
        return StepReport(loss=value / micro_batches, grad_norm=float(norm.value), lr_multiplier=lr_multiplier,
                          step=self.step, tokens=micro_batches * self.batch * self.seq)

    def device_bytes(self) -> int:
        return int(self._lib.onano_device_bytes(self._h))


def nanolab_step_flops(spec: NanolabSpec, batch: int, seq: int) -> float:
    """Algorithmic FLOPs of one step: 6 N P over the weights that take part in products (the
    projections, the gate, the SwiGLU matrices and the tied head) and causal attention at half the
    square (forward 2, backward 5 products)."""
    d, q, kv = spec.n_embd, spec.n_head * spec.head_dim, spec.n_kv_head * spec.head_dim
    per_block = d * q + 2 * d * kv + q * d + spec.n_head * d + 3 * d * spec.hidden
    n = batch * seq
    attention = 7.0 * batch * spec.n_head * seq * seq * spec.head_dim * spec.n_layer
    return 6.0 * n * (spec.n_layer * per_block + spec.vocab * d) + attention


def spec_nanolab_124m() -> NanolabSpec:
    """`ModelSpec::nanolab_124m` (ojas-model/src/spec.rs:74-91)."""
    return NanolabSpec(n_layer=12, n_embd=768, n_head=12, n_kv_head=12, head_dim=64, hidden=2048, vocab=50304,
                       rms_eps=1e-6, rope_base=10000.0, window=None, max_seq=1024)


# ---- the checkpoint directory (ojas-model/src/checkpoint.rs:1-60) ----
MODEL_FILE, OPTIM_FILE, STATE_FILE = "model.safetensors", "optim.safetensors", "state.ojck"
STATE_FORMAT = "ojas-train-v1"


def rust_f64(x: float) -> str:
    """An f64 the way Rust's `{:?}` prints it (shortest digits; exponent form below 1e-4 and from
    1e16 on, without '+' or padding; otherwise at least one fractional digit)."""
    if x != x or x in (math.inf, -math.inf):
        raise ValueError("not a finite number")
    sign, digits, exp = Decimal(repr(float(x))).as_tuple()
    digits = "".join(map(str, digits)).lstrip("0") or "0"
    if digits == "0":
        return "-0.0" if sign else "0.0"
    stripped = digits.rstrip("0")
    exp += len(digits) - len(stripped)
    digits = stripped
    sci = len(digits) - 1 + exp  # value = d.ddd x 10^sci
    if sci < -4 or sci >= 16:
        body = digits[0] + ("." + digits[1:] if len(digits) > 1 else "") + "e" + str(sci)
    elif exp >= 0:
        body = digits + "0" * exp + ".0"
    elif -exp < len(digits):
        body = digits[:exp] + "." + digits[exp:]
    else:
        body = "0." + "0" * (-exp - len(digits)) + digits
    return ("-" if sign else "") + body


def spec_to_json(spec: NanolabSpec) -> str:
    """`ModelSpec::to_json` (ojas-model/src/spec.rs:246-268): `ojas-spec-v1`, or v2 with a window."""
    if spec.max_seq <= 0:
        raise OjasError(OUT_OF_RANGE, "ModelSpec: max_seq is not set")
    fmt, window = ("ojas-spec-v1", "") if spec.window is None else ("ojas-spec-v2", f',"window":{spec.window}')
    return (f'{{"format":"{fmt}","arch":"nanolab-gpt","vocab":{spec.vocab},"n_embd":{spec.n_embd},'
            f'"n_layer":{spec.n_layer},"n_head":{spec.n_head},"n_kv_head":{spec.n_kv_head},"head_dim":{spec.head_dim},'
            f'"hidden":{spec.hidden},"max_seq":{spec.max_seq},"rope_base":{rust_f64(spec.rope_base)},'
            f'"rms_eps":{rust_f64(spec.rms_eps)},"tie_embeddings":true,"qk_norm":true,"gated_attention":true,'
            f'"value_residual":true{window}}}')


def spec_from_json(text: str) -> NanolabSpec:
    """`ModelSpec::from_json` (spec.rs:280-360): the keys of v1 / v2, the four flags true."""
    d = json.loads(text)
    want = {"ojas-spec-v1": False, "ojas-spec-v2": True}
    if d.get("format") not in want or d.get("arch") != "nanolab-gpt":
        raise OjasError(OUT_OF_RANGE, f"ModelSpec: format {d.get('format')!r} / arch {d.get('arch')!r}")
    if ("window" in d) != want[d["format"]]:
        raise OjasError(OUT_OF_RANGE, "ModelSpec: window belongs to ojas-spec-v2 only")
    for flag in ("tie_embeddings", "qk_norm", "gated_attention", "value_residual"):
        if d.get(flag) is not True:
            raise OjasError(OUT_OF_RANGE, f"ModelSpec: {flag} must be true")
    return NanolabSpec(n_layer=d["n_layer"], n_embd=d["n_embd"], n_head=d["n_head"], n_kv_head=d["n_kv_head"],
                       head_dim=d["head_dim"], hidden=d["hidden"], vocab=d["vocab"], rms_eps=float(d["rms_eps"]),
                       rope_base=float(d["rope_base"]), window=d.get("window"), max_seq=d["max_seq"])


@dataclass
class TrainConfig:
    """`ojas_model::TrainConfig` (ojas-model/src/trainer.rs): the fields its JSON carries."""
    seq_len: int
    batch: int
    accum: int = 1
    adam_lr: float = 6e-4
    matrix_lr: float = 0.025
    grad_clip: float = 1.0
    data_seed: int = 0
    schedule: str = "cosine"
    decay_frac: float = 0.0
    total_steps: int = 0
    warmup_steps: int = 0
    chunk_rows: int = 1024
    chunk_cols: int = 8192
    ignore_index: Optional[int] = None
    on_nonfinite: str = "abort"
    muon_ns5_bf16: bool = False

    def to_json(self) -> str:
        """`TrainConfig::to_json` (trainer.rs:179-221): sorted keys, optional ones absent at their defaults."""
        ns5 = '"muon_ns5":"bf16",' if self.muon_ns5_bf16 else ""
        return (f'{{"accum":{self.accum},"adam_lr":{rust_f64(self.adam_lr)},"batch":{self.batch},'
                f'"chunk_cols":{self.chunk_cols},"chunk_rows":{self.chunk_rows},"data_seed":{self.data_seed},'
                f'"decay_frac":{rust_f64(self.decay_frac)},"grad_clip":{rust_f64(self.grad_clip)},'
                f'"ignore":{"true" if self.ignore_index is not None else "false"},"ignore_index":{self.ignore_index or 0},'
                f'"matrix_lr":{rust_f64(self.matrix_lr)},{ns5}"on_nonfinite":{json.dumps(self.on_nonfinite)},'
                f'"schedule":{json.dumps(self.schedule)},"seq_len":{self.seq_len},"total_steps":{self.total_steps},'
                f'"warmup_steps":{self.warmup_steps}}}')


def save_checkpoint(trainer: NanolabTrainer, directory, cfg: TrainConfig, cursor: Tuple[int, int] = (0, 0),
                    run: str = "run", tokenizer_hash: bytes = bytes(32), git_sha: bytes = bytes(20)):
    """`Trainer::save` (ojas-model/src/checkpoint.rs:540-640): `model.safetensors` (F32 weights, table
    order, metadata ojas.spec / ojas.step / ojas.run), `optim.safetensors` (`muon.<name>`,
    `adam_m.<name>`, `adam_v.<name>` of every trained parameter, table order) and `state.ojck`
    (checkpoint v1 with empty tensor sections: step, cursor, the sampler's rng_state, and the config
    object {"format","run","spec","train"}). One tensor is read back at a time."""
    from .data import rng_state_encode
    from .io import CheckpointV1, write_checkpoint, write_safetensors

    directory = Path(directory)
    directory.mkdir(parents=True, exist_ok=True)
    be, step = trainer.be, str(trainer.step)
    spec_json = spec_to_json(trainer.spec)
    write_safetensors(directory / MODEL_FILE, {n: be.download(trainer.params[n]) for n in trainer.names},
                      {"ojas.spec": spec_json, "ojas.step": step, "ojas.run": run})
    moments = {}
    for n in trainer.trainable:
        if n in trainer.muon:
            moments[f"muon.{n}"] = be.download(trainer.state[n][0])
        else:
            moments[f"adam_m.{n}"] = be.download(trainer.state[n][0])
            moments[f"adam_v.{n}"] = be.download(trainer.state[n][1])
    write_safetensors(directory / OPTIM_FILE, moments, {"ojas.step": step, "ojas.run": run})
    config = (f'{{"format":{json.dumps(STATE_FORMAT)},"run":{json.dumps(run)},"spec":{spec_json},'
              f'"train":{cfg.to_json()}}}')
    write_checkpoint(directory / STATE_FILE,
                     CheckpointV1(config=config.encode(), tokenizer_hash=tokenizer_hash, git_sha=git_sha,
                                  step=trainer.step, cursor=cursor, rng_state=rng_state_encode(cfg.data_seed)))


def resume_checkpoint(be: MiBackend, directory, cfg: TrainConfig, tokenizer_hash: bytes = bytes(32)):
    """`Trainer::resume_from` (ojas-model/src/checkpoint.rs:700-900): refuses unless step and run agree
    across the three files, the saved train config and tokenizer hash equal the caller's, the
    rng_state is the sampler's v1 layout with the caller's data_seed, and names, dtypes and shapes
    are exactly the expected ones. Returns (trainer, cursor, run)."""
    from .data import rng_state_decode
    from .io import IoError, SafeTensors, read_checkpoint

    directory = Path(directory)
    state = read_checkpoint(directory / STATE_FILE)
    if any(state.sections()):
        raise IoError("state.ojck: tensor sections are not empty")
    conf = json.loads(state.config)
    if conf.get("format") != STATE_FORMAT:
        raise IoError(f"state.ojck: format {conf.get('format')!r}, expected {STATE_FORMAT!r}")
    if conf.get("train") != json.loads(cfg.to_json()):
        raise IoError("state.ojck: the saved train config is not the caller's")
    if state.tokenizer_hash != tokenizer_hash:
        raise IoError("state.ojck: tokenizer hash differs from the caller's")
    if rng_state_decode(state.rng_state) != cfg.data_seed:
        raise IoError("state.ojck: rng_state seed differs from the caller's data_seed")
    model, optim = SafeTensors(directory / MODEL_FILE), SafeTensors(directory / OPTIM_FILE)
    run = conf.get("run")
    for what, meta in ((MODEL_FILE, model.metadata()), (OPTIM_FILE, optim.metadata())):
        if meta.get("ojas.step") != str(state.step) or meta.get("ojas.run") != run:
            raise IoError(f"{what}: step / run disagree with state.ojck")
    spec = spec_from_json(model.metadata().get("ojas.spec", ""))
    if json.loads(spec_to_json(spec)) != conf.get("spec"):
        raise IoError("model.safetensors: ojas.spec disagrees with state.ojck")
    shapes = spec.param_shapes()
    if model.names() != sorted(spec.param_names(), key=str.encode):
        raise IoError("model.safetensors: tensor names are not the model's")
    host = {}
    for n in spec.param_names():
        info = model.info(n)
        if info.dtype != "F32" or info.shape != tuple(shapes[n]):
            raise IoError(f"model.safetensors: {n} is {info.dtype} {info.shape}, expected F32 {tuple(shapes[n])}")
        host[n] = model.read(n)
    trainer = NanolabTrainer(be, spec, host, adam_lr=cfg.adam_lr, matrix_lr=cfg.matrix_lr, grad_clip=cfg.grad_clip,
                             ns5_bf16=cfg.muon_ns5_bf16)
    expected = []
    for n in trainer.trainable:
        expected += [f"muon.{n}"] if n in trainer.muon else [f"adam_m.{n}", f"adam_v.{n}"]
    if optim.names() != sorted(expected, key=str.encode):
        raise IoError("optim.safetensors: tensor names are not the trained parameters' moments")
    for n in trainer.trainable:
        keys = [f"muon.{n}"] if n in trainer.muon else [f"adam_m.{n}", f"adam_v.{n}"]
        for slot, key in enumerate(keys):
            info = optim.info(key)
            if info.dtype != "F32" or info.shape != tuple(shapes[n]):
                raise IoError(f"optim.safetensors: {key} is {info.dtype} {info.shape}")
            trainer.state[n][slot] = be.upload(optim.read(key))
    trainer.step = state.step
    return trainer, state.cursor, run
