"""`GptTrainer`: ctypes binding of the host-side step driver (libojas_gpt.so).

The driver plays the part of the reference's generic callers (`Tape<B>` and
`Trainer<B>`, ojas-model/src/trainer.rs:754-1046) for the GPT-2-shaped graph of
the benchmark configurations; see include/ojas_gpt.h. No arithmetic lives here.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path
from typing import List, Optional, Tuple

import numpy as np

from .backend import OK, AdamWConfig, MiBackend, OjasError

LIB_PATH = Path(__file__).resolve().parent / "libojas_gpt.so"


class GptConfig(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in
                ("layers", "d_model", "heads", "head_dim", "mlp", "ctx", "vocab", "batch", "gelu_tanh", "bf16")]


# The benchmark configurations (BASELINE.json configs[0] and configs[2]).
def config_tiny_f32() -> GptConfig:
    return GptConfig(4, 256, 4, 64, 1024, 256, 8192, 8, 0, 0)


def config_gpt124m_bf16() -> GptConfig:
    return GptConfig(12, 768, 12, 64, 3072, 1024, 50304, 16, 0, 1)


def matmul_params(c: GptConfig) -> int:
    """Weights that take part in matmuls: L(4 d^2 + 2 d mlp) + V d (tied head)."""
    return c.layers * (4 * c.d_model * c.d_model + 2 * c.d_model * c.mlp) + c.vocab * c.d_model


def step_flops(c: GptConfig) -> float:
    """Algorithmic FLOPs of one training step: 6 N P_mm for the matmuls plus
    causal attention counted at half the square (forward 2, backward 5 products)."""
    n = c.batch * c.ctx
    matmul = 6.0 * n * matmul_params(c)
    attention = 7.0 * c.batch * c.heads * c.ctx * c.ctx * c.head_dim * c.layers
    return matmul + attention


class GptTrainer:
    def __init__(self, backend: MiBackend, config: GptConfig):
        if not LIB_PATH.exists():
            raise OjasError(10, f"{LIB_PATH} is not built; run __graft_entry__.build()")
        self._lib = C.CDLL(str(LIB_PATH))
        self._lib.ogpt_param_count.restype = C.c_uint64
        self._lib.ogpt_param_len.restype = C.c_uint64
        self._lib.ogpt_steps.restype = C.c_uint64
        self._lib.ogpt_device_bytes.restype = C.c_uint64
        self.backend = backend
        self.config = config
        h = C.c_void_p()
        rc = self._lib.ogpt_create(backend._ctx, C.byref(config), C.byref(h))
        self._h = h if rc == OK else None
        backend._check(rc)

    def close(self):
        if self._h:
            self._lib.ogpt_destroy(self._h)
            self._h = None

    def param_lens(self) -> List[int]:
        n = int(self._lib.ogpt_param_count(self._h))
        return [int(self._lib.ogpt_param_len(self._h, C.c_uint64(i))) for i in range(n)]

    def set_params(self, params):
        for i, p in enumerate(params):
            p = np.ascontiguousarray(p, np.float32).reshape(-1)
            self.backend._check(self._lib.ogpt_set_param(self._h, C.c_uint64(i), p.ctypes.data_as(C.c_void_p)))

    def _get(self, fn) -> List[np.ndarray]:
        out = []
        for i, n in enumerate(self.param_lens()):
            a = np.empty(n, np.float32)
            self.backend._check(fn(self._h, C.c_uint64(i), a.ctypes.data_as(C.c_void_p)))
            out.append(a)
        return out

    def params(self) -> List[np.ndarray]:
        return self._get(self._lib.ogpt_get_param)

    def grads(self) -> List[np.ndarray]:
        return self._get(self._lib.ogpt_get_grad)

    def state(self, slot: int) -> List[np.ndarray]:
        """Every parameter's optimizer state: slot 0 the first moment (Muon's momentum for a matrix
        under `step_hybrid`), slot 1 AdamW's second moment."""
        return self._get(lambda h, i, a: self._lib.ogpt_get_state(h, i, C.c_uint32(slot), a))

    def set_state(self, slot: int, arrays):
        for i, a in enumerate(arrays):
            a = np.ascontiguousarray(a, np.float32).reshape(-1)
            self.backend._check(self._lib.ogpt_set_state(self._h, C.c_uint64(i), C.c_uint32(slot),
                                                         a.ctypes.data_as(C.c_void_p)))

    def set_steps(self, steps: int):
        self.backend._check(self._lib.ogpt_set_steps(self._h, C.c_uint64(steps)))

    def init(self, seed: int):
        self.backend._check(self._lib.ogpt_init(self._h, C.c_uint64(seed)))

    def set_batch(self, ids: np.ndarray, targets: np.ndarray):
        ids = np.ascontiguousarray(ids, np.uint32).reshape(-1)
        targets = np.ascontiguousarray(targets, np.uint32).reshape(-1)
        n = self.config.batch * self.config.ctx
        if ids.size != n or targets.size != n:
            raise OjasError(1, f"set_batch: expected {n} ids and targets")
        self.backend._check(self._lib.ogpt_set_batch(self._h, ids.ctypes.data_as(C.c_void_p),
                                                     targets.ctypes.data_as(C.c_void_p)))

    def loss_and_grads(self) -> float:
        loss = C.c_float()
        self.backend._check(self._lib.ogpt_loss_and_grads(self._h, C.byref(loss)))
        return float(loss.value)

    def step(self, adamw: AdamWConfig, grad_clip: float = 1.0) -> Tuple[float, float]:
        """One optimizer step; returns (loss, grad_norm) like `StepReport` (trainer.rs:281-297)."""
        loss, norm = C.c_float(), C.c_float()
        self.backend._check(self._lib.ogpt_step(self._h, C.byref(adamw), C.c_float(grad_clip), C.byref(loss),
                                                C.byref(norm)))
        return float(loss.value), float(norm.value)

    def step_hybrid(self, muon, adamw: AdamWConfig, grad_clip: float = 1.0) -> Tuple[float, float]:
        """One step with Muon-NS5 on the hidden matrices and AdamW on tables and norms
        (`Trainer::apply`, trainer.rs:1004-1028); `muon` is a `MuonNs5Config`."""
        loss, norm = C.c_float(), C.c_float()
        self.backend._check(self._lib.ogpt_step_hybrid(self._h, C.byref(muon), C.byref(adamw), C.c_float(grad_clip),
                                                       C.byref(loss), C.byref(norm)))
        return float(loss.value), float(norm.value)

    def steps(self) -> int:
        return int(self._lib.ogpt_steps(self._h))

    def device_bytes(self) -> int:
        return int(self._lib.ogpt_device_bytes(self._h))


def synthetic_batch(c: GptConfig, seed: int) -> Tuple[np.ndarray, np.ndarray]:
    """Token ids uniform over the vocabulary from SplitMix64(seed) (`next_u64 % V`,
    as `SplitMix64::below`, ojas-test-support/src/rng.rs:26-28), drawn as windows of
    ctx + 1 tokens; targets are the ids shifted by one (ojas-data/src/sampler.rs:3-5)."""
    mask = (1 << 64) - 1
    state = seed & mask
    out = np.empty((c.batch, c.ctx + 1), np.uint32)
    flat = out.reshape(-1)
    for i in range(flat.size):
        state = (state + 0x9E3779B97F4A7C15) & mask
        z = state
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
        z ^= z >> 31
        flat[i] = z % c.vocab
    return np.ascontiguousarray(out[:, :-1]), np.ascontiguousarray(out[:, 1:])
