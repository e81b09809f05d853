"""`LoraTrainer`: ctypes binding of the LoRA fine-tune step driver (libojas_lora.so).

The driver plays the part of the reference's callers for this workload: `Tape<B>` over the
`lora_linear` graph (ojas-model/src/lora.rs:292-344) on the q, k, v and o projections of a frozen
int8 decoder, and the trainer step (ojas-model/src/trainer.rs:754-1046) on the adapters only; see
include/ojas_lora.h. No arithmetic lives here.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path
from typing import List, Tuple

import numpy as np

from .backend import OK, AdamWConfig, MiBackend, OjasError

LIB_PATH = Path(__file__).resolve().parent / "libojas_lora.so"

# Base matrices of a block, in `set_matrix` order, and the adapters of a block, in index order.
BASE_MATRICES = ("wq", "wk", "wv", "wo", "wgate", "wup", "wdown")
ADAPTERS = ("Aq", "Bq", "Ak", "Bk", "Av", "Bv", "Ao", "Bo")


class LoraConfig(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("layers", "d_model", "heads", "head_dim", "hidden", "vocab", "batch", "seq",
                                          "rank")] + [("rms_eps", C.c_float), ("lora_scale", C.c_float),
                                                      ("rope_base", C.c_double)]


def config_lora1b() -> LoraConfig:
    """BASELINE.json configs[4]: 16 layers, d 2048, 16 heads of 128, SwiGLU 8192, ctx 2048, batch 4,
    vocabulary 32000, rank 16 (alpha = rank)."""
    return LoraConfig(16, 2048, 16, 128, 8192, 32000, 4, 2048, 16, 1e-6, 1.0, 10000.0)


def base_params(c: LoraConfig) -> int:
    """Frozen weights that take part in matmuls: L (4 d^2 + 3 d hidden) + V d (tied head)."""
    return c.layers * (4 * c.d_model * c.d_model + 3 * c.d_model * c.hidden) + c.vocab * c.d_model


def adapter_params(c: LoraConfig) -> int:
    return c.layers * 8 * c.rank * c.d_model


def step_flops(c: LoraConfig) -> float:
    """Algorithmic FLOPs of one step: forward and input gradient of the frozen base (4 N P), the
    adapters' three products each way (6 N P_adapter), causal attention at half the square
    (forward 2, backward 5 products)."""
    n = c.batch * c.seq
    attention = 7.0 * c.batch * c.heads * c.seq * c.seq * c.head_dim * c.layers
    return 4.0 * n * base_params(c) + 6.0 * n * adapter_params(c) + attention


class LoraTrainer:
    def __init__(self, backend: MiBackend, config: LoraConfig):
        if not LIB_PATH.exists():
            raise OjasError(10, f"{LIB_PATH} is not built; run __graft_entry__.build()")
        self._lib = C.CDLL(str(LIB_PATH))
        for name in ("olora_adapter_count", "olora_adapter_len", "olora_steps", "olora_device_bytes"):
            getattr(self._lib, name).restype = C.c_uint64
        self.backend = backend
        self.config = config
        h = C.c_void_p()
        rc = self._lib.olora_create(backend._ctx, C.byref(config), C.byref(h))
        self._h = h if rc == OK else None
        backend._check(rc)

    def close(self):
        if self._h:
            self._lib.olora_destroy(self._h)
            self._h = None

    # ---- the frozen base ----
    def set_embedding(self, table: np.ndarray):
        table = np.ascontiguousarray(table, np.float32)
        self.backend._check(self._lib.olora_set_embedding(self._h, table.ctypes.data_as(C.c_void_p)))

    def set_norm(self, layer: int, which: int, w: np.ndarray):
        w = np.ascontiguousarray(w, np.float32)
        self.backend._check(self._lib.olora_set_norm(self._h, C.c_uint32(layer), C.c_uint32(which),
                                                     w.ctypes.data_as(C.c_void_p)))

    def set_matrix(self, layer: int, which: int, codes: np.ndarray, scales: np.ndarray):
        codes, scales = np.ascontiguousarray(codes, np.int8), np.ascontiguousarray(scales, np.float32)
        self.backend._check(self._lib.olora_set_matrix(self._h, C.c_uint32(layer), C.c_uint32(which),
                                                       codes.ctypes.data_as(C.c_void_p),
                                                       scales.ctypes.data_as(C.c_void_p)))

    def init_base(self, seed: int, std: float = 0.02):
        self.backend._check(self._lib.olora_init_base(self._h, C.c_uint64(seed), C.c_float(std)))

    # ---- the adapters ----
    def adapter_lens(self) -> List[int]:
        n = int(self._lib.olora_adapter_count(self._h))
        return [int(self._lib.olora_adapter_len(self._h, C.c_uint64(i))) for i in range(n)]

    def set_adapters(self, adapters):
        for i, a in enumerate(adapters):
            a = np.ascontiguousarray(a, np.float32).reshape(-1)
            self.backend._check(self._lib.olora_set_adapter(self._h, C.c_uint64(i), a.ctypes.data_as(C.c_void_p)))

    def _get(self, fn) -> List[np.ndarray]:
        out = []
        for i, n in enumerate(self.adapter_lens()):
            a = np.empty(n, np.float32)
            self.backend._check(fn(self._h, C.c_uint64(i), a.ctypes.data_as(C.c_void_p)))
            out.append(a)
        return out

    def adapters(self) -> List[np.ndarray]:
        return self._get(self._lib.olora_get_adapter)

    def grads(self) -> List[np.ndarray]:
        return self._get(self._lib.olora_get_grad)

    def init_adapters(self, seed: int, std: float = 0.02):
        self.backend._check(self._lib.olora_init_adapters(self._h, C.c_uint64(seed), C.c_float(std)))

    # ---- steps ----
    def set_batch(self, ids: np.ndarray, targets: np.ndarray):
        ids = np.ascontiguousarray(ids, np.uint32).reshape(-1)
        targets = np.ascontiguousarray(targets, np.uint32).reshape(-1)
        n = self.config.batch * self.config.seq
        if ids.size != n or targets.size != n:
            raise OjasError(1, f"set_batch: expected {n} ids and targets")
        self.backend._check(self._lib.olora_set_batch(self._h, ids.ctypes.data_as(C.c_void_p),
                                                      targets.ctypes.data_as(C.c_void_p)))

    def loss_and_grads(self) -> float:
        loss = C.c_float()
        self.backend._check(self._lib.olora_loss_and_grads(self._h, C.byref(loss)))
        return float(loss.value)

    def step(self, adamw: AdamWConfig, grad_clip: float = 1.0) -> Tuple[float, float]:
        loss, norm = C.c_float(), C.c_float()
        self.backend._check(self._lib.olora_step(self._h, C.byref(adamw), C.c_float(grad_clip), C.byref(loss),
                                                 C.byref(norm)))
        return float(loss.value), float(norm.value)

    def steps(self) -> int:
        return int(self._lib.olora_steps(self._h))

    def device_bytes(self) -> int:
        return int(self._lib.olora_device_bytes(self._h))
