"""CPU restatement of the reference's fresh parameter init (test infrastructure: the parity checker
for `onano_init_reference`; nothing in the product imports it).

Follows ojas-model/src/init.rs:15-114 and the parameter table of ojas-model/src/names.rs:188-300 in
plain Python integers and `math` (the C library's log, sin and cos, as Rust's std uses the
platform's). Pure-Python loops: meant for parameters of up to a few hundred thousand values.

Pinned by (tests/test_init_reference.py): FNV-1a's published vectors (init.rs:127-133), the pinned
SplitMix64 reference stream (ojas-data/src/rng.rs:58-66), exact zeros and ones, the identities
Box-Muller fixes (z0^2 + z1^2 = -2 ln u1 recomputed from the raw draws, the cosine branch first),
sample moments, and independence of the streams of two names. No fixture of the reference holds
`init_params` bits, so beyond those checks its value bits are parity unpinned.
"""
from __future__ import annotations

import math
from typing import Iterator, List, Tuple

import numpy as np

MASK = (1 << 64) - 1
INIT_STD_F32 = float(np.float32(0.02))  # names.rs:16, widened to f64 as init.rs:108 does

ZEROS, ONES, NORMAL = 0, 1, 2


def fnv1a(data: bytes) -> int:
    """init.rs:15-29."""
    h = 0xCBF29CE484222325
    for byte in data:
        h = ((h ^ byte) * 0x00000100000001B3) & MASK
    return h


class CounterRng:
    """SplitMix64 (ojas-kernels/src/rng.rs; re-exported as CounterRng, ojas-data/src/rng.rs:10)."""

    def __init__(self, seed: int):
        self.state = seed & MASK

    def next_u64(self) -> int:
        self.state = (self.state + 0x9E3779B97F4A7C15) & MASK
        z = self.state
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK
        return z ^ (z >> 31)


def normal_stream(seed: int) -> Iterator[float]:
    """init.rs:35-59: pairs from Box-Muller, the cosine branch first, the sine branch next."""
    rng = CounterRng(seed)
    ulp53 = 1.0 / float(1 << 53)
    while True:
        u1 = float((rng.next_u64() >> 11) + 1) * ulp53
        u2 = float(rng.next_u64() >> 11) * ulp53
        radius = math.sqrt(-2.0 * math.log(u1))
        angle = math.tau * u2
        yield radius * math.cos(angle)
        yield radius * math.sin(angle)


def init_values(name: str, n: int, init: int, seed: int, std: float = INIT_STD_F32) -> np.ndarray:
    """init.rs:75-112."""
    if init == ZEROS:
        return np.zeros(n, np.float32)
    if init == ONES:
        return np.ones(n, np.float32)
    if not (math.isfinite(std) and std > 0.0):
        raise ValueError(f"{name}: std {std} is not positive and finite")
    stream = normal_stream(seed ^ fnv1a(name.encode()))
    return np.array([std * next(stream) for _ in range(n)], np.float64).astype(np.float32)


def param_table(n_layer: int, n_embd: int, n_head: int, n_kv_head: int, head_dim: int, hidden: int,
                vocab: int) -> List[Tuple[str, Tuple[int, ...], int]]:
    """names.rs:188-300: (name, shape, init rule) in canonical order."""
    d, q, kv = n_embd, n_head * head_dim, n_kv_head * head_dim
    rows = [("tok_emb.weight", (vocab, d), NORMAL)]
    for i in range(n_layer):
        p, m = f"blocks.{i}", f"blocks.{i}.mixer"
        rows += [
            (f"{p}.norm1.weight", (d,), ONES),
            (f"{m}.q_proj.weight", (q, d), NORMAL),
            (f"{m}.k_proj.weight", (kv, d), NORMAL),
            (f"{m}.v_proj.weight", (kv, d), NORMAL),
            (f"{m}.o_proj.weight", (d, q), ZEROS),
            (f"{m}.q_norm.weight", (head_dim,), ONES),
            (f"{m}.k_norm.weight", (head_dim,), ONES),
            (f"{m}.gate.weight", (n_head, d), NORMAL),
            (f"{m}.gate.bias", (n_head,), ZEROS),
            (f"{m}.vr_lambda", (1,), ZEROS),
            (f"{p}.norm2.weight", (d,), ONES),
            (f"{p}.ffn.gate.weight", (hidden, d), NORMAL),
            (f"{p}.ffn.up.weight", (hidden, d), NORMAL),
            (f"{p}.ffn.down.weight", (d, hidden), ZEROS),
        ]
    rows.append(("norm_f.weight", (d,), ONES))
    return rows
