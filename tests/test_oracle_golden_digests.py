"""The oracle against the reference's bit-exact digests.

The fixture generator below restates ojas-cpu/tests/exact_golden.rs:60-199
(seeds, shapes, scales, call order); the digests in
tests/golden/exact_golden_digests.json are that file's GOLDEN table (:206-276).
`ce_loss` depends on the platform's libm `ln` and was recorded on Apple
silicon only (exact_golden.rs:201-204), so it is not compared.
"""
import json
from pathlib import Path

import numpy as np
import pytest

import oracle_api as orc

GOLDEN = json.loads((Path(__file__).parent / "golden" / "exact_golden_digests.json").read_text())["digests"]

LINEAR = [(1, 1, 1), (3, 5, 9), (73, 11, 13), (127, 67, 131), (64, 128, 96), (70, 80, 100), (257, 129, 65),
          (65, 257, 129), (129, 65, 257), (97, 255, 95), (33, 1000, 17), (200, 300, 520)]


def compute_digests():
    out = {}
    for i, (rows, kin, nout) in enumerate(LINEAR):
        rng = orc.SplitMix64(100 + i)
        x = rng.vec(rows * kin, 0.5).reshape(rows, kin)
        w = rng.vec(nout * kin, 0.5).reshape(nout, kin)
        gy = rng.vec(rows * nout, 0.5).reshape(rows, nout)
        y = orc.linear_forward(x, w)
        gx, gw = orc.linear_backward(x, w, gy)
        tag = f"{rows}x{kin}x{nout}"
        out[f"linear_fwd {tag}"] = orc.fnv(y)
        out[f"linear_gx {tag}"] = orc.fnv(gx)
        out[f"linear_gw {tag}"] = orc.fnv(gw)
    for i, (rows, cols) in enumerate([(64, 48), (48, 64), (130, 70), (97, 97)]):
        rng = orc.SplitMix64(200 + i)
        p = rng.vec(rows * cols, 0.1).reshape(rows, cols)
        g = rng.vec(rows * cols, 0.1).reshape(rows, cols)
        m = rng.vec(rows * cols, 0.01).reshape(rows, cols)
        p2, m2 = orc.muon_ns5_step(p, g, m)  # MuonNs5Config::nanolab_default (backend.rs:559-568)
        out[f"muon_p {rows}x{cols}"] = orc.fnv(p2)
        out[f"muon_m {rows}x{cols}"] = orc.fnv(m2)
    for i, shape in enumerate([[2, 3, 33, 24], [1, 2, 300, 64], [2, 2, 64, 16]]):
        n = int(np.prod(shape))
        rng = orc.SplitMix64(300 + i)
        q, k, v, gy = (rng.vec(n, 0.5).reshape(shape) for _ in range(4))
        y, lse = orc.causal_sdpa_forward(q, k, v)
        gq, gk, gv = orc.causal_sdpa_backward(q, k, v, y, lse, gy)
        tag = "[" + ", ".join(str(s) for s in shape) + "]"
        for name, val in (("fwd", y), ("lse", lse), ("gq", gq), ("gk", gk), ("gv", gv)):
            out[f"sdpa_{name} {tag}"] = orc.fnv(val)
    rows, dim = 300, 256
    rng = orc.SplitMix64(400)
    x = rng.vec(rows * dim, 1.0).reshape(rows, dim)
    w = (np.float32(1.0) + rng.vec(dim, 0.1)).astype(np.float32)
    gy = rng.vec(rows * dim, 1.0).reshape(rows, dim)
    out["rms_fwd"] = orc.fnv(orc.rms_norm_forward(x, w, 1e-6))
    gx, gw = orc.rms_norm_backward(x, w, gy, 1e-6)
    out["rms_gx"] = orc.fnv(gx)
    out["rms_gw"] = orc.fnv(gw)
    b, t, h, d = 2, 64, 4, 32
    rng = orc.SplitMix64(500)
    x = rng.vec(b * t * h * d, 1.0).reshape(b, t, h, d)
    cos = rng.vec(t * d, 1.0).reshape(t, d)
    sin = rng.vec(t * d, 1.0).reshape(t, d)
    out["rope_fwd"] = orc.fnv(orc.rope_forward(x, cos, sin))
    out["rope_bwd"] = orc.fnv(orc.rope_backward(x, cos, sin))
    rows, vocab = 257, 500
    rng = orc.SplitMix64(600)
    logits = rng.vec(rows * vocab, 4.0).reshape(rows, vocab)
    targets = np.array([7 if i % 11 == 3 else rng.below(vocab) for i in range(rows)], dtype=np.uint32)
    out["ce_grad"] = orc.fnv(orc.cross_entropy_mean_backward(logits, targets, ignore=7))
    n = 100_003
    rng = orc.SplitMix64(700)
    p = rng.vec(n, 1.0)
    g = rng.vec(n, 0.1)
    m1 = rng.vec(n, 0.01)
    m2 = np.abs(rng.vec(n, 0.01))
    p2, m1n, m2n = orc.adamw_step(p, g, m1, m2, 9, 3e-3, 0.9, 0.95, 1e-8, 0.1, exact=True)
    out["adamw_p"] = orc.fnv(p2)
    out["adamw_m1"] = orc.fnv(m1n)
    out["adamw_m2"] = orc.fnv(m2n)
    return out


@pytest.fixture(scope="module")
def digests():
    return compute_digests()


@pytest.mark.parametrize("name", [k for k in GOLDEN if k != "ce_loss"])
def test_digest_matches_reference(digests, name):
    assert f"{digests[name]:016x}" == GOLDEN[name], name


def test_all_68_platform_independent_digests_are_covered(digests):
    assert set(GOLDEN) - {"ce_loss"} == set(digests)
    assert len(digests) == 68


@pytest.mark.parametrize("threads", [2, 3, 7])
def test_digests_do_not_depend_on_thread_count(digests, threads):
    # exact_golden.rs:285-300: every thread count reproduces the same bits.
    before = orc.get_threads()
    orc.set_threads(threads)
    try:
        again = compute_digests()
    finally:
        orc.set_threads(before)
    assert again == digests
