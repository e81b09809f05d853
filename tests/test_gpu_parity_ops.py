"""GPU-vs-oracle parity, one op at a time, through the C ABI.

Template: the reference's GPU-vs-CPU gate (ojas-wgpu/tests/parity.rs:1-6,
tests/common/mod.rs:11,90-118): every op on shapes that break tiles (1x1,
primes, 63/64/65, 127/128/129; T = 1, 17, 257) against CPU Exact.

Tolerances (written where used):
  * integer / bit work (gather, casts, permute, argmax, top-k, embedding
    scatter-add order): bit-exact;
  * f32 tier: max|gpu - cpu| <= 1e-5 * max(1, max|cpu|)  (BASELINE "1e-5 relative");
  * bf16 tier: 2e-2 per element relative to max(1, max|cpu|), inputs rounded to
    bf16 on both sides so only accumulation order and output rounding differ.
"""
import numpy as np
import pytest

import oracle_api as orc

pytestmark = pytest.mark.gpu

F32_TOL = 1e-5
BF16_TOL = 2e-2


@pytest.fixture(scope="module")
def be():
    from ojas_amd.backend import MiBackend

    backend = MiBackend(0)
    assert backend.device_name().startswith("gfx950")
    yield backend
    backend.close()


def close(got, want, tol, what=""):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    scale = max(1.0, float(np.max(np.abs(want))) if want.size else 1.0)
    err = float(np.max(np.abs(got - want))) if want.size else 0.0
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    assert err <= tol * scale, f"{what}: max err {err:.3e} > {tol:.0e} * {scale:.3e}"


def rng_vec(seed, n, scale=1.0):
    return orc.SplitMix64(seed).vec(n, scale)


LINEAR_SHAPES = [(1, 1, 1), (3, 5, 9), (73, 11, 13), (127, 67, 131), (64, 128, 96), (63, 64, 65), (129, 127, 128),
                 (257, 129, 65), (33, 1000, 17), (200, 300, 520), (256, 256, 768)]


@pytest.mark.parametrize("rows,kin,nout", LINEAR_SHAPES)
def test_linear_f32(be, rows, kin, nout):
    print(f"linear f32 {rows}x{kin}x{nout}", flush=True)
    r = orc.SplitMix64(1000 + rows * 7 + kin)
    x = r.vec(rows * kin, 0.5).reshape(rows, kin)
    w = r.vec(nout * kin, 0.5).reshape(nout, kin)
    gy = r.vec(rows * nout, 0.5).reshape(rows, nout)
    dx, dw, dgy = be.upload(x), be.upload(w), be.upload(gy)
    y = be.download(be.linear_forward(dx, dw))
    close(y, orc.linear_forward(x, w), F32_TOL, "linear_forward")
    gx, gw = be.linear_backward(dx, dw, dgy)
    ogx, ogw = orc.linear_backward(x, w, gy)
    close(be.download(gx), ogx, F32_TOL, "linear_backward gx")
    close(be.download(gw), ogw, F32_TOL, "linear_backward gw")
    gx_only = be.linear_backward_input(dw, dgy)
    assert np.array_equal(be.download(gx_only), be.download(gx)), "linear_backward_input bits differ from gx"


@pytest.mark.parametrize("rows,kin,nout", LINEAR_SHAPES)
def test_linear_bf16(be, rows, kin, nout):
    from ojas_amd.backend import BF16, F32

    print(f"linear bf16 {rows}x{kin}x{nout}", flush=True)
    r = orc.SplitMix64(2000 + rows * 7 + kin)
    x = orc.round_bf16(r.vec(rows * kin, 0.5)).reshape(rows, kin)
    w = orc.round_bf16(r.vec(nout * kin, 0.5)).reshape(nout, kin)
    gy = orc.round_bf16(r.vec(rows * nout, 0.5)).reshape(rows, nout)
    dx, dw, dgy = be.upload(x, BF16), be.upload(w, BF16), be.upload(gy, BF16)
    # f32 output of bf16 operands: exact products, f32 accumulation -> f32-tier tolerance.
    close(be.download(be.linear_forward(dx, dw)), orc.linear_forward(x, w), F32_TOL, "linear_forward bf16->f32")
    ybf = be.download_f32(be.linear_forward(dx, dw, out_dtype=BF16))
    close(ybf, orc.linear_forward(x, w), BF16_TOL, "linear_forward bf16->bf16")
    gx, gw = be.linear_backward(dx, dw, dgy, gx_dtype=F32)
    ogx, ogw = orc.linear_backward(x, w, gy)
    close(be.download(gx), ogx, F32_TOL, "gx")
    close(be.download(gw), ogw, F32_TOL, "gw")


def test_linear_mixed_operands_and_gemm_accumulate(be):
    from ojas_amd.backend import BF16

    r = orc.SplitMix64(77)
    x = r.vec(70 * 96, 0.5).reshape(70, 96)
    w = orc.round_bf16(r.vec(40 * 96, 0.5)).reshape(40, 96)
    y = be.download(be.linear_forward(be.upload(x), be.upload(w, BF16)))
    close(y, orc.linear_forward(x, w), F32_TOL, "f32 input, bf16 weight")
    # gemm_acc: C += A.B continues the stored chain (gemm.rs:365-388).
    a = r.vec(50 * 30, 0.5).reshape(50, 30)
    b = r.vec(30 * 20, 0.5).reshape(30, 20)
    c0 = r.vec(50 * 20, 0.5).reshape(50, 20)
    dc = be.upload(c0)
    be.gemm(be.upload(a), (30, 1), be.upload(b), (20, 1), 50, 30, 20, c=dc)
    close(be.download(dc), orc.gemm(a, b, c0), F32_TOL, "gemm accumulate")


@pytest.mark.parametrize("rows,dim", [(1, 1), (5, 64), (300, 256), (17, 63), (9, 65), (130, 768), (4, 1000), (3, 2048)])
def test_rms_norm_f32(be, rows, dim):
    print(f"rms {rows}x{dim}", flush=True)
    r = orc.SplitMix64(400 + rows + dim)
    x = r.vec(rows * dim, 1.0).reshape(rows, dim)
    w = (np.float32(1.0) + r.vec(dim, 0.1)).astype(np.float32)
    gy = r.vec(rows * dim, 1.0).reshape(rows, dim)
    dx, dw, dgy = be.upload(x), be.upload(w), be.upload(gy)
    close(be.download(be.rms_norm_forward(dx, dw, 1e-6)), orc.rms_norm_forward(x, w, 1e-6), F32_TOL, "rms fwd")
    gx, gw = be.rms_norm_backward(dx, dw, dgy, 1e-6)
    ogx, ogw = orc.rms_norm_backward(x, w, gy, 1e-6)
    close(be.download(gx), ogx, F32_TOL, "rms gx")
    close(be.download(gw), ogw, F32_TOL, "rms gw")


def test_rms_norm_bf16_storage(be):
    from ojas_amd.backend import BF16

    rows, dim = 70, 768
    r = orc.SplitMix64(4242)
    x = orc.round_bf16(r.vec(rows * dim, 1.0)).reshape(rows, dim)
    w = (np.float32(1.0) + r.vec(dim, 0.1)).astype(np.float32)
    gy = orc.round_bf16(r.vec(rows * dim, 1.0)).reshape(rows, dim)
    y = be.download_f32(be.rms_norm_forward(be.upload(x, BF16), be.upload(w)))
    close(y, orc.rms_norm_forward(x, w), BF16_TOL, "rms fwd bf16")
    gx, gw = be.rms_norm_backward(be.upload(x, BF16), be.upload(w), be.upload(gy, BF16))
    ogx, ogw = orc.rms_norm_backward(x, w, gy)
    close(be.download_f32(gx), ogx, BF16_TOL, "rms gx bf16")
    close(be.download(gw), ogw, 1e-4, "rms gw (f32 sums of bf16 inputs)")


@pytest.mark.parametrize("tokens,vocab,dim", [(1, 1, 1), (12, 10, 8), (257, 500, 64), (1000, 37, 65), (64, 8192, 256)])
def test_embedding_is_bit_exact(be, tokens, vocab, dim):
    print(f"embedding {tokens} {vocab} {dim}", flush=True)
    r = orc.SplitMix64(31 + tokens)
    table = r.vec(vocab * dim, 1.0).reshape(vocab, dim)
    table[0, 0] = -0.0
    ids = np.array([r.below(vocab) for _ in range(tokens)], dtype=np.uint32)
    grad = r.vec(tokens * dim, 1.0).reshape(tokens, dim)
    out = be.download(be.embedding_forward(be.upload(table), be.upload(ids)))
    assert np.array_equal(out.view(np.uint32), orc.embedding_forward(table, ids).view(np.uint32))
    # Scatter-add in ascending token order: the same f32 sums, so the same bits.
    tg = be.download(be.embedding_backward(be.upload(ids), be.upload(grad), vocab))
    assert np.array_equal(tg.view(np.uint32), orc.embedding_backward(ids, grad, vocab).view(np.uint32))


def test_embedding_heavy_collisions_and_bf16_table(be):
    from ojas_amd.backend import BF16

    tokens, vocab, dim = 700, 3, 96
    r = orc.SplitMix64(5)
    ids = np.array([r.below(vocab) for _ in range(tokens)], dtype=np.uint32)
    grad = r.vec(tokens * dim, 1.0).reshape(tokens, dim)
    tg = be.download(be.embedding_backward(be.upload(ids), be.upload(grad), vocab))
    assert np.array_equal(tg.view(np.uint32), orc.embedding_backward(ids, grad, vocab).view(np.uint32))
    table = orc.round_bf16(r.vec(vocab * dim, 1.0)).reshape(vocab, dim)
    out = be.download(be.embedding_forward(be.upload(table, BF16), be.upload(ids)))
    assert np.array_equal(out.view(np.uint32), orc.embedding_forward(table, ids).view(np.uint32))


@pytest.mark.parametrize("tokens,vocab,dim", [(16384, 50, 48), (70000, 7, 8), (65, 1, 16)])
def test_embedding_backward_with_one_id_filling_the_batch(be, tokens, vocab, dim):
    """Rows with more than 64 tokens take the bitmap sort (windows of 32768 tokens: the second case
    crosses two window edges); one id that takes most of the batch must cost no more than its share
    and keep the ascending-token order of the sums bit for bit."""
    print(f"embedding long segments {tokens} {vocab} {dim}", flush=True)
    r = orc.SplitMix64(77 + tokens)
    ids = np.array([r.below(vocab) for _ in range(tokens)], dtype=np.uint32)
    ids[np.arange(tokens) % 3 != 0] = 0  # two thirds of the batch are id 0
    grad = r.vec(tokens * dim, 1.0).reshape(tokens, dim)
    tg = be.download(be.embedding_backward(be.upload(ids), be.upload(grad), vocab))
    assert np.array_equal(tg.view(np.uint32), orc.embedding_backward(ids, grad, vocab).view(np.uint32))


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("tokens,vocab,dim", [(12, 10, 8), (257, 500, 64), (1000, 37, 65), (4096, 50304, 768)])
def test_embedding_backward_accumulate_is_the_scatter_then_the_sum(be, tokens, vocab, dim, bf16):
    """`embedding_backward_accumulate` leaves in the table gradient the bits of `embedding_backward`
    into a fresh buffer followed by `accumulate_grad`: the oracle's scatter, then one f32 add per
    element, and rows that no id names keep their bits (a -0.0 planted there stays -0.0)."""
    from ojas_amd.backend import BF16

    print(f"embedding accumulate {tokens} {vocab} {dim} bf16={bf16}", flush=True)
    r = orc.SplitMix64(4242 + tokens)
    ids = np.array([r.below(vocab) for _ in range(tokens)], dtype=np.uint32)
    grad = r.vec(tokens * dim, 1.0).reshape(tokens, dim)
    if bf16:
        grad = orc.round_bf16(grad)
    base = r.vec(vocab * dim, 1.0).reshape(vocab, dim)
    unnamed = np.setdiff1d(np.arange(vocab), ids)
    if unnamed.size:
        base[unnamed[0], 0] = -0.0
    acc = be.upload(base)
    be.embedding_backward_accumulate(be.upload(ids), be.upload(grad, BF16) if bf16 else be.upload(grad), acc)
    want = base + orc.embedding_backward(ids, grad, vocab)
    if unnamed.size:
        want[unnamed] = base[unnamed]
    assert np.array_equal(be.download(acc).view(np.uint32), want.view(np.uint32))
    # ... and the two ops in sequence on the device give the same.
    two = be.upload(base)
    be.accumulate_grad(two, be.embedding_backward(be.upload(ids), be.upload(grad, BF16) if bf16 else be.upload(grad), vocab))
    named = np.unique(ids)
    assert np.array_equal(be.download(two)[named].view(np.uint32), want[named].view(np.uint32))


def test_embedding_out_of_range_id_is_reported_at_sync(be):
    from ojas_amd.backend import OUT_OF_RANGE, OjasError

    table = be.upload(np.ones((4, 8), np.float32))
    ids = be.upload(np.array([0, 9, 1], np.uint32))
    be.embedding_forward(table, ids)
    with pytest.raises(OjasError) as e:
        be.sync()
    assert e.value.code == OUT_OF_RANGE and "embedding_forward" in e.value.detail
    be.sync()  # the fault word was cleared


@pytest.mark.parametrize("rows,vocab", [(1, 1), (1, 2), (257, 500), (17, 1023), (5, 8192), (3, 50304)])
def test_cross_entropy_f32(be, rows, vocab):
    print(f"ce {rows}x{vocab}", flush=True)
    r = orc.SplitMix64(600 + rows)
    logits = r.vec(rows * vocab, 4.0).reshape(rows, vocab)
    targets = np.array([7 % vocab if i % 11 == 3 else r.below(vocab) for i in range(rows)], dtype=np.uint32)
    ignore = 7 if vocab > 8 and rows > 4 else None
    dl, dt = be.upload(logits), be.upload(targets)
    loss = be.download(be.cross_entropy_mean_forward(dl, dt, ignore))[0]
    want = orc.cross_entropy_mean_forward(logits, targets, ignore)
    assert abs(float(loss) - float(want)) <= F32_TOL * max(1.0, abs(float(want)))
    grad = be.download(be.cross_entropy_mean_backward(dl, dt, ignore))
    og = orc.cross_entropy_mean_backward(logits, targets, ignore)
    close(grad, og, F32_TOL, "ce grad")
    # Invariant: every valid row of the gradient sums to 0 (numerical_invariants.rs T1).
    assert np.max(np.abs(grad.astype(np.float64).sum(axis=1))) < 1e-6


def test_cross_entropy_collapse_row_and_all_ignored(be):
    from ojas_amd.backend import NON_FINITE, OjasError

    # A planted margin: the target logit dominates by 60, so the plain softmax
    # gradient of the target rounds to 0 and the collapse rule takes over.
    rows, vocab = 4, 300
    r = orc.SplitMix64(9)
    logits = r.vec(rows * vocab, 1.0).reshape(rows, vocab)
    targets = np.array([3, 100, 7, 299], np.uint32)
    logits[1, 100] = 60.0
    dl, dt = be.upload(logits), be.upload(targets)
    loss = be.download(be.cross_entropy_mean_forward(dl, dt))[0]
    want = orc.cross_entropy_mean_forward(logits, targets)
    assert abs(float(loss) - float(want)) <= F32_TOL * max(1.0, abs(float(want)))
    grad = be.download(be.cross_entropy_mean_backward(dl, dt))
    og = orc.cross_entropy_mean_backward(logits, targets)
    close(grad, og, F32_TOL, "ce grad")
    assert grad[1, 100] < 0.0, "collapse rule keeps a non-zero target gradient"
    rel = abs(grad[1, 100] - og[1, 100]) / abs(og[1, 100])
    assert rel < 1e-4, rel
    # All rows ignored: NonFinite, reported at the next sync.
    dt2 = be.upload(np.full(rows, 5, np.uint32))
    be.cross_entropy_mean_forward(dl, dt2, 5)
    with pytest.raises(OjasError) as e:
        be.sync()
    assert e.value.code == NON_FINITE and "cross_entropy_mean_forward" in e.value.detail


@pytest.mark.parametrize("rows,dim,vocab,chunk", [(10, 16, 300, (1024, 8192)), (70, 48, 1000, (32, 256)),
                                                  (129, 64, 513, (64, 8192)), (33, 24, 97, (7, 40)),
                                                  (130, 64, 1024, (64, 8192)), (9, 32, 32768, (1024, 32768))])
def test_linear_cross_entropy_matches_composed_path(be, rows, dim, vocab, chunk):
    print(f"linear_ce {rows} {dim} {vocab} {chunk}", flush=True)
    r = orc.SplitMix64(800 + rows)
    x = r.vec(rows * dim, 1.0).reshape(rows, dim)
    w = r.vec(vocab * dim, 0.3).reshape(vocab, dim)
    targets = np.array([r.below(vocab) for _ in range(rows)], np.uint32)
    targets[::5] = 2
    loss, gx, gw = be.linear_cross_entropy_mean(be.upload(x), be.upload(w), be.upload(targets), 2, chunk)
    oloss, ogx, ogw = orc.linear_cross_entropy_mean(x, w, targets, 2)
    assert abs(float(be.download(loss)[0]) - float(oloss)) <= F32_TOL * max(1.0, abs(float(oloss)))
    close(be.download(gx), ogx, F32_TOL, "fused gx")
    close(be.download(gw), ogw, F32_TOL, "fused gw")
    # Loss alone and one gradient alone (CeGrads::EACH).
    l2, g2, w2 = be.linear_cross_entropy_mean(be.upload(x), be.upload(w), be.upload(targets), 2, chunk, (False, False))
    assert g2 is None and w2 is None
    assert abs(float(be.download(l2)[0]) - float(oloss)) <= F32_TOL * max(1.0, abs(float(oloss)))
    _, g3, w3 = be.linear_cross_entropy_mean(be.upload(x), be.upload(w), be.upload(targets), 2, chunk, (True, False))
    assert w3 is None
    close(be.download(g3), ogx, F32_TOL, "fused gx alone")


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("rows,dim,vocab,chunk_rows", [(300, 64, 50304, 128), (70, 128, 8192, 1024), (40, 64, 8, 16)])
def test_linear_cross_entropy_one_read_kernel_agrees_with_the_two_kernels(be, bf16, rows, dim, vocab, chunk_rows):
    """With the whole vocabulary in one tile the statistics and gradient passes run as one kernel
    over one read of the logits. Same formulas as the two-kernel path (`ce_fused` 0); only the
    row sum's partial sums are grouped differently, so the two agree to 2e-6 (f32 rounding of a
    sum of positive terms) and, with bf16 logit gradients, to 1e-4 (the last bit of the row sum
    flips the bf16 rounding of a few of them), with ignored rows; both are within their gate of
    the oracle."""
    from ojas_amd.backend import BF16

    print(f"linear_ce one-read {rows} {dim} {vocab} bf16={bf16}", flush=True)
    r = orc.SplitMix64(900 + vocab)
    x = orc.round_bf16(r.vec(rows * dim, 1.0)).reshape(rows, dim)
    w = orc.round_bf16(r.vec(vocab * dim, 0.3)).reshape(vocab, dim)
    targets = np.array([r.below(vocab) for _ in range(rows)], np.uint32)
    targets[::7] = 3
    up = (lambda a: be.upload(a, BF16)) if bf16 else be.upload
    got = {}
    for fused in (1, 0):
        be.set_option("ce_fused", fused)
        loss, gx, gw = be.linear_cross_entropy_mean(up(x), up(w), be.upload(targets), 3, (chunk_rows, vocab))
        got[fused] = (be.download(loss), be.download(gx), be.download(gw))
    be.set_option("ce_fused", 1)
    for a, b in zip(got[1], got[0]):
        assert np.max(np.abs(a.astype(np.float64) - b)) <= (1e-4 if bf16 else 2e-6) * max(np.max(np.abs(b)), 1e-30)
    oloss, ogx, ogw = orc.linear_cross_entropy_mean(x, w, targets, 3)
    tol = BF16_TOL if bf16 else F32_TOL
    assert abs(float(got[1][0][0]) - float(oloss)) <= (1e-3 if bf16 else F32_TOL) * max(1.0, abs(float(oloss)))
    f32 = lambda a: be_f32(a)
    close(f32(got[1][1]), ogx, tol, "one-read gx")
    close(got[1][2], ogw, tol, "one-read gw")


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("poison", ["nan", "+inf", "-inf"])
@pytest.mark.parametrize("as_target", [False, True])
def test_linear_cross_entropy_one_read_kernel_reports_a_non_finite_logit(be, bf16, poison, as_target):
    """One vocabulary column of NaN, +inf or -inf logits (a poisoned weight row), either never the
    target (it enters the row sums) or every row's target (it is only ever the picked logit): the
    one-read kernel raises NonFinite either way, reported at the next sync."""
    from ojas_amd.backend import BF16, NON_FINITE, OjasError

    print(f"linear_ce one-read non-finite bf16={bf16} {poison} target={as_target}", flush=True)
    rows, dim, vocab, col = 24, 64, 520, 77
    r = orc.SplitMix64(77)
    x = orc.round_bf16(np.abs(r.vec(rows * dim, 1.0)) + 0.5).reshape(rows, dim)
    w = orc.round_bf16(r.vec(vocab * dim, 0.3)).reshape(vocab, dim)
    w[col] = {"nan": np.nan, "+inf": 3e38, "-inf": -3e38}[poison]
    targets = np.full(rows, col if as_target else 5, np.uint32)
    up = (lambda a: be.upload(a, BF16)) if bf16 else be.upload
    be.sync()
    be.linear_cross_entropy_mean(up(x), up(orc.round_bf16(w)), be.upload(targets), None, (rows, vocab))
    with pytest.raises(OjasError) as e:
        be.sync()
    assert e.value.code == NON_FINITE and "linear_cross_entropy" in e.value.detail, e.value.detail
    be.sync()


def be_f32(a):
    """Widens a downloaded bf16 bit array; f32 arrays pass through."""
    return (a.astype(np.uint32) << 16).view(np.float32) if a.dtype == np.uint16 else a


SDPA_SHAPES = [([2, 3, 33, 24], 3, None), ([1, 2, 300, 64], 2, None), ([2, 2, 64, 16], 2, None),
               ([1, 1, 1, 8], 1, None), ([1, 2, 17, 64], 2, None), ([1, 4, 257, 32], 2, None),
               ([1, 4, 130, 64], 1, 40), ([2, 2, 65, 128], 2, 7)]


@pytest.mark.parametrize("shape,hkv,window", SDPA_SHAPES)
def test_causal_sdpa_f32(be, shape, hkv, window):
    print(f"sdpa f32 {shape} hkv {hkv} window {window}", flush=True)
    b, h, t, d = shape
    r = orc.SplitMix64(300 + t + d)
    q = r.vec(b * h * t * d, 0.5).reshape(b, h, t, d)
    k = r.vec(b * hkv * t * d, 0.5).reshape(b, hkv, t, d)
    v = r.vec(b * hkv * t * d, 0.5).reshape(b, hkv, t, d)
    gy = r.vec(b * h * t * d, 0.5).reshape(b, h, t, d)
    oy, olse = orc.causal_sdpa_forward(q, k, v, window or 0)
    ogq, ogk, ogv = orc.causal_sdpa_backward(q, k, v, oy, olse, gy, window or 0)
    dq, dk, dv, dgy = be.upload(q), be.upload(k), be.upload(v), be.upload(gy)
    y, lse = be.causal_sdpa_forward(dq, dk, dv, window)
    close(be.download(y), oy, F32_TOL, "sdpa out")
    close(be.download(lse), olse, F32_TOL, "sdpa lse")
    gq, gk, gv = be.causal_sdpa_backward(dq, dk, dv, y, lse, dgy, window)
    close(be.download(gq), ogq, F32_TOL, "sdpa gq")
    close(be.download(gk), ogk, F32_TOL, "sdpa gk")
    close(be.download(gv), ogv, F32_TOL, "sdpa gv")


@pytest.mark.parametrize("shape,hkv,window", [([1, 4, 333, 64], 2, 100), ([2, 2, 200, 128], 2, None),
                                              ([1, 6, 129, 32], 3, 64), ([3, 2, 64, 16], 1, 5),
                                              ([1, 2, 1024, 64], 2, None)])
def test_causal_sdpa_f32_tiled_kernels_agree_with_the_row_kernels(be, shape, hkv, window):
    """The f32 tier's LDS-tiled attention kernels (head_dim 16 / 32 / 64 / 128) against the
    one-wave-per-row kernels (`sdpa_tiled` 0) and the oracle: several 64-row blocks, windows that
    start inside an earlier block, grouped heads, a ragged last block."""
    print(f"sdpa f32 tiled {shape} hkv {hkv} window {window}", flush=True)
    b, h, t, d = shape
    r = orc.SplitMix64(500 + t + d)
    q = r.vec(b * h * t * d, 0.5).reshape(b, h, t, d)
    k = r.vec(b * hkv * t * d, 0.5).reshape(b, hkv, t, d)
    v = r.vec(b * hkv * t * d, 0.5).reshape(b, hkv, t, d)
    gy = r.vec(b * h * t * d, 0.5).reshape(b, h, t, d)
    dq, dk, dv, dgy = be.upload(q), be.upload(k), be.upload(v), be.upload(gy)
    got = {}
    try:
        for tiled in (1, 0):
            be.set_option("sdpa_tiled", tiled)
            y, lse = be.causal_sdpa_forward(dq, dk, dv, window)
            gq, gk, gv = be.causal_sdpa_backward(dq, dk, dv, y, lse, dgy, window)
            got[tiled] = [be.download(x) for x in (y, lse, gq, gk, gv)]
    finally:
        be.set_option("sdpa_tiled", 1)
    for name, a, c in zip(("out", "lse", "gq", "gk", "gv"), got[1], got[0]):
        close(a, c, F32_TOL, "tiled against rows: " + name)
    if t <= 400:
        orc.set_threads(8)
        oy, olse = orc.causal_sdpa_forward(q, k, v, window or 0)
        ogq, ogk, ogv = orc.causal_sdpa_backward(q, k, v, oy, olse, gy, window or 0)
        for name, a, c in zip(("out", "lse", "gq", "gk", "gv"), got[1], (oy, olse, ogq, ogk, ogv)):
            close(a, c, F32_TOL, "tiled against the oracle: " + name)


def test_causal_sdpa_f32_with_more_planes_than_a_grid_axis_holds(be):
    """65536 (batch, head) planes of a short sequence: above the 65535 a grid's second axis takes,
    so the call goes to the row kernels (decided on the host) instead of failing at launch."""
    b, h, hkv, t, d = 8192, 8, 8, 8, 16
    print(f"sdpa f32 many planes {[b, h, t, d]}", flush=True)
    r = orc.SplitMix64(77)
    q, k, v, gy = (r.vec(b * h * t * d, 0.5).reshape(b, h, t, d) for _ in range(4))
    orc.set_threads(8)
    oy, olse = orc.causal_sdpa_forward(q, k, v, 0)
    ogq, ogk, ogv = orc.causal_sdpa_backward(q, k, v, oy, olse, gy, 0)
    dq, dk, dv, dgy = be.upload(q), be.upload(k), be.upload(v), be.upload(gy)
    y, lse = be.causal_sdpa_forward(dq, dk, dv, None)
    gq, gk, gv = be.causal_sdpa_backward(dq, dk, dv, y, lse, dgy, None)
    be.sync()
    for name, a, c in zip(("out", "lse", "gq", "gk", "gv"), (y, lse, gq, gk, gv), (oy, olse, ogq, ogk, ogv)):
        close(be.download(a), c, F32_TOL, "many planes: " + name)


def test_adamw_matches_fast_f32_contract_bitwise_and_exact_within_1e6(be):
    from ojas_amd.backend import AdamWConfig

    n = 100_003
    r = orc.SplitMix64(700)
    p, g, m1 = r.vec(n, 1.0), r.vec(n, 0.1), r.vec(n, 0.01)
    m2 = np.abs(r.vec(n, 0.01))
    dp, dg, dm1, dm2 = be.upload(p), be.upload(g), be.upload(m1), be.upload(m2)
    be.adamw_step(dp, dg, dm1, dm2, 9, AdamWConfig.nanolab(3e-3, 0.1))
    fp, fm1, fm2 = orc.adamw_step(p, g, m1, m2, 9, 3e-3, 0.9, 0.95, 1e-8, 0.1, exact=False)
    ep, em1, em2 = orc.adamw_step(p, g, m1, m2, 9, 3e-3, 0.9, 0.95, 1e-8, 0.1, exact=True)
    gp, gm1, gm2 = be.download(dp), be.download(dm1), be.download(dm2)
    # Same f32 operations in the same order as the CPU Fast contract (optim.rs:302-395).
    for got, fast, name in ((gp, fp, "p"), (gm1, fm1, "m1"), (gm2, fm2, "m2")):
        close(got, fast, 2e-7, f"adamw {name} vs Fast")
    # Fast-vs-Exact gate of the reference: 1e-6 (ojas-cpu/src/lib.rs:57).
    for got, exact, name in ((gp, ep, "p"), (gm1, em1, "m1"), (gm2, em2, "m2")):
        close(got, exact, 1e-6, f"adamw {name} vs Exact")


def test_adamw_writes_nothing_when_any_value_is_non_finite(be):
    from ojas_amd.backend import NON_FINITE, AdamWConfig, OjasError

    n = 5000
    r = orc.SplitMix64(3)
    p, g, m1 = r.vec(n, 1.0), r.vec(n, 0.1), r.vec(n, 0.01)
    m2 = np.abs(r.vec(n, 0.01))
    g[4321] = np.inf
    dp, dg, dm1, dm2 = be.upload(p), be.upload(g), be.upload(m1), be.upload(m2)
    be.adamw_step(dp, dg, dm1, dm2, 0, AdamWConfig.nanolab(1e-3, 0.0))
    with pytest.raises(OjasError) as e:
        be.sync()
    assert e.value.code == NON_FINITE and "adamw_step" in e.value.detail
    assert np.array_equal(be.download(dp), p) and np.array_equal(be.download(dm1), m1)
    assert np.array_equal(be.download(dm2), m2)


def test_adamw_bounded_form_skips_the_check_only_when_nothing_can_overflow(be):
    """`omx_adamw_step_bounded`: the bits of `omx_adamw_step` in every case; the flag reports stored
    values at or above 2^60; a caller's word is not taken when the scalars could overflow."""
    from ojas_amd.backend import NON_FINITE, U32, AdamWConfig, OjasError

    n = 70_001
    r = orc.SplitMix64(41)
    p, g, m1 = r.vec(n, 1.0), r.vec(n, 0.1), r.vec(n, 0.01)
    m2 = np.abs(r.vec(n, 0.01))
    cfg = AdamWConfig.nanolab(3e-3, 0.1)

    def run(pp, gg, mm1, mm2, step, config, bounded=None):
        dp, dg, dm1, dm2 = be.upload(pp), be.upload(gg), be.upload(mm1), be.upload(mm2)
        flag = be.upload(np.zeros(1, np.uint32))
        if bounded is None:
            be.adamw_step(dp, dg, dm1, dm2, step, config)
        else:
            be.adamw_step_bounded(dp, dg, dm1, dm2, step, config, bounded, flag)
        fault = None
        try:
            be.sync()
        except OjasError as e:
            fault = e
        return be.download(dp), be.download(dm1), be.download(dm2), int(be.download(flag)[0]), fault

    want = run(p, g, m1, m2, 3, cfg)
    for bounded in (True, False):
        got = run(p, g, m1, m2, 3, cfg, bounded)
        assert all(np.array_equal(a, b) for a, b in zip(got[:3], want[:3])) and got[3] == 0 and got[4] is None
    # A stored value at 2^61: finite, so the update is written; the flag says the next call must check.
    big = m1.copy()
    big[17] = 2.0 ** 61
    want = run(p, g, big, m2, 3, cfg)
    got = run(p, g, big, m2, 3, cfg, False)
    assert all(np.array_equal(a, b) for a, b in zip(got[:3], want[:3])) and got[3] == 1 and got[4] is None
    # A non-finite gradient (the caller sees a non-finite norm, so it does not vouch): refused, nothing
    # written, and the flag describes the inputs that stay in memory.
    bad = g.copy()
    bad[n - 1] = np.nan
    got = run(p, bad, m1, m2, 3, cfg, False)
    assert got[4] is not None and got[4].code == NON_FINITE
    assert np.array_equal(got[0], p) and np.array_equal(got[1], m1) and np.array_equal(got[2], m2) and got[3] == 0
    # A step size above 2^20: bounded inputs no longer rule out an overflow, so the caller's word is
    # not enough and the check runs: 1e30 * m / denom overflows and the update is refused.
    wild = AdamWConfig.nanolab(1e30, 0.0)
    got = run(p, np.full(n, 3e10, np.float32), m1, m2, 3, wild, True)
    assert got[4] is not None and got[4].code == NON_FINITE and np.array_equal(got[0], p)


def test_adamw_config_refusals(be):
    from ojas_amd.backend import NON_FINITE, OUT_OF_RANGE, AdamWConfig, OjasError

    t = be.upload(np.ones(8, np.float32))
    for cfg, code in ((AdamWConfig(1e-3, 1.0, 0.95, 1e-8, 0.0), OUT_OF_RANGE),
                      (AdamWConfig(-1e-3, 0.9, 0.95, 1e-8, 0.0), OUT_OF_RANGE),
                      (AdamWConfig(1e-3, 0.9, 0.95, 0.0, 0.0), OUT_OF_RANGE),
                      (AdamWConfig(float("nan"), 0.9, 0.95, 1e-8, 0.0), NON_FINITE)):
        with pytest.raises(OjasError) as e:
            be.adamw_step(t, t, t, t, 0, cfg)
        assert e.value.code == code
    with pytest.raises(OjasError) as e:
        be.adamw_step(t, t, t, t, 2**64 - 1, AdamWConfig.nanolab(1e-3, 0.0))
    assert e.value.code == OUT_OF_RANGE


def test_clip_grad_norm(be):
    r = orc.SplitMix64(11)
    grads = [r.vec(n, 1.0) for n in (1, 1000, 70_001, 300_000)]
    for max_norm in (1.0, 1e9):
        dg = [be.upload(g) for g in grads]
        norm = be.clip_grad_norm(dg, max_norm)
        onorm, oclipped = orc.clip_grad_norm(grads, max_norm)
        assert abs(norm - float(onorm)) <= 1e-6 * float(onorm)
        for got, want in zip(dg, oclipped):
            close(be.download(got), want, 1e-6, "clipped grad")
    # No clipping leaves the bits alone.
    dg = [be.upload(g) for g in grads]
    be.clip_grad_norm(dg, 1e9)
    for got, want in zip(dg, grads):
        assert np.array_equal(be.download(got), want)
    # A tensor that does not start on a 16-byte boundary (the kernel's one-by-one path).
    from ojas_amd.backend import F32, DeviceTensor

    base = be.upload(grads[3])
    view = DeviceTensor(be, base.ptr + 4, (grads[3].size - 1,), F32, owns=False)
    want = float(np.sqrt(np.sum(grads[3][1:].astype(np.float64) ** 2)))
    assert abs(be.clip_grad_norm([view], 1e9) - want) <= 1e-6 * want


def test_elementwise_ops(be):
    n = 70_001
    r = orc.SplitMix64(21)
    x, y = r.vec(n, 3.0), r.vec(n, 3.0)
    dx, dy = be.upload(x), be.upload(y)
    assert np.array_equal(be.download(be.residual_add_forward(dx, dy)), orc.residual_add(x, y))
    acc = be.upload(x)
    be.accumulate_grad(acc, dy)
    assert np.array_equal(be.download(acc), x + y)
    be.scale_grad(acc, 0.25)
    assert np.array_equal(be.download(acc), (x + y) * np.float32(0.25))
    close(be.download(be.gelu_erf_forward(dx)), orc.gelu_erf_forward(x), F32_TOL, "gelu erf")
    close(be.download(be.gelu_erf_backward(dx, dy)), orc.gelu_erf_backward_vec(x, y), F32_TOL, "gelu erf bwd")
    close(be.download(be.gelu_tanh_forward(dx)), orc.gelu_tanh_forward(x), F32_TOL, "gelu tanh")
    close(be.download(be.gelu_tanh_backward(dx, dy)), orc.gelu_tanh_backward_vec(x, y), F32_TOL, "gelu tanh bwd")


def test_casts_and_permute_are_bit_exact(be):
    from ojas_amd.backend import BF16

    r = orc.SplitMix64(55)
    x = r.vec(10_007, 100.0)
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0 + 2.0**-8, 1.0 + 2.0**-8 + 2.0**-20, 3.3895e38,
                        -3.4e38, 1e-40], np.float32)
    nan_payload = np.array([0x7F800001, 0xFFC12345, 0x7FBFFFFF], np.uint32).view(np.float32)
    x = np.concatenate([x, special, nan_payload]).astype(np.float32)
    dx = be.upload(x)
    assert np.array_equal(be.download(be.to_bf16(dx)), orc.to_bf16(x))
    assert np.array_equal(be.download(be.cast_bf16(dx)).view(np.uint32), orc.round_bf16(x).view(np.uint32))
    bits = orc.to_bf16(x)
    assert np.array_equal(be.download(be.to_f32(be.upload(bits))).view(np.uint32), orc.bf16_to_f32(bits).view(np.uint32))
    for shape in ([2, 3, 5, 7], [1, 64, 4, 64], [2, 17, 3, 16]):
        a = r.vec(int(np.prod(shape)), 1.0).reshape(shape)
        got = be.download(be.permute(be.upload(a), [0, 2, 1, 3]))
        assert np.array_equal(got, orc.permute_0213(a)) and np.array_equal(got, a.transpose(0, 2, 1, 3))
        gb = be.download(be.permute(be.upload(a, BF16), [0, 2, 1, 3]))
        assert np.array_equal(gb, orc.to_bf16(a).transpose(0, 2, 1, 3))


def test_bf16_rounding_carries_the_integer_rule_over_every_exponent_and_low_half(be):
    """The device rounds f32 to bf16 with its conversion instruction; the reference's rule is integer
    arithmetic on the bits (ojas-core/src/autocast.rs:70-96: round to nearest even on the dropped 16
    bits, a NaN keeps sign and payload and gains the quiet bit). Every combination of exponent
    (256, zero / denormals and infinity / NaN included), the kept mantissa's low bit and a full or
    an empty kept mantissa (ties to even, the carry into the exponent and into infinity), sign and
    all 65536 values of the dropped half: 134 M patterns, each equal to the rule written in numpy."""
    low = np.arange(1 << 16, dtype=np.uint32)
    for sign in (0, 1):
        for high in (0x00, 0x01, 0x7E, 0x7F):  # kept mantissa bits 22..16
            exps = np.arange(256, dtype=np.uint32)
            bits = ((sign << 31) | (exps[:, None] << 23) | (high << 16) | low[None, :]).astype(np.uint32).reshape(-1)
            x = bits.view(np.float32)
            nan = (bits & 0x7FFFFFFF) > 0x7F800000
            wide = bits.astype(np.uint64)
            rule = np.where(nan, (wide >> 16) | 0x40, (wide + 0x7FFF + ((wide >> 16) & 1)) >> 16).astype(np.uint16)
            got = be.download(be.to_bf16(be.upload(x)))
            assert np.array_equal(got, rule), (sign, high, int(np.flatnonzero(got != rule)[0]))
            rounded = be.download(be.cast_bf16(be.upload(x))).view(np.uint32)
            assert np.array_equal(rounded, rule.astype(np.uint32) << 16)
    # and the oracle's own cast is that rule
    x = (np.arange(1 << 20, dtype=np.uint32) * np.uint32(4099)).view(np.float32)
    bits = x.view(np.uint32)
    nan = (bits & 0x7FFFFFFF) > 0x7F800000
    rule = np.where(nan, (bits >> 16) | 0x40, (bits.astype(np.uint64) + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(orc.to_bf16(x), rule)


def test_argmax_and_topk_are_bit_exact(be):
    from ojas_amd.backend import NON_FINITE, OjasError

    r = orc.SplitMix64(91)
    for rows, cols, k in ((1, 1, 1), (7, 65, 5), (33, 1000, 50), (4, 50304, 8)):
        x = np.round(r.vec(rows * cols, 8.0)).reshape(rows, cols).astype(np.float32)  # many ties
        x[0, 0] = -0.0
        if cols > 3:
            x[0, 3] = 0.0
        dx = be.upload(x)
        assert np.array_equal(be.download(be.argmax_rows(dx)), orc.argmax_rows(x))
        xv = x.copy()
        if cols > 2:
            xv[-1, 1] = -np.inf  # allowed by top-k, sorts last
        vals, ids = be.topk_rows(be.upload(xv), k)
        ov, oi = orc.topk_rows(xv, k)
        assert np.array_equal(be.download(ids), oi)
        assert np.array_equal(be.download(vals).view(np.uint32), ov.view(np.uint32))
    bad = np.ones((2, 9), np.float32)
    bad[1, 4] = np.nan
    be.argmax_rows(be.upload(bad))
    with pytest.raises(OjasError) as e:
        be.sync()
    assert e.value.code == NON_FINITE and "argmax_rows" in e.value.detail


def test_deferred_non_finite_names_the_first_faulting_op(be):
    from ojas_amd.backend import NON_FINITE, OjasError

    x = np.ones((4, 8), np.float32)
    x[2, 3] = np.nan
    w = np.ones((5, 8), np.float32)
    dx, dw = be.upload(x), be.upload(w)
    y = be.linear_forward(dx, dw)            # first fault
    be.residual_add_forward(y, y)            # second fault, later in recording order
    with pytest.raises(OjasError) as e:
        be.download(y)
    assert e.value.code == NON_FINITE and e.value.detail == "linear_forward"


def test_budget_refuses_rather_than_clamps_and_unsupported_ops_name_themselves(be):
    from ojas_amd.backend import CAPACITY_EXCEEDED, UNSUPPORTED, MiBackend, OjasError

    small = MiBackend(0, budget_bytes=1 << 20)
    a = small.empty((100_000,))
    assert small.budget()["live"] == 400_000
    with pytest.raises(OjasError) as e:
        small.empty((200_000,))
    assert e.value.code == CAPACITY_EXCEEDED
    del a
    assert small.budget()["live"] == 0 and small.budget()["peak"] == 400_000
    with pytest.raises(OjasError) as e:
        small.layer_norm_forward(None, None)
    assert e.value.code == UNSUPPORTED and "layer_norm_forward" in e.value.detail
    small.close()


FLASH_SHAPES = [([1, 1, 1, 64], 1, None), ([1, 2, 17, 64], 2, None), ([2, 3, 64, 64], 3, None),
                ([1, 2, 128, 64], 2, None), ([1, 2, 129, 64], 1, None), ([1, 4, 300, 64], 2, None),
                ([2, 2, 257, 64], 2, 40), ([1, 2, 200, 64], 2, 1), ([1, 1, 1024, 64], 1, None),
                ([1, 2, 520, 64], 2, 130),
                # sequence ends at every position inside a 128-row block's waves, tiles and half tiles
                ([1, 1, 33, 64], 1, None), ([1, 1, 65, 64], 1, None), ([1, 2, 96, 64], 1, None),
                ([1, 1, 160, 64], 1, None), ([1, 1, 192, 64], 1, None), ([1, 2, 448, 64], 2, None),
                ([1, 1, 96, 128], 1, None), ([1, 1, 192, 128], 1, None),
                # head_dim 128 (the dK / dV pass walks a key block once per gradient)
                ([1, 1, 1, 128], 1, None), ([1, 2, 33, 128], 2, None), ([2, 2, 128, 128], 2, None),
                ([1, 4, 300, 128], 2, None), ([1, 2, 257, 128], 1, 40), ([1, 1, 1024, 128], 1, None),
                ([1, 2, 520, 128], 2, 130)]


@pytest.mark.parametrize("per_key", [0.002, 0.05, 0.7])
def test_causal_sdpa_bf16_scores_that_keep_growing(be, per_key):
    """Scores that rise steadily along the keys (by `per_key` nats per key: 0.13, 3.2 and 45 nats
    per 64-key tile). The forward moves the reference point of its exponents only when a row's
    maximum has grown by more than 8 binary orders, so the first case never moves it after the
    first tile, the second moves it every other tile and the third on every tile; output and
    log-sum-exp must not care. The gradients (which do not use the forward's reference point)
    are checked on the first two; on the third the keys reach 90 in magnitude and the bf16
    rounding of dS against them is past the bf16 gate whatever the kernel."""
    from ojas_amd.backend import BF16, F32

    b, h, t, d = 1, 2, 512, 64
    r = orc.SplitMix64(1234)
    unit = np.zeros(d, np.float32)
    unit[:8] = 1.0
    q = orc.round_bf16(np.broadcast_to(unit * 4.0, (b, h, t, d)) + r.vec(b * h * t * d, 0.05).reshape(b, h, t, d))
    # q . k / 8 = 4 * 8 * ramp / 8 = 4 * ramp
    ramp = (np.arange(t, dtype=np.float32) * per_key / 4.0).reshape(1, 1, t, 1)
    k = orc.round_bf16(np.broadcast_to(unit, (b, h, t, d)) * ramp + r.vec(b * h * t * d, 0.05).reshape(b, h, t, d))
    v = orc.round_bf16(r.vec(b * h * t * d, 1.0).reshape(b, h, t, d))
    gy = orc.round_bf16(r.vec(b * h * t * d, 1.0).reshape(b, h, t, d))
    oy, olse = orc.causal_sdpa_forward(q, k, v, 0)
    dq, dk, dv, dgy = (be.upload(a, BF16) for a in (q, k, v, gy))
    y32, lse = be.causal_sdpa_forward(dq, dk, dv, None, out_dtype=F32)
    close(be.download(y32), oy, 1e-2, "growing scores: out")
    close(be.download(lse), olse, 1e-5, "growing scores: lse")
    y16, lse16 = be.causal_sdpa_forward(dq, dk, dv, None, out_dtype=BF16)
    close(be.download_f32(y16), oy, BF16_TOL, "growing scores: out (bf16 store)")
    if per_key > 0.1:
        return
    ogq, ogk, ogv = orc.causal_sdpa_backward(q, k, v, orc.round_bf16(oy), olse, gy, 0)
    gq, gk, gv = be.causal_sdpa_backward(dq, dk, dv, y16, lse16, dgy, None, grad_dtype=F32)
    close(be.download(gq), ogq, BF16_TOL, "growing scores: gq")
    close(be.download(gk), ogk, BF16_TOL, "growing scores: gk")
    close(be.download(gv), ogv, BF16_TOL, "growing scores: gv")


@pytest.fixture(params=["one block per workgroup", "mirrored pairs"])
def flash_schedule(request, be):
    """Both block schedules of the flash kernels, whichever the chip's size would pick by itself."""
    be.set_option("flash_schedule", 1 if request.param == "one block per workgroup" else 2)
    yield request.param
    be.set_option("flash_schedule", 0)


@pytest.mark.parametrize("shape,hkv,window", FLASH_SHAPES)
def test_causal_sdpa_bf16_mfma(be, shape, hkv, window, flash_schedule):
    """head_dim 64 or 128 with bf16 operands takes the MFMA flash kernels. Inputs are
    bf16-exact on both sides; the GPU additionally rounds P and dS to bf16 for
    the second product, so the gate is the bf16 one (2e-2 of the largest value)."""
    from ojas_amd.backend import BF16, F32

    print(f"sdpa bf16 {shape} hkv {hkv} window {window} schedule: {flash_schedule}", flush=True)
    b, h, t, d = shape
    r = orc.SplitMix64(900 + t)
    mk = lambda n, sh: orc.round_bf16(r.vec(n, 1.0)).reshape(sh)
    q = mk(b * h * t * d, (b, h, t, d))
    k = mk(b * hkv * t * d, (b, hkv, t, d))
    v = mk(b * hkv * t * d, (b, hkv, t, d))
    gy = mk(b * h * t * d, (b, h, t, d))
    oy, olse = orc.causal_sdpa_forward(q, k, v, window or 0)
    dq, dk, dv, dgy = (be.upload(a, BF16) for a in (q, k, v, gy))
    y32, lse = be.causal_sdpa_forward(dq, dk, dv, window, out_dtype=F32)
    close(be.download(y32), oy, 1e-2, "flash out (f32 store)")
    close(be.download(lse), olse, 1e-5, "flash lse")
    y16, lse16 = be.causal_sdpa_forward(dq, dk, dv, window, out_dtype=BF16)
    close(be.download_f32(y16), oy, BF16_TOL, "flash out (bf16 store)")
    # Backward from the oracle's saved output rounded to bf16, as a bf16-tier caller saves it.
    oy16 = orc.round_bf16(oy)
    ogq, ogk, ogv = orc.causal_sdpa_backward(q, k, v, oy16, olse, gy, window or 0)
    gq, gk, gv = be.causal_sdpa_backward(dq, dk, dv, be.upload(oy16, BF16), be.upload(olse), dgy, window, grad_dtype=F32)
    close(be.download(gq), ogq, BF16_TOL, "flash gq")
    close(be.download(gk), ogk, BF16_TOL, "flash gk")
    close(be.download(gv), ogv, BF16_TOL, "flash gv")
    gq16, gk16, gv16 = be.causal_sdpa_backward(dq, dk, dv, y16, lse16, dgy, window, grad_dtype=BF16)
    close(be.download_f32(gq16), ogq, BF16_TOL, "flash gq bf16")
    close(be.download_f32(gk16), ogk, BF16_TOL, "flash gk bf16")
    close(be.download_f32(gv16), ogv, BF16_TOL, "flash gv bf16")


@pytest.mark.parametrize("dim", [64, 128])
@pytest.mark.parametrize("shared", [(0, 4, 0), (0, 0, 4), (4, 4, 4)])
def test_causal_attention_keeps_its_accuracy_when_rows_share_a_component(be, dim, shared):
    """Query, key and value rows that share a vector `shared` times their spread, as the rows of a
    residual stream do after a block or two. Attention does not see a vector added to every value
    row beyond passing it through (the weights sum to one), and dQ does not see one added to every
    key row (a row of dS sums to zero). In bf16 both sums are off by their rounding, which the
    shared part multiplies: with the output divided by the sum of the weights as computed, and dQ
    taken from the rounded dS as it stands, these cases measured 1e-2 (keys), 3e-3 (values) and
    3.4e-2 (all three) normwise in dQ against 2.4e-3 on plain inputs. The forward divides by the
    sum of the weights it multiplied, and the dQ pass takes (row sum of the rounded dS) x (mean key)
    off; every case must then stay at the plain level: 4e-3 normwise on the output and all three
    gradients (measured at most 2.9e-3)."""
    from ojas_amd.backend import BF16

    cq, ck, cv = shared
    b, t, h = 1, 512, 4
    rng = np.random.default_rng(1)

    def rows(c):
        x = rng.normal(0, 1, (b, t, h, dim)) + c * rng.normal(0, 1, (1, 1, h, dim))
        return orc.round_bf16(x.astype(np.float32))

    q, k, v = rows(cq), rows(ck), rows(cv)
    gy = orc.round_bf16(rng.normal(0, 1, (b, t, h, dim)).astype(np.float32))
    tq, tk, tv, tg = (np.ascontiguousarray(a.transpose(0, 2, 1, 3)) for a in (q, k, v, gy))
    oo, ol = orc.causal_sdpa_forward(tq, tk, tv)
    want = (oo,) + tuple(orc.causal_sdpa_backward(tq, tk, tv, oo, ol, tg))
    dq, dk, dv, dg = (be.upload(a, BF16) for a in (q, k, v, gy))
    out, lse, residual = be.causal_attention_forward(dq, dk, dv, saving=True)
    got = (out,) + tuple(be.causal_attention_backward(dq, dk, dv, out, lse, dg, residual=residual))
    for name, g, w in zip(("out", "gq", "gk", "gv"), got, want):
        g = be.download_f32(g).transpose(0, 2, 1, 3)
        rel = float(np.linalg.norm(g - w) / np.linalg.norm(w))
        assert rel <= 4e-3, (name, rel)


@pytest.mark.parametrize("shape,hkv,window", [((1, 2, 200, 64), 2, None), ((2, 4, 129, 64), 2, 50),
                                              ((1, 2, 70, 24), 1, None)])
def test_causal_sdpa_backward_reads_out_and_grad_output_in_their_own_dtypes(be, shape, hkv, window):
    """bf16 operands with the forward's default f32 output, and an f32 grad_output: the backward
    reads both as stored (head_dim 64: the MFMA kernels, from bf16 + rounding residual; head_dim
    24: the row kernels). The gradients must equal those of the oracle on the same values; an
    output read in the wrong storage type is off by orders of magnitude. Then the one-call
    recompute form (causal_sdpa_backward_recompute), which runs the forward itself."""
    from ojas_amd.backend import BF16, F32

    print(f"sdpa backward dtypes {shape} hkv {hkv} window {window}", flush=True)
    b, h, t, d = shape
    r = orc.SplitMix64(7700 + t)
    mk = lambda sh: orc.round_bf16(r.vec(int(np.prod(sh)), 1.0)).reshape(sh)
    q, k, v = mk((b, h, t, d)), mk((b, hkv, t, d)), mk((b, hkv, t, d))
    gy = r.vec(b * h * t * d, 1.0).reshape(b, h, t, d)  # f32, not bf16-exact
    oy, olse = orc.causal_sdpa_forward(q, k, v, window or 0)
    ogq, ogk, ogv = orc.causal_sdpa_backward(q, k, v, oy, olse, gy, window or 0)
    dq, dk, dv = (be.upload(a, BF16) for a in (q, k, v))
    dgy = be.upload(gy)
    y32, lse = be.causal_sdpa_forward(dq, dk, dv, window)  # default out dtype: f32
    assert y32.dtype == F32
    for name, grads in (("saved f32 out", be.causal_sdpa_backward(dq, dk, dv, y32, lse, dgy, window)),
                        ("recompute", be.causal_sdpa_backward_recompute(dq, dk, dv, dgy, window))):
        for g, og, what in zip(grads, (ogq, ogk, ogv), ("gq", "gk", "gv")):
            close(be.download(g), og, BF16_TOL, f"{name}: {what}")
    # All-f32: the recompute form equals forward + backward bit for bit (same kernels, same order).
    fq, fk, fv = (be.upload(a) for a in (q, k, v))
    y, l = be.causal_sdpa_forward(fq, fk, fv, window)
    two = be.causal_sdpa_backward(fq, fk, fv, y, l, dgy, window)
    one = be.causal_sdpa_backward_recompute(fq, fk, fv, dgy, window)
    for a, c2, og in zip(one, two, (ogq, ogk, ogv)):
        assert np.array_equal(be.download(a), be.download(c2))
        close(be.download(a), og, F32_TOL, "f32 recompute")
