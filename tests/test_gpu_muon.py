"""Muon NS5 on the GPU against the CPU oracle (whose f32 path is pinned bit for
bit by the reference's muon_p / muon_m digests).

Gates: the momentum buffer is one f32 multiply-add per value and must carry the
oracle's bits; the parameter goes through five Newton-Schulz iterations of
re-ordered f32 sums, gated like the reference's device runs (1e-4 of the
largest value, ojas-wgpu/tests/common/mod.rs:11); the bf16 iteration is gated
at the reference's own bf16-NS5 parameter bound (5e-2 of the update's scale,
ojas-oracle/src/parity.rs:29-74)."""
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


@pytest.mark.parametrize("rows,cols", [(64, 48), (48, 64), (130, 70), (97, 97), (768, 768), (768, 3072), (3072, 768)])
def test_muon_f32_matches_cpu_exact(be, rows, cols):
    from ojas_amd.backend import MuonNs5Config

    print(f"muon f32 {rows}x{cols}", flush=True)
    r = orc.SplitMix64(200 + rows)
    p = r.vec(rows * cols, 0.1).reshape(rows, cols)
    g = r.vec(rows * cols, 0.1).reshape(rows, cols)
    m = r.vec(rows * cols, 0.01).reshape(rows, cols)
    orc.set_threads(8)
    op, om = orc.muon_ns5_step(p, g, m)
    dp, dg, dm = be.upload(p), be.upload(g), be.upload(m)
    be.muon_ns5_step(dp, dg, dm, MuonNs5Config.nanolab_default())
    assert np.array_equal(be.download(dm), om), "momentum buffer bits"
    gp = be.download(dp)
    assert np.max(np.abs(gp - op)) <= 1e-4 * max(1.0, np.max(np.abs(op)))
    # The update itself (p_new - p * decay), relative to its own size.
    decay = np.float32(1.0 - 0.025 * 0.1)
    upd_gpu, upd_cpu = gp - p * decay, op - p * decay
    assert np.max(np.abs(upd_gpu - upd_cpu)) <= 2e-3 * np.max(np.abs(upd_cpu))


@pytest.mark.parametrize("rows,cols", [(64, 48), (130, 70), (768, 768), (3072, 768)])
def test_muon_bf16_iteration(be, rows, cols):
    from ojas_amd.backend import MuonNs5Config

    print(f"muon bf16 {rows}x{cols}", flush=True)
    r = orc.SplitMix64(300 + rows)
    p = r.vec(rows * cols, 0.1).reshape(rows, cols)
    g = r.vec(rows * cols, 0.1).reshape(rows, cols)
    m = r.vec(rows * cols, 0.01).reshape(rows, cols)
    orc.set_threads(8)
    op, om = orc.muon_ns5_step(p, g, m, lr=0.02, momentum=0.95, weight_decay=0.0, nesterov=True, bf16=True)
    dp, dg, dm = be.upload(p), be.upload(g), be.upload(m)
    be.muon_ns5_step(dp, dg, dm, MuonNs5Config(0.02, 0.95, 0.0, 1, 1))
    assert np.array_equal(be.download(dm), om)
    upd_gpu, upd_cpu = be.download(dp) - p, op - p
    assert np.max(np.abs(upd_gpu - upd_cpu)) <= 5e-2 * np.max(np.abs(upd_cpu))


def test_muon_is_all_or_nothing_and_refuses_bad_configs(be):
    from ojas_amd.backend import NON_FINITE, OUT_OF_RANGE, MuonNs5Config, OjasError

    rows, cols = 40, 24
    r = orc.SplitMix64(7)
    p, g, m = (r.vec(rows * cols, 0.1).reshape(rows, cols) for _ in range(3))
    g[3, 3] = np.nan
    dp, dg, dm = be.upload(p), be.upload(g), be.upload(m)
    be.muon_ns5_step(dp, dg, dm, MuonNs5Config.nanolab_default())
    with pytest.raises(OjasError) as e:
        be.sync()
    assert e.value.code == NON_FINITE and "muon_ns5_step" in e.value.detail
    assert np.array_equal(be.download(dp), p) and np.array_equal(be.download(dm), m)
    with pytest.raises(OjasError) as e:
        be.muon_ns5_step(dp, dg, dm, MuonNs5Config(-0.1, 0.9, 0.0, 1, 0))
    assert e.value.code == OUT_OF_RANGE
    assert be._lib.omx_muon_scratch_bytes(768, 3072) >= 4 * 768 * 3072 * 4


@pytest.mark.parametrize("rows,cols,count,bf16", [(64, 48, 5, 0), (48, 64, 3, 1), (130, 70, 2, 0), (256, 256, 7, 1),
                                                  (768, 768, 48, 1), (768, 3072, 12, 1), (3072, 768, 12, 0),
                                                  (32, 32, 70, 0)])
def test_batched_step_matches_the_oracle_per_tensor(be, rows, cols, count, bf16):
    """`omx_muon_ns5_step_batched` holds each tensor to the oracle at the single op's gates (momentum
    bit for bit; update 2e-3 of its largest element in f32, 5e-2 with the bf16 iteration). 70 tensors
    go through in two launches of at most 64."""
    from ojas_amd.backend import BF16, MuonNs5Config

    print(f"muon batched {count} x {rows}x{cols} bf16={bf16}", flush=True)
    r = np.random.default_rng(rows * 7 + cols + count)
    ps = [r.standard_normal((rows, cols)).astype(np.float32) * 0.1 for _ in range(count)]
    gs = [r.standard_normal((rows, cols)).astype(np.float32) * (0.02 + 0.05 * i / count) for i in range(count)]
    ms = [r.standard_normal((rows, cols)).astype(np.float32) * 0.01 for _ in range(count)]
    cfg = MuonNs5Config(0.02, 0.95, 0.1, 1, bf16)
    dp, dg, dm = [be.upload(x) for x in ps], [be.upload(x) for x in gs], [be.upload(x) for x in ms]
    mirrors = [be.upload(np.zeros((rows, cols), np.float32), BF16) if i % 2 == 0 else None for i in range(count)]
    be.muon_ns5_step_batched(dp, dg, dm, cfg, mirrors)
    be.sync()
    orc.set_threads(8)
    decay = np.float32(1.0 - 0.02 * 0.1)
    check = range(count) if rows * cols <= 1 << 17 else (0, count // 2, count - 1)  # the oracle is slow on big ones
    for i in check:
        op, om = orc.muon_ns5_step(ps[i], gs[i], ms[i], lr=0.02, momentum=0.95, weight_decay=0.1, nesterov=True,
                                   bf16=bool(bf16))
        assert np.array_equal(be.download(dm[i]), om), i
        got = be.download(dp[i])
        upd_gpu, upd_cpu = got - ps[i] * decay, op - ps[i] * decay
        assert np.max(np.abs(upd_gpu - upd_cpu)) <= (5e-2 if bf16 else 2e-3) * np.max(np.abs(upd_cpu)), i
        if mirrors[i] is not None:
            assert np.array_equal(be.download(mirrors[i]), orc.to_bf16(got)), i


def test_batched_step_refuses_the_whole_batch(be):
    from ojas_amd.backend import NON_FINITE, MuonNs5Config, OjasError

    print("muon batched refusal", flush=True)
    r = np.random.default_rng(1)
    ps = [r.standard_normal((64, 32)).astype(np.float32) for _ in range(4)]
    gs = [r.standard_normal((64, 32)).astype(np.float32) for _ in range(4)]
    gs[2][5, 7] = np.nan
    dp, dg = [be.upload(x) for x in ps], [be.upload(x) for x in gs]
    dm = [be.zeros((64, 32)) for _ in range(4)]
    be.muon_ns5_step_batched(dp, dg, dm, MuonNs5Config.nanolab_default())
    with pytest.raises(OjasError) as e:
        be.sync()
    assert e.value.code == NON_FINITE and "muon_ns5_step" in str(e.value)
    for i in range(4):
        assert np.array_equal(be.download(dp[i]), ps[i]) and not be.download(dm[i]).any()


@pytest.mark.parametrize("rows,cols,count", [(64, 48, 2), (130, 70, 3), (768, 768, 6), (768, 3072, 2), (3072, 768, 2),
                                             (2048, 2048, 2), (2048, 2048, 1)])
def test_bf16_iteration_sums_in_the_store_pass_carry_the_separate_kernels_bits(be, rows, cols, count):
    """The bf16 iteration forms b A + c A^2 and a X + B X in the store passes of the products that
    feed them (`muon_fused_sums`, the default, for calls on more than one tensor): same roundings in
    the same order as the separate kernels, so parameters, momenta and bf16 copies are the same bits; and a NaN gradient leaves
    every tensor of the call untouched under either setting."""
    from ojas_amd.backend import BF16, NON_FINITE, MuonNs5Config, OjasError

    print(f"muon fused sums {count} x {rows}x{cols}", flush=True)
    r = np.random.default_rng(rows + 3 * cols + count)
    ps = [r.standard_normal((rows, cols)).astype(np.float32) * 0.1 for _ in range(count)]
    gs = [r.standard_normal((rows, cols)).astype(np.float32) * 0.03 for _ in range(count)]
    ms = [r.standard_normal((rows, cols)).astype(np.float32) * 0.01 for _ in range(count)]
    cfg = MuonNs5Config(0.02, 0.95, 0.1, 1, 1)
    got = {}
    try:
        for fused in (1, 0):
            be.set_option("muon_fused_sums", fused)
            dp, dg, dm = [be.upload(x) for x in ps], [be.upload(x) for x in gs], [be.upload(x) for x in ms]
            mirrors = [be.upload(np.zeros((rows, cols), np.float32), BF16) for _ in range(count)]
            be.muon_ns5_step_batched(dp, dg, dm, cfg, mirrors)
            be.sync()
            got[fused] = [be.download(t) for t in dp + dm + mirrors]
            # all or nothing
            bad = [g.copy() for g in gs]
            bad[-1][rows // 2, cols // 3] = np.nan
            dp, dg, dm = [be.upload(x) for x in ps], [be.upload(x) for x in bad], [be.upload(x) for x in ms]
            be.muon_ns5_step_batched(dp, dg, dm, cfg, None)
            with pytest.raises(OjasError) as e:
                be.sync()
            assert e.value.code == NON_FINITE and "muon" in e.value.detail
            for t, want in zip(dp + dm, ps + ms):
                assert np.array_equal(be.download(t), want)
    finally:
        be.set_option("muon_fused_sums", 1)
    for a, b in zip(got[1], got[0]):
        assert np.array_equal(a, b)
    assert any(np.any(a != p) for a, p in zip(got[1][:count], ps))
