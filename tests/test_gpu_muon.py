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
