"""The oracle's KV-cache ops (ojas-cpu/src/kv.rs). The reference holds no digest for them; what pins
them is what its documentation states (ojas-core/src/backend.rs:2526-2542): with `kv_len == Tq` the op
is `causal_sdpa_forward` after the layout permute, and, since every row runs the same per-row kernel
oldest key first, for ANY cache rotation the rows are the last Tq rows of `causal_sdpa_forward` over
the whole sequence, bit for bit (that routine is digest-pinned). A wrong slot, a wrong first visible
position or a wrong KV head each breaks one of these. An f64 softmax covers the values."""
import numpy as np
import pytest

import oracle_api as orc


def ring(seq, capacity, kv_len):
    """[B, T, Hkv, D] positions 0..kv_len written into a ring of `capacity` slots; junk elsewhere."""
    b, _, hkv, d = seq.shape
    cache = np.full((b, capacity, hkv, d), np.nan, np.float32)  # unread slots may hold anything
    for j in range(max(0, kv_len - capacity), kv_len):
        cache[:, j % capacity] = seq[:, j]
    return cache


def data(seed, b, t, h, hkv, d):
    r = np.random.default_rng(seed)
    q = r.standard_normal((b, t, h, d)).astype(np.float32)
    k = r.standard_normal((b, t, hkv, d)).astype(np.float32)
    v = r.standard_normal((b, t, hkv, d)).astype(np.float32)
    return q, k, v


@pytest.mark.parametrize("h,hkv", [(4, 4), (4, 2), (6, 1)])
@pytest.mark.parametrize("window", [0, 5])
def test_full_prefill_is_causal_sdpa_after_the_permute(h, hkv, window):
    b, t, d = 2, 19, 16
    q, k, v = data(1, b, t, h, hkv, d)
    want, _ = orc.causal_sdpa_forward(q.transpose(0, 2, 1, 3), k.transpose(0, 2, 1, 3), v.transpose(0, 2, 1, 3), window)
    got = orc.cached_attention_forward(q, k, v, kv_len=t, window=window)
    assert np.array_equal(got, want.transpose(0, 2, 1, 3))


@pytest.mark.parametrize("tq,kv_len,capacity,window", [(1, 37, 64, 0), (1, 37, 37, 0), (3, 37, 40, 0), (1, 37, 8, 8),
                                                       (4, 37, 12, 9), (5, 37, 37, 11), (1, 100, 16, 16), (2, 5, 5, 7)])
def test_decode_rows_are_the_last_rows_of_the_whole_sequence_for_any_rotation(tq, kv_len, capacity, window):
    b, h, hkv, d = 2, 4, 2, 8
    q, k, v = data(2, b, kv_len, h, hkv, d)
    eff = 0 if window >= kv_len else window
    want, _ = orc.causal_sdpa_forward(q.transpose(0, 2, 1, 3), k.transpose(0, 2, 1, 3), v.transpose(0, 2, 1, 3), eff)
    want = want.transpose(0, 2, 1, 3)[:, kv_len - tq:]
    got = orc.cached_attention_forward(q[:, kv_len - tq:], ring(k, capacity, kv_len), ring(v, capacity, kv_len),
                                       kv_len=kv_len, window=window)
    assert np.array_equal(got, want)


def test_values_against_an_f64_softmax():
    b, h, hkv, d, kv_len, tq, cap, window = 1, 4, 2, 16, 23, 2, 32, 6
    q, k, v = data(3, b, kv_len, h, hkv, d)
    got = orc.cached_attention_forward(q[:, -tq:], ring(k, cap, kv_len), ring(v, cap, kv_len), kv_len, window)
    for i in range(tq):
        p = kv_len - tq + i
        lo = max(0, p + 1 - window)
        for head in range(h):
            kk = k[0, lo:p + 1, head // (h // hkv)].astype(np.float64)
            vv = v[0, lo:p + 1, head // (h // hkv)].astype(np.float64)
            s = kk @ q[0, p, head].astype(np.float64) / np.sqrt(d)
            w = np.exp(s - s.max())
            ref = (w / w.sum()) @ vv
            assert np.allclose(got[0, i, head], ref, rtol=0, atol=2e-6)


def test_refusals_follow_the_validator():
    q, k, v = data(4, 1, 8, 2, 2, 4)
    with pytest.raises(orc.OracleError) as e:
        orc.cached_attention_forward(q[:, :3], k, v, kv_len=2)  # kv_len below the new positions
    assert e.value.code == 3
    with pytest.raises(orc.OracleError) as e:
        orc.cached_attention_forward(q[:, :1], k[:, :4], v[:, :4], kv_len=6)  # the ring no longer holds position 0
    assert e.value.code == 3
    assert orc.cached_attention_forward(q[:, :1], ring(k, 4, 6), ring(v, 4, 6), kv_len=6, window=4).shape == (1, 1, 2, 4)
    bad = k.copy()
    bad[0, 2, 0, 0] = np.inf
    with pytest.raises(orc.OracleError) as e:
        orc.cached_attention_forward(q[:, :1], bad, v, kv_len=8)
    assert e.value.code == 4
    # ... but a non-finite value in a slot no query reads is never looked at.
    assert np.isfinite(orc.cached_attention_forward(q[:, :1], bad, v, kv_len=8, window=3)).all()
    with pytest.raises(orc.OracleError):
        orc.cached_attention_forward(np.zeros((1, 1, 3, 4), np.float32), k, v, kv_len=8)  # 3 heads over 2


def test_cache_write_is_a_ring_and_all_or_nothing():
    r = np.random.default_rng(5)
    cache = r.standard_normal((2, 6, 2, 4)).astype(np.float32)
    src = r.standard_normal((2, 4, 2, 4)).astype(np.float32)
    out = orc.kv_cache_write(cache, src, at=4)  # positions 4, 5, 6, 7 -> slots 4, 5, 0, 1
    want = cache.copy()
    for j in range(4):
        want[:, (4 + j) % 6] = src[:, j]
    assert np.array_equal(out, want)
    assert np.array_equal(orc.kv_cache_write(cache, src, at=6 * 1000 + 2)[:, 2:6], src)
    with pytest.raises(orc.OracleError) as e:
        orc.kv_cache_write(cache, r.standard_normal((2, 7, 2, 4)).astype(np.float32), at=0)
    assert e.value.code == 3
    src[1, 3, 1, 2] = np.nan
    with pytest.raises(orc.OracleError) as e:
        orc.kv_cache_write(cache, src, at=0)
    assert e.value.code == 4
