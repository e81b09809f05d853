"""KV-cache attention and cache writes on the device (`omx_cached_attention_forward`,
`omx_kv_cache_write`) against the CPU oracle (ojas-cpu/src/kv.rs restated, tests/test_oracle_kv.py
pins it): f32 tier tolerance 1e-5 * max(1, max|ref|); cache writes are bit copies."""
import numpy as np
import pytest

import oracle_api as orc

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.fixture(scope="module")
def be():
    from ojas_amd.backend import MiBackend

    backend = MiBackend(0)
    yield backend
    backend.close()


def ring(seq, capacity, kv_len, junk):
    b, _, hkv, d = seq.shape
    cache = np.full((b, capacity, hkv, d), junk, np.float32)
    for j in range(max(0, kv_len - capacity), kv_len):
        cache[:, j % capacity] = seq[:, j]
    return cache


CASES = [  # b, tq, h, hkv, d, capacity, kv_len, window
    (2, 1, 4, 4, 16, 40, 37, None),      # tiny model shape, plain prefix
    (2, 1, 4, 2, 64, 64, 64, None),      # one full tile
    (1, 1, 12, 12, 64, 1024, 1000, None),  # GPT-124M decode, ragged last tile
    (2, 3, 8, 2, 64, 300, 257, None),    # grouped heads x 3 queries: 12 rows per KV head, 2 row chunks
    (1, 1, 8, 1, 128, 96, 500, 96),      # ring wrapped several times, window = capacity
    (2, 5, 4, 2, 32, 37, 37, 11),        # window narrower than the new block + ring exactly full
    (1, 2, 2, 2, 256, 130, 129, None),   # widest head
    (1, 16, 4, 4, 64, 4096, 4096, None),  # prefill of 16 onto 4080: many parts per row
    (1, 1, 4, 4, 8, 8, 3, 1),            # a window of one: every row sees only itself
]


@pytest.mark.parametrize("case", CASES + [(2, 2, 6, 2, 24, 70, 69, None), (1, 3, 4, 4, 80, 200, 150, 64)],
                         ids=lambda c: "b{}tq{}h{}kv{}d{}cap{}len{}w{}".format(*c))
@pytest.mark.parametrize("bf16_cache", [False, True])
@pytest.mark.parametrize("kernel", ["by_head_dim", "lds_tiled"])
def test_cached_attention_matches_the_oracle(be, case, bf16_cache, kernel):
    from ojas_amd.backend import BF16

    b, tq, h, hkv, d, cap, kv_len, window = case
    print(f"cached attention {case} bf16_cache={bf16_cache} kernel={kernel}", flush=True)
    be.set_option("kv_attention", 1 if kernel == "lds_tiled" else 0)
    r = np.random.default_rng(hash(case) % 2**32)
    q = r.standard_normal((b, tq, h, d)).astype(np.float32)
    k = r.standard_normal((b, kv_len, hkv, d)).astype(np.float32)
    v = r.standard_normal((b, kv_len, hkv, d)).astype(np.float32)
    if bf16_cache:  # values a bf16 cache holds exactly
        k, v = orc.round_bf16(k), orc.round_bf16(v)
    # Slots no query reads hold NaN: they must never be looked at.
    kc, vc = ring(k, cap, kv_len, np.nan), ring(v, cap, kv_len, np.nan)
    if bf16_cache:
        kc[np.isnan(kc)] = 0.0  # NaN does not survive the f32 -> bf16 upload path's rounding check
        vc[np.isnan(vc)] = 0.0
    want = orc.cached_attention_forward(q, np.nan_to_num(kc), np.nan_to_num(vc), kv_len, window or 0)
    dk = be.upload(kc, BF16) if bf16_cache else be.upload(kc)
    dv = be.upload(vc, BF16) if bf16_cache else be.upload(vc)
    got = be.download(be.cached_attention_forward(be.upload(q), dk, dv, kv_len, window))
    be.sync()
    be.set_option("kv_attention", 0)
    assert np.abs(got - want).max() <= TOL * max(1.0, np.abs(want).max())


def test_decode_loop_write_then_attend(be):
    """Token by token: write position t, attend over 0..=t, against the whole-sequence oracle."""
    print("kv cache decode loop", flush=True)
    b, h, hkv, d, cap, steps = 2, 4, 2, 64, 24, 40
    r = np.random.default_rng(7)
    q = r.standard_normal((b, steps, h, d)).astype(np.float32)
    k = r.standard_normal((b, steps, hkv, d)).astype(np.float32)
    v = r.standard_normal((b, steps, hkv, d)).astype(np.float32)
    kc, vc = be.zeros((b, cap, hkv, d)), be.zeros((b, cap, hkv, d))
    host_k = np.zeros((b, cap, hkv, d), np.float32)
    window = cap  # a ring of `cap` slots serves a window of `cap`
    full, _ = orc.causal_sdpa_forward(q.transpose(0, 2, 1, 3), k.transpose(0, 2, 1, 3), v.transpose(0, 2, 1, 3), window)
    full = full.transpose(0, 2, 1, 3)
    for t in range(steps):
        be.kv_cache_write(kc, be.upload(k[:, t:t + 1]), t)
        be.kv_cache_write(vc, be.upload(v[:, t:t + 1]), t)
        host_k = orc.kv_cache_write(host_k, k[:, t:t + 1], t)
        out = be.download(be.cached_attention_forward(be.upload(q[:, t:t + 1]), kc, vc, t + 1, window))
        assert np.abs(out - full[:, t:t + 1]).max() <= TOL * max(1.0, np.abs(full).max()), t
    assert np.array_equal(be.download(kc), host_k)  # the ring holds the last `cap` positions, bit for bit


def test_cache_write_block_wraps_and_is_all_or_nothing(be):
    from ojas_amd.backend import BF16, NON_FINITE, OUT_OF_RANGE, OjasError

    print("kv cache write", flush=True)
    r = np.random.default_rng(9)
    cache = r.standard_normal((3, 10, 2, 16)).astype(np.float32)
    src = r.standard_normal((3, 7, 2, 16)).astype(np.float32)
    dc = be.upload(cache)
    be.kv_cache_write(dc, be.upload(src), 10 * 123 + 6)
    assert np.array_equal(be.download(dc), orc.kv_cache_write(cache, src, 6))
    db = be.upload(cache, BF16)
    be.kv_cache_write(db, be.upload(src), 6)
    assert np.array_equal(be.download_f32(db), orc.round_bf16(orc.kv_cache_write(cache, src, 6)))
    with pytest.raises(OjasError) as e:
        be.kv_cache_write(dc, be.upload(r.standard_normal((3, 11, 2, 16)).astype(np.float32)), 0)
    assert e.value.code == OUT_OF_RANGE
    before = be.download(dc)
    bad = src.copy()
    bad[2, 6, 1, 15] = np.inf
    be.kv_cache_write(dc, be.upload(bad), 0)
    with pytest.raises(OjasError) as e:
        be.sync()
    assert e.value.code == NON_FINITE and "kv_cache_write" in str(e.value)
    assert np.array_equal(be.download(dc), before)  # nothing was written


def test_refusals_and_the_deferred_fault(be):
    from ojas_amd.backend import NON_FINITE, OUT_OF_RANGE, SHAPE, UNSUPPORTED_HEAD_DIM, OjasError

    print("cached attention refusals", flush=True)
    q = be.upload(np.ones((1, 3, 2, 8), np.float32))
    c8 = be.upload(np.ones((1, 8, 2, 8), np.float32))
    for kw, code in ((dict(kv_len=2), OUT_OF_RANGE), (dict(kv_len=12), OUT_OF_RANGE), (dict(kv_len=8, window=0), SHAPE)):
        with pytest.raises(OjasError) as e:
            be.cached_attention_forward(q, c8, c8, **kw)
        assert e.value.code == code, kw
    be.cached_attention_forward(q, c8, c8, kv_len=12, window=4)  # 3 + 4 - 1 = 6 positions fit the ring
    with pytest.raises(OjasError) as e:
        be.cached_attention_forward(be.upload(np.ones((1, 1, 3, 8), np.float32)), c8, c8, kv_len=4)
    assert e.value.code == SHAPE
    c6 = be.upload(np.ones((1, 8, 2, 6), np.float32))
    with pytest.raises(OjasError) as e:
        be.cached_attention_forward(be.upload(np.ones((1, 1, 2, 6), np.float32)), c6, c6, kv_len=4)
    assert e.value.code == UNSUPPORTED_HEAD_DIM
    be.sync()
    poisoned = np.ones((1, 8, 2, 8), np.float32)
    poisoned[0, 5, 1, 3] = np.nan
    dp = be.upload(poisoned)
    be.cached_attention_forward(be.upload(np.ones((1, 1, 2, 8), np.float32)), dp, c8, kv_len=5)  # slot 5 not read
    be.sync()
    be.cached_attention_forward(be.upload(np.ones((1, 1, 2, 8), np.float32)), dp, c8, kv_len=6)
    with pytest.raises(OjasError) as e:
        be.sync()
    assert e.value.code == NON_FINITE and "cached_attention_forward" in str(e.value)
