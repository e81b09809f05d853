"""Batches built on the device from a token bin resident in HBM (`omx_token_windows`) against the
host sampler (`odata_sampler_next_batch`), which the reference's own dumps pin
(tests/test_token_data.py): integer work, bit-exact."""
import json
from pathlib import Path

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TINY = Path(__file__).parent / "golden" / "tiny"


@pytest.fixture(scope="module")
def be():
    from ojas_amd.backend import MiBackend

    backend = MiBackend(0)
    yield backend
    backend.close()


def test_the_tiny_trace_batches_from_a_resident_bin(be):
    from ojas_amd.data import BatchSampler, TokenBin

    print("token windows: tiny trace bin", flush=True)
    doc = json.loads((TINY / "batch_starts.json").read_text())
    tokens = TokenBin.open_headerless_u16(TINY / "tokens.bin")
    resident = be.upload(tokens.read_raw(0, len(tokens)))
    t, b = doc["seq_len"], doc["batch"]
    rows = np.array(doc["rows"], np.uint32).reshape(-1, t + 1)
    host = BatchSampler(tokens, t, b, doc["seed"])
    dev = BatchSampler(len(tokens), t, b, doc["seed"])
    for i in range(doc["steps"] * doc["accum"]):
        x, y = be.token_windows(resident, dev.next_starts(), t)
        want = host.next_batch()
        gx, gy = be.download(x), be.download(y)
        assert np.array_equal(gx, want.x) and np.array_equal(gy, want.y)
        assert np.array_equal(gx, rows[i * b:(i + 1) * b, :-1])
    assert dev.cursor() == host.cursor()


@pytest.mark.parametrize("width", [2, 4])
def test_large_batches_both_token_widths_and_refusals(be, width, tmp_path):
    from ojas_amd.backend import OUT_OF_RANGE, OjasError
    from ojas_amd.data import BatchSampler, TokenBin

    print(f"token windows: width {width}", flush=True)
    n, t, b = 1_000_003, 1024, 64
    r = np.random.default_rng(width)
    words = r.integers(0, 65536 if width == 2 else 2**32, n, dtype=np.uint64).astype("<u2" if width == 2 else "<u4")
    path = tmp_path / "big.bin"
    words.tofile(path)
    tokens = TokenBin.open_headerless_u16(path) if width == 2 else TokenBin.open_headerless_u32(path)
    resident = be.upload(tokens.read_raw(0, n))
    host, dev = BatchSampler(tokens, t, b, 11), BatchSampler(n, t, b, 11)
    for _ in range(20):  # 1280 windows of 976 per epoch: crosses an epoch boundary
        x, y = be.token_windows(resident, dev.next_starts(), t)
        want = host.next_batch()
        assert np.array_equal(be.download(x), want.x) and np.array_equal(be.download(y), want.y)
    assert dev.cursor().shard == 1
    last = np.array([n - t - 1], np.uint64)
    x, y = be.token_windows(resident, last, t)
    assert int(be.download(y)[0, -1]) == int(words[-1])
    with pytest.raises(OjasError) as e:
        be.token_windows(resident, last + 1, t)
    assert e.value.code == OUT_OF_RANGE
