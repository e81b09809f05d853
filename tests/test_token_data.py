"""The data step in front of the path (`include/ojas_data.h`, `ojas_amd/data.py`) against the
reference's own vectors: the pinned window starts of `permutation_is_pinned`
(ojas-data/tests/sampler.rs:231-254) and the 160 starts / 5280 row tokens that
`ojas-oracle/examples/dump_batch_starts` wrote for the tiny trace (batch_starts.json over tokens.bin),
plus the behaviours the reference's tests assert (ojas-data/tests/sampler.rs, tokens.rs tests)."""
import json
import struct
from pathlib import Path

import numpy as np
import pytest

from ojas_amd.data import (Batch, BatchSampler, DataCursor, DataError, TokenBin, rng_state_decode, rng_state_encode)

GOLD = Path(__file__).parent / "golden"
TINY = GOLD / "tiny"


def write_bin(path, n):
    """The reference tests' bin: token i is i % 65521 (ojas-data/tests/sampler.rs:24-36)."""
    (np.arange(n) % 65521).astype("<u2").tofile(path)
    return TokenBin.open_headerless(path)


def fnv1a64(data: bytes) -> int:
    h = 0xCBF29CE484222325
    for b in data:
        h = ((h ^ b) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return h


def test_permutation_is_pinned(tmp_path):
    pins = json.loads((GOLD / "sampler_pins.json").read_text())
    tokens = write_bin(tmp_path / "t.bin", pins["bin_tokens"])
    for case in pins["cases"]:
        s = BatchSampler(tokens, pins["seq_len"], 1, case["seed"])
        assert s.windows_per_epoch() == pins["windows"]
        got = [s.window_start(case["epoch"], o) for o in range(8)]
        assert got == case["starts"], case


def test_the_tiny_trace_batches_are_reproduced_token_for_token():
    doc = json.loads((TINY / "batch_starts.json").read_text())
    assert fnv1a64((TINY / "tokens.bin").read_bytes()) == int(doc["bin_fnv1a64"], 16)
    tokens = TokenBin.open_headerless_u16(TINY / "tokens.bin")
    assert len(tokens) == doc["bin_tokens"] and tokens.bytes_per_token() == 2
    s = BatchSampler(tokens, doc["seq_len"], doc["batch"], doc["seed"])
    assert s.windows_per_epoch() == doc["windows_per_epoch"]
    t, b = doc["seq_len"], doc["batch"]
    rows = np.array(doc["rows"], np.uint32).reshape(-1, t + 1)
    starts = doc["starts"]
    twin = BatchSampler(len(tokens), t, b, doc["seed"])  # the same stream without the bin
    for i in range(doc["steps"] * doc["accum"]):
        assert twin.next_starts().tolist() == starts[i * b:(i + 1) * b]
        got = s.next_batch()
        assert isinstance(got, Batch) and got.x.shape == (b, t) and got.x.dtype == np.uint32
        want = rows[i * b:(i + 1) * b]
        assert np.array_equal(got.x, want[:, :-1]) and np.array_equal(got.y, want[:, 1:])
    assert s.cursor() == DataCursor(*doc["cursor_after"]) == twin.cursor()


def test_every_window_is_visited_once_per_epoch_and_y_is_x_shifted(tmp_path):
    tokens = write_bin(tmp_path / "t.bin", 7 * 13 + 1 + 5)  # 13 windows of 7 and a ragged tail
    s = BatchSampler(tokens, 7, 4, 99)
    w = s.windows_per_epoch()
    assert w == 13
    for epoch in range(3):
        starts = sorted(s.window_start(epoch, o) for o in range(w))
        assert starts == [7 * k for k in range(w)]
    seen = []
    for _ in range(13):  # 52 windows = 4 epochs exactly, batches straddle epoch ends
        b = s.next_batch()
        assert np.array_equal(b.x[:, 1:], b.y[:, :-1])
        seen += (b.x[:, 0] // 1).tolist()
    for e in range(4):
        assert sorted(seen[e * 13:(e + 1) * 13]) == [7 * k for k in range(13)]
    assert s.cursor() == DataCursor(4, 0)


def test_same_seed_same_batches_other_seed_other_order_and_batch_size_does_not_matter(tmp_path):
    tokens = write_bin(tmp_path / "t.bin", 4001)
    a, b, c = (BatchSampler(tokens, 8, 5, seed) for seed in (7, 7, 8))
    xa = np.concatenate([a.next_batch().x for _ in range(6)])
    xb = np.concatenate([b.next_batch().x for _ in range(6)])
    xc = np.concatenate([c.next_batch().x for _ in range(6)])
    assert np.array_equal(xa, xb) and not np.array_equal(xa, xc)
    d = BatchSampler(tokens, 8, 3, 7)
    xd = np.concatenate([d.next_batch().x for _ in range(10)])
    assert np.array_equal(xa, xd)


def test_resume_from_any_cursor_reproduces_the_uninterrupted_stream(tmp_path):
    tokens = write_bin(tmp_path / "t.bin", 301)
    whole = BatchSampler(tokens, 6, 4, 5)
    stream = []
    cursors = []
    for _ in range(30):
        cursors.append(whole.cursor())
        stream.append(whole.next_batch().x)
    for i in (0, 1, 11, 12, 13, 29):
        again = BatchSampler(tokens, 6, 4, 5, cursors[i])
        for j in range(i, min(i + 3, 30)):
            assert np.array_equal(again.next_batch().x, stream[j])
    with pytest.raises(DataError, match="past the 50 windows"):
        BatchSampler(tokens, 6, 4, 5, DataCursor(0, 50))


def test_shapes_that_cannot_produce_a_window_are_refused(tmp_path):
    tokens = write_bin(tmp_path / "t.bin", 10)
    for t, b in ((0, 1), (1, 0)):
        with pytest.raises(DataError, match="non-zero"):
            BatchSampler(tokens, t, b, 1)
    with pytest.raises(DataError, match="needs 11 tokens"):
        BatchSampler(tokens, 10, 1, 1)
    one = BatchSampler(tokens, 9, 3, 1)  # a single window repeats every epoch
    assert one.windows_per_epoch() == 1
    batch = one.next_batch()
    assert np.array_equal(batch.x, np.tile(np.arange(9, dtype=np.uint32), (3, 1)))
    assert one.cursor() == DataCursor(3, 0)
    with pytest.raises(DataError, match="window 1 past 1"):
        one.window_start(0, 1)
    with pytest.raises(DataError, match="holds no token bin"):
        BatchSampler(10, 9, 3, 1).next_batch()


def test_rng_state_layout_is_exact_and_refuses_anything_else():
    data = rng_state_encode(0x0123456789ABCDEF)
    assert data == struct.pack("<IIQ", 1, 1, 0x0123456789ABCDEF)
    assert rng_state_decode(data) == 0x0123456789ABCDEF
    assert rng_state_decode(rng_state_encode(2**64 - 1)) == 2**64 - 1
    for n in (0, 1, 8, 15, 17, 32):
        with pytest.raises(DataError, match="bytes"):
            rng_state_decode(data.ljust(n, b"\0")[:n])
    for version in (0, 2, 2**32 - 1):
        with pytest.raises(DataError, match="version"):
            rng_state_decode(struct.pack("<I", version) + data[4:])
    for gen in (0, 2, 2**32 - 1):
        with pytest.raises(DataError, match="generator"):
            rng_state_decode(data[:4] + struct.pack("<I", gen) + data[8:])


def fineweb(magic, version, count, tokens, dtype="<u2"):
    header = np.zeros(256, "<i4")
    header[:3] = (magic, version, count)
    return header.tobytes() + np.asarray(tokens, dtype).tobytes()


def test_fineweb_headers_and_their_refusals(tmp_path):
    p = tmp_path / "f.bin"
    p.write_bytes(fineweb(20240520, 1, 5, [1, 2, 3, 4, 65535]))
    b = TokenBin.open_fineweb(p)
    assert len(b) == 5 and b.bytes_per_token() == 2
    assert b.read_into_u32(1, 4).tolist() == [2, 3, 4, 65535]
    assert b.read_into(0, 2).tolist() == [1, 2] and b.read_into_u32(5, 0).size == 0
    with pytest.raises(DataError, match=r"token window \[3, 6\) past length 5"):
        b.read_into_u32(3, 3)
    with pytest.raises(DataError, match="expected u32"):
        TokenBin.open_fineweb_u32(p)
    p.write_bytes(fineweb(20240801, 7, 3, [70000, 5, 248320], "<u4"))
    w = TokenBin.open_fineweb(p)
    assert len(w) == 3 and w.bytes_per_token() == 4 and w.read_into_u32(0, 3).tolist() == [70000, 5, 248320]
    assert TokenBin.open_fineweb_u32(p).read_raw(1, 2).tolist() == [5, 248320]
    with pytest.raises(DataError, match=r"token 70000 at index 0 exceeds u16::MAX \(65535\)"):
        w.read_into(0, 3)
    with pytest.raises(DataError, match="248320"):
        w.read_into(2, 1)
    assert w.read_into(1, 1).tolist() == [5]
    with pytest.raises(DataError, match="expected u16"):
        TokenBin.open_fineweb_u16(p)
    p.write_bytes(fineweb(20240801, 1, 1, [9], "<u4"))
    assert len(TokenBin.open_fineweb(p)) == 1  # version 1 is accepted for u32 streams
    for blob, what in ((fineweb(1, 1, 1, [7]), "magic"), (fineweb(20240520, 2, 1, [7]), "version"),
                       (fineweb(20240801, 6, 1, [7], "<u4"), "version"), (fineweb(20240520, 1, -1, [7]), "negative"),
                       (fineweb(20240520, 1, 2, [7]), "size"), (fineweb(20240520, 1, 1, [7, 8]), "size"),
                       (b"\0" * 100, "truncated")):
        p.write_bytes(blob)
        with pytest.raises(DataError, match=what):
            TokenBin.open_fineweb(p)


def test_headerless_bins(tmp_path):
    p = tmp_path / "h.bin"
    p.write_bytes(np.array([3, 1, 4, 1, 5, 9], "<u2").tobytes())
    assert TokenBin.open_headerless(p).read_into_u32(2, 4).tolist() == [4, 1, 5, 9]
    assert len(TokenBin.open_headerless_u32(p)) == 3
    p.write_bytes(b"\1\2\3")
    with pytest.raises(DataError, match="multiple of 2"):
        TokenBin.open_headerless(p)
    p.write_bytes(b"\1\2\3\4\5\6")
    with pytest.raises(DataError, match="multiple of 4"):
        TokenBin.open_headerless_u32(p)
    with pytest.raises(DataError, match="No such file"):
        TokenBin.open_headerless(tmp_path / "absent.bin")
    with pytest.raises(DataError, match="not a regular file"):
        TokenBin.open_headerless(tmp_path)
