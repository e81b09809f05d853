"""safetensors and checkpoint-v1 files (`include/ojas_io.h`, `ojas_amd/io.py`).

safetensors: the checker is the `safetensors` Python library, an independent implementation of the
format: every file the reference's tests ship is read by both and compared byte for byte, files
written here are read back by it, and the refusals are the ones the reference's own tests list
(ojas-io/src/safetensors.rs:1810-3079). checkpoint v1: the reference holds no golden bytes, only round
trips; the layout is pinned here by a file assembled by hand from the tables of
docs/checkpoint-v1.md, and the refusals follow ojas-io/src/checkpoint.rs:487-866."""
import json
import struct
from pathlib import Path

import numpy as np
import pytest
from safetensors import safe_open
from safetensors.numpy import save_file

from ojas_amd.io import (CKPT_BF16, CKPT_F32, CKPT_U32, CheckpointV1, IoError, NamedBlob, SafeTensors,
                         checkpoint_file_len, read_checkpoint, write_checkpoint, write_safetensors)

GOLD = Path(__file__).parent / "golden"
REF = Path("/root/reference")


def fixture_files():
    files = sorted(GOLD.rglob("*.safetensors"))
    if REF.exists():  # in the build container: every file the reference's tests hold
        files += sorted(p for p in REF.rglob("*.safetensors") if p.stat().st_size < 64 << 20)
    return files


@pytest.mark.parametrize("path", fixture_files(), ids=lambda p: "/".join(p.parts[-3:]))
def test_reads_what_the_safetensors_library_reads(path):
    ours = SafeTensors(path)
    with safe_open(str(path), "np") as theirs:
        assert ours.metadata() == (theirs.metadata() or {})
        assert ours.names() == sorted(theirs.keys(), key=lambda k: k.encode())
        for name in theirs.keys():
            sl = theirs.get_slice(name)
            info = ours.info(name)
            assert info.dtype == sl.get_dtype() and list(info.shape) == list(sl.get_shape())
            if info.dtype == "BF16":  # numpy cannot hold it: compare through the exact widening
                import torch
                from safetensors.torch import load_file
                want = load_file(str(path))[name].to(torch.float32).numpy()
                assert np.array_equal(ours.read_f32(name).view(np.uint32), want.view(np.uint32))
                continue
            want = theirs.get_tensor(name)
            assert ours.read_bytes(name) == np.ascontiguousarray(want).tobytes()
            if info.dtype in ("F32", "F16"):
                assert np.array_equal(ours.read_f32(name).view(np.uint32), want.astype(np.float32).view(np.uint32))
            if info.nbytes >= 8:
                assert ours.read_bytes(name, 3, 5) == np.ascontiguousarray(want).tobytes()[3:8]


def test_files_written_here_are_read_by_the_library_and_by_the_reader(tmp_path):
    r = np.random.default_rng(0)
    tensors = {"b.weight": r.standard_normal((3, 5)).astype(np.float32), "a": np.arange(7, dtype=np.int64),
               "z/ids": r.integers(0, 2**32, (2, 2, 2), dtype=np.uint64).astype(np.uint32),
               "empty": np.zeros((0, 4), np.float32), "scalar": np.array(2.5, np.float32),
               "half": r.standard_normal(9).astype(np.float16), "bits": r.integers(0, 65536, 6).astype(np.uint16),
               'quo"te\\né': np.ones(1, np.uint8)}
    meta = {"ojas.spec": json.dumps({"n_layer": 2}), "k": 'v"\\\n\t\x01é'}
    path = tmp_path / "w.safetensors"
    write_safetensors(path, tensors, meta, dtypes={"bits": "BF16"})
    raw = path.read_bytes()
    (hlen,) = struct.unpack("<Q", raw[:8])
    assert hlen % 8 == 0 and raw[8 + hlen - 1:8 + hlen] in (b" ", b"}")
    ours = SafeTensors(path)
    assert ours.metadata() == meta and ours.info("bits").dtype == "BF16"
    with safe_open(str(path), "np") as theirs:
        assert theirs.metadata() == meta
        for name, arr in tensors.items():
            if name == "bits":
                continue
            assert np.array_equal(theirs.get_tensor(name), arr), name
            assert np.array_equal(ours.read(name), arr), name
    want = (tensors["bits"].astype(np.uint32) << 16).view(np.float32)
    assert np.array_equal(ours.read_f32("bits").view(np.uint32), want.view(np.uint32))
    # Rewriting replaces the file in one step and leaves no temporary behind.
    write_safetensors(path, {"only": np.zeros(2, np.float32)})
    assert SafeTensors(path).names() == ["only"] and [p.name for p in tmp_path.iterdir()] == ["w.safetensors"]
    for bad, what in (({"": np.zeros(1, np.float32)}, "empty"), ({"__metadata__": np.zeros(1, np.float32)}, "not a tensor")):
        with pytest.raises(IoError, match=what):
            write_safetensors(path, bad)
    assert SafeTensors(path).names() == ["only"]


def frame(header: bytes, payload: bytes = b"") -> bytes:
    return struct.pack("<Q", len(header)) + header + payload


GOOD = b'{"__metadata__":{"k":"v"},"w":{"dtype":"U16","shape":[1],"data_offsets":[0,2]}}'


def refused(tmp_path, blob: bytes, what: str):
    p = tmp_path / "bad.safetensors"
    p.write_bytes(blob)
    with pytest.raises(IoError, match=what or None):
        SafeTensors(p)


def test_header_refuses_floats_bools_nulls_and_negatives_everywhere(tmp_path):
    p = tmp_path / "good.safetensors"
    p.write_bytes(frame(GOOD, b"\0\0"))
    assert SafeTensors(p).read("w").tolist() == [0]
    edits = [(b'"shape":[1]', b'"shape":[1.0]'), (b'"shape":[1]', b'"shape":[1e0]'), (b'"shape":[1]', b'"shape":[true]'),
             (b'"shape":[1]', b'"shape":[null]'), (b'"shape":[1]', b'"shape":[-1]'), (b'"shape":[1]', b'"shape":[-0]'),
             (b'"shape":[1]', b'"shape":null'), (b'"data_offsets":[0,2]', b'"data_offsets":[0,2.0]'),
             (b'"data_offsets":[0,2]', b'"data_offsets":[-0,2]'), (b'"data_offsets":[0,2]', b'"data_offsets":[false,2]'),
             (b'"dtype":"U16"', b'"dtype":true'), (b'"dtype":"U16"', b'"dtype":null'), (b'"k":"v"', b'"k":null'),
             (b'"k":"v"', b'"k":1.5'), (b'"k":"v"', b'"k":false'), (b'"__metadata__":{"k":"v"}', b'"__metadata__":null')]
    for old, new in edits:
        assert old in GOOD
        refused(tmp_path, frame(GOOD.replace(old, new, 1), b"\0\0"), "")
    for root in (b"[]", b"null", b"true", b"1.5", b"-1", b'"s"'):
        refused(tmp_path, frame(root), "not a JSON object")


def test_malformed_files_are_refused(tmp_path):
    one = lambda entry, payload=b"\0" * 4: frame(b'{"w":' + entry + b"}", payload)
    cases = [
        (b"", "header length"), (b"\x05\0\0", "header length"),
        (struct.pack("<Q", 0) + b"{}", "outside 1"), (struct.pack("<Q", 10**9) + b"{}", "outside 1"),
        (struct.pack("<Q", 2**64 - 4) + b"{}", "outside 1"),  # would wrap when 8 is added
        (struct.pack("<Q", 50) + b"{}", "runs past the end"),
        (frame(b'{"a":{"dtype":"U8","shape":[1],"data_offsets":[0,1]},"a":{"dtype":"U8","shape":[1],"data_offsets":[1,2]}}',
               b"\0\0"), "duplicate key"),
        (frame(b'{"a":{"dtype":"U8","shape":[1],"data_offsets":[0,1]},"\\u0061":{"dtype":"U8","shape":[1],"data_offsets":[1,2]}}',
               b"\0\0"), "duplicate key"),
        (frame(b'{"a":{"dtype":"U8","shape":[2],"data_offsets":[0,2]},"b":{"dtype":"U8","shape":[2],"data_offsets":[1,3]}}',
               b"\0\0\0"), "gap or overlap"),
        (frame(b'{"a":{"dtype":"U8","shape":[1],"data_offsets":[1,2]}}', b"\0\0"), "gap or overlap"),
        (one(b'{"dtype":"U8","shape":[2],"data_offsets":[0,2]}'), "unindexed gap"),
        (one(b'{"dtype":"F32","shape":[2],"data_offsets":[0,4]}'), "4 bytes in data_offsets"),
        (one(b'{"dtype":"F32","shape":[1],"data_offsets":[0,8]}'), "outside the 4-byte data buffer"),
        (one(b'{"dtype":"F32","shape":[1],"data_offsets":[4,0]}'), "outside"),
        (one(b'{"dtype":"U8","shape":[4294967296,4294967296,2],"data_offsets":[0,4]}'), "overflows"),
        (one(b'{"dtype":"U8","shape":[2,4294967296,4294967296],"data_offsets":[0,4]}'), "overflows"),
        (one(b'{"dtype":"F4","shape":[3],"data_offsets":[0,2]}'), "whole number of bytes"),
        (one(b'{"dtype":"F33","shape":[1],"data_offsets":[0,4]}'), "unknown dtype"),
        (one(b'{"dtype":"F32","shape":[1],"data_offsets":[0,4],"extra":1}'), "unexpected or mistyped"),
        (one(b'{"dtype":"F32","shape":[1]}'), "needs dtype, shape and data_offsets"),
        (one(b'{"dtype":"F32","shape":[1],"data_offsets":[0,4,8]}'), r"not \[begin, end\]"),
        (one(b'{"dtype":"F32","shape":[[1]],"data_offsets":[0,4]}'), "deeper|non-integer"),
        (one(b'[1]'), "not an object"),
        (frame(b'{"":{"dtype":"F32","shape":[1],"data_offsets":[0,4]}}', b"\0" * 4), "name is empty"),
        (frame(b'{"w\xff":{"dtype":"F32","shape":[1],"data_offsets":[0,4]}}', b"\0" * 4), "UTF-8"),
        (frame(b'{"w":{"dtype":"F32","shape":[01],"data_offsets":[0,4]}}', b"\0" * 4), "leading zero"),
        (frame(b'{"w":{"dtype":"F32","shape":[1],"data_offsets":[0,4]}} x', b"\0" * 4), "trailing"),
        (frame(b'{"w":{"dtype":"F32","shape":[1],"data_offsets":[0,4]}', b"\0" * 4), "expected|end of JSON"),
        (frame(b'{"w":{"dtype":"F32","shape":[18446744073709551616],"data_offsets":[0,4]}}', b"\0" * 4), "exceeds u64"),
        (frame(b'{"w":{"dtype":"F\\ud800","shape":[1],"data_offsets":[0,4]}}', b"\0" * 4), "surrogate"),
    ]
    for blob, what in cases:
        refused(tmp_path, blob, what)
    # An empty tensor with a valid dtype is fine, and so is a header padded with spaces.
    p = tmp_path / "ok.safetensors"
    p.write_bytes(frame(b'{"e":{"dtype":"F32","shape":[0,3],"data_offsets":[0,0]}}   '))
    assert SafeTensors(p).read("e").shape == (0, 3)
    with pytest.raises(IoError, match="No such file"):
        SafeTensors(tmp_path / "absent")
    with pytest.raises(IoError, match="not a regular file"):
        SafeTensors(tmp_path)


def test_reads_are_bounded_and_notice_a_file_that_changed(tmp_path):
    p = tmp_path / "t.safetensors"
    save_file({"w": np.arange(10, dtype=np.float32), "i": np.arange(3, dtype=np.int64)}, str(p))
    s = SafeTensors(p)
    assert s.read_bytes("w", 36, 4) == np.float32(9).tobytes() and s.read_bytes("w", 40, 0) == b""
    for off, n in ((37, 4), (41, 0), (0, 41)):
        with pytest.raises(IoError, match="outside its 40 bytes"):
            s.read_bytes("w", off, n)
    with pytest.raises(IoError, match="no tensor named"):
        s.info("nope")
    with pytest.raises(IoError, match="is not F32, BF16 or F16"):
        s.read_f32("i")
    with open(p, "ab") as f:
        f.write(b"\0")
    with pytest.raises(IoError, match="changed since it was opened"):
        s.read("w")


def le(fmt, *v):
    return struct.pack("<" + fmt, *v)


def test_checkpoint_layout_is_the_documented_one(tmp_path):
    """Assembled by hand from docs/checkpoint-v1.md: prefix, body order, section framing, record fields."""
    w0 = np.arange(6, dtype=np.float32).tobytes()
    ids = np.arange(4, dtype=np.uint32).tobytes()
    ckpt = CheckpointV1(config=b'{"lr":0.1}', tokenizer_hash=bytes(range(32)), git_sha=bytes(range(100, 120)), step=7,
                        cursor=(3, 41), rng_state=le("IIQ", 1, 1, 1337),
                        weights=[NamedBlob("tok_emb.weight", CKPT_F32, (2, 3), 0, w0),
                                 NamedBlob("ids", CKPT_U32, (2,), 8, ids)],
                        muon_momentum=[NamedBlob("m", CKPT_BF16, (1, 2), 0, b"\x80\x3f\x00\x40")],
                        adamw_first_moment=[], adamw_second_moment=[NamedBlob("v", CKPT_F32, (), 0, le("f", 0.5))])

    def record(name, tag, shape, off, payload):
        return (le("Q", len(name)) + name.encode() + le("II", tag, len(shape)) + b"".join(le("Q", d) for d in shape) +
                le("QQ", off, len(payload)) + payload)

    def section(*records):
        body = le("Q", len(records)) + b"".join(records)
        return le("Q", len(body)) + body

    want = (b"OJAS0001" + le("I", 1) + le("Q", 10) + b'{"lr":0.1}' + bytes(range(32)) + bytes(range(100, 120)) +
            le("QQQ", 7, 3, 41) + le("Q", 16) + le("IIQ", 1, 1, 1337) +
            section(record("tok_emb.weight", 0, (2, 3), 0, w0), record("ids", 3, (2,), 8, ids)) +
            section(record("m", 1, (1, 2), 0, b"\x80\x3f\x00\x40")) + section() +
            section(record("v", 0, (), 0, le("f", 0.5))))
    path = tmp_path / "state.ojck"
    write_checkpoint(path, ckpt)
    assert path.read_bytes() == want and checkpoint_file_len(ckpt) == len(want)
    assert read_checkpoint(path) == ckpt
    assert [p.name for p in tmp_path.iterdir()] == ["state.ojck"]
    # Every shorter file is refused; so are trailing bytes, another magic and another version.
    bad = tmp_path / "bad.ojck"
    for n in list(range(0, 130)) + [len(want) - 1]:
        bad.write_bytes(want[:n])
        with pytest.raises(IoError, match="truncated|read_prefix|section|cannot fit"):
            read_checkpoint(bad)
    for blob, what in ((want + b"\0", "trailing bytes"), (b"OJAS0002" + want[8:], "bad magic"),
                       (want[:8] + le("I", 2) + want[12:], "version 2")):
        bad.write_bytes(blob)
        with pytest.raises(IoError, match=what):
            read_checkpoint(bad)


def test_checkpoint_refusals_and_random_round_trips(tmp_path):
    path = tmp_path / "c.ojck"
    blob = lambda **kw: NamedBlob(**{"name": "w", "dtype_tag": CKPT_F32, "shape": (2,), "byte_offset": 0,
                                    "payload": bytes(8), **kw})
    for bad, what in (([blob(byte_offset=1)], "exceeds payload"), ([blob(shape=(3,))], "exceeds payload"),
                      ([blob(), blob()], "duplicate key"), ([blob(shape=(2**40, 2**40))], "overflows"),
                      ([blob(dtype_tag=9)], "unknown dtype tag")):
        with pytest.raises(IoError, match=what):
            write_checkpoint(path, CheckpointV1(weights=bad))
    assert not path.exists()
    # The same name in two different sections is fine; a zero extent makes any window fit.
    ok = CheckpointV1(weights=[blob(), blob(name="z", shape=(0, 2**60), payload=b"")], adamw_first_moment=[blob()])
    write_checkpoint(path, ok)
    assert read_checkpoint(path) == ok
    # A record count or rank that its section cannot hold is refused before anything is allocated.
    head = b"OJAS0001" + le("I", 1) + le("Q", 0) + bytes(52) + le("QQQ", 0, 0, 0) + le("Q", 0)
    empty = le("QQ", 8, 0)
    path.write_bytes(head + le("QQ", 8, 2**61) + empty * 3)
    with pytest.raises(IoError, match="cannot fit the section"):
        read_checkpoint(path)
    rec = le("Q", 1) + b"w" + le("II", 0, 2**31) + le("QQ", 0, 0)
    path.write_bytes(head + le("QQ", 8 + len(rec), 1) + rec + empty * 3)
    with pytest.raises(IoError, match="rank .* cannot fit"):
        read_checkpoint(path)
    rec = le("Q", 1) + b"w" + le("II", 0, 1) + le("Q", 4) + le("QQ", 0, 8) + bytes(8)  # 4 floats in 8 bytes
    path.write_bytes(head + le("QQ", 8 + len(rec), 1) + rec + empty * 3)
    with pytest.raises(IoError, match="exceeds payload"):
        read_checkpoint(path)
    r = np.random.default_rng(3)
    for trial in range(20):
        def blobs(k):
            out = []
            for i in range(k):
                shape = tuple(int(x) for x in r.integers(0, 5, r.integers(0, 4)))
                tag = int(r.integers(0, 4))
                size = int(np.prod(shape, dtype=np.int64)) * (4 if tag in (0, 3) else 2)
                off = int(r.integers(0, 9))
                out.append(NamedBlob(f"t{trial}.{i}é", tag, shape, off, r.bytes(off + size + int(r.integers(0, 3)))))
            return out
        c = CheckpointV1(config=r.bytes(int(r.integers(0, 40))), tokenizer_hash=r.bytes(32), git_sha=r.bytes(20),
                         step=int(r.integers(0, 2**63)), cursor=(int(r.integers(0, 2**40)), int(r.integers(0, 2**40))),
                         rng_state=r.bytes(int(r.integers(0, 20))), weights=blobs(3), muon_momentum=blobs(2),
                         adamw_first_moment=blobs(1), adamw_second_moment=blobs(0))
        write_checkpoint(path, c)
        assert path.stat().st_size == checkpoint_file_len(c)
        assert read_checkpoint(path) == c


def test_spec_and_train_config_json_follow_the_reference_formats():
    from ojas_amd.nanolab import NanolabSpec, TrainConfig, rust_f64, spec_from_json, spec_to_json

    for x, want in ((1e-6, "1e-6"), (1e-5, "1e-5"), (3e-5, "3e-5"), (0.0001, "0.0001"), (0.0006, "0.0006"), (1.0, "1.0"),
                    (10000.0, "10000.0"), (1e15, "1000000000000000.0"), (1e16, "1e16"), (2.5e20, "2.5e20"),
                    (1.5e-7, "1.5e-7"), (0.1, "0.1"), (123456.789, "123456.789"), (0.0, "0.0"), (-0.5, "-0.5")):
        assert rust_f64(x) == want and float(rust_f64(x)) == x
    # The spec the reference's oracle wrote into the tiny fixture parses, and re-encodes to the same object.
    meta = SafeTensors(GOLD / "tiny" / "init.safetensors").metadata()["ojas.spec"]
    spec = spec_from_json(meta)
    assert (spec.n_layer, spec.n_embd, spec.head_dim, spec.vocab, spec.max_seq) == (2, 64, 16, 256, 32)
    text = spec_to_json(spec)
    assert json.loads(text) == json.loads(meta)
    assert text.startswith('{"format":"ojas-spec-v1","arch":"nanolab-gpt","vocab":256,') and '"rms_eps":1e-6,' in text
    windowed = NanolabSpec(2, 64, 4, 2, 16, 192, 256, window=8, max_seq=32)
    assert '"format":"ojas-spec-v2"' in spec_to_json(windowed) and spec_from_json(spec_to_json(windowed)) == windowed
    cfg = TrainConfig(seq_len=32, batch=2, accum=2, data_seed=1337, total_steps=40, warmup_steps=4)
    assert cfg.to_json() == ('{"accum":2,"adam_lr":0.0006,"batch":2,"chunk_cols":8192,"chunk_rows":1024,"data_seed":1337,'
                             '"decay_frac":0.0,"grad_clip":1.0,"ignore":false,"ignore_index":0,"matrix_lr":0.025,'
                             '"on_nonfinite":"abort","schedule":"cosine","seq_len":32,"total_steps":40,"warmup_steps":4}')
    assert list(json.loads(cfg.to_json())) == sorted(json.loads(cfg.to_json()))
