"""safetensors files and the checkpoint-v1 state file: the host-side mirror of `ojas_io`
(ojas-io/src/safetensors.rs, ojas-io/src/checkpoint.rs) over the C ABI of `include/ojas_io.h`.
No parsing or arithmetic here; one `IoError` with a message, as in the reference."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from pathlib import Path
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

LIB_PATH = Path(__file__).resolve().parent / "libojas_io.so"

# dtype tag -> numpy dtype for the tags numpy can hold (BF16 is kept as its 16 bits).
NUMPY_OF = {"F32": np.float32, "F16": np.float16, "BF16": np.uint16, "F64": np.float64, "I64": np.int64,
            "I32": np.int32, "I16": np.int16, "I8": np.int8, "U64": np.uint64, "U32": np.uint32, "U16": np.uint16,
            "U8": np.uint8, "BOOL": np.bool_}
# checkpoint-v1 dtype tags (ojas-core/src/checkpoint.rs)
CKPT_F32, CKPT_BF16, CKPT_F16, CKPT_U32 = 0, 1, 2, 3


class IoError(RuntimeError):
    """`ojas_io::IoError`."""


class _TensorOut(C.Structure):
    _fields_ = [("name", C.c_char_p), ("dtype", C.c_char_p), ("rank", C.c_uint32), ("shape", C.POINTER(C.c_uint64)),
                ("data", C.c_void_p), ("nbytes", C.c_uint64)]


class _Blob(C.Structure):
    _fields_ = [("name", C.c_char_p), ("dtype_tag", C.c_uint32), ("rank", C.c_uint32), ("shape", C.POINTER(C.c_uint64)),
                ("byte_offset", C.c_uint64), ("payload", C.c_void_p), ("payload_len", C.c_uint64)]


class _Checkpoint(C.Structure):
    _fields_ = [("config", C.c_void_p), ("config_len", C.c_uint64), ("tokenizer_hash", C.c_uint8 * 32),
                ("git_sha", C.c_uint8 * 20), ("step", C.c_uint64), ("cursor_shard", C.c_uint64),
                ("cursor_token_index", C.c_uint64), ("rng_state", C.c_void_p), ("rng_state_len", C.c_uint64),
                ("sections", C.POINTER(_Blob) * 4), ("counts", C.c_uint64 * 4)]


_lib: Optional[C.CDLL] = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise IoError(f"{LIB_PATH} is not built; run __graft_entry__.build()")
        _lib = C.CDLL(str(LIB_PATH))
        _lib.oio_last_error.restype = C.c_size_t
        for name in ("oio_st_count", "oio_st_metadata_count"):
            getattr(_lib, name).restype = C.c_uint64
        for name in ("oio_st_name", "oio_st_metadata_key", "oio_st_metadata"):
            getattr(_lib, name).restype = C.c_char_p
        _lib.oio_st_close.restype = None
        _lib.oio_ckpt_free.restype = None
    return _lib


def _check(rc: int):
    if rc != 0:
        n = lib().oio_last_error(None, C.c_size_t(0))
        buf = C.create_string_buffer(n + 1)
        lib().oio_last_error(buf, C.c_size_t(n + 1))
        raise IoError(buf.value.decode("utf-8", "replace"))


@dataclass
class TensorInfo:
    dtype: str
    shape: Tuple[int, ...]
    nbytes: int


class SafeTensors:
    """`SafeTensors::open` (safetensors.rs:408): the header is parsed and checked at open, tensors are
    read on demand."""

    def __init__(self, path):
        self._h = C.c_void_p()
        _check(lib().oio_st_open(str(path).encode(), C.byref(self._h)))

    def close(self):
        if self._h:
            lib().oio_st_close(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def names(self) -> List[str]:
        return [lib().oio_st_name(self._h, C.c_uint64(i)).decode() for i in range(lib().oio_st_count(self._h))]

    def metadata(self) -> Dict[str, str]:
        out = {}
        for i in range(lib().oio_st_metadata_count(self._h)):
            key = lib().oio_st_metadata_key(self._h, C.c_uint64(i))
            out[key.decode()] = lib().oio_st_metadata(self._h, key).decode()
        return out

    def info(self, name: str) -> TensorInfo:
        dtype, rank, nbytes = C.c_char_p(), C.c_uint32(), C.c_uint64()
        shape = (C.c_uint64 * 16)()
        _check(lib().oio_st_info(self._h, name.encode(), C.byref(dtype), C.byref(rank), shape, C.c_uint32(16),
                                 C.byref(nbytes)))
        return TensorInfo(dtype.value.decode(), tuple(int(shape[i]) for i in range(rank.value)), int(nbytes.value))

    def read_bytes(self, name: str, offset: int = 0, n: Optional[int] = None) -> bytes:
        n = self.info(name).nbytes - offset if n is None else n
        buf = C.create_string_buffer(max(n, 1))
        _check(lib().oio_st_read(self._h, name.encode(), C.c_uint64(offset), buf, C.c_uint64(n)))
        return buf.raw[:n]

    def read(self, name: str) -> np.ndarray:
        """The tensor in its own dtype (BF16 as uint16 bit patterns)."""
        info = self.info(name)
        if info.dtype not in NUMPY_OF:
            raise IoError(f"{name}: dtype {info.dtype} has no numpy form; use read_bytes")
        return np.frombuffer(self.read_bytes(name), dtype=NUMPY_OF[info.dtype]).reshape(info.shape).copy()

    def read_f32(self, name: str) -> np.ndarray:
        """`read_f32_widened`: F32 as is, BF16 / F16 widened exactly."""
        info = self.info(name)
        out = np.empty(info.shape, np.float32)
        _check(lib().oio_st_read_f32(self._h, name.encode(), out.ctypes.data_as(C.c_void_p), C.c_uint64(out.size)))
        return out


def write_safetensors(path, tensors: Dict[str, np.ndarray], metadata: Optional[Dict[str, str]] = None,
                      dtypes: Optional[Dict[str, str]] = None):
    """`write_safetensors` (safetensors.rs:1224): tensors in dict order. `dtypes` overrides the tag
    numpy's dtype gives (a uint16 array holding bf16 bits is written as "BF16")."""
    tag_of = {np.dtype(v): k for k, v in NUMPY_OF.items() if k != "BF16"}
    n = len(tensors)
    outs = (_TensorOut * max(n, 1))()
    keep = []
    for i, (name, arr) in enumerate(tensors.items()):
        arr = np.require(arr, requirements="C")  # keeps a 0-d array 0-d
        tag = (dtypes or {}).get(name) or tag_of.get(arr.dtype)
        if tag is None:
            raise IoError(f"{name}: numpy dtype {arr.dtype} has no safetensors tag")
        shape = (C.c_uint64 * max(arr.ndim, 1))(*arr.shape)
        keep += [arr, shape]
        outs[i] = _TensorOut(name.encode(), tag.encode(), arr.ndim, shape, arr.ctypes.data, arr.nbytes)
    meta = metadata or {}
    keys = (C.c_char_p * max(len(meta), 1))(*[k.encode() for k in meta])
    vals = (C.c_char_p * max(len(meta), 1))(*[v.encode() for v in meta.values()])
    _check(lib().oio_st_write(str(path).encode(), outs, C.c_uint64(n), keys, vals, C.c_uint64(len(meta))))


@dataclass
class NamedBlob:
    """`ojas_core::NamedBlob` (ojas-core/src/checkpoint.rs:69-80)."""
    name: str
    dtype_tag: int
    shape: Tuple[int, ...]
    byte_offset: int
    payload: bytes


@dataclass
class CheckpointV1:
    """`ojas_core::CheckpointV1` (ojas-core/src/checkpoint.rs:104-115)."""
    config: bytes = b""
    tokenizer_hash: bytes = bytes(32)
    git_sha: bytes = bytes(20)
    step: int = 0
    cursor: Tuple[int, int] = (0, 0)
    rng_state: bytes = b""
    weights: List[NamedBlob] = field(default_factory=list)
    muon_momentum: List[NamedBlob] = field(default_factory=list)
    adamw_first_moment: List[NamedBlob] = field(default_factory=list)
    adamw_second_moment: List[NamedBlob] = field(default_factory=list)

    def sections(self):
        return [self.weights, self.muon_momentum, self.adamw_first_moment, self.adamw_second_moment]


def _to_c(ckpt: CheckpointV1):
    c = _Checkpoint()
    keep = []

    def blob_ptr(data: bytes):
        buf = C.create_string_buffer(data, max(len(data), 1))
        keep.append(buf)
        return C.cast(buf, C.c_void_p)

    if len(ckpt.tokenizer_hash) != 32 or len(ckpt.git_sha) != 20:
        raise IoError("checkpoint: tokenizer_hash is 32 bytes and git_sha is 20")
    c.config, c.config_len = blob_ptr(ckpt.config), len(ckpt.config)
    c.tokenizer_hash[:] = ckpt.tokenizer_hash
    c.git_sha[:] = ckpt.git_sha
    c.step, (c.cursor_shard, c.cursor_token_index) = ckpt.step, ckpt.cursor
    c.rng_state, c.rng_state_len = blob_ptr(ckpt.rng_state), len(ckpt.rng_state)
    for s, blobs in enumerate(ckpt.sections()):
        arr = (_Blob * max(len(blobs), 1))()
        for i, b in enumerate(blobs):
            shape = (C.c_uint64 * max(len(b.shape), 1))(*b.shape)
            keep.append(shape)
            arr[i] = _Blob(b.name.encode(), b.dtype_tag, len(b.shape), shape, b.byte_offset, blob_ptr(b.payload),
                           len(b.payload))
        keep.append(arr)
        c.sections[s] = arr
        c.counts[s] = len(blobs)
    return c, keep


def checkpoint_file_len(ckpt: CheckpointV1) -> int:
    c, _keep = _to_c(ckpt)
    n = C.c_uint64()
    _check(lib().oio_ckpt_file_len(C.byref(c), C.byref(n)))
    return int(n.value)


def write_checkpoint(path, ckpt: CheckpointV1):
    c, _keep = _to_c(ckpt)
    _check(lib().oio_ckpt_write(str(path).encode(), C.byref(c)))


def read_checkpoint(path) -> CheckpointV1:
    h, view = C.c_void_p(), _Checkpoint()
    _check(lib().oio_ckpt_read(str(path).encode(), C.byref(h), C.byref(view)))
    try:
        out = CheckpointV1(config=C.string_at(view.config, view.config_len), tokenizer_hash=bytes(view.tokenizer_hash),
                           git_sha=bytes(view.git_sha), step=int(view.step),
                           cursor=(int(view.cursor_shard), int(view.cursor_token_index)),
                           rng_state=C.string_at(view.rng_state, view.rng_state_len))
        for s, target in enumerate(out.sections()):
            for i in range(view.counts[s]):
                b = view.sections[s][i]
                target.append(NamedBlob(b.name.decode(), int(b.dtype_tag), tuple(int(b.shape[d]) for d in range(b.rank)),
                                        int(b.byte_offset), C.string_at(b.payload, b.payload_len)))
        return out
    finally:
        lib().oio_ckpt_free(h)
