"""`TokenBin` and `BatchSampler`: the host-side mirror of the reference's data step
(ojas-data/src/tokens.rs, ojas-data/src/sampler.rs) over the C ABI of `include/ojas_data.h`.

Same names, argument meaning and error behaviour (one `DataError` with a message); no arithmetic
here. `BatchSampler.next_starts` + `MiBackend.token_windows` build a batch on the device from a bin
that is resident in HBM.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from pathlib import Path
from typing import Optional, Tuple

import numpy as np

LIB_PATH = Path(__file__).resolve().parent / "libojas_data.so"
HEADERLESS, FINEWEB = 0, 1
WIDTH_ANY, WIDTH_U16, WIDTH_U32 = 0, 2, 4


class DataError(RuntimeError):
    """`ojas_data::DataError` (ojas-data/src/error.rs)."""


def _load() -> C.CDLL:
    if not LIB_PATH.exists():
        raise DataError(f"{LIB_PATH} is not built; run __graft_entry__.build()")
    lib = C.CDLL(str(LIB_PATH))
    lib.odata_last_error.restype = C.c_size_t
    lib.odata_bin_len.restype = C.c_uint64
    lib.odata_sampler_windows_per_epoch.restype = C.c_uint64
    for name in ("odata_bin_close", "odata_sampler_free", "odata_sampler_cursor", "odata_rng_state_encode"):
        getattr(lib, name).restype = None
    return lib


_lib: Optional[C.CDLL] = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def _check(rc: int):
    if rc != 0:
        n = lib().odata_last_error(None, C.c_size_t(0))
        buf = C.create_string_buffer(n + 1)
        lib().odata_last_error(buf, C.c_size_t(n + 1))
        raise DataError(buf.value.decode("utf-8", "replace"))


@dataclass(frozen=True)
class DataCursor:
    """`ojas_core::DataCursor`: `shard` is the epoch, `token_index` the next window's ordinal."""
    shard: int = 0
    token_index: int = 0


@dataclass
class Batch:
    """`ojas_data::Batch` (sampler.rs:128-134): x, y are u32 [batch, seq_len]."""
    x: np.ndarray
    y: np.ndarray
    batch: int
    seq_len: int


class TokenBin:
    def __init__(self, path, layout: int, width: int):
        self._h = C.c_void_p()
        _check(lib().odata_bin_open(str(path).encode(), C.c_int32(layout), C.c_int32(width), C.byref(self._h)))

    @classmethod
    def open_headerless_u16(cls, path) -> "TokenBin":
        return cls(path, HEADERLESS, WIDTH_U16)

    open_headerless = open_headerless_u16

    @classmethod
    def open_headerless_u32(cls, path) -> "TokenBin":
        return cls(path, HEADERLESS, WIDTH_U32)

    @classmethod
    def open_fineweb(cls, path) -> "TokenBin":
        return cls(path, FINEWEB, WIDTH_ANY)

    @classmethod
    def open_fineweb_u16(cls, path) -> "TokenBin":
        return cls(path, FINEWEB, WIDTH_U16)

    @classmethod
    def open_fineweb_u32(cls, path) -> "TokenBin":
        return cls(path, FINEWEB, WIDTH_U32)

    def close(self):
        if self._h:
            lib().odata_bin_close(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __len__(self) -> int:
        return int(lib().odata_bin_len(self._h))

    def bytes_per_token(self) -> int:
        return int(lib().odata_bin_bytes_per_token(self._h))

    def read_into_u32(self, index: int, n: int) -> np.ndarray:
        out = np.empty(n, np.uint32)
        _check(lib().odata_bin_read_u32(self._h, C.c_uint64(index), out.ctypes.data_as(C.c_void_p), C.c_uint64(n)))
        return out

    def read_into(self, index: int, n: int) -> np.ndarray:
        out = np.empty(n, np.uint16)
        _check(lib().odata_bin_read_u16(self._h, C.c_uint64(index), out.ctypes.data_as(C.c_void_p), C.c_uint64(n)))
        return out

    def read_raw(self, index: int, n: int) -> np.ndarray:
        """The little-endian token words themselves (u16 or u32 by the bin's width)."""
        out = np.empty(n, np.uint16 if self.bytes_per_token() == 2 else np.uint32)
        _check(lib().odata_bin_read_raw(self._h, C.c_uint64(index), out.ctypes.data_as(C.c_void_p), C.c_uint64(n)))
        return out


class BatchSampler:
    """`BatchSampler::new` / `resume` (sampler.rs:153-214). `bin` is a `TokenBin`, or a token count
    for a bin held elsewhere (then only `next_starts` and `window_start` work)."""

    def __init__(self, bin, seq_len: int, batch: int, seed: int, cursor: DataCursor = DataCursor()):
        self._h = C.c_void_p()
        self._bin = bin  # keeps the bin alive
        self.seq_len, self.batch, self.seed = seq_len, batch, seed
        args = (C.c_uint64(seq_len), C.c_uint64(batch), C.c_uint64(seed), C.c_uint64(cursor.shard),
                C.c_uint64(cursor.token_index), C.byref(self._h))
        if isinstance(bin, TokenBin):
            _check(lib().odata_sampler_new(bin._h, *args))
        else:
            _check(lib().odata_sampler_new_detached(C.c_uint64(int(bin)), *args))

    def __del__(self):
        try:
            if self._h:
                lib().odata_sampler_free(self._h)
                self._h = C.c_void_p()
        except Exception:
            pass

    def windows_per_epoch(self) -> int:
        return int(lib().odata_sampler_windows_per_epoch(self._h))

    def cursor(self) -> DataCursor:
        e, o = C.c_uint64(), C.c_uint64()
        lib().odata_sampler_cursor(self._h, C.byref(e), C.byref(o))
        return DataCursor(int(e.value), int(o.value))

    def window_start(self, epoch: int, ordinal: int) -> int:
        start = C.c_uint64()
        _check(lib().odata_sampler_window_start(self._h, C.c_uint64(epoch), C.c_uint64(ordinal), C.byref(start)))
        return int(start.value)

    def next_batch(self) -> Batch:
        x = np.empty((self.batch, self.seq_len), np.uint32)
        y = np.empty((self.batch, self.seq_len), np.uint32)
        _check(lib().odata_sampler_next_batch(self._h, x.ctypes.data_as(C.c_void_p), y.ctypes.data_as(C.c_void_p)))
        return Batch(x, y, self.batch, self.seq_len)

    def next_starts(self) -> np.ndarray:
        starts = np.empty(self.batch, np.uint64)
        _check(lib().odata_sampler_next_starts(self._h, starts.ctypes.data_as(C.c_void_p)))
        return starts


def rng_state_encode(seed: int) -> bytes:
    out = (C.c_uint8 * 16)()
    lib().odata_rng_state_encode(C.c_uint64(seed), out)
    return bytes(out)


def rng_state_decode(data: bytes) -> int:
    seed = C.c_uint64()
    buf = (C.c_uint8 * max(len(data), 1)).from_buffer_copy(data.ljust(1, b"\0"))
    _check(lib().odata_rng_state_decode(buf, C.c_uint64(len(data)), C.byref(seed)))
    return int(seed.value)
