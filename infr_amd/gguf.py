"""Host-side mirror of ``infr_gguf::Gguf`` over the reader in ``libinfr_hip.so``.

``Gguf.open(path)`` maps a GGUF file, or the whole ``gguf-split`` shard set the file belongs to,
and exposes what the reference's ``WeightSource`` does (crates/infr-core/src/loader.rs:85-92;
crates/infr-gguf/src/lib.rs:476-1008): ``metadata()``, ``tensors()``, ``tensor_bytes(name)``,
``tensor_file_range(name)``, ``shards()``, ``chat_template()``. ``upload(be, name)`` copies a
tensor's raw blocks from the mapping into a weights buffer of a ``HipBackend``. All parsing and
checking happens in the native library; this file only converts handles into Python values.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass

import numpy as np

from .backend import Buffer, HipBackend, InfrError, Status, _GgufTensor, _vp, load_library

BOOL, U64, I64, F64, STR, ARR = range(6)


@dataclass(frozen=True)
class TensorInfo:
    """infr_core::loader::TensorInfo. ``shape[0]`` is the fastest-varying axis."""
    name: str
    shape: tuple[int, ...]
    dtype: int          # ggml type id
    offset: int         # first byte in the concatenated file address space
    nbytes: int


@dataclass(frozen=True)
class Shard:
    """gguf_split::Shard (crates/infr-core/src/gguf_split.rs:13-25)."""
    base: str
    index: int
    total: int
    width: int


def _err() -> str:
    return (load_library().infr_gguf_last_error() or b"").decode(errors="replace")


def _check(rc: int) -> None:
    if rc != 0:
        raise InfrError(rc, _err())


def parse_shard(fname: str) -> Shard | None:
    """``<base>-NNNNN-of-MMMMM.gguf`` -> Shard, else None (gguf_split.rs:44-68)."""
    lib = load_library()
    raw = fname.encode()
    base = C.create_string_buffer(len(raw) + 1)
    n, idx, tot, w = C.c_size_t(), C.c_uint32(), C.c_uint32(), C.c_size_t()
    if not lib.infr_gguf_parse_shard(raw, base, len(raw) + 1, C.byref(n), C.byref(idx), C.byref(tot), C.byref(w)):
        return None
    return Shard(base.raw[: n.value].decode(), idx.value, tot.value, w.value)


def shard_set(chosen: str) -> list[str]:
    """Every file name of the set ``chosen`` belongs to, in order (gguf_split.rs:72-88)."""
    lib = load_library()
    raw = chosen.encode()
    out = C.create_string_buffer(len(raw) + 16)
    n = lib.infr_gguf_shard_set(raw, 0, out, len(out))
    names = [out.value.decode()]
    for i in range(1, n):
        lib.infr_gguf_shard_set(raw, i, out, len(out))
        names.append(out.value.decode())
    return names


def block_layout(ggml_type: int) -> tuple[int, int]:
    """(elements, bytes) per block for every ggml type the reader accepts."""
    e, b = C.c_int(), C.c_int()
    if not load_library().infr_gguf_block_layout(int(ggml_type), C.byref(e), C.byref(b)):
        raise InfrError(Status.Unsupported, f"ggml type {ggml_type}")
    return e.value, b.value


def nbytes(ggml_type: int, numel: int) -> int:
    """infr_gguf::nbytes (lib.rs:428-430): rounded up to whole blocks."""
    ok = C.c_int()
    n = load_library().infr_gguf_nbytes(int(ggml_type), numel, C.byref(ok))
    if not ok.value:
        raise InfrError(Status.Loader, f"nbytes({ggml_type}, {numel}): unknown type or overflow")
    return n


def _value(lib, v):
    kind = lib.infr_gguf_value_kind(v)
    if kind == BOOL:
        o = C.c_int()
        lib.infr_gguf_value_bool(v, C.byref(o))
        return bool(o.value)
    if kind == U64:
        o = C.c_uint64()
        lib.infr_gguf_value_u64(v, C.byref(o))
        return o.value
    if kind == I64:
        o = C.c_int64()
        lib.infr_gguf_value_i64(v, C.byref(o))
        return o.value
    if kind == F64:
        o = C.c_double()
        lib.infr_gguf_value_f64(v, C.byref(o))
        return o.value
    if kind == STR:
        p, n = _vp(), C.c_size_t()
        lib.infr_gguf_value_str(v, C.byref(p), C.byref(n))
        return C.string_at(p.value, n.value).decode() if n.value else ""
    n = C.c_size_t()
    lib.infr_gguf_value_arr_len(v, C.byref(n))
    return [_value(lib, lib.infr_gguf_value_arr_at(v, i)) for i in range(n.value)]


class Metadata:
    """infr_core::loader::Metadata (loader.rs:52-68) over the first shard's key/value store."""

    def __init__(self, owner: "Gguf"):
        self._g = owner

    def keys(self) -> list[str]:
        lib, h = load_library(), self._g._handle()
        return [lib.infr_gguf_meta_key(h, i).decode() for i in range(lib.infr_gguf_n_meta(h))]

    def kind(self, key: str) -> int | None:
        lib = load_library()
        v = lib.infr_gguf_meta_get(self._g._handle(), key.encode())
        return lib.infr_gguf_value_kind(v) if v else None

    def get(self, key: str):
        lib = load_library()
        v = lib.infr_gguf_meta_get(self._g._handle(), key.encode())
        return _value(lib, v) if v else None

    def u64(self, key: str) -> int | None:
        """U64, or a non-negative I64; anything else is None (loader.rs:20-29, 62-64)."""
        lib = load_library()
        v = lib.infr_gguf_meta_get(self._g._handle(), key.encode())
        o = C.c_uint64()
        return o.value if v and lib.infr_gguf_value_u64(v, C.byref(o)) else None

    def f64(self, key: str) -> float | None:
        lib = load_library()
        v = lib.infr_gguf_meta_get(self._g._handle(), key.encode())
        o = C.c_double()
        return o.value if v and lib.infr_gguf_value_f64(v, C.byref(o)) else None

    def str(self, key: str) -> str | None:
        lib = load_library()
        v = lib.infr_gguf_meta_get(self._g._handle(), key.encode())
        return _value(lib, v) if v and lib.infr_gguf_value_kind(v) == STR else None


class Gguf:
    """A parsed, memory-mapped GGUF model: one file or a whole shard set (lib.rs:79-97)."""

    def __init__(self, handle: int):
        self._h = handle

    @classmethod
    def open(cls, path: str | os.PathLike) -> "Gguf":
        h = _vp()
        _check(load_library().infr_gguf_open(os.fspath(path).encode(), C.byref(h)))
        return cls(h.value)

    def _handle(self) -> int:
        if not self._h:
            raise InfrError(Status.Invalid, "the GGUF file is closed")
        return self._h

    def close(self) -> None:
        """Unmap the files. Arrays returned by ``tensor_bytes`` must not be used afterwards."""
        if self._h:
            load_library().infr_gguf_close(self._h)
        self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def metadata(self) -> Metadata:
        return Metadata(self)

    def tensors(self) -> list[TensorInfo]:
        lib, h = load_library(), self._handle()
        out, t = [], _GgufTensor()
        for i in range(lib.infr_gguf_n_tensors(h)):
            _check(lib.infr_gguf_tensor(h, i, C.byref(t)))
            out.append(TensorInfo(t.name.decode(), tuple(t.shape[: t.n_dims]), t.ggml_type, t.offset, t.nbytes))
        return out

    def tensor(self, name: str) -> TensorInfo:
        lib, h = load_library(), self._handle()
        i = lib.infr_gguf_find(h, name.encode())
        if i < 0:
            raise InfrError(Status.Loader, f"tensor not found: '{name}'")
        t = _GgufTensor()
        _check(lib.infr_gguf_tensor(h, i, C.byref(t)))
        return TensorInfo(t.name.decode(), tuple(t.shape[: t.n_dims]), t.ggml_type, t.offset, t.nbytes)

    def tensor_bytes(self, name: str) -> np.ndarray:
        """Read-only uint8 view of the tensor's bytes inside the mapping (no copy)."""
        p, n = _vp(), C.c_size_t()
        _check(load_library().infr_gguf_tensor_bytes(self._handle(), name.encode(), C.byref(p), C.byref(n)))
        if n.value == 0:
            return np.empty(0, np.uint8)
        a = np.ctypeslib.as_array((C.c_uint8 * n.value).from_address(p.value))
        a.flags.writeable = False
        return a

    def tensor_file_range(self, name: str) -> tuple[int, int]:
        off, n = C.c_uint64(), C.c_size_t()
        _check(load_library().infr_gguf_tensor_file_range(self._handle(), name.encode(), C.byref(off), C.byref(n)))
        return off.value, n.value

    def shards(self) -> list[tuple[str, int]]:
        lib, h = load_library(), self._handle()
        out = []
        for i in range(lib.infr_gguf_n_shards(h)):
            p, n = C.c_char_p(), C.c_uint64()
            _check(lib.infr_gguf_shard(h, i, C.byref(p), C.byref(n)))
            out.append((p.value.decode(), n.value))
        return out

    def chat_template(self) -> str | None:
        s = load_library().infr_gguf_chat_template(self._handle())
        return s.decode() if s is not None else None

    def upload(self, be: HipBackend, name: str) -> Buffer:
        """Allocate a weights buffer on ``be`` holding the tensor's raw blocks."""
        h = _vp()
        _check(load_library().infr_gguf_upload(self._handle(), name.encode(), be._h, C.byref(h)))
        return Buffer(be, h.value)

    def upload_concat(self, be: HipBackend, names: list[str]) -> tuple[Buffer, list[int]]:
        """Several same-typed tensors back to back in one buffer; returns it and the byte offsets."""
        arr = (C.c_char_p * len(names))(*[n.encode() for n in names])
        offs = (C.c_size_t * len(names))()
        h = _vp()
        _check(load_library().infr_gguf_upload_concat(self._handle(), arr, len(names), be._h, C.byref(h), offs))
        return Buffer(be, h.value), list(offs)


# ───────────────────────────── fixture writer ─────────────────────────────
# The reference only reads GGUF; its tests assemble small files byte by byte
# (crates/infr-gguf/src/lib.rs:1019-1077, 1601-1656). This writer does the same job for this
# package's tests and benchmarks: synthetic banks become a file the reader opens like a real one.

_VT_U8, _VT_I8, _VT_U16, _VT_I16, _VT_U32, _VT_I32, _VT_F32, _VT_BOOL, _VT_STR, _VT_ARR, _VT_U64, _VT_I64, \
    _VT_F64 = range(13)


def _gstr(s: str | bytes) -> bytes:
    raw = s.encode() if isinstance(s, str) else s
    return len(raw).to_bytes(8, "little") + raw


def _gvalue(v, vtype: int | None = None) -> tuple[int, bytes]:
    """(value type, encoded bytes). Python ints default to UINT32/INT32/UINT64 by range."""
    import struct
    if isinstance(v, tuple) and len(v) == 2 and vtype is None and isinstance(v[0], int) and not isinstance(v[1], tuple):
        return _gvalue(v[1], v[0])  # (explicit value type, value)
    if isinstance(v, bool):
        return _VT_BOOL, bytes([1 if v else 0])
    if isinstance(v, int):
        if vtype is None:
            vtype = _VT_I32 if -2**31 <= v < 0 else _VT_U32 if 0 <= v < 2**32 else _VT_U64 if v >= 0 else _VT_I64
        fmt = {_VT_U8: "<B", _VT_I8: "<b", _VT_U16: "<H", _VT_I16: "<h", _VT_U32: "<I", _VT_I32: "<i",
               _VT_U64: "<Q", _VT_I64: "<q"}[vtype]
        return vtype, struct.pack(fmt, v)
    if isinstance(v, float):
        vtype = _VT_F32 if vtype is None else vtype
        return vtype, struct.pack("<f" if vtype == _VT_F32 else "<d", v)
    if isinstance(v, (str, bytes)):
        return _VT_STR, _gstr(v)
    if isinstance(v, list):
        enc = [_gvalue(e) for e in v]
        et = enc[0][0] if enc else (_VT_U32 if vtype is None else vtype)
        if any(t != et for t, _ in enc):
            raise ValueError("GGUF arrays hold one element type")
        return _VT_ARR, et.to_bytes(4, "little") + len(enc).to_bytes(8, "little") + b"".join(b for _, b in enc)
    raise TypeError(f"cannot encode {type(v).__name__} as a GGUF value")


def _gguf_chunks(metadata: dict, tensors, version: int, alignment: int | None):
    md = dict(metadata)
    if alignment is not None:
        md["general.alignment"] = (_VT_U32, alignment)
    align = alignment or 32
    head = bytearray()
    head += (0x46554747).to_bytes(4, "little") + version.to_bytes(4, "little")
    head += len(tensors).to_bytes(8, "little") + len(md).to_bytes(8, "little")
    for k, v in md.items():
        t, b = _gvalue(v)
        head += _gstr(k) + t.to_bytes(4, "little") + b
    off = 0
    views = [memoryview(np.ascontiguousarray(d)).cast("B") if isinstance(d, np.ndarray) else memoryview(d)
             for _, _, _, d in tensors]
    for (name, shape, ggml_type, _), data in zip(tensors, views):
        head += _gstr(name) + len(shape).to_bytes(4, "little")
        for d in shape:
            head += int(d).to_bytes(8, "little")
        head += int(ggml_type).to_bytes(4, "little") + off.to_bytes(8, "little")
        off += -(-len(data) // align) * align
    head += bytes(-len(head) % align)
    yield bytes(head)
    for i, data in enumerate(views):
        yield data
        if len(data) % align and i + 1 < len(views):
            yield bytes(-len(data) % align)


def gguf_bytes(metadata: dict, tensors: list[tuple[str, tuple[int, ...], int, bytes]], *, version: int = 3,
               alignment: int | None = None) -> bytes:
    """Encode one GGUF file. ``tensors`` are (name, shape with shape[0] fastest, ggml type, raw bytes
    or a numpy array); data is laid out in order, each tensor but the last padded to the alignment (32 unless
    ``alignment`` is given, in which case ``general.alignment`` is written too)."""
    return b"".join(bytes(c) for c in _gguf_chunks(metadata, tensors, version, alignment))


def write_gguf(path: str | os.PathLike, metadata: dict,
               tensors: list[tuple[str, tuple[int, ...], int, bytes]], *, version: int = 3,
               alignment: int | None = None) -> None:
    """``gguf_bytes`` streamed to ``path`` tensor by tensor."""
    with open(path, "wb") as f:
        for c in _gguf_chunks(metadata, tensors, version, alignment):
            f.write(c)
