"""GGUF files through the library's reader (``lkh_gguf_*``), and a writer for test fixtures.

The reader is the C++ one (``csrc/host_gguf.hip``); this module only gives it Python names. The
writer follows the field order the reference's own tests write by hand
(src/tensor/quantized/gguf_file.rs:150-204, 959-1010): header, key/values, tensor directory with
dimensions innermost-first, zero padding to the alignment, tensor payloads each at an aligned
offset.
"""
from __future__ import annotations

import ctypes as C
import struct
from dataclasses import dataclass
from typing import Any

from . import lib

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_SCALAR = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B",
           U64: "<Q", I64: "<q", F64: "<d"}
# block type id -> (values per block, bytes per block), src/tensor/quantized/dtype.rs:66-96
BLOCKS = {0: (1, 4), 1: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 9: (32, 36),
          10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 15: (256, 292),
          30: (1, 2), 24: (1, 1), 39: (32, 17)}


class GgufError(RuntimeError):
    pass


# ----------------------------------------------------------------------------- writer
def _string(s: str) -> bytes:
    raw = s.encode()
    return struct.pack("<Q", len(raw)) + raw


def _value(vtype: int, v: Any) -> bytes:
    if vtype == STRING:
        return _string(v)
    if vtype == ARRAY:
        elem, items = v
        return struct.pack("<IQ", elem, len(items)) + b"".join(_value(elem, x) for x in items)
    return struct.pack(_SCALAR[vtype], v)


def write_bytes(kvs, tensors, version: int = 3, alignment: int | None = None, magic: bytes = b"GGUF") -> bytes:
    """kvs: [(key, type, value)] (ARRAY value = (elem type, items)); tensors: [(name, row-major dims,
    block type id, payload bytes)]. `alignment` adds the ``general.alignment`` key."""
    kvs = list(kvs)
    if alignment is not None:
        kvs.append(("general.alignment", U32, alignment))
    align = alignment or 32
    out = bytearray(magic + struct.pack("<IQQ", version, len(tensors), len(kvs)))
    for key, vtype, v in kvs:
        out += _string(key) + struct.pack("<I", vtype) + _value(vtype, v)
    offsets, at = [], 0
    for _, _, _, payload in tensors:
        offsets.append(at)
        at = -(-(at + len(payload)) // align) * align
    for (name, dims, dtype, _), off in zip(tensors, offsets):
        out += _string(name) + struct.pack("<I", len(dims))
        out += b"".join(struct.pack("<Q", d) for d in reversed(dims))
        out += struct.pack("<IQ", dtype, off)
    out += b"\0" * (-len(out) % align)
    for _, _, _, payload in tensors:
        out += payload + b"\0" * (-len(payload) % align)
    return bytes(out)


# ----------------------------------------------------------------------------- reader
@dataclass
class TensorInfo:
    index: int
    name: str
    dims: tuple
    dtype: int
    offset: int
    nbytes: int


@dataclass
class Facts:
    architecture: str | None
    file_type: int | None
    parameter_count: int | None
    pools: bool
    split_parts: int | None


class GgufFile:
    """A parsed GGUF header over a mapped file (``path``) or over bytes the object keeps alive."""

    def __init__(self, path: str | None = None, data: bytes | None = None):
        self._l = lib.load()
        err = C.create_string_buffer(512)
        self._keep = data
        if path is not None:
            self._h = self._l.lkh_gguf_open(str(path).encode(), err, len(err))
        else:
            self._buf = C.create_string_buffer(data, len(data))
            self._h = self._l.lkh_gguf_over(C.addressof(self._buf), len(data), err, len(err))
        if not self._h:
            raise GgufError(err.value.decode())
        v, ntens, nkv = C.c_int(), C.c_int(), C.c_int()
        a, off = C.c_uint64(), C.c_uint64()
        self._l.lkh_gguf_layout(self._h, C.byref(v), C.byref(a), C.byref(off), C.byref(ntens), C.byref(nkv))
        self.version, self.alignment, self.data_offset = v.value, a.value, off.value
        self.tensor_count, self.kv_count = ntens.value, nkv.value

    def close(self):
        if getattr(self, "_h", None):
            self._l.lkh_gguf_close(self._h)
            self._h = None

    __del__ = close

    # -- tensors
    def tensor(self, which) -> TensorInfo:
        index = which if isinstance(which, int) else self._l.lkh_gguf_find_tensor(self._h, which.encode())
        if index < 0:
            raise GgufError(f"gguf: no tensor `{which}`")
        name, dtype, nd = C.c_char_p(), C.c_int(), C.c_int()
        dims = (C.c_int64 * 8)()
        off, nbytes = C.c_uint64(), C.c_uint64()
        lib.check("lkh_gguf_tensor", self._l.lkh_gguf_tensor(self._h, index, C.byref(name), C.byref(dtype), C.byref(nd),
                                                             dims, 8, C.byref(off), C.byref(nbytes)))
        return TensorInfo(index, name.value.decode(), tuple(dims[: nd.value]), dtype.value, off.value, nbytes.value)

    def tensors(self):
        return [self.tensor(i) for i in range(self.tensor_count)]

    def tensor_bytes(self, which) -> bytes:
        t = self.tensor(which)
        p = self._l.lkh_gguf_tensor_data(self._h, t.index)
        if not p:
            raise GgufError(f"gguf: tensor `{t.name}` lies outside the file")
        return C.string_at(p, t.nbytes)

    # -- metadata
    def keys(self):
        out = []
        for i in range(self.kv_count):
            key = C.c_char_p()
            self._l.lkh_gguf_kv(self._h, i, C.byref(key), None, None, None)
            out.append(key.value.decode())
        return out

    def _scalar(self, vtype: int, getter_prefix: str, index: int, item=None):
        args = (self._h, index) if item is None else (self._h, index, item)
        if vtype == STRING:
            s, n = C.c_char_p(), C.c_uint64()
            lib.check(getter_prefix + "str", getattr(self._l, getter_prefix + "str")(*args, C.byref(s), C.byref(n)))
            return C.string_at(s, n.value).decode()
        if vtype in (F32, F64):
            d = C.c_double()
            lib.check(getter_prefix + "f64", getattr(self._l, getter_prefix + "f64")(*args, C.byref(d)))
            return d.value
        if vtype == BOOL and item is None:
            b = C.c_int()
            lib.check("lkh_gguf_kv_bool", self._l.lkh_gguf_kv_bool(self._h, index, C.byref(b)))
            return bool(b.value)
        if vtype in (U8, U16, U32, U64, BOOL):
            u = C.c_uint64()
            lib.check(getter_prefix + "u64", getattr(self._l, getter_prefix + "u64")(*args, C.byref(u)))
            return u.value
        i = C.c_int64()
        lib.check(getter_prefix + "i64", getattr(self._l, getter_prefix + "i64")(*args, C.byref(i)))
        return i.value

    def get(self, key: str, default=None):
        index = self._l.lkh_gguf_find_key(self._h, key.encode())
        if index < 0:
            return default
        vtype, elem, count = C.c_int(), C.c_int(), C.c_uint64()
        self._l.lkh_gguf_kv(self._h, index, None, C.byref(vtype), C.byref(elem), C.byref(count))
        if vtype.value == ARRAY:
            return [self._scalar(elem.value, "lkh_gguf_kv_item_", index, i) for i in range(count.value)]
        return self._scalar(vtype.value, "lkh_gguf_kv_", index)

    def kind(self, key: str):
        index = self._l.lkh_gguf_find_key(self._h, key.encode())
        if index < 0:
            return None
        vtype, elem = C.c_int(), C.c_int()
        self._l.lkh_gguf_kv(self._h, index, None, C.byref(vtype), C.byref(elem), None)
        return (vtype.value, elem.value) if vtype.value == ARRAY else vtype.value

    def as_u64(self, key: str):
        """The reference's ``to_u64``: any whole-number kind that fits, else None."""
        index = self._l.lkh_gguf_find_key(self._h, key.encode())
        u = C.c_uint64()
        return u.value if index >= 0 and self._l.lkh_gguf_kv_u64(self._h, index, C.byref(u)) == lib.LK_OK else None

    def as_i64(self, key: str):
        index = self._l.lkh_gguf_find_key(self._h, key.encode())
        i = C.c_int64()
        return i.value if index >= 0 and self._l.lkh_gguf_kv_i64(self._h, index, C.byref(i)) == lib.LK_OK else None

    def facts(self) -> Facts:
        arch = C.c_char_p()
        ft, pc, sp = C.c_int64(), C.c_int64(), C.c_int64()
        pools = C.c_int()
        lib.check("lkh_gguf_facts", self._l.lkh_gguf_facts(self._h, C.byref(arch), C.byref(ft), C.byref(pc),
                                                           C.byref(pools), C.byref(sp)))
        opt = lambda v: None if v.value < 0 else v.value
        return Facts(arch.value.decode() if arch.value is not None else None, opt(ft), opt(pc), bool(pools.value), opt(sp))

    # -- device
    def upload(self, which, device: int = 0, stream: int = 0):
        """-> (device pointer, allocation bytes); free with ``free_blob``."""
        t = self.tensor(which)
        n = C.c_uint64()
        p = self._l.lkh_gguf_upload(self._h, t.index, device, stream, C.byref(n))
        if not p:
            raise GgufError(f"gguf: upload of `{t.name}` failed")
        return p, n.value

    def linear(self, name: str, device: int = 0, stream: int = 0):
        """-> (QKernelMatMul handle, device blob): ``lkh_qkernel_matmul_*`` take the handle."""
        blob = C.c_void_p()
        err = C.create_string_buffer(512)
        h = self._l.lkh_gguf_linear(self._h, name.encode(), device, stream, C.byref(blob), err, len(err))
        if not h:
            raise GgufError(err.value.decode())
        return h, blob.value


def free_blob(ptr) -> None:
    lib.load().lkh_gguf_free_blob(ptr)
