"""Host mirror of the reference's GGUF reader and ternary tensor loader over the C ABI.

`read_gguf(buf)` answers like tritium_format::read_gguf (crates/tritium-format/src/gguf.rs:550-664):
a GgufFile with version, alignment, tensor_data_offset, the tensor table and metadata getters.
`GgufFile.load_ternary(buf, name)` is load_ternary of the model loader
(crates/tritium-nn/src/model/weights.rs:177-333) up to the backend call: packed rows, their format
and one scale per output row; `Mi355xBackend.upload_weights_gguf` finishes it on the device.
"""
import ctypes as C
import enum
from dataclasses import dataclass

import numpy as np

from . import _lib
from .backend import InvalidInput, TernaryFormat, _check

GGML_TYPE_TQ1_0, GGML_TYPE_TQ2_0, GGML_TYPE_I2_S, GGML_TYPE_Q2_0 = 34, 35, 36, 42
DEFAULT_ALIGNMENT = 32


class GgufErrorKind(enum.IntEnum):
    """GgufError's variants (crates/tritium-format/src/gguf.rs:63-96)."""
    Ok = 0
    BadMagic = 1
    UnsupportedVersion = 2
    Truncated = 3
    StringTooLong = 4
    DimsOverflow = 5
    InvalidTensorShape = 6
    InvalidAlignment = 7
    InvalidBoolean = 8
    OffsetOutOfBounds = 9
    UnknownValueType = 10
    InvalidUtf8 = 11


class GgufError(InvalidInput):
    def __init__(self, kind, detail, message):
        super().__init__(message)
        self.kind = GgufErrorKind(kind)
        self.detail = detail  # the value UnsupportedVersion / InvalidBoolean / UnknownValueType carry


@dataclass(frozen=True)
class TensorInfo:
    name: str
    dims: tuple
    ggml_type: int
    offset: int
    n_bytes: int

    def element_count(self):
        n = 1
        for d in self.dims:
            n *= d
        return n


def _bytes(buf):
    return np.ascontiguousarray(np.frombuffer(buf, dtype=np.uint8) if not isinstance(buf, np.ndarray) else buf,
                                dtype=np.uint8).reshape(-1)


class GgufFile:
    def __init__(self, handle):
        self._lib = _lib.load()
        self._h = handle

    def close(self):
        if self._h:
            self._lib.tk_gguf_close(self._h)
            self._h = None

    __del__ = close

    @property
    def version(self):
        return self._lib.tk_gguf_version(self._h)

    def alignment(self):
        return self._lib.tk_gguf_alignment(self._h)

    @property
    def tensor_data_offset(self):
        return self._lib.tk_gguf_tensor_data_offset(self._h)

    def _info(self, t):
        return TensorInfo(t.name.decode(), tuple(t.dims[i] for i in range(t.n_dims)), t.ggml_type, t.offset, t.n_bytes)

    @property
    def tensors(self):
        out, t = [], _lib.GgufTensor()
        for i in range(self._lib.tk_gguf_tensor_count(self._h)):
            self._lib.tk_gguf_tensor_at(self._h, i, C.byref(t))
            out.append(self._info(t))
        return out

    def _raw(self, name):
        t = _lib.GgufTensor()
        return t if self._lib.tk_gguf_tensor_find(self._h, name.encode(), C.byref(t)) else None

    def tensor(self, name):
        t = self._raw(name)
        return self._info(t) if t is not None else None

    def metadata_count(self):
        return self._lib.tk_gguf_metadata_count(self._h)

    def _get(self, fn, ctype, key, index):
        v = ctype()
        return v.value if fn(self._h, key.encode(), index, C.byref(v)) else None

    def as_u64(self, key, index=-1):
        return self._get(self._lib.tk_gguf_meta_u64, C.c_uint64, key, index)

    def as_i64(self, key, index=-1):
        return self._get(self._lib.tk_gguf_meta_i64, C.c_int64, key, index)

    def as_f64(self, key, index=-1):
        return self._get(self._lib.tk_gguf_meta_f64, C.c_double, key, index)

    def as_f32(self, key, index=-1):
        return self._get(self._lib.tk_gguf_meta_f32, C.c_float, key, index)

    def as_bool(self, key, index=-1):
        v = self._get(self._lib.tk_gguf_meta_bool, C.c_int, key, index)
        return None if v is None else bool(v)

    def as_str(self, key, index=-1):
        p, n = C.c_char_p(), C.c_size_t()
        if not self._lib.tk_gguf_meta_str(self._h, key.encode(), index, C.byref(p), C.byref(n)):
            return None
        return C.string_at(p, n.value).decode()

    def value_type(self, key, index=-1):
        """(value type id, child type id, array length) or None when the key is absent."""
        vt, ct, n = C.c_uint32(), C.c_uint32(), C.c_uint64()
        if not self._lib.tk_gguf_meta_type(self._h, key.encode(), index, C.byref(vt), C.byref(ct), C.byref(n)):
            return None
        return vt.value, ct.value, n.value

    def payload_span(self, file_len, name):
        """(absolute offset, length) of the tensor's payload in the file."""
        t = self._raw(name)
        if t is None:
            raise InvalidInput(f"missing tensor: {name}")
        off, n = C.c_uint64(), C.c_uint64()
        _check(self._lib.tk_gguf_tensor_payload(self._h, file_len, C.byref(t), C.byref(off), C.byref(n)))
        return off.value, n.value

    def ternary_shape(self, name):
        n, k, f = C.c_size_t(), C.c_size_t(), C.c_int()
        _check(self._lib.tk_gguf_ternary_shape(self._h, name.encode(), C.byref(n), C.byref(k), C.byref(f)))
        return n.value, k.value, TernaryFormat(f.value)

    def load_ternary(self, buf, name):
        """-> (packed rows, format, row scales [n] f32, n, k)"""
        b = _bytes(buf)
        n, k, fmt = self.ternary_shape(name)
        packed = np.zeros(self._lib.tk_packed_len(n, k, int(fmt)), np.uint8)
        scales = np.zeros(n, np.float32)
        _check(self._lib.tk_gguf_load_ternary(self._h, b.ctypes.data, b.size, name.encode(), packed.ctypes.data,
                                              packed.size, scales.ctypes.data, n))
        return packed, fmt, scales, n, k


def read_gguf(buf):
    b = _bytes(buf)
    lib = _lib.load()
    h, kind, detail = C.c_void_p(), C.c_int(), C.c_uint64()
    rc = lib.tk_gguf_open(b.ctypes.data if b.size else None, b.size, C.byref(h), C.byref(kind), C.byref(detail))
    if rc != 0:
        raise GgufError(kind.value, detail.value, lib.tk_last_error().decode())
    return GgufFile(h)
