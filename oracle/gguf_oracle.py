"""TEST INFRASTRUCTURE ONLY: CPU restatement (plain Python + numpy) of the reference's GGUF container
reader and ternary tensor loader. Only tests may import it; the product never does.

  read_gguf      crates/tritium-format/src/gguf.rs:550-664 (values :297-355, sizes :407-455,
                 alignment :509-526, coercions :217-292)
  load_ternary   crates/tritium-nn/src/model/weights.rs:146-166 (payload), :177-333 (scales rule)

Pinned by: the reference's own GGUF file written by the official `gguf` Python writer
(crates/tritium-format/tests/fixtures/bitnet_tiny.gguf, expectations from tests/real_gguf.rs:12-51,
which were read back with gguf.GGUFReader), every case of gguf.rs:740-935 and of
weights.rs:392-442, and hand-written byte strings in tests/test_oracle_gguf.py.
The block decoders passed to load_ternary are the C oracle's, pinned elsewhere.
"""
import struct

import numpy as np

GGML_TYPE_TQ1_0, GGML_TYPE_TQ2_0, GGML_TYPE_I2_S, GGML_TYPE_Q2_0 = 34, 35, 36, 42
MAX_STRING_LEN = 64 * 1024 * 1024
MAX_COUNT = 1 << 32
MAX_METADATA_DEPTH = 8
MAX_METADATA_ARRAY_ELEMENTS = 16_000_000
MAX_DIMS = 8
U64_MAX = (1 << 64) - 1

BLOCK_LAYOUT = {0: (4, 1), 1: (2, 1), 8: (34, 32), 24: (1, 1), 25: (2, 1), 26: (4, 1), 30: (2, 1),
                GGML_TYPE_TQ1_0: (54, 256), GGML_TYPE_TQ2_0: (66, 256), GGML_TYPE_Q2_0: (18, 64)}


class GgufError(Exception):
    def __init__(self, kind, detail=None):
        super().__init__(kind if detail is None else f"{kind}({detail})")
        self.kind, self.detail = kind, detail


class Value:
    """One metadata value: `type` is the GGUF type id, `v` the Python value (list of Value for arrays)."""

    def __init__(self, type_, v, child=None):
        self.type, self.v, self.child = type_, v, child

    def as_u64(self):
        if self.type in (0, 2, 4, 10):
            return self.v
        if self.type in (1, 3, 5, 11) and self.v >= 0:
            return self.v
        return None

    def as_i64(self):
        if self.type in (0, 1, 2, 3, 4, 5, 11):
            return self.v
        if self.type == 10 and self.v < (1 << 63):
            return self.v
        return None

    def as_f64(self):
        return float(self.v) if self.type in (6, 12) else None

    def as_f32(self):
        return self.v if self.type == 6 else None

    def as_bool(self):
        return self.v if self.type == 7 else None

    def as_str(self):
        return self.v if self.type == 8 else None


class _Cursor:
    def __init__(self, buf):
        self.buf, self.pos = bytes(buf), 0

    def take(self, n):
        if self.pos + n > len(self.buf):
            raise GgufError("Truncated")
        out = self.buf[self.pos:self.pos + n]
        self.pos += n
        return out

    def num(self, fmt):
        return struct.unpack("<" + fmt, self.take(struct.calcsize(fmt)))[0]

    def string(self):
        n = self.num("Q")
        if n > MAX_STRING_LEN:
            raise GgufError("StringTooLong")
        raw = self.take(n)
        try:
            return raw.decode("utf-8", errors="strict")
        except UnicodeDecodeError:
            raise GgufError("InvalidUtf8") from None


_SCALARS = {0: "B", 1: "b", 2: "H", 3: "h", 4: "I", 5: "i", 10: "Q", 11: "q", 12: "d"}


def _read_value(cur, vt, depth, total):
    if vt in _SCALARS:
        return Value(vt, cur.num(_SCALARS[vt]))
    if vt == 6:  # keep the f32 as numpy's float32 so that comparisons are in single precision
        return Value(6, np.frombuffer(cur.take(4), "<f4")[0])
    if vt == 7:
        b = cur.num("B")
        if b > 1:
            raise GgufError("InvalidBoolean", b)
        return Value(7, b != 0)
    if vt == 8:
        return Value(8, cur.string())
    if vt == 9:
        if depth >= MAX_METADATA_DEPTH:
            raise GgufError("DimsOverflow")
        child = cur.num("I")
        if child > 12:
            raise GgufError("UnknownValueType", child)
        count = cur.num("Q")
        if count > MAX_COUNT:
            raise GgufError("DimsOverflow")
        total[0] += count
        if total[0] > MAX_METADATA_ARRAY_ELEMENTS:
            raise GgufError("DimsOverflow")
        return Value(9, [_read_value(cur, child, depth + 1, total) for _ in range(count)], child)
    raise GgufError("UnknownValueType", vt)


def _n_bytes(ggml_type, dims):
    if ggml_type not in BLOCK_LAYOUT:
        return 0
    bb, be = BLOCK_LAYOUT[ggml_type]
    row = dims[0] if dims else 1
    if row % be:
        raise GgufError("InvalidTensorShape")
    rows = 1
    for d in dims[1:]:
        rows *= d
        if rows > U64_MAX:
            raise GgufError("DimsOverflow")
    out = (row // be) * bb
    if out > U64_MAX or out * rows > U64_MAX:
        raise GgufError("DimsOverflow")
    return out * rows


class GgufFile:
    def __init__(self):
        self.version, self.metadata, self.tensors, self.tensor_data_offset, self.alignment = 0, {}, [], 0, 32

    def tensor(self, name):
        return next((t for t in self.tensors if t["name"] == name), None)


def read_gguf(buf):
    cur, f = _Cursor(buf), GgufFile()
    if cur.take(4) != b"GGUF":
        raise GgufError("BadMagic")
    f.version = cur.num("I")
    if f.version not in (2, 3):
        raise GgufError("UnsupportedVersion", f.version)
    n_tensors, n_kv = cur.num("Q"), cur.num("Q")
    if n_tensors > MAX_COUNT or n_kv > MAX_COUNT:
        raise GgufError("DimsOverflow")
    total = [0]
    for _ in range(n_kv):
        key = cur.string()
        f.metadata[key] = _read_value(cur, cur.num("I"), 0, total)
    al = f.metadata.get("general.alignment")
    if al is not None:
        if al.type != 4 or al.v == 0 or al.v % 8:
            raise GgufError("InvalidAlignment")
        f.alignment = al.v
    raw = []
    for _ in range(n_tensors):
        name = cur.string()
        nd = cur.num("I")
        if nd > MAX_DIMS:
            raise GgufError("DimsOverflow")
        dims = [cur.num("Q") for _ in range(nd)]
        raw.append((name, dims, cur.num("I"), cur.num("Q")))
    f.tensor_data_offset = (cur.pos + f.alignment - 1) // f.alignment * f.alignment
    data_len = max(0, len(cur.buf) - f.tensor_data_offset)
    for name, dims, ty, off in raw:
        n = 1
        for d in dims:
            n *= d
            if n > U64_MAX:
                raise GgufError("DimsOverflow")
        nbytes = _n_bytes(ty, dims)
        if nbytes > 0:
            if off + nbytes > U64_MAX:
                raise GgufError("DimsOverflow")
            if off + nbytes > data_len:
                raise GgufError("OffsetOutOfBounds")
        elif off > data_len:
            raise GgufError("OffsetOutOfBounds")
        f.tensors.append({"name": name, "dims": dims, "ggml_type": ty, "offset": off, "n_bytes": nbytes})
    return f


class LoadError(Exception):
    pass


def load_ternary(f, buf, name, unpack_row, unpack_i2s_tensor, f16_to_f32, f32_to_f16_to_f32):
    """-> (trits [n,k] int8, row scales [n] f32). The four callables are the pinned block decoders
    and half-precision conversions; unpack_row(row_bytes, k, ggml_type) -> (trits, f16 scale bits)."""
    info = f.tensor(name)
    if info is None:
        raise LoadError("missing tensor")
    if len(info["dims"]) != 2:
        raise LoadError("shape")
    k, n = info["dims"]
    ty = info["ggml_type"]
    start = f.tensor_data_offset + info["offset"]
    length = n * k // 4 + 32 if ty == GGML_TYPE_I2_S else info["n_bytes"]
    if start + length > len(buf):
        raise LoadError("payload out of bounds")
    p = bytes(buf[start:start + length])
    if ty == GGML_TYPE_I2_S:
        trits, scale = unpack_i2s_tensor(p, n * k)
        return np.asarray(trits, np.int8).reshape(n, k), np.full(n, scale, np.float32)
    if ty not in (GGML_TYPE_TQ1_0, GGML_TYPE_TQ2_0):
        raise LoadError("unsupported tensor type")
    bb = 54 if ty == GGML_TYPE_TQ1_0 else 66
    nb = -(-k // 256)
    rb = nb * bb
    trits = np.zeros((n, k), np.int8)
    rows, tensor_scale, uniform = [], None, True
    for r in range(n):
        t, hs = unpack_row(p[r * rb:(r + 1) * rb], k, ty)
        t = np.array(t, np.int8)
        row_scale = None
        for bi, h in enumerate(hs):
            dv = np.float32(f16_to_f32(h))
            if dv == 0:
                t[bi * 256:min((bi + 1) * 256, k)] = 0
            elif row_scale is None:
                row_scale = dv
            elif not row_scale == dv:
                raise LoadError("non-uniform block scales")
        trits[r] = t
        if row_scale is not None:
            if tensor_scale is None:
                tensor_scale = row_scale
            elif tensor_scale != row_scale:
                uniform = False
        rows.append(np.float32(0) if row_scale is None else row_scale)
    if not uniform:
        fill = tensor_scale if tensor_scale is not None else np.float32(0)
        return trits, np.array([fill if s == 0 else s for s in rows], np.float32)
    exact = f.metadata.get("tritium.i2s_scale." + name)
    exact = exact.as_f32() if exact is not None else None
    if exact is not None:
        if tensor_scale is not None and tensor_scale != np.float32(f32_to_f16_to_f32(exact)):
            raise LoadError("stale tritium.i2s_scale metadata")
        scale = exact
    else:
        scale = tensor_scale if tensor_scale is not None else np.float32(0)
    return trits, np.full(n, scale, np.float32)
