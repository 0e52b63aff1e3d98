"""ctypes binding of the oracle's SALT part (oracle/salt_oracle.c): the sparse residual plane, the SALT row
sidecar (legacy v1, progressive v2), the SALT V2 codecs and exact matrix-vector product. Tests only."""
import ctypes as C

import numpy as np

import oracle_lib
from oracle_lib import _p, f32p, i8p, u8p, u16p

u32p = C.POINTER(C.c_uint32)
sz = C.c_size_t
szp = C.POINTER(sz)

(BAD_MAGIC, UNSUPPORTED_VERSION, WRONG_LEN, INVALID_PLANE_TAG, SPARSE_BASE_PLANE, OUT_OF_RANGE, NONCANONICAL_INDICES,
 ROW_TOO_LONG, NONZERO_PADDING, INVALID_DENSITY, TOO_MANY_PLANES) = range(20, 31)
(V2_WRONG_PACKED_LENGTH, V2_INVALID_D2_CODE, V2_INVALID_B3_CODE, V2_NONCANONICAL_TRIT_PADDING,
 V2_S34_NOT_MULTIPLE_OF_FOUR, V2_S34_ZERO_COUNT, V2_NONCANONICAL_BIT_PADDING, V2_NONFINITE_ACTIVATION,
 V2_NONFINITE_OUTPUT) = range(40, 49)
D2, B3, S34 = 0, 1, 2


class SaltOracle:
    def __init__(self, lib):
        self.lib = L = lib
        L.to_sparse_plane_packed_len.restype = sz
        L.to_sparse_plane_packed_len.argtypes = [sz, sz]
        L.to_sparse_from_tq2_0.argtypes = [u8p, sz, sz, u16p, u32p, i8p, szp]
        L.to_sparse_to_tq2_0.argtypes = [sz, u16p, sz, u32p, i8p, sz, u8p, sz]
        L.to_pack_sparse_plane.argtypes = [sz, u16p, sz, u32p, i8p, sz, u8p, sz]
        L.to_unpack_sparse_plane.argtypes = [u8p, sz, szp, u16p, sz, u32p, i8p, sz, szp]
        pp = C.POINTER(C.c_void_p)
        L.to_pack_salt_row.argtypes = [sz, pp, sz, u8p, sz, szp]
        L.to_pack_progressive_salt_row.argtypes = [sz, pp, sz, C.c_float, u8p, sz, szp]
        L.to_packed_salt_row_len.argtypes = [u8p, sz, szp]
        L.to_unpack_salt_row_prefix.argtypes = [u8p, sz, sz, szp, szp, u8p, sz]
        L.to_salt_v2_payload_bytes.argtypes = [C.c_int, sz, szp]
        L.to_salt_v2_pack.argtypes = [C.c_int, i8p, sz, u8p, sz]
        L.to_salt_v2_unpack.argtypes = [C.c_int, u8p, sz, sz, i8p]
        L.to_salt_v2_forward.argtypes = [C.c_int, sz, u8p, sz, u16p, sz, u8p, sz, sz, sz, f32p, sz, f32p]
        L.to_salt_v2_coefficient.argtypes = [C.c_int, sz, u8p, sz, u16p, sz, u8p, sz, sz, sz, sz, f32p]

    @staticmethod
    def _nb(k):
        return (k + 255) // 256

    # ---- sparse plane ----
    def sparse_from_tq2_0(self, packed, k):
        packed = np.ascontiguousarray(packed, np.uint8)
        scales = np.zeros(max(self._nb(k), 1), np.uint16)
        idx, sign, nnz = np.zeros(max(k, 1), np.uint32), np.zeros(max(k, 1), np.int8), sz(0)
        rc = self.lib.to_sparse_from_tq2_0(_p(packed, u8p), packed.size, k, _p(scales, u16p), _p(idx, u32p), _p(sign, i8p),
                                           C.byref(nnz))
        return rc, scales[: self._nb(k)], idx[: nnz.value].copy(), sign[: nnz.value].copy()

    def pack_sparse_plane(self, k, scales, idx, sign):
        scales, idx, sign = (np.ascontiguousarray(scales, np.uint16), np.ascontiguousarray(idx, np.uint32),
                             np.ascontiguousarray(sign, np.int8))
        out = np.zeros(self.lib.to_sparse_plane_packed_len(k, idx.size), np.uint8)
        rc = self.lib.to_pack_sparse_plane(k, _p(scales, u16p), scales.size, _p(idx, u32p), _p(sign, i8p), idx.size,
                                           _p(out, u8p), out.size)
        return rc, out

    def unpack_sparse_plane(self, data):
        data = np.ascontiguousarray(data, np.uint8)
        cap = max(data.size // 4, 1)
        k, nnz = sz(0), sz(0)
        scales, idx, sign = np.zeros(cap + 1, np.uint16), np.zeros(cap, np.uint32), np.zeros(cap, np.int8)
        rc = self.lib.to_unpack_sparse_plane(_p(data, u8p), data.size, C.byref(k), _p(scales, u16p), scales.size,
                                             _p(idx, u32p), _p(sign, i8p), cap, C.byref(nnz))
        return rc, k.value, scales[: self._nb(k.value)].copy(), idx[: nnz.value].copy(), sign[: nnz.value].copy()

    def sparse_to_tq2_0(self, k, scales, idx, sign):
        scales, idx, sign = (np.ascontiguousarray(scales, np.uint16), np.ascontiguousarray(idx, np.uint32),
                             np.ascontiguousarray(sign, np.int8))
        out = np.zeros(self._nb(k) * 66, np.uint8)
        rc = self.lib.to_sparse_to_tq2_0(k, _p(scales, u16p), scales.size, _p(idx, u32p), _p(sign, i8p), idx.size,
                                         _p(out, u8p), out.size)
        return rc, out

    # ---- SALT rows ----
    @staticmethod
    def _planes(planes):
        bs = [np.ascontiguousarray(p, np.uint8) for p in planes]
        arr = (C.c_void_p * max(len(bs), 1))(*[b.ctypes.data for b in bs])
        return bs, arr

    def pack_salt_row(self, k, planes):
        bs, arr = self._planes(planes)
        out, n = np.zeros(10 + len(bs) * self._nb(k) * 66 + 16, np.uint8), sz(0)
        rc = self.lib.to_pack_salt_row(k, arr, len(bs), _p(out, u8p), out.size, C.byref(n))
        return rc, out[: n.value].copy()

    def pack_progressive_salt_row(self, k, planes, max_density=0.10):
        bs, arr = self._planes(planes)
        out, n = np.zeros(10 + len(bs) * (5 + self._nb(k) * 66) + 16, np.uint8), sz(0)
        rc = self.lib.to_pack_progressive_salt_row(k, arr, len(bs), max_density, _p(out, u8p), out.size, C.byref(n))
        return rc, out[: n.value].copy()

    def packed_salt_row_len(self, data):
        data = np.ascontiguousarray(data, np.uint8)
        n = sz(0)
        rc = self.lib.to_packed_salt_row_len(_p(data, u8p), data.size, C.byref(n))
        return rc, n.value

    def unpack_salt_row(self, data, max_planes=1 << 30):
        """(rc, k, [dense TQ2_0 plane rows])"""
        data = np.ascontiguousarray(data, np.uint8)
        k, t = sz(0), sz(0)
        out = np.zeros(max(data.size, 1) * 0 + 256 * 70 * 8 + data.size * 40, np.uint8)
        rc = self.lib.to_unpack_salt_row_prefix(_p(data, u8p), data.size, max_planes, C.byref(k), C.byref(t), _p(out, u8p), out.size)
        pb = self._nb(k.value) * 66
        return rc, k.value, [out[i * pb:(i + 1) * pb].copy() for i in range(t.value)]

    # ---- SALT V2 ----
    def v2_payload_bytes(self, codec, trits):
        n = sz(0)
        rc = self.lib.to_salt_v2_payload_bytes(codec, trits, C.byref(n))
        return rc, n.value

    def v2_pack(self, codec, trits):
        trits = np.ascontiguousarray(trits, np.int8)
        rc, need = self.v2_payload_bytes(codec, trits.size)
        if rc:
            return rc, None
        out = np.zeros(max(need, 1), np.uint8)
        rc = self.lib.to_salt_v2_pack(codec, _p(trits, i8p), trits.size, _p(out, u8p), need)
        return rc, out[:need]

    def v2_unpack(self, codec, packed, n):
        packed = np.ascontiguousarray(packed, np.uint8)
        out = np.zeros(max(n, 1), np.int8)
        rc = self.lib.to_salt_v2_unpack(codec, _p(packed, u8p), packed.size, n, _p(out, i8p))
        return rc, out[:n]

    def v2_forward(self, t, act, m):
        act = np.ascontiguousarray(act, np.float32)
        out = np.full(max(m * t.n, 1), np.float32(19.0))
        rc = self.lib.to_salt_v2_forward(t.codec, t.scale_group, _p(t.payload, u8p), t.payload.size, _p(t.scales, u16p),
                                         t.scales.size, _p(t.plane_counts, u8p), t.plane_counts.size, t.n, t.k,
                                         _p(act, f32p), m, _p(out, f32p))
        return rc, out[: m * t.n].reshape(m, t.n)

    def v2_coefficient(self, t, index):
        v = C.c_float(0)
        rc = self.lib.to_salt_v2_coefficient(t.codec, t.scale_group, _p(t.payload, u8p), t.payload.size, _p(t.scales, u16p),
                                             t.scales.size, _p(t.plane_counts, u8p), t.plane_counts.size, t.n, t.k, index,
                                             C.byref(v))
        return rc, np.float32(v.value)


class V2Tensor:
    """A SALT V2 matrix in the runtime form the reference's device code takes (crates/tritium-cuda/kernels/
    salt_v2.cu:114-131): concatenated codec payloads and f16 scales, tile after tile, and per-tile plane counts.
    Built from per-tile trit planes with the ORACLE's packer."""

    def __init__(self, so, codec, scale_group, n, k, tiles):
        """tiles: list of (trits [planes, len] int8, scales [planes, groups] uint16 f16 bits)"""
        self.codec, self.scale_group, self.n, self.k = codec, scale_group, n, k
        payload, scales, counts = [], [], []
        for trits, sc in tiles:
            counts.append(trits.shape[0])
            for j in range(trits.shape[0]):
                rc, b = so.v2_pack(codec, trits[j])
                assert rc == 0, rc
                payload.append(b)
                scales.append(np.ascontiguousarray(sc[j], np.uint16))
        self.payload = np.ascontiguousarray(np.concatenate(payload) if payload else np.zeros(0, np.uint8))
        self.scales = np.ascontiguousarray(np.concatenate(scales) if scales else np.zeros(0, np.uint16))
        self.plane_counts = np.array(counts, np.uint8)
        self.tiles = tiles

    def dense(self):
        """float64 weights [n,k]: sum over planes of trit * scale (independent of the kernels' order)."""
        w = np.zeros(self.n * self.k, np.float64)
        for ti, (trits, sc) in enumerate(self.tiles):
            ln = trits.shape[1]
            s = sc.view(np.float16).astype(np.float64)
            grp = np.arange(ln) // self.scale_group
            for j in range(trits.shape[0]):
                w[ti * 256: ti * 256 + ln] += trits[j].astype(np.float64) * s[j][grp]
        return w.reshape(self.n, self.k)


def random_v2_tensor(so, rng, codec, n, k, plane_counts=None, scale_group=128):
    total = n * k
    ntiles = (total + 255) // 256
    if plane_counts is None:
        plane_counts = rng.integers(1, 4, ntiles)
    tiles = []
    for ti in range(ntiles):
        ln = min(256, total - ti * 256)
        p = int(plane_counts[ti])
        if codec == S34:
            assert ln % 4 == 0
            trits = np.zeros((p, ln), np.int8)
            for j in range(p):
                g = rng.choice([-1, 1], (ln // 4, 4)).astype(np.int8)
                g[np.arange(ln // 4), rng.integers(0, 4, ln // 4)] = 0
                trits[j] = g.reshape(-1)
        else:
            trits = rng.choice([-1, 0, 1], (p, ln), p=[0.3, 0.4, 0.3]).astype(np.int8)
        groups = (ln + scale_group - 1) // scale_group
        sc = rng.uniform(0.01, 2.0, (p, groups)).astype(np.float16).view(np.uint16)
        tiles.append((trits, sc))
    return V2Tensor(so, codec, scale_group, n, k, tiles)


def load():
    return SaltOracle(oracle_lib.load().lib)
