"""ctypes binding of the CPU oracle (oracle/libtritium_oracle.so). Tests only.

The oracle is the checker: nothing under tritium_amd/ imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
SO = os.path.join(ORACLE_DIR, "libtritium_oracle.so")

FMT_TQ1_0, FMT_TQ2_0 = 1, 2
OK, ERR_SHAPE, ERR_FORMAT, ERR_INVALID, ERR_BACKEND = 0, 1, 2, 4, 5
F16_ONE = 0x3C00

u8p = C.POINTER(C.c_uint8)
i8p = C.POINTER(C.c_int8)
f32p = C.POINTER(C.c_float)
u16p = C.POINTER(C.c_uint16)
i32p = C.POINTER(C.c_int32)


class Vector(C.Structure):
    _fields_ = [("id", C.c_char * 40), ("m", C.c_size_t), ("n", C.c_size_t), ("k", C.c_size_t),
                ("format", C.c_int), ("activation", f32p), ("weights", i8p), ("scales", f32p),
                ("expected", f32p)]


class VectorSet(C.Structure):
    _fields_ = [("count", C.c_size_t), ("v", C.POINTER(Vector))]


def _p(a, t):
    return a.ctypes.data_as(t)


class Oracle:
    def __init__(self, lib):
        self.lib = lib
        L = lib
        L.to_num_blocks.restype = C.c_size_t
        L.to_num_blocks.argtypes = [C.c_size_t]
        L.to_row_bytes.restype = C.c_size_t
        L.to_row_bytes.argtypes = [C.c_size_t, C.c_int]
        L.to_generate_vectors.restype = C.POINTER(VectorSet)
        L.to_generate_vectors.argtypes = [C.c_uint64, C.c_size_t]
        L.to_free_vectors.argtypes = [C.POINTER(VectorSet)]
        L.to_xorshift64_next.restype = C.c_uint64
        L.to_xorshift64_next.argtypes = [C.POINTER(C.c_uint64)]
        L.to_f32_to_bf16.restype = C.c_uint16
        L.to_f32_to_bf16.argtypes = [C.c_float]
        L.to_bf16_to_f32.restype = C.c_float
        L.to_bf16_to_f32.argtypes = [C.c_uint16]
        L.to_accepts_with_floor.argtypes = [C.c_float, C.c_float, C.c_float, C.c_int, C.c_float]
        sz = C.c_size_t
        L.to_pack_row.argtypes = [i8p, sz, u16p, sz, C.c_int, u8p, sz]
        L.to_unpack_row.argtypes = [u8p, sz, C.c_int, i8p, sz, u16p, sz]
        L.to_pack_matrix.argtypes = [i8p, sz, sz, C.c_int, u8p, sz]
        L.to_reference_mpgemm.argtypes = [f32p, sz, i8p, sz, f32p, sz, sz, sz, sz, f32p, sz]
        L.to_quantize_act_int8.argtypes = [f32p, sz, sz, f32p, f32p]
        L.to_quantize_act_int8.restype = None
        L.to_unpack_i2s_block.argtypes = [u8p, sz, i8p, sz]
        L.to_unpack_i2s_tensor.argtypes = [u8p, sz, sz, i8p, sz, f32p]
        L.to_convert_i2s_to_tq2_0.argtypes = [u8p, sz, sz, sz, u8p, sz, f32p]
        L.to_f16_to_f32.argtypes = [C.c_uint16]
        L.to_f16_to_f32.restype = C.c_float
        L.to_salt_dequant_row.argtypes = [C.POINTER(C.c_void_p), sz, sz, f32p]
        L.to_salt_mpgemm.argtypes = [C.POINTER(C.c_void_p), sz, sz, sz, f32p, sz, f32p]
        L.to_sum_squares_canonical.argtypes = [f32p, sz]
        L.to_sum_squares_canonical.restype = C.c_float
        L.to_rmsnorm.argtypes = [f32p, f32p, sz, C.c_float, C.c_int, f32p]
        L.to_rmsnorm.restype = None
        L.to_rmsnorm_quant.argtypes = [f32p, f32p, sz, sz, C.c_float, C.c_int, f32p, f32p]
        L.to_rmsnorm_quant.restype = None
        L.to_cpu_upload_check.argtypes = [u8p, sz, sz, sz, C.c_int, C.POINTER(C.c_long)]
        L.to_cpu_mpgemm.argtypes = [u8p, sz, C.c_int, f32p, sz, f32p, sz, sz, sz, sz, f32p, sz]
        L.to_cpu_mpgemm_with_act_quant.argtypes = L.to_cpu_mpgemm.argtypes
        L.to_int8_accumulators.argtypes = [u8p, sz, C.c_int, i8p, sz, sz, sz, i32p]
        pp = C.POINTER(C.c_void_p)
        L.to_cpu_mpgemm_planes.argtypes = [pp, C.POINTER(sz), C.c_int, pp, sz, f32p, sz, sz, sz, f32p]
        L.to_cpu_linear_a8_planes.argtypes = L.to_cpu_mpgemm_planes.argtypes
        L.to_cpu_projected_vjp.argtypes = [u8p, sz, C.c_int, f32p, sz, f32p, sz, f32p, sz, sz, sz, sz, f32p, sz, f32p, sz,
                                           f32p, sz]
        L.to_cpu_mpgemm_fast.argtypes = [u8p, sz, C.c_int, f32p, f32p, sz, sz, sz, f32p, C.c_int,
                                         C.POINTER(C.c_int), C.POINTER(C.c_int)]
        u32p = C.POINTER(C.c_uint32)
        L.to_compute_zero_bitmap.argtypes = [u8p, sz, sz, u32p, sz]
        L.to_compute_zero_bitmaps.argtypes = [u8p, sz, sz, sz, sz, u32p, sz]
        for name in ("to_pack_tq2_0_block", "to_pack_tq1_0_block"):
            getattr(L, name).argtypes = [i8p, C.c_uint16, u8p]
        for name in ("to_unpack_tq2_0_block", "to_unpack_tq1_0_block"):
            getattr(L, name).argtypes = [u8p, i8p, u16p]

    # ---- format ----
    def num_blocks(self, k):
        return self.lib.to_num_blocks(k)

    def row_bytes(self, k, fmt):
        return self.lib.to_row_bytes(k, fmt)

    def pack_block(self, trits, fmt, scale=F16_ONE):
        t = np.ascontiguousarray(trits, dtype=np.int8)
        assert t.size == 256
        out = np.zeros(66 if fmt == FMT_TQ2_0 else 54, dtype=np.uint8)
        fn = self.lib.to_pack_tq2_0_block if fmt == FMT_TQ2_0 else self.lib.to_pack_tq1_0_block
        assert fn(_p(t, i8p), scale, _p(out, u8p)) == 0
        return out

    def unpack_block(self, block, fmt):
        b = np.ascontiguousarray(block, dtype=np.uint8)
        t = np.zeros(256, dtype=np.int8)
        s = C.c_uint16(0)
        fn = self.lib.to_unpack_tq2_0_block if fmt == FMT_TQ2_0 else self.lib.to_unpack_tq1_0_block
        rc = fn(_p(b, u8p), _p(t, i8p), C.byref(s))
        return rc, t, s.value

    def pack_row(self, trits, fmt, scales=None):
        t = np.ascontiguousarray(trits, dtype=np.int8)
        k = t.size
        nb = self.num_blocks(k)
        sc = np.full(nb, F16_ONE, dtype=np.uint16) if scales is None else np.ascontiguousarray(scales, np.uint16)
        out = np.zeros(self.row_bytes(k, fmt), dtype=np.uint8)
        rc = self.lib.to_pack_row(_p(t, i8p), k, _p(sc, u16p), sc.size, fmt, _p(out, u8p), out.size)
        return rc, out

    def unpack_row(self, packed, k, fmt):
        b = np.ascontiguousarray(packed, dtype=np.uint8)
        nb = self.num_blocks(k)
        t = np.zeros(k, dtype=np.int8)
        sc = np.zeros(max(nb, 1), dtype=np.uint16)
        rc = self.lib.to_unpack_row(_p(b, u8p), b.size, fmt, _p(t, i8p), k, _p(sc, u16p), nb)
        return rc, t, sc[:nb]

    def pack_matrix(self, trits, n, k, fmt):
        t = np.ascontiguousarray(trits, dtype=np.int8).reshape(-1)
        assert t.size == n * k
        out = np.zeros(n * self.row_bytes(k, fmt), dtype=np.uint8)
        rc = self.lib.to_pack_matrix(_p(t, i8p), n, k, fmt, _p(out, u8p), out.size)
        assert rc == 0, rc
        return out

    # ---- compute ----
    def reference_mpgemm(self, act, trits, scales, m, n, k):
        a = np.ascontiguousarray(act, np.float32).reshape(-1)
        w = np.ascontiguousarray(trits, np.int8).reshape(-1)
        s = np.ascontiguousarray(scales, np.float32).reshape(-1)
        out = np.zeros(m * n, np.float32)
        rc = self.lib.to_reference_mpgemm(_p(a, f32p), a.size, _p(w, i8p), w.size, _p(s, f32p), s.size,
                                          m, n, k, _p(out, f32p), out.size)
        return rc, out.reshape(m, n)

    def quantize_act_int8(self, act, m, k):
        a = np.ascontiguousarray(act, np.float32).reshape(-1)
        assert a.size == m * k
        q = np.zeros(m * k, np.float32)
        s = np.zeros(m, np.float32)
        self.lib.to_quantize_act_int8(_p(a, f32p), m, k, _p(q, f32p), _p(s, f32p))
        return q.reshape(m, k), s

    def unpack_i2s_block(self, block, trits_len=128):
        b = np.ascontiguousarray(block, np.uint8).reshape(-1)
        t = np.zeros(trits_len, np.int8)
        rc = self.lib.to_unpack_i2s_block(_p(b, u8p), b.size, _p(t, i8p), t.size)
        return rc, t

    def unpack_i2s_tensor(self, payload, n_elements, trits_len=None):
        b = np.ascontiguousarray(payload, np.uint8).reshape(-1)
        t = np.zeros(n_elements if trits_len is None else trits_len, np.int8)
        s = np.zeros(1, np.float32)
        rc = self.lib.to_unpack_i2s_tensor(_p(b, u8p), b.size, n_elements, _p(t, i8p), t.size, _p(s, f32p))
        return rc, t, s[0]

    def convert_i2s_to_tq2_0(self, payload, n, k):
        b = np.ascontiguousarray(payload, np.uint8).reshape(-1)
        out = np.zeros(n * self.row_bytes(k, FMT_TQ2_0), np.uint8)
        s = np.zeros(1, np.float32)
        rc = self.lib.to_convert_i2s_to_tq2_0(_p(b, u8p), b.size, n, k, _p(out, u8p), out.size, _p(s, f32p))
        return rc, out, s[0]

    def f16_to_f32(self, h):
        return np.float32(self.lib.to_f16_to_f32(int(h)))

    def salt_dequant_row(self, plane_rows, k):
        """plane_rows: list of T packed TQ2_0 rows (one per plane) of one output channel."""
        bs = [np.ascontiguousarray(b, np.uint8) for b in plane_rows]
        pa = (C.c_void_p * len(bs))(*[b.ctypes.data for b in bs])
        out = np.zeros(k, np.float32)
        rc = self.lib.to_salt_dequant_row(pa, len(bs), k, _p(out, f32p))
        return rc, out

    def salt_mpgemm(self, planes, n, k, act, m):
        """planes: list of T arrays, each the n packed TQ2_0 rows (with block scales) of one plane."""
        bs = [np.ascontiguousarray(b, np.uint8) for b in planes]
        pa = (C.c_void_p * len(bs))(*[b.ctypes.data for b in bs])
        a = np.ascontiguousarray(act, np.float32).reshape(-1)
        assert a.size == m * k
        out = np.zeros(m * n, np.float32)
        rc = self.lib.to_salt_mpgemm(pa, len(bs), n, k, _p(a, f32p), m, _p(out, f32p))
        return rc, out.reshape(m, n)

    def pack_matrix_scaled(self, trits, block_scales_f16, n, k, fmt=FMT_TQ2_0):
        """Rows packed with the given f16 block scales (uint16 bit patterns [n, nb])."""
        t = np.ascontiguousarray(trits, np.int8).reshape(n, k)
        sc = np.ascontiguousarray(block_scales_f16, np.uint16).reshape(n, -1)
        rows = [self.pack_row(t[r], fmt, sc[r]) for r in range(n)]
        assert all(rc == 0 for rc, _ in rows)
        return np.concatenate([b for _, b in rows])

    def sum_squares_canonical(self, x):
        a = np.ascontiguousarray(x, np.float32).reshape(-1)
        return np.float32(self.lib.to_sum_squares_canonical(_p(a, f32p), a.size))

    def rmsnorm(self, x, w, eps, zero_centered=False):
        a = np.ascontiguousarray(x, np.float32).reshape(-1)
        ww = np.ascontiguousarray(w, np.float32).reshape(-1)
        assert a.size == ww.size
        out = np.zeros(a.size, np.float32)
        self.lib.to_rmsnorm(_p(a, f32p), _p(ww, f32p), a.size, eps, int(zero_centered), _p(out, f32p))
        return out

    def rmsnorm_quant(self, x, w, m, k, eps, zero_centered=False):
        a = np.ascontiguousarray(x, np.float32).reshape(-1)
        ww = np.ascontiguousarray(w, np.float32).reshape(-1)
        assert a.size == m * k and ww.size == k
        q = np.zeros(m * k, np.float32)
        s = np.zeros(m, np.float32)
        self.lib.to_rmsnorm_quant(_p(a, f32p), _p(ww, f32p), m, k, eps, int(zero_centered), _p(q, f32p), _p(s, f32p))
        return q.reshape(m, k), s

    def compute_zero_bitmap(self, packed_row, k):
        b = np.ascontiguousarray(packed_row, np.uint8).reshape(-1)
        nb = (k + 255) // 256
        words = np.zeros((nb + 31) // 32, np.uint32)
        rc = self.lib.to_compute_zero_bitmap(_p(b, u8p), b.size, k, words.ctypes.data_as(C.POINTER(C.c_uint32)), words.size)
        return rc, words

    def compute_zero_bitmaps(self, packed, n, k, row_bytes, words_len=None):
        b = np.ascontiguousarray(packed, np.uint8).reshape(-1)
        nb = (k + 255) // 256
        if words_len is None:
            words_len = n * ((nb + 31) // 32)
        words = np.zeros(max(words_len, 1), np.uint32)
        rc = self.lib.to_compute_zero_bitmaps(_p(b, u8p), b.size, n, k, row_bytes,
                                              words.ctypes.data_as(C.POINTER(C.c_uint32)), words_len)
        return rc, words[:words_len]

    def upload_check(self, packed, n, k, fmt):
        b = np.ascontiguousarray(packed, np.uint8)
        bad = C.c_long(-2)
        rc = self.lib.to_cpu_upload_check(_p(b, u8p), b.size, n, k, fmt, C.byref(bad))
        return rc, bad.value

    def _mp(self, fn, packed, fmt, act, scales, m, n, k, out_len=None):
        b = np.ascontiguousarray(packed, np.uint8)
        a = np.ascontiguousarray(act, np.float32).reshape(-1)
        s = np.ascontiguousarray(scales, np.float32).reshape(-1)
        out = np.zeros(m * n if out_len is None else out_len, np.float32)
        rc = fn(_p(b, u8p), b.size, fmt, _p(a, f32p), a.size, _p(s, f32p), s.size, m, n, k,
                _p(out, f32p), out.size)
        return rc, (out.reshape(m, n) if out_len is None else out)

    def cpu_mpgemm(self, packed, fmt, act, scales, m, n, k, out_len=None):
        return self._mp(self.lib.to_cpu_mpgemm, packed, fmt, act, scales, m, n, k, out_len)

    def cpu_mpgemm_with_act_quant(self, packed, fmt, act, scales, m, n, k, out_len=None):
        return self._mp(self.lib.to_cpu_mpgemm_with_act_quant, packed, fmt, act, scales, m, n, k, out_len)

    def int8_accumulators(self, packed, fmt, q, m, n, k):
        b = np.ascontiguousarray(packed, np.uint8)
        qq = np.ascontiguousarray(q, np.int8).reshape(-1)
        assert qq.size == m * k
        acc = np.zeros(m * n, np.int32)
        rc = self.lib.to_int8_accumulators(_p(b, u8p), b.size, fmt, _p(qq, i8p), m, n, k, _p(acc, i32p))
        assert rc == 0, rc
        return acc.reshape(m, n)

    def _planes(self, fn, packed_list, fmt, scales_list, act, m, n, k):
        P = len(packed_list)
        bs = [np.ascontiguousarray(b, np.uint8) for b in packed_list]
        ss = [np.ascontiguousarray(s, np.float32) for s in scales_list]
        pa = (C.c_void_p * P)(*[b.ctypes.data for b in bs])
        la = (C.c_size_t * P)(*[b.size for b in bs])
        sa = (C.c_void_p * P)(*[s.ctypes.data for s in ss])
        a = np.ascontiguousarray(act, np.float32).reshape(-1)
        assert a.size == m * k
        out = np.zeros(m * n, np.float32)
        rc = fn(pa, la, fmt, sa, P, _p(a, f32p), m, n, k, _p(out, f32p))
        assert rc == 0, rc
        return out.reshape(m, n)

    def cpu_mpgemm_planes(self, packed_list, fmt, scales_list, act, m, n, k):
        return self._planes(self.lib.to_cpu_mpgemm_planes, packed_list, fmt, scales_list, act, m, n, k)

    def cpu_linear_a8_planes(self, packed_list, fmt, scales_list, act, m, n, k):
        return self._planes(self.lib.to_cpu_linear_a8_planes, packed_list, fmt, scales_list, act, m, n, k)

    def cpu_projected_vjp(self, packed, fmt, act, scales, grad_output, m, n, k, bias=True, lens=None):
        """(rc, grad_act [m,k], grad_w [n,k], grad_bias [n] or None); outputs start as NaN so that an
        early error return is seen to have written nothing. `lens` overrides the output lengths
        (grad_act, grad_w, grad_bias) to provoke the shape errors."""
        b = np.ascontiguousarray(packed, np.uint8)
        a = np.ascontiguousarray(act, np.float32).reshape(-1)
        s = np.ascontiguousarray(scales, np.float32).reshape(-1)
        gy = np.ascontiguousarray(grad_output, np.float32).reshape(-1)
        la, lw, lb = lens or (m * k, n * k, n)
        ga, gw, gb = (np.full(max(x, 1), np.nan, np.float32) for x in (la, lw, lb))
        rc = self.lib.to_cpu_projected_vjp(_p(b, u8p), b.size, fmt, _p(a, f32p), a.size, _p(s, f32p), s.size,
                                           _p(gy, f32p), gy.size, m, n, k, _p(ga, f32p), la, _p(gw, f32p), lw,
                                           _p(gb, f32p) if bias else None, lb if bias else 0)
        return rc, ga[:la].reshape(m, k) if la == m * k else ga[:la], \
            gw[:lw].reshape(n, k) if lw == n * k else gw[:lw], (gb[:lb] if bias else None)

    def cpu_mpgemm_fast(self, packed, fmt, act, scales, m, n, k, threads):
        b = np.ascontiguousarray(packed, np.uint8)
        a = np.ascontiguousarray(act, np.float32).reshape(-1)
        s = np.ascontiguousarray(scales, np.float32).reshape(-1)
        out = np.zeros(m * n, np.float32)
        tu, ku = C.c_int(0), C.c_int(0)
        rc = self.lib.to_cpu_mpgemm_fast(_p(b, u8p), b.size, fmt, _p(a, f32p), _p(s, f32p), m, n, k,
                                         _p(out, f32p), threads, C.byref(tu), C.byref(ku))
        assert rc == 0, rc
        return out.reshape(m, n), tu.value, ku.value

    def accepts(self, got, want, rel=1e-4, bit_exact=False, floor=1.0):
        return bool(self.lib.to_accepts_with_floor(float(got), float(want), rel, int(bit_exact), floor))

    def generate_vectors(self, seed, count):
        ps = self.lib.to_generate_vectors(seed, count)
        out = []
        try:
            s = ps.contents
            for i in range(s.count):
                v = s.v[i]
                m, n, k = v.m, v.n, v.k
                out.append(dict(
                    id=v.id.decode(), m=m, n=n, k=k, format=v.format,
                    activation=np.ctypeslib.as_array(v.activation, (m * k,)).copy(),
                    weights=np.ctypeslib.as_array(v.weights, (n * k,)).copy(),
                    scales=np.ctypeslib.as_array(v.scales, (n,)).copy(),
                    expected=np.ctypeslib.as_array(v.expected, (m * n,)).copy()))
        finally:
            self.lib.to_free_vectors(ps)
        return out

    def f32_to_bf16(self, x):
        return self.lib.to_f32_to_bf16(float(x))

    def bf16_to_f32(self, h):
        return self.lib.to_bf16_to_f32(int(h))


def build():
    subprocess.check_call(["make", "-s", "-C", ORACLE_DIR])


def load():
    if not os.path.exists(SO):
        build()
    return Oracle(C.CDLL(SO))
