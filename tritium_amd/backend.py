"""Host-side mirror of the reference's backend adapter for this path.

Names, argument meaning and error behaviour follow `TernaryBackend`, `MpGemm`, `DeviceBuffer`,
`DeviceCaps`, `BackendError` (crates/tritium-spec/src/lib.rs:64-78,147-158,166-333,382-405;
caps.rs:7-67) and the registration record (crates/tritium-runtime/src/lib.rs:73-217). Everything
computes in the HIP library behind the C ABI; nothing here has a CPU path.
"""
import ctypes as C
import enum
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

from . import _lib as L


# ---- BackendError (crates/tritium-spec/src/lib.rs:382-405) -----------------------------------

class BackendError(Exception):
    """Base of every error a backend returns; backends never panic on bad input."""


class ShapeMismatch(BackendError):
    def __init__(self, expected, got, msg=None):
        super().__init__(msg or f"shape mismatch: expected {expected}, got {got}")
        self.expected, self.got = expected, got


class UnsupportedFormat(BackendError):
    pass


class OutOfMemory(BackendError):
    def __init__(self, requested, msg=None):
        super().__init__(msg or f"out of device memory: requested {requested} bytes")
        self.requested = requested


class InvalidInput(BackendError):
    pass


class Backend(BackendError):
    """Device-specific failure, stringified (BackendError::Backend)."""


def _raise(code):
    lib = L.load()
    msg = (lib.tk_last_error() or b"").decode()
    if code == L.TK_ERR_SHAPE_MISMATCH:
        e, g = C.c_size_t(0), C.c_size_t(0)
        lib.tk_last_mismatch(C.byref(e), C.byref(g))
        raise ShapeMismatch(e.value, g.value, msg)
    if code == L.TK_ERR_UNSUPPORTED_FORMAT:
        raise UnsupportedFormat(msg)
    if code == L.TK_ERR_OUT_OF_MEMORY:
        e, g = C.c_size_t(0), C.c_size_t(0)
        lib.tk_last_mismatch(C.byref(e), C.byref(g))
        raise OutOfMemory(e.value, msg)
    if code == L.TK_ERR_INVALID_INPUT:
        raise InvalidInput(msg)
    raise Backend(msg)


def _check(code):
    if code != L.TK_OK:
        _raise(code)


# ---- vocabulary (crates/tritium-core/src/{shape.rs:10-38,dtype.rs:89-107}) --------------------

class TernaryFormat(enum.IntEnum):
    Tq1_0 = 1
    Tq2_0 = 2
    I2sInt8 = 3


@dataclass(frozen=True)
class GemmShape:
    m: int
    n: int
    k: int

    def macs(self):
        return self.m * self.n * self.k

    def buffers_fit(self, act_len, weight_len, out_len):
        return act_len == self.m * self.k and weight_len == self.n * self.k and out_len == self.m * self.n


@dataclass
class DeviceCaps:
    backend: str
    device_name: str
    features: List[str] = field(default_factory=list)
    total_memory_bytes: int = 0
    supports_imma: bool = False
    supports_fp8: bool = False

    def has_feature(self, name):
        return name in self.features


class DeviceBuffer:
    """Opaque handle to device-resident memory owned by a backend."""

    def len_bytes(self):
        raise NotImplementedError

    def is_empty(self):
        return self.len_bytes() == 0


@dataclass
class MpGemm:
    """Operands of one ternary mixed-precision GEMM call (crates/tritium-spec/src/lib.rs:64-78)."""
    act: np.ndarray          # [M,K] f32, row-major (flat or 2-D)
    weights: DeviceBuffer
    scales: np.ndarray       # [N] f32
    shape: GemmShape
    format: TernaryFormat
    out: np.ndarray          # [M,N] f32, overwritten


@dataclass
class MpGemmProjectedVjp:
    """Operands of the VJP of one packed ternary mpGEMM (crates/tritium-spec/src/lib.rs:93-117).
    grad_projected_weight is the gradient with respect to P[n,k] = scales[n] * trit[n,k]."""
    act: np.ndarray                    # [M,K] f32
    weights: DeviceBuffer
    scales: np.ndarray                 # [N] f32
    grad_output: np.ndarray            # [M,N] f32
    shape: GemmShape
    format: TernaryFormat
    grad_act: np.ndarray               # [M,K] f32, overwritten
    grad_projected_weight: np.ndarray  # [N,K] f32, overwritten
    grad_bias: Optional[np.ndarray] = None  # [N] f32, overwritten when given


DTYPES = {"f32": L.TK_F32, "bf16": L.TK_BF16, "i8": L.TK_I8, "i32": L.TK_I32}
_NP = {L.TK_F32: np.float32, L.TK_BF16: np.uint16, L.TK_I8: np.int8, L.TK_I32: np.int32}


class DeviceArray:
    """A device allocation with a dtype tag; bf16 travels as uint16 bit patterns on the host."""

    def __init__(self, backend, ptr, count, dtype):
        self.backend, self.ptr, self.count, self.dtype = backend, ptr, count, dtype

    @property
    def nbytes(self):
        return self.count * np.dtype(_NP[self.dtype]).itemsize

    def to_host(self):
        out = np.empty(self.count, _NP[self.dtype])
        _check(L.load().tk_memcpy_d2h(self.backend._ctx, out.ctypes.data, self.ptr, out.nbytes))
        return out

    def copy_from(self, host):
        h = np.ascontiguousarray(host, _NP[self.dtype]).reshape(-1)
        assert h.size == self.count, (h.size, self.count)
        _check(L.load().tk_memcpy_h2d(self.backend._ctx, self.ptr, h.ctypes.data, h.nbytes))
        return self

    def free(self):
        if self.ptr:
            _check(L.load().tk_free(self.backend._ctx, self.ptr))
            self.ptr = None


class SaltV2Tensor:
    """A SALT V2 matrix resident on the device (tk_salt_v2)."""

    def __init__(self, backend, handle, n, k):
        self._backend, self._h, self.n, self.k = backend, handle, n, k

    def forward(self, act, m, out):
        """out[m,n] = act[m,k] x W^T in the reference's pinned order (device f32 arrays); raises InvalidInput
        and leaves out untouched when an activation or a result is not finite."""
        _check(L.load().tk_salt_v2_forward(self._backend._ctx, self._h, act.ptr, m, out.ptr))

    def gather_rows(self, rows, out):
        r = np.ascontiguousarray(rows, np.uint32).reshape(-1)
        _check(L.load().tk_salt_v2_gather_rows(self._backend._ctx, self._h, r.ctypes.data, r.size, out.ptr))

    def free(self):
        if self._h:
            L.load().tk_salt_v2_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Mi355xBuffer(DeviceBuffer):
    """Packed ternary weights resident on the device; frees its memory when dropped."""

    def __init__(self, backend, handle):
        self._backend, self._h = backend, handle

    def len_bytes(self):
        return L.load().tk_weights_len_bytes(self._h)

    @property
    def n(self):
        return L.load().tk_weights_n(self._h)

    @property
    def k(self):
        return L.load().tk_weights_k(self._h)

    @property
    def format(self):
        return TernaryFormat(L.load().tk_weights_format(self._h))

    def zero_chunks(self):
        """(all-zero 1-KiB chunks, chunks, whether the upload kept a skip map for them)."""
        z, t, kept = C.c_size_t(0), C.c_size_t(0), C.c_int(0)
        _check(L.load().tk_weights_zero_chunks(self._h, C.byref(z), C.byref(t), C.byref(kept)))
        return z.value, t.value, bool(kept.value)

    def base3_bytes(self):
        """Bytes of this buffer's base-3 stream (0 when the upload kept none)."""
        return L.load().tk_weights_base3_bytes(self._h)

    def download_trits(self):
        out = np.empty(self.n * self.k, np.int8)
        _check(L.load().tk_weights_download_trits(self._backend._ctx, self._h, out.ctypes.data, out.size))
        return out.reshape(self.n, self.k)

    def free(self):
        if self._h and self._backend._ctx:
            L.load().tk_free_weights(self._h)
        self._h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Linear:
    """Device-resident additive-plane linear layer: plane handles + per-plane scale vectors."""

    def __init__(self, backend, planes, scales):
        self.backend, self.planes, self.scales = backend, list(planes), list(scales)
        assert 1 <= len(self.planes) <= L.TK_MAX_PLANES and len(self.planes) == len(self.scales)
        self.n, self.k = self.planes[0].n, self.planes[0].k
        d = L.LinearDesc()
        for i, (p, s) in enumerate(zip(self.planes, self.scales)):
            d.planes[i] = p._h
            d.scales[i] = s.ptr
        d.n_planes = len(self.planes)
        self.desc = d

    def free(self):
        for p in self.planes:
            p.free()
        for s in self.scales:
            s.free()


class Group:
    def __init__(self, backend, handle, keep):
        self.backend, self._h, self._keep = backend, handle, keep

    def launch(self):
        _check(L.load().tk_group_launch(self.backend._ctx, self._h))

    def launch_parts(self, prep=True, main=True):
        _check(L.load().tk_group_launch_parts(self.backend._ctx, self._h, int(prep), int(main)))

    def destroy(self):
        if self._h:
            L.load().tk_group_destroy(self._h)
            self._h = None


class Event:
    def __init__(self, backend):
        self.backend = backend
        h = C.c_void_p()
        _check(L.load().tk_event_create(backend._ctx, C.byref(h)))
        self._h = h

    def record(self):
        _check(L.load().tk_event_record(self.backend._ctx, self._h))
        return self

    def elapsed_ms(self, stop):
        ms = C.c_float(0)
        _check(L.load().tk_event_elapsed_ms(self._h, stop._h, C.byref(ms)))
        return ms.value

    def destroy(self):
        if self._h:
            L.load().tk_event_destroy(self._h)
            self._h = None


def _flat(a, dtype, name):
    arr = np.ascontiguousarray(a, dtype=dtype).reshape(-1)
    return arr


class Mi355xBackend:
    """`impl TernaryBackend` for one MI355X (gfx950). Thread-safe; calls are synchronous."""

    NAME = "mi355x"

    def __init__(self, ordinal=0):
        self._lib = L.load()
        ctx = C.c_void_p()
        _check(self._lib.tk_init(ordinal, C.byref(ctx)))
        self._ctx = ctx
        info = L.DeviceInfo()
        _check(self._lib.tk_device_info_get(ctx, C.byref(info)))
        self.info = info

    def close(self):
        if self._ctx:
            self._lib.tk_destroy(self._ctx)
            self._ctx = None

    # ---- TernaryBackend ----
    def device_id(self):
        return self._lib.tk_device_id(self._ctx).decode()

    def physical_device_id(self):
        return self.device_id()

    def capabilities(self):
        return DeviceCaps(backend="mi355x", device_name=self.info.name.decode(),
                          features=["hip", self.info.arch.decode().split(":")[0], "tq2_0", "tq1_0", "mfma_i8",
                                    "act_quant_i8", "additive_planes", "rmsnorm_quant_i8", "salt_block_scales"],
                          total_memory_bytes=int(self.info.total_memory_bytes), supports_imma=True,
                          supports_fp8=False)

    def upload_weights(self, packed, shape, format):
        b = np.ascontiguousarray(packed, dtype=np.uint8).reshape(-1)
        h = C.c_void_p()
        _check(self._lib.tk_upload_weights(self._ctx, b.ctypes.data, b.size, shape.n, shape.k, int(format),
                                           C.byref(h)))
        return Mi355xBuffer(self, h)

    def upload_weights_i2s(self, payload, shape):
        """I2_S tensor payload (quants + per-tensor f32 scale) -> (device buffer in TQ2_0 form, scale):
        convert_i2s_to_tq2_0 (crates/tritium-format/src/i2s_int8.rs:36-68) followed by upload_weights."""
        b = np.ascontiguousarray(payload, dtype=np.uint8).reshape(-1)
        h, sc = C.c_void_p(), C.c_float(0.0)
        _check(self._lib.tk_upload_weights_i2s(self._ctx, b.ctypes.data, b.size, shape.n, shape.k, C.byref(h),
                                               C.byref(sc)))
        return Mi355xBuffer(self, h), np.float32(sc.value)

    def upload_weights_gguf(self, gguf, buf, name):
        """One ternary weight tensor of a GGUF file onto the device -> (device buffer, row scales [n] f32):
        load_ternary of the model loader (crates/tritium-nn/src/model/weights.rs:177-333)."""
        b = np.ascontiguousarray(buf, dtype=np.uint8).reshape(-1)
        n, _, _ = gguf.ternary_shape(name)
        h, scales = C.c_void_p(), np.zeros(n, np.float32)
        _check(self._lib.tk_upload_weights_gguf(self._ctx, gguf._h, b.ctypes.data, b.size, name.encode(), C.byref(h),
                                                scales.ctypes.data, n))
        return Mi355xBuffer(self, h), scales

    def upload_weights_scaled(self, packed, shape):
        """TQ2_0 rows whose f16 block scales are kept on the device (block-scale planes)."""
        b = np.ascontiguousarray(packed, dtype=np.uint8).reshape(-1)
        h = C.c_void_p()
        _check(self._lib.tk_upload_weights_scaled(self._ctx, b.ctypes.data, b.size, shape.n, shape.k, C.byref(h)))
        return Mi355xBuffer(self, h)

    def upload_salt_rows(self, data, n, k, max_planes=1 << 30):
        """A SALT tensor -- n encoded rows ("TSLT" version 1 or 2, sparse residuals allowed) back to back -- as
        block-scale planes for linear_salt; max_planes keeps a prefix of every row."""
        b = np.ascontiguousarray(data, dtype=np.uint8).reshape(-1)
        hs, count = (C.c_void_p * L.TK_MAX_PLANES)(), C.c_int(0)
        _check(self._lib.tk_upload_salt_rows(self._ctx, b.ctypes.data, b.size, n, k, max_planes, hs, C.byref(count)))
        return [Mi355xBuffer(self, C.c_void_p(hs[i])) for i in range(count.value)]

    def salt_v2_upload(self, codec, scale_group, payload, scales_f16, plane_counts, n, k):
        """A SALT V2 matrix [n,k] from its runtime parts: codec payload, f16 scale bits, per-tile plane counts."""
        pay = np.ascontiguousarray(payload, np.uint8).reshape(-1)
        sc = np.ascontiguousarray(scales_f16, np.uint16).reshape(-1)
        pc = np.ascontiguousarray(plane_counts, np.uint8).reshape(-1)
        h = C.c_void_p()
        _check(self._lib.tk_salt_v2_upload(self._ctx, int(codec), scale_group, pay.ctypes.data, pay.size, sc.ctypes.data, sc.size,
                                           pc.ctypes.data, pc.size, n, k, C.byref(h)))
        return SaltV2Tensor(self, h, n, k)

    def linear_salt(self, planes, act, m, out, seq=False):
        """Block-scale additive planes on float activations: planes = buffers from
        upload_weights_scaled; seq=True takes the host's summation order for every output."""
        d = L.SaltDesc()
        for i, w in enumerate(planes):
            d.planes[i] = w._h
        d.n_planes = len(planes)
        fn = self._lib.tk_linear_salt_seq if seq else self._lib.tk_linear_salt
        _check(fn(self._ctx, C.byref(d), act.ptr, act.dtype, m, out.ptr, out.dtype))

    def _host_call(self, fn, p):
        if not isinstance(p.weights, Mi355xBuffer) or p.weights._backend is not self or not p.weights._h:
            raise InvalidInput("buffer is not a Mi355xBuffer of this backend")
        if not (isinstance(p.out, np.ndarray) and p.out.dtype == np.float32 and p.out.flags.c_contiguous):
            raise InvalidInput("out must be a C-contiguous float32 numpy array")
        act = _flat(p.act, np.float32, "act")
        scales = _flat(p.scales, np.float32, "scales")
        s = p.shape
        _check(fn(self._ctx, act.ctypes.data, act.size, p.weights._h, scales.ctypes.data, scales.size,
                  s.m, s.n, s.k, int(p.format), p.out.ctypes.data, p.out.size))

    def mpgemm(self, p):
        self._host_call(self._lib.tk_mpgemm, p)

    def mpgemm_with_act_quant(self, p):
        self._host_call(self._lib.tk_mpgemm_with_act_quant, p)

    def mpgemm_projected_vjp(self, p):
        """grad_act, grad_projected_weight and the optional grad_bias of one packed mpGEMM, with the
        bits of the CPU backend's scalar path (crates/tritium-cpu/src/kernel.rs:281-317)."""
        if not isinstance(p.weights, Mi355xBuffer) or p.weights._backend is not self or not p.weights._h:
            raise InvalidInput("buffer is not a Mi355xBuffer of this backend")
        outs = [p.grad_act, p.grad_projected_weight] + ([p.grad_bias] if p.grad_bias is not None else [])
        for o in outs:
            if not (isinstance(o, np.ndarray) and o.dtype == np.float32 and o.flags.c_contiguous):
                raise InvalidInput("gradient outputs must be C-contiguous float32 numpy arrays")
        act = _flat(p.act, np.float32, "act")
        scales = _flat(p.scales, np.float32, "scales")
        up = _flat(p.grad_output, np.float32, "grad_output")
        s = p.shape
        gb = p.grad_bias
        _check(self._lib.tk_mpgemm_projected_vjp(
            self._ctx, act.ctypes.data, act.size, p.weights._h, scales.ctypes.data, scales.size, up.ctypes.data,
            up.size, s.m, s.n, s.k, int(p.format), p.grad_act.ctypes.data, p.grad_act.size,
            p.grad_projected_weight.ctypes.data, p.grad_projected_weight.size,
            gb.ctypes.data if gb is not None else None, gb.size if gb is not None else 0))

    def projected_vjp(self, weights, scales, act, grad_output, m, grad_act, grad_w, grad_bias=None):
        """The same gradients on device-resident f32 arrays; enqueued, not synchronised. An output
        given as None is skipped."""
        ptr = lambda a: a.ptr if a is not None else None  # noqa: E731
        _check(self._lib.tk_projected_vjp(self._ctx, weights._h, scales.ptr, ptr(act), grad_output.ptr, m, ptr(grad_act),
                                          ptr(grad_w), ptr(grad_bias)))

    def as_concrete(self):
        return self

    # ---- device-resident extension ----
    def empty(self, count, dtype="f32"):
        dt = DTYPES[dtype] if isinstance(dtype, str) else dtype
        ptr = C.c_void_p()
        _check(self._lib.tk_malloc(self._ctx, count * np.dtype(_NP[dt]).itemsize, C.byref(ptr)))
        return DeviceArray(self, ptr, count, dt)

    def to_device(self, host, dtype):
        dt = DTYPES[dtype] if isinstance(dtype, str) else dtype
        h = np.ascontiguousarray(host, _NP[dt]).reshape(-1)
        return self.empty(h.size, dt).copy_from(h)

    def sync(self):
        _check(self._lib.tk_sync(self._ctx))

    def stream_handle(self):
        """The hipStream_t every call of this backend enqueues on, as an integer (for callers that record events on
        it, wait for it from another stream, or capture it into a HIP graph)."""
        return int(self._lib.tk_stream(self._ctx) or 0)

    def linear(self, packed_planes, scales_planes, n, k, format=TernaryFormat.Tq2_0):
        shape = GemmShape(0, n, k)  # upload is called with m = 0 (crates/tritium-nn/src/layers/linear.rs:97)
        planes = [self.upload_weights(p, shape, format) for p in packed_planes]
        scales = [self.to_device(s, "f32") for s in scales_planes]
        for s in scales:
            if s.count != n:
                raise ShapeMismatch(n, s.count)
        return Linear(self, planes, scales)

    def _lin(self, fn, layer, act, m, out):
        _check(fn(self._ctx, C.byref(layer.desc), act.ptr, act.dtype, m, out.ptr, out.dtype))

    def linear_float(self, layer, act, m, out):
        self._lin(self._lib.tk_linear_float, layer, act, m, out)

    def linear_a8(self, layer, act, m, out):
        self._lin(self._lib.tk_linear_a8, layer, act, m, out)

    def linear_a8_noalloc(self, layer, act, m, out):
        """linear_a8 on the static device scratch: no allocation; refuses shapes that do not fit."""
        self._lin(self._lib.tk_linear_a8_noalloc, layer, act, m, out)

    def linear_a8_residual(self, layer, act, m, residual, out):
        """out = residual + linear_a8(act); residual has the output's dtype and may be `out` itself."""
        _check(self._lib.tk_linear_a8_residual(self._ctx, C.byref(layer.desc), act.ptr, act.dtype, m, residual.ptr,
                                               out.ptr, out.dtype))

    def linear_i8_residual(self, layer, q, act_scale, m, residual, out):
        _check(self._lib.tk_linear_i8_residual(self._ctx, C.byref(layer.desc), q.ptr,
                                               act_scale.ptr if act_scale is not None else None, m, residual.ptr,
                                               out.ptr, out.dtype))

    def linear_float_seq(self, layer, act, m, out):
        self._lin(self._lib.tk_linear_float_seq, layer, act, m, out)

    def linear_i8(self, layer, q, act_scale, m, out):
        _check(self._lib.tk_linear_i8(self._ctx, C.byref(layer.desc), q.ptr,
                                      act_scale.ptr if act_scale is not None else None, m, out.ptr, out.dtype))

    def act_quant_i8(self, act, m, k, q, act_scale, nonfinite=None):
        _check(self._lib.tk_act_quant_i8(self._ctx, act.ptr, act.dtype, m, k, q.ptr, act_scale.ptr,
                                         nonfinite.ptr if nonfinite is not None else None))

    @staticmethod
    def _norm(weight, eps, zero_centered):
        nm = L.RmsNorm()
        nm.weight = weight.ptr if weight is not None else None
        nm.eps = eps
        nm.zero_centered = int(bool(zero_centered))
        return nm

    def rmsnorm_quant_i8(self, x, weight, eps, m, k, q, act_scale, nonfinite=None, zero_centered=False):
        """RMSNorm of each row of x [m,k], then the per-token int8 quantization, in one launch."""
        nm = self._norm(weight, eps, zero_centered)
        _check(self._lib.tk_rmsnorm_quant_i8(self._ctx, x.ptr, x.dtype, C.byref(nm), m, k, q.ptr, act_scale.ptr,
                                             nonfinite.ptr if nonfinite is not None else None))

    def linear_rmsnorm_a8(self, layer, x, weight, eps, m, out, zero_centered=False):
        """linear_a8 on RMSNorm(x): weight is a device array of k floats."""
        nm = self._norm(weight, eps, zero_centered)
        _check(self._lib.tk_linear_rmsnorm_a8(self._ctx, C.byref(layer.desc), x.ptr, x.dtype, C.byref(nm), m, out.ptr,
                                              out.dtype))

    def group(self, members, mode, act_dtype, out_dtype, norms=None):
        """members: list of (Linear, act DeviceArray, m, out DeviceArray). norms (W1.58A8 groups
        only): one entry per member, None or (weight DeviceArray, eps, zero_centered)."""
        arr = (L.GroupMember * len(members))()
        for i, (layer, act, m, out) in enumerate(members):
            arr[i].layer = layer.desc
            arr[i].act = act.ptr
            arr[i].m = m
            arr[i].out = out.ptr
        h = C.c_void_p()
        if norms is None:
            _check(self._lib.tk_group_create(self._ctx, arr, len(members), mode, DTYPES[act_dtype],
                                             DTYPES[out_dtype], C.byref(h)))
            return Group(self, h, members)
        if mode != 1 or len(norms) != len(members):
            raise ValueError("norms need a W1.58A8 group and one entry per member")
        narr = (L.RmsNorm * len(members))()
        for i, nm in enumerate(norms):
            narr[i] = self._norm(*nm) if nm is not None else self._norm(None, 0.0, False)
        _check(self._lib.tk_group_create_normed(self._ctx, arr, narr, len(members), DTYPES[act_dtype],
                                                DTYPES[out_dtype], C.byref(h)))
        return Group(self, h, (members, norms))

    def set_gemm_min_m(self, v):
        _check(self._lib.tk_set_gemm_min_m(self._ctx, v))

    def gemm_min_m(self):
        return self._lib.tk_get_gemm_min_m(self._ctx)

    def set_decode_kernel(self, variant):
        """0 automatic, 1 K-split, 2 streaming, 3 flow."""
        _check(self._lib.tk_set_decode_kernel(self._ctx, variant))

    def set_flow_run_tiles(self, tiles):
        _check(self._lib.tk_set_flow_run_tiles(self._ctx, tiles))

    def set_flow_ring(self, positions):
        _check(self._lib.tk_set_flow_ring(self._ctx, positions))

    def set_flow_mfma(self, rows):
        _check(self._lib.tk_set_flow_mfma(self._ctx, rows))

    def set_gemm_tiles(self, tiles):
        """0 automatic, 2 or 4 output tiles per wave of the one-plane prefill kernel."""
        _check(self._lib.tk_set_gemm_tiles(self._ctx, tiles))

    def set_gemm_two_by_two(self, on):
        """One-plane prefill kernel, 64 x 128 form: waves two by two instead of four side by side (same bits)."""
        _check(self._lib.tk_set_gemm_two_by_two(self._ctx, 1 if on else 0))

    def set_prep_team_rows(self, rows):
        """Activation prep: launches of up to `rows` tokens give a token the whole workgroup (default 384)."""
        _check(self._lib.tk_set_prep_team_rows(self._ctx, rows))

    def set_group_overlap(self, on):
        """Grouped launches of two kernels (flow part + prefill-kernel part): side by side (default) or in turn."""
        _check(self._lib.tk_set_group_overlap(self._ctx, 1 if on else 0))

    def set_host_direct_bytes(self, nbytes):
        """Host-slice calls (`mpgemm`, `mpgemm_with_act_quant`) of up to `nbytes` of operands go through the context's
        pinned host block instead of four pageable transfers (default 1 MiB, 0 = never)."""
        _check(self._lib.tk_set_host_direct_bytes(self._ctx, nbytes))

    def set_fuse_tokens(self, tokens):
        """Decode calls (and groups created afterwards) of up to `tokens` tokens (1..4) build their operand rows inside
        the decode kernel: one launch instead of two. 0 = always the separate prep launch, -1 (default) = chosen per
        call (one token; two under the int8 contract in single narrow calls)."""
        _check(self._lib.tk_set_fuse_tokens(self._ctx, tokens))

    def fused_calls(self):
        """Calls so far that ran as one launch (the decode kernel built the operand rows itself)."""
        c = C.c_ulonglong(0)
        _check(self._lib.tk_get_fused_calls(self._ctx, C.byref(c)))
        return int(c.value)

    def last_kernel(self):
        """Name of the contraction kernel the last single call took ("flow", "gemm64_ksplit", "gemm128", ...)."""
        return self._lib.tk_last_kernel(self._ctx).decode()

    def set_gemm_rows(self, rows):
        """0 = automatic, 64 / 128 / 256 = rows of the workgroup tile for one-plane int8-contract prefill launches."""
        _check(self._lib.tk_set_gemm_rows(self._ctx, rows))

    def set_gemm256_form(self, form):
        """The 256-row prefill kernel: 0 = 4 waves x 224 outputs, 1 = 8 waves x 224, 2 = 4 waves x (128 | 96) outputs with
        two workgroups per CU, -1 = chosen per launch (same bits)."""
        _check(self._lib.tk_set_gemm256_form(self._ctx, form))

    def set_gemm_ksplit(self, slices):
        """0 automatic, 1 off, 2..64 K slices of the prefill kernel in single launches."""
        _check(self._lib.tk_set_gemm_ksplit(self._ctx, slices))

    def set_zero_skip(self, mode):
        """Later uploads: 0 keep a zero-chunk map by the 0.5% threshold, 1 never, 2 always."""
        _check(self._lib.tk_set_zero_skip(self._ctx, mode))

    def set_flow_operand_order(self, weights_first):
        """Decode kernel under the int8 contract: 1 weights as the first operand of the matrix instruction (one wide
        store per lane), 0 activations first (same bits)."""
        _check(self._lib.tk_set_flow_operand_order(self._ctx, weights_first))

    def set_flow_workgroup_waves(self, waves):
        """Decode kernel, 17..32 operand rows beyond 80 KiB (one workgroup per CU): 0 automatic, 8 or 16 waves per
        workgroup (same bits)."""
        _check(self._lib.tk_set_flow_workgroup_waves(self._ctx, waves))

    def set_base3_stream(self, mode):
        """Later uploads: 0 no base-3 copy, 1 TQ1_0 uploads keep one beside the 2-bit codes, 2 every upload."""
        _check(self._lib.tk_set_base3_stream(self._ctx, mode))

    def set_stream_min_groups(self, groups):
        _check(self._lib.tk_set_stream_min_groups(self._ctx, groups))

    def stream_min_groups(self):
        return self._lib.tk_get_stream_min_groups(self._ctx)

    def set_exact_max_macs(self, macs):
        _check(self._lib.tk_set_exact_max_macs(self._ctx, macs))

    def exact_max_macs(self):
        return self._lib.tk_get_exact_max_macs(self._ctx)

    def event(self):
        return Event(self)

    def copy_kernel(self, dst, src, nbytes):
        _check(self._lib.tk_copy_kernel(self._ctx, dst.ptr, src.ptr, nbytes))


# ---- host-side packing (tritium-format rows, as TernaryLinear::pack_rows uses them) -----------

def packed_len(n, k, format):
    return L.load().tk_packed_len(n, k, int(format))


def salt_row_len(data):
    """Length of the first encoded SALT row in data (packed_salt_row_len)."""
    b = np.ascontiguousarray(data, np.uint8).reshape(-1)
    n = C.c_size_t(0)
    _check(L.load().tk_salt_row_len(b.ctypes.data, b.size, C.byref(n)))
    return n.value


def salt_row_unpack(data, max_planes=1 << 30):
    """One encoded SALT row -> (k, [dense TQ2_0 plane rows]); sparse residuals are expanded."""
    b = np.ascontiguousarray(data, np.uint8).reshape(-1)
    k, planes, version = C.c_size_t(0), C.c_size_t(0), C.c_int(0)
    _check(L.load().tk_salt_row_info(b.ctypes.data, b.size, C.byref(k), C.byref(planes), C.byref(version)))
    pb = (k.value + 255) // 256 * 66
    keep = min(planes.value, max_planes)
    out = np.zeros(max(keep * pb, 1), np.uint8)
    kk, got = C.c_size_t(0), C.c_size_t(0)
    _check(L.load().tk_salt_row_unpack(b.ctypes.data, b.size, max_planes, out.ctypes.data, keep * pb, C.byref(kk), C.byref(got)))
    return kk.value, [out[i * pb:(i + 1) * pb].copy() for i in range(got.value)]


def sparse_plane_to_tq2_0(data):
    """One encoded sparse residual plane ("TSSP") -> (k, the dense TQ2_0 row it stands for)."""
    b = np.ascontiguousarray(data, np.uint8).reshape(-1)
    if b.size < 10:
        k_hint = 0
    else:
        k_hint = int.from_bytes(bytes(b[6:10]), "little")
    out = np.zeros(max((k_hint + 255) // 256 * 66, 1), np.uint8)
    k = C.c_size_t(0)
    _check(L.load().tk_sparse_plane_to_tq2_0(b.ctypes.data, b.size, out.ctypes.data, (k_hint + 255) // 256 * 66, C.byref(k)))
    return k.value, out[: (k.value + 255) // 256 * 66]


SALT_V2_D2, SALT_V2_B3, SALT_V2_S34 = 0, 1, 2


def salt_v2_payload_bytes(codec, trits):
    n = C.c_size_t(0)
    _check(L.load().tk_salt_v2_payload_bytes(int(codec), trits, C.byref(n)))
    return n.value


def salt_v2_pack(codec, trits):
    t = np.ascontiguousarray(trits, np.int8).reshape(-1)
    out = np.zeros(max(salt_v2_payload_bytes(codec, t.size), 1), np.uint8)
    need = salt_v2_payload_bytes(codec, t.size)
    _check(L.load().tk_salt_v2_pack(int(codec), t.ctypes.data, t.size, out.ctypes.data, need))
    return out[:need]


def salt_v2_unpack(codec, packed, n):
    b = np.ascontiguousarray(packed, np.uint8).reshape(-1)
    out = np.zeros(max(n, 1), np.int8)
    _check(L.load().tk_salt_v2_unpack(int(codec), b.ctypes.data, b.size, n, out.ctypes.data))
    return out[:n]


def pack_rows(trits, n, k, format=TernaryFormat.Tq2_0):
    t = np.ascontiguousarray(trits, dtype=np.int8).reshape(-1)
    out = np.empty(packed_len(n, k, format), np.uint8)
    _check(L.load().tk_pack_rows(t.ctypes.data, t.size, n, k, int(format), out.ctypes.data, out.size))
    return out


def compute_zero_bitmaps(packed, n, k, row_bytes):
    """Per-row zero-block bitmaps of packed TQ2_0 rows (crates/tritium-format/src/tq2.rs:134-181):
    uint32 words, ceil(nb/32) per row."""
    b = np.ascontiguousarray(packed, dtype=np.uint8).reshape(-1)
    nb = (k + 255) // 256
    want = n * ((nb + 31) // 32)
    # the library checks the rows against the buffer before it touches the words: an absurd n is
    # refused there, so only a believable word count is allocated here
    words = np.zeros(want if nb and n * row_bytes <= b.size else 0, np.uint32)
    _check(L.load().tk_compute_zero_bitmaps(b.ctypes.data, b.size, n, k, row_bytes, words.ctypes.data,
                                            min(want, (1 << 63) - 1)))
    return words


def convert_i2s_to_tq2_0(payload, n, k):
    """(TQ2_0 rows with unit block scales, per-tensor scale) of an I2_S tensor payload
    (crates/tritium-format/src/i2s_int8.rs:36-68)."""
    b = np.ascontiguousarray(payload, dtype=np.uint8).reshape(-1)
    out = np.empty(packed_len(n, k, TernaryFormat.Tq2_0), np.uint8)
    sc = C.c_float(0.0)
    _check(L.load().tk_convert_i2s_to_tq2_0(b.ctypes.data, b.size, n, k, out.ctypes.data, out.size, C.byref(sc)))
    return out, np.float32(sc.value)


def unpack_rows(packed, n, k, format=TernaryFormat.Tq2_0):
    b = np.ascontiguousarray(packed, dtype=np.uint8).reshape(-1)
    out = np.empty(n * k, np.int8)
    _check(L.load().tk_unpack_rows(b.ctypes.data, b.size, n, k, int(format), out.ctypes.data, out.size))
    return out.reshape(n, k)


# ---- registration (crates/tritium-runtime/src/lib.rs:73-217) -----------------------------------

@dataclass
class BackendEntry:
    name: str
    init: object  # () -> backend, raises BackendError when the device is unavailable


BACKENDS: List[BackendEntry] = [BackendEntry(Mi355xBackend.NAME, lambda: Mi355xBackend(0))]


class Registry:
    """Initialises every registered backend; a failing init is logged to stderr and skipped."""

    def __init__(self, entries=None):
        import sys
        self.backends = []
        for entry in (BACKENDS if entries is None else entries):
            try:
                self.backends.append((entry.name, entry.init()))
            except BackendError as err:
                print(f"tritium-runtime: backend `{entry.name}` failed to initialise, skipping: {err}",
                      file=sys.stderr)

    def get(self, name) -> Optional[Mi355xBackend]:
        for n, b in self.backends:
            if n == name:
                return b
        return None

    def enumerate(self):
        return [b.capabilities() for _, b in self.backends]

    def __len__(self):
        return len(self.backends)

    def is_empty(self):
        return not self.backends
