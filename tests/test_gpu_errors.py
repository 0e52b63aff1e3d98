"""Error behaviour through the C ABI, as the reference's backends behave
(crates/tritium-cpu/src/lib.rs:801-886; crates/tritium-rocm/src/rocm.rs:446-535)."""
import numpy as np
import pytest

import tritium_amd as T

pytestmark = pytest.mark.gpu


def _buf(backend, n, k, fmt=T.TernaryFormat.Tq2_0, fill=0):
    packed = T.pack_rows(np.full(n * k, fill, np.int8), n, k, fmt)
    return backend.upload_weights(packed, T.GemmShape(0, n, k), fmt)


def test_upload_rejects_wrong_length(backend):
    short = np.zeros(2 * 66 - 1, np.uint8)
    with pytest.raises(T.InvalidInput):
        backend.upload_weights(short, T.GemmShape(1, 2, 256), T.TernaryFormat.Tq2_0)
    with pytest.raises(T.UnsupportedFormat):
        backend.upload_weights(np.zeros(64, np.uint8), T.GemmShape(1, 1, 256), T.TernaryFormat.I2sInt8)


def test_upload_accepts_correct_length(backend):
    buf = _buf(backend, 3, 256)
    assert buf.len_bytes() == 3 * 66 and not buf.is_empty()
    assert (buf.n, buf.k, buf.format) == (3, 256, T.TernaryFormat.Tq2_0)
    empty = backend.upload_weights(np.zeros(0, np.uint8), T.GemmShape(0, 0, 256), T.TernaryFormat.Tq2_0)
    assert empty.is_empty()


def test_mpgemm_rejects_foreign_buffer(backend):
    class Foreign(T.DeviceBuffer):
        def len_bytes(self):
            return 0
    out = np.zeros(1, np.float32)
    with pytest.raises(T.InvalidInput):
        backend.mpgemm(T.MpGemm(np.zeros(256, np.float32), Foreign(), np.ones(1, np.float32),
                                T.GemmShape(1, 1, 256), T.TernaryFormat.Tq2_0, out))


def test_mpgemm_rejects_bad_operand_lengths(backend):
    buf = _buf(backend, 1, 256)
    out = np.zeros(2, np.float32)
    with pytest.raises(T.ShapeMismatch) as e:  # act too short for M=2
        backend.mpgemm(T.MpGemm(np.zeros(256, np.float32), buf, np.ones(1, np.float32), T.GemmShape(2, 1, 256),
                                T.TernaryFormat.Tq2_0, out))
    assert (e.value.expected, e.value.got) == (512, 256)
    with pytest.raises(T.ShapeMismatch):       # scales
        backend.mpgemm(T.MpGemm(np.zeros(512, np.float32), buf, np.ones(2, np.float32), T.GemmShape(2, 1, 256),
                                T.TernaryFormat.Tq2_0, out))
    with pytest.raises(T.ShapeMismatch):       # out
        backend.mpgemm(T.MpGemm(np.zeros(512, np.float32), buf, np.ones(1, np.float32), T.GemmShape(2, 1, 256),
                                T.TernaryFormat.Tq2_0, np.zeros(3, np.float32)))
    with pytest.raises(T.ShapeMismatch):       # fused path validates the same lengths
        backend.mpgemm_with_act_quant(T.MpGemm(np.zeros(256, np.float32), buf, np.ones(1, np.float32),
                                               T.GemmShape(2, 1, 256), T.TernaryFormat.Tq2_0, out))


def test_mpgemm_rejects_identity_mismatch(backend):
    buf = _buf(backend, 2, 256)
    out = np.zeros(3, np.float32)
    with pytest.raises(T.InvalidInput):  # buffer is [2,256], call says N=3
        backend.mpgemm(T.MpGemm(np.zeros(256, np.float32), buf, np.ones(3, np.float32), T.GemmShape(1, 3, 256),
                                T.TernaryFormat.Tq2_0, out))
    with pytest.raises(T.InvalidInput):  # format differs
        backend.mpgemm(T.MpGemm(np.zeros(256, np.float32), buf, np.ones(2, np.float32), T.GemmShape(1, 2, 256),
                                T.TernaryFormat.Tq1_0, np.zeros(2, np.float32)))


def test_empty_shapes_are_ok(backend):
    buf = _buf(backend, 2, 256)
    backend.mpgemm(T.MpGemm(np.zeros(0, np.float32), buf, np.ones(2, np.float32), T.GemmShape(0, 2, 256),
                            T.TernaryFormat.Tq2_0, np.zeros(0, np.float32)))
    empty = backend.upload_weights(np.zeros(0, np.uint8), T.GemmShape(0, 0, 256), T.TernaryFormat.Tq2_0)
    backend.mpgemm(T.MpGemm(np.zeros(256, np.float32), empty, np.ones(0, np.float32), T.GemmShape(1, 0, 256),
                            T.TernaryFormat.Tq2_0, np.zeros(0, np.float32)))


def test_reserved_code_reported_at_mpgemm(backend):
    """Upload accepts the bytes; the contraction reports the row, like the CPU backend's unpack
    (crates/tritium-cpu/src/lib.rs:213,282-292)."""
    packed = T.pack_rows(np.zeros(3 * 256, np.int8), 3, 256)
    packed[66 * 2 + 7] = 0xC0  # slot 3 of a byte of row 2 holds code 3
    buf = backend.upload_weights(packed, T.GemmShape(0, 3, 256), T.TernaryFormat.Tq2_0)
    with pytest.raises(T.Backend, match="unpack row 2"):
        backend.mpgemm(T.MpGemm(np.zeros(256, np.float32), buf, np.ones(3, np.float32), T.GemmShape(1, 3, 256),
                                T.TernaryFormat.Tq2_0, np.zeros(3, np.float32)))


def test_gemm_min_m_knob(backend):
    assert backend.gemm_min_m() == 65
    backend.set_gemm_min_m(32)
    assert backend.gemm_min_m() == 32
    with pytest.raises(T.InvalidInput):
        backend.set_gemm_min_m(1)
    backend.set_gemm_min_m(65)


def test_exact_max_macs_knob(backend):
    assert backend.exact_max_macs() == 1 << 20
    backend.set_exact_max_macs(0)
    assert backend.exact_max_macs() == 0
    backend.set_exact_max_macs(1 << 20)


def test_one_backend_shared_by_threads(backend, oracle):
    """TernaryBackend is Send + Sync: one object serves concurrent callers
    (crates/tritium-spec/src/lib.rs:166; crates/tritium-rocm/src/rocm.rs:207-211). Four threads issue
    fused calls of different shapes at the same time; every result has the oracle's bits, and an
    error raised in one thread does not leak into another's last-error text."""
    import threading

    from helpers import same_bits, scales, ternary
    from oracle_lib import FMT_TQ2_0

    rng = np.random.default_rng(77)
    jobs = []
    for m, n, k in ((1, 48, 512), (3, 33, 700), (5, 130, 300), (2, 64, 1280)):
        w, sc = ternary(rng, n, k), scales(rng, n)
        packed = oracle.pack_matrix(w, n, k, FMT_TQ2_0)
        buf = backend.upload_weights(packed, T.GemmShape(0, n, k), T.TernaryFormat.Tq2_0)
        act = rng.standard_normal((m, k)).astype(np.float32)
        rc, want = oracle.cpu_mpgemm_with_act_quant(packed, FMT_TQ2_0, act, sc, m, n, k)
        assert rc == 0
        jobs.append((buf, act, sc, (m, n, k), want))
    failures = []

    def worker(job, idx):
        buf, act, sc, (m, n, k), want = job
        try:
            for it in range(25):
                out = np.zeros((m, n), np.float32)
                backend.mpgemm_with_act_quant(T.MpGemm(act, buf, sc, T.GemmShape(m, n, k), T.TernaryFormat.Tq2_0, out))
                if not same_bits(out, want):
                    failures.append((idx, it, "bits"))
                if idx == 0 and it % 5 == 0:  # a failing call in one thread, while the others compute
                    try:
                        backend.mpgemm(T.MpGemm(act[:, :-1], buf, sc, T.GemmShape(m, n, k), T.TernaryFormat.Tq2_0, out))
                        failures.append((idx, it, "no error"))
                    except T.ShapeMismatch as e:
                        if (e.expected, e.got) != (m * k, m * (k - 1)):
                            failures.append((idx, it, "mismatch fields"))
        except Exception as e:  # noqa: BLE001 - reported below
            failures.append((idx, "exception", repr(e)))

    threads = [threading.Thread(target=worker, args=(job, i)) for i, job in enumerate(jobs)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures[:5]
    for job in jobs:
        job[0].free()
