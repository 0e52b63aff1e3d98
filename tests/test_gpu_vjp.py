"""TernaryBackend::mpgemm_projected_vjp through the C ABI: the reference's own cases
(crates/tritium-cpu/src/lib.rs:496-700, crates/tritium-cuda/src/cuda/tests.rs:724-800), bit for bit
against the CPU oracle's scalar path (the reference's bar between backends is 1e-4 relative)."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import same_bits, ternary
from oracle_lib import FMT_TQ1_0, FMT_TQ2_0

pytestmark = pytest.mark.gpu


def _vjp(backend, packed, fmt, act, scales, gy, m, n, k, bias=True):
    buf = backend.upload_weights(packed, T.GemmShape(m, n, k), T.TernaryFormat(fmt))
    ga = np.full((m, k), np.nan, np.float32)
    gw = np.full((n, k), np.nan, np.float32)
    gb = np.full(n, np.nan, np.float32) if bias else None
    backend.mpgemm_projected_vjp(T.MpGemmProjectedVjp(
        act=np.asarray(act, np.float32), weights=buf, scales=np.asarray(scales, np.float32),
        grad_output=np.asarray(gy, np.float32), shape=T.GemmShape(m, n, k), format=T.TernaryFormat(fmt),
        grad_act=ga, grad_projected_weight=gw, grad_bias=gb))
    return ga, gw, gb


def test_reference_known_answer(backend, oracle):
    """crates/tritium-cpu/src/lib.rs:500-533."""
    packed = oracle.pack_matrix(np.array([[1, 0, -1], [-1, 1, 1]], np.int8), 2, 3, FMT_TQ2_0)
    ga, gw, gb = _vjp(backend, packed, FMT_TQ2_0, [1.0, 2.0, 3.0, -1.0, 4.0, 0.5], [2.0, 0.5], [3.0, -2.0, 4.0, 1.0], 2, 2, 3)
    assert ga.reshape(-1).tolist() == [7.0, -1.0, -7.0, 7.5, 0.5, -7.5]
    assert gw.reshape(-1).tolist() == [-1.0, 22.0, 11.0, -3.0, 0.0, -5.5]
    assert gb.tolist() == [7.0, -1.0]


@pytest.mark.parametrize("fmt", [FMT_TQ2_0, FMT_TQ1_0])
@pytest.mark.parametrize("m,n,k", [(2, 3, 5), (7, 4, 257), (1, 33, 64), (2, 3, 257), (17, 35, 576), (33, 130, 1100),
                                   (70, 16, 256), (16, 64, 1024)])
def test_bits_of_the_cpu_scalar_path(backend, oracle, fmt, m, n, k):
    """The first three shapes are the reference's device test (tests.rs:734), the fourth its
    packed-decode test (lib.rs:536), (17, 35, 576) its training shape (tests.rs:818-820); the rest
    cross every tile edge of the kernels (16 tokens, 16 / 64 rows, 64 / 256 / 1024 columns)."""
    print("case vjp", fmt, m, n, k, flush=True)
    rng = np.random.default_rng(m * 1000 + n * 10 + k)
    w = ternary(rng, n, k)
    packed = oracle.pack_matrix(w, n, k, fmt)
    act = rng.uniform(-2, 2, (m, k)).astype(np.float32)
    sc = rng.uniform(0.05, 1.5, n).astype(np.float32)
    sc[0] = -sc[0]
    gy = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    rc, ga_w, gw_w, gb_w = oracle.cpu_projected_vjp(packed, fmt, act, sc, gy, m, n, k)
    assert rc == 0
    ga, gw, gb = _vjp(backend, packed, fmt, act, sc, gy, m, n, k)
    assert same_bits(ga, ga_w) and same_bits(gw, gw_w) and same_bits(gb, gb_w)
    ga, gw, gb = _vjp(backend, packed, fmt, act, sc, gy, m, n, k, bias=False)
    assert same_bits(ga, ga_w) and same_bits(gw, gw_w) and gb is None


def test_non_finite_values_follow_the_host(backend, oracle):
    """Inf upstream times a zero trit is NaN on the host (upstream * (0 * scale)); so it is here."""
    rng = np.random.default_rng(12)
    m, n, k = 3, 20, 300
    w = ternary(rng, n, k)
    packed = oracle.pack_matrix(w, n, k, FMT_TQ2_0)
    act = rng.standard_normal((m, k)).astype(np.float32)
    act[1, 7] = np.nan
    sc = rng.uniform(0.1, 1, n).astype(np.float32)
    sc[3] = np.inf
    gy = rng.standard_normal((m, n)).astype(np.float32)
    gy[0, 5] = np.inf
    gy[2, 9] = -np.inf
    rc, ga_w, gw_w, gb_w = oracle.cpu_projected_vjp(packed, FMT_TQ2_0, act, sc, gy, m, n, k)
    ga, gw, gb = _vjp(backend, packed, FMT_TQ2_0, act, sc, gy, m, n, k)
    for got, want in ((ga, ga_w), (gw, gw_w), (gb, gb_w)):
        nan = np.isnan(want)
        assert (np.isnan(got) == nan).all() and same_bits(got[~nan], want[~nan])


def test_device_resident_form_equals_the_host_form(backend, oracle):
    rng = np.random.default_rng(13)
    m, n, k = 40, 100, 700
    packed = oracle.pack_matrix(ternary(rng, n, k), n, k, FMT_TQ2_0)
    act = rng.standard_normal((m, k)).astype(np.float32)
    sc = rng.uniform(0.1, 1, n).astype(np.float32)
    gy = rng.standard_normal((m, n)).astype(np.float32)
    ga_w, gw_w, gb_w = _vjp(backend, packed, FMT_TQ2_0, act, sc, gy, m, n, k)
    buf = backend.upload_weights(packed, T.GemmShape(0, n, k), T.TernaryFormat(FMT_TQ2_0))
    d = [backend.to_device(x, "f32") for x in (sc, act, gy)]
    o = [backend.empty(c, "f32") for c in (m * k, n * k, n)]
    backend.projected_vjp(buf, d[0], d[1], d[2], m, o[0], o[1], o[2])
    backend.sync()
    assert same_bits(o[0].to_host(), ga_w) and same_bits(o[1].to_host(), gw_w) and same_bits(o[2].to_host(), gb_w)
    for a in d + o:
        a.free()


def test_reserved_code_is_refused_before_any_write(backend, oracle):
    """lib.rs:600-638."""
    for corrupt in (0, 1):
        packed = oracle.pack_matrix(np.ones((1, 1), np.int8), 1, 1, FMT_TQ2_0).copy()
        packed[corrupt] |= 3
        buf = backend.upload_weights(packed, T.GemmShape(1, 1, 1), T.TernaryFormat.Tq2_0)
        ga, gw, gb = np.array([41.0], np.float32), np.array([42.0], np.float32), np.array([43.0], np.float32)
        with pytest.raises(T.Backend, match="unpack row 0: decoded value 2 outside ternary range"):
            backend.mpgemm_projected_vjp(T.MpGemmProjectedVjp(
                act=np.ones(1, np.float32), weights=buf, scales=np.ones(1, np.float32), grad_output=np.ones(1, np.float32),
                shape=T.GemmShape(1, 1, 1), format=T.TernaryFormat.Tq2_0, grad_act=ga, grad_projected_weight=gw, grad_bias=gb))
        assert (ga[0], gw[0], gb[0]) == (41.0, 42.0, 43.0)


def test_zero_dimensions(backend, oracle):
    """lib.rs:640-666 (k = 0: the bias is still summed); m = 0 and n = 0 zero-fill (kernel.rs:122-129)."""
    buf = backend.upload_weights(np.zeros(0, np.uint8), T.GemmShape(2, 3, 0), T.TernaryFormat.Tq2_0)
    gb = np.full(3, np.nan, np.float32)
    backend.mpgemm_projected_vjp(T.MpGemmProjectedVjp(
        act=np.zeros(0, np.float32), weights=buf, scales=np.array([1, 2, 3], np.float32),
        grad_output=np.array([1, 2, 3, 1, 2, 4], np.float32), shape=T.GemmShape(2, 3, 0), format=T.TernaryFormat.Tq2_0,
        grad_act=np.zeros(0, np.float32), grad_projected_weight=np.zeros(0, np.float32), grad_bias=gb))
    assert gb.tolist() == [2.0, 4.0, 7.0]
    n, k = 5, 40
    rng = np.random.default_rng(2)
    packed = oracle.pack_matrix(ternary(rng, n, k), n, k, FMT_TQ2_0)
    buf = backend.upload_weights(packed, T.GemmShape(0, n, k), T.TernaryFormat.Tq2_0)
    gw, gb = np.full((n, k), np.nan, np.float32), np.full(n, np.nan, np.float32)
    backend.mpgemm_projected_vjp(T.MpGemmProjectedVjp(
        act=np.zeros(0, np.float32), weights=buf, scales=np.ones(n, np.float32), grad_output=np.zeros(0, np.float32),
        shape=T.GemmShape(0, n, k), format=T.TernaryFormat.Tq2_0, grad_act=np.zeros(0, np.float32),
        grad_projected_weight=gw, grad_bias=gb))
    assert not gw.any() and not gb.any()


def test_length_and_identity_errors(backend, oracle):
    """lib.rs:668-700 and the order of kernel.rs:102-120; identity first (lib.rs:363)."""
    packed = oracle.pack_matrix(np.ones((1, 1), np.int8), 1, 1, FMT_TQ2_0)
    buf = backend.upload_weights(packed, T.GemmShape(1, 1, 1), T.TernaryFormat.Tq2_0)
    one = lambda: np.ones(1, np.float32)  # noqa: E731

    def call(**kw):
        args = dict(act=one(), weights=buf, scales=one(), grad_output=one(), shape=T.GemmShape(1, 1, 1),
                    format=T.TernaryFormat.Tq2_0, grad_act=one(), grad_projected_weight=one(), grad_bias=None)
        args.update(kw)
        backend.mpgemm_projected_vjp(T.MpGemmProjectedVjp(**args))

    with pytest.raises(T.ShapeMismatch) as e:
        call(grad_act=np.zeros(0, np.float32))
    assert (e.value.expected, e.value.got) == (1, 0)
    with pytest.raises(T.ShapeMismatch) as e:
        call(act=np.zeros(3, np.float32), grad_output=np.zeros(2, np.float32))  # act is checked first
    assert (e.value.expected, e.value.got) == (1, 3)
    with pytest.raises(T.ShapeMismatch) as e:
        call(grad_bias=np.zeros(2, np.float32))
    assert (e.value.expected, e.value.got) == (1, 2)
    with pytest.raises(T.InvalidInput):
        call(shape=T.GemmShape(1, 2, 1), act=np.zeros(7, np.float32))  # identity before lengths
    call()
