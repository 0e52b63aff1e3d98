"""RMSNorm fused in front of the int8 activation quantization, through the device-resident C ABI.

The reference pins its fused decode kernel to the host's rmsnorm followed by the host's int8
quantization, bit for bit (crates/tritium-cuda/src/cuda/tests.rs:4675-4771); the same inputs and the
same bar are used here, with the CPU oracle as the host side."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import bf16_bits_to_f32, f32_to_bf16_bits, same_bits, scales, ternary
from oracle_lib import FMT_TQ2_0

pytestmark = pytest.mark.gpu

EPS = 1e-5


def reference_inputs(n, rows=1):
    """x [rows,n] then w [n] from the xorshift stream of the reference's test
    (crates/tritium-cuda/src/cuda/tests.rs:4728-4737): values in [-4, 4)."""
    s = (0x0FEDCBA987654321 ^ ((n * 0x9E3779B9) & 0xFFFFFFFFFFFFFFFF)) & 0xFFFFFFFFFFFFFFFF
    out = np.empty(rows * n + n, np.float32)
    two53 = np.float32(2.0 ** 53)
    for i in range(out.size):
        s ^= (s << 13) & 0xFFFFFFFFFFFFFFFF
        s ^= s >> 7
        s ^= (s << 17) & 0xFFFFFFFFFFFFFFFF
        out[i] = np.float32(np.float32(np.uint64(s >> 11)) / two53) * np.float32(8.0) - np.float32(4.0)
    return out[:rows * n].reshape(rows, n), out[rows * n:]


def _quant(backend, x_dev, w_dev, m, k, zero_centered=False):
    q, sc, nf = backend.empty(m * k, "i8"), backend.empty(m, "f32"), backend.empty(m, "i32")
    backend.rmsnorm_quant_i8(x_dev, w_dev, EPS, m, k, q, sc, nf, zero_centered=zero_centered)
    got = q.to_host().reshape(m, k), sc.to_host(), nf.to_host()
    for a in (q, sc, nf):
        a.free()
    return got


@pytest.mark.parametrize("n", [2560, 6912, 1, 17, 256, 2559])
@pytest.mark.parametrize("zero_centered", [False, True])
def test_rmsnorm_quant_bit_matches_host(backend, oracle, n, zero_centered):
    print("case rmsnorm-quant", n, zero_centered, flush=True)
    rows = 3
    x, w = reference_inputs(n, rows)
    dx, dw = backend.to_device(x, "f32"), backend.to_device(w, "f32")
    q, sc, nf = _quant(backend, dx, dw, rows, n, zero_centered)
    q_want, sc_want = oracle.rmsnorm_quant(x, w, rows, n, EPS, zero_centered)
    assert same_bits(sc, sc_want)
    assert (q.astype(np.float32) == q_want).all()
    assert not nf.any()
    dx.free()
    dw.free()


def test_rmsnorm_quant_bf16_rows_and_zero_row(backend, oracle):
    rng = np.random.default_rng(5)
    m, k = 4, 1000
    bits = f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32) * 2)
    bits[2] = 0  # an all-zero row: zeros and scale 0 (tests.rs:4759-4771)
    x = bf16_bits_to_f32(bits).reshape(m, k)
    w = rng.uniform(-2, 2, k).astype(np.float32)
    dx, dw = backend.to_device(bits, "bf16"), backend.to_device(w, "f32")
    q, sc, nf = _quant(backend, dx, dw, m, k)
    q_want, sc_want = oracle.rmsnorm_quant(x, w, m, k, EPS)
    assert same_bits(sc, sc_want) and (q.astype(np.float32) == q_want).all()
    assert sc[2] == 0.0 and not q[2].any()
    dx.free()
    dw.free()


@pytest.mark.parametrize("decode_kernel", [0, 1, 2, 3])
@pytest.mark.parametrize("m,n,k,planes", [(1, 48, 2560, 1), (5, 130, 700, 2), (40, 72, 1280, 1), (70, 64, 512, 2)])
def test_linear_rmsnorm_a8_equals_norm_then_linear(backend, oracle, decode_kernel, m, n, k, planes):
    """out has the bits of: host rmsnorm, then the backend trait's fused quantize + contract + fold on
    the normalized rows, for every decode kernel and (m = 70) the prefill kernel."""
    print("case linear-rmsnorm", decode_kernel, m, n, k, planes, flush=True)
    rng = np.random.default_rng(m * 31 + n)
    ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7)[:planes]]
    scs = [scales(rng, n) for _ in range(planes)]
    packed = [oracle.pack_matrix(w, n, k, FMT_TQ2_0) for w in ws]
    layer = backend.linear(packed, scs, n, k, T.TernaryFormat(FMT_TQ2_0))
    x = (rng.standard_normal((m, k)) * 3).astype(np.float32)
    w = rng.uniform(0.5, 1.5, k).astype(np.float32)
    y = np.stack([oracle.rmsnorm(x[r], w, EPS) for r in range(m)])
    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, y, m, n, k)
    dx, dw, dout = backend.to_device(x, "f32"), backend.to_device(w, "f32"), backend.empty(m * n, "f32")
    backend.set_decode_kernel(decode_kernel)
    try:
        backend.linear_rmsnorm_a8(layer, dx, dw, EPS, m, dout)
        assert same_bits(dout.to_host(), want)
    finally:
        backend.set_decode_kernel(0)
        for a in (dx, dw, dout):
            a.free()
        layer.free()


def test_rows_with_nan_or_inf_follow_the_host(backend, oracle):
    """A NaN makes the whole normalized row NaN; an Inf makes inv 0 and that element NaN. The host
    quantizer never takes NaN as the row maximum (crates/tritium-spec/src/lib.rs:354-360), and the
    contraction of the resulting values is what the device has to reproduce."""
    rng = np.random.default_rng(8)
    m, n, k = 4, 40, 600
    wt, sc = ternary(rng, n, k), scales(rng, n)
    packed = oracle.pack_matrix(wt, n, k, FMT_TQ2_0)
    layer = backend.linear([packed], [sc], n, k, T.TernaryFormat(FMT_TQ2_0))
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[1, 17] = np.nan
    x[3, 5] = np.inf
    w = rng.uniform(0.5, 1.5, k).astype(np.float32)
    y = np.stack([oracle.rmsnorm(x[r], w, EPS) for r in range(m)])
    rc, want = oracle.cpu_mpgemm_with_act_quant(packed, FMT_TQ2_0, y, sc, m, n, k)
    dx, dw, dout = backend.to_device(x, "f32"), backend.to_device(w, "f32"), backend.empty(m * n, "f32")
    backend.linear_rmsnorm_a8(layer, dx, dw, EPS, m, dout)
    assert same_bits(dout.to_host(), want)
    for a in (dx, dw, dout):
        a.free()
    layer.free()


@pytest.mark.parametrize("zero_centered", [False, True])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("m,k", [(1, 256), (3, 2560), (2, 4096), (4, 6912), (1, 8192), (300, 1024)])
def test_rows_of_whole_blocks_take_one_pass(backend, oracle, m, k, dtype, zero_centered):
    """Rows of whole K blocks up to K = 8192 go through the kernel that reads the row once (the sum of squares folds in
    the canonical order through LDS and lane shuffles): same bits as the host's rmsnorm + quantization for plain rows,
    an all-zero row, a row with NaN and a row with Inf (whose normalized values the exact fallback reads back)."""
    print("case rmsnorm-one-pass", m, k, dtype, zero_centered, flush=True)
    rng = np.random.default_rng(m * 13 + k + zero_centered)
    n = 40
    wt, sc = ternary(rng, n, k), scales(rng, n)
    packed = oracle.pack_matrix(wt, n, k, FMT_TQ2_0)
    layer = backend.linear([packed], [sc], n, k, T.TernaryFormat(FMT_TQ2_0))
    x = (rng.standard_normal((m, k)) * 10.0 ** rng.integers(-2, 3)).astype(np.float32)
    if m >= 2:
        x[1] = 0.0
    if m >= 3:
        x[2, k // 2] = np.nan
    if m >= 4:
        x[3, 7] = np.inf
    host = f32_to_bf16_bits(x) if dtype == "bf16" else x
    seen = bf16_bits_to_f32(host).reshape(m, k) if dtype == "bf16" else x
    w = (rng.uniform(-0.5, 0.5, k) if zero_centered else rng.uniform(0.5, 1.5, k)).astype(np.float32)
    y = np.stack([oracle.rmsnorm(seen[r], w, EPS, zero_centered) for r in range(m)])
    rc, want = oracle.cpu_mpgemm_with_act_quant(packed, FMT_TQ2_0, y, sc, m, n, k)
    dx, dw, dout = backend.to_device(host, dtype), backend.to_device(w, "f32"), backend.empty(m * n, "f32")
    backend.linear_rmsnorm_a8(layer, dx, dw, EPS, m, dout, zero_centered=zero_centered)
    got = dout.to_host()
    fin = ~np.isnan(want.reshape(-1))
    assert (np.isnan(got) == ~fin).all() and same_bits(got[fin], want.reshape(-1)[fin])
    for a in (dx, dw, dout):
        a.free()
    layer.free()


def test_group_shares_one_norm_per_activation(backend, oracle):
    """q/k/v read norm1(hid), o reads att as it is, gate/up read norm2(hid): one grouped launch equals
    the single launches, bit for bit, and relaunching it changes nothing."""
    rng = np.random.default_rng(9)
    m, h, f, kv = 2, 512, 768, 128
    hid = backend.to_device((rng.standard_normal((m, h)) * 2).astype(np.float32), "f32")
    att = backend.to_device(rng.standard_normal((m, h)).astype(np.float32), "f32")
    w1 = backend.to_device(rng.uniform(0.5, 1.5, h).astype(np.float32), "f32")
    w2 = backend.to_device(rng.uniform(-0.5, 0.5, h).astype(np.float32), "f32")
    spec = [("q", h, hid, (w1, EPS, False)), ("k", kv, hid, (w1, EPS, False)), ("v", kv, hid, (w1, EPS, False)),
            ("o", h, att, None), ("gate", f, hid, (w2, EPS, True)), ("up", f, hid, (w2, EPS, True))]
    members, norms, singles = [], [], []
    for name, n, src, nm in spec:
        layer = backend.linear([oracle.pack_matrix(ternary(rng, n, h), n, h, FMT_TQ2_0)], [scales(rng, n)], n, h,
                               T.TernaryFormat(FMT_TQ2_0))
        out_g, out_s = backend.empty(m * n, "f32"), backend.empty(m * n, "f32")
        members.append((layer, src, m, out_g))
        norms.append(nm)
        singles.append(out_s)
    grp = backend.group(members, 1, "f32", "f32", norms=norms)
    grp.launch()
    grp.launch()
    for (layer, src, _, out_g), nm, out_s in zip(members, norms, singles):
        if nm is None:
            backend.linear_a8(layer, src, m, out_s)
        else:
            backend.linear_rmsnorm_a8(layer, src, nm[0], nm[1], m, out_s, zero_centered=nm[2])
        assert same_bits(out_g.to_host(), out_s.to_host())
    grp.destroy()


def test_rmsnorm_argument_errors(backend, oracle):
    rng = np.random.default_rng(10)
    n, k = 16, 256
    layer = backend.linear([oracle.pack_matrix(ternary(rng, n, k), n, k, FMT_TQ2_0)], [scales(rng, n)], n, k,
                           T.TernaryFormat(FMT_TQ2_0))
    x, w, out = backend.to_device(np.ones((1, k), np.float32), "f32"), backend.to_device(np.ones(k, np.float32), "f32"), \
        backend.empty(n, "f32")
    with pytest.raises(T.InvalidInput):
        backend.linear_rmsnorm_a8(layer, x, None, EPS, 1, out)
    with pytest.raises(T.InvalidInput):
        backend.linear_rmsnorm_a8(layer, x, w, -1.0, 1, out)
    with pytest.raises(T.InvalidInput):
        backend.linear_rmsnorm_a8(layer, x, w, float("nan"), 1, out)
    for a in (x, w, out):
        a.free()
    layer.free()
