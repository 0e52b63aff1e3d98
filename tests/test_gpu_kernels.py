"""Kernel parity through the device-resident C ABI: bit-exact integer paths, bounded float paths.

Shapes follow the reference's GPU tail-shape tests (crates/tritium-cuda/src/cuda/tests.rs:1886-1934,
2026-2215) and the BASELINE configs; the expected values come from the CPU oracle."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import (accepts, bf16_bits_to_f32, f32_to_bf16_bits, rel_err, same_bits, scales, ternary)
from oracle_lib import FMT_TQ1_0, FMT_TQ2_0

pytestmark = pytest.mark.gpu

DECODE_SHAPES = [(1, 1, 1), (1, 7, 300), (5, 130, 257), (64, 3, 2560), (3, 33, 6912), (1, 1, 8192),
                 (16, 8, 256), (33, 13, 512), (7, 9, 1024), (1, 16, 256), (17, 17, 513), (2, 100, 4096)]
GEMM_SHAPES = [(65, 8, 256), (100, 50, 700), (130, 257, 512), (128, 40, 2560), (200, 129, 300), (257, 16, 256)]


@pytest.fixture(params=["ksplit", "stream", "flow", "flow32"], autouse=True)
def decode_kernel(request, backend):
    """Every case runs through all decode kernels: K-split (default for narrow launches), streaming
    and flow (forced here; the defaults for launches that fill the chip), the last with 17..64
    operand rows on each of its two matrix instructions ("flow" 16x16x64, "flow32" 32x32x32)."""
    backend.set_decode_kernel({"ksplit": 1, "stream": 2, "flow": 3, "flow32": 3}[request.param])
    backend.set_flow_mfma(32 if request.param == "flow32" else 16)
    yield request.param
    backend.set_decode_kernel(0)
    backend.set_flow_mfma(0)


def _layer(backend, oracle, ws, scs, fmt=FMT_TQ2_0):
    n, k = ws[0].shape
    packed = [oracle.pack_matrix(w, n, k, fmt) for w in ws]
    return packed, backend.linear(packed, scs, n, k, T.TernaryFormat(fmt))


@pytest.mark.parametrize("m,n,k", DECODE_SHAPES + GEMM_SHAPES)
def test_int8_accumulators_bit_exact(backend, oracle, m, n, k):
    print("case int8-acc", m, n, k, flush=True)
    rng = np.random.default_rng(m * 131 + n * 17 + k)
    w = ternary(rng, n, k)
    q = rng.integers(-128, 128, (m, k)).astype(np.int8)
    q.flat[0], q.flat[-1] = -128, 127
    packed, layer = _layer(backend, oracle, [w], [np.ones(n, np.float32)])
    dq = backend.to_device(q, "i8")
    dacc = backend.empty(m * n, "i32")
    backend.linear_i8(layer, dq, None, m, dacc)
    got = dacc.to_host().reshape(m, n)
    want = oracle.int8_accumulators(packed[0], FMT_TQ2_0, q, m, n, k)
    assert (got == want).all()
    for a in (dq, dacc):
        a.free()
    layer.free()


@pytest.mark.parametrize("m,n,k", [(1, 7, 300), (5, 130, 257), (3, 33, 6912), (33, 13, 512), (100, 50, 700)])
@pytest.mark.parametrize("fmt", [FMT_TQ2_0, FMT_TQ1_0])
def test_a8_linear_bit_exact(backend, oracle, m, n, k, fmt):
    """quantize on device -> int32 contraction -> ((float)acc·s_w[n])·s_a[m] == the CPU composition."""
    print("case a8", m, n, k, fmt, flush=True)
    rng = np.random.default_rng(m + n + k + fmt)
    w, sc = ternary(rng, n, k), scales(rng, n)
    act = rng.standard_normal((m, k)).astype(np.float32)
    if m > 2:
        act[1] = 0.0  # a zero token: zero quants, zero scale
    packed, layer = _layer(backend, oracle, [w], [sc], fmt)
    dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
    backend.linear_a8(layer, dact, m, dout)
    got = dout.to_host()
    rc, want = oracle.cpu_mpgemm_with_act_quant(packed[0], fmt, act, sc, m, n, k)
    assert rc == 0 and same_bits(got, want)
    # the same through bf16 activations and bf16 output
    ab = f32_to_bf16_bits(act)
    dab, dob = backend.to_device(ab, "bf16"), backend.empty(m * n, "bf16")
    backend.linear_a8(layer, dab, m, dob)
    rc, want = oracle.cpu_mpgemm_with_act_quant(packed[0], fmt, bf16_bits_to_f32(ab), sc, m, n, k)
    assert (dob.to_host() == f32_to_bf16_bits(want).reshape(-1)).all()
    for a in (dact, dout, dab, dob):
        a.free()
    layer.free()


def test_act_quant_kernel_bit_exact(backend, oracle):
    rng = np.random.default_rng(11)
    m, k = 9, 777
    act = (rng.standard_normal((m, k)) * 3).astype(np.float32)
    act[3] = 0.0
    act[4, :6] = [1.0, -2.0, 0.5, -0.5, 2.0, -1.0]
    g = np.array([0x3F0F475A], np.uint32).view(np.float32)[0]
    a = np.array([0x3EFDD71B], np.uint32).view(np.float32)[0]
    act[5] = 0.0
    act[5, :3] = [g, a, -a]  # the order-of-operations / ties-to-even pin
    dact = backend.to_device(act, "f32")
    dq, ds, dn = backend.empty(m * k, "i8"), backend.empty(m, "f32"), backend.empty(m, "i32")
    backend.act_quant_i8(dact, m, k, dq, ds, dn)
    q, s = oracle.quantize_act_int8(act, m, k)
    assert (dq.to_host().reshape(m, k) == q.astype(np.int8)).all()
    assert same_bits(ds.to_host(), s) and (dn.to_host() == 0).all()
    assert dq.to_host().reshape(m, k)[5, :3].tolist() == [127, 112, -112]
    # golden row of the reference (crates/tritium-spec/src/lib.rs:458-466) alone in a tensor
    d1 = backend.to_device(np.array([1.0, -2.0, 0.5, -0.5, 2.0, -1.0], np.float32), "f32")
    q1, s1 = backend.empty(6, "i8"), backend.empty(1, "f32")
    backend.act_quant_i8(d1, 1, 6, q1, s1)
    assert q1.to_host().tolist() == [64, -127, 32, -32, 127, -64]
    assert s1.to_host()[0] == np.float32(2.0) / np.float32(127.0)


@pytest.mark.parametrize("m", [1, 2, 4, 8, 16, 33])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_float_linear_two_planes(backend, oracle, m, dtype):
    """BASELINE config 2 in small: two additive planes (P(0)=0.4 and 0.7), bf16 or f32 activations.
    Bound: |got-want| <= 1e-3·max|want| (north star) and the reference's own 1e-4·max(1,|want|)."""
    print("case float2p", m, dtype, flush=True)
    n, k = 192, 2048
    rng = np.random.default_rng(100 + m)
    ws = [ternary(rng, n, k, 0.4), ternary(rng, n, k, 0.7)]
    scs = [scales(rng, n), scales(rng, n)]
    act = rng.standard_normal((m, k)).astype(np.float32)
    packed, layer = _layer(backend, oracle, ws, scs)
    if dtype == "bf16":
        bits = f32_to_bf16_bits(act)
        act = bf16_bits_to_f32(bits).reshape(m, k)
        dact = backend.to_device(bits, "bf16")
    else:
        dact = backend.to_device(act, "f32")
    dout = backend.empty(m * n, "f32")
    backend.linear_float(layer, dact, m, dout)
    got = dout.to_host().reshape(m, n)
    want = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
    assert rel_err(got, want) <= 1e-3
    assert accepts(got, want, rel=1e-4, floor=1.0).all()
    # against an exact (float64) evaluation the fixed-point path is tighter than the f32 fold
    exact = sum((act.astype(np.float64) @ w.T.astype(np.float64)) * s.astype(np.float64) for w, s in zip(ws, scs))
    assert np.abs(got - exact).max() <= np.abs(want - exact).max() + 1e-6
    # reference-order kernel: bit-identical to the CPU for any float input
    dseq = backend.empty(m * n, "f32")
    backend.linear_float_seq(layer, dact, m, dseq)
    assert same_bits(dseq.to_host(), want)
    for a in (dact, dout, dseq):
        a.free()
    layer.free()


@pytest.mark.parametrize("m,n,k", DECODE_SHAPES[:8] + GEMM_SHAPES[:3])
def test_float_linear_tail_shapes(backend, oracle, m, n, k):
    print("case float-tail", m, n, k, flush=True)
    rng = np.random.default_rng(7 * m + n + k)
    w, sc = ternary(rng, n, k), scales(rng, n)
    act = (rng.standard_normal((m, k)) * rng.uniform(0.1, 30)).astype(np.float32)
    packed, layer = _layer(backend, oracle, [w], [sc])
    dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
    backend.linear_float(layer, dact, m, dout)
    got = dout.to_host().reshape(m, n)
    rc, want = oracle.cpu_mpgemm(packed[0], FMT_TQ2_0, act, sc, m, n, k)
    assert rc == 0 and accepts(got, want, rel=1e-4, floor=1.0).all()
    for a in (dact, dout):
        a.free()
    layer.free()


def test_integer_valued_floats_are_exact(backend, oracle):
    """mpgemm on int8-valued f32 (what TernaryLinear feeds a backend) is exact: bits equal the CPU's."""
    rng = np.random.default_rng(5)
    m, n, k = 6, 40, 2560
    w, sc = ternary(rng, n, k), scales(rng, n)
    act = rng.integers(-128, 128, (m, k)).astype(np.float32)
    packed, layer = _layer(backend, oracle, [w], [sc])
    dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
    backend.linear_float(layer, dact, m, dout)
    rc, want = oracle.cpu_mpgemm(packed[0], FMT_TQ2_0, act, sc, m, n, k)
    assert same_bits(dout.to_host(), want)


def test_nan_inf_propagate_like_the_reference(backend, oracle):
    """crates/tritium-cpu/src/lib.rs:982-1003 and reference.rs:44-48: NaN/Inf under a non-zero trit
    propagate, under a zero trit they are skipped. Rows holding them take the in-kernel sequential
    path, so the bits equal the CPU's."""
    rng = np.random.default_rng(9)
    m, n, k = 4, 20, 512
    w, sc = ternary(rng, n, k), scales(rng, n)
    act = rng.standard_normal((m, k)).astype(np.float32)
    act[0, 3] = np.nan
    act[1, 100] = np.inf
    act[2, 7] = -np.inf
    act[2, 9] = np.nan
    packed, layer = _layer(backend, oracle, [w], [sc])
    dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
    backend.linear_float(layer, dact, m, dout)
    got = dout.to_host().reshape(m, n)
    rc, want = oracle.cpu_mpgemm(packed[0], FMT_TQ2_0, act, sc, m, n, k)
    assert (np.isnan(got) == np.isnan(want)).all()
    fin = ~np.isnan(want)
    assert same_bits(got[:3][fin[:3]], want[:3][fin[:3]])
    assert accepts(got[3], want[3]).all()
    assert np.isnan(got[0]).any() and not np.isnan(got[0]).all()  # zero trits really skip
    # fused path: the quantizer's NaN/Inf behaviour too
    backend.linear_a8(layer, dact, m, dout)
    got = dout.to_host().reshape(m, n)
    rc, want = oracle.cpu_mpgemm_with_act_quant(packed[0], FMT_TQ2_0, act, sc, m, n, k)
    assert (np.isnan(got) == np.isnan(want)).all()
    assert same_bits(got[~np.isnan(want)], want[~np.isnan(want)])


def test_tq1_equals_tq2_and_download(backend, oracle):
    """The same trits through either packing give identical bits (cuda tests.rs:5520), and the
    device-resident planes decode back to the trits that were packed."""
    rng = np.random.default_rng(13)
    m, n, k = 3, 37, 777
    w, sc = ternary(rng, n, k), scales(rng, n)
    act = rng.standard_normal((m, k)).astype(np.float32)
    outs = []
    for fmt in (FMT_TQ2_0, FMT_TQ1_0):
        packed, layer = _layer(backend, oracle, [w], [sc], fmt)
        assert (layer.planes[0].download_trits() == w).all()
        dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
        backend.linear_a8(layer, dact, m, dout)
        outs.append(dout.to_host())
        backend.linear_float(layer, dact, m, dout)
        outs.append(dout.to_host())
    assert same_bits(outs[0], outs[2]) and same_bits(outs[1], outs[3])


def test_three_planes_a8(backend, oracle):
    """BASELINE config 5 in small: three planes, P(0)=0.4/0.7/0.85, batch 64 -> decode kernel; batch
    96 -> GEMM kernel. out = (Σ_p (float)acc_p·s_p[n])·s_a[m] in plane order."""
    rng = np.random.default_rng(21)
    n, k = 80, 1024
    ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7, 0.85)]
    scs = [scales(rng, n) for _ in range(3)]
    packed, layer = _layer(backend, oracle, ws, scs)
    for m in (1, 64, 96):
        print("case 3planes", m, flush=True)
        act = rng.standard_normal((m, k)).astype(np.float32)
        dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
        backend.linear_a8(layer, dact, m, dout)
        want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
        assert same_bits(dout.to_host(), want)
        dact.free()
        dout.free()


@pytest.mark.parametrize("m,n,k,planes", [(56, 48, 3072, 2), (64, 200, 2816, 3), (40, 16400, 4352, 1), (36, 48, 4864, 1),
                                            (28, 16400, 6144, 1)])
def test_single_launch_with_rows_beyond_lds(backend, oracle, m, n, k, planes, decode_kernel):
    """One launch whose operand rows exceed LDS (more than 32 rows, or more than 16 on a layer of at
    least 16384 outputs) goes through the prefill kernel by default; forced back onto the decode kernels it gives the same
    bits, and both equal the CPU backend's."""
    if decode_kernel != "stream":
        pytest.skip("single configuration")
    print("case rows-beyond-lds", m, n, k, planes, flush=True)
    backend.set_decode_kernel(0)  # automatic choice
    rng = np.random.default_rng(m + n)
    ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7, 0.85)[:planes]]
    scs = [scales(rng, n) for _ in range(planes)]
    packed, layer = _layer(backend, oracle, ws, scs)
    act = rng.standard_normal((m, k)).astype(np.float32)
    dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
    backend.linear_a8(layer, dact, m, dout)
    a = dout.to_host()
    backend.set_decode_kernel(2)  # the streaming decode kernel
    try:
        backend.linear_a8(layer, dact, m, dout)
        b = dout.to_host()
    finally:
        backend.set_decode_kernel(0)  # the float call below is on the automatic choice too
    rows = np.arange(m) if n * k <= 1 << 21 else np.array([0, m // 2, m - 1])
    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act[rows], len(rows), n, k)
    assert same_bits(a, b) and same_bits(a.reshape(m, n)[rows], want)
    if m <= 16 * 4:  # the float contract on the same path: 4 digit rows per token
        mf = m // 4
        dout2 = backend.empty(mf * n, "f32")
        backend.linear_float(layer, dact, mf, dout2)
        got = dout2.to_host().reshape(mf, n)
        wantf = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, act[:mf], mf, n, k)
        assert rel_err(got, wantf) <= 1e-3 and accepts(got, wantf, rel=1e-4, floor=1.0).all()
        dout2.free()
    dact.free()
    dout.free()
    layer.free()


def test_gemm_crossover_is_bit_neutral(backend, oracle):
    """Decode kernel and GEMM kernel give identical bits (cuda tests.rs:2100-2190: IMMA == dp4a)."""
    rng = np.random.default_rng(23)
    m, n, k = 48, 72, 1280
    w, sc = ternary(rng, n, k), scales(rng, n)
    act = rng.standard_normal((m, k)).astype(np.float32)
    packed, layer = _layer(backend, oracle, [w], [sc])
    dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
    backend.linear_a8(layer, dact, m, dout)
    a = dout.to_host()
    backend.set_gemm_min_m(2)
    try:
        backend.linear_a8(layer, dact, m, dout)
        b = dout.to_host()
    finally:
        backend.set_gemm_min_m(65)
    rc, want = oracle.cpu_mpgemm_with_act_quant(packed[0], FMT_TQ2_0, act, sc, m, n, k)
    assert same_bits(a, b) and same_bits(a, want)


@pytest.mark.parametrize("m,n,k", [(65, 64, 512), (150, 136, 768), (130, 131, 512), (300, 520, 256)])
def test_gemm_epilogue_variants(backend, oracle, m, n, k, decode_kernel):
    """The prefill kernel's two ways out -- rows staged through LDS when the output rows are 16-byte
    aligned, direct stores otherwise -- for every output type, both activation contracts, and with
    tokens that take the exact NaN/Inf path in the middle of a tile."""
    if decode_kernel != "ksplit":
        pytest.skip("the prefill kernel does not depend on the decode kernel choice")
    print("case gemm-epilogue", m, n, k, flush=True)
    rng = np.random.default_rng(m * 7 + n)
    ws = [ternary(rng, n, k, 0.4), ternary(rng, n, k, 0.7)]
    scs = [scales(rng, n), scales(rng, n)]
    act = rng.standard_normal((m, k)).astype(np.float32)
    act[3, 5] = np.nan
    act[m - 2, k - 1] = np.inf
    act[40] = 0.0
    packed, layer = _layer(backend, oracle, ws, scs)
    dact = backend.to_device(act, "f32")
    want_a8 = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k).reshape(m, n)
    want_f = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, act, m, n, k).reshape(m, n)
    fin = np.isfinite(want_f)
    for dtype in ("f32", "bf16"):
        dout = backend.empty(m * n, dtype)
        backend.linear_a8(layer, dact, m, dout)
        got = dout.to_host().reshape(m, n)
        if dtype == "bf16":
            ok = ~np.isnan(want_a8)
            assert (np.isnan(bf16_bits_to_f32(got).reshape(m, n)) == ~ok).all()
            assert (got[ok] == f32_to_bf16_bits(want_a8).reshape(m, n)[ok]).all()
        else:
            assert (np.isnan(got) == np.isnan(want_a8)).all()
            assert same_bits(got[~np.isnan(want_a8)], want_a8[~np.isnan(want_a8)])
        backend.linear_float(layer, dact, m, dout)
        got = dout.to_host().reshape(m, n)
        if dtype == "bf16":
            got = bf16_bits_to_f32(got).reshape(m, n)
            assert (np.isnan(got) == np.isnan(want_f)).all()
            assert accepts(got[fin], want_f[fin], rel=1e-2, floor=1.0).all()  # bf16 keeps 8 bits
        else:
            assert (np.isnan(got) == np.isnan(want_f)).all()
            assert accepts(got[fin], want_f[fin], rel=1e-4, floor=1.0).all()
            # rows with NaN/Inf are computed in the reference's order: bits equal the CPU's
            assert same_bits(got[3][fin[3]], want_f[3][fin[3]]) and same_bits(got[m - 2][fin[m - 2]], want_f[m - 2][fin[m - 2]])
        dout.free()
    # raw accumulators of one plane
    q = rng.integers(-128, 128, (m, k)).astype(np.int8)
    single = backend.linear([packed[0]], [scs[0]], n, k, T.TernaryFormat(FMT_TQ2_0))
    dq, dacc = backend.to_device(q, "i8"), backend.empty(m * n, "i32")
    backend.linear_i8(single, dq, None, m, dacc)
    assert (dacc.to_host().reshape(m, n) == oracle.int8_accumulators(packed[0], FMT_TQ2_0, q, m, n, k)).all()
    for a in (dact, dq, dacc):
        a.free()
    single.free()
    layer.free()


@pytest.mark.parametrize("nb", [1, 2, 3, 4, 5, 6, 7, 9, 27])
@pytest.mark.parametrize("planes", [1, 2])
def test_flow_runs_of_several_tiles(backend, oracle, nb, planes, decode_kernel):
    """A wave of the flow kernel walks runs of consecutive tiles as one stream behind a prefetch
    ring; every K block count relative to the ring size, runs of 2 and 5 tiles, ragged last run,
    one, two and four row tiles (the last two on either matrix instruction)."""
    if decode_kernel not in ("flow", "flow32"):
        pytest.skip("flow kernel only")
    k = nb * 256 - 13
    n = 16 * 37 + 5
    rng = np.random.default_rng(1000 + nb * 10 + planes)
    ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7)[:planes]]
    scs = [np.ones(n, np.float32) for _ in range(planes)]
    packed, layer = _layer(backend, oracle, ws, scs)
    try:
        for run_tiles in (2, 5):
            backend.set_flow_run_tiles(run_tiles)
            for m in ((1, 16, 17, 64) if decode_kernel == "flow" else (17, 33, 64)):
                print("case flow-runs", nb, planes, run_tiles, m, flush=True)
                q = rng.integers(-128, 128, (m, k)).astype(np.int8)
                dq, dout = backend.to_device(q, "i8"), backend.empty(m * n, "f32")
                backend.linear_i8(layer, dq, None, m, dout)
                got = dout.to_host().reshape(m, n)
                want = sum(q.astype(np.int32) @ w.T.astype(np.int32) for w in ws).astype(np.float32)
                assert same_bits(got, want)  # exact: the sums stay far below 2^24
                dq.free()
                dout.free()
    finally:
        backend.set_flow_run_tiles(0)
        layer.free()


def test_group_launch_equals_single_launches(backend, oracle):
    rng = np.random.default_rng(29)
    k = 768
    act = rng.standard_normal((2, k)).astype(np.float32)
    dact = backend.to_device(act, "f32")
    members, singles = [], []
    for n in (48, 20, 129):  # q/k/v-like: one activation, three projections
        w, sc = ternary(rng, n, k), scales(rng, n)
        _, layer = _layer(backend, oracle, [w], [sc])
        out_g, out_s = backend.empty(2 * n, "f32"), backend.empty(2 * n, "f32")
        members.append((layer, dact, 2, out_g))
        singles.append((layer, out_s))
    for mode, fn in ((1, backend.linear_a8), (0, backend.linear_float)):
        grp = backend.group(members, mode, "f32", "f32")
        grp.launch()
        grp.launch()  # relaunch is idempotent
        for (layer, _, _, out_g), (_, out_s) in zip(members, singles):
            fn(layer, dact, 2, out_s)
            assert same_bits(out_g.to_host(), out_s.to_host())
        grp.destroy()


def test_group_with_rows_beyond_lds_takes_the_prefill_kernel(backend, oracle, decode_kernel):
    """Grouped decode whose operand rows do not fit in LDS (40 tokens x K=4500 int8, 12 tokens x 4
    digit rows x K=4500) runs as one grouped launch of the prefill kernel; bits equal the single
    launches and the CPU composition. Two projections share an activation, a third has its own."""
    if decode_kernel != "ksplit":
        pytest.skip("automatic kernel choice only")
    backend.set_decode_kernel(0)
    rng = np.random.default_rng(37)
    for mode, m, fn in ((1, 40, backend.linear_a8), (0, 12, backend.linear_float)):
        k = 4500
        act_a = rng.standard_normal((m, k)).astype(np.float32)
        act_b = rng.standard_normal((m, k)).astype(np.float32)
        act_c = rng.standard_normal((m, 768)).astype(np.float32)  # these rows do fit: the flow kernel's share
        da, db, dc = backend.to_device(act_a, "f32"), backend.to_device(act_b, "f32"), backend.to_device(act_c, "f32")
        members, singles, hosts = [], [], []
        for n, src, act in ((136, da, act_a), (200, dc, act_c), (72, da, act_a), (257, db, act_b), (48, dc, act_c)):
            k = act.shape[1]
            ws = [ternary(rng, n, k, 0.4), ternary(rng, n, k, 0.7)]
            scs = [scales(rng, n), scales(rng, n)]
            packed, layer = _layer(backend, oracle, ws, scs)
            out_g, out_s = backend.empty(m * n, "f32"), backend.empty(m * n, "f32")
            members.append((layer, src, m, out_g))
            singles.append((layer, src, out_s))
            hosts.append((packed, scs, act, n))
        grp = backend.group(members, mode, "f32", "f32")
        # the group's two kernels (flow part, prefill-kernel part) one after the other, then side by side on
        # two streams (the default), several launches in a row: every launch leaves the same bits
        backend.set_group_overlap(False)
        grp.launch()
        in_turn = [out_g.to_host().copy() for _, _, _, out_g in members]
        backend.set_group_overlap(True)
        for _ in range(3):
            for _, _, _, out_g in members:
                out_g.copy_from(np.full(out_g.count, np.float32(-7.0)))
            grp.launch()
            for (_, _, _, out_g), ref in zip(members, in_turn):
                assert same_bits(out_g.to_host(), ref)
        for (layer, src, _, out_g), (_, _, out_s), (packed, scs, act, n) in zip(members, singles, hosts):
            k = act.shape[1]
            fn(layer, src, m, out_s)
            got = out_g.to_host()
            assert same_bits(got, out_s.to_host())
            if mode == 1:
                assert same_bits(got, oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k))
            else:
                want = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
                assert accepts(got.reshape(m, n), want.reshape(m, n), rel=1e-4, floor=1.0).all()
        grp.destroy()


def test_ternary_linear_forward(backend, oracle):
    """tritium-nn/tests/layers.rs:138+ : TernaryLinear on the backend vs the inline reference, ragged K."""
    rng = np.random.default_rng(31)
    n, k, m = 24, 300, 5
    w = ternary(rng, n, k)
    lin = T.TernaryLinear.new(backend, w, n, k, 0.037)
    act = rng.standard_normal((m, k)).astype(np.float32)
    out = np.zeros(m * n, np.float32)
    lin.forward(backend, act, m, out)
    packed = oracle.pack_matrix(w, n, k, FMT_TQ2_0)
    rc, want = oracle.cpu_mpgemm_with_act_quant(packed, FMT_TQ2_0, act, np.full(n, 0.037, np.float32), m, n, k)
    assert same_bits(out, want)
    with pytest.raises(T.ShapeMismatch):
        lin.forward(backend, act[:, :-1], m, out)


def test_streaming_kernel_by_default_on_wide_launch(backend, oracle, decode_kernel):
    """A launch wide enough to take the streaming kernel on its own (>= one workgroup per CU), ragged
    tile count, three planes, 64 operand rows -> two LDS passes over K."""
    if decode_kernel != "stream":
        pytest.skip("single configuration")
    backend.set_decode_kernel(0)
    rng = np.random.default_rng(41)
    m, n, k = 64, 33000, 1300
    ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7, 0.85)]
    scs = [scales(rng, n) for _ in range(3)]
    packed = [T.pack_rows(w, n, k) for w in ws]
    layer = backend.linear(packed, scs, n, k)
    q = rng.integers(-128, 128, (m, k)).astype(np.int8)
    s_a = rng.uniform(0.001, 0.1, m).astype(np.float32)
    dq, ds, dout = backend.to_device(q, "i8"), backend.to_device(s_a, "f32"), backend.empty(m * n, "f32")
    backend.linear_i8(layer, dq, ds, m, dout)
    got = dout.to_host().reshape(m, n)
    accs = [q.astype(np.int32) @ w.T.astype(np.int32) for w in ws]  # exact integer reference
    want = np.zeros((m, n), np.float32)
    for p, (a, sc) in enumerate(zip(accs, scs)):
        t = a.astype(np.float32) * sc[None, :]
        want = t if p == 0 else want + t
    want = want * s_a[:, None]
    assert same_bits(got, want)
    rows = [0, 31, 63]
    for p in range(3):
        assert (oracle.int8_accumulators(packed[p], FMT_TQ2_0, q[rows], 3, n, k) == accs[p][rows]).all()


def test_flow_kernel_by_default_on_wide_launch(backend, oracle, decode_kernel):
    """Wide launch whose operand rows fit in LDS: takes the flow kernel on its own. Ragged tile count
    (runs clamp at the end of the plane), two planes, bf16 in, bf16 out."""
    if decode_kernel != "flow":
        pytest.skip("single configuration")
    backend.set_decode_kernel(0)
    rng = np.random.default_rng(43)
    m, n, k = 3, 70001, 700
    ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7)]
    scs = [scales(rng, n) for _ in range(2)]
    packed = [T.pack_rows(w, n, k) for w in ws]
    layer = backend.linear(packed, scs, n, k)
    bits = f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
    act = bf16_bits_to_f32(bits).reshape(m, k)
    dact, dout = backend.to_device(bits, "bf16"), backend.empty(m * n, "f32")
    backend.linear_float(layer, dact, m, dout)
    got = dout.to_host().reshape(m, n)
    want = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
    assert rel_err(got, want) <= 1e-3 and accepts(got, want).all()
    dob = backend.empty(m * n, "bf16")
    backend.linear_a8(layer, dact, m, dob)
    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
    assert (dob.to_host() == f32_to_bf16_bits(want).reshape(-1)).all()
